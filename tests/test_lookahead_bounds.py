"""The row-group kernels read their per-entry arrays ahead of the entry in use (software pipeline).  This test
replays the kernels' index arithmetic on real plans, with the look-ahead constants taken from the kernel source,
and checks that the largest index every per-entry array is read at lies inside what the plan allocates
(entries + GROUP_PAD_ENTRIES padding) and that every v_readlane index is a lane id.  CPU only."""
import os
import re

import numpy as np
import pytest

from bpt_amd import graphbuilder as gb
from bpt_amd import plan as plan_mod

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = open(os.path.join(ROOT, "bpt_amd", "csrc", "bptattn.hip")).read()


def _const(name):
    m = re.search(r"constexpr int " + name + r" = (\d+);", SRC)
    assert m, name
    return int(m.group(1))


CHUNK, PAD, NB = _const("GRP_CHUNK"), _const("GRP_PAD_ENTRIES"), _const("MFMA_NB")
BATCHES = (1, 2)          # grp_batch<EPL>(): entries whose rows are loaded together


def _pipeline_reads(begin, end, batch):
    """Entry positions (and lane ids) that the two-stage pipeline of the vector row-group kernels touches through
    load_batch for one group: load_batch(A, 0), then per step load_batch(B, b + batch), load_batch(A, b + 2 * batch)."""
    worst_entry, worst_lane = -1, -1
    for p0 in range(begin, end, CHUNK):
        cnt = min(CHUNK, end - p0)
        starts = [0] + [b + s * batch for b in range(0, cnt, 2 * batch) for s in (1, 2)]
        top = max(starts) + batch - 1
        worst_entry, worst_lane = max(worst_entry, p0 + top), max(worst_lane, top)
    return worst_entry, worst_lane


def _mfma_reads(begin, end, last_padded):
    """The same for k_attn_fwd_mfma: load_half(0), load_half(NB), then load_half(b + 2 * NB) per batch; the edge-id
    list is read at min(position, last padded entry), the entry list through v_readlane of lane b + NB/2 * wave + e."""
    worst_clamped, worst_raw, worst_lane = -1, -1, -1
    for p0 in range(begin, end, CHUNK):
        cnt = min(CHUNK, end - p0)
        starts = [0, NB] + [b + 2 * NB for b in range(0, cnt, NB)]
        top = max(starts) + NB - 1
        worst_raw = max(worst_raw, p0 + top)
        worst_clamped = max(worst_clamped, min(p0 + top, last_padded))
        worst_lane = max(worst_lane, max(starts) + (NB // 2) * 1 + (NB // 2 - 1))
    return worst_clamped, worst_raw, worst_lane


def _plans(L, triu, step):
    g = gb.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n, as_torch=False)
    for units, ip, csr in ((COL, IC, in_csr), (ROW, IR, out_csr)):
        arrays, _ = plan_mod.build_plan_host(units, ip, csr[2], csr[1], n, n)
        for R in (4, 8):
            for order in (plan_mod.GROUP_ORDER, plan_mod.GROUP_ORDER_SRC):
                yield plan_mod.build_groups_host(arrays, n, R=R, order_mode=order)


def test_constants_match_the_host_side():
    assert PAD == plan_mod.GROUP_PAD_ENTRIES
    assert CHUNK % (2 * max(BATCHES)) == 0 and CHUNK + 3 * max(BATCHES) <= 64 and CHUNK % NB == 0


@pytest.mark.parametrize("L,triu,step", [(512, False, 4), (300, True, 2), (1024, True, 4), (97, False, 1)])
def test_every_lookahead_read_is_inside_the_padded_arrays(L, triu, step):
    overshoot_without_clamp = 0
    for grp in _plans(L, triu, step):
        n_entries = len(grp["entries"])
        allocated = n_entries + PAD                  # grp_eids, grp_pairs, the (p, ds) scratch: entries + padding
        ptr = grp["grp_ptr"]
        assert ptr[-1] == n_entries
        for g in range(len(ptr) - 1):
            begin, end = int(ptr[g]), int(ptr[g + 1])
            if end == begin:
                continue
            for batch in BATCHES:
                entry, lane = _pipeline_reads(begin, end, batch)
                assert entry < allocated, (g, begin, end, batch, entry, allocated)
                assert lane < 64
            clamped, raw, lane = _mfma_reads(begin, end, allocated - 1)
            assert clamped < allocated and lane < 64
            overshoot_without_clamp = max(overshoot_without_clamp, raw - (end - 1))
    # the matrix-core forward looks up to 2 * NB + NB - 1 entries past a group's last one, more than the padding:
    # the clamp in the kernel is what keeps the last group's reads inside the list
    assert overshoot_without_clamp <= 3 * NB - 1
    assert re.search(r"grp_eids\[\(size_t\)min\(p0 \+ b \+ e, eid_last\)", SRC), "k_attn_fwd_mfma must clamp its look-ahead"
