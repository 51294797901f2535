"""The numpy model of the device-side plan construction: its base plan equals the host builder's, its row groups
satisfy the structural invariants of every group plan, and the kernels' walk over them reproduces the oracle."""
import numpy as np
import pytest

import parallel_plan_model as model
from bpt_amd import graphbuilder as gb
from bpt_amd.plan import GROUP_PAD_ENTRIES, build_plan_host
from test_group_plan import GRAPHS, bpt, check_emulated_walks, check_group_invariants


def sides(name, seg):
    src, dst, n = GRAPHS[name]()
    csr = gb.get_csrs(src, dst, n, as_torch=False)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    return src, dst, n, csr, (COL, IC, in_csr[2], in_csr[1]), (ROW, IR, out_csr[2], out_csr[1])


@pytest.mark.parametrize("seg", [8, 64])
@pytest.mark.parametrize("name", sorted(GRAPHS))
def test_model_base_plan_equals_host_plan(name, seg):
    src, dst, n, csr, a_in, a_out = sides(name, seg)
    for row, ip, eid, idx in (a_in, a_out):
        host, info = build_plan_host(row, ip, eid, idx, n, n, seg)
        mod, minfo = model.base_plan(row, ip, eid, idx, n, n, seg)
        for k in ("rowptr", "idx", "eid", "items", "heavy"):
            assert np.array_equal(host[k], mod[k]), k
        assert (info.n_items, info.n_heavy, info.n_slots, info.max_degree, bool(info.flags & 1)) == \
               (minfo["n_items"], minfo["n_heavy"], minfo["n_slots"], minfo["max_degree"], minfo["perm"])


@pytest.mark.parametrize("R", [4, 8, 16])
@pytest.mark.parametrize("by_mask", [0, 1, 2])
@pytest.mark.parametrize("seg", [8, 64])
@pytest.mark.parametrize("name", sorted(GRAPHS))
def test_model_group_plan_invariants(name, seg, by_mask, R):
    src, dst, n, csr, a_in, a_out = sides(name, seg)
    for (row, ip, eid, idx), rows_of, cols_of in ((a_in, dst, src), (a_out, src, dst)):
        arrays, _ = model.base_plan(row, ip, eid, idx, n, n, seg)
        grp = model.group_plan(arrays, n, R, by_mask)
        check_group_invariants(arrays, grp, rows_of, cols_of, len(src), R, by_mask == 1)


@pytest.mark.parametrize("name,seg,R", [("bpt64c", 64, 4), ("bpt37", 8, 8), ("multi", 8, 4), ("bpt300c", 64, 8)])
def test_model_group_walk_matches_oracle(name, seg, R):
    src, dst, n, csr, a_in, a_out = sides(name, seg)
    pin, _ = model.base_plan(*a_in, n, n, seg)
    pout, _ = model.base_plan(*a_out, n, n, seg)
    gin, gout = model.group_plan(pin, n, R, 1), model.group_plan(pout, n, R, 2)
    check_emulated_walks(src, dst, n, csr, pin, gin, gout, model.link_groups(gin, gout, len(src), GROUP_PAD_ENTRIES))


def test_model_grouping_reduces_row_loads_on_the_headline_graph():
    src, dst, n = bpt(8192, True, 4)
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n, as_torch=False)
    for row, ip, eid, idx, bound in ((COL, IC, in_csr[2], in_csr[1], 0.21), (ROW, IR, out_csr[2], out_csr[1], 0.27)):
        arrays, _ = build_plan_host(row, ip, eid, idx, n, n)
        grp = model.group_plan(arrays, n, 8, False)
        assert len(grp["entries"]) < bound * len(src)
