"""Row-group plans (host): structural invariants, and a numpy emulation of the walk the row-group
kernels perform over them, checked against the oracle (no GPU needed)."""
import numpy as np
import pytest

import oracle
from bpt_amd import graphbuilder as gb
from bpt_amd.plan import GROUP_PAD_ENTRIES, GROUP_R, build_groups_host, build_plan_host, link_groups_host


def bpt(L, triu, step):
    g = gb.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    return src, dst, g.number_of_nodes


def multigraph(n=40, E=600, seed=3):
    rng = np.random.default_rng(seed)
    src = rng.integers(0, n, E); dst = rng.integers(0, n, E)
    dst[: E // 3] = 1; src[E // 3: E // 2] = 2
    src[src == 0] = 3; dst[dst == 0] = 3
    src[-3:] = src[-4]; dst[-3:] = dst[-4]            # an edge with multiplicity 4
    return src.astype(np.int64), dst.astype(np.int64), n


GRAPHS = {"bpt64c": lambda: bpt(64, True, 4), "bpt37": lambda: bpt(37, False, 2), "bpt300c": lambda: bpt(300, True, 2),
          "multi": multigraph, "bpt1": lambda: bpt(1, False, 1)}


def plans(name, seg=64):
    src, dst, n = GRAPHS[name]()
    csr = gb.get_csrs(src, dst, n, as_torch=False)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    pin, _ = build_plan_host(COL, IC, in_csr[2], in_csr[1], n, n, seg)
    pout, _ = build_plan_host(ROW, IR, out_csr[2], out_csr[1], n, n, seg)
    return src, dst, n, csr, pin, pout


def check_group_invariants(arrays, grp, rows_of, cols_of, E, GROUP_R, masks_sorted):
    members, gptr, entries, pair_eid = grp["members"], grp["grp_ptr"], grp["entries"], grp["pair_eid"]
    ch = grp["chunks"]
    assert ch[0] == 0 and ch[8] == len(members) and np.all(np.diff(ch) >= 0)
    items = arrays["items"]
    ng = len(members)
    assert members.shape == (ng, GROUP_R, 2) and len(gptr) == ng + 1
    assert gptr[0] == 0 and gptr[-1] == len(entries) and np.all(np.diff(gptr) >= 0)
    # every item is a member of exactly one group
    used = [(r, s) for r, s in members.reshape(-1, 2).tolist() if r >= 0]
    assert sorted(used) == sorted((r, s) for r, _, _, s in items.tolist())
    assert np.all(members[:, 0, 0] >= 0)                      # no empty group
    # every edge is exactly one pair
    assert sorted(pair_eid.tolist()) == list(range(E))
    # entries: masks valid, pairs numbered consecutively, every pair is an edge (entry idx -> member row)
    seg_of = {(r, s): (b, e) for r, b, e, s in items.tolist()}
    eid_slot = {int(e): p for p, e in enumerate(arrays["eid"].tolist())}
    slot_eid = grp["slot_eid"]
    assert slot_eid.shape == (len(entries), GROUP_R)
    n_pairs = 0
    for g in range(ng):
        masks = entries[gptr[g]:gptr[g + 1], 1]
        if masks_sorted:
            assert np.all(np.diff(masks) <= 0)                # equal masks adjacent, larger first
        for u in range(gptr[g], gptr[g + 1]):
            idx, mask, pb, _ = entries[u].tolist()
            assert 0 < mask < (1 << GROUP_R) and pb == n_pairs
            for m in range(GROUP_R):
                if not mask >> m & 1:
                    assert slot_eid[u, m] == -1
                else:
                    row, slot = members[g, m].tolist()
                    e = int(pair_eid[n_pairs]); n_pairs += 1
                    assert slot_eid[u, m] == e
                    assert rows_of[e] == row and cols_of[e] == idx
                    b, en = seg_of[(row, slot)]
                    assert b <= eid_slot[e] < en              # the edge lies in this member's segment
    assert n_pairs == E


@pytest.mark.parametrize("GROUP_R", [4, 16])
@pytest.mark.parametrize("order_mode", [0, 1, 2, 6, 10])
@pytest.mark.parametrize("seg", [8, 64])
@pytest.mark.parametrize("name", sorted(GRAPHS))
def test_group_plan_invariants(name, seg, order_mode, GROUP_R):
    src, dst, n, csr, pin, pout = plans(name, seg)
    E = len(src)
    for arrays, rows_of, cols_of in ((pin, dst, src), (pout, src, dst)):
        grp = build_groups_host(arrays, n, R=GROUP_R, order_mode=order_mode)
        check_group_invariants(arrays, grp, rows_of, cols_of, E, GROUP_R, bool(order_mode & 4 and not order_mode & 8))


def emulate_forward(arrays, grp, q, k, v, scale):
    """What k_attn_fwd_grp + k_attn_fwd_combine compute, in float64 numpy."""
    n, h, d = q.shape
    o = np.zeros_like(q); lse = np.zeros((n, h))
    part = {}
    GROUP_R = grp["R"]
    for g in range(len(grp["members"])):
        st = [dict(m=np.full(h, -np.inf), l=np.zeros(h), acc=np.zeros((h, d))) for _ in range(GROUP_R)]
        for u in range(grp["grp_ptr"][g], grp["grp_ptr"][g + 1]):
            idx, mask, _, _ = grp["entries"][u].tolist()
            for m in range(GROUP_R):
                if mask >> m & 1:
                    row = grp["members"][g, m, 0]
                    s = (q[row] * k[idx]).sum(-1) * scale
                    mx = np.maximum(st[m]["m"], s)
                    a = np.exp(st[m]["m"] - mx); p = np.exp(s - mx)
                    st[m]["l"] = st[m]["l"] * a + p
                    st[m]["acc"] = st[m]["acc"] * a[:, None] + p[:, None] * v[idx]
                    st[m]["m"] = mx
        for m in range(GROUP_R):
            row, slot = grp["members"][g, m].tolist()
            if row < 0:
                continue
            if slot < 0:
                has = st[m]["l"] > 0
                o[row] = np.where(has[:, None], st[m]["acc"] / np.where(has, st[m]["l"], 1)[:, None], 0)
            else:
                part[slot] = st[m]
    for row, s0, ns in arrays["heavy"].tolist():
        M = np.max([part[s0 + i]["m"] for i in range(ns)], axis=0)
        l = sum(part[s0 + i]["l"] * np.exp(part[s0 + i]["m"] - M) for i in range(ns))
        acc = sum(part[s0 + i]["acc"] * np.exp(part[s0 + i]["m"] - M)[:, None] for i in range(ns))
        o[row] = acc / l[:, None]
    return o


def check_emulated_walks(src, dst, n, csr, pin, gin, gout, xpos):
    """Forward walk over the destination-side groups, backward walks over both sides, against the oracle."""
    GROUP_R = gin["R"]
    assert gout["R"] == GROUP_R
    rng = np.random.default_rng(0)
    h, d = 2, 8
    q, k, v, do = (rng.standard_normal((n, h, d)) / 2 for _ in range(4))
    ro, ra = oracle.attention_forward(csr, q, k, v)
    o = emulate_forward(pin, gin, q, k, v, 1 / np.sqrt(d))
    assert np.allclose(o, ro, rtol=1e-10, atol=1e-12)
    # backward walk: destination side writes (p, ds) at the source side's pair numbers, source side reads them in order
    spare = (len(gout["entries"]) + GROUP_PAD_ENTRIES) * GROUP_R - 1
    assert len(xpos) == (len(gin["entries"]) + GROUP_PAD_ENTRIES) * GROUP_R and np.all(xpos[len(gin["entries"]) * GROUP_R:] == spare)
    assert np.all(xpos[:len(gin["entries"]) * GROUP_R][gin["slot_eid"].reshape(-1) < 0] == spare)
    rdq, rdk, rdv = oracle.attention_backward(csr, q, k, v, ra, do)
    scale = 1 / np.sqrt(d)
    delta = (do * ro).sum(-1)
    # log-sum-exp per (node, head) from the oracle's probabilities: p = exp(s*scale - lse)
    lse = np.zeros((n, h)); z = np.zeros((n, h)); mrow = np.full((n, h), -np.inf)
    sc = (k[src] * q[dst]).sum(-1) * scale
    np.maximum.at(mrow, dst, sc)
    np.add.at(z, dst, np.exp(sc - mrow[dst]))
    has = z > 0
    lse[has] = mrow[has] + np.log(z[has])
    pds = np.full((len(gout["entries"]) * GROUP_R, h, 2), np.nan)     # scratch indexed by source-side (entry, member)
    dq = np.zeros_like(q)
    for g in range(len(gin["members"])):
        for u in range(gin["grp_ptr"][g], gin["grp_ptr"][g + 1]):
            idx, mask, _, _ = gin["entries"][u].tolist()
            for m in range(GROUP_R):
                if mask >> m & 1:
                    row = gin["members"][g, m, 0]
                    p = np.exp((q[row] * k[idx]).sum(-1) * scale - lse[row])
                    ds = p * ((do[row] * v[idx]).sum(-1) - delta[row]) * scale
                    dq[row] += ds[:, None] * k[idx]
                    t = xpos[u * GROUP_R + m]
                    assert np.isnan(pds[t]).all()                      # every position written once
                    pds[t, :, 0] = p; pds[t, :, 1] = ds
    assert np.isnan(pds[:, 0, 0]).sum() == len(pds) - len(src) and np.allclose(dq, rdq, rtol=1e-9, atol=1e-12)
    dk = np.zeros_like(k); dv = np.zeros_like(v)
    for g in range(len(gout["members"])):
        for u in range(gout["grp_ptr"][g], gout["grp_ptr"][g + 1]):
            idx, mask, _, _ = gout["entries"][u].tolist()
            for m in range(GROUP_R):
                if mask >> m & 1:
                    row = gout["members"][g, m, 0]
                    dk[row] += pds[u * GROUP_R + m, :, 1][:, None] * q[idx]
                    dv[row] += pds[u * GROUP_R + m, :, 0][:, None] * do[idx]
    assert np.allclose(dk, rdk, rtol=1e-9, atol=1e-12) and np.allclose(dv, rdv, rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("name,seg", [("bpt64c", 64), ("bpt37", 8), ("multi", 8), ("bpt300c", 64)])
def test_emulated_group_walk_matches_oracle(name, seg):
    src, dst, n, csr, pin, pout = plans(name, seg)
    gin, gout = build_groups_host(pin, n), build_groups_host(pout, n)
    check_emulated_walks(src, dst, n, csr, pin, gin, gout, link_groups_host(gin, gout, len(src)))


def test_grouping_reduces_row_loads_on_the_headline_graph():
    src, dst, n = bpt(8192, True, 4)
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n, as_torch=False)
    pin, _ = build_plan_host(COL, IC, in_csr[2], in_csr[1], n, n)
    pout, _ = build_plan_host(ROW, IR, out_csr[2], out_csr[1], n, n)
    for arrays in (pin, pout):
        g16 = build_groups_host(arrays, n, R=16)
        assert len(g16["entries"]) < 0.18 * len(src)        # neighbour-row fetches per kernel vs one per edge
        assert len(g16["members"]) < 0.08 * len(arrays["items"])
        grp = build_groups_host(arrays, n, R=4)
        assert len(grp["entries"]) < 0.42 * len(src)
        # XCD chunks carry about equal work (pairs)
        pc = np.array([bin(m).count("1") for m in grp["entries"][:, 1]])
        cum = np.concatenate([[0], np.cumsum(pc)])
        ch = grp["chunks"]
        per = [cum[grp["grp_ptr"][ch[x + 1]]] - cum[grp["grp_ptr"][ch[x]]] for x in range(8)]
        assert max(per) < 1.10 * min(per)      # balanced on pairs + a fixed cost per group


def test_link_groups_rejects_incomplete_source_side():
    """bptg_link_groups: the source-side groups must hold every edge exactly once."""
    src, dst, n, csr, pin, pout = plans(sorted(GRAPHS)[0], 64)
    gd = build_groups_host(pin, n, R=4)
    gs = build_groups_host(pout, n, R=4)
    pairs = link_groups_host(gd, gs, len(src))
    assert pairs.dtype == np.int32 and len(pairs) == (len(gd["entries"]) + 8) * 4
    broken = dict(gs)
    broken["slot_eid"] = gs["slot_eid"].copy()
    r, c = np.argwhere(broken["slot_eid"] >= 0)[0]
    broken["slot_eid"][r, c] = -1                      # one edge missing
    with pytest.raises(ValueError):
        link_groups_host(gd, broken, len(src))
