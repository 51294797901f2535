"""Plans built on the GPU (libbptplan): bit for bit against the numpy model of the same construction (and, for the
base plan, against the host builder), rejection of malformed arrays without a fault, and the attention kernels
running on such plans against the oracle."""
import numpy as np
import pytest
import torch

import oracle
import parallel_plan_model as model
from test_gpu_parity import GTOL, TOL, Case, close, f64, rand

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _graphs():
    from bpt_amd import graphbuilder as gb

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

    def batch():
        parts = [bpt(L, True, 4) for L in (171, 99, 260, 64)]
        shift, srcs, dsts = 0, [], []
        for s, d, n in parts:
            srcs.append(s + shift); dsts.append(d + shift); shift += n
        return np.concatenate(srcs), np.concatenate(dsts), shift

    return {"bpt64c": lambda: bpt(64, True, 4), "bpt37": lambda: bpt(37, False, 2), "bpt300c": lambda: bpt(300, True, 2),
            "multi": multigraph, "bpt1": lambda: bpt(1, False, 1), "bpt2048c": lambda: bpt(2048, True, 4), "batch": batch}


GRAPHS = _graphs()
_cache = {}


def sides(name):
    """(src, dst, n, csr, host arrays of the in side, of the out side, the same as device tensors)."""
    if name not in _cache:
        from bpt_amd import graphbuilder as gb
        src, dst, n = GRAPHS[name]()
        csr = gb.get_csrs(src, dst, n, as_torch=False)
        out_csr, in_csr, ROW, IR, COL, IC = csr
        a_in, a_out = (COL, IC, in_csr[2], in_csr[1]), (ROW, IR, out_csr[2], out_csr[1])
        t = lambda arrs: tuple(torch.from_numpy(a).to(DEV) for a in arrs)
        _cache[name] = (src, dst, n, csr, a_in, a_out, t(a_in), t(a_out))
    return _cache[name]


def host(t):
    return t.cpu().numpy()


def check_base(dp, arrays, info):
    d = dp._dev
    assert (dp.n_items, dp.n_heavy, dp.n_slots, dp.max_degree, dp.covers_all_edges) == \
           (info["n_items"], info["n_heavy"], info["n_slots"], info["max_degree"], info["perm"])
    assert np.array_equal(host(d["rowptr"]), arrays["rowptr"])
    E = len(arrays["eid"])
    assert np.array_equal(host(d["idx"])[:E], arrays["idx"]) and np.array_equal(host(d["eid"])[:E], arrays["eid"])
    assert np.array_equal(host(d["items"])[:dp.n_items], arrays["items"])
    assert np.array_equal(host(d["heavy"])[:dp.n_heavy], arrays["heavy"])


def check_groups(hit, grp, n_edges):
    from bpt_amd.plan import GROUP_PAD_ENTRIES
    st, dev, R = hit["struct"], hit["dev"], grp["R"]
    ng, ne = len(grp["members"]), len(grp["entries"])
    assert (st.n_groups, st.n_grp_entries, st.grp_R) == (ng, ne, R)
    assert st.grp_max_chunk == (int(np.diff(grp["chunks"]).max()) if ng else 0)
    assert np.array_equal(host(dev["chunks"]), grp["chunks"])
    assert np.array_equal(host(dev["members"]), grp["members"])
    assert np.array_equal(host(dev["grp_ptr"]), grp["grp_ptr"])
    ent = host(dev["entries"])
    assert np.array_equal(ent[:ne], grp["entries"]) and np.all(ent[ne] == 0)
    assert np.array_equal(host(dev["pair_eid"])[:n_edges], grp["pair_eid"])
    eids = host(dev["eids"])
    want = np.full((ne + GROUP_PAD_ENTRIES, R), n_edges, dtype=np.int32)
    want[:ne] = np.where(grp["slot_eid"] >= 0, grp["slot_eid"], n_edges)
    assert np.array_equal(eids, want.reshape(-1))


@pytest.mark.parametrize("seg", [8, 64])
@pytest.mark.parametrize("name", sorted(GRAPHS))
def test_device_plan_equals_model_and_host(name, seg):
    from bpt_amd.plan import GROUP_ORDER_SRC, GROUP_PAD_ENTRIES, DevicePlan, build_plan_host
    src, dst, n, csr, a_in, a_out, t_in, t_out = sides(name)
    plans = []
    for arrs, tens in ((a_in, t_in), (a_out, t_out)):
        dp = DevicePlan(*tens, n, n, DEV, seg)
        arrays, info = model.base_plan(*arrs, n, n, seg)
        check_base(dp, arrays, info)
        harr, _ = build_plan_host(*arrs, n, n, seg)
        assert np.array_equal(host(dp._dev["items"])[:dp.n_items], harr["items"])       # and the host builder's
        plans.append((dp, arrays))
    for R in (4, 8, 16):
        grps = []
        for (dp, arrays), by_mask in zip(plans, (1, 2) if R != 16 else (0, 5)):       # (5: entries by mask, groups in locality order)
            hit = dp.ensure_groups(R, {0: 2, 1: 6, 2: 10, 5: 4}[by_mask])
            grp = model.group_plan(arrays, n, R, by_mask)
            check_groups(hit, grp, len(src))
            grps.append(grp)
        if R != 16:
            st = plans[0][0].linked_to(plans[1][0], R)
            want = model.link_groups(grps[0], grps[1], len(src), GROUP_PAD_ENTRIES)
            got = host(plans[0][0]._links[(id(plans[1][0]), R, None, GROUP_ORDER_SRC)][1])
            assert np.array_equal(got, want) and st.grp_pairs
        else:
            # the tile kernels link the other way round: source side -> destination side, both in the default order
            grps = [model.group_plan(arrays, n, R, 1) for dp, arrays in plans]
            st = plans[1][0].linked_to(plans[0][0], R, partner_order=None)
            want = model.link_groups(grps[1], grps[0], len(src), GROUP_PAD_ENTRIES)
            got = host(plans[1][0]._links[(id(plans[0][0]), R, None, None)][1])
            assert np.array_equal(got, want) and st.grp_pairs
            # ... and by pair numbers (what the tile kernels' scratch is indexed by): the number of the same edge's pair
            # on the destination side, from the model's own pair lists
            from bpt_amd.plan import pair_numbers_host
            st = plans[1][0].linked_to(plans[0][0], R, partner_order=None, pair_numbers=True)
            got = host(plans[1][0]._links[(id(plans[0][0]), R, None, None, True)][1])
            want = pair_numbers_host(grps[1], grps[0], len(src))
            assert np.array_equal(got, want) and st.grp_pairs
            number = {int(e): i for i, e in enumerate(grps[0]["pair_eid"])}
            se = np.asarray(grps[1]["slot_eid"]).reshape(-1)
            assert all(want[i] == number[int(e)] for i, e in enumerate(se) if e >= 0) and not want[len(se):].any()


def test_device_plan_without_indices_and_with_uncovered_slots():
    """Plans of the ops that take no indices keep the row order; units that leave edge slots out give a plan that
    is valid for the per-row kernels and has no groups."""
    from bpt_amd.plan import DevicePlan
    src, dst, n, csr, a_in, a_out, t_in, t_out = sides("bpt37")
    dp = DevicePlan(t_in[0], t_in[1], t_in[2], None, n, n, DEV, 8)
    arrays, info = model.base_plan(a_in[0], a_in[1], a_in[2], None, n, n, 8)
    rowsorted = arrays["items"][np.argsort(arrays["items"][:, 1], kind="stable")]       # the model always sorts by locality
    assert np.array_equal(host(dp._dev["items"])[:dp.n_items][:, :3], rowsorted[:, :3])
    # drop the last unit: the slots it covered belong to no row any more
    row, ip = a_in[0][:-1], a_in[1][:-1]
    dp = DevicePlan(torch.from_numpy(row).to(DEV), torch.from_numpy(ip).to(DEV), t_in[2], t_in[3], n, n, DEV, 8)
    arrays, info = model.base_plan(row, ip, a_in[2], a_in[3], n, n, 8)
    assert not dp.covers_all_edges and not info["perm"]
    check_base(dp, arrays, info)
    assert dp.ensure_groups(4)["struct"].n_groups == 0


def test_device_plan_rejects_malformed_arrays():
    from bpt_amd.plan import DevicePlan
    src, dst, n, csr, a_in, a_out, t_in, t_out = sides("bpt64c")
    row, ip, eid, idx = (t.clone() for t in t_in)
    bad = idx.clone(); bad[5] = n
    with pytest.raises(ValueError, match="out of range"):
        DevicePlan(row, ip, eid, bad, n, n, DEV, 64)
    bad = idx.clone(); bad[7] = -1
    with pytest.raises(ValueError, match="out of range"):
        DevicePlan(row, ip, eid, bad, n, n, DEV, 64)
    bad = eid.clone(); bad[0] = len(eid)
    with pytest.raises(ValueError, match="out of range"):
        DevicePlan(row, ip, bad, idx, n, n, DEV, 64)
    bad = row.clone(); bad[3], bad[4] = row[4] + 1, row[3]
    with pytest.raises(ValueError, match="not sorted"):
        DevicePlan(bad, ip, eid, idx, n, n, DEV, 64)
    bad = ip.clone(); bad[2] = bad[3] + 1
    with pytest.raises(ValueError, match="not sorted"):
        DevicePlan(row, bad, eid, idx, n, n, DEV, 64)
    bad = row.clone(); bad[-1] = n
    with pytest.raises(ValueError, match="out of range"):
        DevicePlan(bad, ip, eid, idx, n, n, DEV, 64)
    # a repeated edge id is no error, but such a plan gets no groups (as on the host)
    dup = eid.clone(); dup[1] = dup[0]
    dp = DevicePlan(row, ip, dup, idx, n, n, DEV, 64)
    assert not dp.covers_all_edges and dp.ensure_groups(4)["struct"].n_groups == 0
    torch.cuda.synchronize()


@pytest.fixture
def device_plans():
    from bpt_amd import plan
    plan.plan_cache.clear()
    old = plan.set_device_build(True)
    yield plan
    plan.set_device_build(old)
    plan.plan_cache.clear()


@pytest.mark.parametrize("R", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gname", ["bpt512_k4", "bpt300_causal_k2", "multigraph", "fc_w100"])
def test_fused_attention_on_device_plans_matches_oracle(device_plans, gname, dtype, R):
    from bpt_amd import graphop
    c = Case(gname)
    h, d = 8, 64
    q, k, v, do = (rand((c.n, h, d), dtype, s, 0.125) for s in range(4))
    old = graphop.set_group_rows(R)
    try:
        qd, kd, vd, dod = (x.to(DEV) for x in (q, k, v, do))
        o, lse = graphop.attention_forward(*c.inn, qd, kd, vd)
        dq, dk, dv = graphop.attention_backward(*c.out, *c.inn, qd, kd, vd, o, lse, dod)
        torch.cuda.synchronize()
        assert isinstance(device_plans.plan_cache.get(*c.inn, c.n, c.n), device_plans.DevicePlan)
    finally:
        graphop.set_group_rows(old)
    ro, ra = oracle.attention_forward(c.csr, f64(q), f64(k), f64(v))
    rdq, rdk, rdv = oracle.attention_backward(c.csr, f64(q), f64(k), f64(v), ra, f64(do))
    close(o, ro, TOL[dtype], "o")
    for got, want, nm in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv")):
        close(got, want, GTOL[dtype], nm)


def test_ops_and_rel_pos_on_device_plans_match_host_plans(device_plans):
    """The unfused ops and the fused path with rel_pos and dropout give the same results on device-built plans as on
    host-built ones: edge outputs bit for bit (a dot product or a row's softmax does not depend on the grouping), row
    sums up to their order of summation."""
    from bpt_amd import graphop, op, plan
    c = Case("bpt512_k4")
    h, d = 8, 64
    q, k, v = (rand((c.n, h, d), torch.float32, s, 0.125).to(DEV) for s in range(3))
    table = rand((30, d), torch.float32, 7, 0.125).to(DEV)
    etype = torch.from_numpy(np.random.default_rng(0).integers(0, 30, c.E)).to(DEV)

    def run():
        e = graphop.maskedmm_csr_forward(*c.out, k, q)
        a = graphop.sparse_softmax_forward(*c.inn[:3], e)
        y = graphop.vector_spmm_forward(*c.inn, a, v)
        qq, kk, vv, tt = (x.clone().requires_grad_(True) for x in (q, k, v, table))
        o = op.bpt_attention(*c.out, *c.inn, qq, kk, vv, rel_table=tt, etype=etype)
        o.sum().backward()
        od = op.bpt_attention(*c.out, *c.inn, q, k, v, dropout_p=0.2, seed=5)      # the mask is keyed by edge id, not by the plan
        torch.cuda.synchronize()
        return e, a, y, o.detach(), qq.grad, kk.grad, vv.grad, tt.grad, od

    dev = run()
    assert isinstance(plan.plan_cache.get(*c.inn, c.n, c.n), plan.DevicePlan)
    plan.set_device_build(False)
    plan.plan_cache.clear()
    hst = run()
    assert isinstance(plan.plan_cache.get(*c.inn, c.n, c.n), plan.Plan)
    for i in range(2):
        assert torch.equal(dev[i], hst[i])
    for got, want in zip(dev[2:], hst[2:]):
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)


def test_device_plan_at_headline_size_and_its_build_time():
    """cfg 3 (L = 8192, k = 4, causal): the device-built plans equal the model, and the kernels accept them."""
    import time
    from bpt_amd import graphbuilder as gb
    from bpt_amd.plan import DevicePlan
    g = gb.BinaryPartition(8192, True, 4, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n, as_torch=False)
    a_in, a_out = (COL, IC, in_csr[2], in_csr[1]), (ROW, IR, out_csr[2], out_csr[1])
    t_in, t_out = (tuple(torch.from_numpy(a).to(DEV) for a in arrs) for arrs in (a_in, a_out))
    for rep in range(2):                                   # the second pass is warm
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pin, pout = DevicePlan(*t_in, n, n, DEV), DevicePlan(*t_out, n, n, DEV)
        pin.linked_to(pout, 8)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    print(f"device plan build (both sides, groups of 8, pair mapping) at cfg 3: {dt * 1e3:.2f} ms")
    for dp, arrs, by_mask in ((pin, a_in, 1), (pout, a_out, 2)):
        arrays, info = model.base_plan(*arrs, n, n, 64)
        check_base(dp, arrays, info)
        check_groups(dp.ensure_groups(8, {0: 2, 1: 6, 2: 10}[by_mask]), model.group_plan(arrays, n, 8, by_mask), len(src))


@pytest.mark.parametrize("chunk", [4, 32])
@pytest.mark.parametrize("name", sorted(GRAPHS))
def test_device_csr_equals_host_csr(name, chunk):
    """get_csrs_device: bit for bit the arrays of get_csrs (the layout of graph/base.py:71-86 + partition_csr)."""
    from bpt_amd import graphbuilder as gb
    src, dst, n = GRAPHS[name]()
    want = gb.get_csrs(src, dst, n, chunk_size=chunk, as_torch=False)
    got = gb.get_csrs_device(torch.from_numpy(src).to(DEV), torch.from_numpy(dst).to(DEV), n, chunk_size=chunk)
    for side in (0, 1):
        for a, b in zip(got[side], want[side]):
            assert a.dtype == torch.int64 and np.array_equal(host(a), b)
    for a, b in zip(got[2:], want[2:]):
        assert a.dtype == torch.int64 and np.array_equal(host(a), b)


def test_device_csr_edge_cases():
    from bpt_amd import graphbuilder as gb
    e = torch.empty(0, dtype=torch.int64, device=DEV)
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs_device(e, e, 5)
    assert host(out_csr[0]).tolist() == [0] * 6 and ROW.numel() == 0 and host(IR).tolist() == [0]
    bad = torch.tensor([0, 7], dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError, match="out of range"):
        gb.get_csrs_device(bad, torch.zeros_like(bad), 5)
    with pytest.raises(ValueError):
        gb.get_csrs_device(bad.cpu(), bad.cpu(), 9)
    torch.cuda.synchronize()


def test_edge_list_to_attention_without_leaving_the_gpu(device_plans):
    """Edge list on the device -> CSRs -> plans -> fused attention forward and backward, against the oracle."""
    from bpt_amd import graphbuilder as gb, graphop
    src, dst, n = GRAPHS["batch"]()
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs_device(torch.from_numpy(src).to(DEV), torch.from_numpy(dst).to(DEV), n)
    h, d = 8, 64
    q, k, v, do = (rand((n, h, d), torch.float32, s, 0.125) for s in range(4))
    qd, kd, vd, dod = (x.to(DEV) for x in (q, k, v, do))
    inn, out = (COL, IC, in_csr[2], in_csr[1]), (ROW, IR, out_csr[2], out_csr[1])
    o, lse = graphop.attention_forward(*inn, qd, kd, vd)
    dq, dk, dv = graphop.attention_backward(*out, *inn, qd, kd, vd, o, lse, dod)
    torch.cuda.synchronize()
    csr = gb.get_csrs(src, dst, n, as_torch=False)
    ro, ra = oracle.attention_forward(csr, f64(q), f64(k), f64(v))
    rdq, rdk, rdv = oracle.attention_backward(csr, f64(q), f64(k), f64(v), ra, f64(do))
    close(o, ro, TOL[torch.float32], "o")
    deg = int(max(np.bincount(src, minlength=n).max(), np.bincount(dst, minlength=n).max()))
    for got, want, nm in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv")):
        close(got, want, GTOL[torch.float32], nm)


@pytest.mark.parametrize("seed", range(12))
def test_device_plan_on_random_graphs(seed):
    """Seeded random multigraphs (empty rows, rows longer than a segment, repeated edges, more index nodes than rows):
    CSR, base plan, groups and pair mapping equal the host builders / the model."""
    from bpt_amd import graphbuilder as gb
    from bpt_amd.plan import GROUP_ORDER_SRC, GROUP_PAD_ENTRIES, DevicePlan
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(1, 300))
    E = int(rng.integers(0, 4000))
    hot = rng.integers(0, n, 3)
    src = np.where(rng.random(E) < 0.3, hot[rng.integers(0, 3, E)], rng.integers(0, n, E)).astype(np.int64)
    dst = np.where(rng.random(E) < 0.3, hot[rng.integers(0, 3, E)], rng.integers(0, max(n // 2, 1), E)).astype(np.int64)
    if E > 10:
        src[-5:], dst[-5:] = src[-6], dst[-6]                        # one edge six times
    seg, R, chunk = int(rng.choice([4, 16, 64])), int(rng.choice([4, 8, 16])), int(rng.choice([3, 32]))
    want = gb.get_csrs(src, dst, n, chunk_size=chunk, as_torch=False)
    got = gb.get_csrs_device(torch.from_numpy(src).to(DEV), torch.from_numpy(dst).to(DEV), n, chunk_size=chunk)
    for a, b in zip((*got[0], *got[1], *got[2:]), (*want[0], *want[1], *want[2:])):
        assert np.array_equal(host(a), b)
    out_csr, in_csr, ROW, IR, COL, IC = got
    w_out, w_in = want[0], want[1]
    sides_ = (((COL, IC, in_csr[2], in_csr[1]), (want[4], want[5], w_in[2], w_in[1]), 1),
              ((ROW, IR, out_csr[2], out_csr[1]), (want[2], want[3], w_out[2], w_out[1]), 2))
    plans, grps = [], []
    for tens, arrs, by_mask in sides_:
        dp = DevicePlan(*tens, n, n, DEV, seg)
        arrays, info = model.base_plan(*arrs, n, n, seg)
        check_base(dp, arrays, info)
        grp = model.group_plan(arrays, n, R, by_mask)
        check_groups(dp.ensure_groups(R, {0: 2, 1: 6, 2: 10}[by_mask]), grp, E)
        plans.append(dp); grps.append(grp)
    plans[0].linked_to(plans[1], R)
    assert np.array_equal(host(plans[0]._links[(id(plans[1]), R, None, GROUP_ORDER_SRC)][1]),
                          model.link_groups(grps[0], grps[1], E, GROUP_PAD_ENTRIES))


def test_batch_merge_on_the_device_and_the_whole_pipeline_time():
    """merge_graphs_device equals merge_graphs; and what a new batch costs from its lengths to plans that the fused
    kernels can run on, on the host and on the GPU (benchmark configuration 2: 32 sequences, causal, k = 4)."""
    import time
    from bpt_amd import graphbuilder as gb, plan
    lengths = np.random.default_rng(2345).integers(64, 1025, 32)
    graphs = [gb.BinaryPartition(int(L), True, 4, 10) for L in lengths]
    want = gb.merge_graphs(graphs)
    got = gb.merge_graphs_device(graphs, DEV)
    for a, b in zip(got[:4], want[:4]):
        assert np.array_equal(host(a), b)
    assert got[4] == want[4] == 33598 and len(want[0]) == 573520

    def on_host():
        src, dst, et, pos, n = gb.merge_graphs(graphs)
        out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n)
        t = [x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1])]
        pin, pout = plan.Plan(*t[4:], n, n, DEV), plan.Plan(*t[:4], n, n, DEV)
        pin.linked_to(pout, 8)
        return pin, pout

    def on_device():
        src, dst, et, pos, n = gb.merge_graphs_device(graphs, DEV)
        out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs_device(src, dst, n)
        pin = plan.DevicePlan(COL, IC, in_csr[2], in_csr[1], n, n, DEV)
        pout = plan.DevicePlan(ROW, IR, out_csr[2], out_csr[1], n, n, DEV)
        pin.linked_to(pout, 8)
        return pin, pout

    times = {}
    for name, fn in (("host", on_host), ("device", on_device)):
        best = 1e9
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            pin, pout = fn()
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        times[name] = best
        assert pin.n_edges == 573520 and pin.covers_all_edges and pout.covers_all_edges
    print(f"lengths -> plans with groups of 8 (cfg 2): host {times['host'] * 1e3:.1f} ms, device {times['device'] * 1e3:.2f} ms")
    # (the two timings are reported, not asserted: a busy host or a cold first launch says nothing about the code)


def test_device_graph_builder_equals_host_builder():
    """Edge lists built on the GPU, bit for bit those of the host builder (itself pinned by the reference's own
    module through tests/golden): all three graph kinds, causal and not, odd sizes, shifts."""
    from bpt_amd import graphbuilder as gb
    graphs = [gb.BinaryPartition(L, triu, step, clip) for L in (1, 2, 3, 5, 6, 7, 13, 33, 100, 511, 512, 1000)
              for triu in (False, True) for step, clip in ((1, 10), (2, 3), (4, 10))]
    graphs += [gb.BinaryPartition(8192, True, 4, 10), gb.BinaryPartition(4097, False, 8, 2), gb.BinaryPartition(32768, True, 8, 10)]
    graphs += [gb.FullyConnected(L, triu, w) for L in (1, 2, 17, 260) for triu in (False, True) for w in (0, 1, 5, 8192)]
    graphs += [gb.OpenAISparse(L, stride, c) for L, stride, c in ((1, 4, 2), (50, 8, 3), (257, 16, 16), (64, 64, 0))]
    for i, g in enumerate(graphs):
        shift = 7 * (i % 3)
        want = g.get_edges(v_shift=shift)
        got = g.get_edges_device(DEV, v_shift=shift)
        for a, b in zip(got, want):
            assert a.dtype == torch.int64 and np.array_equal(host(a), b), (type(g).__name__, g.__reduce__()[1])


@pytest.mark.parametrize("device_side", ["in", "out"])
def test_one_side_planned_on_the_gpu_and_the_other_on_the_host(device_side):
    """The two CSR sides of a graph can be planned in different places (a bipartite graph whose sides fall on either
    side of the size rule): the pair mapping and the backward pass still work."""
    from bpt_amd import graphop, plan
    c = Case("bpt300_causal_k2")
    h, d = 8, 64
    q, k, v, do = (rand((c.n, h, d), torch.float32, s, 0.125).to(DEV) for s in range(4))
    plan.plan_cache.clear()
    old = plan.set_device_build(device_side == "in")
    try:
        p_in = plan.plan_cache.get(*c.inn, c.n, c.n)
        plan.set_device_build(device_side != "in")
        p_out = plan.plan_cache.get(*c.out, c.n, c.n)
        assert isinstance(p_in, plan.DevicePlan) != isinstance(p_out, plan.DevicePlan)
        # the cache key carries the setting: look the plans up under the setting they were built with
        plan.set_device_build(device_side == "in")
        o, lse = graphop.attention_forward(*c.inn, q, k, v)
        st = p_in.linked_to(p_out, 4)
        assert st.grp_pairs
        import ctypes
        from bpt_amd._lib import attn_lib
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        out_st = p_out.ensure_groups(4, plan.GROUP_ORDER_SRC)["struct"]
        lib = attn_lib()
        nws = lib.bpt_workspace_bytes(6, ctypes.byref(st), ctypes.byref(out_st), h, d, 0)
        ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
        status = lib.bpt_attention_backward(ctypes.byref(st), ctypes.byref(out_st), q.data_ptr(), k.data_ptr(), v.data_ptr(), None,
                                            o.data_ptr(), do.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                            None, ws.data_ptr(), nws, 0.125, 0.0, 0, h, d, 0, torch.cuda.current_stream().cuda_stream)
        assert status == 0
        torch.cuda.synchronize()
    finally:
        plan.set_device_build(old)
        plan.plan_cache.clear()
    ro, ra = oracle.attention_forward(c.csr, f64(q), f64(k), f64(v))
    rdq, rdk, rdv = oracle.attention_backward(c.csr, f64(q), f64(k), f64(v), ra, f64(do))
    close(o, ro, TOL[torch.float32], "o")
    for got, want, nm in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv")):
        close(got, want, GTOL[torch.float32], nm)
