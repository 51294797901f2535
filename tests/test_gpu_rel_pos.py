"""GPU parity of the rel_pos score term's own kernels (modules/attention.py:55-56,69-71: embed_ak looked up per edge, then
node_mul_edge, and their autograd) against the CPU oracle's node_mul_edge on the looked-up rows.

Tolerances as everywhere: fp32 outputs rtol 1e-5 / atol 1e-5, fp32 gradients rtol 1e-4, bf16 2e-2.  The oracle runs in
float64 on the same float32 / bf16 input values.
"""
import numpy as np
import pytest
import torch

import oracle
from test_gpu_parity import DEV, GTOL, TOL, case, close, f64, rand

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from bpt_amd import graphop, op
    return graphop, op


def edge_types(E, n_types, n_used, seed):
    """E edge types out of n_types of which exactly min(n_used, E) occur, scattered over the range."""
    rng = np.random.default_rng(seed)
    pool = np.sort(rng.choice(n_types, size=min(n_used, n_types), replace=False))
    et = pool[rng.integers(0, len(pool), E)]
    m = min(len(pool), E)
    et[rng.permutation(E)[:m]] = pool[:m]                # every type of the pool occurs
    return et.astype(np.int64)


def used_map(etype_slot, n_types, seed=None):
    """(used, used_types, number_slot): the types that occur (ascending, or shuffled with `seed`: any order is allowed),
    the number of every type in that list (-1: does not occur) and the number of every slot's type."""
    used_types = np.unique(etype_slot).astype(np.int32)
    if seed is not None:
        used_types = np.random.default_rng(seed).permutation(used_types)
    used = np.full(n_types, -1, dtype=np.int32)
    used[used_types] = np.arange(len(used_types), dtype=np.int32)
    return used, used_types, used[etype_slot].astype(np.int64)


def dev(a):
    return torch.from_numpy(a).to(DEV)


SHAPES = [(torch.float32, 8), (torch.float32, 4), (torch.float32, 16), (torch.bfloat16, 8), (torch.bfloat16, 16)]
GRAPH_NAMES = ["bpt512_k4", "bpt300_causal_k2", "multigraph", "fc_w100", "blocks8x30"]


def _score_cases():
    """Every graph and shape with the table rows on chip; the kernel that gathers them by type on two graphs."""
    return [(g, dt, h, True) for g in GRAPH_NAMES for dt, h in SHAPES] + \
           [(g, dt, h, False) for g in ("bpt512_k4", "multigraph") for dt, h in SHAPES]


@pytest.mark.parametrize("gname,dtype,h,on_chip", _score_cases())
def test_score_term_matches_node_mul_edge_of_the_looked_up_rows(ops, gname, dtype, h, on_chip):
    """on_chip: the kernel that keeps the table rows in use in LDS (plan indices = type numbers); otherwise the one that
    gathers table rows by type."""
    graphop, _ = ops
    d, n_types = 64, 1000
    c = case(gname)
    q = rand((c.n, h, d), dtype, 11, 0.5).to(DEV)
    table = rand((n_types, d), dtype, 12, 0.5).to(DEV)
    et = edge_types(c.E, n_types, 55, 13)
    etype_slot = et[c.np_in[2]]
    if on_chip:
        used, used_types, number_slot = used_map(etype_slot, n_types, seed=14)
        bias = graphop.rel_bias_forward(*c.inn[:3], dev(number_slot), q, table, used_types=dev(used_types))
    else:
        bias = graphop.rel_bias_forward(*c.inn[:3], dev(etype_slot), q, table)
    assert bias.shape == (c.E + 1, h) and bias.dtype == torch.float32
    want = oracle.node_mul_edge_forward(*c.np_in[:3], f64(q), f64(table)[et])
    close(bias[:c.E], want, TOL[dtype], "score term")
    assert float(bias[c.E].abs().max()) == 0.0


def _gradient_cases():
    """55 of 1000 and 37 of 37 types on every graph; 100 and 230 used types (two and one wavefronts per workgroup of the
    kernel instead of four) and a single type on two graphs."""
    return [(g, dt, h, nt, nu) for g in GRAPH_NAMES for dt, h in SHAPES for nt, nu in ((1000, 55), (37, 37))] + \
           [(g, dt, h, nt, nu) for g in ("bpt512_k4", "multigraph") for dt, h in SHAPES for nt, nu in ((1000, 100), (400, 230), (5, 1))]


@pytest.mark.parametrize("gname,dtype,h,n_types,n_used", _gradient_cases())
def test_score_term_gradients_match_node_mul_edge_backward(ops, gname, dtype, h, n_types, n_used):
    """dq gains node_mul_edge's dA, dtable is its dB summed per edge type (the embedding's gradient)."""
    graphop, _ = ops
    d = 64
    c = case(gname)
    q = rand((c.n, h, d), dtype, 21, 0.5).to(DEV)
    table = rand((n_types, d), dtype, 22, 0.5).to(DEV)
    ds = torch.cat([rand((c.E, h), torch.float32, 23, 0.1), torch.zeros(1, h)]).to(DEV)     # (E + 1, h) as the fused backward returns it
    dq0 = rand((c.n, h, d), dtype, 24, 0.5).to(DEV)
    et = edge_types(c.E, n_types, n_used, 25)
    used, used_types, number_slot = used_map(et[c.np_in[2]], n_types, seed=26 if n_used == 55 else None)
    assert len(used_types) == min(n_used, c.E)
    args = (*c.inn[:3], dev(number_slot), dev(used), dev(used_types), ds, q, table)
    dq = dq0.clone()
    dtable = graphop.rel_bias_backward(*args, dq)
    dA, dB = oracle.node_mul_edge_backward(*c.np_in[:3], f64(q), f64(table)[et], f64(ds[:c.E]))
    want_table = np.zeros((n_types, d))
    np.add.at(want_table, et, dB)
    # both are raw sums of unnormalised N(0, 0.1) x N(0, 0.5) products: max_deg terms for a row of dq (on top of dq0), h * E / n_used
    # for a row of the table (terms)
    close(dq, f64(dq0) + dA, GTOL[dtype], "dq", c.max_deg)
    close(dtable, want_table, GTOL[dtype], "dtable", h * c.E / max(len(used_types), 1))
    again = graphop.rel_bias_backward(*args, dq0.clone())
    assert torch.equal(again, dtable), "the sums have a fixed order: the same bits every run"


@pytest.mark.parametrize("dtype,h", SHAPES)
@pytest.mark.parametrize("gname", ["bpt512_k4", "multigraph", "fc_w100"])
def test_head_major_form_of_the_score_term_kernels(ops, gname, dtype, h):
    """by_pair: the term goes to, and its gradient comes from, (h, E) arrays at the places the plan's eid array names (any
    permutation of the edges will do here): the same bits as the (E, h) form, moved."""
    graphop, _ = ops
    d, n_types = 64, 1000
    c = case(gname)
    q = rand((c.n, h, d), dtype, 71, 0.5).to(DEV)
    table = rand((n_types, d), dtype, 72, 0.5).to(DEV)
    et = edge_types(c.E, n_types, 55, 73)
    used, used_types, number_slot = used_map(et[c.np_in[2]], n_types)
    place = torch.from_numpy(np.random.default_rng(74).permutation(c.E)).to(DEV)           # place of edge e
    place_slot = place.index_select(0, c.inn[2]).contiguous()
    tail = (dev(number_slot), q, table)
    by_eid = graphop.rel_bias_forward(*c.inn[:3], *tail, used_types=dev(used_types))
    moved = graphop.rel_bias_forward(*c.inn[:2], place_slot, *tail, used_types=dev(used_types), by_pair=True)
    assert moved.shape == (h, c.E)
    assert torch.equal(moved.t().index_select(0, place), by_eid[:c.E])
    ds = rand((c.E, h), torch.float32, 75, 0.1).to(DEV)
    ds_moved = torch.empty_like(ds).index_copy_(0, place, ds).t().contiguous()
    dq0 = rand((c.n, h, d), dtype, 76, 0.5).to(DEV)
    maps = (dev(number_slot), dev(used), dev(used_types))
    dq_a, dq_b = dq0.clone(), dq0.clone()
    dt_a = graphop.rel_bias_backward(*c.inn[:3], *maps, torch.cat([ds, torch.zeros(1, h, device=DEV)]), q, table, dq_a)
    dt_b = graphop.rel_bias_backward(*c.inn[:2], place_slot, *maps, ds_moved, q, table, dq_b, by_pair=True)
    assert torch.equal(dt_a, dt_b) and torch.equal(dq_a, dq_b)
    with pytest.raises(ValueError, match="used_types"):
        graphop.rel_bias_forward(*c.inn[:2], place_slot, dev(et[c.np_in[2]]), q, table, by_pair=True)


@pytest.mark.parametrize("dtype,h", SHAPES)
@pytest.mark.parametrize("gname,n_types,n_used", [("bpt512_k4", 1000, 55), ("bpt300_causal_k2", 37, 37), ("multigraph", 400, 230),
                                                  ("fc_w100", 1000, 100), ("blocks8x30", 5, 1)])
def test_score_term_over_the_tile_plan(ops, gname, dtype, h, n_types, n_used):
    """rel_bias_forward_tiles: the term in the tiles' pair order, head-major, against node_mul_edge of the looked-up rows."""
    graphop, _ = ops
    d = 64
    c = case(gname)
    q = rand((c.n, h, d), dtype, 81, 0.5).to(DEV)
    table = rand((n_types, d), dtype, 82, 0.5).to(DEV)
    et = edge_types(c.E, n_types, n_used, 83)
    used, used_types, _ = used_map(et, n_types, seed=84)
    pair = graphop.attention_pair_rows(*c.out, *c.inn, q, q)
    member = graphop.attention_pair_members(*c.out, *c.inn, q, q)
    assert pair is not None and member.shape == (c.E,) and member.dtype == torch.int32 and 0 <= int(member.min()) and int(member.max()) < 16
    number_pair = torch.empty(c.E, dtype=torch.int32, device=DEV).index_copy_(0, pair, dev(used[et]))
    bias = graphop.rel_bias_forward_tiles(*c.out, *c.inn, q, q, table, dev(used_types), (number_pair | (member << 8)).contiguous())
    assert bias.shape == (h, c.E) and bias.dtype == torch.float32
    want = oracle.node_mul_edge_forward(*c.np_in[:3], f64(q), f64(table)[et])
    close(bias.t().index_select(0, pair), want, TOL[dtype], "score term")


@pytest.mark.parametrize("gname", ["bpt512_k4", "multigraph"])
def test_layer_with_the_term_is_the_same_on_host_built_and_gpu_built_plans(ops, gname):
    """The pair order and the member index of every pair come from either builder's tile groups (which need not be the same
    groups): the same step within the stated tolerances."""
    from bpt_amd import plan
    _, op = ops
    h, d, n_types = 8, 64, 40
    c = case(gname)
    etype = torch.from_numpy(np.random.default_rng(91).integers(0, n_types, c.E)).to(DEV)
    got = []
    for on_gpu in (False, True):
        plan.plan_cache.clear()
        old = plan.set_device_build(on_gpu)
        try:
            q, k, v, do = (rand((c.n, h, d), torch.float32, s, 1.0 / 8).to(DEV) for s in (92, 93, 94, 95))
            table = rand((n_types, d), torch.float32, 96, 1.0 / 8).to(DEV)
            for t in (q, k, v, table):
                t.requires_grad_(True)
            o = op.bpt_attention(*c.out, *c.inn, q, k, v, rel_table=table, etype=etype)
            o.backward(do)
            got.append((o.detach(), q.grad, k.grad, v.grad, table.grad))
        finally:
            plan.set_device_build(old)
            plan.plan_cache.clear()
    for a, b, what in zip(*got, ("o", "dq", "dk", "dv", "dtable")):
        close(a, f64(b), TOL[torch.float32] if what == "o" else GTOL[torch.float32], what)


def test_layer_falls_back_to_the_in_csr_kernel_where_the_tile_form_is_refused(ops, monkeypatch):
    """BPTRelAttention where rel_bias_forward_tiles reports an unsupported configuration (forced here): the term comes from
    the kernel over the in-CSR, in the same layout, and the step is the same within the stated tolerances."""
    graphop, op = ops
    h, d, n_types = 8, 64, 60
    c = case("bpt512_k4")
    etype = torch.from_numpy(np.random.default_rng(111).integers(0, n_types, c.E)).to(DEV)
    def step():
        q, k, v, do = (rand((c.n, h, d), torch.float32, s, 1.0 / 8).to(DEV) for s in (112, 113, 114, 115))
        table = rand((n_types, d), torch.float32, 116, 1.0 / 8).to(DEV)
        for t in (q, k, v, table):
            t.requires_grad_(True)
        o = op.bpt_attention(*c.out, *c.inn, q, k, v, rel_table=table, etype=etype)
        o.backward(do)
        return o.detach(), q.grad, k.grad, v.grad, table.grad
    want = step()
    calls = []
    def refused(*a, **kw):
        calls.append(1)
        raise graphop.BptStatusError(graphop.BPT_ERR_UNSUPPORTED, "rel_bias_forward_tiles")
    monkeypatch.setattr(graphop, "rel_bias_forward_tiles", refused)
    got = step()
    assert calls, "the tile form was not asked for: the test does not reach the fallback"
    for a, b, what in zip(got, want, ("o", "dq", "dk", "dv", "dtable")):
        close(a, f64(b), TOL[torch.float32] if what == "o" else GTOL[torch.float32], what)


def test_too_many_used_types_is_refused_and_the_layer_takes_the_spmm_form(ops):
    graphop, op = ops
    h, d, n_types = 8, 64, 1000
    c = case("bpt512_k4")
    q, k, v, do = (rand((c.n, h, d), torch.float32, s, 1.0 / 8).to(DEV) for s in (31, 32, 33, 34))
    table = rand((n_types, d), torch.float32, 35, 1.0 / 8).to(DEV)
    et = edge_types(c.E, n_types, 300, 36)
    used, used_types, number_slot = used_map(et[c.np_in[2]], n_types)
    assert len(used_types) == 300 > graphop.REL_MAX_USED_TYPES
    ds = torch.zeros(c.E + 1, h, device=DEV)
    with pytest.raises(RuntimeError, match="status -7"):
        graphop.rel_bias_forward(*c.inn[:3], dev(number_slot), q, table, used_types=dev(used_types))
    with pytest.raises(RuntimeError, match="status -7"):
        graphop.rel_bias_backward(*c.inn[:3], dev(number_slot), dev(used), dev(used_types), ds, q, table, torch.zeros_like(q))
    from oracle import torch_ops
    etype = torch.from_numpy(et).to(DEV)
    for t in (q, k, v, table):
        t.requires_grad_(True)
    o = op.bpt_attention(*c.out, *c.inn, q, k, v, rel_table=table, etype=etype)
    o.backward(do)
    t64 = lambda x: x.detach().cpu().double()
    ro, rdq, rdk, rdv, rdak = torch_ops.attention_fwd_bwd(torch.from_numpy(c.src), torch.from_numpy(c.dst), t64(q), t64(k), t64(v), t64(do),
                                                          ak=t64(table)[etype.cpu()])
    rdt = torch.zeros(n_types, d, dtype=torch.float64).index_add_(0, etype.cpu(), rdak)
    close(o, ro.numpy(), TOL[torch.float32], "o")
    close(q.grad, rdq.numpy(), GTOL[torch.float32], "dq")
    close(table.grad, rdt.numpy(), GTOL[torch.float32], "dtable", h * c.E / 300)


def test_graph_without_edges_gives_a_zero_table_gradient(ops):
    graphop, _ = ops
    h, d, n_types = 8, 64, 12
    i64 = lambda *a: torch.tensor(a, dtype=torch.int64, device=DEV)
    col, indptr, eid, et = i64(), i64(0), i64(), i64()
    q = rand((5, h, d), torch.float32, 41).to(DEV)
    table = rand((n_types, d), torch.float32, 42).to(DEV)
    dq = torch.ones_like(q)
    used = torch.full((n_types,), -1, dtype=torch.int32, device=DEV)
    used_types = torch.zeros(0, dtype=torch.int32, device=DEV)
    dtable = graphop.rel_bias_backward(col, indptr, eid, et, used, used_types, torch.zeros(1, h, device=DEV), q, table, dq)
    assert float(dtable.abs().max()) == 0.0 and torch.equal(dq, torch.ones_like(q))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gname", ["bpt512_k4", "multigraph", "fc_w100"])
@pytest.mark.parametrize("p", [0.0, 0.25])
def test_score_term_in_the_order_of_the_tiles_gives_the_same_step(ops, gname, dtype, p):
    """A score term stored head-major at the tile plan's pair numbers (attention_pair_rows, bias_by_pair) instead of by
    edge id: the same o, lse, dq, dk, dv bit for bit, and ds the same values in the other layout."""
    graphop, _ = ops
    h, d = 8, 64
    c = case(gname)
    q, k, v, do = (rand((c.n, h, d), dtype, s, 1.0 / 8).to(DEV) for s in (51, 52, 53, 54))
    term = rand((c.E, h), torch.float32, 55, 0.5).to(DEV)
    pair = graphop.attention_pair_rows(*c.out, *c.inn, q, k, p)
    assert pair is not None and pair.shape == (c.E,) and torch.equal(torch.sort(pair).values, torch.arange(c.E, device=DEV))
    zero = torch.zeros(1, h, device=DEV)
    by_eid = torch.cat([term, zero])
    by_pair = torch.empty_like(term).index_copy_(0, pair, term).t().contiguous()          # (h, E)
    got = {}
    for name, bias, flag in (("eid", by_eid, False), ("pair", by_pair, True)):
        o, lse = graphop.attention_forward(*c.inn, q, k, v, dropout_p=p, seed=77, bias=bias, bias_by_pair=flag)
        got[name] = (o, lse) + tuple(graphop.attention_backward(*c.out, *c.inn, q, k, v, o, lse, do, dropout_p=p, seed=77, bias=bias,
                                                               bias_by_pair=flag))
    for a, b, what in zip(got["eid"][:5], got["pair"][:5], ("o", "lse", "dq", "dk", "dv")):
        assert torch.equal(a, b), what
    assert got["pair"][5].shape == (h, c.E)
    assert torch.equal(got["eid"][5], got["pair"][5].t().index_select(0, pair)), "ds"


def test_the_order_of_the_tiles_is_offered_only_where_both_passes_run_on_tiles(ops):
    graphop, _ = ops
    c = case("bpt512_k4")
    q, k, v = (rand((c.n, 8, 64), torch.float32, s, 1.0 / 8).to(DEV) for s in (61, 62, 63))
    assert graphop.attention_pair_rows(*c.out, *c.inn, q, k) is not None
    old = graphop.set_group_rows(4)                       # row groups of 4: no tiles
    try:
        assert graphop.attention_pair_rows(*c.out, *c.inn, q, k) is None
        bias = torch.zeros(8, c.E, device=DEV)
        with pytest.raises(RuntimeError, match="bias_by_pair"):
            graphop.attention_forward(*c.inn, q, k, v, bias=bias, bias_by_pair=True)
    finally:
        graphop.set_group_rows(old)
    q32 = rand((c.n, 8, 32), torch.float32, 64, 1.0 / 8).to(DEV)          # 32 columns per head: no tile kernels
    assert graphop.attention_pair_rows(*c.out, *c.inn, q32, q32) is None
