"""Host-side argument checks of the operator surface (bpt_amd/graphop.py): a tensor whose shape does not fit the
graph or the other operands raises ValueError before any plan is built or kernel launched.  Runs without a GPU: the
device check of graphop.cpp:4-6 is switched off and the library handle replaced by one that fails on any call."""
import pytest
import torch

from bpt_amd import graphbuilder as gb


class _NoLaunch:
    def __getattr__(self, name):
        raise AssertionError(f"{name} was called although an argument was malformed")


@pytest.fixture()
def g(monkeypatch):
    from bpt_amd import graphop, plan
    monkeypatch.setattr(graphop, "_check_input", lambda t, name: None)
    monkeypatch.setattr(graphop, "_LIB", _NoLaunch())
    monkeypatch.setattr(plan.plan_cache, "get", lambda *a, **k: (_ for _ in ()).throw(AssertionError("plan requested")))
    return graphop


def _graph():
    b = gb.BinaryPartition(16, True, 2, 10)
    src, dst, _ = b.get_edges()
    n = b.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n)
    return n, len(src), (ROW, IR, out_csr[2], out_csr[1]), (COL, IC, in_csr[2], in_csr[1])


N, E, OUT, INN = _graph()
H, D = 8, 64
node = lambda n=N, h=H, d=D: torch.zeros(n, h, d)
edge = lambda e=E, h=H: torch.zeros(e, h)


def test_maskedmm_checks(g):
    with pytest.raises(ValueError):
        g.maskedmm_csr_forward(*OUT, node(), node(h=4))                       # B has other heads
    with pytest.raises(ValueError):
        g.maskedmm_csr_forward(*OUT, node(), node(d=32))                      # B has another head size
    with pytest.raises(ValueError):
        g.maskedmm_csr_forward(OUT[0], OUT[1], OUT[2], OUT[3][:-1], node(), node())   # indices shorter than eid
    with pytest.raises(ValueError):
        g.maskedmm_csr_backward(*OUT, *INN, node(), node(), edge(e=E - 1))    # dy misses an edge
    with pytest.raises(ValueError):
        g.maskedmm_csr_backward(*OUT, *INN, node(), node(), edge(h=4))
    with pytest.raises(ValueError):
        g.maskedmm_csr_backward(*OUT, INN[0], INN[1], INN[2][:-1], INN[3][:-1], node(), node(), edge())


def test_node_mul_edge_checks(g):
    with pytest.raises(ValueError):
        g.node_mul_edge_forward(*INN[:3], node(), torch.zeros(E - 1, D))      # B is not (E, d)
    with pytest.raises(ValueError):
        g.node_mul_edge_forward(*INN[:3], node(), torch.zeros(E, D // 2))
    with pytest.raises(ValueError):
        g.node_mul_edge_backward(*INN[:3], node(), torch.zeros(E, D), edge(e=E + 1))
    with pytest.raises(ValueError):
        g.node_mul_edge_backward(*INN[:3], node(), torch.zeros(E, D, 2), edge())


def test_softmax_checks(g):
    with pytest.raises(ValueError):
        g.sparse_softmax_forward(*INN[:3], edge(e=E - 3))
    with pytest.raises(ValueError):
        g.sparse_softmax_forward(*INN[:3], torch.zeros(E, H, 2))
    with pytest.raises(ValueError):
        g.sparse_softmax_backward(*INN[:3], edge(), edge(h=4))
    with pytest.raises(ValueError):
        g.sparse_softmax_backward(*INN[:3], edge(e=E + 1), edge(e=E + 1))


def test_vector_spmm_checks(g):
    with pytest.raises(ValueError):
        g.vector_spmm_forward(*INN, edge(e=E - 1), node())
    with pytest.raises(ValueError):
        g.vector_spmm_forward(*INN, edge(h=4), node())
    with pytest.raises(ValueError):
        g.vector_spmm_forward(*INN, torch.zeros(E), node())                   # (E,) goes with (n, d) tensors only
    with pytest.raises(ValueError):
        g.vector_spmm_backward(*INN, *OUT, edge(), node(d=32), node())        # dy has another head size than x
    with pytest.raises(ValueError):
        g.vector_spmm_backward(*INN, *OUT, edge(e=E - 1), node(), node())


def test_attention_checks(g):
    lse = torch.zeros(N, H)
    with pytest.raises(ValueError):
        g.attention_forward(*INN, node(), node(), node(n=N - 1))              # v and k differ
    with pytest.raises(ValueError):
        g.attention_forward(*INN, node(), node(h=4), node(h=4))               # k, v have other heads than q
    with pytest.raises(ValueError):
        g.attention_backward(*OUT, *INN, node(), node(), node(), node(n=N - 1), lse, node())       # o
    with pytest.raises(ValueError):
        g.attention_backward(*OUT, *INN, node(), node(), node(), node(), lse, node(d=32))          # do
    with pytest.raises(ValueError):
        g.attention_backward(*OUT, *INN, node(), node(), node(), node(), torch.zeros(N, H - 1), node())   # lse shape
    with pytest.raises(ValueError):
        g.attention_backward(*OUT, *INN, node(), node(), node(), node(), lse.double(), node())            # lse dtype
    with pytest.raises(ValueError):
        g.attention_forward(*INN, node(), node(), node(), bias=torch.zeros(E, H))                  # bias needs E + 1 rows
    with pytest.raises(ValueError):
        g.rel_bias_forward(*INN[:3], INN[3][:-1], node(), torch.zeros(1000, D))                    # a type per slot


def test_rel_bias_checks(g):
    """The score term's own ops: every tensor against the graph and the table before a plan is asked for."""
    i32 = lambda n, v=0: torch.full((n,), v, dtype=torch.int32)
    table, used, used_types, ds = torch.zeros(1000, D), i32(1000, -1), i32(3), torch.zeros(E + 1, H)
    ok = (*INN[:3], INN[3], used, used_types, ds, node(), table, node())
    def bad(**kw):
        names = ("col", "indptr_c", "eid_c", "number_slot", "used", "used_types", "ds", "q", "table", "dq")
        args = [kw.get(n, a) for n, a in zip(names, ok)]
        with pytest.raises(ValueError):
            g.rel_bias_backward(*args)
    bad(table=torch.zeros(1000, D // 2))                 # other head size
    bad(used=i32(999, -1))                               # one entry per table row
    bad(used=torch.full((1000,), -1, dtype=torch.int64))
    bad(used_types=torch.zeros(3, dtype=torch.int64))
    bad(used_types=i32(1001))                            # more used types than types
    bad(ds=torch.zeros(E - 1, H))                        # a row per edge
    bad(ds=torch.zeros(E + 1, H - 1))
    bad(ds=torch.zeros(E + 1, H, dtype=torch.float64))
    bad(dq=node(n=N - 1))
    bad(number_slot=INN[3][:-1])                         # a type number per slot
    with pytest.raises(AssertionError):
        g.rel_bias_backward(*ok)                         # (well formed: reaches the plan cache)
    with pytest.raises(ValueError):
        g.rel_bias_forward(*INN[:3], INN[3], node(), table, used_types=torch.zeros(3, dtype=torch.int64))
    with pytest.raises(ValueError):
        g.rel_bias_forward(*INN[:3], INN[3], node(), table, used_types=i32(1001))
    with pytest.raises(ValueError):
        g.rel_bias_forward(*INN[:3], INN[3], node(), torch.zeros(1000, D + 1), used_types=i32(3))
    with pytest.raises(AssertionError):
        g.rel_bias_forward(*INN[:3], INN[3], node(), table, used_types=i32(3))


def test_score_term_in_pair_order_checks(g):
    """The (h, E) forms: the term over the tile plan, ds of the gradient op, bias of the fused calls."""
    i32 = lambda n, v=0: torch.full((n,), v, dtype=torch.int32)
    table, used_types = torch.zeros(1000, D), i32(3)
    def tiles(**kw):
        args = dict(q=node(), k=node(), table=table, used_types=used_types, pair_types=i32(E))
        args.update(kw)
        return g.rel_bias_forward_tiles(*OUT, *INN, args["q"], args["k"], args["table"], args["used_types"], args["pair_types"])
    for kw in (dict(pair_types=i32(E - 1)), dict(pair_types=torch.zeros(E, dtype=torch.int64)), dict(table=torch.zeros(1000, D // 2)),
               dict(used_types=torch.zeros(3, dtype=torch.int64)), dict(used_types=i32(1001))):
        with pytest.raises(ValueError):
            tiles(**kw)
    with pytest.raises(RuntimeError, match="tile kernels"):
        tiles()                                          # (well formed, but no tile kernels run on host tensors)
    used = i32(1000, -1)
    for ds in (torch.zeros(E + 1, H), torch.zeros(H, E + 1), torch.zeros(H, E, dtype=torch.float64)):
        with pytest.raises(ValueError):
            g.rel_bias_backward(*INN[:3], INN[3], used, used_types, ds, node(), table, node(), by_pair=True)
    with pytest.raises(ValueError, match="used_types"):
        g.rel_bias_forward(*INN[:3], INN[3], node(), table, by_pair=True)
    for bias in (torch.zeros(E + 1, H), torch.zeros(H, E + 1)):
        with pytest.raises(ValueError):
            g.attention_forward(*INN, node(), node(), node(), bias=bias, bias_by_pair=True)
        with pytest.raises(ValueError):
            g.attention_backward(*OUT, *INN, node(), node(), node(), node(), torch.zeros(N, H), node(), bias=bias, bias_by_pair=True)


def test_well_formed_calls_get_past_the_checks(g):
    # the same calls with fitting tensors reach the plan cache (which this fixture turns into an AssertionError)
    with pytest.raises(AssertionError):
        g.maskedmm_csr_forward(*OUT, node(), node())
    with pytest.raises(AssertionError):
        g.attention_backward(*OUT, *INN, node(), node(n=N + 3), node(n=N + 3), node(), torch.zeros(N, H), node())
    with pytest.raises(AssertionError):
        g.vector_spmm_forward(*INN, torch.zeros(E), torch.zeros(N, D))        # single head: (E,) with (n, d)
    with pytest.raises(AssertionError):
        g.vector_spmm_backward(*INN, *OUT, edge(), node(n=N - 1), node())     # rectangular: y has other rows than x
