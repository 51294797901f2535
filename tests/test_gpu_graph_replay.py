"""The fused step under HIP graph capture: a caller that records forward + backward once and replays it (a training
loop with a fixed graph) must get, on every replay, exactly what the eager launches give.  The graph is replayed
several times with eager work of the same library and synchronisations in between, inputs are changed in place
between replays, and every replay is compared bit for bit with an eager step on the same inputs.  The tile kernels
forward and backward in float32 and bfloat16, and in float32 also the tile forward with the row-group backward; with and
without dropout (a function of seed, edge id and head: the same under replay)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.mark.parametrize("dtype,dropout,tile_backward", [(torch.float32, 0.0, None), (torch.bfloat16, 0.0, None), (torch.float32, 0.2, None),
                                                         (torch.float32, 0.0, False), (torch.float32, 0.2, False)])
@pytest.mark.parametrize("L", [1024, 8192])
def test_graph_replay_equals_eager(L, dtype, dropout, tile_backward, monkeypatch):
    """tile_backward None: the library's choice (tiles); False: the backward on the row groups."""
    from bpt_amd import graphbuilder as gb
    from bpt_amd import graphop
    monkeypatch.setattr(graphop, "TILE_BACKWARD", tile_backward)
    g = gb.BinaryPartition(L, True, 4, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n)
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(77)
    q, k, v, do = ((torch.randn(n, 8, 64, generator=gen) / 8).to(dtype).to(DEV) for _ in range(4))
    seed = 1234

    def step():
        o, lse = graphop.attention_forward(*args[4:], q, k, v, dropout_p=dropout, seed=seed)
        return (o, lse) + tuple(graphop.attention_backward(*args, q, k, v, o, lse, do, dropout_p=dropout, seed=seed))

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):                      # plans are built and cached before the capture
        for _ in range(2):
            step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gout = step()
    for rep in range(4):
        if rep:                                        # new inputs, written in place: the graph reads the same buffers
            for t in (q, k, v, do):
                t.mul_(-0.5).add_(0.01 * rep)
        want = step()                                  # eager work of the same library between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b, name in zip(gout, want, ("o", "lse", "dq", "dk", "dv")):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager result"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graph_replay_of_the_step_with_the_rel_pos_term_equals_eager(dtype):
    """The same with the rel_pos score term: its score kernel, the fused kernels that add it, and the kernels that form
    the gradients of q and of the table from the per-edge ds (more than 64 KB of LDS per workgroup, partial tables in
    the kept workspace), the table changed in place between replays like the other inputs."""
    import numpy as np
    from bpt_amd import graphbuilder as gb
    from bpt_amd import graphop, op
    g = gb.BinaryPartition(8192, True, 4, 10)
    src, dst, etype = g.get_edges()
    n = g.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n)
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(78)
    q, k, v, do = ((torch.randn(n, 8, 64, generator=gen) / 8).to(dtype).to(DEV) for _ in range(4))
    table = (torch.randn(1000, 64, generator=gen) / 8).to(dtype).to(DEV)
    aux = op._rel_aux(torch.from_numpy(np.asarray(etype, dtype=np.int64)).to(DEV), *args[4:7], 1000)
    assert 1 < aux["n_used"] <= graphop.REL_MAX_USED_TYPES

    def step():
        bias = graphop.rel_bias_forward(*args[4:7], aux["number_slot"], q, table, used_types=aux["used_types"])
        o, lse = graphop.attention_forward(*args[4:], q, k, v, bias=bias)
        dq, dk, dv, ds = graphop.attention_backward(*args, q, k, v, o, lse, do, bias=bias)
        dtable = graphop.rel_bias_backward(*args[4:7], aux["number_slot"], aux["used"], aux["used_types"], ds, q, table, dq)
        return o, lse, dq, dk, dv, dtable

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):                      # plans are built and cached before the capture
        for _ in range(2):
            step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gout = step()
    for rep in range(4):
        if rep:
            for t in (q, k, v, do, table):
                t.mul_(-0.5).add_(0.01 * rep)
        want = step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b, name in zip(gout, want, ("o", "lse", "dq", "dk", "dv", "dtable")):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager result"


def test_kept_workspaces_give_the_same_results_and_can_be_released():
    """Ops keep one workspace per device and stream and reuse it from call to call: results equal those with a fresh
    allocation per call, two different ops in a row do not disturb each other, and release_workspaces() drops the buffers."""
    from bpt_amd import graphbuilder as gb
    from bpt_amd import graphop
    g = gb.BinaryPartition(2048, False, 4, 10)            # non-causal: rows of 2048 edges, split rows on both sides
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n)
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(5)
    q, k, v, do = ((torch.randn(n, 8, 64, generator=gen) / 8).to(DEV) for _ in range(4))
    w = torch.randn(len(src), 8, generator=gen).to(DEV)

    def run():
        o, lse = graphop.attention_forward(*args[4:], q, k, v)
        y = graphop.vector_spmm_forward(*args[4:], w, v)                       # another op between forward and backward
        return (o, lse, y) + tuple(graphop.attention_backward(*args, q, k, v, o, lse, do))

    graphop.release_workspaces()
    assert not graphop._SCRATCH
    kept = run()
    assert len(graphop._SCRATCH) == 1
    again = run()
    old, graphop.KEEP_WORKSPACES = graphop.KEEP_WORKSPACES, False
    try:
        fresh = run()
    finally:
        graphop.KEEP_WORKSPACES = old
    torch.cuda.synchronize()
    for a, b, c in zip(kept, again, fresh):
        assert torch.equal(a, b) and torch.equal(a, c)
    graphop.release_workspaces()
    assert not graphop._SCRATCH
