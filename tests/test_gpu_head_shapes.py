"""Fused attention for the head shapes of the reference's other configs: 6 heads x 50 (configs/imdb-4.yml:10-12,
configs/snli.yml:11-13) and 8 x 40 (configs/ptb-6.yml:12-14).  The reference's kernels take any d
(graph_kernel/graphop_kernel.cu:269-304, 509-542); here `op.bpt_attention` runs the fused kernels on heads zero-padded to
64 columns.  Checked against the float64 oracle at the stated tolerances (fp32 outputs rtol / atol 1e-5, gradients rtol
1e-4; bf16 2e-2), with and without the rel_pos term, on the benchmark's small graph, a multigraph with empty and heavy
rows and a batch of merged graphs of different lengths."""
import numpy as np
import pytest
import torch

import oracle
from test_gpu_parity import DEV, GTOL, TOL, Case, GRAPHS, close, f64, rand

pytestmark = pytest.mark.gpu


def _tc_batch():
    """Block-diagonal merge of causal BPT graphs of different lengths (graph/text_classification.py:26-77)."""
    from bpt_amd import graphbuilder as gb
    lengths = np.random.default_rng(7).integers(20, 200, 6)
    src, dst, _, _, n = gb.merge_graphs([gb.BinaryPartition(int(L), True, 4, 10) for L in lengths])
    return np.asarray(src), np.asarray(dst), n


GRAPHS.setdefault("tc_batch6", _tc_batch)
_cases = {}


def _case(name):
    if name not in _cases:
        _cases[name] = Case(name)
    return _cases[name]


@pytest.fixture(scope="module")
def ops():
    from bpt_amd import graphop, op
    return graphop, op


@pytest.mark.parametrize("rel", [False, True], ids=["plain", "rel_pos"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hd", [(6, 50), (8, 40)], ids=["6x50", "8x40"])
@pytest.mark.parametrize("gname", ["bpt512_k4", "multigraph", "tc_batch6"])
def test_fused_attention_on_narrow_heads(ops, monkeypatch, gname, hd, dtype, rel):
    from oracle import torch_ops
    graphop, op = ops
    h, d = hd
    c = _case(gname)
    n_types = 23
    q, k, v, do = (rand((c.n, h, d), dtype, s, 1.0 / 8).to(DEV) for s in (51, 52, 53, 54))
    table = rand((n_types, d), dtype, 55, 1.0 / 8).to(DEV)
    etype = torch.from_numpy(np.random.default_rng(56).integers(0, n_types, c.E)).to(DEV)
    for t in (q, k, v, table):
        t.requires_grad_(True)
    assert graphop.attention_padded_shape(q) == (8, 64) and not graphop.attention_supported(q)
    fused_calls, chain_calls = [], []
    real_fwd, real_mm = graphop.attention_forward, graphop.maskedmm_csr_forward
    monkeypatch.setattr(graphop, "attention_forward", lambda *a, **kw: (fused_calls.append(a[4].shape), real_fwd(*a, **kw))[1])
    monkeypatch.setattr(op, "maskedmm_csr_forward", lambda *a, **kw: (chain_calls.append(1), real_mm(*a, **kw))[1])
    o = op.bpt_attention(*c.out, *c.inn, q, k, v, **(dict(rel_table=table, etype=etype) if rel else {}))    # default kernel choice
    o.backward(do)
    assert fused_calls == [(c.n, 8, 64)] and not chain_calls, "the fused kernels did not run"
    assert o.shape == (c.n, h, d) and o.is_contiguous()
    t64 = lambda x: x.detach().cpu().double()
    if rel:
        et = etype.cpu()
        ro, rdq, rdk, rdv, rdak = torch_ops.attention_fwd_bwd(torch.from_numpy(c.src), torch.from_numpy(c.dst), t64(q), t64(k), t64(v), t64(do),
                                                              ak=t64(table)[et])
        rdt = torch.zeros(n_types, d, dtype=torch.float64).index_add_(0, et, rdak)
        ro, rdq, rdk, rdv = (x.numpy() for x in (ro, rdq, rdk, rdv))
    else:
        ro, ra = oracle.attention_forward(c.csr, f64(q), f64(k), f64(v))
        rdq, rdk, rdv = oracle.attention_backward(c.csr, f64(q), f64(k), f64(v), ra, f64(do))
    close(o, ro, TOL[dtype], "o")
    close(q.grad, rdq, GTOL[dtype], "dq"); close(k.grad, rdk, GTOL[dtype], "dk"); close(v.grad, rdv, GTOL[dtype], "dv")
    if rel:
        # a table row is a raw sum over all edges of its type and all heads (h * E / n_types products): terms
        close(table.grad, rdt.numpy(), GTOL[dtype], "dtable", h * c.E / n_types)


def test_narrow_heads_chain_and_fused_agree(ops):
    """The op chain (shape-generic kernels, what `fused=False` runs) and the padded fused kernels give the same layer."""
    graphop, op = ops
    c = _case("bpt512_k4")
    q, k, v, do = (rand((c.n, 6, 50), torch.float32, s, 1.0 / 8).to(DEV) for s in (61, 62, 63, 64))
    outs = []
    for fused in (False, None):
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o = op.bpt_attention(*c.out, *c.inn, qq, kk, vv, fused=fused)
        o.backward(do)
        outs.append((o.detach(), qq.grad, kk.grad, vv.grad))
    for a, b, nm in zip(outs[0], outs[1], ("o", "dq", "dk", "dv")):
        close(a, f64(b), TOL[torch.float32] if nm == "o" else GTOL[torch.float32], nm)
