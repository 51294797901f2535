"""TEST INFRASTRUCTURE — PyTorch-CPU restatement of the attention layer's op semantics.

The same arithmetic as modules/attention.py:66-77 (masked_mm over the out-CSR, scale by
1/sqrt(d_k), sparse_softmax over each destination's in-edges, vec_spmm) written with gather /
index_add / scatter_reduce over the edge list, backward by autograd.  Used (a) as an independent
fp64 cross-check of the C oracle and (b) as the multi-threaded CPU baseline timed by bench.py
(the reference has no CPU path of its own: README.md:53-54).  Never imported by the product.
"""
import math

import torch


def attention(src, dst, q, k, v, ak=None, drop=None):
    """src, dst: (E,) int64 edge endpoints (edge e: src[e] -> dst[e]); q,k,v: (N,H,D).

    Returns o (N,H,D) with o[dst] = sum_e softmax_dst(q[dst].k[src]/sqrt(D)) * v[src].  ak (E,D): rows of the
    relative-position table per edge (attention.py:69-71).  drop (E,H): multipliers that dropout applies to the
    attention probabilities, 0 or 1/(1-p) (attention.py:73)."""
    n, h, d = q.shape
    s = (k[src] * q[dst]).sum(-1)                              # (E,H)   attention.py:66-67
    if ak is not None:
        s = s + (q[dst] * ak.unsqueeze(1)).sum(-1)             # attention.py:69-71
    s = s / math.sqrt(d)
    idx = dst.unsqueeze(-1).expand(-1, h)
    m = torch.full((n, h), -1e9, dtype=s.dtype).scatter_reduce(0, idx, s.detach(), "amax", include_self=True)
    p = torch.exp(s - m[dst])                                  # graphop_kernel.cu:180-192
    z = torch.zeros((n, h), dtype=s.dtype).index_add_(0, dst, p)
    a = p / z[dst]                                             # graphop_kernel.cu:194-202
    if drop is not None:
        a = a * drop                                           # attention.py:73
    o = torch.zeros((n,) + tuple(v.shape[1:]), dtype=v.dtype).index_add_(0, dst, a.unsqueeze(-1) * v[src])   # attention.py:74-77
    return o


def attention_fwd_bwd(src, dst, q, k, v, do, ak=None, drop=None):
    q = q.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    v = v.detach().clone().requires_grad_(True)
    leaves = [q, k, v]
    if ak is not None:
        ak = ak.detach().clone().requires_grad_(True)
        leaves.append(ak)
    o = attention(src, dst, q, k, v, ak, drop)
    grads = torch.autograd.grad(o, leaves, do)
    return (o.detach(),) + tuple(grads)
