"""The transformer block of the reference (modules/attention.py:22-81) on the HIP attention kernels.

Same sub-modules, parameter names and initialisation as the reference's `BPTBlock`, so its
`state_dict` loads here unchanged: `norm_in`, `norm_inter`, `proj_q/k/v/o` (bias-free), `embed_ak`
(when `rel_pos`), `ffn.0.w_1`, `ffn.0.w_2`.  The reference keeps node features and edge types in a
DGL graph object (`g.ndata['h']`, `g.edata['etype']`) and writes the result back into it; here
`forward(h, csr, etype)` takes and returns plain tensors, `csr` being the 6-tuple that
`graph/base.py:71-86` (`bpt_amd.graphbuilder.get_csrs`) produces.

Attention core: the fused kernels (`op.bpt_attention`: rel_pos term and attention dropout included), or with
`fused=False` the four operators composed exactly as attention.py:66-77 does.
Projections, LayerNorm and the feed-forward are torch modules (rocBLAS GEMMs).
"""
import math

import torch
import torch.nn as nn

from .op import bpt_attention, edge_type_embedding, masked_mm, node_mul_edge, sparse_softmax, vec_spmm

__all__ = ["PositionwiseFeedForward", "BPTBlock", "BPTMemBlock"]


class PositionwiseFeedForward(nn.Module):
    """FFN(x) = max(0, x W_1 + b_1) W_2 + b_2   (modules/attention.py:8-19)"""

    def __init__(self, dim_model, dim_ff, dropout=0.1):
        super().__init__()
        self.w_1 = nn.Linear(dim_model, dim_ff)
        self.w_2 = nn.Linear(dim_ff, dim_model)
        self.dropout = nn.Dropout(dropout)

    def forward(self, x):
        return self.w_2(self.dropout(torch.relu(self.w_1(x))))


class BPTBlock(nn.Module):
    MAX_ETYPE = 1000        # modules/attention.py:23

    def __init__(self, dim_model, h, dim_ff, rel_pos=False, drop_h=0.1, drop_a=0.1, fused=True):
        super().__init__()
        self.fused = fused          # False: the four operators composed exactly as attention.py:66-77 does
        self.dim_model, self.h, self.dim_ff = dim_model, h, dim_ff
        self.d_k = dim_model // h
        self.rel_pos = rel_pos
        self.drop_h = nn.Dropout(drop_h)
        self.drop_att = nn.Dropout(drop_a)
        self.norm_in = nn.LayerNorm(dim_model)
        self.norm_inter = nn.LayerNorm(dim_model)
        self.proj_q = nn.Linear(dim_model, self.d_k * h, bias=False)
        self.proj_k = nn.Linear(dim_model, self.d_k * h, bias=False)
        self.proj_v = nn.Linear(dim_model, self.d_k * h, bias=False)
        self.proj_o = nn.Linear(self.d_k * h, dim_model, bias=False)
        if rel_pos:
            self.embed_ak = nn.Embedding(self.MAX_ETYPE, self.d_k)
        self.ffn = nn.Sequential(PositionwiseFeedForward(dim_model, dim_ff, dropout=drop_h), nn.Dropout(drop_h))

    def reset_parameters(self):
        # modules/attention.py:49-52
        for p in self.parameters():
            if p.dim() > 1:
                nn.init.xavier_uniform_(p)

    def attention(self, q, k, v, csr, etype=None):
        """attention.py:66-77: (n, h, d_k) q, k, v -> (n, h * d_k)."""
        out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C = csr
        graph = (ROW, INDPTR_R, out_csr[2], out_csr[1], COL, INDPTR_C, in_csr[2], in_csr[1])
        att_dropout = self.drop_att.p if self.training else 0.0
        if self.rel_pos and etype is None:
            raise ValueError("rel_pos=True needs the edge types (etype)")
        if self.fused:
            rel = dict(rel_table=self.embed_ak.weight, etype=etype) if self.rel_pos else {}
            return bpt_attention(*graph, q, k, v, dropout_p=att_dropout, **rel).view(-1, self.d_k * self.h)
        e = masked_mm(*graph, k, q)
        if self.rel_pos:
            e = e + node_mul_edge(COL, INDPTR_C, in_csr[2], q, edge_type_embedding(self.embed_ak.weight, etype))
        e = self.drop_att(sparse_softmax(COL, INDPTR_C, in_csr[2], e / math.sqrt(self.d_k)))
        return vec_spmm(COL, INDPTR_C, in_csr[2], in_csr[1], ROW, INDPTR_R, out_csr[2], out_csr[1], e, v).view(
            -1, self.d_k * self.h)

    def forward(self, h, csr, etype=None):
        # three GEMMs: one strided-batched GEMM over the stacked weights (its (3, n, h * d_k) result holds q, k, v as the
        # contiguous tensors the kernels need) measured slower, 3.38 against 3.17 ms per layer fwd+bwd at n = 16 383 in float32
        q = self.proj_q(h).view(-1, self.h, self.d_k)
        k = self.proj_k(h).view(-1, self.h, self.d_k)
        v = self.proj_v(h).view(-1, self.h, self.d_k)
        a = self.attention(q, k, v, csr, etype)
        h = self.norm_in(h + self.drop_h(self.proj_o(a)))
        return self.norm_inter(h + self.ffn(h))


def _graph_args(csr):
    out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C = csr
    return (ROW, INDPTR_R, out_csr[2], out_csr[1], COL, INDPTR_C, in_csr[2], in_csr[1])


class BPTMemBlock(nn.Module):
    """The decoder-side block of the reference (modules/attention.py:84-172): self-attention over the block's own
    graph, then attention to a memory (encoder states) over an inter graph, then the feed-forward.  Same sub-modules,
    parameter names and initialisation as the reference's `BPTMemBlock` (`proj_q.0` ... `proj_o.1`, `norm_in.0/1`,
    `norm_inter`, `embed_ak`, `ffn.0.w_1/w_2`), so its `state_dict` loads unchanged.

    forward(h, csr, mem, csr_inter, etype=None): h (n, dim_model) states of this block's nodes, mem (n_mem, dim_model)
    the memory, csr / csr_inter the 6-tuples of get_csrs; returns the new (n, dim_model) states.  csr_inter may be

      * the reference's square form (graph/mt.py:340-344): both CSRs over max(n, n_mem) nodes.  Queries are then
        padded with zero rows up to the in-CSR's row count as attention.py:148-149 does, and cut back afterwards; or
      * the bipartite form of graphbuilder.get_csrs_bipartite: out-CSR over the n_mem memory nodes, in-CSR over the n
        query nodes; nothing is padded (and n > n_mem, which the reference cannot run, works too).

    Both attention cores run the fused kernels (`op.bpt_attention`) where they cover the shape; `fused=False` composes
    the four operators exactly as the reference does."""
    MAX_ETYPE = 1000        # modules/attention.py:85

    def __init__(self, dim_model, h, dim_ff, rel_pos=False, drop_h=0.1, drop_a=0.1, fused=True):
        super().__init__()
        self.fused = fused
        self.dim_model, self.h, self.dim_ff = dim_model, h, dim_ff
        self.d_k = dim_model // h
        self.rel_pos = rel_pos
        self.drop_h = nn.ModuleList([nn.Dropout(drop_h) for _ in range(2)])
        self.drop_att = nn.ModuleList([nn.Dropout(drop_a) for _ in range(2)])
        self.norm_in = nn.ModuleList([nn.LayerNorm(dim_model) for _ in range(2)])
        self.norm_inter = nn.LayerNorm(dim_model)
        lin = lambda i, o: nn.ModuleList([nn.Linear(i, o, bias=False) for _ in range(2)])
        self.proj_q, self.proj_k, self.proj_v = (lin(dim_model, self.d_k * h) for _ in range(3))
        self.proj_o = lin(self.d_k * h, dim_model)
        if rel_pos:
            self.embed_ak = nn.Embedding(self.MAX_ETYPE, self.d_k)
        self.ffn = nn.Sequential(PositionwiseFeedForward(dim_model, dim_ff, dropout=drop_h), nn.Dropout(drop_h))

    def reset_parameters(self):
        # modules/attention.py:112-115
        for p in self.parameters():
            if p.dim() > 1:
                nn.init.xavier_uniform_(p)

    def _attend(self, which, q, k, v, csr, etype=None):
        """attention.py:130-141 (which = 0, with rel_pos) and :156-163 (which = 1): (n_q, h, d_k) -> (n_q, h * d_k)."""
        graph = _graph_args(csr)
        drop = self.drop_att[which]
        p = drop.p if self.training else 0.0
        rel = self.rel_pos and which == 0
        if rel and etype is None:
            raise ValueError("rel_pos=True needs the edge types (etype)")
        if self.fused:
            extra = dict(rel_table=self.embed_ak.weight, etype=etype) if rel else {}
            return bpt_attention(*graph, q, k, v, dropout_p=p, **extra).view(-1, self.d_k * self.h)
        COL, INDPTR_C, in_eid, in_idx = graph[4:]
        e = masked_mm(*graph, k, q)
        if rel:
            e = e + node_mul_edge(COL, INDPTR_C, in_eid, q, edge_type_embedding(self.embed_ak.weight, etype))
        e = drop(sparse_softmax(COL, INDPTR_C, in_eid, e / math.sqrt(self.d_k)))
        return vec_spmm(COL, INDPTR_C, in_eid, in_idx, *graph[:4], e, v,
                        n_rows=None if q.size(0) == v.size(0) else q.size(0)).view(-1, self.d_k * self.h)

    def forward(self, h, csr, mem, csr_inter, etype=None):
        heads = lambda proj, x: proj(x).view(-1, self.h, self.d_k)
        # Part I: self-attention (attention.py:118-142)
        a = self._attend(0, heads(self.proj_q[0], h), heads(self.proj_k[0], h), heads(self.proj_v[0], h), csr, etype)
        h = self.norm_in[0](h + self.drop_h[0](self.proj_o[0](a)))
        # Part II: attention to memory (attention.py:144-168)
        n = h.size(0)
        n_q = csr_inter[1][0].numel() - 1                  # rows of the inter graph's in-CSR
        if n_q < n:
            raise ValueError("the inter graph has fewer destination nodes than the block has states")
        hq = h if n_q == n else torch.cat([h, h.new_zeros(n_q - n, h.size(1))], 0)        # attention.py:148-149
        a = self._attend(1, heads(self.proj_q[1], hq), heads(self.proj_k[1], mem), heads(self.proj_v[1], mem), csr_inter)[:n]
        h = self.norm_in[1](h + self.drop_h[1](self.proj_o[1](a)))
        # FFN (attention.py:170-171)
        return self.norm_inter(h + self.ffn(h))
