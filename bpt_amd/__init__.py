"""bpt_amd — MI355X-native graph-attention kernel layer of BP-Transformer.

  bpt_amd.graphbuilder  host graph construction (reference module `graphbuilder`)
  bpt_amd.graphop       the eight device ops of the reference's `graphop` extension + fused attention
  bpt_amd.op            autograd Functions with the surface of the reference's modules/op.py
  bpt_amd.plan          per-graph launch plans (row ownership instead of atomics)

`graphop`/`op` need the built HIP library and raise at import if it is missing.
"""
from . import graphbuilder  # noqa: F401  (host only; safe without a GPU)
