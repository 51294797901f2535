"""Host-side (CPU-runnable) logic of bpt_amd/op.py and bpt_amd/block.py."""
import numpy as np
import pytest
import torch

from bpt_amd import graphbuilder as gb


@pytest.mark.parametrize("seed", range(5))
def test_type_csr_equals_partition_csr_of_the_sorted_edge_types(seed):
    """The CSR over edge types (rows = types, slots = edges of that type in ascending edge id), built with tensor ops
    where etype lives, equals a stable argsort + builder.pyx:305-321's partition_csr."""
    from bpt_amd import op
    rng = np.random.default_rng(seed)
    n_types = 37
    et = torch.from_numpy(rng.integers(0, n_types, int(rng.integers(1, 5000)))) if seed else torch.zeros(0, dtype=torch.int64)
    if seed == 2:
        et[et == 5] = 6                      # a type without edges
    row, units, order = op._type_csr(et, n_types)
    e = et.numpy()
    indptr = np.zeros(n_types + 1, dtype=np.int64)
    np.cumsum(np.bincount(e, minlength=n_types), out=indptr[1:])
    want_row, want_units = gb.partition_csr(indptr)
    assert np.array_equal(order.numpy(), np.argsort(e, kind="stable"))
    assert np.array_equal(row.numpy(), want_row) and np.array_equal(units.numpy(), want_units)
    with pytest.raises(ValueError):
        op._type_csr(torch.tensor([0, n_types]), n_types)
