"""The module names the reference imports resolve to this package when `shims/` is on the path
(modules/op.py:2 `from graphop import *`; graph/base.py:1,69 `from graphbuilder import ...`)."""
import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIMS = os.path.join(ROOT, "shims")


@pytest.fixture()
def shim_path():
    sys.path.insert(0, SHIMS)
    for name in ("graphop", "graphbuilder"):
        sys.modules.pop(name, None)
    yield
    sys.path.remove(SHIMS)
    for name in ("graphop", "graphbuilder"):
        sys.modules.pop(name, None)


def test_graphop_star_import_gives_the_eight_reference_names(shim_path):
    ns = {}
    exec("from graphop import *", ns)
    names = sorted(k for k in ns if not k.startswith("__"))
    # graph_kernel/graphop.cpp:216-225
    assert names == sorted(["maskedmm_csr_forward", "maskedmm_csr_backward", "node_mul_edge_forward", "node_mul_edge_backward",
                            "sparse_softmax_forward", "sparse_softmax_backward", "vector_spmm_forward", "vector_spmm_backward"])
    import bpt_amd.graphop as real
    assert all(ns[k] is getattr(real, k) for k in names)
    assert importlib.import_module("graphop").__file__.startswith(SHIMS)


def test_graphbuilder_names_of_the_reference_import(shim_path):
    ns = {}
    exec("from graphbuilder import BinaryPartition, FullyConnected, OpenAISparse, partition_csr", ns)    # graph/base.py:1,69
    g = ns["BinaryPartition"](8, True, 2, 10)
    src, dst, et = g.get_edges()
    assert g.number_of_edges == len(src) == len(dst) == len(et) and g.number_of_nodes == 15
    row, indptr = ns["partition_csr"](np.array([0, 4, 8, 10], dtype=np.int64), 4)     # graph_kernel/part_csr.py:29-32
    assert list(row) == [0, 1, 2] and list(indptr) == [0, 4, 8, 10]
    assert ns["FullyConnected"](5, True, 2).number_of_nodes == 6
    assert ns["OpenAISparse"](8, 4, 1).number_of_nodes >= 8
    # the star import of graph/base.py:1 brings the same four
    star = {}
    exec("from graphbuilder import *", star)
    assert {"BinaryPartition", "FullyConnected", "OpenAISparse", "partition_csr"} <= set(star)
