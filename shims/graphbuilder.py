"""Module name the reference imports (`from graphbuilder import *`, graph/base.py:1; `partition_csr`, graph/base.py:69).

Put this directory and the repository root on PYTHONPATH: the classes and functions of graph_builder/builder.pyx
(BinaryPartition, FullyConnected, OpenAISparse, partition_csr) then come from bpt_amd's C++ builder."""
from bpt_amd.graphbuilder import *          # noqa: F401,F403
from bpt_amd.graphbuilder import __all__    # noqa: F401
