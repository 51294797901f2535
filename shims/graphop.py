"""Module name the reference imports (`from graphop import *`, modules/op.py:2; graph_kernel/test.py:2).

Put this directory and the repository root on PYTHONPATH: the star import then yields exactly the eight functions
the reference's pybind module exports (graph_kernel/graphop.cpp:216-225), served by the HIP kernels of bpt_amd."""
from bpt_amd.graphop import *          # noqa: F401,F403
from bpt_amd.graphop import __all__    # noqa: F401
