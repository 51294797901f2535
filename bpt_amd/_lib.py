"""ctypes bindings of the two native libraries (C ABIs in include/bptgraph.h and include/bptattn.h).

There is no Python or CPU fallback for the device ops: if libbptattn.so is missing, importing
`bpt_amd.graphop` raises.  Build with `python -m bpt_amd._build`.
"""
import ctypes
import os

from ._build import ATTN_SO, GRAPH_SO, PLAN_SO

c_i64 = ctypes.c_int64
c_vp = ctypes.c_void_p


class PlanStruct(ctypes.Structure):
    """Mirror of `bpt_plan` (include/bptattn.h)."""
    _fields_ = [("rowptr", c_vp), ("idx", c_vp), ("eid", c_vp), ("items", c_vp), ("heavy", c_vp),
                ("n_rows", c_i64), ("n_edges", c_i64), ("n_items", c_i64), ("n_heavy", c_i64), ("n_slots", c_i64),
                ("grp_members", c_vp), ("grp_ptr", c_vp), ("grp_entries", c_vp), ("grp_pairs", c_vp),
                ("grp_chunks", c_vp), ("n_groups", c_i64), ("grp_R", c_i64), ("grp_max_chunk", c_i64),
                ("n_grp_entries", c_i64), ("grp_eids", c_vp), ("bias_by_pair", c_i64),
                ("n_index_nodes", c_i64)]


class PlanInfo(ctypes.Structure):
    """Mirror of `bptg_plan_info` (include/bptgraph.h)."""
    _fields_ = [("n_items", c_i64), ("n_heavy", c_i64), ("n_slots", c_i64), ("max_degree", c_i64), ("flags", c_i64)]


# every exported symbol with (restype, argtypes); tests check the libraries export exactly these
GRAPH_API = {
    "bptg_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "bptg_graph_sizes": (ctypes.c_int, [ctypes.c_int, c_i64, ctypes.c_int, c_i64, c_i64, c_vp, c_vp, c_vp]),
    "bptg_graph_fill": (ctypes.c_int, [ctypes.c_int, c_i64, ctypes.c_int, c_i64, c_i64, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "bptg_partition_csr_count": (ctypes.c_int, [c_vp, c_i64, c_i64, c_vp]),
    "bptg_partition_csr_fill": (ctypes.c_int, [c_vp, c_i64, c_i64, c_vp, c_vp]),
    "bptg_build_csr": (ctypes.c_int, [c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp]),
    "bptg_plan_sizes": (ctypes.c_int, [c_vp, c_vp, c_i64, c_i64, c_i64, ctypes.POINTER(PlanInfo)]),
    "bptg_plan_fill": (ctypes.c_int, [c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64,
                                      c_vp, c_vp, c_vp, c_vp, c_vp, ctypes.POINTER(PlanInfo)]),
    "bptg_group_plan": (ctypes.c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_i64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                       ctypes.c_int32, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "bptg_link_groups": (ctypes.c_int, [c_vp, c_i64, ctypes.c_int32, c_vp, c_i64, ctypes.c_int32, c_i64, ctypes.c_int32, c_vp]),
}

_PP = ctypes.POINTER(PlanStruct)
_tail = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_vp]          # h, d, dtype, stream
ATTN_API = {
    "bpt_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "bpt_plan_struct_bytes": (c_i64, []),
    "bpt_set_force_generic": (ctypes.c_int, [ctypes.c_int]),
    "bpt_profile_kernel": (ctypes.c_int, [ctypes.c_int, c_vp, c_vp]),
    "bpt_gather_probe": (ctypes.c_int, [c_vp, c_i64, ctypes.c_int, ctypes.c_int, ctypes.c_int, c_vp, c_vp]),
    "bpt_workspace_bytes": (c_i64, [ctypes.c_int, _PP, _PP, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "bpt_maskedmm_csr_forward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp] + _tail),
    "bpt_maskedmm_csr_backward": (ctypes.c_int, [_PP, _PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64] + _tail),
    "bpt_node_mul_edge_forward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp] + _tail),
    "bpt_node_mul_edge_backward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64] + _tail),
    "bpt_sparse_softmax_forward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_i64, ctypes.c_int, ctypes.c_int, c_vp]),
    "bpt_sparse_softmax_backward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_i64, ctypes.c_int, ctypes.c_int, c_vp]),
    "bpt_vector_spmm_forward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_i64] + _tail),
    "bpt_vector_spmm_accumulate": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_i64] + _tail),
    "bpt_vector_spmm_backward": (ctypes.c_int, [_PP, _PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64] + _tail),
    "bpt_rel_bias_forward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_i64, c_vp] + _tail),
    "bpt_rel_bias_forward_tiles": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_i64, c_vp, c_vp] + _tail),
    "bpt_rel_bias_backward_workspace_bytes": (c_i64, [_PP, c_i64, ctypes.c_int]),
    "bpt_rel_bias_backward_supported": (ctypes.c_int, [c_i64, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "bpt_rel_bias_backward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_i64] + _tail),
    "bpt_attention_forward": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, ctypes.c_float, ctypes.c_float,
                                            ctypes.c_uint64] + _tail),
    "bpt_attention_forward_noalloc": (ctypes.c_int, [_PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, ctypes.c_float, ctypes.c_float,
                                                    ctypes.c_uint64] + _tail),
    "bpt_attention_backward": (ctypes.c_int, [_PP, _PP, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
                                             c_i64, ctypes.c_float, ctypes.c_float, ctypes.c_uint64] + _tail),
}

c_i32 = ctypes.c_int32
# libbptplan (include/bptplan.h): plans built on the GPU
PLAN_API = {
    "bpt_graph_count_device": (ctypes.c_int, [ctypes.c_int, c_i64, ctypes.c_int, c_i64, c_i64, c_vp, c_vp, c_i64, c_vp]),
    "bpt_graph_fill_device": (ctypes.c_int, [ctypes.c_int, c_i64, ctypes.c_int, c_i64, c_i64, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp]),
    "bpt_csr_device_bounds": (ctypes.c_int, [c_i64, c_i64, c_i32, ctypes.POINTER(c_i64 * 2)]),
    "bpt_csr_build_device": (ctypes.c_int, [c_vp, c_vp, c_i64, c_i64, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp]),
    "bpt_plan_device_bounds": (ctypes.c_int, [c_i64, c_i64, c_i64, c_i32, c_i32, ctypes.POINTER(c_i64 * 4)]),
    "bpt_plan_build_device": (ctypes.c_int, [c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32,
                                             c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp]),
    "bpt_plan_group_device": (ctypes.c_int, [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32,
                                             c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp]),
    "bpt_plan_link_device": (ctypes.c_int, [c_vp, c_vp, c_i32, c_vp, c_vp, c_i32, c_i64, c_i32, c_vp, c_vp, c_i64, c_vp]),
}

_graph = None
_attn = None
_plan = None


def _load(path, api, what):
    if not os.path.exists(path):
        raise ImportError(f"{what} is not built ({path} missing): run `python -m bpt_amd._build`")
    lib = ctypes.CDLL(path)
    for name, (res, args) in api.items():
        fn = getattr(lib, name)          # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    return lib


def graph_lib():
    global _graph
    if _graph is None:
        _graph = _load(GRAPH_SO, GRAPH_API, "libbptgraph")
    return _graph


def attn_lib():
    global _attn
    if _attn is None:
        lib = _load(ATTN_SO, ATTN_API, "libbptattn (HIP kernels)")
        if lib.bpt_plan_struct_bytes() != ctypes.sizeof(PlanStruct):
            raise ImportError(f"libbptattn was built for a bpt_plan of {lib.bpt_plan_struct_bytes()} bytes, this binding passes "
                              f"{ctypes.sizeof(PlanStruct)}: rebuild with `python -m bpt_amd._build`")
        _attn = lib
    return _attn


def plan_lib():
    global _plan
    if _plan is None:
        _plan = _load(PLAN_SO, PLAN_API, "libbptplan (plans built on the GPU)")
    return _plan


def check_graph(status):
    if status != 0:
        raise ValueError("bptgraph: " + graph_lib().bptg_strerror(status).decode())


class BptStatusError(RuntimeError):
    """A non-zero status of a libbptattn call; `.status` is the code (negative: bpt_status, positive: hipError_t)."""

    def __init__(self, status, what):
        super().__init__(f"{what}: " + attn_lib().bpt_strerror(status).decode() + f" (status {status})")
        self.status = int(status)


BPT_ERR_UNSUPPORTED = -7


def check_attn(status, what):
    if status != 0:
        raise BptStatusError(status, what)
