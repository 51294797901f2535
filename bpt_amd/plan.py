"""Launch plans: the int32 row-level form of one CSR side plus the wavefront work list.

The reference's ops receive (row, indptr, eid, indices) as int64 device tensors on every call
(modules/op.py:10-70).  The HIP kernels want row ownership, so the first call that sees a given
set of index tensors copies them to the host once, lets libbptgraph validate them and derive the
plan (bptg_plan_fill), uploads the plan and caches it; later calls with the same tensors (all 12
layers, forward and backward) hit the cache.  The cache keeps the key tensors alive, so a
`data_ptr` can not be recycled for another graph while its entry exists.
"""
import collections
import ctypes
import threading

import numpy as np
import torch

from ._lib import PlanInfo, PlanStruct, check_graph, graph_lib

DEFAULT_SEG_LEN = 64
GROUP_R = 4            # rows per group: 4 = one wavefront per group (default, fastest measured); 16 = a team of 4 wavefronts x 4 rows sharing rows through LDS
GROUP_WINDOW = 32      # how many following items the greedy grouping examines per group
GROUP_ORDER = 2        # order of the groups inside an XCD chunk: 0 locality, 1 big first / small last, 2 decreasing work
_CACHE_SIZE = 64


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _host_i64(t):
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=np.int64)


def build_plan_host(row, indptr, eid, indices, n_rows, n_index_nodes, seg_len=DEFAULT_SEG_LEN):
    """Pure host step (no GPU): returns (arrays, info) with arrays = dict of int32 numpy arrays
    rowptr, idx, eid, items (n_items, 4), heavy (n_heavy, 3).  Raises ValueError on malformed input."""
    row, indptr, eid, indices = map(_host_i64, (row, indptr, eid, indices))
    if len(indptr) != len(row) + 1:
        raise ValueError("indptr must have len(row) + 1 entries")
    if indices is not None and len(indices) != len(eid):
        raise ValueError("indices and eid must have the same length")
    lib = graph_lib()
    info = PlanInfo()
    check_graph(lib.bptg_plan_sizes(_ptr(row), _ptr(indptr), len(row), int(n_rows), int(seg_len), ctypes.byref(info)))
    E = len(eid)
    arrays = {
        "rowptr": np.empty(n_rows + 1, dtype=np.int32),
        "idx": np.empty(E, dtype=np.int32),
        "eid": np.empty(E, dtype=np.int32),
        "items": np.empty((info.n_items, 4), dtype=np.int32),
        "heavy": np.empty((info.n_heavy, 3), dtype=np.int32),
    }
    check_graph(lib.bptg_plan_fill(_ptr(row), _ptr(indptr), len(row), _ptr(eid), _ptr(indices), E,
                                   int(n_rows), int(n_index_nodes), int(seg_len),
                                   _ptr(arrays["rowptr"]), _ptr(arrays["idx"]), _ptr(arrays["eid"]),
                                   _ptr(arrays["items"]), _ptr(arrays["heavy"]), ctypes.byref(info)))
    return arrays, info


def build_groups_host(arrays, n_index_nodes, R=None, window=GROUP_WINDOW, order_mode=None):
    """Pure host step: clusters the plan's items into row groups (bptg_group_plan).  Returns a dict
    with members (n_groups, R, 2), grp_ptr (n_groups + 1), entries (n_entries, 4), pair_eid (n_edges),
    chunks (9,)."""
    order_mode = GROUP_ORDER if order_mode is None else order_mode
    R = GROUP_R if R is None else R
    items = np.ascontiguousarray(arrays["items"], dtype=np.int32)
    idx = np.ascontiguousarray(arrays["idx"], dtype=np.int32)
    eid = np.ascontiguousarray(arrays["eid"], dtype=np.int32)
    n_items, E = len(items), len(eid)
    members = np.empty((max(n_items, 1), R, 2), dtype=np.int32)
    grp_ptr = np.empty(n_items + 1, dtype=np.int32)
    entries = np.zeros((E + 1, 4), dtype=np.int32)      # one zero row of padding: kernels may peek at entries[n_entries]
    pair_eid = np.empty(max(E, 1), dtype=np.int32)
    chunks = np.zeros(9, dtype=np.int32)
    ng, ne = ctypes.c_int64(), ctypes.c_int64()
    check_graph(graph_lib().bptg_group_plan(_ptr(items), n_items, _ptr(idx), _ptr(eid), E, int(n_index_nodes), R, window,
                                            int(order_mode), _ptr(members), _ptr(grp_ptr), _ptr(entries), _ptr(pair_eid),
                                            _ptr(chunks), ctypes.byref(ng), ctypes.byref(ne)))
    return {"members": members[:ng.value].copy(), "grp_ptr": grp_ptr[:ng.value + 1].copy(),
            "entries": entries[:ne.value].copy(), "entries_padded": entries[:ne.value + 1].copy(),
            "pair_eid": pair_eid[:E].copy(), "chunks": chunks, "R": R}


class Plan:
    """Device-resident plan of one CSR side; `.struct` is the `bpt_plan` passed to the C ABI."""

    def __init__(self, row, indptr, eid, indices, n_rows, n_index_nodes, device, seg_len=DEFAULT_SEG_LEN):
        arrays, info = build_plan_host(row, indptr, eid, indices, n_rows, n_index_nodes, seg_len)
        self.n_rows, self.n_edges = int(n_rows), len(arrays["eid"])
        self.n_items, self.n_heavy, self.n_slots = info.n_items, info.n_heavy, info.n_slots
        self.max_degree = info.max_degree
        self.covers_all_edges = bool(info.flags & 1)
        self.has_indices = indices is not None
        self.device = torch.device(device)
        self.n_index_nodes = int(n_index_nodes)
        self._host = arrays                  # kept for the (lazy) row-group construction
        self._groups = None
        self._links = {}
        self._lock = threading.Lock()
        # one allocation, 256-byte aligned sections (the items array is read as 16-byte vectors)
        self._dev = {k: torch.from_numpy(v).to(self.device) for k, v in arrays.items()}
        d = self._dev
        self.struct = PlanStruct(
            d["rowptr"].data_ptr(), d["idx"].data_ptr() if self.n_edges else None,
            d["eid"].data_ptr() if self.n_edges else None, d["items"].data_ptr() if self.n_items else None,
            d["heavy"].data_ptr() if self.n_heavy else None,
            self.n_rows, self.n_edges, self.n_items, self.n_heavy, self.n_slots)

    @property
    def ref(self):
        return ctypes.byref(self.struct)

    # ---- row groups for the fused attention kernels ----
    def ensure_groups(self):
        """Builds the row-group arrays once (host) and uploads them; returns the host dict."""
        with self._lock:
            if self._groups is None or self._groups["R"] != GROUP_R:
                self._links = {}
                grp = build_groups_host(self._host, self.n_index_nodes)
                self._grp_dev = {k: torch.from_numpy(grp[k]).to(self.device)
                                 for k in ("members", "grp_ptr", "entries_padded", "chunks")}
                d = self._grp_dev
                self.n_groups = len(grp["members"])
                self.struct.grp_members = d["members"].data_ptr() if self.n_groups else None
                self.struct.grp_ptr = d["grp_ptr"].data_ptr()
                self.struct.grp_entries = d["entries_padded"].data_ptr()
                self.struct.grp_pairs = None
                self.struct.grp_chunks = d["chunks"].data_ptr()
                self.struct.grp_max_chunk = int(np.diff(grp["chunks"]).max()) if self.n_groups else 0
                self.struct.n_groups = self.n_groups
                self.struct.grp_R = grp["R"]
                self._groups = grp
        return self._groups

    def linked_to(self, plan_src):
        """`bpt_plan` of this (destination-side) plan whose grp_pairs maps each of its pairs to the number of
        the same edge's pair in `plan_src` (the source-side plan of the same graph)."""
        mine, theirs = self.ensure_groups(), plan_src.ensure_groups()
        key = (id(plan_src), GROUP_R)
        with self._lock:
            hit = self._links.get(key)
            if hit is None:
                if self.n_edges != plan_src.n_edges or not (self.covers_all_edges and plan_src.covers_all_edges):
                    raise ValueError("the two plans do not describe the same edge set")
                pos_of_eid = np.empty(self.n_edges, dtype=np.int32)
                pos_of_eid[theirs["pair_eid"]] = np.arange(self.n_edges, dtype=np.int32)
                pairs = torch.from_numpy(pos_of_eid[mine["pair_eid"]]).to(self.device)
                st = PlanStruct.from_buffer_copy(self.struct)
                st.grp_pairs = pairs.data_ptr() if self.n_edges else None
                hit = (st, pairs, plan_src)          # keeps the mapping and the partner alive
                self._links[key] = hit
        return hit[0]


class PlanCache:
    def __init__(self, capacity=_CACHE_SIZE):
        self._d = collections.OrderedDict()
        self._cap = capacity
        self._lock = threading.Lock()     # forward runs on the Python thread, backward on autograd's
        self.hits = self.misses = 0

    @staticmethod
    def _key(tensors, n_rows, n_index, seg_len):
        return tuple((t.data_ptr(), t.numel(), t._version, str(t.device)) if t is not None else None
                     for t in tensors) + (n_rows, n_index, seg_len)

    def get(self, row, indptr, eid, indices, n_rows=None, n_index_nodes=None, seg_len=DEFAULT_SEG_LEN):
        """n_rows None: as many rows as `row` mentions (ops that only produce edge outputs)."""
        tensors = (row, indptr, eid, indices)
        key = self._key(tensors, n_rows, n_index_nodes, seg_len)
        with self._lock:
            hit = self._d.get(key)
            if hit is not None:
                self._d.move_to_end(key)
                self.hits += 1
                return hit[0]
        self.misses += 1
        row_h = _host_i64(row)
        nr = n_rows if n_rows is not None else (int(row_h[-1]) + 1 if len(row_h) else 0)
        ni = n_index_nodes if n_index_nodes is not None else nr
        plan = Plan(row_h, indptr, eid, indices, nr, ni, eid.device, seg_len)
        with self._lock:
            self._d[key] = (plan, tensors)          # tensors kept alive with the entry
            while len(self._d) > self._cap:
                self._d.popitem(last=False)
        return plan

    def clear(self):
        with self._lock:
            self._d.clear()


plan_cache = PlanCache()
