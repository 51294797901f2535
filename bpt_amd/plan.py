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

from ._lib import PlanInfo, PlanStruct, check_graph, graph_lib, plan_lib

DEFAULT_SEG_LEN = None  # edges per work item: None = chosen per plan by auto_seg_len
FORCE_SEG_LEN = None    # testing hook: when set, replaces the automatic choice for plans built from now on
GROUP_R = 4            # default rows per group (the row-group kernels exist for 4 and, float32 with h <= 8 and h*d <= 512, 8)
GROUP_WINDOW = 32      # how many following items the greedy grouping examines per group
GROUP_ORDER = 2 + 4    # groups inside an XCD chunk by decreasing work (2); entries of a group sorted by member mask (+4)
GROUP_ORDER_SRC = 2 + 8  # source-side groups of the fused backward: aligned entry order (+8), which lowers that kernel's HBM reads
GROUP_MAX_PAIRS = None  # cap on the edges of one group: None = 48 per member row, 0 = no cap
GROUP_PAD_ENTRIES = 8  # the kernels' software pipeline reads per-entry arrays this far past the end
TILE_GROUP_R = 16      # rows per group of the dense-tile kernels
TILE_ORDER_SRC = None   # order of the SOURCE-side tile groups of the fused backward: None = tile_order_src()'s choice


def tile_order_src(n_rows, n_edges):
    """Order of the source-side tile groups.  On large sparse graphs the groups of an XCD's range keep their locality order
    (0: groups that run at the same time read the same q / dO rows; measured at L = 8192, k = 4: that kernel's HBM reads
    245 -> 115 MB and 55 -> 51 us; L = 32768, k = 8 in bfloat16: 455 -> 418 us; the 32-graph batch 95 -> 91 us); on small or
    dense graphs the order by decreasing work (2 + 4) wins, whose last groups are the lightest (L = 4096, k = 32: 57 against
    70 us in locality order)."""
    if TILE_ORDER_SRC is not None:
        return TILE_ORDER_SRC
    return 0 if (n_rows >= 12288 and n_edges <= 64 * n_rows) else 2 + 4
TILE_ORDER_DST = None   # order of the DESTINATION-side tile groups (the forward's and the fused backward's): None = tile_order_dst()'s choice


def tile_order_dst(n_index_nodes):
    """Order of the destination-side tile groups (what ensure_groups takes for groups of TILE_GROUP_R rows when no order is
    named).  By decreasing work inside an XCD's range (2 + 4: the last groups are the lightest) tiles that read the same
    K / V rows do not run at the same time and the rows are fetched about twice; that costs nothing while K and V fit the
    memory-side cache, and locality order (4) is slower there (L = 8192, k = 4: 0.142 against 0.144 ms; the 32-graph
    batch 0.264 against 0.267; 32 767 nodes level).  Beyond it the second fetch is HBM traffic and locality order wins:
    65 535 nodes, 8 heads float32 0.669 -> 0.641 ms (bfloat16 level), 131 071 nodes 1.425 -> 1.268 (bfloat16
    0.813 -> 0.786), L = 32768, k = 8 with 16 heads float32 1.547 -> 1.447, bfloat16 0.912 -> 0.895."""
    if TILE_ORDER_DST is not None:
        return TILE_ORDER_DST
    return 4 if n_index_nodes >= 49152 else 2 + 4
TILE_MAX_PAIRS = 0     # cap on the edges of such a group (0 = none, None = as the other groups)
_CACHE_SIZE = 64                 # plans kept by the cache (PlanCache.set_limits)
_CACHE_BYTES = 2 << 30           # and the device memory they may hold together: least recently used plans go first
DEVICE_BUILD = None     # where new plans are built: True = on the GPU (libbptplan), False = on the host, None = by size
DEVICE_BUILD_MIN_ROWS = 24576   # None: graphs with at least this many rows are planned on the GPU (measured: their
                                # simpler grouping runs the fused kernels 4-9 % faster there and builds 10-30 x faster),
DEVICE_BUILD_MIN_DEGREE = 32    # and so are graphs of at least 2^17 edges with this average degree (L = 4096: k = 8, 16,
                                # 32 run 5, 3 and 18 % faster on GPU-built groups, k = 1 and 4 run 8 and 1 % slower)
DEVICE_BUILD_DENSE_MIN_ROWS = 2048   # if they have this many rows: the CSR of 1000 edge types over 430 k edges (the table
                                     # gradient of the rel_pos term) runs its SpMM in 40 us on host-built groups, 130 us on GPU-built ones


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _host_i64(t):
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=np.int64)


def auto_seg_len(row, indptr, n_rows):
    """Edges per work item.  Rows longer than this are cut into segments whose partial results cost a workspace
    round trip and a combine pass, so on graphs with enough rows to keep every wavefront slot of the GPU busy
    with whole rows (8 rows per slot) it is the smallest of 64, 128, 256 that leaves 90 % of the non-empty rows
    whole; on smaller graphs the extra wavefronts that segments of 64 provide are worth more (both measured)."""
    if len(row) == 0 or n_rows < 8 * 3072:
        return 64
    r = np.asarray(row)
    if r.min() < 0 or r.max() >= max(n_rows, 1):
        return 64                                   # malformed: the C validation reports it
    deg = np.bincount(r, weights=np.diff(np.asarray(indptr)).astype(np.float64), minlength=max(n_rows, 1))
    deg = deg[deg > 0]
    if len(deg) == 0:
        return 64
    q90 = float(np.quantile(deg, 0.9))
    return 64 if q90 <= 64 else (128 if q90 <= 128 else 256)


def build_plan_host(row, indptr, eid, indices, n_rows, n_index_nodes, seg_len=DEFAULT_SEG_LEN):
    """Pure host step (no GPU): returns (arrays, info) with arrays = dict of int32 numpy arrays
    rowptr, idx, eid, items (n_items, 4), heavy (n_heavy, 3).  Raises ValueError on malformed input."""
    row, indptr, eid, indices = map(_host_i64, (row, indptr, eid, indices))
    if len(indptr) != len(row) + 1:
        raise ValueError("indptr must have len(row) + 1 entries")
    if seg_len is None:
        seg_len = FORCE_SEG_LEN if FORCE_SEG_LEN is not None else auto_seg_len(row, indptr, int(n_rows))
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
    arrays["seg_len"] = int(seg_len)
    return arrays, info


def build_groups_host(arrays, n_index_nodes, R=None, window=GROUP_WINDOW, order_mode=None, max_pairs=None):
    """Pure host step: clusters the plan's items into row groups (bptg_group_plan).  Returns a dict
    with members (n_groups, R, 2), grp_ptr (n_groups + 1), entries (n_entries, 4), pair_eid (n_edges),
    chunks (9,), and slot_eid (n_entries, R): the edge id of (entry, member), -1 where the entry's
    mask has no such member."""
    order_mode = GROUP_ORDER if order_mode is None else order_mode
    R = GROUP_R if R is None else R
    if max_pairs is None:      # 48 edges per member row, more where the work items themselves are longer than 64 edges
        max_pairs = 48 * R * max(1, arrays.get("seg_len", 64) // 64) if GROUP_MAX_PAIRS is None else GROUP_MAX_PAIRS
    items = np.ascontiguousarray(arrays["items"], dtype=np.int32)
    idx = np.ascontiguousarray(arrays["idx"], dtype=np.int32)
    eid = np.ascontiguousarray(arrays["eid"], dtype=np.int32)
    n_items, E = len(items), len(eid)
    members = np.empty((max(n_items, 1), R, 2), dtype=np.int32)
    grp_ptr = np.empty(n_items + 1, dtype=np.int32)
    entries = np.empty((E + 1, 4), dtype=np.int32)
    pair_eid = np.empty(max(E, 1), dtype=np.int32)
    slot_eid = np.empty((max(E, 1), R), dtype=np.int32)
    chunks = np.zeros(9, dtype=np.int32)
    ng, ne = ctypes.c_int64(), ctypes.c_int64()
    check_graph(graph_lib().bptg_group_plan(_ptr(items), n_items, _ptr(idx), _ptr(eid), E, int(n_index_nodes), R, window,
                                            int(order_mode), int(max_pairs), _ptr(members), _ptr(grp_ptr), _ptr(entries), _ptr(pair_eid),
                                            _ptr(slot_eid), _ptr(chunks), ctypes.byref(ng), ctypes.byref(ne)))
    entries[ne.value] = 0                  # one zero row of padding: kernels may peek at entries[n_entries]
    return {"members": members[:ng.value].copy(), "grp_ptr": grp_ptr[:ng.value + 1].copy(),
            "entries": entries[:ne.value].copy(), "pair_eid": pair_eid[:E].copy(), "slot_eid": slot_eid[:ne.value].copy(),
            "chunks": chunks, "R": R}


def link_groups_host(grp_dst, grp_src, n_edges):
    """Pure host step (bptg_link_groups): for every (entry, member) of the destination-side groups, the position
    entry' * R + member' of the same edge in the source-side groups; where the entry has no such member, and in
    the GROUP_PAD_ENTRIES * R elements of padding, the spare position (n_entries_src + GROUP_PAD_ENTRIES) * R - 1
    (the last one of the source side's padding, which no kernel uses).  int32, length
    (n_entries_dst + GROUP_PAD_ENTRIES) * R."""
    sd = np.ascontiguousarray(grp_dst["slot_eid"], dtype=np.int32)
    ss = np.ascontiguousarray(grp_src["slot_eid"], dtype=np.int32)
    out = np.empty((len(sd) + GROUP_PAD_ENTRIES) * grp_dst["R"], dtype=np.int32)
    st = graph_lib().bptg_link_groups(_ptr(sd), len(sd), grp_dst["R"], _ptr(ss), len(ss), grp_src["R"], int(n_edges),
                                      GROUP_PAD_ENTRIES, _ptr(out))
    if st == -4:          # BPTG_ERR_RANGE
        raise ValueError("the source-side groups do not cover every edge exactly once")
    check_graph(st)
    return out


def _bias_rows_of(groups_struct, pair_eid, eids, n_edges):
    """For a plan's tile groups: the struct with bias_by_pair set (the per-edge score term is read, and its gradient
    written, head-major at the plan's own pair numbers), the pair number of every edge id, and for every pair number its
    member index in its tile (the position of its bit in its entry's mask), int32."""
    pair_of_eid = torch.empty(n_edges, dtype=torch.int64, device=pair_eid.device)
    pair_of_eid[pair_eid[:n_edges].to(torch.int64)] = torch.arange(n_edges, dtype=torch.int64, device=pair_eid.device)
    # eids is (entries, R) with n_edges where an entry has no such member: the pairs in their own order are its other elements
    R = int(groups_struct.grp_R)
    member = (torch.nonzero(eids.reshape(-1) < n_edges).flatten() % R).to(torch.int32)
    st = PlanStruct.from_buffer_copy(groups_struct)
    st.bias_by_pair = 1
    return {"struct": st, "pair_of_eid": pair_of_eid, "member_of_pair": member}


def pair_numbers_host(grp_mine, grp_theirs, n_edges):
    """For every (entry, member) of `grp_mine` the number, among the pairs of `grp_theirs`, of the pair that is the same
    edge (pairs are numbered entry by entry, members ascending: grp["pair_eid"][number] = edge id); 0 where the entry has
    no such member and in the GROUP_PAD_ENTRIES * R elements of padding.  int32, length (n_entries + GROUP_PAD_ENTRIES) * R."""
    pe = np.asarray(grp_theirs["pair_eid"], dtype=np.int64)
    if len(pe) != n_edges or (n_edges and (np.bincount(pe, minlength=n_edges) != 1).any()):
        raise ValueError("the partner's groups do not cover every edge exactly once")
    number = np.zeros(n_edges + 1, dtype=np.int32)
    number[pe] = np.arange(n_edges, dtype=np.int32)
    se = np.asarray(grp_mine["slot_eid"], dtype=np.int64)
    out = np.zeros((len(se) + GROUP_PAD_ENTRIES) * grp_mine["R"], dtype=np.int32)
    out[:se.size] = np.where(se >= 0, number[np.maximum(se, 0)], 0).reshape(-1)
    return out


def _tensor_bytes(obj):
    """Bytes of the torch tensors reachable from a plan's containers (dicts, tuples, lists)."""
    if isinstance(obj, torch.Tensor):
        return obj.numel() * obj.element_size()
    if isinstance(obj, dict):
        return sum(_tensor_bytes(v) for k, v in obj.items() if k != "host")
    if isinstance(obj, (tuple, list)):
        return sum(_tensor_bytes(v) for v in obj if not isinstance(v, (Plan, DevicePlan)))
    return 0


class Plan:
    """Device-resident plan of one CSR side; `.struct` is the `bpt_plan` passed to the C ABI."""

    def device_bytes(self):
        """Device memory held by this plan, its row groups and pair mappings."""
        return (_tensor_bytes(self._dev) + _tensor_bytes(list(self._groups.values())) + _tensor_bytes(list(self._links.values()))
                + _tensor_bytes(list(self._bias_rows.values())))

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
        self._groups = {}
        self._links = {}
        self._bias_rows = {}
        self._lock = threading.Lock()
        # one allocation, 256-byte aligned sections (the items array is read as 16-byte vectors)
        self.seg_len = arrays["seg_len"]
        self._dev = {k: torch.from_numpy(v).to(self.device) for k, v in arrays.items() if isinstance(v, np.ndarray)}
        d = self._dev
        self.struct = PlanStruct(
            d["rowptr"].data_ptr(), d["idx"].data_ptr() if self.n_edges else None,
            d["eid"].data_ptr() if self.n_edges else None, d["items"].data_ptr() if self.n_items else None,
            d["heavy"].data_ptr() if self.n_heavy else None,
            self.n_rows, self.n_edges, self.n_items, self.n_heavy, self.n_slots)
        self.struct.n_index_nodes = self.n_index_nodes

    @property
    def ref(self):
        return ctypes.byref(self.struct)

    # ---- row groups for the fused attention kernels ----
    def default_order(self, R):
        """The group order where a caller names none: tile groups by tile_order_dst, the others GROUP_ORDER."""
        return tile_order_dst(self.n_index_nodes) if R == TILE_GROUP_R else GROUP_ORDER

    def ensure_groups(self, R=GROUP_R, order_mode=None):
        """Builds the row-group arrays for groups of R rows once (host) and uploads them.  Returns a dict with
        the host arrays ("host") and the `bpt_plan` carrying them ("struct").  Groups of TILE_GROUP_R rows (the dense-tile
        kernels) have no cap on their edges: a tile costs the same whether its pairs exist or not."""
        order_mode = self.default_order(R) if order_mode is None else order_mode
        with self._lock:
            hit = self._groups.get((R, order_mode))
            if hit is None:
                grp = build_groups_host(self._host, self.n_index_nodes, R=R, order_mode=order_mode,
                                        max_pairs=TILE_MAX_PAIRS if R == TILE_GROUP_R else None)
                # edge id of every (entry, member); absent members and the padding point at the spare row n_edges
                eids = np.full((len(grp["entries"]) + GROUP_PAD_ENTRIES, R), self.n_edges, dtype=np.int32)
                se = grp["slot_eid"]
                eids[:len(se)] = np.where(se >= 0, se, self.n_edges)
                grp["eids"] = eids
                dev = {k: torch.from_numpy(grp[k]).to(self.device) for k in ("members", "grp_ptr", "entries", "chunks", "eids")}
                n_groups = len(grp["members"])
                st = PlanStruct.from_buffer_copy(self.struct)
                st.grp_members = dev["members"].data_ptr() if n_groups else None
                st.grp_ptr = dev["grp_ptr"].data_ptr()
                st.grp_entries = dev["entries"].data_ptr() if len(grp["entries"]) else None
                st.grp_pairs = None
                st.grp_chunks = dev["chunks"].data_ptr()
                st.grp_max_chunk = int(np.diff(grp["chunks"]).max()) if n_groups else 0
                st.n_groups = n_groups
                st.grp_R = R
                st.n_grp_entries = len(grp["entries"])
                st.grp_eids = dev["eids"].data_ptr()
                hit = {"host": grp, "dev": dev, "struct": st}
                self._groups[(R, order_mode)] = hit
        return hit

    def bias_rows(self, R=TILE_GROUP_R):
        """The tile groups for a per-edge score term stored in the order of the plan's own pairs (bias_by_pair): dict
        with "struct" (the `bpt_plan`), "pair_of_eid" (the pair number of every edge id) and "member_of_pair" (the member
        index of every pair in its tile).  Needs a plan that covers every edge."""
        with self._lock:
            hit = self._bias_rows.get(R)
        if hit is None:
            g = self.ensure_groups(R)
            pair_eid = torch.from_numpy(np.ascontiguousarray(g["host"]["pair_eid"])).to(self.device)
            hit = _bias_rows_of(g["struct"], pair_eid, g["dev"]["eids"], self.n_edges)
            if self.device.type == "cuda":
                torch.cuda.current_stream(self.device).synchronize()      # complete before another stream may read it
            with self._lock:
                self._bias_rows[R] = hit
        return hit

    def linked_to(self, plan_src, R=GROUP_R, order=None, partner_order=GROUP_ORDER_SRC, pair_numbers=False):
        """`bpt_plan` of this plan whose grp_pairs maps each (entry, member) of its groups (built with `order`) to the
        position entry' * R + member' of the same edge in the groups of `plan_src` (the plan of the other CSR side of the
        same graph, groups built with `partner_order`) or, with pair_numbers, to the NUMBER of that pair there (the
        entry's first pair + the rank of the member in its mask; 0 where the pair does not exist).  The row-group kernels
        link the destination side to the source side by positions, the tile kernels the source side to the destination
        side by pair numbers."""
        o_mine, o_theirs = (self.default_order(R) if order is None else order), (plan_src.default_order(R) if partner_order is None else partner_order)
        if isinstance(plan_src, Plan) and plan_src is not self and (R, o_mine) not in self._groups and (R, o_theirs) not in plan_src._groups:
            # both sides still to be grouped: the partner's groups are built on a second thread meanwhile (the builder
            # is a plain C function, called with the interpreter lock released)
            other = _group_pool().submit(plan_src.ensure_groups, R, partner_order)
            mine = self.ensure_groups(R, order)
            theirs = other.result()
        else:
            mine, theirs = self.ensure_groups(R, order), plan_src.ensure_groups(R, partner_order)
        key = (id(plan_src), R, order, partner_order) + ((True,) if pair_numbers else ())
        with self._lock:
            hit = self._links.get(key)
            if hit is None:
                if self.n_edges != plan_src.n_edges or not (self.covers_all_edges and plan_src.covers_all_edges):
                    raise ValueError("the two plans do not describe the same edge set")
                if pair_numbers:
                    pairs = torch.from_numpy(pair_numbers_host(mine["host"], theirs["host"], self.n_edges)).to(self.device)
                else:
                    pairs = torch.from_numpy(link_groups_host(mine["host"], theirs["host"], self.n_edges)).to(self.device)
                st = PlanStruct.from_buffer_copy(mine["struct"])
                st.grp_pairs = pairs.data_ptr()
                hit = (st, pairs, plan_src)          # keeps the mapping and the partner alive
                self._links[key] = hit
        return hit[0]


_GROUP_POOL = None


def _group_pool():
    global _GROUP_POOL
    if _GROUP_POOL is None:
        import concurrent.futures
        _GROUP_POOL = concurrent.futures.ThreadPoolExecutor(max_workers=1, thread_name_prefix="bpt-groups")
    return _GROUP_POOL


def set_device_build(on):
    """Plans of graphs seen from now on are built on the GPU (True: DevicePlan), on the host (False: Plan), or where
    their size says (None, the default: on the GPU from DEVICE_BUILD_MIN_ROWS rows, or from 2^17 edges at an average
    degree of DEVICE_BUILD_MIN_DEGREE and DEVICE_BUILD_DENSE_MIN_ROWS rows).  Returns the old setting."""
    global DEVICE_BUILD
    old, DEVICE_BUILD = DEVICE_BUILD, (None if on is None else bool(on))
    return old


def _build_on_device(eid, n_rows):
    if not eid.is_cuda:
        return False
    if DEVICE_BUILD is None:
        if n_rows is None:
            return False
        n_edges = int(eid.numel())
        return n_rows >= DEVICE_BUILD_MIN_ROWS or (n_rows >= DEVICE_BUILD_DENSE_MIN_ROWS and n_edges >= (1 << 17) and
                                                   n_edges >= DEVICE_BUILD_MIN_DEGREE * n_rows)
    return DEVICE_BUILD


_PLAN_ERRORS = {1: "row id, column id or edge id out of range", 2: "row / indptr not sorted", 3: "sizes out of the int32 range"}


def _check_plan(status, what):
    if status != 0:
        raise RuntimeError(f"{what}: status {status}" + (" (HIP error)" if status > 0 else ""))


class _Groups(dict):
    """Row-group record of a DevicePlan; the host copies ("host") are downloaded when first asked for."""

    def __missing__(self, key):
        if key != "host":
            raise KeyError(key)
        dev, R = self["dev"], self["R"]
        ne = self["struct"].n_grp_entries
        eids = dev["eids"][:ne * R].view(ne, R).cpu().numpy()
        host = {"members": dev["members"].cpu().numpy(), "grp_ptr": dev["grp_ptr"].cpu().numpy(),
                "entries": dev["entries"][:ne].cpu().numpy(), "pair_eid": dev["pair_eid"].cpu().numpy(),
                "slot_eid": np.where(eids < self["n_edges"], eids, -1).astype(np.int32),
                "chunks": dev["chunks"].cpu().numpy(), "R": R}
        self["host"] = host
        return host


class DevicePlan:
    """Plan of one CSR side built on the GPU from the reference's int64 device tensors (include/bptplan.h): no copy
    of the index arrays to the host, only the 16-int size blocks come back.  Same interface as Plan."""

    device_bytes = Plan.device_bytes

    def __init__(self, row, indptr, eid, indices, n_rows, n_index_nodes, device, seg_len=DEFAULT_SEG_LEN):
        self.device = torch.device(device)
        self.n_rows, self.n_edges, self.n_index_nodes = int(n_rows), int(eid.numel()), int(n_index_nodes)
        self.has_indices = indices is not None
        if indptr.numel() != row.numel() + 1:
            raise ValueError("indptr must have len(row) + 1 entries")
        if indices is not None and indices.numel() != eid.numel():
            raise ValueError("indices and eid must have the same length")
        if seg_len is None:
            seg_len = FORCE_SEG_LEN if FORCE_SEG_LEN is not None else self._auto_seg_len(row, indptr)
        self.seg_len = int(seg_len)
        self._groups, self._links, self._bias_rows, self._lock = {}, {}, {}, threading.Lock()
        lib = plan_lib()
        U, E = int(row.numel()), self.n_edges
        b = (ctypes.c_int64 * 4)()
        _check_plan(lib.bpt_plan_device_bounds(U, E, self.n_rows, self.seg_len, 0, ctypes.byref(b)), "bpt_plan_device_bounds")
        self._max_items, max_heavy = int(b[0]), int(b[1])
        i32 = lambda *shape: torch.empty(shape, dtype=torch.int32, device=self.device)
        rowptr, idx, eid32 = i32(self.n_rows + 1), i32(max(E, 1)), i32(max(E, 1))
        items, heavy, info = i32(max(self._max_items, 1), 4), i32(max(max_heavy, 1), 3), i32(16)
        ws = torch.empty(int(b[3]), dtype=torch.uint8, device=self.device)
        with torch.cuda.device(self.device):
            st = lib.bpt_plan_build_device(row.data_ptr() if U else None, indptr.data_ptr() if U else None, U,
                                           eid.data_ptr() if E else None,
                                           indices.data_ptr() if (indices is not None and E) else None, E, self.n_rows,
                                           self.n_index_nodes, self.seg_len, rowptr.data_ptr(), idx.data_ptr(),
                                           eid32.data_ptr(), items.data_ptr(), heavy.data_ptr(), info.data_ptr(),
                                           ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
        _check_plan(st, "bpt_plan_build_device")
        h = info.cpu().tolist()                       # the one synchronisation of the build
        if h[0] != 0:
            raise ValueError("bptplan: " + _PLAN_ERRORS.get(h[0], f"error {h[0]}"))
        self.n_items, self.n_heavy, self.n_slots, self.max_degree = h[1], h[2], h[3], h[4]
        self.covers_all_edges = bool(h[5] & 1)
        self._info = info
        # the work lists were allocated for their upper bounds: keep what the build produced
        items, heavy = items[:max(self.n_items, 1)].clone(), heavy[:max(self.n_heavy, 1)].clone()
        self._max_items = max(self.n_items, 1)
        self._dev = {"rowptr": rowptr, "idx": idx, "eid": eid32, "items": items, "heavy": heavy}
        d = self._dev
        torch.cuda.current_stream(self.device).synchronize()      # the plan is complete before any stream can use it
        self.struct = PlanStruct(
            d["rowptr"].data_ptr(), d["idx"].data_ptr() if E else None, d["eid"].data_ptr() if E else None,
            d["items"].data_ptr() if self.n_items else None, d["heavy"].data_ptr() if self.n_heavy else None,
            self.n_rows, E, self.n_items, self.n_heavy, self.n_slots)
        self.struct.n_index_nodes = self.n_index_nodes

    def _auto_seg_len(self, row, indptr):
        """auto_seg_len on the device: the 90 % quantile of the non-empty rows' degrees."""
        if row.numel() == 0 or self.n_rows < 8 * 3072:
            return 64
        if int(row.min()) < 0 or int(row.max()) >= self.n_rows:
            return 64                                   # malformed: the validation kernels report it
        deg = torch.zeros(self.n_rows, dtype=torch.int64, device=row.device).index_add_(0, row, indptr[1:] - indptr[:-1])
        deg = deg[deg > 0]
        if deg.numel() == 0:
            return 64
        q90 = float(np.quantile(deg.cpu().numpy(), 0.9))
        return 64 if q90 <= 64 else (128 if q90 <= 128 else 256)

    @property
    def ref(self):
        return ctypes.byref(self.struct)

    def default_order(self, R):
        """The group order where a caller names none: tile groups by tile_order_dst, the others GROUP_ORDER."""
        return tile_order_dst(self.n_index_nodes) if R == TILE_GROUP_R else GROUP_ORDER

    def ensure_groups(self, R=GROUP_R, order_mode=None):
        """Row groups of R rows built on the GPU (bpt_plan_group_device).  Of order_mode only the entry order counts:
        by member mask (+4), or for the aligned order of the host builder (+8), which is sequential by construction, its
        parallel stand-in (entries by neighbour id mod 16, then id); else ascending neighbour."""
        order_mode = self.default_order(R) if order_mode is None else order_mode
        by_mask = (2 if order_mode & 8 else (1 if order_mode & 4 else 0)) + (0 if order_mode & 2 else 4)
        with self._lock:
            hit = self._groups.get((R, by_mask))
            if hit is None:
                lib = plan_lib()
                E = self.n_edges
                b = (ctypes.c_int64 * 4)()
                _check_plan(lib.bpt_plan_device_bounds(0, E, self.n_rows, self.seg_len, R, ctypes.byref(b)),
                            "bpt_plan_device_bounds")
                max_groups = (self._max_items + R - 1) // R
                i32 = lambda *shape: torch.empty(shape, dtype=torch.int32, device=self.device)
                members, grp_ptr, entries = i32(max(max_groups, 1), R, 2), i32(max_groups + 1), i32(E + 1, 4)
                pair_eid, eids, chunks, ginfo = i32(max(E, 1)), i32((E + GROUP_PAD_ENTRIES) * R), i32(9), i32(16)
                ws = torch.empty(int(b[3]), dtype=torch.uint8, device=self.device)
                d = self._dev
                with torch.cuda.device(self.device):
                    st = lib.bpt_plan_group_device(d["items"].data_ptr(), d["idx"].data_ptr(), d["eid"].data_ptr(),
                                                   self._info.data_ptr(), self._max_items, E, self.n_index_nodes,
                                                   self.seg_len, R, int(by_mask), members.data_ptr(), grp_ptr.data_ptr(),
                                                   entries.data_ptr(), pair_eid.data_ptr(), eids.data_ptr(),
                                                   chunks.data_ptr(), ginfo.data_ptr(), ws.data_ptr(), ws.numel(),
                                                   torch.cuda.current_stream().cuda_stream)
                _check_plan(st, "bpt_plan_group_device")
                ng, ne, max_chunk = ginfo.cpu().tolist()[:3]
                dev = {"members": members[:ng].clone(), "grp_ptr": grp_ptr[:ng + 1].clone(),
                       "entries": entries[:ne + 1].clone(), "pair_eid": pair_eid[:E].clone(),
                       "eids": eids[:(ne + GROUP_PAD_ENTRIES) * R].clone(), "chunks": chunks, "ginfo": ginfo}
                st = PlanStruct.from_buffer_copy(self.struct)
                st.grp_members = dev["members"].data_ptr() if ng else None
                st.grp_ptr = dev["grp_ptr"].data_ptr()
                st.grp_entries = dev["entries"].data_ptr()
                st.grp_pairs = None
                st.grp_chunks = dev["chunks"].data_ptr()
                st.grp_max_chunk = max_chunk
                st.n_groups = ng
                st.grp_R = R
                st.n_grp_entries = ne
                st.grp_eids = dev["eids"].data_ptr()
                hit = _Groups(dev=dev, struct=st, R=R, n_edges=E)
                torch.cuda.current_stream(self.device).synchronize()      # the clones above ran on the building stream
                self._groups[(R, by_mask)] = hit
        return hit

    def bias_rows(self, R=TILE_GROUP_R):
        """As Plan.bias_rows, from the groups built on the GPU."""
        with self._lock:
            hit = self._bias_rows.get(R)
        if hit is None:
            g = self.ensure_groups(R)
            hit = _bias_rows_of(g["struct"], g["dev"]["pair_eid"], g["dev"]["eids"], self.n_edges)
            torch.cuda.current_stream(self.device).synchronize()      # complete before another stream may read it
            with self._lock:
                self._bias_rows[R] = hit
        return hit

    def linked_to(self, plan_src, R=GROUP_R, order=None, partner_order=GROUP_ORDER_SRC, pair_numbers=False):
        """As Plan.linked_to, with the pair mapping computed on the GPU (bpt_plan_link_device; the pair numbers by an
        inverse permutation and a gather)."""
        mine, theirs = self.ensure_groups(R, order), plan_src.ensure_groups(R, partner_order)
        key = (id(plan_src), R, order, partner_order) + ((True,) if pair_numbers else ())
        with self._lock:
            hit = self._links.get(key)
            if hit is None:
                if self.n_edges != plan_src.n_edges or not (self.covers_all_edges and plan_src.covers_all_edges):
                    raise ValueError("the two plans do not describe the same edge set")
                E = self.n_edges
                if not isinstance(plan_src, DevicePlan):
                    # the partner was planned on the host (the two sides of a bipartite graph can fall on either side
                    # of the size rule): map the pairs there, from the downloaded group arrays
                    mapped = (pair_numbers_host if pair_numbers else link_groups_host)(mine["host"], theirs["host"], E)
                    pairs = torch.from_numpy(mapped).to(self.device)
                    st = PlanStruct.from_buffer_copy(mine["struct"])
                    st.grp_pairs = pairs.data_ptr()
                    hit = (st, pairs, plan_src)
                    self._links[key] = hit
                    return hit[0]
                if pair_numbers:
                    number = torch.zeros(E + 1, dtype=torch.int32, device=self.device)
                    number[theirs["dev"]["pair_eid"][:E].long()] = torch.arange(E, dtype=torch.int32, device=self.device)
                    pairs = number[mine["dev"]["eids"].long()]          # absent members carry the edge id E: number 0
                    torch.cuda.current_stream(self.device).synchronize()
                    st = PlanStruct.from_buffer_copy(mine["struct"])
                    st.grp_pairs = pairs.data_ptr()
                    hit = (st, pairs, plan_src)
                    self._links[key] = hit
                    return hit[0]
                n_pairs = (mine["struct"].n_grp_entries + GROUP_PAD_ENTRIES) * R
                pairs = torch.empty((E + GROUP_PAD_ENTRIES) * R, dtype=torch.int32, device=self.device)
                ws = torch.empty(4 * max(E, 1) + 512, dtype=torch.uint8, device=self.device)
                with torch.cuda.device(self.device):
                    st = plan_lib().bpt_plan_link_device(mine["dev"]["eids"].data_ptr(), mine["dev"]["ginfo"].data_ptr(), R,
                                                         theirs["dev"]["eids"].data_ptr(), theirs["dev"]["ginfo"].data_ptr(), R,
                                                         E, GROUP_PAD_ENTRIES, pairs.data_ptr(), ws.data_ptr(), ws.numel(),
                                                         torch.cuda.current_stream().cuda_stream)
                _check_plan(st, "bpt_plan_link_device")
                pairs = pairs[:n_pairs].clone()
                torch.cuda.current_stream(self.device).synchronize()      # complete before another stream may read it
                st = PlanStruct.from_buffer_copy(mine["struct"])
                st.grp_pairs = pairs.data_ptr()
                hit = (st, pairs, plan_src)
                self._links[key] = hit
        return hit[0]


class PlanCache:
    """Least-recently-used cache of plans, bounded by a number of entries AND by the device memory the entries hold
    (index arrays, work lists, row groups, pair mappings: about 45 MB per graph at L = 8192, k = 4).  A training loop
    that builds a new graph per batch (graph/lm.py:53-98) therefore keeps at most `max_bytes` of plans alive."""

    def __init__(self, capacity=_CACHE_SIZE, max_bytes=_CACHE_BYTES):
        self._d = collections.OrderedDict()
        self._cap = capacity
        self._max_bytes = max_bytes
        self._lock = threading.Lock()     # forward runs on the Python thread, backward on autograd's
        self.hits = self.misses = 0

    def set_limits(self, capacity=None, max_bytes=None):
        """Change the number of plans kept and / or the device bytes they may hold together; returns the old pair."""
        with self._lock:
            old = (self._cap, self._max_bytes)
            if capacity is not None:
                self._cap = max(1, int(capacity))
            if max_bytes is not None:
                self._max_bytes = max(0, int(max_bytes))
            self._evict()
        return old

    def device_bytes(self):
        with self._lock:
            return sum(p.device_bytes() + _tensor_bytes(list(t for t in ts if t is not None and t.is_cuda)) for p, ts in self._d.values())

    def _evict(self):
        # called with the lock held; the newest entry always stays
        while len(self._d) > self._cap:
            self._d.popitem(last=False)
        if len(self._d) > 1:
            total = sum(p.device_bytes() for p, _ in self._d.values())
            while len(self._d) > 1 and total > self._max_bytes:
                _, (p, _) = self._d.popitem(last=False)
                total -= p.device_bytes()

    @staticmethod
    def _key(tensors, n_rows, n_index, seg_len, on_device):
        return tuple((t.data_ptr(), t.numel(), t._version, t.device) if t is not None else None
                     for t in tensors) + (n_rows, n_index, seg_len, on_device)

    def get(self, row, indptr, eid, indices, n_rows=None, n_index_nodes=None, seg_len=DEFAULT_SEG_LEN, prefer_device=False):
        """n_rows None: as many rows as `row` mentions (ops that only produce edge outputs).  prefer_device: build on the GPU
        whatever the graph's size, unless set_device_build() fixed the place (the tile kernels ask for this: the GPU
        builder's groups of 16 run them as fast or faster on every graph measured)."""
        tensors = (row, indptr, eid, indices)
        on_device = _build_on_device(eid, n_rows) or bool(prefer_device and DEVICE_BUILD is None and eid.is_cuda and n_rows is not None)
        key = self._key(tensors, n_rows, n_index_nodes, seg_len, on_device)
        with self._lock:
            hit = self._d.get(key)
            if hit is not None:
                self._d.move_to_end(key)
                self.hits += 1
                if self.hits % 64 == 0:
                    self._evict()                   # row groups and pair mappings are added to plans after insertion
                return hit[0]
        self.misses += 1
        if on_device:
            nr = n_rows if n_rows is not None else (int(row[-1]) + 1 if row.numel() else 0)
            ni = n_index_nodes if n_index_nodes is not None else nr
            plan = DevicePlan(row, indptr, eid, indices, nr, ni, eid.device, seg_len)
        else:
            row_h = _host_i64(row)
            nr = n_rows if n_rows is not None else (int(row_h[-1]) + 1 if len(row_h) else 0)
            ni = n_index_nodes if n_index_nodes is not None else nr
            plan = Plan(row_h, indptr, eid, indices, nr, ni, eid.device, seg_len)
        with self._lock:
            self._d[key] = (plan, tensors)          # tensors kept alive with the entry
            self._evict()
        return plan

    def clear(self):
        with self._lock:
            self._d.clear()

    def held(self):
        """The plans in the cache right now (with the index tensors they were built from), as a list the caller keeps.
        Launched kernels read plan arrays through raw pointers that only these objects keep alive: whoever replays work
        later than the cache may evict its plans (a captured HIP graph of a step, replayed after many other graphs went
        through the cache) holds on to this list for as long as the replay may run."""
        with self._lock:
            return list(self._d.values())


plan_cache = PlanCache()
