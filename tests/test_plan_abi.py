"""Host logic of the launch plan, and that the shared libraries load and export every symbol
their headers declare (no GPU needed, no compute calls)."""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle
from bpt_amd import _lib
from bpt_amd import graphbuilder as gb
from bpt_amd.plan import build_plan_host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"\w+)\s*\(", text)))


def test_libraries_export_every_declared_symbol():
    g = _declared("bptgraph.h", "bptg_")
    a = sorted(_declared("bptattn.h", "bpt_") + _declared("bptattn_measure.h", "bpt_"))
    assert len(g) >= 8 and len(a) >= 13
    # the drop-in header carries no process-global hooks: those live in the measurement header
    assert not {"bpt_profile_kernel", "bpt_gather_probe", "bpt_set_force_generic"} & set(_declared("bptattn.h", "bpt_"))
    glib, alib = _lib.graph_lib(), _lib.attn_lib()
    for name in g:
        assert hasattr(glib, name), name
    for name in a:
        assert hasattr(alib, name), name
    p = sorted(_declared("bptplan.h", "bpt_plan_") + _declared("bptplan.h", "bpt_csr_") + _declared("bptplan.h", "bpt_graph_"))
    assert len(p) == 8
    plib = _lib.plan_lib()
    for name in p:
        assert hasattr(plib, name), name
    # the Python bindings cover exactly the declared API
    assert sorted(_lib.GRAPH_API) == g and sorted(_lib.ATTN_API) == a and sorted(_lib.PLAN_API) == p


def _header_plan_fields():
    """(name, is_pointer) of every member of `bpt_plan` as include/bptattn.h declares it, in order."""
    text = open(os.path.join(ROOT, "include", "bptattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    body = re.search(r"typedef struct \{(.*?)\} bpt_plan;", text, flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        m = re.match(r"(const\s+)?(int32_t|int64_t)\s+(.*)", decl, flags=re.S)
        assert m, decl
        for name in m.group(3).split(","):
            name = name.strip()
            fields.append((name.lstrip("* "), name.startswith("*")))
    return fields


def test_binding_mirrors_the_plan_struct_of_the_header():
    """The ctypes mirror has the header's members in the header's order, and its size is the library's sizeof(bpt_plan):
    a binding that is one member short would make the library read past the caller's struct."""
    fields = _header_plan_fields()
    mirror = [(n, t is ctypes.c_void_p) for n, t in _lib.PlanStruct._fields_]
    assert mirror == fields
    assert all(t in (ctypes.c_void_p, ctypes.c_int64) for _, t in _lib.PlanStruct._fields_)
    assert _lib.attn_lib().bpt_plan_struct_bytes() == ctypes.sizeof(_lib.PlanStruct) == 8 * len(fields)


def test_integration_document_shows_the_whole_plan_struct():
    """The ctypes stub printed for integrators names every member of bpt_plan."""
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    for name, _ in _header_plan_fields():
        assert '"' + name + '"' in doc, name
    assert "bpt_plan_struct_bytes" in doc


def test_error_strings_and_argument_errors_without_gpu():
    alib = _lib.attn_lib()
    assert alib.bpt_strerror(0) == b"ok" and b"workspace" in alib.bpt_strerror(-5)
    # argument errors are detected before anything touches the device
    assert alib.bpt_maskedmm_csr_forward(None, None, None, None, 8, 64, 0, None) == -1
    plan = _lib.PlanStruct(None, None, None, None, None, 0, 0, 0, 0, 0)
    assert alib.bpt_sparse_softmax_forward(ctypes.byref(plan), None, None, None, 0, 8, 7, None) == -3          # dtype
    assert alib.bpt_vector_spmm_forward(ctypes.byref(plan), None, None, None, None, 0, 0, 64, 0, None) == -4   # h = 0
    plan_bad = _lib.PlanStruct(None, None, None, None, None, 0, -1, 0, 0, 0)
    assert alib.bpt_sparse_softmax_forward(ctypes.byref(plan_bad), None, None, None, 0, 8, 0, None) == -2
    assert alib.bpt_workspace_bytes(5, ctypes.byref(plan), None, 8, 64, 0) == 0
    assert _lib.graph_lib().bptg_strerror(-4).startswith(b"row id")
    plib = _lib.plan_lib()
    assert plib.bpt_plan_device_bounds(0, -1, 0, 64, 0, ctypes.byref((ctypes.c_int64 * 4)())) == -2            # size
    assert plib.bpt_plan_device_bounds(0, 0, 0, 64, 0, None) == -1
    assert plib.bpt_plan_group_device(None, None, None, None, 0, 0, 0, 64, 17, 0, None, None, None, None, None, None, None,
                                      None, 0, None) == -4                                                    # R
    assert plib.bpt_plan_link_device(None, None, 4, None, None, 4, 10, 8, None, None, 0, None) == -1
    assert plib.bpt_csr_device_bounds(10, 10, 0, ctypes.byref((ctypes.c_int64 * 2)())) == -4                  # chunk size
    assert plib.bpt_csr_build_device(None, None, -1, 0, 32, None, None, None, None, None, None, None, 0, None) == -2
    assert plib.bpt_graph_count_device(0, 0, 1, 4, 10, None, None, 0, None) == -2                             # length < 1
    assert plib.bpt_graph_fill_device(2, 8, 1, 4, 5, 0, None, 0, None, None, None, None) == -2                # c > stride


def _bpt_csr(L, triu, step):
    g = gb.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    return g, src, dst, gb.get_csrs(src, dst, g.number_of_nodes, as_torch=False)


@pytest.mark.parametrize("seg", [4, 64])
@pytest.mark.parametrize("L,triu,step", [(64, True, 4), (37, False, 2), (1, False, 1)])
def test_plan_properties(L, triu, step, seg):
    g, src, dst, (out_csr, in_csr, ROW, IR, COL, IC) = _bpt_csr(L, triu, step)
    n, E = g.number_of_nodes, g.number_of_edges
    for (indptr, indices, eid), units, ip in ((out_csr, ROW, IR), (in_csr, COL, IC)):
        arr, info = build_plan_host(units, ip, eid, indices, n, n, seg)
        assert np.array_equal(arr["rowptr"], indptr)                      # row-level indptr recovered from the units
        assert np.array_equal(arr["idx"], indices) and np.array_equal(arr["eid"], eid)
        items, heavy = arr["items"], arr["heavy"]
        assert info.flags & 1 and info.max_degree == np.diff(indptr).max()
        # items tile every row exactly once, in order, each at most seg long
        assert np.all(items[:, 2] - items[:, 1] <= seg)
        assert set(items[:, 0].tolist()) == set(range(n))
        # locality order: non-decreasing smallest neighbour id (empty rows: their own id)
        keys = [indices[b:e].min() if e > b else r for r, b, e, _ in items.tolist()]
        assert np.all(np.diff(keys) >= 0)
        pos = 0
        for r, b, e, slot in sorted(items.tolist(), key=lambda it: (it[1], it[2])):
            if e > b:
                assert b == pos
                pos = e
            assert indptr[r] <= b and e <= indptr[r + 1]
            assert (slot >= 0) == (indptr[r + 1] - indptr[r] > seg)
        assert pos == E
        # heavy rows: consecutive slots, ceil(deg / seg) each
        slots = items[items[:, 3] >= 0]
        slots = slots[np.argsort(slots[:, 3])]
        assert np.array_equal(slots[:, 3], np.arange(info.n_slots))
        for r, s0, ns in heavy.tolist():
            assert ns == -(-(indptr[r + 1] - indptr[r]) // seg)
            assert np.all(slots[s0:s0 + ns, 0] == r)
        assert heavy[:, 2].sum() == info.n_slots


def test_plan_handles_empty_rows_and_partial_edge_cover():
    # 5 nodes, rows 1 and 3 have slots; eid covers 0..4 but the units stop before the last slot
    row = np.array([1, 3]); ip = np.array([0, 2, 4]); eid = np.array([4, 0, 2, 1, 3]); idx = np.array([0, 1, 2, 3, 4])
    arr, info = build_plan_host(row, ip, eid, idx, 5, 5, 64)
    assert arr["rowptr"].tolist() == [0, 0, 2, 2, 4, 4] and info.n_items == 5 and not (info.flags & 1)
    assert arr["items"].tolist() == [[0, 0, 0, -1], [1, 0, 2, -1], [2, 2, 2, -1], [3, 2, 4, -1], [4, 4, 4, -1]]


def test_plan_rejects_malformed_graphs():
    ok = dict(row=np.array([0, 1]), indptr=np.array([0, 1, 2]), eid=np.array([0, 1]), indices=np.array([1, 0]))
    build_plan_host(**ok, n_rows=2, n_index_nodes=2)
    bad = [dict(ok, row=np.array([1, 0])),                 # rows not grouped
           dict(ok, indptr=np.array([0, 2, 1])),           # indptr decreasing
           dict(ok, indices=np.array([1, 2])),             # index out of range
           dict(ok, eid=np.array([0, 2])),                 # edge id out of range
           dict(ok, row=np.array([0, 2])),                 # row id out of range
           dict(ok, indptr=np.array([0, 1, 3]))]           # units beyond the edge arrays
    for kw in bad:
        with pytest.raises(ValueError):
            build_plan_host(**kw, n_rows=2, n_index_nodes=2)
    with pytest.raises(ValueError):
        build_plan_host(ok["row"], np.array([0, 1]), ok["eid"], ok["indices"], 2, 2)


def test_cfg3_plan_numbers():
    """Headline graph: L=8192, k=4, causal."""
    g, src, dst, (out_csr, in_csr, ROW, IR, COL, IC) = _bpt_csr(8192, True, 4)
    assert (g.number_of_nodes, g.number_of_edges, len(COL), len(ROW)) == (16383, 430237, 25475, 21902)
    deg_in = np.diff(in_csr[0])
    assert deg_in[:8192].max() == 46 and deg_in.max() == 8192 and np.diff(out_csr[0]).max() == 3587
    arr, info = build_plan_host(COL, IC, in_csr[2], in_csr[1], 16383, 16383, 64)
    assert info.n_heavy == 127 and info.n_slots == 896


def test_plan_cache_is_bounded_by_entries_and_by_bytes():
    import torch
    from bpt_amd import plan as pm
    graphs = []
    for L in (64, 80, 96, 112):
        g, src, dst, (out_csr, in_csr, ROW, IR, COL, IC) = _bpt_csr(L, True, 2)
        graphs.append((g.number_of_nodes, tuple(torch.from_numpy(a) for a in (COL, IC, in_csr[2], in_csr[1]))))
    cache = pm.PlanCache(capacity=3, max_bytes=1 << 30)
    plans = [cache.get(*args, n, n) for n, args in graphs]
    assert len(cache._d) == 3 and cache.misses == 4                      # the oldest entry went
    assert cache.get(*graphs[3][1], graphs[3][0], graphs[3][0]) is plans[3] and cache.hits == 1
    one = plans[3].device_bytes()
    plans[3].ensure_groups(8)
    assert plans[3].device_bytes() > one                                 # row groups count towards the bytes
    assert cache.device_bytes() >= sum(p.device_bytes() for p in plans[1:])
    old = cache.set_limits(max_bytes=plans[3].device_bytes() + 1)
    assert old == (3, 1 << 30) and len(cache._d) == 1                    # least recently used plans evicted, newest stays
    cache.get(*graphs[0][1], graphs[0][0], graphs[0][0])
    assert len(cache._d) == 1                                            # a plan larger than the budget is still usable once


def test_noalloc_entry_refuses_a_plan_that_does_not_fit_its_scratch():
    alib = _lib.attn_lib()
    big = _lib.PlanStruct(None, None, None, None, None, 0, 0, 0, 0, 10 ** 6)       # a million partial rows
    assert alib.bpt_attention_forward_noalloc(ctypes.byref(big), None, None, None, None, None, None, 0.125, 0.0, 0, 8, 64, 0, None) == -8
    assert b"scratch" in alib.bpt_strerror(-8)


def test_pair_numbers_of_host_built_groups():
    """plan.pair_numbers_host: every (entry, member) of the source-side groups gets the number of the same edge's pair in
    the destination-side groups (pairs numbered entry by entry, members ascending), checked through the edge ids."""
    import numpy as np
    from bpt_amd import graphbuilder as gb, plan
    g = gb.BinaryPartition(300, True, 2, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n, as_torch=False)
    a_in, _ = plan.build_plan_host(COL, IC, in_csr[2], in_csr[1], n, n, 64)
    a_out, _ = plan.build_plan_host(ROW, IR, out_csr[2], out_csr[1], n, n, 64)
    g_in = plan.build_groups_host(a_in, n, R=16, max_pairs=0)
    g_out = plan.build_groups_host(a_out, n, R=16, max_pairs=0)
    pairs = plan.pair_numbers_host(g_out, g_in, len(src))
    se = np.asarray(g_out["slot_eid"]).reshape(-1)
    assert len(pairs) == (len(g_out["slot_eid"]) + plan.GROUP_PAD_ENTRIES) * 16 and not pairs[len(se):].any()
    assert np.array_equal(np.asarray(g_in["pair_eid"])[pairs[:len(se)][se >= 0]], se[se >= 0])      # same edge on both sides
    assert not pairs[:len(se)][se < 0].any()
    # the pair number of (entry, member) on the destination side = the entry's first pair + rank of the member in its mask
    ent = np.asarray(g_in["entries"]).reshape(-1, 4)
    sd = np.asarray(g_in["slot_eid"]).reshape(-1, 16)
    for u in (0, len(ent) // 2, len(ent) - 1):
        members = [m for m in range(16) if (ent[u, 1] >> m) & 1]
        assert [int(g_in["pair_eid"][ent[u, 2] + i]) for i in range(len(members))] == [int(sd[u, m]) for m in members]
    with pytest.raises(ValueError):
        bad = dict(g_in, pair_eid=np.zeros_like(g_in["pair_eid"]))
        plan.pair_numbers_host(g_out, bad, len(src))
