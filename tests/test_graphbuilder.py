"""Host graph builder of the product (libbptgraph) against the golden vectors written by the
reference's own builder, and against the independent oracle restatement."""
import hashlib
import json
import os
import pickle

import numpy as np
import pytest

import oracle
from bpt_amd import graphbuilder as gb

GOLD = os.path.join(os.path.dirname(__file__), "golden")
SMALL = np.load(os.path.join(GOLD, "builder_small.npz"))
DIGESTS = json.load(open(os.path.join(GOLD, "builder_digests.json")))


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(np.asarray(a).astype("<i8")).tobytes())
    return h.hexdigest()


def _keys(prefix):
    return sorted({k[:-4] for k in SMALL.files if k.startswith(prefix) and k.endswith("_src") and "shift" not in k})


def _args(key):
    return [int(p[1:]) for p in key.split("_")[1:]]


@pytest.mark.parametrize("key", _keys("bp_L"))
def test_binary_partition_golden(key):
    L, triu, step, clip = _args(key)
    g = gb.BinaryPartition(L, bool(triu), step, clip)
    src, dst, et = g.get_edges()
    assert src.dtype == np.int64
    assert [g.number_of_nodes, g.number_of_edges, g.number_of_levels] == SMALL[key + "_meta"].tolist()
    assert np.array_equal(src, SMALL[key + "_src"]) and np.array_equal(dst, SMALL[key + "_dst"])
    assert np.array_equal(et, SMALL[key + "_etype"]) and np.array_equal(g.get_pos(), SMALL[key + "_pos"])


@pytest.mark.parametrize("key", sorted(DIGESTS))
def test_large_digests(key):
    a = _args(key)
    g = gb.BinaryPartition(a[0], bool(a[1]), a[2], a[3]) if key.startswith("bp_") else gb.FullyConnected(a[0], bool(a[1]), a[2])
    src, dst, et = g.get_edges()
    assert (g.number_of_nodes, g.number_of_edges) == (DIGESTS[key]["n_nodes"], DIGESTS[key]["n_edges"])
    assert digest(src, dst, et, g.get_pos()) == DIGESTS[key]["sha256_src_dst_etype_pos"]


@pytest.mark.parametrize("key", _keys("fc_"))
def test_fully_connected_golden(key):
    L, triu, window = _args(key)
    g = gb.FullyConnected(L, bool(triu), window)
    src, dst, et = g.get_edges()
    assert np.array_equal(src, SMALL[key + "_src"]) and np.array_equal(dst, SMALL[key + "_dst"])
    assert np.array_equal(et, SMALL[key + "_etype"]) and np.array_equal(g.get_pos(), SMALL[key + "_pos"])


@pytest.mark.parametrize("key", _keys("oa_"))
def test_openai_sparse_golden(key):
    L, stride, c = _args(key)
    g = gb.OpenAISparse(L, stride, c)
    src, dst, et = g.get_edges()
    assert np.array_equal(src, SMALL[key + "_src"]) and np.array_equal(dst, SMALL[key + "_dst"])
    assert np.array_equal(et, SMALL[key + "_etype"]) and np.array_equal(g.get_pos(), SMALL[key + "_pos"])


def test_api_surface_and_pickle():
    g = gb.BinaryPartition(13, True, 2, 10)
    s, d, _ = g.get_edges(v_shift=100)
    assert np.array_equal(s, SMALL["bp_shift_src"]) and np.array_equal(d, SMALL["bp_shift_dst"])
    assert np.array_equal(g.leaf_ids(v_shift=100, start=3), SMALL["bp_shift_leaf"])
    assert np.array_equal(g.internal_ids(v_shift=100), SMALL["bp_shift_internal"])
    assert g.root_id(v_shift=100) == SMALL["bp_shift_root"][0] and g.is_triu
    assert [g.number_of_nodes_at_lvl(i) for i in range(g.number_of_levels)] == SMALL["bp_shift_lvls"].tolist()
    g2 = pickle.loads(pickle.dumps(g))                    # builder.pyx:38-39
    assert all(np.array_equal(a, b) for a, b in zip(g.get_edges(), g2.get_edges()))
    f2 = pickle.loads(pickle.dumps(gb.FullyConnected(5, True, 3)))
    assert f2.number_of_edges == gb.FullyConnected(5, True, 3).number_of_edges
    with pytest.raises(ValueError):
        gb.BinaryPartition(0)
    with pytest.raises(AssertionError):
        gb.OpenAISparse(8, 4, 1, triu=False)


@pytest.mark.parametrize("i", range(5))
def test_partition_csr_golden(i):
    row, ip = gb.partition_csr(SMALL[f"pc{i}_indptr"], int(SMALL[f"pc{i}_chunk"][0]))
    assert row.dtype == np.int64 and ip.dtype == np.int64
    assert np.array_equal(row, SMALL[f"pc{i}_row"]) and np.array_equal(ip, SMALL[f"pc{i}_out"])


def test_partition_csr_errors():
    with pytest.raises(ValueError):
        gb.partition_csr(np.array([0, 4]), 0)
    with pytest.raises(ValueError):
        gb.partition_csr(np.array([0, 4, 2]), 4)


@pytest.mark.parametrize("L,triu,step", [(37, False, 2), (100, True, 4), (5, False, 1)])
def test_get_csrs_matches_oracle(L, triu, step):
    g = gb.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    got = gb.get_csrs(src, dst, g.number_of_nodes, as_torch=False)
    want = oracle.get_csrs(src, dst, g.number_of_nodes)
    for a, b in zip(got[0] + got[1] + got[2:], want[0] + want[1] + want[2:]):
        assert a.dtype == np.int64 and np.array_equal(a, b)
    t = gb.get_csrs(src, dst, g.number_of_nodes)
    import torch
    assert t[2].dtype == torch.long and t[0][1].dtype == torch.long


def test_build_csr_rejects_out_of_range():
    with pytest.raises(ValueError):
        gb.build_csr(np.array([0, 5]), np.array([0, 1]), 3)


def test_batch_merge_cfg2_shape():
    """benchmark configuration 2: 32 causal graphs with seeded lengths merged block-diagonally."""
    lengths = np.random.default_rng(2345).integers(64, 1025, 32)
    assert lengths[:4].tolist() == [171, 550, 518, 514] and lengths.sum() == 16736
    cache = {}
    gs = [cache.setdefault(int(L), gb.BinaryPartition(int(L), True, 4, 10)) for L in lengths]
    src, dst, et, pos, n = gb.merge_graphs(gs)
    assert (n, len(src)) == (33598, 573520)
    ogs = [oracle.BinaryPartition(int(L), True, 4, 10) for L in lengths[:3]]
    osrc, odst, oet, opos, on = oracle.merge_graphs(ogs)
    assert np.array_equal(src[:len(osrc)], osrc) and np.array_equal(dst[:len(osrc)], odst)
    assert np.array_equal(et[:len(osrc)], oet) and np.array_equal(pos[:on], opos)


@pytest.mark.parametrize("L,triu,step", [(37, False, 2), (100, True, 4), (5, False, 1)])
def test_get_csrs_src_ordered_in_csr(L, triu, step):
    """The opt-in in-CSR order (source, edge id): same indptr, same (index, edge id) pairs per row as the default,
    rows sorted by (source, edge id), which is what scipy's transpose of the out-CSR produces; out-CSR unchanged."""
    import scipy.sparse as sp
    g = gb.BinaryPartition(L, triu, step, 10)        # the non-causal graphs carry duplicate edges
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    base = gb.get_csrs(src, dst, n, as_torch=False)
    alt = gb.get_csrs(src, dst, n, as_torch=False, in_order="src_eid")
    for a, b in zip(base[0] + base[2:], alt[0] + alt[2:]):
        assert np.array_equal(a, b)                                       # out-CSR and the units of both sides
    (ip0, ix0, e0), (ip1, ix1, e1) = base[1], alt[1]
    assert np.array_equal(ip0, ip1)
    for r in range(n):
        a, b = slice(ip0[r], ip0[r + 1]), slice(ip1[r], ip1[r + 1])
        assert sorted(zip(ix0[a], e0[a])) == list(zip(ix1[b], e1[b]))      # same pairs, (source, edge id) ascending
        assert np.all(np.diff(e0[a]) > 0)                                  # default: ascending edge id
    assert np.array_equal(src[e1], ix1) and np.array_equal(dst[e1], np.repeat(np.arange(n), np.diff(ip1)))
    # independent construction: CSR of (dst, src) with data = edge id + 1, duplicates kept, columns sorted stably
    m = sp.csr_matrix((np.arange(len(src)) + 1, (dst, src)), shape=(n, n))
    assert m.nnz == len(src) or not triu          # scipy sums duplicates in the constructor: only compare without them
    if m.nnz == len(src):
        m.sort_indices()
        assert np.array_equal(m.indptr, ip1) and np.array_equal(m.indices, ix1) and np.array_equal(m.data - 1, e1)
    with pytest.raises(ValueError):
        gb.get_csrs(src, dst, n, in_order="random")


def test_inter_graph_edges_follow_the_reference_construction():
    """graph/mt.py:286-321: per sentence pair and segment, np.repeat(source tokens, #target) / np.tile(target tokens,
    #source), node ids shifted by the node counts of the graphs before; graph/nli.py:60-87 for the two-way form."""
    enc = [gb.BinaryPartition(7, False, 2, 10), gb.BinaryPartition(12, False, 2, 10), gb.BinaryPartition(3, False, 2, 10)]
    dec = [gb.BinaryPartition(5, True, 2, 10), gb.BinaryPartition(9, True, 2, 10), gb.BinaryPartition(4, True, 2, 10)]
    seg_e = [None, [0, 4, 12], None]
    seg_d = [None, [0, 6, 9], None]
    src, dst, n_enc, n_dec = gb.inter_graph_edges(enc, dec, seg_e, seg_d)
    assert n_enc == sum(g.number_of_nodes for g in enc) and n_dec == sum(g.number_of_nodes for g in dec)
    # brute force from the definition: (s, t) for every source token s and target token t of the same pair and segment
    want, ve, vd = [], 0, 0
    for ge, gd, se, sd in zip(enc, dec, seg_e, seg_d):
        le, ld = len(ge.leaf_ids()), len(gd.leaf_ids())
        se, sd = se or [0, le], sd or [0, ld]
        for i in range(1, len(se)):
            for s in range(se[i - 1], se[i]):
                for t in range(sd[i - 1], sd[i]):
                    want.append((ve + s, vd + t))
        ve += ge.number_of_nodes
        vd += gd.number_of_nodes
    assert list(zip(src.tolist(), dst.tolist())) == want
    assert len(src) == 7 * 5 + 4 * 6 + 8 * 3 + 3 * 4
    # only tokens carry inter edges: span nodes of both sides have none
    leaf_e = np.concatenate([g.leaf_ids(v_shift=s) for g, s in zip(enc, np.cumsum([0] + [g.number_of_nodes for g in enc[:-1]]))])
    assert set(src.tolist()) <= set(leaf_e.tolist())
    # square (reference) and bipartite CSR forms describe the same edges
    sq = gb.get_csrs(src, dst, max(n_enc, n_dec), as_torch=False)
    bi = gb.get_csrs_bipartite(src, dst, n_enc, n_dec, as_torch=False)
    assert len(bi[0][0]) == n_enc + 1 and len(bi[1][0]) == n_dec + 1
    assert np.array_equal(sq[0][0][:n_enc + 1], bi[0][0]) and np.array_equal(sq[1][0][:n_dec + 1], bi[1][0])
    assert np.array_equal(sq[0][1], bi[0][1]) and np.array_equal(sq[1][2], bi[1][2])
    with pytest.raises(ValueError):
        gb.inter_graph_edges(enc, dec[:2])
    with pytest.raises(ValueError):
        gb.inter_graph_edges(enc[:1], dec[:1], [[0, 3, 7]], [[0, 5]])
    with pytest.raises(ValueError):
        gb.get_csrs_bipartite(src, dst, n_enc, int(dst.max()))

    prem = [gb.BinaryPartition(4, False, 1, 10), gb.BinaryPartition(6, False, 1, 10)]
    hypo = [gb.BinaryPartition(3, False, 1, 10), gb.BinaryPartition(2, False, 1, 10)]
    s2, d2, n2 = gb.nli_inter_graph_edges(prem, hypo)
    assert n2 == sum(g.number_of_nodes for g in prem + hypo) and len(s2) == 2 * (4 * 3 + 6 * 2)
    pairs = set(zip(s2.tolist(), d2.tolist()))
    assert len(pairs) == len(s2) and all((b, a) in pairs for a, b in pairs)                  # two-way, no duplicates
    v0 = prem[0].number_of_nodes
    assert (0, v0) in pairs and (v0 + 2, 3) in pairs and (4, v0) not in pairs                  # node 4 is a span node
