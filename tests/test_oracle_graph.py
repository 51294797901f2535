"""Pins the oracle's graph routines against vectors written by the reference's own Cython builder
(tests/golden/make_builder_golden.py) and against facts the construction fixes by itself."""
import hashlib
import json
import os

import numpy as np
import pytest

import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden")
SMALL = np.load(os.path.join(GOLD, "builder_small.npz"))
DIGESTS = json.load(open(os.path.join(GOLD, "builder_digests.json")))


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(np.asarray(a).astype("<i8")).tobytes())
    return h.hexdigest()


def _bp_keys():
    return sorted({k[: -len("_meta")] for k in SMALL.files if k.startswith("bp_L") and k.endswith("_meta")})


def _parse(key):
    parts = key.split("_")
    return int(parts[1][1:]), bool(int(parts[2][1:])), int(parts[3][1:]), int(parts[4][1:])


@pytest.mark.parametrize("key", _bp_keys())
def test_binary_partition_golden(key):
    L, triu, step, clip = _parse(key)
    g = oracle.BinaryPartition(L, triu, step, clip)
    src, dst, et = g.get_edges()
    assert [g.number_of_nodes, g.number_of_edges, g.number_of_levels] == SMALL[key + "_meta"].tolist()
    assert np.array_equal(src, SMALL[key + "_src"])
    assert np.array_equal(dst, SMALL[key + "_dst"])
    assert np.array_equal(et, SMALL[key + "_etype"])
    assert np.array_equal(g.get_pos(), SMALL[key + "_pos"])


@pytest.mark.parametrize("key", sorted(k for k in DIGESTS if k.startswith("bp_")))
def test_binary_partition_digest(key):
    L, triu, step, clip = _parse(key)
    g = oracle.BinaryPartition(L, triu, step, clip)
    src, dst, et = g.get_edges()
    ref = DIGESTS[key]
    assert (g.number_of_nodes, g.number_of_edges, g.number_of_levels) == (ref["n_nodes"], ref["n_edges"], ref["n_levels"])
    assert digest(src, dst, et, g.get_pos()) == ref["sha256_src_dst_etype_pos"]


def test_shift_and_id_helpers():
    g = oracle.BinaryPartition(13, True, 2, 10)
    s, d, _ = g.get_edges(v_shift=100)
    assert np.array_equal(s, SMALL["bp_shift_src"]) and np.array_equal(d, SMALL["bp_shift_dst"])
    assert np.array_equal(g.leaf_ids(v_shift=100, start=3), SMALL["bp_shift_leaf"])
    assert np.array_equal(g.internal_ids(v_shift=100), SMALL["bp_shift_internal"])
    assert g.root_id(v_shift=100) == SMALL["bp_shift_root"][0]
    assert [g.number_of_nodes_at_lvl(i) for i in range(g.number_of_levels)] == SMALL["bp_shift_lvls"].tolist()


@pytest.mark.parametrize("key", sorted({k[:-4] for k in SMALL.files if k.startswith("fc_") and k.endswith("_src")}))
def test_fully_connected_golden(key):
    parts = key.split("_")
    g = oracle.FullyConnected(int(parts[1][1:]), bool(int(parts[2][1:])), int(parts[3][1:]))
    src, dst, et = g.get_edges()
    assert np.array_equal(src, SMALL[key + "_src"]) and np.array_equal(dst, SMALL[key + "_dst"])
    assert np.array_equal(et, SMALL[key + "_etype"]) and np.array_equal(g.get_pos(), SMALL[key + "_pos"])


@pytest.mark.parametrize("key", sorted(k for k in DIGESTS if k.startswith("fc_")))
def test_fully_connected_digest(key):
    parts = key.split("_")
    g = oracle.FullyConnected(int(parts[1][1:]), bool(int(parts[2][1:])), int(parts[3][1:]))
    src, dst, et = g.get_edges()
    assert (g.number_of_nodes, g.number_of_edges) == (DIGESTS[key]["n_nodes"], DIGESTS[key]["n_edges"])
    assert digest(src, dst, et, g.get_pos()) == DIGESTS[key]["sha256_src_dst_etype_pos"]


@pytest.mark.parametrize("key", sorted({k[:-4] for k in SMALL.files if k.startswith("oa_") and k.endswith("_src")}))
def test_openai_sparse_golden(key):
    parts = key.split("_")
    g = oracle.OpenAISparse(int(parts[1][1:]), int(parts[2][1:]), int(parts[3][1:]))
    src, dst, et = g.get_edges()
    assert np.array_equal(src, SMALL[key + "_src"]) and np.array_equal(dst, SMALL[key + "_dst"])
    assert np.array_equal(et, SMALL[key + "_etype"]) and np.array_equal(g.get_pos(), SMALL[key + "_pos"])


@pytest.mark.parametrize("i", range(5))
def test_partition_csr_golden(i):
    row, ip = oracle.partition_csr(SMALL[f"pc{i}_indptr"], int(SMALL[f"pc{i}_chunk"][0]))
    assert np.array_equal(row, SMALL[f"pc{i}_row"]) and np.array_equal(ip, SMALL[f"pc{i}_out"])


def test_partition_csr_known_answer():
    # graph_kernel/part_csr.py:29-32
    row, ip = oracle.partition_csr(np.array([0, 4, 8, 10]), 4)
    assert row.tolist() == [0, 1, 2] and ip.tolist() == [0, 4, 8, 10]


def test_hand_cases():
    g = oracle.BinaryPartition(1, False, 1, 10)
    assert (g.number_of_nodes, g.number_of_edges) == (1, 1)
    assert [a.tolist() for a in g.get_edges()] == [[0], [0], [0]]
    g = oracle.BinaryPartition(2, True, 4, 10)
    s, d, e = g.get_edges()
    assert list(zip(s.tolist(), d.tolist(), e.tolist())) == [(0, 0, 0), (0, 2, 9), (0, 1, 1), (1, 1, 0), (1, 2, 9)]
    # non power-of-two, non causal: the right-overlap rule emits the duplicate edge 5 -> 3
    g = oracle.BinaryPartition(5, False, 1, 10)
    s, d, e = g.get_edges()
    assert (g.number_of_nodes, g.number_of_edges) == (11, 40)
    assert sum(1 for a, b in zip(s.tolist(), d.tolist()) if (a, b) == (5, 3)) == 2


@pytest.mark.parametrize("L", [1, 2, 3, 7, 64, 100, 257])
@pytest.mark.parametrize("step", [1, 2, 4, 8])
def test_causal_cover_invariant(L, step):
    """Causal graph: the spans of a token's in-neighbours tile [0, i] exactly once."""
    g = oracle.BinaryPartition(L, True, step, 10)
    src, dst, _ = g.get_edges()
    n_lvl = g.number_of_levels
    sizes = [g.number_of_nodes_at_lvl(j) for j in range(n_lvl)]
    shift = np.concatenate([[0], np.cumsum(sizes)])
    assert g.number_of_nodes == sum(-(-L // (1 << j)) for j in range(n_lvl) if -(-L // (1 << j)) >= 1 and (j == 0 or -(-L // (1 << (j - 1))) >= 2))
    lvl_of = np.searchsorted(shift, src, side="right") - 1
    lo = (src - shift[lvl_of]) << lvl_of
    hi = np.minimum(lo + (1 << lvl_of), L)
    tok = dst < L
    cover = np.zeros((L, L + 1), dtype=np.int64)
    for a, b, i in zip(lo[tok], hi[tok], dst[tok]):
        cover[i, a:b] += 1
    for i in range(L):
        assert cover[i, : i + 1].tolist() == [1] * (i + 1) and cover[i, i + 1:].sum() == 0
    # bottom-up edges: one per token per level
    assert int((~tok).sum()) + L == L * n_lvl


def test_get_csrs_layout():
    g = oracle.BinaryPartition(37, False, 2, 10)
    src, dst, _ = g.get_edges()
    n, E = g.number_of_nodes, g.number_of_edges
    out_csr, in_csr, ROW, IR, COL, IC = oracle.get_csrs(src, dst, n)
    for (indptr, indices, eid), rows, cols in ((out_csr, src, dst), (in_csr, dst, src)):
        assert indptr[0] == 0 and indptr[-1] == E and np.all(np.diff(indptr) >= 0)
        assert sorted(eid.tolist()) == list(range(E))
        assert np.array_equal(cols[eid], indices)
        assert np.array_equal(np.repeat(np.arange(n), np.diff(indptr)), rows[eid])
        for r in range(n):                      # inside a row: ascending edge id
            assert np.all(np.diff(eid[indptr[r]:indptr[r + 1]]) > 0)
    for row, ip, indptr in ((ROW, IR, out_csr[0]), (COL, IC, in_csr[0])):
        assert np.all(np.diff(row) >= 0) and np.all(np.diff(ip) <= 32) and np.all(np.diff(ip) > 0)
        assert ip[0] == 0 and ip[-1] == E
        assert np.all(ip[:-1] >= indptr[row]) and np.all(ip[1:] <= indptr[row + 1])


def test_merge_graphs():
    gs = [oracle.BinaryPartition(L, True, 4, 10) for L in (5, 9, 1)]
    src, dst, et, pos, n = oracle.merge_graphs(gs)
    assert n == sum(g.number_of_nodes for g in gs) and len(src) == sum(g.number_of_edges for g in gs)
    off = gs[0].number_of_nodes
    s1, d1, e1 = gs[1].get_edges()
    sl = slice(gs[0].number_of_edges, gs[0].number_of_edges + gs[1].number_of_edges)
    assert np.array_equal(src[sl], s1 + off) and np.array_equal(dst[sl], d1 + off) and np.array_equal(et[sl], e1)
    assert np.array_equal(pos[off:off + gs[1].number_of_nodes], gs[1].get_pos())
