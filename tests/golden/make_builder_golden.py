#!/usr/bin/env python3
"""Write golden vectors for the host graph builder from the reference's own Cython module.

Runs ONLY in the build container (needs /root/reference). It cythonizes
/root/reference/graph_builder/builder.pyx where it lies, compiles the generated C++ into
oracle/_ref/ (git-ignored; nothing of the reference enters the repository) and dumps, for a grid
of constructor arguments, the arrays the reference returns:

  BinaryPartition(length, triu, step, clip_dist)  -> get_edges(), get_pos(), counts
  FullyConnected(length, triu, window)            -> get_edges(), get_pos()
  OpenAISparse(length, stride, c)                 -> get_edges(), get_pos()
  partition_csr(indptr, chunk_size)               -> row, indptr_

Small cases are stored verbatim in builder_small.npz; large cases (the benchmark sizes) are stored
as SHA-256 digests of the little-endian int64 arrays in builder_digests.json.

Usage:  python tests/golden/make_builder_golden.py
"""
import hashlib
import importlib.util
import json
import os
import subprocess
import sys
import sysconfig

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF_PYX = "/root/reference/graph_builder/builder.pyx"
OUT_DIR = os.path.join(ROOT, "oracle", "_ref")


def build_reference_builder():
    """Compile the reference's builder.pyx into oracle/_ref/ (the built module only).  The generated C++
    is reference source in another form: it is written to a temporary directory and removed after the
    compile, so that it neither stays in the tree nor travels anywhere with it."""
    import shutil
    import tempfile
    os.makedirs(OUT_DIR, exist_ok=True)
    stale = os.path.join(OUT_DIR, "ref_builder.cpp")
    if os.path.exists(stale):
        os.remove(stale)
    # cython names the module after the .pyx file: PyInit_builder
    so = os.path.join(OUT_DIR, "builder" + sysconfig.get_config_var("EXT_SUFFIX"))
    tmp = tempfile.mkdtemp(prefix="bpt_ref_builder_")
    try:
        cpp = os.path.join(tmp, "ref_builder.cpp")
        subprocess.check_call([sys.executable, "-m", "cython", "--cplus", "-2", REF_PYX, "-o", cpp])
        subprocess.check_call([
            "g++", "-O2", "-shared", "-fPIC", "-w",
            "-DNPY_NO_DEPRECATED_API=NPY_1_7_API_VERSION",
            "-I", sysconfig.get_paths()["include"], "-I", np.get_include(),
            cpp, "-o", so])
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    spec = importlib.util.spec_from_file_location("builder", so)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(np.asarray(a).astype("<i8")).tobytes())
    return h.hexdigest()


def main():
    gb = build_reference_builder()
    small = {}
    digests = {}

    # ---- BinaryPartition: small grid stored verbatim
    lengths = [1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 16, 17, 31, 33, 64, 100]
    for L in lengths:
        for triu in (False, True):
            for step in (1, 2, 3, 4, 8):
                for clip in (2, 10):
                    if clip == 2 and step not in (1, 4):
                        continue
                    g = gb.BinaryPartition(L, triu, step, clip)
                    src, dst, et = g.get_edges()
                    key = f"bp_L{L}_t{int(triu)}_s{step}_c{clip}"
                    small[key + "_src"] = src.astype(np.int32)
                    small[key + "_dst"] = dst.astype(np.int32)
                    small[key + "_etype"] = et.astype(np.int32)
                    small[key + "_pos"] = g.get_pos().astype(np.int32)
                    small[key + "_meta"] = np.array(
                        [g.number_of_nodes, g.number_of_edges, g.number_of_levels], dtype=np.int64)
    # v_shift / id helpers on one case
    g = gb.BinaryPartition(13, True, 2, 10)
    s, d, e = g.get_edges(v_shift=100)
    small["bp_shift_src"] = s.astype(np.int64)
    small["bp_shift_dst"] = d.astype(np.int64)
    small["bp_shift_leaf"] = g.leaf_ids(v_shift=100, start=3).astype(np.int64)
    small["bp_shift_internal"] = g.internal_ids(v_shift=100).astype(np.int64)
    small["bp_shift_root"] = np.array([g.root_id(v_shift=100)], dtype=np.int64)
    small["bp_shift_lvls"] = np.array(
        [g.number_of_nodes_at_lvl(i) for i in range(g.number_of_levels)], dtype=np.int64)

    # ---- BinaryPartition: large cases as digests (benchmark configurations)
    big = [(512, False, 4, 10), (512, True, 4, 10), (1000, False, 4, 10), (1023, True, 8, 3),
           (4096, True, 1, 10), (4096, True, 32, 10), (4096, False, 16, 10),
           (8192, True, 4, 10), (8192, True, 64, 7), (32768, True, 8, 10)]
    for (L, triu, step, clip) in big:
        g = gb.BinaryPartition(L, triu, step, clip)
        src, dst, et = g.get_edges()
        digests[f"bp_L{L}_t{int(triu)}_s{step}_c{clip}"] = {
            "n_nodes": int(g.number_of_nodes), "n_edges": int(g.number_of_edges),
            "n_levels": int(g.number_of_levels),
            "sha256_src_dst_etype_pos": digest(src, dst, et, g.get_pos())}

    # ---- FullyConnected
    for L in (1, 2, 5, 17):
        for triu in (False, True):
            for window in (1, 3, 8192):
                g = gb.FullyConnected(L, triu, window)
                src, dst, et = g.get_edges()
                key = f"fc_L{L}_t{int(triu)}_w{window}"
                small[key + "_src"] = src.astype(np.int32)
                small[key + "_dst"] = dst.astype(np.int32)
                small[key + "_etype"] = et.astype(np.int32)
                small[key + "_pos"] = g.get_pos().astype(np.int32)
    for (L, triu, window) in [(4096, True, 128), (4096, False, 128)]:
        g = gb.FullyConnected(L, triu, window)
        src, dst, et = g.get_edges()
        digests[f"fc_L{L}_t{int(triu)}_w{window}"] = {
            "n_nodes": int(g.number_of_nodes), "n_edges": int(g.number_of_edges),
            "sha256_src_dst_etype_pos": digest(src, dst, et, g.get_pos())}

    # ---- OpenAISparse (strided baseline graph)
    for (L, stride, c) in [(1, 4, 1), (9, 4, 2), (32, 8, 3)]:
        g = gb.OpenAISparse(L, stride, c)
        src, dst, et = g.get_edges()
        key = f"oa_L{L}_s{stride}_c{c}"
        small[key + "_src"] = src.astype(np.int32)
        small[key + "_dst"] = dst.astype(np.int32)
        small[key + "_etype"] = et.astype(np.int32)
        small[key + "_pos"] = g.get_pos().astype(np.int32)

    # ---- partition_csr
    rng = np.random.default_rng(7)
    cases = [(np.array([0, 4, 8, 10], dtype=np.int64), 4),
             (np.array([0, 0, 0], dtype=np.int64), 32),
             (np.array([0, 33, 33, 97, 100], dtype=np.int64), 32),
             (np.concatenate([[0], np.cumsum(rng.integers(0, 90, 40))]).astype(np.int64), 32),
             (np.concatenate([[0], np.cumsum(rng.integers(0, 20, 40))]).astype(np.int64), 5)]
    for i, (indptr, chunk) in enumerate(cases):
        row, ip = gb.partition_csr(indptr, chunk)
        small[f"pc{i}_indptr"] = indptr
        small[f"pc{i}_chunk"] = np.array([chunk], dtype=np.int64)
        small[f"pc{i}_row"] = row
        small[f"pc{i}_out"] = ip

    np.savez_compressed(os.path.join(HERE, "builder_small.npz"), **small)
    with open(os.path.join(HERE, "builder_digests.json"), "w") as f:
        json.dump(digests, f, indent=1, sort_keys=True)
    print("wrote", len(small), "arrays and", len(digests), "digests")


if __name__ == "__main__":
    main()
