#!/usr/bin/env python3
"""Benchmark of the BPT graph-attention hot path on one MI355X.

A step = one fused attention layer forward + backward (SDDMM -> edge softmax -> SpMM and their
gradients) over one synthetic graph batch, inputs resident in HBM.  Default workload: the headline
configuration (cfg3), L=8192 tokens, k=4, causal binary-partition graph, 8 heads x 64, fp32.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg1|cfg2|cfg5|cfg4-kN|cfg4-w128]
                  [--dtype f32|bf16] [--no-cpu-baseline] [--no-graph] [--block-layers N]

Prints ONE JSON line on stdout (details go to stderr).  `value` = graph edges per second of the
whole fwd+bwd step; `roofline` describes the dominant kernel, timed live with HIP events on the
launch stream; `cpu_baseline` is the PyTorch-CPU restatement of the same arithmetic (oracle/), timed
on this host's cores on the same workload.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published peak


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_workload(name):
    """Returns (description, list of graphs, h, d, default dtype)."""
    import numpy as np
    from bpt_amd import graphbuilder as gb
    if name == "cfg1":
        return "cfg1: L=512 k=4 non-causal BPT graph, 8x64", [gb.BinaryPartition(512, False, 4, 10)], 8, 64, "f32"
    if name == "cfg2":
        lengths = np.random.default_rng(2345).integers(64, 1025, 32)
        cache = {}
        gs = [cache.setdefault(int(L), gb.BinaryPartition(int(L), True, 4, 10)) for L in lengths]
        return "cfg2: 32 causal BPT graphs, L~U[64,1024] (seed 2345), k=4, 8x64", gs, 8, 64, "f32"
    if name == "cfg3":
        return "cfg3: L=8192 k=4 causal BPT graph, 8x64", [gb.BinaryPartition(8192, True, 4, 10)], 8, 64, "f32"
    if name.startswith("long-"):            # e.g. long-32768: cfg3's graph family at another length
        L = int(name[5:])
        return f"L={L} k=4 causal BPT graph, 8x64", [gb.BinaryPartition(L, True, 4, 10)], 8, 64, "f32"
    if name == "cfg5":
        return "cfg5: L=32768 k=8 causal BPT graph, 16x64", [gb.BinaryPartition(32768, True, 8, 10)], 16, 64, "bf16"
    if name.startswith("cfg4-k"):
        k = int(name[6:])
        return f"cfg4: L=4096 k={k} causal BPT graph, 8x64", [gb.BinaryPartition(4096, True, k, 10)], 8, 64, "f32"
    if name == "cfg4-w128":
        return "cfg4: L=4096 window-128 causal dense graph, 8x64", [gb.FullyConnected(4096, True, 128)], 8, 64, "f32"
    raise SystemExit(f"unknown workload {name}")


def algorithmic_bytes(N, E, H, D, s):
    """Compulsory HBM traffic of the fused fwd+bwd step (every distinct input read once per pass, every
    output written once): 12*N*C*s + 2*N*H*4 + 3*E*4 + 2*(N+1)*4, split over the three main kernels so that
    the parts add up to the total: q and dO, which both backward kernels read, are charged half to each."""
    C = H * D
    fwd = 4 * N * C * s + N * H * 4 + E * 4 + (N + 1) * 4          # read q,k,v; write o, lse; in-CSR
    bwd_dst = 5 * N * C * s + N * H * 4 + E * 4                    # read k,v,o + half of (q,dO), lse; write dq; in-CSR
    bwd_src = 3 * N * C * s + E * 4 + (N + 1) * 4                  # half of (q,dO); write dk,dv; out-CSR
    return {"attn_fwd": fwd, "attn_bwd_dst": bwd_dst, "attn_bwd_src": bwd_src, "total": fwd + bwd_dst + bwd_src}


def cpu_baseline(src, dst, N, H, D, seed, budget_s=25.0):
    """PyTorch-CPU gather / index_add restatement (oracle/torch_ops.py), all host threads, fp32."""
    import torch
    from oracle import torch_ops
    gen = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(N, H, D, generator=gen) / 8 for _ in range(4))
    s, d_ = torch.from_numpy(src), torch.from_numpy(dst)
    cores = torch.get_num_threads()
    t0 = time.perf_counter()
    torch_ops.attention_fwd_bwd(s, d_, q, k, v, do)                 # warm-up (allocator, threads)
    warm = time.perf_counter() - t0
    times = []
    while len(times) < 5 and (sum(times) + warm) < budget_s:
        t0 = time.perf_counter()
        torch_ops.attention_fwd_bwd(s, d_, q, k, v, do)
        times.append(time.perf_counter() - t0)
    if not times:
        times = [warm]
    med = sorted(times)[len(times) // 2]
    return {"value": len(src) / med, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": f"{len(times)} timed fwd+bwd passes of the full workload after 1 warm-up (median {med * 1e3:.1f} ms), fp32"}


def timed(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t) / steps


def timed_runs(fn, steps, warmups):
    """Seconds per call of fn, one figure per entry of `warmups` (that many untimed calls, then `steps` timed ones between
    two synchronisations).  Python's cyclic garbage collector is off from before the first warm-up to after the last run,
    as in timeit: a full collection of this process's heap takes 25-45 ms, which a timed region of 30 ms cannot absorb (it
    showed as one run in three at twice the time of the others), and a collection between the runs would leave the GPU
    idle right before a timed region."""
    import gc
    gc_was_on = gc.isenabled()
    gc.collect()
    gc.disable()
    try:
        return [timed(fn, steps, w) for w in warmups]
    finally:
        if gc_was_on:
            gc.enable()


def median(xs):
    return sorted(xs)[len(xs) // 2]


def graph_replay_runs(step, ref, steps, warmup, runs=3):
    """Three timed runs of the replay of a HIP graph of `step`, or [] where capture fails or a replay does not
    reproduce the eager results `ref` bit for bit."""
    import torch
    try:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            gout = step()
        g.replay(); torch.cuda.synchronize()
        g.replay(); torch.cuda.synchronize()
        if ref is not None and not all(torch.equal(a, b) for a, b in zip(gout, ref)):
            log("HIP graph replay did not reproduce the eager result; using eager timing")
            return []
        out = timed_runs(g.replay, steps, [warmup if i == 0 else 2 for i in range(runs)])
        if ref is not None and not all(torch.equal(a, b) for a, b in zip(gout, ref)):
            log("HIP graph replay did not reproduce the eager result; using eager timing")
            return []
        return out
    except Exception as exc:          # graph capture is an optimisation of the launch path only
        log("HIP graph capture unavailable:", exc)
        return []


def device_inputs(workload, dtype_name, dev, seed=2345):
    """Graph arguments and node tensors of a workload on the device: (desc, N, E, H, D, gargs, (q, k, v, do), host parts)."""
    import torch
    from bpt_amd import graphbuilder as gb
    desc, graphs, H, D, default_dtype = make_workload(workload)
    dtype_name = dtype_name or default_dtype
    tdtype = {"f32": torch.float32, "bf16": torch.bfloat16}[dtype_name]
    t0 = time.perf_counter()
    src, dst, etype, _, N = gb.merge_graphs(graphs)
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, N)
    t_graph = time.perf_counter() - t0
    gargs = tuple(x.to(dev) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(seed)
    qkvd = tuple((torch.randn(N, H, D, generator=gen) / 8).to(tdtype).to(dev) for _ in range(4))
    host = dict(src=src, dst=dst, etype=etype, out_csr=out_csr, in_csr=in_csr, ROW=ROW, IR=IR, COL=COL, IC=IC, t_graph=t_graph, gen=gen)
    return desc, dtype_name, N, len(src), H, D, gargs, qkvd, host


def measure_side_workload(name, dtype_name, dev, steps, no_graph, label=None):
    """ms per fused fwd+bwd step of another BASELINE configuration (median and shortest of three runs of `steps` steps,
    eager launches or HIP-graph replay, whichever median is lower), with its edges/s and share of the HBM roofline."""
    import torch
    from bpt_amd import graphop
    from bpt_amd import plan as plan_mod
    desc, dtype_name, N, E, H, D, gargs, (q, k, v, do), host = device_inputs(name, dtype_name, dev)
    scale = None

    def step():
        o, lse = graphop.attention_forward(*gargs[4:], q, k, v)
        dq, dk, dv = graphop.attention_backward(*gargs, q, k, v, o, lse, do)
        return o, dq, dk, dv

    ref = step()
    torch.cuda.synchronize()
    runs = timed_runs(step, steps, [max(10, steps // 10), 2, 2])
    t, tmin, mode = median(runs), min(runs), "eager"
    if not no_graph:
        gr = graph_replay_runs(step, ref, steps, 10)
        if gr and median(gr) < t:
            t, tmin, mode = median(gr), min(gr), "hipgraph-replay"
    esize = {"f32": 4, "bf16": 2}[dtype_name]
    alg = algorithmic_bytes(N, E, H, D, esize)["total"]
    flops = 2.0 * 12 * E * H * D                     # 12 E C multiply-adds per step
    res = {"workload": desc, "dtype": dtype_name, "n_nodes": N, "n_edges": E, "ms_per_step": round(t * 1e3, 5), "ms_per_step_min": round(tmin * 1e3, 5),
           "launch": mode, "edges_per_s": round(E / t, 1), "algorithmic_bytes": alg,
           "step_frac_of_hbm_peak": round(alg / t / 1e9 / HBM_PEAK_GBS, 4),
           "useful_tflops": round(flops / t / 1e12, 2), "matrix_peak_tflops": {"f32": 157.3, "bf16": 2500.0}[dtype_name]}
    del q, k, v, do, gargs, ref
    plan_mod.plan_cache.clear()
    graphop.release_workspaces()
    torch.cuda.empty_cache()
    log(f"workload {label or name}: {res}")
    return res


def measure_narrow_heads(dev, steps, no_graph, h=6, d=50):
    """The reference's other head shape (6 heads x 50, configs/imdb-4.yml:10-12) on cfg2's batch of 32 graphs, float32, through
    `op.bpt_attention` and autograd: the fused kernels on zero-padded heads against the unfused op chain on the shape-generic
    kernels (median of three runs each, eager launches or HIP-graph replay, whichever median is lower)."""
    import torch
    from bpt_amd import graphop, op
    from bpt_amd import plan as plan_mod
    desc, _, N, E, _, _, gargs, _, host = device_inputs("cfg2", "f32", dev)
    gen = torch.Generator().manual_seed(2345)
    q, k, v, do = ((torch.randn(N, h, d, generator=gen) / math.sqrt(d)).to(dev) for _ in range(4))

    def make(fused):
        def step():
            qq, kk, vv = (x.detach().requires_grad_(True) for x in (q, k, v))
            o = op.bpt_attention(*gargs, qq, kk, vv, fused=fused)
            o.backward(do)
            return o, qq.grad, kk.grad, vv.grad
        return step

    res = {"workload": desc.replace("8x64", f"{h}x{d}") + " (op.bpt_attention fwd+bwd through autograd)", "dtype": "f32", "n_nodes": N, "n_edges": E}
    for name, fused in (("fused_padded", None), ("op_chain", False)):
        step = make(fused)
        ref = step()
        torch.cuda.synchronize()
        t = median(timed_runs(step, steps, [5, 2, 2]))
        if not no_graph:
            gr = graph_replay_runs(step, None, steps, 5)
            if gr:
                t = min(t, median(gr))
        res[name + "_ms_per_step"] = round(t * 1e3, 5)
    res["edges_per_s"] = round(E / (res["fused_padded_ms_per_step"] * 1e-3), 1)
    res["fused_over_chain"] = round(res["op_chain_ms_per_step"] / res["fused_padded_ms_per_step"], 2)
    del q, k, v, do, gargs
    plan_mod.plan_cache.clear()
    graphop.release_workspaces()
    torch.cuda.empty_cache()
    log(f"workload tc32-{h}x{d}: {res}")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg3")
    ap.add_argument("--dtype", default=None, choices=[None, "f32", "bf16"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="accepted for older command lines: the 256 MiB device-to-device copies (known HBM bytes, by which "
                         "counter runs are scaled) now run every time")
    ap.add_argument("--group-rows", type=int, default=None, choices=[4, 8], help="rows per wavefront group of the fused kernels (default: 8 where available, else 4)")
    ap.add_argument("--rows", action="store_true", help="fused kernels with one wavefront per row (no row groups)")
    ap.add_argument("--unfused", action="store_true", help="time the unfused op chain of the reference's surface")
    ap.add_argument("--dropout", type=float, default=0.0, help="dropout on the attention probabilities inside the fused kernels (attention.py:73)")
    ap.add_argument("--rel-pos", action="store_true",
                    help="add the relative-position score term q[dst].table[etype[e]] (table (1000, d_head), modules/attention.py:23,42,69-71)")
    ap.add_argument("--plan", default="auto", choices=["auto", "host", "device"],
                    help="where launch plans and row groups are built: on the host (libbptgraph), on the GPU (libbptplan), "
                         "or by graph size and density (the library's default)")
    ap.add_argument("--tile-backward", default="auto", choices=["auto", "on", "off"],
                    help="fused backward on the dense tiles of 16 rows (on), on the row groups (off), or the library's choice by dtype and graph")
    ap.add_argument("--side-workloads", default="auto", choices=["auto", "all", "none"],
                    help="also time the other BASELINE configurations (cfg1, cfg2, cfg3 bf16, cfg4 k=1 / k=32 / window 128, cfg5 bf16), "
                         "50 steps x 3 runs each, reported as `workloads`; auto: with the default headline line only")
    ap.add_argument("--block-layers", type=int, default=None,
                    help="also time fwd+bwd of a stack of this many transformer blocks (d_model = heads*d_head, d_ff = 4x) on the "
                         "workload's graph, a few steps, reported as block_stack; default: 12 for the headline workload, else 0")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.block_layers is None:
        args.block_layers = 12 if (args.workload == "cfg3" and not args.unfused and not args.rel_pos and not args.rows) else 0

    import numpy as np
    import torch
    from bpt_amd import graphbuilder as gb
    from bpt_amd import graphop
    from bpt_amd._lib import attn_lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    graphop.set_row_groups(not args.rows)
    graphop.TILE_BACKWARD = {"auto": None, "on": True, "off": False}[args.tile_backward]
    graphop.set_group_rows(args.group_rows)
    from bpt_amd import plan as plan_mod
    plan_mod.set_device_build({"auto": None, "host": False, "device": True}[args.plan])
    desc, dtype_name, N, E, H, D, gargs, (q, k, v, do), host = device_inputs(args.workload, args.dtype, dev)
    tdtype = {"f32": torch.float32, "bf16": torch.bfloat16}[dtype_name]
    esize = {"f32": 4, "bf16": 2}[dtype_name]
    src, dst, etype, out_csr, in_csr, gen = host["src"], host["dst"], host["etype"], host["out_csr"], host["in_csr"], host["gen"]
    ROW, IR, COL, IC = host["ROW"], host["IR"], host["COL"], host["IC"]
    log(f"{desc}: N={N} E={E} dtype={dtype_name}; host graph+CSR build {host['t_graph'] * 1e3:.1f} ms")

    if args.rel_pos and not args.unfused:
        # rel_pos inside the fused kernels: per-edge score term from the (1000, d) table, table gradient by SpMMs
        from bpt_amd import op
        table = (torch.randn(1000, D, generator=gen) / 8).to(tdtype).to(dev)
        et = torch.from_numpy(np.asarray(etype, dtype=np.int64)).to(dev)

        def step():
            qq, kk, vv, tt = (x.detach().requires_grad_(True) for x in (q, k, v, table))
            o = op.bpt_attention(*gargs, qq, kk, vv, dropout_p=args.dropout, seed=2345, rel_table=tt, etype=et)
            o.backward(do)
            return o, qq.grad, kk.grad, vv.grad
    elif args.rel_pos:
        # the op sequence of modules/attention.py:66-77 with rel_pos on; the (E, d) rows of the table are
        # gathered per step as the reference's nn.Embedding does (backward: segment sums per edge type)
        from bpt_amd import op
        table = (torch.randn(1000, D, generator=gen) / 8).to(tdtype).to(dev)
        et = torch.from_numpy(np.asarray(etype, dtype=np.int64)).to(dev)

        def step():
            qq, kk, vv, tt = (x.detach().requires_grad_(True) for x in (q, k, v, table))
            e = op.masked_mm(*gargs, kk, qq) + op.node_mul_edge(*gargs[4:7], qq, op.edge_type_embedding(tt, et))
            a = op.sparse_softmax(*gargs[4:7], e / math.sqrt(D))
            o = op.vec_spmm(*gargs[4:], *gargs[:4], a, vv)
            o.backward(do)
            return o, qq.grad, kk.grad, vv.grad
    elif args.unfused:
        from bpt_amd import op

        def step():
            qq, kk, vv = (x.detach().requires_grad_(True) for x in (q, k, v))
            o = op.bpt_attention(*gargs, qq, kk, vv, fused=False)
            o.backward(do)
            return o, qq.grad, kk.grad, vv.grad
    else:
        def step():
            o, lse = graphop.attention_forward(*gargs[4:], q, k, v, dropout_p=args.dropout, seed=2345)
            dq, dk, dv = graphop.attention_backward(*gargs, q, k, v, o, lse, do, dropout_p=args.dropout, seed=2345)
            return o, dq, dk, dv

    ref = step()                                   # builds + caches the plans
    torch.cuda.synchronize()

    # what a new graph costs before its first step: the plans of both CSR sides, the groups both passes use and the pair
    # mapping, built from the int64 device tensors the ops receive = a fused step on a cold plan cache (libraries loaded),
    # less a warm step
    plan_build = None
    if not args.rows and not args.unfused and not args.rel_pos:
        step()
        ts = []
        for _ in range(3):
            plan_mod.plan_cache.clear()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            step()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        where = sorted({"device" if isinstance(p_, plan_mod.DevicePlan) else "host" for p_, _ in plan_mod.plan_cache._d.values()})
        plan_build = {"where": "+".join(where), "cold_step_ms": round(min(ts) * 1e3, 3)}
        log(f"plan build: {plan_build}")
        ref = step()
        torch.cuda.synchronize()

    # The timed region is exactly --steps steps between two synchronisations.  It is run three times; the MEDIAN run is
    # the reported ms_per_step and the shortest one is kept beside it (all three are in the JSON line): the host of a
    # shared box stalls now and then for tens of milliseconds, which shows as one slow run of the three.
    runs_eager = timed_runs(step, args.steps, [args.warmup, 2, 2])
    t_eager, t_eager_min = median(runs_eager), min(runs_eager)
    t_step, t_step_min, mode = t_eager, t_eager_min, "eager"
    t_graph_replay, runs_graph = None, []
    if not args.no_graph:
        runs_graph = graph_replay_runs(step, ref, args.steps, args.warmup)
        if runs_graph:
            t_graph_replay = median(runs_graph)
            if t_graph_replay < t_step:
                t_step, t_step_min, mode = t_graph_replay, min(runs_graph), "hipgraph-replay"

    # ---- per-kernel durations, HIP events recorded by the library around the kernel on its launch stream
    lib = attn_lib()
    kernels = {}
    if not args.unfused and not args.rel_pos:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record(); ev1.record(); torch.cuda.synchronize()
        for which, name in ((1, "attn_fwd"), (2, "attn_bwd_dst"), (3, "attn_bwd_src")):
            lib.bpt_profile_kernel(which, ev0.cuda_event, ev1.cuda_event)
            ts = []
            for i in range(min(args.steps, 100) + 5):
                step()
                torch.cuda.synchronize()
                if i >= 5:
                    ts.append(ev0.elapsed_time(ev1))
            lib.bpt_profile_kernel(0, None, None)
            kernels[name] = sum(ts) / len(ts)          # ms, average launch duration
    alg = algorithmic_bytes(N, E, H, D, esize)
    roofline = None
    if kernels:
        dom = max(kernels, key=kernels.get)
        achieved = alg[dom] / (kernels[dom] * 1e-3) / 1e9
        traffic = None
        tpath = os.path.join(ROOT, "profiles", "traffic.json")
        if os.path.exists(tpath):
            traffic = json.load(open(tpath)).get(f"{args.workload}-{dtype_name}", {}).get(dom)
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                    "traffic_source": "profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, scaled by the "
                                      "256 MiB copies of the same run (profiles/attn_fused_cfg3_f32_hbm_traffic.txt); not measured in this run",
                    "algorithmic_bytes": alg[dom], "avg_launch_ms": round(kernels[dom], 5)}

    # what this GPU's memory system delivers to a plain streaming kernel: device-to-device copies of 256 MiB (read +
    # write = 512 MiB of HBM traffic per launch, far larger than the caches), timed with events on the current stream
    a = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
    b = torch.empty_like(a)
    for _ in range(3):
        b.copy_(a)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    for _ in range(10):
        b.copy_(a)
    c1.record()
    torch.cuda.synchronize()
    copy_gbs = 10 * 2 * a.numel() * 4 / (c0.elapsed_time(c1) * 1e-3) / 1e9
    del a, b
    log(f"measured device copy bandwidth: {copy_gbs:.0f} GB/s (read + write)")
    # ... and to the access pattern of these kernels: pseudo-random 1 KB rows (a node row's share of one wavefront) of a
    # region the size of the K and V tensors, at the occupancies the attention kernels run at (8 and 16 wavefronts per CU)
    gather = {}
    region = torch.zeros(max(2 * N * H * D * esize, 1 << 20), dtype=torch.uint8, device=dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    for waves in (8, 16, 32):
        iters, in_flight = 100, 4
        for rep in range(2):
            c0.record()
            st = lib.bpt_gather_probe(region.data_ptr(), region.numel(), waves, in_flight, iters, sink.data_ptr(),
                                      torch.cuda.current_stream().cuda_stream)
            c1.record()
            torch.cuda.synchronize()
        assert st == 0, st
        gather[f"{waves}_waves_per_cu"] = round(256 * waves * iters * in_flight * 1024 / (c0.elapsed_time(c1) * 1e-3) / 1e9, 1)
    del region
    log(f"measured 1 KB row-gather bandwidth from a {2 * N * H * D * esize / 1e6:.0f} MB region, GB/s: {gather}")
    if roofline is not None:
        roofline["measured_copy_GBps"] = round(copy_gbs, 1)
        roofline["frac_of_measured_copy"] = round(roofline["achieved"] / copy_gbs, 4)
        roofline["measured_row_gather_GBps"] = gather

    block = None
    if args.block_layers > 0 and not args.unfused:
        # the reference's layer (modules/attention.py:22-81) around the attention core, dropout off, no rel_pos
        from bpt_amd.block import BPTBlock
        dm = H * D
        csr_dev = (tuple(t.to(dev) for t in out_csr), tuple(t.to(dev) for t in in_csr), *(x.to(dev) for x in (ROW, IR, COL, IC)))
        torch.manual_seed(2345)
        layers = torch.nn.ModuleList([BPTBlock(dm, H, 4 * dm, rel_pos=False, drop_h=0.0, drop_a=0.0) for _ in range(args.block_layers)])
        layers = layers.to(dev).to(tdtype)
        h0 = (torch.randn(N, dm, generator=torch.Generator().manual_seed(1)) / 8).to(tdtype).to(dev).requires_grad_(True)
        gh = (torch.randn(N, dm, generator=torch.Generator().manual_seed(2)) / 8).to(tdtype).to(dev)

        def stack_step():
            x = h0
            for blk in layers:
                x = blk(x, csr_dev)
            x.backward(gh)
            return x

        t_stack = median(timed_runs(stack_step, 5, [2, 2, 2]))
        block = {"layers": args.block_layers, "d_model": dm, "d_ff": 4 * dm, "ms_per_layer_fwd_bwd": round(t_stack / args.block_layers * 1e3, 4),
                 "attention_ms_per_layer": round(t_step * 1e3, 4), "attention_share": round(t_step * args.block_layers / t_stack, 3)}
        log(f"block stack: {block}")

    variants = None
    if args.block_layers > 0 and not args.unfused and not args.rel_pos and args.dropout == 0:
        # the same step with the layer's two optional terms inside the fused kernels (modules/attention.py:69-73), eager,
        # shortest of three short runs each: the rel_pos score term (table (1000, d_head), the graph's own edge types) and
        # attention dropout 0.1
        from bpt_amd import op as op_mod
        table = (torch.randn(1000, D, generator=torch.Generator().manual_seed(3)) / 8).to(tdtype).to(dev)
        et = torch.from_numpy(np.asarray(etype, dtype=np.int64)).to(dev)

        def variant_step(**kw):
            def f():
                qq, kk, vv, tt = (x.detach().requires_grad_(True) for x in (q, k, v, table))
                if "rel" in kw:
                    kw2 = dict(rel_table=tt, etype=et)
                else:
                    kw2 = {}
                o = op_mod.bpt_attention(*gargs, qq, kk, vv, dropout_p=kw.get("p", 0.0), seed=2345, **kw2)
                o.backward(do)
            return f

        def best_of_eager_and_replay(fn):
            # as for the headline step: eager launches (through autograd here, about 0.2 ms of host work per step) or the
            # replay of a HIP graph of the same step, whichever median of three runs is lower
            t = median(timed_runs(fn, 100, [10, 10, 10]))
            if not args.no_graph:
                gr = graph_replay_runs(fn, None, 100, 10)
                if gr:
                    t = min(t, median(gr))
            return t

        variants = {name: round(best_of_eager_and_replay(variant_step(**kw)) * 1e3, 4)
                    for name, kw in (("rel_pos_ms_per_step", dict(rel=True)), ("dropout_0.1_ms_per_step", dict(p=0.1)),
                                     ("rel_pos_dropout_0.1_ms_per_step", dict(rel=True, p=0.1)))}
        log(f"variants: {variants}")

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(src, dst, N, H, D, 2345)

    # the other BASELINE configurations, a short run each (the default line only: --side-workloads none switches them off)
    side = None
    if args.side_workloads == "all" or (args.side_workloads == "auto" and args.block_layers > 0 and args.workload == "cfg3"
                                        and dtype_name == "f32" and not args.unfused and not args.rel_pos and args.dropout == 0):
        del q, k, v, do
        plan_mod.plan_cache.clear()
        graphop.release_workspaces()
        torch.cuda.empty_cache()
        side = {}
        for label, wl, dt in (("cfg1", "cfg1", "f32"), ("cfg2", "cfg2", "f32"), ("cfg3-bf16", "cfg3", "bf16"), ("cfg4-k1", "cfg4-k1", "f32"),
                              ("cfg4-k32", "cfg4-k32", "f32"), ("cfg4-w128", "cfg4-w128", "f32"), ("cfg5-bf16", "cfg5", "bf16")):
            side[label] = measure_side_workload(wl, dt, dev, args.steps, args.no_graph, label)      # (as many steps as the headline: 50 read 3-5 % long)
        side["tc32-6x50"] = measure_narrow_heads(dev, max(30, args.steps // 4), args.no_graph)

    step_gbs = alg["total"] / t_step / 1e9
    out = {
        "metric": "attention edges/s fwd+bwd at n=8192 k=4 8h\u00d764; % of HBM roofline",
        "value": E / t_step, "unit": "edges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": t_step * 1e3, "ms_per_step_min": t_step_min * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype_name, "data": "synthetic",
        "config": {"workload": desc + (" (op chain with rel_pos)" if args.rel_pos and args.unfused else " (fused fwd+bwd with rel_pos)" if args.rel_pos else " (unfused op chain)" if args.unfused else
                                       f" (fused fwd+bwd, attention dropout {args.dropout})" if args.dropout > 0 else " (fused fwd+bwd)"), "n_nodes": N,
                   "n_edges": E, "heads": H, "d_head": D, "launch": mode,
                   "kernels": "per-row" if args.rows else f"row groups of {args.group_rows}" if args.group_rows else
                              "auto (tiles of 16 rows or row groups of 4 / 8, by dtype and graph)"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "step_roofline": {"algorithmic_bytes": alg["total"], "achieved_GBps": round(step_gbs, 1),
                          "frac_of_hbm_peak": round(step_gbs / HBM_PEAK_GBS, 4),
                          "measured_copy_GBps": round(copy_gbs, 1), "frac_of_measured_copy": round(step_gbs / copy_gbs, 4)},
        "ms_per_step_eager": t_eager * 1e3,
        "ms_per_step_graph": None if t_graph_replay is None else t_graph_replay * 1e3,
        "timed_runs_ms_per_step": {"eager": [round(t * 1e3, 5) for t in runs_eager], "graph": [round(t * 1e3, 5) for t in runs_graph],
                                   "reported": "ms_per_step = median of three runs of --steps steps each (of the faster launch mode); ms_per_step_min = the shortest"},
        "kernel_ms": {k_: round(v_, 5) for k_, v_ in kernels.items()},
    }
    if plan_build is not None:
        plan_build["ms"] = round(plan_build.pop("cold_step_ms") - t_step * 1e3, 3)
        out["plan_build"] = plan_build
    if block is not None:
        out["block_stack"] = block
    if variants is not None:
        out["variants"] = variants
    if side is not None:
        out["workloads"] = side
    log(json.dumps(out, indent=1))
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
