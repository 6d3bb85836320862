#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

A "step" is one decode GEMV of the headline workload: Q4_K weights, rows=14336, cols=4096
(Llama-3-8B FFN gate/up), one f32 activation vector quantized to Q8_K on the device, f32 output.
Operands are resident in HBM before the timed region.  Every step reads a different one of
COPIES weight copies (COPIES x 33 MB > the 256 MB Infinity Cache), so the weights come from HBM
and not from cache.  The metric is the reference's: quantized weight bytes / seconds per step
(crates/frink-cuda/examples/matvec_bench.rs:56-61), in GB/s.

The timed region is K steps captured in HIP graphs of at most GRAPH_STEPS steps and replayed
(config.graph says how many steps one replay held: a replay starts with a few microseconds of
nothing, which 400 steps dilute and 20 do not).

Prints ONE JSON line (see the fields at the bottom).  `--read-sweep` prints, instead, the time of a
read-only stream against its size (cache-cold), the floor under any kernel that reads that much.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0  # dense int8 MFMA
COPIES = 16
HEADLINE_KERNEL = "gemv_q4_k_lines_kernel<16, 0, 8, false, 4, false>"
# steps captured per HIP graph in the two timed loops of the headline (a multiple of COPIES): a graph
# replay starts with a few microseconds of nothing, which 400 steps dilute and 16 would not
GRAPH_STEPS = 400
# HBM bytes per launch of the roofline kernel: not measurable from inside this script (hardware counters
# need rocprofv3 around it), so the record carries what the last two rocprofv3 --pmc runs of this script
# found -- FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each scaled by what the same counter reads for
# copy_kernel over a known size -- read from the summary those runs are kept in, and names that file.
TRAFFIC_PROFILE = os.path.join("profiles", "bench_kernels_hbm_traffic_pmc.txt")


def traffic_from_profile(kernel_prefix):
    """(bytes per launch, source) from the lines `traffic <kernel> fetch_kib=F write_kib=W` and
    `calibration copy_kernel kib=K fetch_kib=F write_kib=W` of TRAFFIC_PROFILE; (None, reason) without them."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return None, "%s is missing" % TRAFFIC_PROFILE

    def fields(line):
        return {k: float(v) for k, v in (w.split("=") for w in line.split() if "=" in w)}
    cal = [fields(l) for l in lines if l.startswith("calibration copy_kernel")]
    mine = [fields(l) for l in lines if l.startswith("traffic " + kernel_prefix)]
    if not cal or not mine:
        return None, "%s has no line for %s" % (TRAFFIC_PROFILE, kernel_prefix)
    c, m = cal[0], mine[0]
    kib = m["fetch_kib"] * c["kib"] / c["fetch_kib"] + m["write_kib"] * c["kib"] / c["write_kib"]
    return int(kib * 1024), "%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, scaled by copy_kernel)" % TRAFFIC_PROFILE


def random_blocks(kind, rows, cols, seed):
    """Structurally valid GGUF blocks with weight-like magnitudes, straight from a seeded
    generator (timing does not depend on the values; the parity tests use encoded N(0, 0.02))."""
    from frink_amd import BLOCK
    bb, be = BLOCK[kind]
    nb = rows * (cols // be)
    rng = np.random.default_rng(seed)
    data = rng.integers(0, 256, (nb, bb), dtype=np.uint8)

    def f16(lo, hi):
        return rng.uniform(lo, hi, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    if kind in (12, 13):  # Q4_K, Q5_K: d, dmin
        data[:, 0:2] = f16(1e-4, 3e-4)
        data[:, 2:4] = f16(1e-3, 3e-3)
    elif kind == 14:    # Q6_K: d
        data[:, 208:210] = f16(2e-5, 6e-5)
    elif kind == 39:    # MXFP4: an E8M0 scale byte, 2^-10 .. 2^-6
        data[:, 0] = rng.integers(118, 123, nb)
    else:               # Q8_0, Q4_0, Q5_0, IQ4_XS: d
        data[:, 0:2] = f16(3e-4, 6e-4)
    return data.reshape(-1)


def time_graph(torch, fn_steps, n_steps, copies):
    """Captures `copies` consecutive steps in one HIP graph (fn_steps(i) chooses its operands by i
    modulo whatever it rotates over) and replays it; returns seconds for exactly n_steps steps (a
    second, shorter graph runs the remainder)."""
    stream = torch.cuda.Stream()
    graphs = []
    with torch.cuda.stream(stream):
        for i in range(copies):
            fn_steps(i)  # warm: sizes the library workspace before capture
        torch.cuda.synchronize()
        full, rem = divmod(n_steps, copies)
        for count in ([copies] if full else []) + ([rem] if rem else []):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(count):
                    fn_steps(i)
            graphs.append((g, count))
        g_full = graphs[0][0] if full else None
        g_rem = graphs[-1][0] if rem else None
        # one untimed replay of each, then a synchronization; a second untimed replay goes out right in
        # front of the timed ones with no synchronization between, so that the timed steps start on a
        # GPU that is already running steps (the state of a decode loop) and not on an idle one
        for g, _ in graphs:
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        graphs[0][0].replay()
        e0.record()
        for _ in range(full):
            g_full.replay()
        if g_rem is not None:
            g_rem.replay()
        e1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    # (the host's clock also saw the untimed replay in front: scaled to the timed steps' share)
    return wall * n_steps / (n_steps + graphs[0][1]), e0.elapsed_time(e1) * 1e-3


def host_cpu():
    """Model name, logical CPUs this process may use, physical cores among them (distinct
    thread_siblings_list entries, as crates/frink-core/src/threads.rs sizes the reference's pool) and
    whether AVX2 and FMA are there."""
    model, flags = "unknown", ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name") and model == "unknown":
                model = line.split(":", 1)[1].strip()
            elif line.startswith("flags") and not flags:
                flags = line.split(":", 1)[1]
    except OSError:
        pass
    cpus = sorted(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else list(range(os.cpu_count() or 1))
    cores = set()
    for c in cpus:
        try:
            cores.add(open("/sys/devices/system/cpu/cpu%d/topology/thread_siblings_list" % c).read().strip())
        except OSError:
            cores.add("cpu%d" % c)
    words = flags.split()
    return {"cpu_model": model, "logical_cpus": len(cpus), "physical_cores": len(cores),
            "avx2_fma": "avx2" in words and "fma" in words}


def best_of(fn, budget_s, max_reps=50):
    reps, spent, best = 0, 0.0, float("inf")
    while reps < 1 or (spent < budget_s and reps < max_reps):
        t = time.perf_counter()
        fn()
        dt = time.perf_counter() - t
        best = min(best, dt)
        spent += dt
        reps += 1
    return best, reps


def cpu_baseline(kind, data, rows, cols, x, y_gpu, xb):
    """Times the CPU forms of the same work on this host's physical cores (rows over OpenMP threads,
    as the reference partitions them): the decode GEMV as the reference's x86 default runs it (AVX2+FMA
    f32 dot), as its integer path runs it (Q8_K + AVX2 integer dot) and as the scalar oracle computes
    it; and the M=512 GEMM as integer dots with the weight row outermost.  Checks the GPU's GEMV
    against the scalar oracle on the way."""
    import oracle as fo
    host = host_cpu()
    threads = max(1, host["physical_cores"])
    want = fo.gemv(kind, data, rows, cols, x, fo.INT_DOT, threads)
    err = float(np.abs(y_gpu - want).max() / np.abs(want).max())
    legs = {}
    t, n = best_of(lambda: fo.gemv(kind, data, rows, cols, x, fo.INT_DOT, threads), 3.0)
    legs["decode_int_dot_scalar_GBs"] = round(data.size / t / 1e9, 2)
    simd = host["avx2_fma"] and fo.have_avx2()
    if simd:
        t, n = best_of(lambda: fo.avx2_gemv_q4_k_f32(data, rows, cols, x, threads), 4.0)
        legs["decode_f32_dot_avx2_GBs"] = round(data.size / t / 1e9, 2)
        headline, what = data.size / t / 1e9, "AVX2+FMA f32 dot (the reference's x86 decode default), best of %d" % n
        t, n = best_of(lambda: fo.avx2_gemm_q4_k_q8k(data, rows, cols, x, threads), 4.0)
        legs["decode_int_dot_avx2_GBs"] = round(data.size / t / 1e9, 2)
        t, n = best_of(lambda: fo.avx2_gemm_q4_k_q8k(data, rows, cols, xb, threads), 8.0, 5)
        legs["gemm_m512_int_dot_avx2_TOPS"] = round(2.0 * xb.shape[0] * rows * cols / t / 1e12, 4)
        legs["gemm_m512_ms"] = round(t * 1e3, 1)
        # batched decode, M=8: the same row-outer integer dots, eight activations per weight row (the shape the
        # reference's 8-row repack tier serves, crates/frink-core/src/weight_matrix.rs:2954-3057)
        t, n = best_of(lambda: fo.avx2_gemm_q4_k_q8k(data, rows, cols, xb[:8], threads), 3.0)
        legs["gemm_m8_int_dot_avx2_GBs"] = round(data.size / t / 1e9, 2)
        legs["gemm_m8_ms"] = round(t * 1e3, 2)
    else:
        headline, what = legs["decode_int_dot_scalar_GBs"], "scalar integer dot (this host has no AVX2+FMA)"
    # the MoE layer (128 experts, top-8, 2048/768, 512 tokens) as the reference's bucket path runs it
    # (Decoder::moe_ffn_batch, crates/frink-models/src/decoder/ffn_batch.rs:343-434): the oracle's scalar integer
    # dots, experts over the threads; one pass (seconds)
    E, K, H, F, T = 128, 8, 2048, 768, 512
    from frink_amd import Q4_K, synth
    gate, up, down = (random_blocks(Q4_K, r, c, seed=80 + j) for j, (r, c) in enumerate(((E * F, H), (E * F, H), (E * H, F))))
    xm = synth.activations(7, T, H)
    logits = synth.normal(8, T * E).reshape(T, E)
    routed = [fo.route_top_k_softmax(l, K, True) for l in logits]
    ids = np.stack([r[0] for r in routed]).astype(np.int32)
    wts = np.stack([r[1] for r in routed])
    t, n = best_of(lambda: fo.moe_ffn(Q4_K, gate, up, down, E, H, F, xm, ids, wts, threads), 6.0, 3)
    legs["moe_layer_512_tokens_scalar_int_dot_ms"] = round(t * 1e3, 1)
    legs["moe_layer_512_tokens_tokens_per_s"] = round(T / t, 1)
    del gate, up, down
    out = {"value": round(headline, 2), "unit": "GB/s", "cores": threads, "kind": "port",
           "sample": "the whole workload (%dx%d Q4_K decode GEMV) as %s; legs: the same GEMV on the integer path "
                     "(Q8_K quantization + AVX2 integer dot, and the scalar oracle), the whole M=512 GEMM and the M=8 batch as "
                     "AVX2 integer dots with the weight row outermost, and one pass of the 128-expert MoE layer at 512 "
                     "tokens on the scalar oracle; %d OpenMP threads = physical cores"
                     % (rows, cols, what, threads),
           "legs": legs, "gpu_vs_cpu_max_err_over_ninf": err}
    out.update(host)
    return out


def read_sweep(torch, fa):
    """time of a read-only stream against its size, every launch reading memory no earlier launch of
    the last 512 MB touched"""
    import ctypes as C
    dev = torch.device("cuda:0")
    pool = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_()
    sink = torch.empty(1 << 16, dtype=torch.uint8, device=dev)
    L = fa.lib()
    print("# read-only stream (frk_hip_read_dev), cache-cold: bytes, us per launch, GB/s")
    for mb in (8, 16, 33, 66, 132, 264):
        nbytes = mb * 1000 * 1000 // 4096 * 4096
        slots = max(2, (1 << 30) // nbytes)

        def rd(i):
            fa.check(L.frk_hip_read_dev(C.c_void_p(pool.data_ptr() + (i % slots) * nbytes), nbytes,
                                        C.c_void_p(sink.data_ptr()), fa._stream()))
        n = 4 * slots if mb >= 132 else 400
        _, t = time_graph(torch, rd, n, min(n, 400))
        print("%10d  %7.2f  %7.1f" % (nbytes, t / n * 1e6, nbytes / (t / n) / 1e9), flush=True)


def read_shapes(torch, fa):
    """frk_hip_read_shape_dev over the headline matrix's 33,030,144 bytes, cache-cold: which span per wavefront,
    wavefronts per workgroup, landing place and cache bits fetch it fastest, with frk_hip_read_dev beside them"""
    import ctypes as C
    dev = torch.device("cuda:0")
    nbytes = 14336 * 4096 // 256 * 144
    slots = COPIES
    pool = torch.empty(slots * nbytes, dtype=torch.uint8, device=dev).random_()
    sink = torch.empty(1 << 16, dtype=torch.uint8, device=dev)
    L = fa.lib()

    def run(fn):
        _, t = time_graph(torch, fn, 400, 400)
        return t / 400 * 1e6

    def plain(i):
        fa.check(L.frk_hip_read_dev(C.c_void_p(pool.data_ptr() + (i % slots) * nbytes), nbytes, C.c_void_p(sink.data_ptr()),
                                    fa._stream()))
    print("# fetch of %d bytes, cache-cold (%d copies in turn), 400 launches in one graph; us per launch" % (nbytes, slots))
    print("frk_hip_read_dev  %6.2f" % run(plain), flush=True)
    print("# span KB  wavefronts/workgroup  landing  policy  us  GB/s")
    names = ("-", "nt", "sc1", "sc0 sc1")
    for to_lds in (0, 1):
        for span in (2, 4, 9, 18):
            for waves in (4, 8, 16):
                if to_lds and waves * min(span, 8) > 160:
                    continue
                for policy in (0, 1, 2, 3):
                    def rd(i):
                        fa.check(L.frk_hip_read_shape_dev(C.c_void_p(pool.data_ptr() + (i % slots) * nbytes), nbytes,
                                                          C.c_void_p(sink.data_ptr()), span, waves, to_lds, policy, fa._stream()))
                    us = run(rd)
                    print("%3d  %3d  %-9s  %-8s  %6.2f  %7.1f" % (span, waves, "LDS" if to_lds else "registers", names[policy], us,
                                                                 nbytes / us / 1e3), flush=True)


def issue_probe(fa):
    """frk_hip_issue_probe: a chain of dependent v_mfma_i32_32x32x32_i8 with N cheap vector instructions behind each,
    two wavefronts per SIMD on every compute unit."""
    import ctypes as C
    out = (C.c_float * 16)()
    fa.check(fa.lib().frk_hip_issue_probe(out))
    print("# v_mfma_i32_32x32x32_i8 (32 clocks of the matrix core) + N x v_and_b32 per MFMA, 2 wavefronts per SIMD")
    print("# N  cycles per MFMA and SIMD  shader MHz  launch us  first wavefront's share of the launch")
    for k, n in enumerate((0, 4, 8, 12)):
        print("%3d  %8.1f  %8.0f  %9.1f  %6.2f" % (n, out[4 * k], out[4 * k + 1], out[4 * k + 2], out[4 * k + 3]), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--read-sweep", action="store_true", help="only: time of a read-only stream against its size")
    ap.add_argument("--read-shapes", action="store_true", help="only: the headline matrix's bytes fetched in the decode "
                    "kernels' shape -- span per wavefront, wavefronts per workgroup, registers or LDS, cache bits")
    ap.add_argument("--issue-probe", action="store_true", help="only: what a matrix-core instruction costs the vector ALU, "
                    "and the shader clock under matrix-core load")
    ap.add_argument("--only", default="", help="comma-separated groups of secondary workloads to run (ceilings, gemv, gemm, "
                    "moe, thin, qkv): a profiler run replays only the kernels it is about")
    ap.add_argument("--graph-steps", type=int, default=GRAPH_STEPS, help="most steps captured in one HIP graph")
    args = ap.parse_args()
    only = set(w for w in args.only.split(",") if w)

    def want(group):
        return not only or group in only
    graph_cap = max(1, args.graph_steps)

    def timed(fn, n, per_graph):
        return time_graph(torch, fn, n, max(1, min(per_graph, graph_cap)))
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch
    import frink_amd as fa

    if args.read_sweep:
        read_sweep(torch, fa)
        return
    if args.read_shapes:
        read_shapes(torch, fa)
        return
    if args.issue_probe:
        issue_probe(fa)
        return
    info = fa.probe()
    dev = torch.device("cuda:0")
    rows, cols, kind = 14336, 4096, fa.Q4_K
    from frink_amd import synth
    data = random_blocks(kind, rows, cols, seed=1234)
    x = synth.activations(4321, 1, cols)[0]
    data_dev = torch.from_numpy(data).to(dev)
    ws = [fa.Weights.from_device(kind, data_dev, rows, cols) for _ in range(COPIES)]
    xd = torch.from_numpy(x).to(dev)
    y = torch.empty(rows, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()

    # ---- headline: whole step (Q8_K quantization + GEMV) ----
    def step(i):
        ws[i % COPIES].gemv(xd, out=y)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    wall, ev = timed(step, args.steps, GRAPH_STEPS)
    sec_per_step = ev / args.steps
    wbytes = data.size
    value = wbytes / sec_per_step / 1e9

    # ---- roofline of the dominant kernel = the one kernel a step launches (quantization inside it):
    # its launch duration is the step's, measured above with events on the stream it runs on ----
    alg_bytes = wbytes + cols * 4 + rows * 4  # W + x + y
    achieved = alg_bytes / sec_per_step / 1e9
    y_gpu = y.cpu().numpy()
    # the same product from an activation quantized beforehand (what a fused producer would hand over)
    acts = fa.quantize_q8_k(xd)

    def gemv_only(i):
        ws[i % COPIES].gemv_q8k(acts, out=y)

    n_k = max(COPIES * 8, min(args.steps, 4000))
    _, ev_k = timed(gemv_only, n_k, GRAPH_STEPS)
    k_sec = ev_k / n_k

    traffic_bytes, traffic_src = traffic_from_profile("gemv_q4_k_lines_kernel")
    out = {
        "metric": "Q4_K GEMV HBM GB/s", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "Q4_K decode GEMV, rows=14336 cols=4096 batch=1 (Llama-3-8B FFN gate/up): Q8_K "
                               "activation quantization + GEMV per step (one kernel), %d weight copies rotated "
                               "(cache-cold)" % COPIES,
                   "graph": "%d steps timed with HIP events as replays of a HIP graph of %d steps, behind one untimed "
                            "replay with no synchronization between" % (args.steps, min(args.steps, GRAPH_STEPS, graph_cap)),
                   "weight_bytes": int(wbytes), "device": info["name"], "arch": info["gcn_arch"],
                   "compute_units": info["compute_units"], "wall_ms_per_step": round(wall / args.steps * 1e3, 6)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_bytes, "traffic_source": traffic_src,
                     "kernel": HEADLINE_KERNEL, "algorithmic_bytes": int(alg_bytes),
                     "avg_launch_us": round(sec_per_step * 1e6, 3), "launches": args.steps,
                     "prequantized_form": {"kernel": "gemv_q4_k_lines_kernel<16, 1, 8, false, 0, false>",
                                           "avg_launch_us": round(k_sec * 1e6, 3), "launches": n_k,
                                           "frac": round((wbytes + cols + cols // 256 * 4 + cols // 16 * 2 + rows * 4)
                                                         / k_sec / 1e9 / HBM_PEAK_GBS, 4)}},
    }

    if not args.no_extra:
        extra = {}
        if want('ceilings'):
            # practical ceilings at the same size: a read-only stream and a copy
            src = [torch.empty(wbytes, dtype=torch.uint8, device=dev).random_() for _ in range(COPIES)]
            dst = torch.empty(wbytes, dtype=torch.uint8, device=dev)
            sink = torch.empty(1 << 16, dtype=torch.uint8, device=dev)
            L, C = fa.lib(), __import__("ctypes")

            def read_only(i):
                fa.check(L.frk_hip_read_dev(C.c_void_p(src[i % COPIES].data_ptr()), wbytes, C.c_void_p(sink.data_ptr()),
                                            fa._stream()))

            def copy(i):
                fa.check(L.frk_hip_copy_dev(C.c_void_p(src[i % COPIES].data_ptr()), C.c_void_p(dst.data_ptr()), wbytes,
                                            fa._stream()))
            _, t = timed(read_only, 800, GRAPH_STEPS)
            extra["read_only_stream_33MB_GBs"] = round(wbytes / (t / 800) / 1e9, 1)
            _, t = timed(copy, 800, GRAPH_STEPS)
            extra["copy_33MB_read_plus_write_GBs"] = round(2 * wbytes / (t / 800) / 1e9, 1)
            del src, dst
        if want('gemv'):
            for name, k2, r2, c2 in (("Q6_K GEMV 4096x14336 (FFN down)", fa.Q6_K, 4096, 14336),
                                     ("Q8_0 GEMV 4096x4096", fa.Q8_0, 4096, 4096),
                                     ("Q5_K GEMV 14336x4096 (one launch)", fa.Q5_K, 14336, 4096),
                                     ("Q4_0 GEMV 14336x4096 (f32 dot)", fa.Q4_0, 14336, 4096),
                                     ("Q4_K GEMV 4096x14336 (a Q4_K down projection)", fa.Q4_K, 4096, 14336),
                                     ("Q4_K GEMV 4096x4096 (attention projection)", fa.Q4_K, 4096, 4096),
                                     ("Q8_0 GEMV 4096x14336", fa.Q8_0, 4096, 14336)):
                d2 = torch.from_numpy(random_blocks(k2, r2, c2, seed=77)).to(dev)
                n_copies = max(COPIES, -(-560_000_000 // d2.numel()))  # (past the 256 MB Infinity Cache, like the headline's copies)
                w2 = [fa.Weights.from_device(k2, d2, r2, c2) for _ in range(n_copies)]
                x2 = torch.from_numpy(synth.activations(5, 1, c2)[0]).to(dev)
                y2 = torch.empty(r2, dtype=torch.float32, device=dev)

                def step2(i):
                    w2[i % n_copies].gemv(x2, out=y2)
                _, t = timed(step2, 1600, 25 * n_copies)
                extra[name] = {"GBs": round(d2.numel() / (t / 1600) / 1e9, 1), "us_per_step": round(t / 1600 * 1e6, 3),
                               "frac_of_hbm_peak": round(d2.numel() / (t / 1600) / 1e9 / HBM_PEAK_GBS, 4)}
                for w in w2:
                    w.release()
            # the other kinds behind the seam, 14336x4096: the f32 dot of the reference's decode path and the integer tier
            for name_o, k2 in (("Q5_0", fa.Q5_0), ("IQ4_XS", fa.IQ4_XS), ("MXFP4", fa.MXFP4)):
                d2 = torch.from_numpy(random_blocks(k2, 14336, 4096, seed=91)).to(dev)
                n_copies = max(COPIES, -(-560_000_000 // d2.numel()))
                w2 = [fa.Weights.from_device(k2, d2, 14336, 4096) for _ in range(n_copies)]
                x2 = torch.from_numpy(synth.activations(5, 1, 4096)[0]).to(dev)
                y2 = torch.empty(14336, dtype=torch.float32, device=dev)
                for mode, label in ((fa.ACT_F32, "f32 dot"), (fa.ACT_INT8, "integer tier, with its quantization launch")):
                    def step2o(i):
                        w2[i % n_copies].gemv(x2, out=y2, act_mode=mode)
                    _, t = timed(step2o, 800, 25 * n_copies)
                    extra["%s GEMV 14336x4096 (%s)" % (name_o, label)] = {
                        "GBs": round(d2.numel() / (t / 800) / 1e9, 1), "us_per_step": round(t / 800 * 1e6, 3),
                        "frac_of_hbm_peak": round(d2.numel() / (t / 800) / 1e9 / HBM_PEAK_GBS, 4)}
                for w in w2:
                    w.release()
        if want('gemm'):
            # prefill GEMM M=512 on the int8 matrix cores: 2*M*rows*cols integer ops per step.  The step is
            # the activations' quantization + the GEMM kernel; the kernel alone is timed over activations
            # quantized beforehand (frk_hip_gemm_acts_dev: a graph of nothing but that kernel, HIP events).
            xb = torch.from_numpy(synth.activations(6, 512, cols, outlier_frac=0.01)).to(dev)
            acts512 = fa.BatchActs(512, cols).quantize(xb)
            gemm_records = []
            for name, r2, kname in (("Q4_K GEMM M=512 4096x4096", 4096, "gemm_q4_k_pipe_kernel<4, 2, 2>"),
                                    ("Q4_K GEMM M=512 14336x4096", 14336, "gemm_q4_k_pipe_kernel<8, 1, 4>")):
                d2 = torch.from_numpy(random_blocks(kind, r2, cols, seed=78)).to(dev)
                w2 = [fa.Weights.from_device(kind, d2, r2, cols) for _ in range(8)]
                yb = torch.empty((512, r2), dtype=torch.float32, device=dev)

                def step3(i):
                    w2[i % 8].gemm(xb, out=yb)

                def step3p(i):
                    w2[i % 8].gemm_acts(acts512, out=yb)
                _, t = timed(step3, 200, 100)
                _, tp = timed(step3p, 200, 100)
                ops = 2.0 * 512 * r2 * cols
                tops = ops / (t / 200) / 1e12
                k_us = tp / 200 * 1e6
                extra[name] = {"TOPS": round(tops, 1), "us_per_step": round(t / 200 * 1e6, 2),
                               "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
                gemm_records.append({"bound": "mfma", "workload": name, "kernel": kname, "achieved": round(ops / k_us / 1e6, 1),
                                     "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": round(ops / k_us / 1e6 / INT8_PEAK_TOPS, 4),
                                     "ops": ops, "avg_launch_us": round(k_us, 2), "launches": 200,
                                     "how": "HIP events around graphs of this kernel alone, over activations quantized beforehand",
                                     "step_us_with_quantization": round(t / 200 * 1e6, 2)})
                for w in w2:
                    w.release()
            out["roofline_gemm"] = gemm_records
            acts512.release()
            # Q5_K at M=512: the tiled matrix-core kernel with the fifth bits as a third int8 plane
            d5g = torch.from_numpy(random_blocks(fa.Q5_K, rows, cols, seed=84)).to(dev)
            w5 = [fa.Weights.from_device(fa.Q5_K, d5g, rows, cols) for _ in range(4)]
            yb5 = torch.empty((512, rows), dtype=torch.float32, device=dev)

            def step3e(i):
                w5[i % 4].gemm(xb, out=yb5)
            _, t = timed(step3e, 40, 20)
            tops = 2.0 * 512 * rows * cols / (t / 40) / 1e12
            extra["Q5_K GEMM M=512 14336x4096 (three int8 planes)"] = {
                "TOPS": round(tops, 1), "us_per_step": round(t / 40 * 1e6, 2), "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
            for w in w5:
                w.release()
            del d5g, yb5
            # the FFN down projection of a Q4_K_M model at M=512: Q6_K on the matrix cores
            d6g = torch.from_numpy(random_blocks(fa.Q6_K, cols, rows, seed=78)).to(dev)
            w6 = [fa.Weights.from_device(fa.Q6_K, d6g, cols, rows) for _ in range(4)]
            xb6 = torch.from_numpy(synth.activations(6, 512, rows)).to(dev)
            yb6 = torch.empty((512, cols), dtype=torch.float32, device=dev)

            def step3b(i):
                w6[i % 4].gemm(xb6, out=yb6)
            _, t = timed(step3b, 100, 50)
            tops = 2.0 * 512 * rows * cols / (t / 100) / 1e12
            extra["Q6_K GEMM M=512 4096x14336"] = {"TOPS": round(tops, 1), "us_per_step": round(t / 100 * 1e6, 2),
                                                   "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
            for w in w6:
                w.release()
            # the shape the reference quotes its int8 Q8_0 GEMM on (crates/frink-cuda/src/mmq/kernel.rs:30-36)
            d8g = torch.from_numpy(random_blocks(fa.Q8_0, cols, rows, seed=79)).to(dev)
            w8 = [fa.Weights.from_device(fa.Q8_0, d8g, cols, rows) for _ in range(4)]

            def step3c(i):
                w8[i % 4].gemm(xb6, out=yb6)
            _, t = timed(step3c, 100, 50)
            tops = 2.0 * 512 * rows * cols / (t / 100) / 1e12
            extra["Q8_0 GEMM M=512 4096x14336"] = {"TOPS": round(tops, 1), "us_per_step": round(t / 100 * 1e6, 2),
                                                   "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
            for w in w8:
                w.release()
            # the same kernel on Q4_0 weights (nibbles turned into signed bytes while they are staged)
            d40 = torch.from_numpy(random_blocks(fa.Q4_0, cols, rows, seed=81)).to(dev)
            w40 = [fa.Weights.from_device(fa.Q4_0, d40, cols, rows) for _ in range(4)]

            def step3d(i):
                w40[i % 4].gemm(xb6, out=yb6)
            _, t = timed(step3d, 100, 50)
            tops = 2.0 * 512 * rows * cols / (t / 100) / 1e12
            extra["Q4_0 GEMM M=512 4096x14336"] = {"TOPS": round(tops, 1), "us_per_step": round(t / 100 * 1e6, 2),
                                                   "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
            for w in w40:
                w.release()
            del d40
            # Q5_0 and MXFP4 batches: decoded into the Q8_0 planar form in scratch memory, then the Q8_0 kernel;
            # IQ4_XS: decoded to signed bytes with integer block scales, the same kernel's form for Q8_K activations
            for kind_o, name_o in ((fa.Q5_0, "Q5_0"), (fa.MXFP4, "MXFP4"), (fa.IQ4_XS, "IQ4_XS")):
                do = torch.from_numpy(random_blocks(kind_o, cols, rows, seed=85)).to(dev)
                wo = [fa.Weights.from_device(kind_o, do, cols, rows) for _ in range(4)]

                def step3f(i):
                    wo[i % 4].gemm(xb6, out=yb6)
                _, t = timed(step3f, 40, 20)
                tops = 2.0 * 512 * rows * cols / (t / 40) / 1e12
                extra["%s GEMM M=512 4096x14336 (decoded to int8 planes per call)" % name_o] = {
                    "TOPS": round(tops, 1), "us_per_step": round(t / 40 * 1e6, 2), "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
                for w in wo:
                    w.keep_decoded()
                _, t = timed(step3f, 40, 20)
                tops = 2.0 * 512 * rows * cols / (t / 40) / 1e12
                extra["%s GEMM M=512 4096x14336 (decoded copy kept)" % name_o] = {
                    "TOPS": round(tops, 1), "us_per_step": round(t / 40 * 1e6, 2), "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4)}
                for w in wo:
                    w.release()
                del do
        if want('moe'):
            # MoE layer: 128 experts, top-8, hidden 2048, ffn 768, 512 tokens (routing done beforehand)
            E, K, H, F, T = 128, 8, 2048, 768, 512
            experts = [fa.Weights.from_device(kind, torch.from_numpy(random_blocks(kind, r, c, seed=80 + j)).to(dev), r, c)
                       for j, (r, c) in enumerate(((E * F, H), (E * F, H), (E * H, F)))]
            xm = torch.from_numpy(synth.activations(7, T, H)).to(dev)
            logits = torch.from_numpy(synth.normal(8, T * E).reshape(T, E)).to(dev)
            ids, wts = fa.route_top_k_softmax(logits, K, True)
            ym = torch.empty((T, H), dtype=torch.float32, device=dev)

            def step4(i):
                fa.moe_ffn(experts[0], experts[1], experts[2], E, xm, ids, wts, out=ym)
            _, t = timed(step4, 100, 50)
            moe_bytes = 3 * E * F * H // 256 * 144 + 2 * T * H * 4 + 2 * T * K * 4
            extra["MoE layer 128x top-8, 2048/768, 512 tokens"] = {
                "us_per_step": round(t / 100 * 1e6, 2), "tokens_per_s": round(T / (t / 100), 0),
                "algorithmic_GBs": round(moe_bytes / (t / 100) / 1e9, 1),
                "frac_of_hbm_peak": round(moe_bytes / (t / 100) / 1e9 / HBM_PEAK_GBS, 4),
                "TOPS": round(2.0 * T * K * 3 * F * H / (t / 100) / 1e12, 1)}
            # the same layer for ONE token (decode): 16 routings in turn that between them visit all 128
            # experts once, so that no expert's weights are still cached when its turn comes again
            perm = np.random.default_rng(11).permutation(E).astype(np.int32).reshape(16, 1, K)
            ids1 = [torch.from_numpy(np.ascontiguousarray(p)).to(dev) for p in perm]
            w1 = torch.full((1, K), 1.0 / K, dtype=torch.float32, device=dev)
            x1 = xm[:1].contiguous()
            y1 = torch.empty((1, H), dtype=torch.float32, device=dev)

            def step4b(i):
                fa.moe_ffn(experts[0], experts[1], experts[2], E, x1, ids1[i % 16], w1, out=y1)
            _, t = timed(step4b, 800, 400)
            tok_bytes = K * 3 * F * H // 256 * 144
            extra["MoE layer 128x top-8, 2048/768, 1 token (decode)"] = {
                "us_per_step": round(t / 800 * 1e6, 2), "algorithmic_GBs": round(tok_bytes / (t / 800) / 1e9, 1),
                "frac_of_hbm_peak": round(tok_bytes / (t / 800) / 1e9 / HBM_PEAK_GBS, 4)}
            # the same layer with its down experts in Q6_K (a Q4_K_M file keeps some layers' that way), 512 tokens and 1
            down6 = fa.Weights.from_device(fa.Q6_K, torch.from_numpy(random_blocks(fa.Q6_K, E * H, F, seed=83)).to(dev), E * H, F)

            def step4c(i):
                fa.moe_ffn(experts[0], experts[1], down6, E, xm, ids, wts, out=ym)
            _, t = timed(step4c, 100, 50)
            moe6_bytes = E * F * H // 256 * (2 * 144 + 210) + 2 * T * H * 4 + 2 * T * K * 4
            extra["MoE layer 128x top-8, 2048/768, 512 tokens, down experts Q6_K"] = {
                "us_per_step": round(t / 100 * 1e6, 2), "tokens_per_s": round(T / (t / 100), 0),
                "algorithmic_GBs": round(moe6_bytes / (t / 100) / 1e9, 1),
                "frac_of_hbm_peak": round(moe6_bytes / (t / 100) / 1e9 / HBM_PEAK_GBS, 4)}

            def step4d(i):
                fa.moe_ffn(experts[0], experts[1], down6, E, x1, ids1[i % 16], w1, out=y1)
            _, t = timed(step4d, 800, 400)
            tok6_bytes = K * F * H // 256 * (2 * 144 + 210)
            extra["MoE layer 128x top-8, 2048/768, 1 token (decode), down experts Q6_K"] = {
                "us_per_step": round(t / 800 * 1e6, 2), "algorithmic_GBs": round(tok6_bytes / (t / 800) / 1e9, 1),
                "frac_of_hbm_peak": round(tok6_bytes / (t / 800) / 1e9 / HBM_PEAK_GBS, 4)}
            down6.release()
            for w in experts:
                w.release()
            # a layer of MXFP4 experts in gpt-oss-20b's shape (32 experts, top-4, 2880/2880), 512 tokens: the experts
            # decoded to signed bytes per call, the grouped form of the Q8_0 matrix-core kernel
            E4, K4, H4, F4 = 32, 4, 2880, 2880
            ex4 = [fa.Weights.from_device(fa.MXFP4, torch.from_numpy(random_blocks(fa.MXFP4, r, c, seed=90 + j)).to(dev), r, c)
                   for j, (r, c) in enumerate(((E4 * F4, H4), (E4 * F4, H4), (E4 * H4, F4)))]
            xm4 = torch.from_numpy(synth.activations(9, T, H4)).to(dev)
            ids4, wts4 = fa.route_top_k_softmax(torch.from_numpy(synth.normal(10, T * E4).reshape(T, E4)).to(dev), K4, True)
            ym4 = torch.empty((T, H4), dtype=torch.float32, device=dev)

            def step4e(i):
                fa.moe_ffn(ex4[0], ex4[1], ex4[2], E4, xm4, ids4, wts4, out=ym4)
            _, t = timed(step4e, 20, 10)
            extra["MoE layer 32x top-4, 2880/2880, 512 tokens, MXFP4 experts"] = {
                "us_per_step": round(t / 20 * 1e6, 2), "tokens_per_s": round(T / (t / 20), 0),
                "TOPS": round(2.0 * T * K4 * 3 * F4 * H4 / (t / 20) / 1e12, 1)}
            # ONE token of that layer (decode): eight routings in turn that between them visit all 32 experts once
            perm4 = np.random.default_rng(12).permutation(E4).astype(np.int32).reshape(8, 1, K4)
            ids41 = [torch.from_numpy(np.ascontiguousarray(p)).to(dev) for p in perm4]
            w41 = torch.full((1, K4), 1.0 / K4, dtype=torch.float32, device=dev)
            x41 = xm4[:1].contiguous()
            y41 = torch.empty((1, H4), dtype=torch.float32, device=dev)

            def step4f(i):
                fa.moe_ffn(ex4[0], ex4[1], ex4[2], E4, x41, ids41[i % 8], w41, out=y41)
            _, t = timed(step4f, 400, 200)
            tok4_bytes = K4 * 3 * F4 * H4 // 32 * 17
            extra["MoE layer 32x top-4, 2880/2880, 1 token (decode), MXFP4 experts"] = {
                "us_per_step": round(t / 400 * 1e6, 2), "algorithmic_GBs": round(tok4_bytes / (t / 400) / 1e9, 1),
                "frac_of_hbm_peak": round(tok4_bytes / (t / 400) / 1e9 / HBM_PEAK_GBS, 4)}
            for w in ex4:
                w.keep_decoded()
            _, t = timed(step4e, 20, 10)
            extra["MoE layer 32x top-4, 2880/2880, 512 tokens, MXFP4 experts (decoded copies kept)"] = {
                "us_per_step": round(t / 20 * 1e6, 2), "tokens_per_s": round(T / (t / 20), 0),
                "TOPS": round(2.0 * T * K4 * 3 * F4 * H4 / (t / 20) / 1e12, 1)}
            for w in ex4:
                w.release()
        if want('thin'):
            # batched decode, M=8 (weights read once per batch), and the whole decode FFN in one call
            # (gate and up share one quantized activation, SwiGLU, down)
            g8 = [fa.Weights.from_device(kind, data_dev, rows, cols) for _ in range(8)]
            u8 = [fa.Weights.from_device(kind, data_dev, rows, cols) for _ in range(8)]
            d6 = torch.from_numpy(random_blocks(fa.Q6_K, cols, rows, seed=79)).to(dev)
            dn = [fa.Weights.from_device(fa.Q6_K, d6, cols, rows) for _ in range(8)]
            x8 = torch.from_numpy(synth.activations(9, 8, cols)).to(dev)
            h8 = torch.from_numpy(synth.activations(10, 8, rows)).to(dev)
            y8 = torch.empty((8, rows), dtype=torch.float32, device=dev)
            z8 = torch.empty((8, cols), dtype=torch.float32, device=dev)
            d5 = torch.from_numpy(random_blocks(fa.Q5_K, rows, cols, seed=80)).to(dev)
            q5 = [fa.Weights.from_device(fa.Q5_K, d5, rows, cols) for _ in range(8)]
            for name, mats, xin, yout in (("Q4_K thin GEMM M=8 14336x4096", g8, x8, y8),
                                          ("Q6_K thin GEMM M=8 4096x14336", dn, h8, z8),
                                          ("Q5_K thin GEMM M=8 14336x4096", q5, x8, y8)):
                def step5(i, mats=mats, xin=xin, yout=yout):
                    mats[i % 8].gemm(xin, out=yout)
                _, t = timed(step5, 400, 200)
                wb = mats[0].rows * (mats[0].cols // 256) * fa.BLOCK[mats[0].kind][0]
                extra[name] = {"us_per_step": round(t / 400 * 1e6, 2), "GBs": round(wb / (t / 400) / 1e9, 1),
                               "frac_of_hbm_peak": round(wb / (t / 400) / 1e9 / HBM_PEAK_GBS, 4)}
            # the same M=8 batches from activations quantized beforehand (by the kernel that produced them, or
            # shared with another projection): the multiplying launch alone
            for name, mats, xin, yout in (("Q4_K thin GEMM M=8 14336x4096, activations quantized beforehand", g8, x8, y8),
                                          ("Q6_K thin GEMM M=8 4096x14336, activations quantized beforehand", dn, h8, z8)):
                acts8 = fa.quantize_q8_k(xin)

                def step5q(i, mats=mats, acts8=acts8, yout=yout):
                    mats[i % 8].gemm_q8k(acts8, 8, out=yout)
                _, t = timed(step5q, 400, 200)
                wb = mats[0].rows * (mats[0].cols // 256) * fa.BLOCK[mats[0].kind][0]
                extra[name] = {"us_per_step": round(t / 400 * 1e6, 2), "GBs": round(wb / (t / 400) / 1e9, 1),
                               "frac_of_hbm_peak": round(wb / (t / 400) / 1e9 / HBM_PEAK_GBS, 4)}
            yf = torch.empty(cols, dtype=torch.float32, device=dev)

            def step6(i):
                fa.ffn_swiglu(g8[i % 8], u8[i % 8], dn[i % 8], xd, out=yf)
            _, t = timed(step6, 400, 200)
            fb = 2 * wbytes + d6.numel()
            extra["decode FFN 4096->14336->4096 (gate, up Q4_K; down Q6_K)"] = {
                "us_per_step": round(t / 400 * 1e6, 2), "GBs": round(fb / (t / 400) / 1e9, 1),
                "frac_of_hbm_peak": round(fb / (t / 400) / 1e9 / HBM_PEAK_GBS, 4)}
            for w in g8 + u8 + dn + q5:
                w.release()
        if want('qkv'):
            # q/k/v of a Llama-3-8B layer (4096, 1024 and 1024 rows of 4096): one launch for the three;
            # 40 sets of weights in turn (566 MB > the 256 MB Infinity Cache)
            qkv_rows = (4096, 1024, 1024)
            qkv_dev = [torch.from_numpy(random_blocks(kind, r, cols, seed=90 + j)).to(dev) for j, r in enumerate(qkv_rows)]
            qkv_sets = [[fa.Weights.from_device(kind, d.clone(), r, cols) for d, r in zip(qkv_dev, qkv_rows)] for _ in range(40)]
            qkv_out = [torch.empty(r, dtype=torch.float32, device=dev) for r in qkv_rows]

            def step7(i):
                fa.gemv_multi(qkv_sets[i % 40], xd, outs=qkv_out)
            _, t = timed(step7, 800, 400)
            qb = sum(qkv_rows) * (cols // 256) * 144
            extra["Q4_K q/k/v multi-GEMV (4096+1024+1024)x4096, one launch"] = {
                "us_per_step": round(t / 800 * 1e6, 2), "GBs": round(qb / (t / 800) / 1e9, 1),
                "frac_of_hbm_peak": round(qb / (t / 800) / 1e9 / HBM_PEAK_GBS, 4)}
            for ws_ in qkv_sets:
                for w in ws_:
                    w.release()
        out["extra"] = extra

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(kind, data, rows, cols, x, y_gpu, synth.activations(6, 512, cols, outlier_frac=0.01))
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
