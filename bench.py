#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

Headline workload (what `value` measures): one decode step (m = 1) through every quantized
linear layer of a Llama-7B-shaped model -- per decoder layer four 4096x4096, two 11008x4096 and one
4096x11008 `fused_linear_with_groupwise_quantized_weight` calls, symmetric int4 weights packed two
per byte, group_size 128 along K, fp16 scales, fp16 bias -- over `--layers` layers with DISTINCT
weights (32 layers = 3.3 GB of packed weights, far beyond L2 + Infinity Cache, so every launch
streams its weights from HBM).  value = algorithmic bytes of all launches / wall time of the step.

The same JSON line carries
  roofline      for the dominant kernel (gemv_w4_m1, the decode kernel for one row of x, on the
                4096-row shapes: four 4096x4096 and one 4096x11008 per layer): algorithmic bytes
                per launch / average launch duration, timed live with events on the launch stream
                over a region that contains only that kernel's launches;
  cpu_baseline  the CPU oracle (scalar C port of the reference composition dequantize -> matmul)
                on one decoder layer's seven GEMVs, single thread;
  secondary     the other BASELINE configurations (prefill W8A16 GEMM at m=2048, dequantize,
                LayerNorm+observer / quantize, int8 matmul_quant, observer/quantize of a
                4096x4096 fp32 weight), each with its own roofline fraction.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the dominant kernel (mean over the launches of the roofline region: four
# of 4096x4096 to one of 4096x11008) from two `rocprofv3 --pmc` runs of `bench.py --pmc-calibration`
# (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for an elementwise
# kernel of known size: x2.0 and x1.0); the summary is
# profiles/gemv_w4_m1__llama7b_decode_m1__hbm_traffic_pmc.txt (11,747,966 B; rounded to 1000 B
# here).  Valid for m = 1 only.
PMC_TRAFFIC_BYTES_PER_LAUNCH_M1 = 11748000
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "i8": 5000.0}

LLAMA7B_LAYER = [  # (name, n, k, count per decoder layer)
    ("qkvo", 4096, 4096, 4),
    ("gate_up", 11008, 4096, 2),
    ("down", 4096, 11008, 1),
]


def gemv_bytes(m, n, k, g=128, bits=4, tsize=2, asym=False):
    """Algorithmic bytes of one fused linear: each tensor once, packed sizes."""
    b = n * k * bits // 8 + n * (k // g) * tsize * (2 if asym else 1)
    return b + m * k * tsize + n * tsize + m * n * tsize


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--m", type=int, default=1, help="decode batch (rows of x), 1..16")
    ap.add_argument("--no-graph", action="store_true", help="launch directly instead of replaying a HIP graph")
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="for a `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE` run: a few direct launches of "
                         "the hot path (plain and fused step), the LayerNorm -> quantize pair, plus an elementwise kernel of known traffic (1 GiB read, "
                         "1 GiB written) to scale the counters by; prints no result line")
    ap.add_argument("--pmc-gemm", action="store_true",
                    help="for a `rocprofv3 --pmc` run on the MFMA kernels: three launches each of the "
                         "prefill linear (with and without its workspace) and of matmul_quant at "
                         "m=2048; prints no result line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is single-GPU by design (the path has no collectives); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import oneflow_amd
    from oneflow_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    L = _lib.lib()
    P = load_probes()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(1234)
    M = args.m
    if args.pmc_gemm:
        pmc_gemm(L, _lib, torch, dev)
        return

    # ---- synthetic Llama-7B-shaped int4 weights, distinct per layer ----------------------------
    layers = []
    for _ in range(args.layers):
        mats = []
        for name, n, k, cnt in LLAMA7B_LAYER:
            for _c in range(cnt):
                w = torch.randint(-128, 128, (n, k // 2), dtype=torch.int8, device=dev)
                scale = torch.empty((n, k // 128), dtype=torch.float16, device=dev).uniform_(1e-3, 1e-2)
                bias = (torch.randn(n, device=dev) * 0.01).to(torch.float16)
                out = torch.empty((max(M, 64), n), dtype=torch.float16, device=dev)
                mats.append((name, n, k, w, scale, bias, out))
        layers.append(mats)
    x_by_k = {k: torch.randn((max(M, 64), k), device=dev).to(torch.float16) for k in (4096, 11008)}

    def launch(mat, m=M):
        name, n, k, w, scale, bias, out = mat
        st = L.ofq_fused_linear_gq(torch.cuda.current_stream().cuda_stream, x_by_k[k].data_ptr(),
                                   w.data_ptr(), scale.data_ptr(), None, bias.data_ptr(),
                                   out.data_ptr(), _lib.I8, _lib.F16, 4, 1, 1, 128, m, n, k, None, 0)
        if st != 0:
            raise RuntimeError(f"ofq_fused_linear_gq status {st}")

    def step_all(m=M):
        for mats in layers:
            for mat in mats:
                launch(mat, m)

    def step_dominant():
        for mats in layers:
            for mat in mats:
                if mat[1] == 4096:
                    launch(mat)

    # the same step with the block's neighbouring ops fused: q/k/v as one grouped launch,
    # o, gate|up with the SiLU gating as one launch, down: 4 launches per layer, not 7 (+ gating)
    glu_y = torch.empty((max(M, 64), 11008), dtype=torch.float16, device=dev)
    vp = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    i64 = lambda v: (ctypes.c_int64 * len(v))(*v)

    def step_fused(m=M):
        stream = torch.cuda.current_stream().cuda_stream
        for mats in layers:
            qkv, o, gate, up, down = mats[0:3], mats[3], mats[4], mats[5], mats[6]
            x4 = x_by_k[4096]
            st = L.ofq_grouped_linear_gq(
                stream, 3, vp([x4] * 3), vp([q[3] for q in qkv]), vp([q[4] for q in qkv]), None,
                vp([q[5] for q in qkv]), vp([q[6] for q in qkv]), i64([m] * 3), i64([4096] * 3),
                i64([4096] * 3), _lib.I8, _lib.F16, 4, 1, 1, 128)
            if st != 0:
                raise RuntimeError(f"ofq_grouped_linear_gq status {st}")
            launch(o, m)
            st = L.ofq_fused_glu_gq(stream, x4.data_ptr(), up[3].data_ptr(), up[4].data_ptr(), None,
                                    up[5].data_ptr(), gate[3].data_ptr(), gate[4].data_ptr(), None,
                                    gate[5].data_ptr(), glu_y.data_ptr(), up[6].data_ptr(),
                                    gate[6].data_ptr(), 5, _lib.I8, _lib.F16, 4, 1, 1, 128, m,
                                    11008, 4096)
            if st != 0:
                raise RuntimeError(f"ofq_fused_glu_gq status {st}")
            launch(down, m)

    def make_runner(fn):
        if args.no_graph:
            return fn
        # warm up outside capture, then capture the launches into one HIP graph
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g.replay

    def time_region(run, steps, warmup):
        for _ in range(warmup):
            run()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            run()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        return e0.elapsed_time(e1), wall_ms

    if args.pmc_calibration:
        src = torch.zeros(256 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)  # vectorized_elementwise_kernel: 2^30 B in, 2^30 B out
        for _ in range(2):
            step_all()
        for _ in range(2):
            step_fused()
        # the activation front end of the int8 path: LayerNorm + observer, then quantisation of the
        # y just written, on fresh buffers each time (is y re-read from HBM or from the caches?)
        mm, kk = 2048, 4096
        gam = torch.randn(kk, device=dev).to(torch.float16)
        bet = torch.randn(kk, device=dev).to(torch.float16)
        sc1 = torch.empty(1, dtype=torch.float32, device=dev)
        zp1 = torch.empty(1, dtype=torch.float32, device=dev)
        lws = torch.empty(mm * 4, dtype=torch.uint8, device=dev)
        stream = torch.cuda.current_stream().cuda_stream
        for _ in range(4):
            xa = torch.randn((mm, kk), device=dev).to(torch.float16)
            ya = torch.empty_like(xa)
            qa = torch.empty((mm, kk), dtype=torch.int8, device=dev)
            st = L.ofq_fused_layer_norm_min_max_observer(stream, xa.data_ptr(), gam.data_ptr(),
                                                         bet.data_ptr(), ya.data_ptr(), sc1.data_ptr(),
                                                         zp1.data_ptr(), _lib.F16, mm, kk, 1e-5, 8,
                                                         lws.data_ptr(), mm * 4)
            st |= L.ofq_quantization(stream, ya.data_ptr(), sc1.data_ptr(), zp1.data_ptr(),
                                     qa.data_ptr(), _lib.F16, _lib.I8, mm * kk, 1, 8, 0, 0, 0)
            if st != 0:
                raise RuntimeError(f"layer norm / quantization status {st}")
        torch.cuda.synchronize()
        return

    bytes_step = sum(gemv_bytes(M, n, k) * cnt for _, n, k, cnt in LLAMA7B_LAYER) * args.layers
    launches_step = sum(cnt for *_, cnt in LLAMA7B_LAYER) * args.layers
    run_all = make_runner(step_all)
    ev_ms, wall_ms = time_region(run_all, args.steps, args.warmup)
    ms_per_step = wall_ms / args.steps
    value = bytes_step / (ms_per_step * 1e-3) / 1e9

    # ---- roofline of the dominant kernel: only the launches with n = 4096 (16-wave instance) -----
    bytes_k4096 = sum(gemv_bytes(M, n, k) * cnt for _, n, k, cnt in LLAMA7B_LAYER if n == 4096) * args.layers
    launches_k4096 = sum(cnt for _, n, k, cnt in LLAMA7B_LAYER if n == 4096) * args.layers
    run_k = make_runner(step_dominant)
    ev_k_ms, _ = time_region(run_k, args.steps, args.warmup)
    avg_launch_us = ev_k_ms * 1e3 / (args.steps * launches_k4096)
    achieved = (bytes_k4096 / launches_k4096) / (avg_launch_us * 1e-6) / 1e9
    roofline = {
        "kernel": "gemv_w4_m1 (a wave owns whole weight rows; n=4096 shapes: 4096x4096 x4, 4096x11008 x1 per layer)",
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": PMC_TRAFFIC_BYTES_PER_LAUNCH_M1 if (M == 1 and args.layers == 32) else None,
        "bytes_per_launch": bytes_k4096 // launches_k4096, "avg_launch_us": round(avg_launch_us, 3),
    }

    result = {
        # the first clause of the reference benchmark's metric, which `value` is; the second
        # clause is reported as `second_metric` below (and in `secondary`)
        "metric": "W4A16 GEMV HBM GB/s (% peak) @M=1" if M == 1 else f"W4A16 GEMV HBM GB/s (% peak) @M={M}",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"llama7b_decode_linears_w4a16_sym_g128_m{M}", "layers": args.layers,
                   "launches_per_step": launches_step, "bytes_per_step": bytes_step,
                   "hip_graph": not args.no_graph, "event_ms_per_step": round(ev_ms / args.steps, 4),
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2)},
        "roofline": roofline,
    }

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(M)
    if not args.no_secondary:
        # the same decode step at the other batch sizes of the decode configuration
        other = {}
        for m in (4, 8):
            if m == M:
                continue
            run_m = make_runner(lambda: step_all(m))
            _, wall_m = time_region(run_m, 10, 2)
            b_m = sum(gemv_bytes(m, n, k) * cnt for _, n, k, cnt in LLAMA7B_LAYER) * args.layers
            gbps = b_m / (wall_m / 10 * 1e-3) / 1e9
            other[f"decode_w4a16_m{m}"] = {
                "ms_per_step": round(wall_m / 10, 4), "gbps": round(gbps, 1),
                "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS,
                             "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4)}}
        for m in sorted({M, 4, 8}):
            run_f = make_runner(lambda: step_fused(m))
            _, wall_f = time_region(run_f, 10, 2)
            b_m = sum(gemv_bytes(m, n, k) * cnt for _, n, k, cnt in LLAMA7B_LAYER) * args.layers
            gbps = (b_m + args.layers * m * 11008 * 2) / (wall_f / 10 * 1e-3) / 1e9
            other[f"decode_w4a16_m{m}_grouped_qkv_and_glu"] = {
                "ms_per_step": round(wall_f / 10, 4), "gbps": round(gbps, 1),
                "launches_per_step": 4 * args.layers,
                "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS,
                             "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4)}}
        # the offline tile-major copy of the weights (ofq_groupwise_repack) for 4 and 8 rows of x;
        # a shape the tiled call does not serve at that m (8 rows of 11008 do not fit LDS) keeps
        # the row-major call, as a caller would
        tiled = {}
        for mats in layers:
            for mat in mats:
                nb = L.ofq_groupwise_repack_bytes(4, mat[1], mat[2])
                t = torch.empty(nb, dtype=torch.int8, device=dev)
                st = L.ofq_groupwise_repack(torch.cuda.current_stream().cuda_stream, mat[3].data_ptr(),
                                            t.data_ptr(), 4, mat[1], mat[2])
                if st != 0:
                    raise RuntimeError(f"ofq_groupwise_repack status {st}")
                tiled[id(mat)] = t

        def launch_tiled(mat, m):
            name, n, k, w, scale, bias, out = mat
            st = L.ofq_fused_linear_gq_tiled(torch.cuda.current_stream().cuda_stream,
                                             x_by_k[k].data_ptr(), tiled[id(mat)].data_ptr(),
                                             scale.data_ptr(), None, bias.data_ptr(), out.data_ptr(),
                                             _lib.I8, _lib.F16, 4, 1, 1, 128, m, n, k)
            if st == 5:  # OFQ_ERR_UNSUPPORTED
                launch(mat, m)
                return False
            if st != 0:
                raise RuntimeError(f"ofq_fused_linear_gq_tiled status {st}")
            return True
        for m in (4, 8):
            run_t = make_runner(lambda: [launch_tiled(mat, m) for mats in layers for mat in mats])
            _, wall_t = time_region(run_t, 10, 2)
            b_m = sum(gemv_bytes(m, n, k) * cnt for _, n, k, cnt in LLAMA7B_LAYER) * args.layers
            gbps = b_m / (wall_t / 10 * 1e-3) / 1e9
            by_shape = {}
            for name, n, k, cnt in LLAMA7B_LAYER:
                mats_s = [mat for mats in layers for mat in mats if mat[0] == name]
                served = launch_tiled(mats_s[0], m)
                run_s = make_runner(lambda: [launch_tiled(mat, m) for mat in mats_s])
                ev_s, _ = time_region(run_s, 10, 2)
                by_shape[f"{n}x{k}"] = {"us": round(ev_s * 1e3 / (10 * len(mats_s)), 2),
                                        "tiled_call_serves_it": served}
            other[f"decode_w4a16_m{m}_tile_major_weights"] = {
                "ms_per_step": round(wall_t / 10, 4), "gbps": round(gbps, 1), "by_shape": by_shape,
                "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS,
                             "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4)}}
        del tiled
        # per shape: the GEMV alone over all layers for 1, 4 and 8 rows of x (and 32 and 64, the
        # batch sizes of a serving loop, which run the multi-tile streaming kernel), and beside it a
        # kernel that only reads the codes of the same weight tensors (ofq_bench_probe_read; 97% of the
        # bytes the GEMV reads, in one launch per tensor) in the same graph-replay harness: what
        # reading those bytes once takes on this box
        sink = torch.zeros(1, dtype=torch.int32, device=dev)

        def read_only(mats):
            stream = torch.cuda.current_stream().cuda_stream
            for mat in mats:
                st = P.ofq_bench_probe_read(stream, mat[3].data_ptr(), mat[3].numel(), sink.data_ptr())
                if st != 0:
                    raise RuntimeError(f"ofq_bench_probe_read status {st}")
        for m in sorted({M, 1, 4, 8, 32, 64}):
            by_shape = {}
            for name, n, k, cnt in LLAMA7B_LAYER:
                mats_s = [mat for mats in layers for mat in mats if mat[0] == name]
                run_s = make_runner(lambda: [launch(mat, m) for mat in mats_s])
                ev_s, _ = time_region(run_s, 10, 2)
                us_s = ev_s * 1e3 / (10 * len(mats_s))
                gb_s = gemv_bytes(m, n, k) / (us_s * 1e-6) / 1e9
                by_shape[f"{n}x{k}"] = {"us": round(us_s, 2), "gbps": round(gb_s, 1),
                                        "frac": round(gb_s / HBM_PEAK_GBPS, 4)}
                if m == M:
                    run_r = make_runner(lambda: read_only(mats_s))
                    ev_r, _ = time_region(run_r, 10, 2)
                    by_shape[f"{n}x{k}"]["read_floor_us"] = round(ev_r * 1e3 / (10 * len(mats_s)), 2)
            other[f"decode_w4a16_m{m}_by_shape"] = by_shape
        # the headline step replayed for at least a second (the timed region of the headline is
        # `--steps` replays, some 20 ms): what the path sustains
        n_sus = max(args.steps, int(1.05e3 / ms_per_step) + 1)
        ev_sus, wall_sus = time_region(run_all, n_sus, 1)
        gb_sus = bytes_step / (wall_sus / n_sus * 1e-3) / 1e9
        other[f"decode_w4a16_m{M}_sustained"] = {
            "replays": n_sus, "seconds": round(wall_sus * 1e-3, 3),
            "ms_per_step": round(wall_sus / n_sus, 4), "gbps": round(gb_sus, 1),
            "roofline": {"bound": "hbm", "achieved": round(gb_sus, 1), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": round(gb_sus / HBM_PEAK_GBPS, 4)}}
        # the ceilings the lines above are read against, in the same graph-replay harness: the
        # fixed cost of a launch (a kernel that does nothing) and a plain copy kernel
        stream_now = lambda: torch.cuda.current_stream().cuda_stream
        run_e = make_runner(lambda: [P.ofq_bench_empty_launch(stream_now(), sink.data_ptr())
                                     for _ in range(224)])
        ev_e, _ = time_region(run_e, 10, 2)
        ceilings = {"empty_kernel_us_per_launch": round(ev_e * 1e3 / (10 * 224), 3), "copy_kernel": {}}
        for mb in (16, 32, 128):
            nbytes = mb << 20
            srcs = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(max(2, 1024 // mb))]
            dsts = [torch.empty_like(t) for t in srcs]

            def copies():
                for a, b in zip(srcs, dsts):
                    if P.ofq_bench_copy(stream_now(), b.data_ptr(), a.data_ptr(), nbytes) != 0:
                        raise RuntimeError("ofq_bench_copy failed")
            run_c = make_runner(copies)
            ev_c, _ = time_region(run_c, 10, 2)
            us_c = ev_c * 1e3 / (10 * len(srcs))
            ceilings["copy_kernel"][f"{mb}MiB"] = {"us": round(us_c, 2),
                                                  "gbps_read_plus_write": round(2 * nbytes / (us_c * 1e-6) / 1e9, 1)}
            del srcs, dsts
        other["ceilings_of_this_box"] = ceilings
        del layers
        torch.cuda.empty_cache()
        result["secondary"] = {**other, **secondary(L, _lib, torch, dev, args)}
        pf = result["secondary"]["prefill_w8a16_bf16_m2048"]
        result["second_metric"] = {"metric": "W8A16 GEMM TFLOPS (% MFMA) @M=2048", "value": pf["tflops"],
                                   "unit": "TFLOP/s", "pct_mfma_peak": round(100 * pf["roofline"]["frac"], 2),
                                   "us": pf["us"]}
    print(json.dumps(result))


def load_probes():
    """The measurement probes (a kernel that only reads, an empty kernel, a plain copy): a
    library of their own next to the product library, outside the ABI of include/ofq.h."""
    path = os.path.join(ROOT, "oneflow_amd", "csrc", "libofq_bench_probes.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with __graft_entry__.build()")
    P = ctypes.CDLL(path)
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    P.ofq_bench_probe_read.argtypes, P.ofq_bench_probe_read.restype = [vp, vp, sz, vp], ctypes.c_int
    P.ofq_bench_empty_launch.argtypes, P.ofq_bench_empty_launch.restype = [vp, vp], ctypes.c_int
    P.ofq_bench_copy.argtypes, P.ofq_bench_copy.restype = [vp, vp, vp, sz], ctypes.c_int
    return P


def cpu_baseline(M):
    """The CPU oracle (scalar C: dequantize in fp16 arithmetic, fp32-accumulated matmul) on the
    seven GEMVs of a few decoder layers; single thread, like the reference's CPU kernels.  Beside
    it, labelled apart, the same dequantize -> matmul decomposition as torch CPU tensor ops on all
    the cores torch uses (the oracle's outputs check it)."""
    import torch
    from oracle import ofq_oracle as O
    rng = np.random.default_rng(0)
    total_bytes = 0
    t_total = 0.0
    reps = 4  # about 10 s of scalar CPU work
    mt_bytes = 0
    t_mt = 0.0
    mt_reps = 8
    for name, n, k, cnt in LLAMA7B_LAYER:
        w = rng.integers(-128, 128, size=(n, k // 2), dtype=np.int8)
        scale = rng.uniform(1e-3, 1e-2, size=(n, k // 128)).astype(np.float16)
        bias = (rng.standard_normal(n) * 0.01).astype(np.float16)
        x = rng.standard_normal((M, k)).astype(np.float16)
        t0 = time.perf_counter()
        for _ in range(cnt * reps):
            ref = O.fused_linear(x, w, scale, None, bias, 4, True, 1, 128)
        t_total += time.perf_counter() - t0
        total_bytes += gemv_bytes(M, n, k) * cnt * reps
        # all cores: unpack (high nibble first), T(q) * s in fp16, fp32 matmul, + bias, round to fp16
        wt, st, bt, xt = map(torch.from_numpy, (w, scale, bias, x))
        t0 = time.perf_counter()
        for _ in range(cnt * mt_reps):
            codes = torch.stack((wt >> 4, (wt << 4) >> 4), dim=2).reshape(n, k)
            wd = (codes.to(torch.float16).reshape(n, k // 128, 128) * st[:, :, None]).reshape(n, k)
            got = (xt.float() @ wd.float().t() + bt.float()).to(torch.float16)
        t_mt += time.perf_counter() - t0
        mt_bytes += gemv_bytes(M, n, k) * cnt * mt_reps
        d = got.float().numpy().astype(np.float64) - ref.astype(np.float64)
        rel = float(np.sqrt((d * d).sum() / max((ref.astype(np.float64) ** 2).sum(), 1e-30)))
        assert rel < 1e-3, f"all-cores CPU decomposition differs from the oracle: rel-L2 {rel:.3e}"
    return {"value": round(total_bytes / t_total / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} Llama-7B decoder layers ({7 * reps} GEMVs, {total_bytes} algorithmic bytes, m={M}) "
                      f"through oracle/ofq_oracle.c in {t_total:.2f} s; host has {os.cpu_count()} cpus",
            "all_cores": {"value": round(mt_bytes / t_mt / 1e9, 4), "unit": "GB/s",
                          "cores": torch.get_num_threads(),
                          "sample": f"{mt_reps} layers, the dequantize -> matmul decomposition as torch CPU ops "
                                    f"(unpack, fp16 multiply, fp32 matmul) in {t_mt:.2f} s"}}


def pmc_gemm(L, _lib, torch, dev):
    """BASELINE configurations 4 and 5 (the GEMM halves), a few direct launches each."""
    cs = torch.cuda.current_stream().cuda_stream
    m, n, k, g = 2048, 11008, 4096, 64
    x = torch.randn((m, k), device=dev).to(torch.bfloat16)
    w = torch.randint(0, 256, (n, k), dtype=torch.uint8, device=dev)
    sc = torch.empty((n, k // g), device=dev).uniform_(1e-3, 1e-2).to(torch.bfloat16)
    ze = torch.empty((n, k // g), device=dev).uniform_(120, 136).to(torch.bfloat16)
    o = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ws_bytes = L.ofq_fused_linear_gq_workspace_bytes(_lib.U8, _lib.BF16, 8, 0, 1, g, m, n, k)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    a8 = torch.randint(-128, 128, (m, k), dtype=torch.int8, device=dev)
    w8 = torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev)
    a_s = torch.full((1,), 0.01, dtype=torch.float32, device=dev)
    b_s = torch.empty(n, dtype=torch.float32, device=dev).uniform_(1e-3, 1e-2)
    o16 = torch.empty((m, n), dtype=torch.float16, device=dev)
    for _ in range(3):
        for wptr, wb in ((ws.data_ptr(), ws_bytes), (None, 0)):
            st = L.ofq_fused_linear_gq(cs, x.data_ptr(), w.data_ptr(), sc.data_ptr(), ze.data_ptr(), None,
                                       o.data_ptr(), _lib.U8, _lib.BF16, 8, 0, 1, g, m, n, k, wptr, wb)
            assert st == 0, st
        st = L.ofq_matmul_quant(cs, a8.data_ptr(), w8.data_ptr(), a_s.data_ptr(), b_s.data_ptr(), None,
                                o16.data_ptr(), _lib.F16, m, n, k)
        assert st == 0, st
    torch.cuda.synchronize()


def secondary(L, _lib, torch, dev, args):
    """The other BASELINE configurations, each timed with events over a replayed HIP graph of
    back-to-back calls."""
    out = {}
    cs = lambda: torch.cuda.current_stream().cuda_stream

    def timeit(fn, iters=20, warmup=3):
        """us per call: `iters` calls captured into one HIP graph (so that the host's launch
        cost, two to four launches per call through ctypes, is not what gets measured) and the
        graph replayed three times between events; plain back-to-back launches with --no-graph."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        run, reps = (lambda: [fn() for _ in range(iters)]), 1
        if not args.no_graph:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for _ in range(iters):
                    fn()
            run, reps = g.replay, 3
            run()
            torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (iters * reps)  # us

    def chk(st, what):
        if st != 0:
            raise RuntimeError(f"{what} status {st}")

    # ---- config 4: prefill W8A16 bf16, asymmetric uint8, g=64, m=2048 -------------------------
    m, n, k, g = 2048, 11008, 4096, 64
    x = torch.randn((m, k), device=dev).to(torch.bfloat16)
    w = torch.randint(0, 256, (n, k), dtype=torch.uint8, device=dev)
    sc = torch.empty((n, k // g), device=dev).uniform_(1e-3, 1e-2).to(torch.bfloat16)
    ze = torch.empty((n, k // g), device=dev).uniform_(120, 136).to(torch.bfloat16)
    o = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ws_bytes = L.ofq_fused_linear_gq_workspace_bytes(_lib.U8, _lib.BF16, 8, 0, 1, g, m, n, k)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)  # the op's tmp_buffer
    us = timeit(lambda: chk(L.ofq_fused_linear_gq(cs(), x.data_ptr(), w.data_ptr(), sc.data_ptr(),
                                                  ze.data_ptr(), None, o.data_ptr(), _lib.U8,
                                                  _lib.BF16, 8, 0, 1, g, m, n, k, ws.data_ptr(),
                                                  ws_bytes), "prefill"))
    us_fused = timeit(lambda: chk(L.ofq_fused_linear_gq(cs(), x.data_ptr(), w.data_ptr(),
                                                        sc.data_ptr(), ze.data_ptr(), None,
                                                        o.data_ptr(), _lib.U8, _lib.BF16, 8, 0, 1,
                                                        g, m, n, k, None, 0), "prefill"))
    flops = 2.0 * m * n * k
    tf = flops / (us * 1e-6) / 1e12
    # Two yardsticks for the same shape, measured here so that they can be checked: (1) the same
    # call on operands that toggle few bits (x = 0, all codes equal): MFMA throughput on this part
    # depends on the data (power and clock), and the headline above is quoted on random operands;
    # (2) the vendor GEMM (torch.matmul, bf16 x bf16 with the weights already dequantised, i.e.
    # without the dequantisation this op has to do) on random operands of the same shape.
    x0 = torch.zeros_like(x)
    w0 = torch.full_like(w, 128)
    us_const = timeit(lambda: chk(L.ofq_fused_linear_gq(cs(), x0.data_ptr(), w0.data_ptr(),
                                                        sc.data_ptr(), ze.data_ptr(), None,
                                                        o.data_ptr(), _lib.U8, _lib.BF16, 8, 0, 1,
                                                        g, m, n, k, ws.data_ptr(), ws_bytes),
                                  "prefill, constant operands"))
    del x0, w0
    us_vendor = None
    try:
        wd = torch.randn((n, k), device=dev).to(torch.bfloat16)
        us_vendor = timeit(lambda: torch.matmul(x, wd.t(), out=o))
        del wd
    except Exception as e:  # the yardstick must not take the benchmark down
        print(f"bench.py: vendor GEMM yardstick failed: {e}", file=sys.stderr)
    out["prefill_w8a16_bf16_m2048"] = {
        "us": round(us, 2), "tflops": round(tf, 1), "workspace_bytes": ws_bytes,
        "us_without_workspace": round(us_fused, 2),
        "us_same_call_constant_operands": round(us_const, 2),
        "us_vendor_gemm_bf16_same_shape_random_operands": None if us_vendor is None else round(us_vendor, 2),
        "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_PEAK_TFLOPS["bf16"],
                     "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS["bf16"], 4)}}
    del x, w, sc, ze, o, ws

    # ---- config 2: groupwise_dequantize 11008x4096 uint8 asym g=128 -> fp16 ---------------------
    n, k, g = 11008, 4096, 128
    reps = 8  # rotate buffers: 8 x 137 MB > caches
    qs = [torch.randint(0, 256, (n, k), dtype=torch.uint8, device=dev) for _ in range(reps)]
    sc = torch.empty((n, k // g), device=dev).uniform_(1e-3, 1e-2).to(torch.float16)
    ze = torch.empty((n, k // g), device=dev).uniform_(100, 156).to(torch.float16)
    os_ = [torch.empty((n, k), dtype=torch.float16, device=dev) for _ in range(reps)]
    it = [0]

    def deq():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_groupwise_dequantize(cs(), qs[i].data_ptr(), sc.data_ptr(), ze.data_ptr(),
                                       os_[i].data_ptr(), _lib.U8, _lib.F16, 8, 0, n * (k // g), g, 1),
            "dequantize")
    us = timeit(deq, iters=40)
    nbytes = n * k + 2 * n * (k // g) * 2 + n * k * 2
    gb = nbytes / (us * 1e-6) / 1e9
    out["dequantize_u8_f16_11008x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1),
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gb / HBM_PEAK_GBPS, 4)}}
    del qs, os_

    # ---- config 5: LayerNorm+observer, quantize to int8, int8 matmul_quant ----------------------
    m, n, k = 2048, 11008, 4096
    reps = 8
    xs = [torch.randn((m, k), device=dev).to(torch.float16) for _ in range(reps)]
    gamma = (1 + 0.1 * torch.randn(k, device=dev)).to(torch.float16)
    beta = (0.1 * torch.randn(k, device=dev)).to(torch.float16)
    ys = [torch.empty((m, k), dtype=torch.float16, device=dev) for _ in range(reps)]
    a8 = [torch.empty((m, k), dtype=torch.int8, device=dev) for _ in range(reps)]
    s = torch.empty(1, dtype=torch.float32, device=dev)
    z = torch.empty(1, dtype=torch.float32, device=dev)
    ws = torch.empty(m * 4, dtype=torch.uint8, device=dev)
    it[0] = 0

    def ln():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fused_layer_norm_min_max_observer(cs(), xs[i].data_ptr(), gamma.data_ptr(),
                                                    beta.data_ptr(), ys[i].data_ptr(), s.data_ptr(),
                                                    z.data_ptr(), _lib.F16, m, k, 1e-5, 8,
                                                    ws.data_ptr(), m * 4), "ln_observer")
    us = timeit(ln, iters=40)
    gb = (2 * m * k * 2) / (us * 1e-6) / 1e9
    out["layer_norm_observer_f16_2048x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1),
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gb / HBM_PEAK_GBPS, 4)}}

    # the same call with the row statistics accumulated in fp64 and rounded once
    def ln_exact():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fused_layer_norm_min_max_observer_stats(
            cs(), xs[i].data_ptr(), None, None, 0.0, 0, gamma.data_ptr(), beta.data_ptr(),
            ys[i].data_ptr(), s.data_ptr(), z.data_ptr(), _lib.F16, m, k, 1e-5, 8,
            _lib.LN_STATS_FP64, ws.data_ptr(), m * 4), "ln_observer_stats")
    us_exact = timeit(ln_exact, iters=40)
    out["layer_norm_observer_f16_2048x4096"]["us_with_fp64_row_statistics"] = round(us_exact, 2)

    def sln():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fused_skip_layer_norm_min_max_observer(
            cs(), xs[i].data_ptr(), None, xs[(i + 1) % reps].data_ptr(), 1.0, gamma.data_ptr(),
            beta.data_ptr(), ys[i].data_ptr(), s.data_ptr(), z.data_ptr(), _lib.F16, m, k, 1e-5, 8,
            ws.data_ptr(), m * 4), "skip_ln_observer")
    us = timeit(sln, iters=40)
    gb = (3 * m * k * 2) / (us * 1e-6) / 1e9
    out["skip_layer_norm_observer_f16_2048x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1),
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gb / HBM_PEAK_GBPS, 4)}}

    def qz():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_quantization(cs(), ys[i].data_ptr(), s.data_ptr(), z.data_ptr(), a8[i].data_ptr(),
                               _lib.F16, _lib.I8, m * k, 1, 8, 0, 0, 0), "quantization")
    us = timeit(qz, iters=40)
    gb = (m * k * 3) / (us * 1e-6) / 1e9
    out["quantize_f16_to_i8_2048x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1),
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gb / HBM_PEAK_GBPS, 4)}}

    # the pair as the model runs it: LayerNorm + observer, then quantization of the y just written
    # with the scale just computed.  Algorithmic bytes: x read, y written, y read, int8 written.
    def ln_qz():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fused_layer_norm_min_max_observer(cs(), xs[i].data_ptr(), gamma.data_ptr(),
                                                    beta.data_ptr(), ys[i].data_ptr(), s.data_ptr(),
                                                    z.data_ptr(), _lib.F16, m, k, 1e-5, 8,
                                                    ws.data_ptr(), m * 4), "ln_observer")
        chk(L.ofq_quantization(cs(), ys[i].data_ptr(), s.data_ptr(), z.data_ptr(), a8[i].data_ptr(),
                               _lib.F16, _lib.I8, m * k, 1, 8, 0, 0, 0), "quantization")
    us = timeit(ln_qz, iters=40)
    gb = (m * k * 7) / (us * 1e-6) / 1e9
    out["layer_norm_observer_then_quantize_f16_2048x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1), "algorithmic_bytes": m * k * 7,
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gb / HBM_PEAK_GBPS, 4)}}

    # the same result from the entry point that never writes the normalised tensor (two kernels:
    # x from HBM, x again from L2, codes out); the bytes are those of the pair above, so that the
    # two entries compare on one scale
    nb = L.ofq_fused_layer_norm_quantization_workspace_bytes(_lib.F16, m, k)
    ws2 = torch.empty(nb, dtype=torch.uint8, device=dev)

    def lnq():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fused_layer_norm_quantization(
            cs(), xs[i].data_ptr(), gamma.data_ptr(), beta.data_ptr(), a8[i].data_ptr(),
            s.data_ptr(), z.data_ptr(), _lib.F16, m, k, 1e-5, 8, _lib.LN_STATS_FP32,
            ws2.data_ptr(), nb), "ln_quantization")
    us = timeit(lnq, iters=40)
    gb = (m * k * 3) / (us * 1e-6) / 1e9
    out["layer_norm_quantization_f16_to_i8_2048x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1), "algorithmic_bytes": m * k * 3,
        "us_of_the_two_ops": out["layer_norm_observer_then_quantize_f16_2048x4096"]["us"],
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gb / HBM_PEAK_GBPS, 4)}}

    wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev)
    wsc = torch.empty(n, device=dev).uniform_(1e-3, 1e-2)
    o = torch.empty((m, n), dtype=torch.float16, device=dev)
    us = timeit(lambda: chk(L.ofq_matmul_quant(cs(), a8[0].data_ptr(), wq.data_ptr(), s.data_ptr(),
                                               wsc.data_ptr(), None, o.data_ptr(), _lib.F16, m, n, k),
                            "matmul_quant"))
    tops = 2.0 * m * n * k / (us * 1e-6) / 1e12

    # yardstick: the vendor int8 GEMM (torch._int_mm: int8 x int8 -> int32, without the scaling to
    # fp16 that this op does in its epilogue) on the same operands
    def vendor_int8(a_i8, w_i8):
        try:
            return round(timeit(lambda: torch._int_mm(a_i8, w_i8.t())), 2)
        except Exception as e:  # the yardstick must not take the benchmark down
            print(f"bench.py: vendor int8 GEMM yardstick failed: {e}", file=sys.stderr)
            return None
    out["matmul_quant_i8_m2048"] = {
        "us": round(us, 2), "tops": round(tops, 1),
        "us_vendor_gemm_int8_to_int32_same_operands": vendor_int8(a8[0], wq),
        "roofline": {"bound": "mfma", "achieved": round(tops, 1), "peak": MFMA_PEAK_TFLOPS["i8"],
                     "unit": "TOP/s", "frac": round(tops / MFMA_PEAK_TFLOPS["i8"], 4)}}
    # a batch of 256 rows on a square weight: 32 x 1 tiles of 128 columns, so K is cut into slices
    # in the workspace the op asks for
    mm, nn = 256, 4096
    wsq = torch.randint(-127, 128, (nn, k), dtype=torch.int8, device=dev)
    wssc = torch.empty(nn, device=dev).uniform_(1e-3, 1e-2)
    osq = torch.empty((mm, nn), dtype=torch.float16, device=dev)
    mq_ws_bytes = L.ofq_matmul_quant_workspace_bytes(mm, nn, k)
    mq_ws = torch.empty(max(mq_ws_bytes, 16), dtype=torch.uint8, device=dev)
    us = timeit(lambda: chk(L.ofq_matmul_quant_ws(cs(), a8[0].data_ptr(), wsq.data_ptr(), s.data_ptr(),
                                                  wssc.data_ptr(), None, osq.data_ptr(), _lib.F16, mm,
                                                  nn, k, mq_ws.data_ptr(), mq_ws_bytes),
                            "matmul_quant k slices"))
    tops = 2.0 * mm * nn * k / (us * 1e-6) / 1e12
    out["matmul_quant_i8_m256_4096x4096"] = {
        "us": round(us, 2), "tops": round(tops, 1), "workspace_bytes": int(mq_ws_bytes),
        "us_vendor_gemm_int8_to_int32_same_operands": vendor_int8(a8[0][:mm], wsq),
        "roofline": {"bound": "mfma", "achieved": round(tops, 1), "peak": MFMA_PEAK_TFLOPS["i8"],
                     "unit": "TOP/s", "frac": round(tops / MFMA_PEAK_TFLOPS["i8"], 4)}}
    del wsq, osq, mq_ws

    # the same op at decode (m = 1 and 16): the streaming int8 kernel; 6 weight sets cycled so that
    # no launch finds its weight in the caches
    reps_w = 6
    wqs = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev) for _ in range(reps_w)]
    for md in (1, 16):
        ad = torch.randint(-128, 128, (md, k), dtype=torch.int8, device=dev)
        od = torch.empty((md, n), dtype=torch.float16, device=dev)

        def mq_dec():
            for i in range(reps_w):
                chk(L.ofq_matmul_quant(cs(), ad.data_ptr(), wqs[i].data_ptr(), s.data_ptr(),
                                       wsc.data_ptr(), None, od.data_ptr(), _lib.F16, md, n, k),
                    "matmul_quant decode")
        us = timeit(mq_dec, iters=10) / reps_w
        nbytes = n * k + n * 4 + md * k + md * n * 2
        gb = nbytes / (us * 1e-6) / 1e9
        out[f"matmul_quant_i8_decode_11008x4096_m{md}"] = {
            "us": round(us, 2), "gbps": round(gb, 1),
            "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBPS, 4)}}
    del xs, ys, a8, wq, o, wqs

    # ---- config 1: observer / quantization / fake_quantization of a 4096x4096 fp32 weight --------
    reps = 6
    wsrc = [(torch.randn((4096, 4096), device=dev) * 0.02) for _ in range(reps)]
    qo = [torch.empty((4096, 4096), device=dev) for _ in range(reps)]
    sc = torch.empty(4096, device=dev)
    zp = torch.empty(4096, device=dev)
    wsb = L.ofq_min_max_observer_workspace_bytes(_lib.F32, 4096 * 4096, 4096)
    ws = torch.empty(wsb, dtype=torch.uint8, device=dev)
    it[0] = 0

    def obs():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_min_max_observer(cs(), wsrc[i].data_ptr(), sc.data_ptr(), zp.data_ptr(), _lib.F32,
                                   4096 * 4096, 4096, 8, 0, 0, ws.data_ptr(), wsb), "observer")

    def qf32():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_quantization(cs(), wsrc[i].data_ptr(), sc.data_ptr(), zp.data_ptr(),
                               qo[i].data_ptr(), _lib.F32, _lib.F32, 4096 * 4096, 4096, 8, 0, 0, 0),
            "quantization f32")

    def fq32():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fake_quantization(cs(), wsrc[i].data_ptr(), sc.data_ptr(), zp.data_ptr(),
                                    qo[i].data_ptr(), _lib.F32, 4096 * 4096, 4096, 8, 0, 0, 0),
            "fake_quantization f32")
    for name, fn, nbytes in (("min_max_observer_f32_4096x4096", obs, 4096 * 4096 * 4),
                             ("quantization_f32_4096x4096", qf32, 4096 * 4096 * 8),
                             ("fake_quantization_f32_4096x4096", fq32, 4096 * 4096 * 8)):
        us = timeit(fn, iters=30)
        gb = nbytes / (us * 1e-6) / 1e9
        out[name] = {"us": round(us, 2), "gbps": round(gb, 1),
                     "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS,
                                  "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBPS, 4)}}
    del wsrc, qo

    # ---- decode of the variants whose w~ is formed with the reference's roundings: W4 with a zero
    # point g=128 in fp16 and bf16, fp16 W8 g=64; m = 1 (a wave owns whole rows) and 16 (MFMA,
    # natural element order), gate/up shape; 8 weight sets cycled so that no launch finds its
    # codes in cache
    n, k = 11008, 4096
    for tag, tcode, tdt, bits, g in (("f16_w4_asym_g128", _lib.F16, torch.float16, 4, 128),
                                     ("bf16_w4_asym_g128", _lib.BF16, torch.bfloat16, 4, 128),
                                     ("f16_w8_asym_g64", _lib.F16, torch.float16, 8, 64)):
        reps = 8
        ws = [torch.randint(0, 256, (n, k * bits // 8), dtype=torch.uint8, device=dev) for _ in range(reps)]
        sc = torch.empty((n, k // g), device=dev).uniform_(1e-3, 1e-2).to(tdt)
        ze = torch.empty((n, k // g), device=dev).uniform_(0.01, 0.05).to(tdt)
        for m in (1, 16):
            xx = torch.randn((m, k), device=dev).to(tdt)
            oo = torch.empty((m, n), dtype=tdt, device=dev)

            def dec():
                for i in range(reps):
                    chk(L.ofq_fused_linear_gq(cs(), xx.data_ptr(), ws[i].data_ptr(), sc.data_ptr(),
                                              ze.data_ptr(), None, oo.data_ptr(), _lib.U8, tcode, bits,
                                              0, 1, g, m, n, k, None, 0), "decode " + tag)
            us = timeit(dec, iters=10) / reps
            nbytes = n * k * bits // 8 + 2 * n * (k // g) * 2 + m * k * 2 + m * n * 2
            gb = nbytes / (us * 1e-6) / 1e9
            out[f"decode_{tag}_11008x4096_m{m}"] = {
                "us": round(us, 2), "gbps": round(gb, 1),
                "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS,
                             "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBPS, 4)}}
        del ws

    # ---- groups along N (group_dim = 0, scale [n/g, k]): fp16 W4 symmetric g=128, m = 1 and 16 ---
    n, k, g = 11008, 4096, 128
    reps = 8
    ws = [torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev) for _ in range(reps)]
    sc = torch.empty((n // g, k), device=dev).uniform_(1e-3, 1e-2).to(torch.float16)
    for m in (1, 16):
        xx = torch.randn((m, k), device=dev).to(torch.float16)
        oo = torch.empty((m, n), dtype=torch.float16, device=dev)

        def dec_gn():
            for i in range(reps):
                chk(L.ofq_fused_linear_gq(cs(), xx.data_ptr(), ws[i].data_ptr(), sc.data_ptr(), None,
                                          None, oo.data_ptr(), _lib.I8, _lib.F16, 4, 1, 0, g, m, n, k,
                                          None, 0), "decode, groups along N")
        us = timeit(dec_gn, iters=10) / reps
        nbytes = n * k // 2 + (n // g) * k * 2 + m * k * 2 + m * n * 2
        gb = nbytes / (us * 1e-6) / 1e9
        out[f"decode_f16_w4_groups_along_n_g128_11008x4096_m{m}"] = {
            "us": round(us, 2), "gbps": round(gb, 1),
            "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBPS, 4)}}
    del ws

    # ---- the same decode kernel on a large weight: an int4 output layer, 128256 x 4096 ---------
    # (263 MB per launch: the fixed cost per launch that bounds the 8-23 MB layer shapes is small
    # here, so this shows what the kernel itself streams at)
    n, k, g = 128256, 4096, 128
    reps = 3
    ws = [torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev) for _ in range(reps)]
    sc = torch.empty((n, k // g), dtype=torch.float16, device=dev).uniform_(1e-3, 1e-2)
    xx = torch.randn((1, k), device=dev).to(torch.float16)
    oo = torch.empty((1, n), dtype=torch.float16, device=dev)
    it[0] = 0

    def head():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_fused_linear_gq(cs(), xx.data_ptr(), ws[i].data_ptr(), sc.data_ptr(), None, None,
                                  oo.data_ptr(), _lib.I8, _lib.F16, 4, 1, 1, g, 1, n, k, None, 0),
            "lm head")
    us = timeit(head, iters=12)
    nbytes = gemv_bytes(1, n, k) - n * 2  # no bias
    gb = nbytes / (us * 1e-6) / 1e9
    out["decode_w4a16_output_layer_128256x4096_m1"] = {
        "us": round(us, 2), "gbps": round(gb, 1),
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBPS, 4)}}
    del ws

    # ---- weight quantise + pack: fp16 [11008,4096] -> symmetric int4, g=128 -------------------
    n, k, g = 11008, 4096, 128
    reps = 6  # 6 x 90 MB of distinct sources: beyond the caches
    wsrc = [(torch.randn((n, k), device=dev) * 0.02).to(torch.float16) for _ in range(reps)]
    qo = torch.empty((n, k // 2), dtype=torch.int8, device=dev)
    so = torch.empty((n, k // g), dtype=torch.float16, device=dev)
    it = [0]

    def wq():
        i = it[0] % reps
        it[0] += 1
        chk(L.ofq_groupwise_quantize(cs(), wsrc[i].data_ptr(), qo.data_ptr(), so.data_ptr(), None,
                                     _lib.F16, _lib.I8, 4, 1, 1, g, n, k), "groupwise_quantize")
    us = timeit(wq, iters=24)
    nbytes = n * k * 2 + n * k // 2 + n * (k // g) * 2
    gb = nbytes / (us * 1e-6) / 1e9
    out["weight_quantize_f16_to_int4_11008x4096"] = {
        "us": round(us, 2), "gbps": round(gb, 1),
        "roofline": {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBPS, 4)}}
    return out


if __name__ == "__main__":
    main()
