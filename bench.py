#!/usr/bin/env python3
"""Benchmark of the fused-kernel hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-rotating] [--only NAME]

A step is one launch of the fused three-stage blur chain (x, y, x; 3 taps of
weight 1/3) on an 8192 x 8192 fp32 image that is already resident in HBM; the
headline value is its whole-job throughput in GB/s of ALGORITHMIC bytes
(logical input read once + logical output written once).  The same line also
carries the other configurations of the metric (row softmax, GEMM fp32 / bf16,
fused QK^T softmax), each with its own roofline fraction, a roofline object
for the dominant kernel timed with HIP events on the launching stream, and the
CPU baseline: the reference library's own CPU lowering of the same composed
pipeline (oracle/_ref/, when it was built) or the CPU oracle, timed on one host
core.

Prints exactly one JSON line on stdout.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 MFMA
FP32_VECTOR_PEAK_TFLOPS = 157.3
# HBM bytes one launch of the headline kernel moves, from the FETCH_SIZE and
# WRITE_SIZE counters scaled by the plain-copy calibration kernel below
# (profiles/bench_all_workloads_hbm_traffic.md).  Counters cannot be read from
# inside this process; the figure is re-measured whenever the kernel changes.
BLUR_XYX_8192_TRAFFIC_BYTES = 548743032


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_launches(fn, warmup, steps, torch, gern_amd):
    """Returns (wall ms per step, event ms per step) over exactly `steps` launches."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = gern_amd.Event(), gern_amd.Event()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, start.elapsed_ms_until(stop) / steps


def per_launch_ms(fn, n, torch, gern_amd):
    """Durations of n single launches, each between its own pair of events."""
    pairs = [(gern_amd.Event(), gern_amd.Event()) for _ in range(n)]
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    return sorted(start.elapsed_ms_until(stop) for start, stop in pairs)


COPY_SRC = r"""
extern "C" __global__ void __launch_bounds__(256) gern_copy_f4(const float4 *in, float4 *out, long long n)
{
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = in[i];
}
typedef float gern_f4 __attribute__((ext_vector_type(4)));
extern "C" __global__ void __launch_bounds__(256) gern_copy_f4_streaming(const gern_f4 *in, gern_f4 *out, long long n)
{
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) __builtin_nontemporal_store(in[i], out + i);
}
"""


def copy_calibration(torch, gern_amd, warmup, steps, kernel="gern_copy_f4", nbytes=256 << 20):
    """A plain float4 copy of 256 MiB through the same C ABI.  gern_copy_f4 is
    the kernel of known size that the FETCH_SIZE / WRITE_SIZE counters are
    scaled by; gern_copy_f4_streaming (nontemporal stores, as the gernels use)
    shows the HBM rate a trivial kernel reaches on this device."""
    import ctypes as C
    hip = gern_amd.hip_lib()
    mod, ker = C.c_void_p(), C.c_void_p()
    names = (C.c_char_p * 1)(kernel.encode())
    if hip.gern_hip_compile(COPY_SRC.encode(), names, 1, None, 0, None, C.byref(mod)) != 0 or \
       hip.gern_hip_get_kernel(mod, kernel.encode(), C.byref(ker)) != 0:
        raise gern_amd.GernError(gern_amd._hip_error())
    src = torch.ones(nbytes // 4, device="cuda")
    dst = torch.zeros_like(src)
    n = C.c_longlong(nbytes // 16)
    a, b = C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr())
    params = (C.c_void_p * 3)(C.cast(C.byref(a), C.c_void_p), C.cast(C.byref(b), C.c_void_p), C.cast(C.byref(n), C.c_void_p))
    grid = (C.c_uint32 * 3)((nbytes // 16 + 255) // 256, 1, 1)
    block = (C.c_uint32 * 3)(256, 1, 1)

    def launch():
        if hip.gern_hip_launch(ker, grid, block, 0, params, None) != 0:
            raise gern_amd.GernError(gern_amd._hip_error())
    wall, ev = time_launches(launch, warmup, steps, torch, gern_amd)
    assert bool((dst == 1).all())
    return {"GB/s": 2 * nbytes / (ev * 1e-3) / 1e9, "ms": ev, "frac_hbm": 2 * nbytes / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "kernel": kernel, "bytes_read": nbytes, "bytes_written": nbytes}


def cpu_baseline_blur(img_np):
    """The same composed pipeline on ONE host core."""
    from oracle import oracle as o
    from oracle import ref
    rows, cols = img_np.shape
    if ref.available():
        kind = "reference"
        # tile sizes must divide the 8190 x 8188 output (the reference handles no ragged tiles)
        run = lambda: ref.blur_chain(img_np, "xyx", 90, 356)  # noqa: E731
        what = "reference library CPU lowering of Tile(rows=90)(Tile(cols=356)(blur_x, blur_y, blur_x)), g++ -O2"
    else:
        kind = "port"
        run = lambda: o.blur_chain_tiled(img_np, "xyx", 90, 356)  # noqa: E731
        what = "CPU oracle (scalar C restatement), same tiling, gcc -O2"
    run()  # warm-up
    times = []
    budget = time.perf_counter() + 20.0
    while len(times) < 5 and (len(times) < 1 or time.perf_counter() < budget):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    nbytes = rows * cols * 4 + (rows - 2) * (cols - 4) * 4
    return {
        "value": nbytes / med / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "host_cores": os.cpu_count(),
        "kind": kind,
        "seconds": med,
        "sample": "full workload (8192x8192 three-stage blur), median of %d runs after one warm-up; %s" % (len(times), what),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-rotating", action="store_true",
                    help="skip the extra timings over rotating buffers (profiles: keeps one kind of launch per kernel)")
    ap.add_argument("--only", default="", help="run only this workload (blur, softmax, gemm_f32, gemm_bf16, qk_softmax, copy)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import numpy as np
    import torch

    import __graft_entry__
    __graft_entry__.ensure_built()  # builds only in a fresh checkout
    import gern_amd
    from gern_amd import inputs

    if gern_amd.device_count() < 1 or not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: there is no CPU fallback")
    lim = gern_amd.device_limits()
    log("device:", lim.arch.decode(), "CUs:", lim.compute_units)

    want = lambda name: (not args.only) or args.only == name  # noqa: E731
    workloads = {}
    result = None

    # ---- config 2: three-stage blur, 8192 x 8192 (the headline) ------------
    if want("blur"):
        rows = cols = 8192
        img = inputs.uniform((rows, cols), 2)
        d_in = torch.from_numpy(img).cuda()
        blur = gern_amd.BlurChain("xyx", tile_rows=4)  # 4 x 224 tiles, line-aligned store windows
        d_out = torch.zeros(blur.out_shape(rows, cols), device="cuda")
        wall, ev = time_launches(lambda: blur(d_in, d_out), args.warmup, args.steps, torch, gern_amd)
        nbytes = img.nbytes + d_out.numel() * 4
        gbs = nbytes / (wall * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": nbytes / (ev * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": nbytes / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": BLUR_XYX_8192_TRAFFIC_BYTES,
                "kernel": blur.kernel_name, "kernel_ms": ev, "algorithmic_bytes": nbytes}
        each = per_launch_ms(lambda: blur(d_in, d_out), 50, torch, gern_amd)
        roof["kernel_ms_median"] = each[len(each) // 2]
        roof["kernel_ms_min"] = each[0]
        workloads["blur_xyx_8192"] = {"GB/s": gbs, "ms": wall, "frac_hbm": gbs / HBM_PEAK_GBS}
        log("blur xyx 8192^2: %.1f us/launch  %.0f GB/s  (%.1f%% of HBM peak)" % (wall * 1e3, gbs, 100 * gbs / HBM_PEAK_GBS))
        if not args.no_rotating:
            # The same launch over ROTATING buffer pairs: the 256 MiB image is exactly the size of the
            # memory-side cache, and with streaming stores a launch finds part of its input there when
            # the previous launch read the same buffer.  Rotating over four pairs takes that away.
            ring = [(d_in, d_out)] + [(d_in.clone(), torch.zeros_like(d_out)) for _ in range(3)]
            turn = [0]

            def rotating():
                a, b = ring[turn[0] % len(ring)]
                turn[0] += 1
                blur(a, b)
            wall_r, ev_r = time_launches(rotating, args.warmup, args.steps, torch, gern_amd)
            workloads["blur_xyx_8192_rotating_buffers"] = {"GB/s": nbytes / (ev_r * 1e-3) / 1e9, "ms": ev_r,
                                                           "frac_hbm": nbytes / (ev_r * 1e-3) / 1e9 / HBM_PEAK_GBS, "buffer_pairs": len(ring)}
            log("blur xyx 8192^2 over %d rotating buffer pairs: %.1f us/launch  %.0f GB/s" % (len(ring), ev_r * 1e3, nbytes / (ev_r * 1e-3) / 1e9))
            # `value`, `achieved` and `frac` follow the reference's own protocol (apps/blur/blur.cu:79-96: warm-up,
            # then N launches on the SAME buffers); the rotating figure is what HBM alone sustains.
            roof["achieved_rotating_buffers"] = nbytes / (ev_r * 1e-3) / 1e9
            roof["frac_rotating_buffers"] = roof["achieved_rotating_buffers"] / HBM_PEAK_GBS
            roof["kernel_ms_rotating_buffers"] = ev_r
            del ring
        result = {
            "metric": "fused 3-stage blur (x,y,x) 8192x8192 fp32, algorithmic GB/s",
            "value": gbs,
            "unit": "GB/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": wall,
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "f32",
            "data": "synthetic",
            "config": {"workload": "three-stage fused separable blur chain (3-tap x, y, x; weights 1/3), 8192x8192 fp32 "
                                   "uniform[0,1) seed 2, valid-region output 8190x8188, one launch per step",
                       "schedule": "one wavefront per 4x224 output tile, store windows moved to whole 128-byte lines, XCD-aware workgroup order",
                       "protocol": "the reference's: warm-up, then `steps` launches on the same buffers "
                                   "(roofline.achieved_rotating_buffers: the same launches over four rotating "
                                   "buffer pairs, which takes the 256 MiB memory-side cache out of the figure)"},
            "roofline": roof,
        }
        if not args.no_cpu:
            result["cpu_baseline"] = cpu_baseline_blur(img)
            log("cpu baseline: %.2f GB/s on 1 core (%s)" % (result["cpu_baseline"]["value"], result["cpu_baseline"]["kind"]))
        del d_in, d_out

    steps2 = max(10, args.steps // 4)
    # ---- config 3: row softmax, 8192 x 4096 --------------------------------
    if want("softmax"):
        x = inputs.normal((8192, 4096), 3, 0.0, 2.0)
        d_x = torch.from_numpy(x).cuda()
        d_y = torch.zeros_like(d_x)
        sm = gern_amd.Softmax(4096)
        wall, ev = time_launches(lambda: sm(d_x, d_y), args.warmup, steps2, torch, gern_amd)
        gbs = 2 * x.nbytes / (ev * 1e-3) / 1e9
        workloads["softmax_8192x4096"] = {"GB/s": gbs, "ms": ev, "frac_hbm": gbs / HBM_PEAK_GBS, "kernel": sm.kernel_name}
        log("softmax 8192x4096: %.1f us  %.0f GB/s (%.1f%%)" % (ev * 1e3, gbs, 100 * gbs / HBM_PEAK_GBS))
        if not args.no_rotating:
            ring = [(d_x, d_y)] + [(d_x.clone(), torch.zeros_like(d_y)) for _ in range(5)]
            turn = [0]

            def rotating_softmax():
                a, b = ring[turn[0] % len(ring)]
                turn[0] += 1
                sm(a, b)
            wall_r, ev_r = time_launches(rotating_softmax, args.warmup, steps2, torch, gern_amd)
            workloads["softmax_8192x4096_rotating_buffers"] = {"GB/s": 2 * x.nbytes / (ev_r * 1e-3) / 1e9, "ms": ev_r,
                                                               "frac_hbm": 2 * x.nbytes / (ev_r * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                                               "buffer_pairs": len(ring)}
            log("softmax 8192x4096 over %d rotating buffer pairs: %.1f us  %.0f GB/s" % (len(ring), ev_r * 1e3, 2 * x.nbytes / (ev_r * 1e-3) / 1e9))
            del ring
        del d_x, d_y

    # ---- config 4: GEMM 4096^3 ---------------------------------------------
    for variant, peak in (("f32", FP32_VECTOR_PEAK_TFLOPS), ("bf16", MFMA_BF16_PEAK_TFLOPS)):
        if not want("gemm_" + variant):
            continue
        n = 4096
        A = inputs.uniform((n, n), 4, -1.0, 1.0)
        B = inputs.uniform((n, n), 5, -1.0, 1.0)
        if variant == "bf16":
            dA = torch.from_numpy(inputs.to_bf16_bits(A).view(np.int16)).cuda()
            dB = torch.from_numpy(inputs.to_bf16_bits(B).view(np.int16)).cuda()
        else:
            dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        dC = torch.zeros((n, n), device="cuda")
        g = gern_amd.Gemm(variant, overwrite=True)  # config 4 is C = A * B
        wall, ev = time_launches(lambda: g(dA, dB, dC), 3, max(5, args.steps // 20), torch, gern_amd)
        tf = 2.0 * n ** 3 / (ev * 1e-3) / 1e12
        workloads["gemm_%s_4096" % variant] = {"TFLOP/s": tf, "ms": ev, "frac_peak": tf / peak, "peak_TFLOP/s": peak,
                                               "kernel": g.kernel_name}
        log("gemm %s 4096^3: %.1f us  %.1f TFLOP/s (%.1f%% of %.0f)" % (variant, ev * 1e3, tf, 100 * tf / peak, peak))
        if variant == "f32":
            # the same product on the kernel that takes every shape (vector-ALU FMAs)
            g = gern_amd.Gemm(variant, overwrite=True, general_only=True)
            wall, ev = time_launches(lambda: g(dA, dB, dC), 3, max(5, args.steps // 20), torch, gern_amd)
            tf = 2.0 * n ** 3 / (ev * 1e-3) / 1e12
            workloads["gemm_f32_4096_vector_alu"] = {"TFLOP/s": tf, "ms": ev, "frac_peak": tf / peak, "peak_TFLOP/s": peak,
                                                     "kernel": g.kernel_name}
            log("gemm f32 4096^3, vector-ALU kernel: %.1f us  %.1f TFLOP/s (%.1f%% of %.0f)" % (ev * 1e3, tf, 100 * tf / peak, peak))
        del dA, dB, dC

    # ---- config 5: fused QK^T -> softmax ------------------------------------
    if want("qk_softmax"):
        m = nk = 4096
        d = 128
        Q = inputs.to_bf16_bits(inputs.normal((m, d), 5))
        K = inputs.to_bf16_bits(inputs.normal((nk, d), 6))
        dQ = torch.from_numpy(Q.view(np.int16)).cuda()
        dK = torch.from_numpy(K.view(np.int16)).cuda()
        dS = torch.zeros((m, nk), device="cuda")
        qk = gern_amd.QKSoftmax(d, nk)
        scale = 1.0 / np.sqrt(float(d))
        wall, ev = time_launches(lambda: qk(dQ, dK, dS, scale), args.warmup, steps2, torch, gern_amd)
        nbytes = Q.nbytes + K.nbytes + m * nk * 4
        gbs = nbytes / (ev * 1e-3) / 1e9
        tf = 2.0 * m * nk * d / (ev * 1e-3) / 1e12
        workloads["qk_softmax_4096x4096x128"] = {"GB/s": gbs, "ms": ev, "frac_hbm": gbs / HBM_PEAK_GBS, "TFLOP/s": tf,
                                                 "frac_mfma": tf / MFMA_BF16_PEAK_TFLOPS, "kernel": qk.kernel_name}
        log("qk softmax 4096x4096x128: %.1f us  %.0f GB/s (%.1f%% HBM)  %.1f TFLOP/s" % (ev * 1e3, gbs, 100 * gbs / HBM_PEAK_GBS, tf))

    # ---- calibration: plain copy of known size ------------------------------
    if want("copy"):
        workloads["copy_256MiB"] = copy_calibration(torch, gern_amd, args.warmup, steps2)
        log("copy 256 MiB: %.1f us  %.0f GB/s" % (workloads["copy_256MiB"]["ms"] * 1e3, workloads["copy_256MiB"]["GB/s"]))
        workloads["copy_256MiB_streaming_stores"] = copy_calibration(torch, gern_amd, args.warmup, steps2,
                                                                     "gern_copy_f4_streaming")
        log("copy 256 MiB, streaming stores: %.1f us  %.0f GB/s" % (workloads["copy_256MiB_streaming_stores"]["ms"] * 1e3,
                                                                   workloads["copy_256MiB_streaming_stores"]["GB/s"]))
        if not args.no_rotating:
            # 1 GiB: far beyond the 256 MiB memory-side cache, i.e. what HBM itself streams
            workloads["copy_1GiB_streaming_stores"] = copy_calibration(torch, gern_amd, args.warmup, max(10, steps2 // 2),
                                                                       "gern_copy_f4_streaming", 1 << 30)
            log("copy 1 GiB, streaming stores: %.1f us  %.0f GB/s" % (workloads["copy_1GiB_streaming_stores"]["ms"] * 1e3,
                                                                     workloads["copy_1GiB_streaming_stores"]["GB/s"]))

    if result is None:
        result = {"metric": "partial run (--only %s)" % args.only, "value": None, "unit": "", "n_gpus": 1,
                  "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True,
                  "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": args.only}}
    result["workloads"] = workloads
    result["device"] = {"arch": lim.arch.decode(), "compute_units": lim.compute_units, "clock_khz": lim.clock_khz}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
