#!/usr/bin/env python3
"""Benchmark of the fused-kernel hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-rotating] [--only NAME]

A step is one launch of the fused three-stage blur chain (x, y, x; 3 taps of
weight 1/3) on an 8192 x 8192 fp32 image that is already resident in HBM; the
headline value is its whole-job throughput in GB/s of ALGORITHMIC bytes
(logical input read once + logical output written once), timed over ROTATING
buffer pairs: the image is 256 MiB, the size of this GPU's memory-side cache,
so launches on one and the same buffer pair are served in part by that cache
(reported beside it as roofline.achieved_same_buffers, not as the value).

The same line carries every other configuration of the metric under
"workloads" (two-stage blur 1024^2, row softmax, GEMM fp32 / bf16, fused QK^T
softmax, the user-level GEMM schedules at 1024^3).  Each entry holds the mean
launch time over the timed steps, the median and minimum over at least 20
launches timed one by one (HIP events on the launching stream), and its own
"roofline" object: algorithmic bytes or flops per launch, the peak it is
priced against, the fraction reached, and the HBM bytes per launch read from
profiles/hbm_traffic.md -- used only when the kernel identity recorded there
(a hash of the generated source and of the gernel headers) is the one that
ran here; otherwise "traffic" is null and "traffic_note" says why.

"cpu_baseline" is the reference library's own CPU lowering of the same
composed pipeline (oracle/_ref/, when it was built) or the CPU oracle, timed
on one host core.

Prints exactly one JSON line on stdout.
"""
import argparse
import glob
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 MFMA
FP32_PEAK_TFLOPS = 157.3       # fp32, matrix or packed vector
MIN_SINGLE_LAUNCHES = 20
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic.md")


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


DEVICE_WARMUP_S = 0.06


def device_warmup(fn, torch):
    """Untimed launches of the workload's own kernel for about 60 ms.  After idling (half a second
    is enough) this GPU runs its first launches 10-25 % slower and takes some 25 ms of load to settle:
    measured on the bf16 GEMM, 131-150 us per launch at first, 117 us from the 200th launch on."""
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < DEVICE_WARMUP_S or n == 0:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        n += 20
    return n


def measure(fn, warmup, steps, torch, gern_amd):
    """Device warm-up, `warmup` more untimed launches, the mean over exactly `steps` back-to-back
    launches, then median and minimum over single launches."""
    device_warmup(fn, torch)
    wall, ev = time_launches(fn, warmup, steps, torch, gern_amd)
    n = max(MIN_SINGLE_LAUNCHES, min(steps, 50))
    each = per_launch_ms(fn, n, torch, gern_amd)
    return {"ms": ev, "wall_ms": wall, "steps": steps, "ms_median": each[len(each) // 2], "ms_min": each[0], "single_launches": n}


_HEADER_HASH = []


def kernel_id(source):
    """Identity of a generated kernel: its source (the code generator numbers functions and variables
    per process, so trailing numbers of identifiers are masked) and every gernel header it may include."""
    if not _HEADER_HASH:
        h = hashlib.sha1()
        for path in sorted(glob.glob(os.path.join(ROOT, "gern_amd", "gernels", "*.h"))):
            with open(path, "rb") as f:
                h.update(f.read())
        _HEADER_HASH.append(h.hexdigest())
    text = re.sub(r"(?:_\d+)+\b", "_N", source)
    return hashlib.sha1((text + _HEADER_HASH[0]).encode()).hexdigest()[:12]


def traffic_table():
    """Rows `| workload | kernel id | fetch bytes | write bytes |` of profiles/hbm_traffic.md."""
    rows = {}
    try:
        with open(TRAFFIC_TABLE) as f:
            for line in f:
                cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
                if len(cells) >= 4 and re.fullmatch(r"[0-9a-f]{12}", cells[1]) and cells[2].isdigit() and cells[3].isdigit():
                    rows[cells[0]] = (cells[1], int(cells[2]), int(cells[3]))
    except OSError:
        pass
    return rows


def roofline(workload, table, bound, algorithmic, timing, pipeline, source=None):
    """bound "hbm": algorithmic bytes against 8 TB/s; "mfma" / "fp32": flops against the matrix peak."""
    ms = timing["ms"]
    if bound == "hbm":
        achieved, peak, unit = algorithmic / (ms * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s"
    else:
        achieved, unit = algorithmic / (ms * 1e-3) / 1e12, "TFLOP/s"
        peak = MFMA_BF16_PEAK_TFLOPS if bound == "mfma" else FP32_PEAK_TFLOPS
    kid = kernel_id(source if source is not None else pipeline.source)
    roof = {"bound": "hbm" if bound == "hbm" else "mfma", "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
            "algorithmic": algorithmic, "algorithmic_unit": "bytes" if bound == "hbm" else "flop",
            "kernel": pipeline.kernel_name, "kernel_id": kid, "kernel_ms": ms,
            "kernel_ms_median": timing["ms_median"], "kernel_ms_min": timing["ms_min"],
            "frac_at_median": achieved * ms / timing["ms_median"] / peak}
    row = table.get(workload)
    if row is None:
        roof["traffic"] = None
        roof["traffic_note"] = "no row for this workload in profiles/hbm_traffic.md"
    elif row[0] != kid:
        roof["traffic"] = None
        roof["traffic_note"] = "the kernel changed since the counters were read (profiles/hbm_traffic.md has %s)" % row[0]
    else:
        roof["traffic"] = row[1] + row[2]
        roof["traffic_fetch"], roof["traffic_write"] = row[1], row[2]
    return roof


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


def copy_calibration(torch, gern_amd, warmup, steps, kernel="gern_copy_f4", nbytes=256 << 20, pairs=1):
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
    # pairs > 1: the launches go round that many buffer pairs, as the rotating-buffer runs of the pipelines do
    srcs = [torch.ones(nbytes // 4, device="cuda") for _ in range(pairs)]
    dsts = [torch.zeros_like(srcs[0]) for _ in range(pairs)]
    n = C.c_longlong(nbytes // 16)
    grid = (C.c_uint32 * 3)((nbytes // 16 + 255) // 256, 1, 1)
    block = (C.c_uint32 * 3)(256, 1, 1)
    args_of = []
    for src, dst in zip(srcs, dsts):
        a, b = C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr())
        args_of.append((a, b, (C.c_void_p * 3)(C.cast(C.byref(a), C.c_void_p), C.cast(C.byref(b), C.c_void_p), C.cast(C.byref(n), C.c_void_p))))
    turn = [0]

    def launch():
        params = args_of[turn[0] % pairs][2]
        turn[0] += 1
        if hip.gern_hip_launch(ker, grid, block, 0, params, None) != 0:
            raise gern_amd.GernError(gern_amd._hip_error())
    device_warmup(launch, torch)
    wall, ev = time_launches(launch, warmup, steps, torch, gern_amd)
    assert all(bool((dst == 1).all()) for dst in dsts)
    out = {"GB/s": 2 * nbytes / (ev * 1e-3) / 1e9, "ms": ev, "frac_hbm": 2 * nbytes / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "kernel": kernel, "bytes_read": nbytes, "bytes_written": nbytes}
    if pairs > 1:
        out["buffer_pairs"] = pairs
    return out


def cpu_blur(img_np, pattern, tile_rows, tile_cols, budget_s, what_size):
    """The same composed pipeline on ONE host core: the reference library's CPU lowering when it
    was built, else the CPU oracle with the same tiling."""
    from oracle import oracle as o
    from oracle import ref
    rows, cols = img_np.shape
    if ref.available():
        kind = "reference"
        run = lambda: ref.blur_chain(img_np, pattern, tile_rows, tile_cols)  # noqa: E731
        what = "reference library CPU lowering of Tile(rows=%d)(Tile(cols=%d)(%s)), g++ -O2" % (
            tile_rows, tile_cols, ", ".join("blur_" + c for c in pattern))
    else:
        kind = "port"
        run = lambda: o.blur_chain_tiled(img_np, pattern, tile_rows, tile_cols)  # noqa: E731
        what = "CPU oracle (scalar C restatement), same tiling, gcc -O2"
    out = run()  # warm-up
    times = []
    budget = time.perf_counter() + budget_s
    while len(times) < 5 and (len(times) < 1 or time.perf_counter() < budget):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    nbytes = img_np.nbytes + out.nbytes
    return out, {
        "value": nbytes / med / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "host_cores": os.cpu_count(),
        "kind": kind,
        "seconds": med,
        "sample": "full workload (%s), median of %d runs after one warm-up; %s" % (what_size, len(times), what),
    }


def cpu_time(run, budget_s, nbytes=None, flop=None, what=""):
    """Median of up to five runs (after one warm-up) of a CPU pipeline on ONE host core."""
    run()
    times = []
    budget = time.perf_counter() + budget_s
    while len(times) < 5 and (len(times) < 1 or time.perf_counter() < budget):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    out = {"cores": 1, "host_cores": os.cpu_count(), "seconds": med, "sample": "%s; median of %d runs after one warm-up" % (what, len(times))}
    if nbytes is not None:
        out.update({"value": nbytes / med / 1e9, "unit": "GB/s"})
    if flop is not None:
        out.update({"value": flop / med / 1e9, "unit": "GFLOP/s"})
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-rotating", action="store_true",
                    help="skip the extra timings over rotating buffers (profiles: keeps one kind of launch per kernel)")
    ap.add_argument("--rotating-only", action="store_true",
                    help="blur and softmax: time ONLY the launches over rotating buffers (counter runs of that regime)")
    ap.add_argument("--only", default="", help="run only these workloads, comma-separated (blur, blur_xy_1024, softmax, gemm_f32, gemm_bf16, "
                                               "qk_softmax, gemm_schedules, copy)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import numpy as np
    import torch

    import __graft_entry__
    __graft_entry__.ensure_built()
    import gern_amd
    from gern_amd import inputs

    if gern_amd.device_count() < 1 or not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: there is no CPU fallback")
    lim = gern_amd.device_limits()
    log("device:", lim.arch.decode(), "CUs:", lim.compute_units)

    only = [w for w in args.only.split(",") if w]
    want = lambda name: (not only) or name in only  # noqa: E731
    table = traffic_table()
    workloads = {}
    result = None
    # every workload is timed over at least MIN_SINGLE_LAUNCHES launches, whatever --steps says
    steps2 = max(MIN_SINGLE_LAUNCHES, args.steps)  # launches of 0.4 ms and less: as many as the headline
    steps_gemm = max(MIN_SINGLE_LAUNCHES, args.steps // 10)

    def rotating(pairs, launch):
        turn = [0]

        def fn():
            a, b = pairs[turn[0] % len(pairs)]
            turn[0] += 1
            launch(a, b)
        return fn

    # ---- config 2: three-stage blur, 8192 x 8192 (the headline) ------------
    if want("blur"):
        rows = cols = 8192
        img = inputs.uniform((rows, cols), 2)
        d_in = torch.from_numpy(img).cuda()
        blur = gern_amd.BlurChain("xyx", tile_rows=4)  # 4 x 224 tiles, line-aligned store windows
        d_out = torch.zeros(blur.out_shape(rows, cols), device="cuda")
        nbytes = img.nbytes + d_out.numel() * 4
        if not args.rotating_only:
            t = measure(lambda: blur(d_in, d_out), args.warmup, args.steps, torch, gern_amd)
            roof = roofline("blur_xyx_8192", table, "hbm", nbytes, t, blur)
            workloads["blur_xyx_8192"] = {"GB/s": roof["achieved"], "ms": t["ms"], "frac_hbm": roof["frac"], "roofline": roof,
                                          "note": "same buffer pair every launch: cache-assisted"}
            log("blur xyx 8192^2, same buffers: %.1f us/launch  %.0f GB/s  (%.1f%% of HBM peak)" % (t["ms"] * 1e3, roof["achieved"], 100 * roof["frac"]))
        if not args.no_rotating:
            # The same launch over ROTATING buffer pairs: the 256 MiB image is exactly the size of the
            # memory-side cache, and with streaming stores a launch finds part of its input there when
            # the previous launch read the same buffer.  Rotating over four pairs takes that away.
            ring = [(d_in, d_out)] + [(d_in.clone(), torch.zeros_like(d_out)) for _ in range(3)]
            tr = measure(rotating(ring, lambda a, b: blur(a, b)), args.warmup, args.steps, torch, gern_amd)
            rroof = roofline("blur_xyx_8192_rotating_buffers", table, "hbm", nbytes, tr, blur)
            workloads["blur_xyx_8192_rotating_buffers"] = {"GB/s": rroof["achieved"], "ms": tr["ms"], "frac_hbm": rroof["frac"],
                                                           "buffer_pairs": len(ring), "roofline": rroof}
            log("blur xyx 8192^2 over %d rotating buffer pairs: %.1f us/launch  %.0f GB/s" % (len(ring), tr["ms"] * 1e3, rroof["achieved"]))
            del ring
        # The headline is the HBM regime: rotating buffers (the reference's own image, 15360^2 = 944 MB,
        # apps/blur/blur.cu:10, is far beyond any cache, so its same-buffer loop measured memory too).
        # --no-rotating / --rotating-only runs (counter and trace runs of one regime) report the regime they timed.
        head, head_t, protocol = None, None, ""
        if not args.no_rotating:
            head, head_t = rroof, tr
            protocol = ("about 60 ms of untimed launches (the GPU settles), `warmup` more untimed launches, then `steps` timed "
                        "launches over four rotating buffer pairs (1 GiB of images and 1 GiB of results: nothing of a launch's "
                        "input is left in the 256 MiB memory-side cache by the previous one)")
            if not args.rotating_only:
                # the reference's own protocol (apps/blur/blur.cu:79-96: N launches on the SAME buffers): cache-assisted here
                head = dict(rroof)
                head["achieved_same_buffers"] = roof["achieved"]
                head["frac_same_buffers"] = roof["frac"]
                head["kernel_ms_same_buffers"] = roof["kernel_ms"]
                head["traffic_same_buffers"] = roof["traffic"]
                head["same_buffers_note"] = "launches on one buffer pair find part of the 256 MiB image in the memory-side cache"
        elif not args.rotating_only:
            head, head_t = roof, t
            protocol = "--no-rotating: `steps` timed launches on the SAME buffer pair (cache-assisted: not the HBM regime)"
        if head is not None:
            gbs = nbytes / (head_t["wall_ms"] * 1e-3) / 1e9
            result = {
                "metric": "fused 3-stage blur (x,y,x) 8192x8192 fp32, algorithmic GB/s",
                "value": gbs,
                "unit": "GB/s",
                "n_gpus": 1,
                "steps": args.steps,
                "warmup": args.warmup,
                "ms_per_step": head_t["wall_ms"],
                "higher_is_better": True,
                "scaling": "weak",
                "vs_baseline": None,  # the reference publishes no number for this metric
                "dtype": "f32",
                "data": "synthetic",
                "config": {"workload": "three-stage fused separable blur chain (3-tap x, y, x; weights 1/3), 8192x8192 fp32 "
                                       "uniform[0,1) seed 2, valid-region output 8190x8188, one launch per step",
                           "schedule": "one wavefront per 4x224 output tile, store windows moved to whole 128-byte lines, "
                                       "XCD-aware workgroup order",
                           "protocol": protocol},
                "roofline": head,
            }
            if not args.no_cpu and not args.rotating_only:
                # tile sizes must divide the 8190 x 8188 output (the reference handles no ragged tiles)
                _, result["cpu_baseline"] = cpu_blur(img, "xyx", 90, 356, 20.0, "8192x8192 three-stage blur")
                log("cpu baseline: %.2f GB/s on 1 core (%s)" % (result["cpu_baseline"]["value"], result["cpu_baseline"]["kind"]))
        del d_in, d_out

    # ---- config 1: two-stage blur, 1024 x 1024 (the reference's CPU-runnable case) ----
    if want("blur_xy_1024") and not args.rotating_only:
        img = inputs.uniform((1024, 1024), 1)
        d_in = torch.from_numpy(img).cuda()
        blur = gern_amd.BlurChain("xy")
        d_out = torch.zeros(blur.out_shape(1024, 1024), device="cuda")
        nbytes = img.nbytes + d_out.numel() * 4
        t = measure(lambda: blur(d_in, d_out), args.warmup, steps2, torch, gern_amd)
        roof = roofline("blur_xy_1024", table, "hbm", nbytes, t, blur)
        workloads["blur_xy_1024"] = {"GB/s": roof["achieved"], "ms": t["ms"], "frac_hbm": roof["frac"], "roofline": roof,
                                     "note": "8 MB of traffic: launch latency, not HBM, bounds a launch this small"}
        log("blur xy 1024^2: %.1f us  %.0f GB/s" % (t["ms"] * 1e3, roof["achieved"]))
        if not args.no_cpu:
            # 1022 x 1022 output = (14 x 73) x (7 x 146) tiles
            want_out, cpu = cpu_blur(img, "xy", 73, 146, 5.0, "1024x1024 two-stage blur")
            torch.cuda.synchronize()
            cpu["gpu_result_identical"] = bool(np.array_equal(d_out.cpu().numpy(), want_out))
            workloads["blur_xy_1024_cpu"] = cpu
            log("blur xy 1024^2 on the CPU: %.2f GB/s on 1 core (%s), GPU result identical: %s" % (cpu["value"], cpu["kind"], cpu["gpu_result_identical"]))
        del d_in, d_out

    # ---- config 3: row softmax, 8192 x 4096 --------------------------------
    if want("softmax"):
        x = inputs.normal((8192, 4096), 3, 0.0, 2.0)
        d_x = torch.from_numpy(x).cuda()
        d_y = torch.zeros_like(d_x)
        sm = gern_amd.Softmax(4096)
        if not args.rotating_only:
            t = measure(lambda: sm(d_x, d_y), args.warmup, steps2, torch, gern_amd)
            roof = roofline("softmax_8192x4096", table, "hbm", 2 * x.nbytes, t, sm)
            workloads["softmax_8192x4096"] = {"GB/s": roof["achieved"], "ms": t["ms"], "frac_hbm": roof["frac"], "roofline": roof}
            log("softmax 8192x4096: %.1f us  %.0f GB/s (%.1f%%)" % (t["ms"] * 1e3, roof["achieved"], 100 * roof["frac"]))
        if not args.no_cpu and not args.rotating_only:
            from oracle import oracle as o
            from oracle import ref
            sample = x[:1024]  # 1024 of the 8192 rows: a bounded sample of the same workload
            if ref.available():
                cpu = cpu_time(lambda: ref.softmax_rows(sample), 5.0, nbytes=2 * sample.nbytes,
                               what="1024 rows of the 8192x4096 softmax, reference library CPU lowering of the fused five-gernel pipeline, g++ -O2")
                cpu["kind"] = "reference"
            else:
                cpu = cpu_time(lambda: o.softmax_rows(sample), 5.0, nbytes=2 * sample.nbytes,
                               what="1024 rows of the 8192x4096 softmax, CPU oracle, gcc -O2")
                cpu["kind"] = "port"
            workloads["softmax_8192x4096_cpu"] = cpu
            log("softmax on the CPU (1024 rows): %.2f GB/s on 1 core (%s)" % (cpu["value"], cpu["kind"]))
        if not args.no_rotating:
            ring = [(d_x, d_y)] + [(d_x.clone(), torch.zeros_like(d_y)) for _ in range(5)]
            tr = measure(rotating(ring, lambda a, b: sm(a, b)), args.warmup, steps2, torch, gern_amd)
            rroof = roofline("softmax_8192x4096_rotating_buffers", table, "hbm", 2 * x.nbytes, tr, sm)
            workloads["softmax_8192x4096_rotating_buffers"] = {"GB/s": rroof["achieved"], "ms": tr["ms"], "frac_hbm": rroof["frac"],
                                                               "buffer_pairs": len(ring), "roofline": rroof}
            log("softmax 8192x4096 over %d rotating buffer pairs: %.1f us  %.0f GB/s" % (len(ring), tr["ms"] * 1e3, rroof["achieved"]))
            del ring
        del d_x, d_y

    # ---- config 4: GEMM 4096^3 ---------------------------------------------
    for variant, bound in (("f32", "fp32"), ("bf16", "mfma")):
        if not want("gemm_" + variant) or args.rotating_only:
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
        # a 0.1 ms launch is timed over `steps` launches (20 ms), a 1 ms launch over a tenth of them
        steps_here = steps_gemm if variant == "f32" else max(steps_gemm, args.steps)
        t = measure(lambda: g(dA, dB, dC), 5, steps_here, torch, gern_amd)
        vendor = {}
        # The vendor library on the same operands, for comparison (not part of the product).  bf16: torch.mm with
        # fp32 output is the same contract (bf16 in, fp32 accumulate, fp32 C); with bf16 output the library writes
        # half the bytes.  fp32: torch.mm (TF32 is off by default).  This build's kernel and the library's are
        # timed in turn, twice, each time with the same warm-up, and every kernel keeps its better turn: on a GPU
        # whose clock follows its power draw and temperature, whichever runs second would otherwise pay for the first.
        if variant == "bf16":
            tA, tB = dA.view(torch.bfloat16), dB.view(torch.bfloat16)
            out_bf16 = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
            calls = {"gemm_bf16_4096_vendor": lambda: torch.mm(tA, tB, out_dtype=torch.float32, out=dC),
                     "gemm_bf16_4096_vendor_bf16_out": lambda: torch.mm(tA, tB, out=out_bf16)}
        else:
            calls = {"gemm_f32_4096_vendor": lambda: torch.mm(dA, dB, out=dC)}
        peak = MFMA_BF16_PEAK_TFLOPS if variant == "bf16" else FP32_PEAK_TFLOPS
        turns = {"ours": [t]}
        for turn in range(2):
            for name, call in calls.items():
                try:
                    turns.setdefault(name, []).append(measure(call, 5, steps_here, torch, gern_amd))
                except Exception as e:  # a torch without out_dtype: say so, do not fail the benchmark
                    vendor[name] = {"error": str(e)[:200]}
            if turn == 0:
                turns["ours"].append(measure(lambda: g(dA, dB, dC), 5, steps_here, torch, gern_amd))
        t = min(turns["ours"], key=lambda x: x["ms"])
        for name in calls:
            if name in turns:
                tv = min(turns[name], key=lambda x: x["ms"])
                tfv = 2.0 * n ** 3 / (tv["ms"] * 1e-3) / 1e12
                vendor[name] = {"TFLOP/s": tfv, "ms": tv["ms"], "ms_median": tv["ms_median"], "ms_min": tv["ms_min"],
                                "ms_turns": [x["ms"] for x in turns[name]],
                                "frac_peak": tfv / peak, "peak_TFLOP/s": peak,
                                "what": "torch.mm (hipBLASLt), %s operands, %s output; comparison only"
                                        % (variant if variant == "bf16" else "fp32", "bf16" if name.endswith("bf16_out") else "fp32")}
        roof = roofline("gemm_%s_4096" % variant, table, bound, 2.0 * n ** 3, t, g)
        workloads["gemm_%s_4096" % variant] = {"TFLOP/s": roof["achieved"], "ms": t["ms"], "frac_peak": roof["frac"],
                                               "peak_TFLOP/s": roof["peak"], "roofline": roof}
        log("gemm %s 4096^3: %.1f us  %.1f TFLOP/s (%.1f%% of %.0f)" % (variant, t["ms"] * 1e3, roof["achieved"], 100 * roof["frac"], roof["peak"]))
        workloads["gemm_%s_4096" % variant]["ms_turns"] = [x["ms"] for x in turns["ours"]]
        workloads.update(vendor)
        for name, v in vendor.items():
            if "ms" in v:
                log("%s: %.1f us  %.1f TFLOP/s (turns: %s)" % (name, v["ms"] * 1e3, v["TFLOP/s"], ", ".join("%.1f" % (x * 1e3) for x in v["ms_turns"])))
        if variant == "f32" and not args.no_cpu:
            from oracle import oracle as o
            from oracle import ref
            As, Bs = A[:512, :512].copy(), B[:512, :512].copy()  # a 512^3 corner of the product: 1/512 of the flops
            if ref.available():
                cpu = cpu_time(lambda: ref.gemm(As, Bs, 64, 64, 64), 8.0, flop=2.0 * 512 ** 3,
                               what="512^3 corner of the 4096^3 fp32 product, reference library CPU lowering of Tile(64)(Tile(64)(Reduce(64)(matrix_multiply))), g++ -O2")
                cpu["kind"] = "reference"
            else:
                cpu = cpu_time(lambda: o.gemm_f32(As, Bs), 8.0, flop=2.0 * 512 ** 3, what="512^3 corner of the 4096^3 fp32 product, CPU oracle, gcc -O2")
                cpu["kind"] = "port"
            workloads["gemm_f32_512_cpu"] = cpu
            log("gemm f32 512^3 on the CPU: %.2f GFLOP/s on 1 core (%s)" % (cpu["value"], cpu["kind"]))
        if variant == "f32":
            # the same product on the kernel that takes every shape (vector-ALU FMAs)
            g = gern_amd.Gemm(variant, overwrite=True, general_only=True)
            t = measure(lambda: g(dA, dB, dC), 3, steps_gemm, torch, gern_amd)
            roof = roofline("gemm_f32_4096_vector_alu", table, bound, 2.0 * n ** 3, t, g)
            workloads["gemm_f32_4096_vector_alu"] = {"TFLOP/s": roof["achieved"], "ms": t["ms"], "frac_peak": roof["frac"],
                                                     "peak_TFLOP/s": roof["peak"], "roofline": roof}
            log("gemm f32 4096^3, vector-ALU kernel: %.1f us  %.1f TFLOP/s (%.1f%% of %.0f)" % (
                t["ms"] * 1e3, roof["achieved"], 100 * roof["frac"], roof["peak"]))
        del dA, dB, dC

    # ---- config 5: fused QK^T -> softmax ------------------------------------
    if want("qk_softmax") and not args.rotating_only:
        m = nk = 4096
        d = 128
        Q = inputs.to_bf16_bits(inputs.normal((m, d), 5))
        K = inputs.to_bf16_bits(inputs.normal((nk, d), 6))
        dQ = torch.from_numpy(Q.view(np.int16)).cuda()
        dK = torch.from_numpy(K.view(np.int16)).cuda()
        dS = torch.zeros((m, nk), device="cuda")
        qk = gern_amd.QKSoftmax(d, nk)
        scale = 1.0 / np.sqrt(float(d))
        t = measure(lambda: qk(dQ, dK, dS, scale), args.warmup, steps2, torch, gern_amd)
        nbytes = Q.nbytes + K.nbytes + m * nk * 4
        roof = roofline("qk_softmax_4096x4096x128", table, "hbm", nbytes, t, qk)
        tf = 2.0 * m * nk * d / (t["ms"] * 1e-3) / 1e12
        workloads["qk_softmax_4096x4096x128"] = {"GB/s": roof["achieved"], "ms": t["ms"], "frac_hbm": roof["frac"], "TFLOP/s": tf,
                                                 "frac_mfma": tf / MFMA_BF16_PEAK_TFLOPS, "roofline": roof}
        log("qk softmax 4096x4096x128: %.1f us  %.0f GB/s (%.1f%% HBM)  %.1f TFLOP/s" % (t["ms"] * 1e3, roof["achieved"], 100 * roof["frac"], tf))
        del dQ, dK, dS

    # ---- schedules written at the level of Gern's API, 1024^3 (the reference times such a
    # kernel in gernels/mm/bench.cu:72-89) ---------------------------------------------------
    if want("gemm_schedules") and not args.rotating_only:
        n = gern_amd.GemmSchedule.SIZE
        dA = torch.from_numpy(inputs.uniform((n, n), 4, -1.0, 1.0)).cuda()
        dB = torch.from_numpy(inputs.uniform((n, n), 5, -1.0, 1.0)).cuda()
        dC = torch.zeros((n, n), device="cuda")
        for schedule, what in ((3, "kernel_3.cu as the reference composes it: 64x64 block tiles staged through LDS one float per lane, "
                                   "4x4 outputs per thread multiplied into C in global memory"),
                               (6, "kernel_6.cu's composition plus a register stage of C: 64x64 block tiles, K tiles of 64 staged "
                                   "16 bytes per lane, 4x4 outputs per thread in registers"),
                               (10, "kernel_10.cu's block -> wavefront -> lane tiling with the lanes of a wavefront on consecutive "
                                    "columns, loads that write LDS directly, one output per lane")):
            g = gern_amd.GemmSchedule(schedule)
            t = measure(lambda: g(dA, dB, dC), 3, MIN_SINGLE_LAUNCHES, torch, gern_amd)
            roof = roofline("gemm_schedule_kernel_%d_1024" % schedule, table, "fp32", 2.0 * n ** 3, t, g)
            workloads["gemm_schedule_kernel_%d_1024" % schedule] = {"TFLOP/s": roof["achieved"], "ms": t["ms"], "frac_peak": roof["frac"],
                                                                    "schedule": what, "roofline": roof}
            log("gemm schedule kernel_%d 1024^3: %.1f us  %.2f TFLOP/s" % (schedule, t["ms"] * 1e3, roof["achieved"]))
        del dA, dB, dC

    # ---- calibration: plain copy of known size ------------------------------
    if want("copy") and not args.rotating_only:
        workloads["copy_256MiB"] = copy_calibration(torch, gern_amd, args.warmup, steps2)
        log("copy 256 MiB: %.1f us  %.0f GB/s" % (workloads["copy_256MiB"]["ms"] * 1e3, workloads["copy_256MiB"]["GB/s"]))
        workloads["copy_256MiB_streaming_stores"] = copy_calibration(torch, gern_amd, args.warmup, steps2,
                                                                     "gern_copy_f4_streaming")
        log("copy 256 MiB, streaming stores: %.1f us  %.0f GB/s" % (workloads["copy_256MiB_streaming_stores"]["ms"] * 1e3,
                                                                   workloads["copy_256MiB_streaming_stores"]["GB/s"]))
        if not args.no_rotating:
            # the blur's bytes in the blur's regime: 256 MiB in, 256 MiB out, round four buffer pairs
            workloads["copy_256MiB_streaming_stores_rotating_buffers"] = copy_calibration(
                torch, gern_amd, args.warmup, steps2, "gern_copy_f4_streaming", pairs=4)
            log("copy 256 MiB, streaming stores, over 4 rotating buffer pairs: %.1f us  %.0f GB/s" % (
                workloads["copy_256MiB_streaming_stores_rotating_buffers"]["ms"] * 1e3,
                workloads["copy_256MiB_streaming_stores_rotating_buffers"]["GB/s"]))
            # 1 GiB: far beyond the 256 MiB memory-side cache, i.e. what HBM itself streams
            workloads["copy_1GiB_streaming_stores"] = copy_calibration(torch, gern_amd, args.warmup, max(10, steps2 // 2),
                                                                       "gern_copy_f4_streaming", 1 << 30)
            log("copy 1 GiB, streaming stores: %.1f us  %.0f GB/s" % (workloads["copy_1GiB_streaming_stores"]["ms"] * 1e3,
                                                                     workloads["copy_1GiB_streaming_stores"]["GB/s"]))

    if result is None:
        result = {"metric": "partial run (--only %s%s)" % (args.only, " --rotating-only" if args.rotating_only else ""),
                  "value": None, "unit": "", "n_gpus": 1,
                  "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True,
                  "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": args.only}}
    result["workloads"] = workloads
    result["device"] = {"arch": lim.arch.decode(), "compute_units": lim.compute_units, "clock_khz": lim.clock_khz}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
