#!/usr/bin/env python3
"""In-kernel clocks of the matrix-core pipelines, and the machine rates they are
judged against, on ONE MI355X.

    python -m gern_amd.microbench [gemm_bf16_phases] [gemm_bf16_split] [gemm_bf16_operands] [vendor_gemm] [qk_phases] [mfma_rate] [write_rate]

gemm_bf16_phases  the bf16 GEMM 4096^3 kernel as the code generator emits it
                  (same gernel calls, gernels/mm.h), with the 100 MHz
                  wall clock and the shader clock read by every workgroup
                  before the K loop, after it, after its stores are issued and
                  after they are acknowledged
gemm_bf16_split   the bf16 GEMM 4096^3 and 8192^3 pipeline built three ways and timed
                  in turn in one process: as it is, moving the data only (no LDS
                  reads, no MFMAs), and computing only (every stage on what the
                  first two loaded)
gemm_bf16_operands  the bf16 GEMM 4096^3 pipeline and torch.matmul on random, all-zero
                  and all-one matrices, in turn: how much of the launch time is the
                  clock the GPU grants for the data it is given
vendor_gemm       torch.matmul (the vendor's GEMM library) on the same shapes,
                  bf16 and fp32: what tuned code of the vendor reaches on this GPU
qk_phases         the same for the QK^T softmax tile kernel (gernels/qk_tiles.h)
mfma_rate         a loop of nothing but v_mfma_f32_32x32x16_bf16 with changing
                  operands on every SIMD for about a millisecond: the sustained
                  matrix rate and clock of this GPU
write_rate        a kernel that only writes 64 MiB (16-byte streaming stores, and
                  16-byte stores written through to memory as the gernels use them):
                  the floor of any kernel that writes a 4096 x 4096 fp32 result

Prints a table per probe on stdout.  These are measurements of the library's
own kernels through the C ABI; nothing here is on the product path.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


class Mat(C.Structure):
    _fields_ = [("data", C.c_void_p), ("row", C.c_int64), ("col", C.c_int64), ("lda", C.c_int64)]


class Exchange(C.Structure):
    _fields_ = [("entries", C.c_void_p), ("state", C.c_void_p), ("pitch", C.c_int32), ("spin_limit", C.c_int32),
                ("capacity", C.c_int64)]


STAMP = r"""
// slot k of this workgroup: wall clock (100 MHz) and shader clock
#define STAMP(k)                                                                               \
    do {                                                                                       \
        if (threadIdx.x == 0) {                                                                \
            unsigned long long *at = stamps + ((blockIdx.y * gridDim.x + blockIdx.x) * 8 + (k)) * 2; \
            at[0] = __builtin_amdgcn_s_memrealtime();                                          \
            at[1] = __builtin_readcyclecounter();                                              \
        }                                                                                      \
    } while (0)
"""

GEMM_SRC = r"""
#include "gernels/mm.h"
""" + STAMP + r"""
// The kernel the code generator emits for Tile(i)(Tile(j)(Reduce(k)(matrix_multiply))) on the
// whole-tile bf16 data structures, with clock reads between its statements.
__global__ void __launch_bounds__(512) gemm_bf16_phases(gernels::MatrixBF16 A, gernels::MatrixBF16 B, gernels::MatrixF32 C,
                                                        int64_t k_dim, unsigned long long *stamps) {
    STAMP(0);
    const int64_t i = (int64_t)blockIdx.y * 256, j = (int64_t)blockIdx.x * 256;
    auto acc = C.template load_acc_mfma8<256, 256>(i, j);
    for (int64_t k = 0; k < k_dim; k += 4096) {
        auto a = A.template view_exact<256, 4096>(i, k);
        auto b = B.template view_exact<4096, 256>(k, j);
        gernels::matrix_multiply(a, b, acc);
    }
    STAMP(1);
    C.store_acc(i, j, acc);
    STAMP(2);
    __builtin_amdgcn_s_waitcnt(0x0070);
    STAMP(3);
}
"""

QK_SRC = r"""
#include "gernels/qk_softmax.h"
#include "gernels/qk_tiles.h"
""" + STAMP + r"""
// The kernel the code generator emits for the tile program of gern_qk_softmax_create,
// with clock reads between its statements.
__global__ void __launch_bounds__(512) qk_phases(gernels::MatrixBF16 K, gernels::MatrixBF16 Q, gernels::MatrixF32 S,
                                                 gernels::RowStatsExchange exchange, float scale, unsigned long long *stamps) {
    STAMP(0);
    const int64_t x = (int64_t)blockIdx.y * 256, y = (int64_t)blockIdx.x * 256;
    auto session = exchange.open();
    auto out = S.template view_score_tile<256, 256>(x, y);
    auto logits = gernels::allocate_score_tile<256, 256>();
    auto q = Q.template view<256, 128>(x, 0);
    auto k = K.template view<256, 128>(y, 0);
    gernels::qk_scaled(q, k, logits, scale);
    STAMP(1);
    gernels::softmax_rows_across_tiles(logits, session, out);
    STAMP(2);
    S.store_score_tile(x, y, out);  // nothing left to do: the rows went out through the view
    __builtin_amdgcn_s_waitcnt(0x0070);
    STAMP(3);
}
"""

RATE_SRC = r"""
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
// Eight wavefronts per workgroup (two per SIMD), each 128 accumulators as in the GEMM gernel; consecutive
// instructions take different operand registers.  spread = 0 makes every operand zero.
extern "C" __global__ void __launch_bounds__(512) mfma_rate(float *sink, int iters, float spread, unsigned long long *stamps) {
    f32x16_t acc[8];
    for (int t = 0; t < 8; t++) for (int i = 0; i < 16; i++) acc[t][i] = 0.f;
    bf16x8_t a[4], b[2];
    // values spread over [-spread, spread) with all mantissa bits in use, as uniform random operands have
    for (int t = 0; t < 4; t++) for (int i = 0; i < 8; i++) a[t][i] = (__bf16)(spread * ((float)((threadIdx.x * 37 + t * 11 + i * 5) % 255) / 127.5f - 1.0f));
    for (int t = 0; t < 2; t++) for (int i = 0; i < 8; i++) b[t][i] = (__bf16)(spread * ((float)((threadIdx.x * 29 + t * 13 + i * 7) % 251) / 125.5f - 1.0f));
    unsigned long long t0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int tm = 0; tm < 4; tm++) {
#pragma unroll
            for (int tn = 0; tn < 2; tn++) {
                acc[tm * 2 + tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[tm], b[tn], acc[tm * 2 + tn], 0, 0, 0);
            }
        }
    }
    unsigned long long t1 = __builtin_amdgcn_s_memrealtime(), c1 = __builtin_readcyclecounter();
    float s = 0.f;
    for (int t = 0; t < 8; t++) for (int i = 0; i < 16; i++) s += acc[t][i];
    if (s == 12345.678f) sink[0] = s;
    if (threadIdx.x == 0) {
        stamps[blockIdx.x * 4 + 0] = t0; stamps[blockIdx.x * 4 + 1] = t1;
        stamps[blockIdx.x * 4 + 2] = c0; stamps[blockIdx.x * 4 + 3] = c1;
    }
}
extern "C" __global__ void __launch_bounds__(256) write_rate(f32x4_t *out, long long n) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const f32x4_t v = {1.f, 2.f, 3.f, 4.f};
    if (i < n) __builtin_nontemporal_store(v, out + i);
}
// the same with stores that are written through to memory (the gernels' store_result16)
extern "C" __global__ void __launch_bounds__(256) write_rate_through(float *out, long long n) {
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const u32x4_t v = {0x3f800000u, 0x40000000u, 0x40400000u, 0x40800000u};
    const __amdgpu_buffer_rsrc_t desc = __builtin_amdgcn_make_buffer_rsrc((void *)out, 0, (int)(n * 16), 0x00020000);
    if (i < n) __builtin_amdgcn_raw_buffer_store_b128(v, desc, (int)(i * 16), 0, 16);
}
"""


def _compile(gern_amd, source, names):
    hip = gern_amd.hip_lib()
    opts = [("-I" + os.path.join(ROOT, "gern_amd")).encode()]
    opts += [w.encode() for w in os.environ.get("GERN_PIPELINE_EXTRA_OPTIONS", "").split()]  # as the pipelines take them
    mod = C.c_void_p()
    c_names = (C.c_char_p * len(names))(*[n.encode() for n in names])
    c_opts = (C.c_char_p * len(opts))(*opts)
    if hip.gern_hip_compile(source.encode(), c_names, len(names), c_opts, len(opts), None, C.byref(mod)) != 0:
        raise gern_amd.GernError(gern_amd._hip_error())
    kernels = []
    for n in names:
        k = C.c_void_p()
        if hip.gern_hip_get_kernel(mod, n.encode(), C.byref(k)) != 0:
            raise gern_amd.GernError(gern_amd._hip_error())
        kernels.append(k)
    return kernels


def _launch(gern_amd, kernel, grid, block, args):
    g, b = (C.c_uint32 * 3)(*grid), (C.c_uint32 * 3)(*block)
    params = (C.c_void_p * len(args))(*[C.cast(C.pointer(a), C.c_void_p) for a in args])
    if gern_amd.hip_lib().gern_hip_launch(kernel, g, b, 0, params, None) != 0:
        raise gern_amd.GernError(gern_amd._hip_error())


def _event_us(gern_amd, torch, fn, warmup, n):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = gern_amd.Event(), gern_amd.Event()
    start.record()
    for _ in range(n):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_ms_until(stop) / n * 1e3


def _phase_table(title, stamps, names, per_launch_us):
    """stamps: (workgroups, 8, 2) of the last launch.  Times in us from the earliest start."""
    wall = stamps[:, :, 0].astype(np.float64) / 100.0
    cyc = stamps[:, :, 1].astype(np.float64)
    t0 = wall[:, 0].min()
    print("%s: %.1f us per launch (HIP events over back-to-back launches)" % (title, per_launch_us))
    print("  %-32s %8s %8s %8s" % ("clock read (us after first start)", "min", "median", "max"))
    for i, name in enumerate(names):
        col = wall[:, i] - t0
        print("  %-32s %8.2f %8.2f %8.2f" % (name, col.min(), np.median(col), col.max()))
    last = len(names) - 1
    span = wall[:, last] - wall[:, 0]
    mhz = (cyc[:, last] - cyc[:, 0]) / span
    print("  shader clock over a workgroup's run: %.0f - %.0f MHz (median %.0f)" % (mhz.min(), mhz.max(), np.median(mhz)))
    return wall, cyc


def gemm_bf16_phases(gern_amd, torch):
    from gern_amd import inputs
    n = 4096
    A = inputs.to_bf16_bits(inputs.uniform((n, n), 4, -1.0, 1.0))
    B = inputs.to_bf16_bits(inputs.uniform((n, n), 5, -1.0, 1.0))
    dA, dB = torch.from_numpy(A.view(np.int16)).cuda(), torch.from_numpy(B.view(np.int16)).cuda()
    dC = torch.zeros((n, n), device="cuda")
    stamps = torch.zeros((256, 8, 2), dtype=torch.int64, device="cuda")
    (k,) = _compile(gern_amd, GEMM_SRC, ["gemm_bf16_phases"])
    args = [Mat(dA.data_ptr(), n, n, n), Mat(dB.data_ptr(), n, n, n), Mat(dC.data_ptr(), n, n, n), C.c_int64(n),
            C.c_void_p(stamps.data_ptr())]
    pipeline = gern_amd.Gemm("bf16", overwrite=True)
    for _ in range(2):  # the second round is the one reported (clocks settle during the first)
        us_pipeline = _event_us(gern_amd, torch, lambda: pipeline(dA, dB, dC), 5, 30)
        us = _event_us(gern_amd, torch, lambda: _launch(gern_amd, k, (16, 16, 1), (512, 1, 1), args), 5, 30)
    print("the pipeline's own kernel (%s), same process, just before: %.1f us per launch" % (pipeline.kernel_name, us_pipeline))
    wall, cyc = _phase_table("bf16 GEMM 4096^3, whole-tile kernel with clock reads", stamps.cpu().numpy(),
                             ["start", "K loop done", "stores issued", "stores acknowledged"], us)
    loop_cycles = cyc[:, 1] - cyc[:, 0]
    mfma_cycles = 4096.0 * 32.0  # v_mfma_f32_32x32x16_bf16 per SIMD x 32 cycles each
    print("  K loop: %.0f - %.0f shader cycles per workgroup; the MFMAs of one SIMD are %.0f cycles: matrix pipe busy %.1f %% of the loop (median)"
          % (loop_cycles.min(), loop_cycles.max(), mfma_cycles, 100.0 * mfma_cycles / np.median(loop_cycles)))
    print("  2 * 4096^3 flop / per-launch time = %.0f TFLOP/s" % (2.0 * n ** 3 / (us * 1e-6) / 1e12))


def gemm_bf16_split(gern_amd, torch):
    from gern_amd import inputs
    for n in (4096, 8192):
        A = inputs.to_bf16_bits(inputs.uniform((n, n), 4, -1.0, 1.0))
        B = inputs.to_bf16_bits(inputs.uniform((n, n), 5, -1.0, 1.0))
        dA, dB = torch.from_numpy(A.view(np.int16)).cuda(), torch.from_numpy(B.view(np.int16)).cuda()
        dC = torch.zeros((n, n), device="cuda")
        builds = [("as it is", ""), ("data movement only", "-DGERN_MM_ONLY=1"), ("compute only", "-DGERN_MM_ONLY=2")]
        pipes = []
        before = os.environ.get("GERN_PIPELINE_EXTRA_OPTIONS")
        for _, opt in builds:
            os.environ["GERN_PIPELINE_EXTRA_OPTIONS"] = ((before or "") + " " + opt).strip()
            pipes.append(gern_amd.Gemm("bf16", overwrite=True))
        if before is None:
            del os.environ["GERN_PIPELINE_EXTRA_OPTIONS"]
        else:
            os.environ["GERN_PIPELINE_EXTRA_OPTIONS"] = before
        times = [[] for _ in builds]
        for _ in range(100):
            pipes[0](dA, dB, dC)
        for rep in range(5):
            for i, p in enumerate(pipes):
                times[i].append(_event_us(gern_amd, torch, lambda: p(dA, dB, dC), 5, 30))
        print("bf16 GEMM %d^3, whole-tile kernel, three builds timed in turn (us per launch, 5 rounds of 30 launches):" % n)
        for (name, _), t in zip(builds, times):
            print("  %-20s %s   min %.1f us = %.0f TFLOP/s-equivalent" % (name + ":", " ".join("%.1f" % x for x in t), min(t),
                                                                          2.0 * n ** 3 / (min(t) * 1e-6) / 1e12))
        del pipes


def gemm_bf16_operands(gern_amd, torch):
    from gern_amd import inputs
    n = 4096
    A = inputs.to_bf16_bits(inputs.uniform((n, n), 4, -1.0, 1.0))
    B = inputs.to_bf16_bits(inputs.uniform((n, n), 5, -1.0, 1.0))
    dA, dB = torch.from_numpy(A.view(np.int16)).cuda(), torch.from_numpy(B.view(np.int16)).cuda()
    sets = [("uniform [-1, 1)", dA, dB), ("all zero", torch.zeros_like(dA), torch.zeros_like(dB)),
            ("all one", torch.full_like(dA, 0x3F80), torch.full_like(dB, 0x3F80))]
    dC = torch.zeros((n, n), device="cuda")
    g = gern_amd.Gemm("bf16", overwrite=True)
    out = torch.empty((n, n), device="cuda", dtype=torch.bfloat16)

    def vendor_us(a, b):
        for _ in range(5):
            torch.matmul(a, b, out=out)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(60):
            torch.matmul(a, b, out=out)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 60 * 1e3

    for _ in range(300):
        g(dA, dB, dC)
    print("bf16 GEMM 4096^3, the same kernel on different operand VALUES (us per launch, 3 rounds of 60 launches, in turn):")
    rows = {name: [] for name, _, _ in sets}
    for _ in range(3):
        for name, a, b in sets:
            rows[name].append(_event_us(gern_amd, torch, lambda: g(a, b, dC), 5, 60))
    for name, t in rows.items():
        print("  this build, %-16s %s   min %.1f us = %.0f TFLOP/s" % (name + ":", " ".join("%.1f" % x for x in t), min(t), 2.0 * n ** 3 / (min(t) * 1e-6) / 1e12))
    views = [(name, a.view(torch.bfloat16), b.view(torch.bfloat16)) for name, a, b in sets]
    for _ in range(200):
        torch.matmul(views[0][1], views[0][2], out=out)
    rows = {name: [] for name, _, _ in sets}
    for _ in range(3):
        for name, a, b in views:
            rows[name].append(vendor_us(a, b))
    for name, t in rows.items():
        print("  torch.matmul, %-16s %s   min %.1f us = %.0f TFLOP/s" % (name + ":", " ".join("%.1f" % x for x in t), min(t), 2.0 * n ** 3 / (min(t) * 1e-6) / 1e12))


def vendor_gemm(gern_amd, torch):
    print("torch.matmul (vendor GEMM library), uniform [-1, 1) operands, us per launch over 5 rounds of 30 launches:")
    for n in (4096, 8192):
        for dt, name in ((torch.bfloat16, "bf16"), (torch.float32, "fp32")):
            A = (torch.rand(n, n, device="cuda") * 2 - 1).to(dt)
            B = (torch.rand(n, n, device="cuda") * 2 - 1).to(dt)
            out = torch.empty(n, n, device="cuda", dtype=dt)
            for _ in range(10):
                torch.matmul(A, B, out=out)
            torch.cuda.synchronize()
            res = []
            for _ in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(30):
                    torch.matmul(A, B, out=out)
                e1.record()
                torch.cuda.synchronize()
                res.append(e0.elapsed_time(e1) / 30 * 1e3)
            print("  %d^3 %s: %s   min %.1f us = %.0f TFLOP/s" % (n, name, " ".join("%.1f" % r for r in res), min(res),
                                                                   2.0 * n ** 3 / (min(res) * 1e-6) / 1e12))


def qk_phases(gern_amd, torch):
    from gern_amd import inputs
    m = n = 4096
    d = 128
    Q = inputs.to_bf16_bits(inputs.normal((m, d), 5))
    K = inputs.to_bf16_bits(inputs.normal((n, d), 6))
    dQ, dK = torch.from_numpy(Q.view(np.int16)).cuda(), torch.from_numpy(K.view(np.int16)).cuda()
    dS = torch.zeros((m, n), device="cuda")
    scratch = torch.zeros(2 * 1024 * 1024 + 256, dtype=torch.uint8, device="cuda")
    stamps = torch.zeros((256, 8, 2), dtype=torch.int64, device="cuda")
    (k,) = _compile(gern_amd, QK_SRC, ["qk_phases"])
    ex = Exchange(scratch.data_ptr() + 256, scratch.data_ptr(), 16, int(os.environ.get('GERN_QK_SPIN_LIMIT', 1 << 18)), (2 * 1024 * 1024) // 8)
    args = [Mat(dK.data_ptr(), n, d, d), Mat(dQ.data_ptr(), m, d, d), Mat(dS.data_ptr(), m, n, n), ex,
            C.c_float(1.0 / np.sqrt(d)), C.c_void_p(stamps.data_ptr())]
    us = _event_us(gern_amd, torch, lambda: _launch(gern_amd, k, (16, 16, 1), (512, 1, 1), args), 10, 50)
    us = _event_us(gern_amd, torch, lambda: _launch(gern_amd, k, (16, 16, 1), (512, 1, 1), args), 10, 50)
    _phase_table("QK^T softmax 4096 x 4096 x 128, tile kernel with clock reads", stamps.cpu().numpy(),
                 ["start", "qk_scaled done", "softmax done, stores issued", "stores acknowledged"], us)
    err = float((dS.double().sum(dim=1) - 1).abs().max())
    print("  rows sum to 1 within %.2g" % err)


def mfma_rate(gern_amd, torch):
    (k, _, _) = _compile(gern_amd, RATE_SRC, ["mfma_rate", "write_rate", "write_rate_through"])
    sink = torch.zeros(16, device="cuda")
    stamps = torch.zeros((256, 4), dtype=torch.int64, device="cuda")
    iters = 6000  # x 8 MFMAs x 32 cycles x 2 wavefronts per SIMD: ~3.1 M cycles
    flop = 256.0 * 8 * iters * 8 * (2.0 * 32 * 32 * 16)
    print("pure MFMA loop (v_mfma_f32_32x32x16_bf16; 256 workgroups x 8 wavefronts x %d x 8 instructions, no memory access):" % iters)
    for what, spread in (("operands spread over [-1, 1)", 1.0), ("all operands zero", 0.0), ("operands spread over [-1, 1)", 1.0)):
        args = [C.c_void_p(sink.data_ptr()), C.c_int(iters), C.c_float(spread), C.c_void_p(stamps.data_ptr())]
        us = _event_us(gern_amd, torch, lambda: _launch(gern_amd, k, (256, 1, 1), (512, 1, 1), args), 2, 5)
        s = stamps.cpu().numpy().astype(np.float64)
        span_us = (s[:, 1] - s[:, 0]) / 100.0
        mhz = (s[:, 3] - s[:, 2]) / span_us
        # the older wavefront of a SIMD is served first and finishes early: the launch, not wavefront 0, times the pipe
        busy = (iters * 16 * 32) / (np.median(mhz) * us)
        print("  %-30s %6.0f us per launch = %4.0f TFLOP/s sustained; shader clock %.0f - %.0f MHz (median %.0f); "
              "matrix pipe busy %.0f %% of the launch at that clock"
              % (what + ":", us, flop / (us * 1e-6) / 1e12, mhz.min(), mhz.max(), np.median(mhz), 100.0 * busy))


def write_rate(gern_amd, torch):
    (_, k, kt) = _compile(gern_amd, RATE_SRC, ["mfma_rate", "write_rate", "write_rate_through"])
    out = torch.zeros(16 * 1024 * 1024, device="cuda")  # 64 MiB
    n = C.c_longlong(out.numel() // 4)
    args = [C.c_void_p(out.data_ptr()), n]
    grid = ((out.numel() // 4 + 255) // 256, 1, 1)
    for name, kernel in (("16-byte streaming stores", k), ("16-byte stores written through to memory", kt)):
        us = _event_us(gern_amd, torch, lambda: _launch(gern_amd, kernel, grid, (256, 1, 1), args), 10, 100)
        us = _event_us(gern_amd, torch, lambda: _launch(gern_amd, kernel, grid, (256, 1, 1), args), 10, 100)
        print("write-only kernel, 64 MiB of %s: %.1f us per launch = %.0f GB/s" % (name, us, out.numel() * 4 / (us * 1e-6) / 1e9))
    assert float(out[1]) == 2.0 and float(out[-1]) == 4.0


def main():
    import torch

    import __graft_entry__
    __graft_entry__.ensure_built()
    import gern_amd
    if gern_amd.device_count() < 1 or not torch.cuda.is_available():
        sys.exit("gern_amd.microbench needs a GPU")
    probes = {"gemm_bf16_phases": gemm_bf16_phases, "gemm_bf16_split": gemm_bf16_split, "gemm_bf16_operands": gemm_bf16_operands, "vendor_gemm": vendor_gemm, "qk_phases": qk_phases, "mfma_rate": mfma_rate, "write_rate": write_rate}
    chosen = sys.argv[1:] or list(probes)
    for name in chosen:
        if name not in probes:
            sys.exit("unknown probe %r (have: %s)" % (name, ", ".join(probes)))
        probes[name](gern_amd, torch)
        print(flush=True)


if __name__ == "__main__":
    main()
