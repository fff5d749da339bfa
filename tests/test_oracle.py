"""Pins the CPU oracle: golden vectors written by the reference's own CPU
lowering, the reference's known-answer tests, and what the mathematics fixes.
No GPU."""
import os
from concurrent.futures import ProcessPoolExecutor

import numpy as np
import pytest

from gern_amd import inputs


# ---------------------------------------------------------------- inputs ----
def test_mt19937_known_answer(oracle):
    # ISO C++ [rand.predef]: the 10000th output of a default-seeded mt19937
    assert int(oracle.mt19937_u32(5489, 10000)[-1]) == 4123659995


def test_mt19937_matches_numpy_raw_words(oracle):
    raw = np.random.RandomState(1234)._bit_generator.random_raw(5000).astype(np.uint32)
    assert np.array_equal(raw, oracle.mt19937_u32(1234, 5000))


def test_input_generators_agree(oracle):
    assert np.array_equal(inputs.uniform((37, 19), 5), oracle.uniform((37, 19), 5))
    assert np.array_equal(inputs.uniform((37, 19), 5, -1.0, 1.0), oracle.uniform((37, 19), 5, -1.0, 1.0))
    a, b = inputs.normal((41, 7), 6, 0.0, 2.0), oracle.normal((41, 7), 6, 0.0, 2.0)
    assert np.array_equal(a, b)
    u = inputs.uniform((100000,), 9)
    assert 0.0 <= u.min() and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.01
    n = inputs.normal((200000,), 9, 0.0, 2.0)
    assert abs(n.mean()) < 0.02 and abs(n.std() - 2.0) < 0.02


def test_bf16_rounding_known_answers(oracle):
    x = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -2.5, 0.0, 3.0e38, 1.0 + 2.0 ** -7], dtype=np.float32)
    bits, val = oracle.to_bf16(x)
    # ties go to even: 1 + 2^-8 -> 1.0 ; 1 + 3*2^-8 -> 1 + 2^-6
    assert list(bits[:3]) == [0x3F80, 0x3F80, 0x3F82]
    assert val[3] == -2.5 and val[4] == 0.0 and val[6] == np.float32(1.0 + 2.0 ** -7)
    assert np.array_equal(bits, inputs.to_bf16_bits(x))


# ------------------------------------------------------------------ blur ----
def test_blur_reference_closed_form(oracle):
    # apps/blur/blur.cpp:96-108: on ascending input X then Y reproduces the
    # input shifted by (1,1) exactly while 3*value < 2^24.
    a = oracle.ascending(1024, 1024)
    out = oracle.blur_chain(a, "xy")
    assert out.shape == (1022, 1022)
    assert np.array_equal(out, a[1:-1, 1:-1])


def test_blur_brute_force_tiny(oracle):
    img = oracle.uniform((7, 9), 3)
    want = np.zeros((5, 5), dtype=np.float32)
    x1 = np.zeros((7, 7), dtype=np.float32)
    three = np.float32(3)
    for i in range(7):
        for j in range(7):
            x1[i, j] = ((np.float32(0) + img[i, j]) + img[i, j + 1] + img[i, j + 2]) / three
    y = np.zeros((5, 7), dtype=np.float32)
    for i in range(5):
        for j in range(7):
            y[i, j] = ((np.float32(0) + x1[i, j]) + x1[i + 1, j] + x1[i + 2, j]) / three
    for i in range(5):
        for j in range(5):
            want[i, j] = ((np.float32(0) + y[i, j]) + y[i, j + 1] + y[i, j + 2]) / three
    assert np.array_equal(oracle.blur_chain(img, "xyx"), want)
    # x and y are not interchangeable on a non-square footprint
    assert oracle.blur_chain(img, "yxy").shape == (3, 7)


def test_blur_constant_image_and_order(oracle):
    c = np.full((20, 30), 0.625, dtype=np.float32)  # 3 * 0.625 is exact
    assert np.array_equal(oracle.blur_chain(c, "xyx"), np.full((18, 26), 0.625, dtype=np.float32))
    img = oracle.uniform((40, 50), 4)
    assert np.array_equal(oracle.blur_chain(img.T.copy(), "y").T, oracle.blur_chain(img, "x"))


@pytest.mark.parametrize("pattern,tile", [("xy", (7, 13)), ("xyx", (5, 11)), ("xyx", (64, 252)), ("y", (3, 3))])
def test_blur_fused_tiles_equal_whole_passes(oracle, pattern, tile):
    img = oracle.uniform((70, 300), 8)
    assert np.array_equal(oracle.blur_chain(img, pattern), oracle.blur_chain_tiled(img, pattern, *tile))


@pytest.mark.parametrize("name,pattern", [("blur_xy", "xy"), ("blur_xyx", "xyx"), ("blur_xyx_wide", "xyx"),
                                          ("blur_xy_asc", "xy")])
def test_blur_golden(oracle, golden, name, pattern):
    assert np.array_equal(oracle.blur_chain(golden[name + "_in"], pattern), golden[name + "_out"])


# --------------------------------------------------------------- softmax ----
@pytest.mark.parametrize("name", ["softmax64", "softmax1000", "softmax4096"])
def test_softmax_golden(oracle, golden, name):
    assert np.array_equal(oracle.softmax_rows(golden[name + "_in"]), golden[name + "_out"])


def test_softmax_invariants(oracle):
    x = oracle.normal((32, 4096), 3, 0.0, 2.0)
    s = oracle.softmax_rows(x)
    assert np.all(np.abs(s.sum(axis=1, dtype=np.float64) - 1.0) < 4096 * 2.0 ** -24)
    # shifting by a power of two is exact in fp32 for these magnitudes
    assert np.allclose(oracle.softmax_rows(x + np.float32(4.0)), s, rtol=2e-6, atol=0)
    const = np.full((3, 512), -1.25, dtype=np.float32)
    assert np.array_equal(oracle.softmax_rows(const), np.full((3, 512), 1.0 / 512, dtype=np.float32))
    # the maximum is found wherever it sits, including at column 0 and for all-negative rows
    neg = -np.abs(x[:4]) - 1.0
    sn = oracle.softmax_rows(neg)
    assert np.all(sn.argmax(axis=1) == neg.argmax(axis=1))
    assert np.all(sn.max(axis=1) <= 1.0) and np.all(np.isfinite(sn))


def test_softmax_against_torch(oracle):
    import torch
    x = oracle.normal((16, 4096), 5, 0.0, 2.0)
    want = torch.softmax(torch.from_numpy(x).double(), dim=1).numpy()
    got = oracle.softmax_rows(x).astype(np.float64)
    assert np.max(np.abs(got - want) / want) < 5e-6


# ------------------------------------------------------------------ GEMM ----
def test_gemm_reference_known_answers(oracle, golden):
    # test/test-cpu-mm.cpp: ascending 4x4 and 10x10, exact small integers
    for n in (4, 10):
        a = oracle.ascending(n, n)
        want = (a.astype(np.int64) @ a.astype(np.int64)).astype(np.float32)
        assert np.array_equal(oracle.gemm_f32(a, a), want)
    assert np.array_equal(oracle.gemm_f32(golden["gemm_asc_A"], golden["gemm_asc_A"]), golden["gemm_asc_C"])
    assert np.array_equal(oracle.gemm_f32(golden["gemm_A"], golden["gemm_B"]), golden["gemm_C"])


def test_gemm_structure(oracle):
    A = oracle.uniform((12, 20), 1, -1.0, 1.0)
    B = oracle.uniform((20, 9), 2, -1.0, 1.0)
    eye = np.eye(20, dtype=np.float32)
    assert np.array_equal(oracle.gemm_f32(A, eye), A)
    perm = eye[:, np.random.RandomState(0).permutation(20)]
    assert np.array_equal(oracle.gemm_f32(A, perm), A @ perm)
    # accumulates INTO C
    c0 = np.full((12, 9), 2.0, dtype=np.float32)
    assert np.allclose(oracle.gemm_f32(A, B, C_in=c0), 2.0 + A.astype(np.float64) @ B.astype(np.float64), rtol=1e-5, atol=1e-5)
    # non-square shapes catch a transposed operand
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.max(np.abs(oracle.gemm_f32(A, B) - want)) < 1e-5
    # sampled rows
    part = oracle.gemm_f32(A, B, rows=(3, 5))
    assert np.array_equal(part[3:5], oracle.gemm_f32(A, B)[3:5]) and not part[:3].any()


def test_gemm_bf16_and_qk_softmax(oracle):
    ai = np.random.RandomState(1).randint(-8, 9, size=(9, 16)).astype(np.float32)
    bi = np.random.RandomState(2).randint(-8, 9, size=(16, 5)).astype(np.float32)
    abits, _ = oracle.to_bf16(ai)
    bbits, _ = oracle.to_bf16(bi)
    assert np.array_equal(oracle.gemm_bf16(abits, bbits), ai @ bi)  # exact small integers
    A = oracle.uniform((8, 64), 3, -1.0, 1.0)
    B = oracle.uniform((64, 6), 4, -1.0, 1.0)
    abits, av = oracle.to_bf16(A)
    bbits, bv = oracle.to_bf16(B)
    assert np.array_equal(oracle.gemm_bf16(abits, bbits), oracle.gemm_f32(av, bv))
    # QK^T softmax is the composition of the two pinned pieces
    Q = oracle.normal((6, 128), 5)
    K = oracle.normal((40, 128), 6)
    qb, qv = oracle.to_bf16(Q)
    kb, kv = oracle.to_bf16(K)
    scale = np.float32(1.0 / np.sqrt(128.0))
    logits = oracle.gemm_f32(qv, kv.T.copy()) * scale
    assert np.array_equal(oracle.qk_softmax(qb, kb, scale), oracle.softmax_rows(logits))


# --------------------------------------------- reference-derived checker ----
def test_oracle_matches_reference_lowering(oracle):
    from oracle import ref
    if not ref.available():
        pytest.skip("oracle/_ref is not built here (needs the reference tree)")
    img = oracle.uniform((1024, 1024), 1)
    assert np.array_equal(ref.blur_chain(img, "xy", 73, 146), oracle.blur_chain(img, "xy"))
    img = oracle.uniform((272, 364), 2)
    assert np.array_equal(ref.blur_chain(img, "xyx", 90, 180), oracle.blur_chain(img, "xyx"))
    x = oracle.normal((64, 4096), 3, 0.0, 2.0)
    assert np.array_equal(ref.softmax_rows(x, 8), oracle.softmax_rows(x))
    A = oracle.uniform((64, 96), 6, -1.0, 1.0)
    B = oracle.uniform((96, 32), 7, -1.0, 1.0)
    assert np.array_equal(ref.gemm(A, B, 16, 8, 96), oracle.gemm_f32(A, B))


# ------------------------------------------------- division by constant ----
def _mismatches(args):
    import ctypes as C
    from oracle import oracle as o
    d, lo, hi = args
    ulp, amin, amax = C.c_uint32(), C.c_float(), C.c_float()
    n = int(o.lib().oracle_quotient_mismatches(d, lo, hi, C.byref(ulp), C.byref(amin), C.byref(amax)))
    return n, ulp.value, amin.value, amax.value


def test_two_fma_division_by_three_matches_ieee_division():
    """quotient_of_sum for three taps: fma(s, c_hi, fma(s, c_lo, +0)) with
    1/3 = c_hi + c_lo.  Over ALL fp32 operands (both signs, subnormals,
    infinities, zeros) it equals (0 + s) / 3 bit for bit, except for
    2^-126 <= |s| < 2^-122, where the correction term underflows and the
    subnormal quotient may be one ulp off: the blur kernels rely on exactly this."""
    chunks = [(3.0, i << 27, min((i + 1) << 27, 0x7F800001)) for i in range(16)]
    chunks += [(3.0, 0x80000000 + (i << 27), min(0x80000000 + ((i + 1) << 27), 0xFF800001)) for i in range(16)]
    workers = min(8, os.cpu_count() or 1)
    with ProcessPoolExecutor(workers) as ex:
        results = list(ex.map(_mismatches, chunks))
    bad = [r for r in results if r[0]]
    assert bad, "expected the known sliver of the subnormal range"
    assert max(r[1] for r in bad) == 1                       # one unit in the last place at most
    assert min(r[2] for r in bad) >= 2.0 ** -126             # only dividends in [2^-126, 2^-122)
    assert max(r[3] for r in bad) < 2.0 ** -122
    # zero of either sign comes out as +0, as (0 + s) / 3 does; infinities stay infinite
    import ctypes as C
    from oracle import oracle as o
    q = o.lib().oracle_quotient_of_sum
    assert np.float32(q(np.float32(-0.0), 3.0)).tobytes() == np.float32(0.0).tobytes()
    assert q(np.float32(np.inf), 3.0) == np.inf and q(np.float32(-np.inf), 3.0) == -np.inf


def _fallback_mismatches(args):
    from oracle import oracle as o
    d, lo, hi = args
    return int(o.lib().oracle_div_const_mismatches(d, lo, hi))


def test_fma_corrected_division_by_three_is_exact():
    """q = x*RN(1/3); q += fma(-3, q, x) * RN(1/3) equals x / 3 for EVERY finite
    fp32 x (both signs, subnormals included): the blur kernels fall back to it for tiles
    that hold tiny values or zeros."""
    chunks = [(3.0, i << 27, min((i + 1) << 27, 0x7F800000)) for i in range(16)]
    chunks += [(3.0, 0x80000000 + (i << 27), min(0x80000000 + ((i + 1) << 27), 0xFF800000)) for i in range(16)]
    workers = min(8, os.cpu_count() or 1)
    with ProcessPoolExecutor(workers) as ex:
        bad = sum(ex.map(_fallback_mismatches, chunks))
    assert bad == 0


def test_division_by_powers_of_two_is_exact(oracle):
    # sampled, including the subnormal range (the product with 2^-k rounds as the quotient does)
    for d in (2.0, 4.0, 8.0):
        for lo, hi in ((0, 1 << 24), (0x3F000000, 0x3F000000 + (1 << 22)), (0x80000000, 0x80000000 + (1 << 24))):
            assert oracle.lib().oracle_quotient_mismatches(d, lo, hi, None, None, None) == 0


def test_max_ulp_known_answers(oracle):
    """max_ulp is the yardstick of the blur parity tests: known distances, so that `== 0` there means
    bit-equal apart from the sign of zero (which those tests compare separately)."""
    one = np.float32(1.0)
    up = np.nextafter(one, np.float32(2.0))
    assert oracle.max_ulp([one], [one]) == 0
    assert oracle.max_ulp([one], [up]) == 1 and oracle.max_ulp([up], [one]) == 1
    three = np.array([0x3F800003], dtype=np.uint32).view(np.float32)
    assert oracle.max_ulp([one], three) == 3
    # the worst element wins, wherever it sits
    a = np.full(1000, 0.375, dtype=np.float32)
    b = a.copy()
    b[617] = np.nextafter(np.nextafter(b[617], np.float32(1.0)), np.float32(1.0))
    assert oracle.max_ulp(a, b) == 2
    # across a binade boundary and across zero the distance counts representable numbers
    below_two = np.nextafter(np.float32(2.0), np.float32(0.0))
    assert oracle.max_ulp([below_two], [np.nextafter(np.float32(2.0), np.float32(3.0))]) == 2
    tiny = np.array([1], dtype=np.uint32).view(np.float32)  # the smallest subnormal
    assert oracle.max_ulp(tiny, -tiny) == 2
    assert oracle.max_ulp([np.float32(0.0)], [np.float32(-0.0)]) == 0  # documented: the sign of zero is not a distance
    # a NaN on either side is never "close"
    assert oracle.max_ulp([np.float32(np.nan)], [one]) == 0xFFFFFFFF
    assert oracle.max_ulp([one], [np.float32(np.nan)]) == 0xFFFFFFFF
    assert oracle.max_ulp([one, np.float32(np.nan)], [one, np.float32(np.nan)]) == 0xFFFFFFFF
    # far apart: one against minus one
    assert oracle.max_ulp([one], [-one]) == 2 * 0x3F800000
