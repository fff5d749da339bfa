"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real
MI355X.  Tolerances are the ones the task states: fp32 stencil within 2 ulp
(measured: bit-exact), fp32 softmax within 1e-5 relative, fp32 GEMM within
1e-4*sqrt(K) relative, bf16-in/fp32-accumulate GEMM within 1e-2 relative."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch
    import gern_amd
    if gern_amd.device_count() < 1 or not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests must run on an MI355X box")
    assert gern_amd.device_limits().arch.decode().startswith("gfx950")
    return gern_amd


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _run_blur(gpu, img, pattern, **kw):
    import torch
    p = gpu.BlurChain(pattern, **kw)
    out = torch.full(p.out_shape(*img.shape), float("nan"), dtype=torch.float32, device="cuda")
    p(_dev(img), out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


# ------------------------------------------------------------------ blur ----
@pytest.mark.parametrize("name,pattern", [("blur_xy", "xy"), ("blur_xyx", "xyx"), ("blur_xyx_wide", "xyx"),
                                          ("blur_xy_asc", "xy")])
def test_blur_golden_vectors(gpu, golden, name, pattern):
    got = _run_blur(gpu, golden[name + "_in"], pattern)
    assert np.array_equal(got, golden[name + "_out"])


@pytest.mark.parametrize("shape,pattern,kw", [
    ((1024, 1024), "xy", {}),                                   # the reference's CPU-runnable configuration
    ((1024, 1024), "xyx", {}),
    ((70, 300), "xyx", {"tile_rows": 4}),                       # ragged in both directions
    ((3, 5), "xy", {}),                                         # a single output element
    ((515, 1027), "xyx", {"tile_rows": 6, "waves_per_block": 4}),  # odd extents: unaligned rows, WARP_X mapping
    ((300, 700), "yxy", {"tile_rows": 8}),
    ((64, 64), "x", {}),
    ((64, 64), "y", {"tile_cols": 128}),
    # the widest tile (stores its own 252 columns) and the default one (224 columns, windows moved to whole lines)
    ((1024, 1024), "xyx", {"tile_rows": 6, "tile_cols": 252}),
    ((100, 1500), "xyx", {"tile_rows": 6, "flags": 16}),        # GERN_PIPELINE_BLUR_PLAIN_STORES
    ((100, 1500), "xyx", {"tile_rows": 5, "tile_cols": 64}),    # narrow line-aligned tiles, result rows 1496 floats apart
    ((61, 2047), "xy", {"tile_rows": 3, "tile_cols": 192, "waves_per_block": 2}),  # result rows 2045 floats apart: mostly unaligned
    ((40, 228), "xyx", {"tile_rows": 8}),                       # exactly one tile of 224 columns
    ((40, 229), "xyx", {"tile_rows": 8}),                       # one column into the second tile
])
def test_blur_matches_oracle_bit_exact(gpu, oracle, shape, pattern, kw):
    img = oracle.uniform(shape, 7)
    got = _run_blur(gpu, img, pattern, **kw)
    want = oracle.blur_chain(img, pattern)
    assert got.shape == want.shape
    assert oracle.max_ulp(got, want) == 0


def test_blur_reference_closed_form_on_gpu(gpu, oracle):
    # apps/blur/blur.cpp:96-108, the reference's own GPU check
    a = oracle.ascending(1024, 1024)
    assert np.array_equal(_run_blur(gpu, a, "xy"), a[1:-1, 1:-1])


def test_blur_full_size_three_stage(gpu, oracle):
    import torch
    img = oracle.uniform((8192, 8192), 2)
    # the schedule bench.py times: one wavefront per 4 x 224 output tile, line-aligned store windows
    got = _run_blur(gpu, img, "xyx", tile_rows=4)
    assert got.shape == (8190, 8188)
    # exact against the oracle on four bands (top, two interior tile seams, bottom)
    for r0 in (0, 4093, 4 * 1100 - 3, 8190 - 64):
        want = oracle.blur_chain(img[r0:r0 + 66], "xyx")
        assert np.array_equal(got[r0:r0 + 64], want)
    # size-independent properties over the whole image: a constant image is a
    # fixed point, and the schedule does not change a single bit
    const = np.full((8192, 8192), 0.375, dtype=np.float32)
    assert np.all(_run_blur(gpu, const, "xyx", tile_rows=4) == np.float32(0.375))
    for kw in ({"tile_rows": 6, "tile_cols": 252}, {"tile_rows": 8, "waves_per_block": 4}):
        assert np.array_equal(got, _run_blur(gpu, img, "xyx", **kw)), kw
    del torch


def test_blur_non_finite_inputs_follow_ieee(gpu, oracle):
    img = oracle.uniform((40, 300), 3)
    img[5, 7] = np.inf
    img[20, 100] = np.nan
    img[30, 200] = -0.0
    got = _run_blur(gpu, img, "xy")
    want = oracle.blur_chain(img, "xy")
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(want)], want[~np.isnan(want)])


def test_blur_signed_zeros_and_negative_values(gpu, oracle):
    # the reference's sums start at +0, so a neighbourhood of -0 gives +0; the
    # kernel leaves the leading zero out of its sums and must still agree in
    # every bit, signs of zeros included
    img = (oracle.uniform((40, 300), 4) - np.float32(0.5)).astype(np.float32)
    img[:12, :] = -0.0
    img[12:20, :64] = 0.0
    img[25, 10:13] = -0.0
    for pattern in ("x", "y", "xy", "xyx"):
        got = _run_blur(gpu, img, pattern)
        want = oracle.blur_chain(img, pattern)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), pattern
    assert not np.any(np.signbit(_run_blur(gpu, np.full((16, 300), -0.0, dtype=np.float32), "xyx")))


def test_blur_tiny_values_and_zeros_stay_exact(gpu, oracle):
    # the two-FMA division by 3 is IEEE-exact except for sums in
    # [2^-126, 2^-122); tiles that could produce such sums (values below 2^-60,
    # zeros) take the slower exact division, so every range matches bit for bit
    base = oracle.uniform((24, 300), 6) + np.float32(0.25)
    for scale in (2.0 ** -59, 2.0 ** -61, 2.0 ** -118, 2.0 ** -125, 2.0 ** -127, 2.0 ** -140):
        img = (base * np.float32(scale)).astype(np.float32)
        for pattern in ("xyx", "y"):
            assert oracle.max_ulp(_run_blur(gpu, img, pattern), oracle.blur_chain(img, pattern)) == 0, (scale, pattern)
    sparse = base.copy()
    sparse[::3, ::5] = 0.0
    sparse[7, 100:140] = np.float32(1e-37)
    got, want = _run_blur(gpu, sparse, "xyx"), oracle.blur_chain(sparse, "xyx")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_blur_on_windows_of_wider_buffers(gpu, oracle):
    # row pitches larger than the widths (ld_in, ld_out of the C ABI), windows
    # that start off the 16-byte grid, and a result written into the middle of
    # a larger buffer whose other elements must stay untouched
    import torch
    big = oracle.uniform((90, 700), 21)
    d_big = _dev(big)
    # result pitches: odd (most rows start off the 16-byte grid and keep their own columns) and a
    # multiple of four floats (every row moves its windows to whole 128-byte lines)
    for (pad, off) in ((9, 5), (12, 8)):
        for (r0, c0, rows, cols) in ((0, 0, 90, 520), (3, 4, 60, 600), (5, 1, 70, 333), (2, 3, 9, 17)):
            win = d_big[r0:r0 + rows, c0:c0 + cols]
            p = gpu.BlurChain("xyx", tile_rows=6)
            orows, ocols = p.out_shape(rows, cols)
            canvas = torch.full((orows + 4, ocols + pad), -7.0, dtype=torch.float32, device="cuda")
            out = canvas[2:2 + orows, off:off + ocols]
            p(win, out)
            torch.cuda.synchronize()
            want = oracle.blur_chain(np.ascontiguousarray(big[r0:r0 + rows, c0:c0 + cols]), "xyx")
            got = canvas.cpu().numpy()
            assert np.array_equal(got[2:2 + orows, off:off + ocols], want), (pad, off, r0, c0, rows, cols)
            frame = got.copy()
            frame[2:2 + orows, off:off + ocols] = -7.0
            assert np.all(frame == -7.0), (pad, off, r0, c0, rows, cols)


# --------------------------------------------------------------- softmax ----
def _run_softmax(gpu, x, **kw):
    import torch
    sm = gpu.Softmax(x.shape[1], **kw)
    out = torch.full(x.shape, float("nan"), dtype=torch.float32, device="cuda")
    sm(_dev(x), out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("name", ["softmax64", "softmax1000", "softmax4096"])
def test_softmax_golden_vectors(gpu, golden, name):
    got = _run_softmax(gpu, golden[name + "_in"])
    want = golden[name + "_out"]
    assert np.max(np.abs(got - want) / want) < 1e-5


# Widths of 1024 columns and more that divide into 256-column chunks spread a
# row over 2, 4 or 8 wavefronts (1024 -> 2 x 512, 2048 -> 4 x 512, 3072 -> 4 x
# 768, 4096 -> 8 x 512, 6144 -> 8 x 768, 8192 -> 8 x 1024); the others keep one
# wavefront per row.  Row counts that leave a partial last workgroup included.
@pytest.mark.parametrize("shape,kw", [((64, 4096), {}), ((33, 1000), {"rows_per_wave": 2}), ((5, 7), {}),
                                      ((128, 256), {"rows_per_wave": 4}), ((16, 8192), {}), ((37, 1024), {}),
                                      ((21, 2048), {"rows_per_wave": 2}), ((19, 3072), {}), ((9, 6144), {}),
                                      ((7, 4096), {"rows_per_wave": 4}), ((40, 1280), {})])
def test_softmax_matches_oracle(gpu, oracle, shape, kw):
    x = oracle.normal(shape, 11, 0.0, 2.0)
    got = _run_softmax(gpu, x, **kw)
    want = oracle.softmax_rows(x)
    assert np.max(np.abs(got - want) / want) < 1e-5


# Rows wider than 8192 columns are cut into 4, 8 or 16 pieces of at most 4096 columns, one per wavefront;
# widths that do not divide leave the last pieces partly used (8200 -> 4 x 2052, the last 2044; 20000 -> 8 x
# 2500; 40004 -> 16 x 2504, the last 2444; 8193 -> 4 x 2052, the last 2037).  The oracle adds a row left to right in fp32, as the reference's CPU
# code does, and over this many terms strays from the exact sum by more than the bar itself: the result is held
# to 1e-5 against the exact (fp64) softmax, and to the oracle within 1e-5 plus the oracle's own distance from it.
@pytest.mark.parametrize("shape", [(5, 8193), (9, 8200), (6, 12288), (33, 16384), (3, 20000), (4, 32768), (2, 40004),
                                   (3, 65536), (1, 65531)])
def test_softmax_rows_wider_than_one_wavefront_holds(gpu, oracle, shape):
    x = oracle.normal(shape, 23 + shape[1] % 97, 0.0, 2.0)
    got = _run_softmax(gpu, x)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    exact = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(got - exact) / exact) < 1e-5, shape
    want = oracle.softmax_rows(x)
    own = float(np.max(np.abs(want - exact) / exact))
    assert np.max(np.abs(got - want) / want) < 1e-5 + own, (shape, own)
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5)
    assert np.all(got.argmax(axis=1) == x.argmax(axis=1))


def test_softmax_wide_rows_in_a_window_and_with_a_wide_range(gpu, oracle):
    import torch
    # a 9000-column window of a wider buffer: the unused part of the last piece lies INSIDE the buffer
    ncol, ld, c0 = 9000, 9300, 4
    x = oracle.normal((7, ld), 29, 0.0, 2.0)
    x[:, c0 + ncol:] = 50.0  # would win every maximum if a reduction read past the window
    dx = _dev(x)
    dy = torch.full((7, ld), -7.0, dtype=torch.float32, device="cuda")
    gpu.Softmax(ncol)(dx[:, c0:c0 + ncol], dy[:, c0:c0 + ncol])
    torch.cuda.synchronize()
    got = dy.cpu().numpy()
    x64 = x[:, c0:c0 + ncol].astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    exact = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(got[:, c0:c0 + ncol] - exact) / exact) < 1e-5
    got[:, c0:c0 + ncol] = -7.0
    assert np.all(got == -7.0)
    # differences of more than 87 from the row maximum on a wide row
    x = oracle.normal((3, 10000), 31, 0.0, 40.0)
    got = _run_softmax(gpu, x)
    want = oracle.softmax_rows(x)
    big = want >= 1e-30
    assert np.max(np.abs(got[big] - want[big]) / want[big]) < 1e-5
    assert np.max(np.abs(got[~big] - want[~big])) < 1e-35
    with pytest.raises(gpu.GernError, match="65536"):
        gpu.Softmax(65537)
    with pytest.raises(gpu.GernError, match="32 x 256"):
        gpu.Softmax(16384, rows_per_wave=4)


def test_softmax_on_a_window_of_a_wider_buffer(gpu, oracle):
    # ld larger than ncol; columns outside the window stay as they were
    import torch
    for ncol, ld, c0 in ((1024, 1280, 0), (1000, 1030, 7), (4096, 4100, 4)):
        x = oracle.normal((19, ld), 13, 0.0, 2.0)
        dx = _dev(x)
        dy = torch.full((19, ld), -7.0, dtype=torch.float32, device="cuda")
        sm = gpu.Softmax(ncol)
        sm(dx[:, c0:c0 + ncol], dy[:, c0:c0 + ncol])
        torch.cuda.synchronize()
        got = dy.cpu().numpy()
        want = oracle.softmax_rows(np.ascontiguousarray(x[:, c0:c0 + ncol]))
        assert np.max(np.abs(got[:, c0:c0 + ncol] - want) / want) < 1e-5, (ncol, ld, c0)
        got[:, c0:c0 + ncol] = -7.0
        assert np.all(got == -7.0), (ncol, ld, c0)


def test_softmax_full_size(gpu, oracle):
    x = oracle.normal((8192, 4096), 3, 0.0, 2.0)
    got = _run_softmax(gpu, x)
    for r0 in (0, 4000, 8192 - 256):
        want = oracle.softmax_rows(x[r0:r0 + 256])
        assert np.max(np.abs(got[r0:r0 + 256] - want) / want) < 1e-5
    # properties over all rows: sums to one, order preserved, shift invariance
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 4096 * 2.0 ** -24)
    assert np.all(got.argmax(axis=1) == x.argmax(axis=1))
    shifted = _run_softmax(gpu, x + np.float32(4.0))
    assert np.allclose(shifted, got, rtol=1e-5, atol=0)


def test_softmax_all_negative_rows_and_constant_rows(gpu, oracle):
    x = -np.abs(oracle.normal((8, 4096), 5, 0.0, 2.0)) - 3.0
    x[3, :] = -7.5
    got = _run_softmax(gpu, x)
    want = oracle.softmax_rows(x)
    assert np.max(np.abs(got - want) / want) < 1e-5
    assert np.all(got[3] == np.float32(1.0 / 4096))


# Results leave through buffer stores with 32-bit byte offsets; a matrix beyond 2 GiB has offsets with
# the top bit set, one beyond 4 GiB takes the other store path.  Every element must be written either way.
@pytest.mark.parametrize("rows", [150000, 270000])
def test_softmax_results_beyond_2_and_4_gib(gpu, rows):
    import torch
    x = torch.randn((rows, 4096), device="cuda")
    y = torch.full_like(x, float("nan"))
    gpu.Softmax(4096)(x, y)
    torch.cuda.synchronize()
    assert int(torch.isnan(y).sum()) == 0
    for lo in (0, rows // 2, rows - 64):
        want = torch.softmax(x[lo:lo + 64].double(), dim=1)
        assert float(((y[lo:lo + 64].double() - want).abs() / want).max()) < 1e-5, lo
    assert float((y.sum(dim=1, dtype=torch.float64) - 1).abs().max()) < 1e-5


@pytest.mark.parametrize("ncol", [1000, 4096])
def test_softmax_rows_with_a_wide_range(gpu, oracle, ncol):
    # differences of more than 87 from the row maximum: exp leaves the range of
    # the fast path (results below 2^-126); both the one-wavefront and the
    # multi-wavefront layout must then agree with the CPU's expf, denormals included
    x = oracle.normal((12, ncol), 17, 0.0, 40.0)
    got = _run_softmax(gpu, x)
    want = oracle.softmax_rows(x)
    big = want >= 1e-30
    assert np.max(np.abs(got[big] - want[big]) / want[big]) < 1e-5
    assert np.max(np.abs(got[~big] - want[~big])) < 1e-35
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5)


# ------------------------------------------------------------------ GEMM ----
def _run_gemm(gpu, variant, A, B, C0=None, general_only=False):
    import torch
    g = gpu.Gemm(variant, general_only=general_only)
    M, N = A.shape[0], B.shape[1]
    dC = torch.zeros((M, N), dtype=torch.float32, device="cuda") if C0 is None else _dev(C0)
    if variant == "bf16":
        dA, dB = _dev(A.view(np.int16)), _dev(B.view(np.int16))
    else:
        dA, dB = _dev(A), _dev(B)
    g(dA, dB, dC)
    torch.cuda.synchronize()
    return dC.cpu().numpy()


def _assert_gemm_close(got, want, A, B, tol, rows=None, c0=None, what=None):
    """Two bounds on got - want (got, want: the rows `rows` of the product of the VALUES A and B):
    norm-wise, max |got - want| <= tol * max |want|, and element by element,
    |got - want|_ij <= tol * (|A| |B| (+ |C0|))_ij in fp64 -- the scale of the rounding errors of THAT
    dot product, so an element near zero may not be wrong by more than its own terms allow."""
    lo, hi = (0, A.shape[0]) if rows is None else rows
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape == (hi - lo, B.shape[1]), (got.shape, want.shape, what)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < tol, what
    scale = np.abs(A[lo:hi].astype(np.float64)) @ np.abs(B.astype(np.float64))
    if c0 is not None:
        scale = scale + np.abs(c0[lo:hi].astype(np.float64))
    excess = np.abs(got - want) - tol * scale
    assert np.all(excess <= 0), (what, float(excess.max()), np.unravel_index(int(excess.argmax()), excess.shape))


def test_gemm_f32_golden_and_known_answers(gpu, oracle, golden):
    got = _run_gemm(gpu, "f32", golden["gemm_A"], golden["gemm_B"])
    want = golden["gemm_C"]
    _assert_gemm_close(got, want, golden["gemm_A"], golden["gemm_B"], 1e-4 * np.sqrt(golden["gemm_A"].shape[1]))
    # test/test-cpu-mm.cpp: ascending 10x10, exact small integers
    a = golden["gemm_asc_A"]
    assert np.array_equal(_run_gemm(gpu, "f32", a, a), golden["gemm_asc_C"])


# general_only keeps the shapes that the matrix-core kernel could take
# (K >= 4) on the vector-ALU kernel.
@pytest.mark.parametrize("general_only", [False, True])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (200, 136, 72), (512, 384, 256), (1, 4, 4), (130, 260, 1032)])
def test_gemm_f32_matches_oracle(gpu, oracle, M, N, K, general_only):
    A = oracle.uniform((M, K), 1, -1.0, 1.0)
    B = oracle.uniform((K, N), 2, -1.0, 1.0)
    got = _run_gemm(gpu, "f32", A, B, general_only=general_only)
    want = oracle.gemm_f32(A, B)
    _assert_gemm_close(got, want, A, B, 1e-4 * np.sqrt(K))


@pytest.mark.parametrize("general_only", [False, True])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (200, 136, 72), (512, 384, 256), (3, 2, 8), (130, 260, 1032)])
def test_gemm_bf16_matches_oracle(gpu, oracle, M, N, K, general_only):
    ab, av = oracle.to_bf16(oracle.uniform((M, K), 1, -1.0, 1.0))
    bb, bv = oracle.to_bf16(oracle.uniform((K, N), 2, -1.0, 1.0))
    got = _run_gemm(gpu, "bf16", ab, bb, general_only=general_only)
    want = oracle.gemm_bf16(ab, bb)
    _assert_gemm_close(got, want, av, bv, 1e-2)
    # exact small integers: products and sums are exact in fp32 in any order
    ai = np.random.RandomState(1).randint(-4, 5, size=(M, K)).astype(np.float32)
    bi = np.random.RandomState(2).randint(-4, 5, size=(K, N)).astype(np.float32)
    aib, _ = oracle.to_bf16(ai)
    bib, _ = oracle.to_bf16(bi)
    assert np.array_equal(_run_gemm(gpu, "bf16", aib, bib, general_only=general_only), ai @ bi)


# Every shape the bf16 pipeline accepts (K % 8 == 0, N % 2 == 0) takes the
# eight-wavefront kernel that loads straight into LDS: one K stage, an odd
# number of stages, several column and row tiles, a K that spans more than one
# 4096-deep Reduce step, partial tiles at the bottom and right edges (one row,
# one 8-column chunk, all but one), a partial last K stage (its missing part
# must read as zero), rows of B off the 16-byte grid (N not a multiple of 8),
# two columns, and K below one stage.
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 256, 192), (256, 768, 128), (768, 512, 4096 + 4096 + 64),
                                   (300, 264, 128), (1, 8, 64), (511, 504, 320), (257, 1000, 64),
                                   (256, 256, 72), (300, 258, 200), (130, 262, 8), (77, 2, 120), (512, 302, 4096 + 56)])
@pytest.mark.parametrize("overwrite", [False, True])
def test_gemm_bf16_whole_tile_kernel(gpu, oracle, M, N, K, overwrite):
    import torch
    # small integers: every product and every partial sum is exact in fp32 in
    # any order, so each element of C pins its own row of A and column of B
    ai = np.random.RandomState(11).randint(-3, 4, size=(M, K)).astype(np.float32)
    bi = np.random.RandomState(12).randint(-3, 4, size=(K, N)).astype(np.float32)
    c0 = np.random.RandomState(13).randint(-5, 6, size=(M, N)).astype(np.float32)
    aib, _ = oracle.to_bf16(ai)
    bib, _ = oracle.to_bf16(bi)
    g = gpu.Gemm("bf16", overwrite=overwrite)
    dC = _dev(c0)
    g(_dev(aib.view(np.int16)), _dev(bib.view(np.int16)), dC)
    torch.cuda.synchronize()
    assert "256, 256" in g.kernel_name and "512" in g.kernel_name.split("<")[1].split(",")[0], g.kernel_name
    want = ai.astype(np.float64) @ bi.astype(np.float64) + (0 if overwrite else c0)
    assert np.array_equal(dC.cpu().numpy().astype(np.float64), want)
    # and ordinary values against the oracle
    ab, av = oracle.to_bf16(oracle.uniform((M, K), 21, -1.0, 1.0))
    bb, bv = oracle.to_bf16(oracle.uniform((K, N), 22, -1.0, 1.0))
    dC = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    g(_dev(ab.view(np.int16)), _dev(bb.view(np.int16)), dC)
    torch.cuda.synchronize()
    rows = (max(M - 2, 0), M)
    want = oracle.gemm_bf16(ab, bb, rows=rows)[rows[0]:rows[1]]
    got = dC.cpu().numpy()
    _assert_gemm_close(got[rows[0]:rows[1]], want, av, bv, 1e-2, rows=rows)
    # every element against fp64 of the same bf16 values
    _assert_gemm_close(got, av.astype(np.float64) @ bv.astype(np.float64), av, bv, 1e-2)


# fp32 shapes with K >= 4 take the eight-wavefront kernel on the fp32
# matrix instruction: one K stage, an odd number of stages, several tiles
# either way, a K beyond one 4096-deep Reduce step, partial tiles at the bottom
# and right edges (one row, one 4-column piece, all but one), a partial last K
# stage (its missing part must read as zero), rows of B off the 16-byte grid
# (N not a multiple of 4), a single column, and K below one stage.
@pytest.mark.parametrize("M,N,K", [(256, 256, 32), (512, 256, 96), (256, 768, 64), (512, 512, 4096 + 4096 + 32),
                                   (300, 260, 128), (1, 4, 32), (511, 508, 160), (257, 1000, 32),
                                   (256, 256, 36), (300, 258, 100), (130, 263, 4), (77, 1, 60), (512, 301, 4096 + 28),
                                   # K not a multiple of 4: the last one to three columns of A are added by a
                                   # second launch of the vector-ALU kernel
                                   (256, 256, 50), (130, 258, 63), (300, 301, 4096 + 33), (65, 12, 5)])
@pytest.mark.parametrize("overwrite", [False, True])
def test_gemm_f32_whole_tile_kernel(gpu, oracle, M, N, K, overwrite):
    import torch
    # small integers: exact in fp32 in any order, so each element of C pins
    # its own row of A and column of B
    ai = np.random.RandomState(31).randint(-3, 4, size=(M, K)).astype(np.float32)
    bi = np.random.RandomState(32).randint(-3, 4, size=(K, N)).astype(np.float32)
    c0 = np.random.RandomState(33).randint(-5, 6, size=(M, N)).astype(np.float32)
    g = gpu.Gemm("f32", overwrite=overwrite)
    dC = _dev(c0)
    g(_dev(ai), _dev(bi), dC)
    torch.cuda.synchronize()
    assert "256, 256" in g.kernel_name and "512" in g.kernel_name.split("<")[1].split(",")[0], g.kernel_name
    want = ai.astype(np.float64) @ bi.astype(np.float64) + (0 if overwrite else c0)
    assert np.array_equal(dC.cpu().numpy().astype(np.float64), want)
    # and ordinary values against the oracle and against fp64
    A = oracle.uniform((M, K), 41, -1.0, 1.0)
    B = oracle.uniform((K, N), 42, -1.0, 1.0)
    dC = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    g(_dev(A), _dev(B), dC)
    torch.cuda.synchronize()
    got = dC.cpu().numpy()
    rows = (max(M - 2, 0), M)
    want = oracle.gemm_f32(A, B, rows=rows)[rows[0]:rows[1]]
    _assert_gemm_close(got[rows[0]:rows[1]], want, A, B, 1e-4 * np.sqrt(K), rows=rows)
    _assert_gemm_close(got, A.astype(np.float64) @ B.astype(np.float64), A, B, 1e-4 * np.sqrt(K))


# The matrix-core fp32 kernel reads rows of A in whole 16-byte pieces; a K
# below 4 has none and stays on the vector-ALU kernel.
@pytest.mark.parametrize("M,N,K", [(256, 256, 3), (7, 5, 2)])
def test_gemm_f32_other_shapes_keep_the_general_kernel(gpu, oracle, M, N, K):
    import torch
    ai = np.random.RandomState(51).randint(-3, 4, size=(M, K)).astype(np.float32)
    bi = np.random.RandomState(52).randint(-3, 4, size=(K, N)).astype(np.float32)
    g = gpu.Gemm("f32")
    dC = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    g(_dev(ai), _dev(bi), dC)
    torch.cuda.synchronize()
    assert "512" not in g.kernel_name.split("<")[1].split(",")[0], g.kernel_name
    assert np.array_equal(dC.cpu().numpy(), ai @ bi)


# Schedules written at the level of Gern's API (the reference's gernels/mm/kernel_3.cu:61-75,
# kernel_6.cu:61-74 and kernel_10.cu:108-131) over the scalar matrix_multiply gernel: every
# output is one fp32 sum in ascending k, so the oracle's loop order gives the same bits.
@pytest.mark.parametrize("schedule", [3, 6, 10])
def test_gemm_user_schedules_match_oracle(gpu, oracle, schedule):
    import torch
    n = gpu.GemmSchedule.SIZE
    g = gpu.GemmSchedule(schedule)
    ai = np.random.RandomState(61).randint(-3, 4, size=(n, n)).astype(np.float32)
    bi = np.random.RandomState(62).randint(-3, 4, size=(n, n)).astype(np.float32)
    c0 = np.random.RandomState(63).randint(-5, 6, size=(n, n)).astype(np.float32)
    dC = _dev(c0)
    g(_dev(ai), _dev(bi), dC)
    torch.cuda.synchronize()
    assert np.array_equal(dC.cpu().numpy().astype(np.float64), ai.astype(np.float64) @ bi.astype(np.float64) + c0)
    A = oracle.uniform((n, n), 64, -1.0, 1.0)
    B = oracle.uniform((n, n), 65, -1.0, 1.0)
    dC = torch.zeros((n, n), dtype=torch.float32, device="cuda")
    g(_dev(A), _dev(B), dC)
    torch.cuda.synchronize()
    got = dC.cpu().numpy()
    for rows in ((0, 8), (60, 68), (n - 4, n)):
        want = oracle.gemm_f32(A, B, rows=rows)[rows[0]:rows[1]]
        _assert_gemm_close(got[rows[0]:rows[1]], want, A, B, 1e-4 * np.sqrt(n), rows=rows)
    _assert_gemm_close(got, A.astype(np.float64) @ B.astype(np.float64), A, B, 1e-4 * np.sqrt(n))


@pytest.mark.parametrize("variant", ["f32", "bf16"])
def test_gemm_accumulates_into_c(gpu, oracle, variant):
    A = oracle.uniform((192, 128), 3, -1.0, 1.0)
    B = oracle.uniform((128, 160), 4, -1.0, 1.0)
    C0 = oracle.uniform((192, 160), 5, -1.0, 1.0)
    if variant == "bf16":
        ab, av = oracle.to_bf16(A)
        bb, bv = oracle.to_bf16(B)
        got = _run_gemm(gpu, variant, ab, bb, C0)
        want = C0 + oracle.gemm_f32(av, bv)
        A, B = av, bv
    else:
        got = _run_gemm(gpu, variant, A, B, C0)
        want = oracle.gemm_f32(A, B, C_in=C0)
    _assert_gemm_close(got, want, A, B, 1e-4, c0=C0)


# general_only: the kernels that take every shape (fp32: vector-ALU FMAs, the kernel BASELINE's config 4a
# names; bf16: the four-wavefront kernel that stages through registers) on the full-size product too.
@pytest.mark.parametrize("variant,tol,general_only", [("f32", 1e-4 * 64, False), ("f32", 1e-4 * 64, True),
                                                      ("bf16", 1e-2, False), ("bf16", 1e-2, True)])
def test_gemm_full_size(gpu, oracle, variant, tol, general_only):
    M = N = K = 4096
    A = oracle.uniform((M, K), 4, -1.0, 1.0)
    B = oracle.uniform((K, N), 5, -1.0, 1.0)
    av, bv = A, B
    if variant == "bf16":
        A, av = oracle.to_bf16(A)
        B, bv = oracle.to_bf16(B)
    got = _run_gemm(gpu, variant, A, B, general_only=general_only)
    # 64 whole rows against the oracle (every column, the last ones included):
    # the first and last rows of the first and last 256-row tiles, both sides of
    # two tile seams, of a wavefront seam and of an MFMA-tile seam inside a tile
    bands = ((0, 8), (248, 264), (1000, 1002), (1148, 1156), (2032, 2048), (2300, 2306), (4088, 4096))
    assert sum(b - a for a, b in bands) == 64
    for rows in bands:
        want = (oracle.gemm_bf16(A, B, rows=rows) if variant == "bf16" else oracle.gemm_f32(A, B, rows=rows))[rows[0]:rows[1]]
        _assert_gemm_close(got[rows[0]:rows[1]], want, av, bv, tol, rows=rows, what=rows)
    # Freivalds-style check of the whole product: C r == A (B r) in fp64
    r = np.random.RandomState(9).randint(0, 2, size=(N,)).astype(np.float64)
    a64, b64 = av.astype(np.float64), bv.astype(np.float64)
    lhs = got.astype(np.float64) @ r
    rhs = a64 @ (b64 @ r)
    assert np.max(np.abs(lhs - rhs)) / np.max(np.abs(rhs)) < 1e-4


def test_gemm_f32_operands_off_the_16_byte_grid_keep_the_general_kernel(gpu):
    # the matrix-core kernel loads 16 bytes per lane; operands that start 4
    # bytes off that grid are legal and take the vector-ALU kernel
    import torch
    M, N, K = 256, 256, 64
    ai = np.random.RandomState(61).randint(-3, 4, size=(M, K)).astype(np.float32)
    bi = np.random.RandomState(62).randint(-3, 4, size=(K, N)).astype(np.float32)
    bufa = torch.zeros(M * K + 1, device="cuda")
    bufb = torch.zeros(K * N + 1, device="cuda")
    dA, dB = bufa[1:].view(M, K), bufb[1:].view(K, N)
    dA.copy_(torch.from_numpy(ai))
    dB.copy_(torch.from_numpy(bi))
    assert dA.data_ptr() % 16 == 4 and dA.is_contiguous()
    g = gpu.Gemm("f32")
    dC = torch.zeros((M, N), device="cuda")
    g(dA, dB, dC)
    torch.cuda.synchronize()
    assert g.kernel_name.split("<")[1].split(",")[0].strip() != "512", g.kernel_name
    assert np.array_equal(dC.cpu().numpy(), ai @ bi)
    # the bf16 kernels read 16-byte pieces of A: an operand off that grid is refused, not read
    h = gpu.Gemm("bf16")
    buf = torch.zeros(M * K + 8, dtype=torch.int16, device="cuda")
    with pytest.raises(gpu.GernError, match="aligned"):
        h(buf[1:1 + M * K].view(M, K), torch.zeros((K, N), dtype=torch.int16, device="cuda"), dC)


def test_gemm_rejects_unsupported_bf16_shapes(gpu):
    import torch
    g = gpu.Gemm("bf16")
    A = torch.zeros((8, 12), dtype=torch.int16, device="cuda")
    B = torch.zeros((12, 8), dtype=torch.int16, device="cuda")
    with pytest.raises(gpu.GernError, match="K % 8"):
        g(A, B, torch.zeros((8, 8), device="cuda"))


# ------------------------------------------------------- QK^T -> softmax ----
def _run_qk(gpu, qb, kb, scale, max_keys, flags=0, faults=0):
    """One run on a fresh pipeline; the pipeline must report `faults` afterwards (None: not looked at)."""
    import torch
    p = gpu.QKSoftmax(qb.shape[1], max_keys, flags=flags)
    S = torch.full((qb.shape[0], kb.shape[0]), float("nan"), dtype=torch.float32, device="cuda")
    p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, scale)
    torch.cuda.synchronize()
    if faults is not None:
        assert p.faults() == faults
    return S.cpu().numpy()


# Head dimensions 64, 128, 192 and 256 take the 256 x 256 tile kernel (row
# statistics exchanged between workgroups), 32 and 96 the row-block kernel
# (32: K streamed through LDS, 96: the register path); flag 32
# (GERN_PIPELINE_QK_ROW_BLOCKS) keeps the row-block kernel for the others too
# (256: two tiles in flight instead of four).  Ragged rows and keys.
@pytest.mark.parametrize("M,N,D,max_keys,flags", [(64, 256, 128, 256, 0), (50, 200, 64, 256, 0), (16, 1024, 128, 1024, 0),
                                                  (37, 1000, 32, 1024, 0), (33, 500, 256, 512, 0), (20, 300, 96, 512, 0),
                                                  (48, 2048, 256, 2048, 0), (300, 1000, 192, 1024, 0), (513, 257, 64, 512, 0),
                                                  (700, 4096, 128, 4096, 0),
                                                  (64, 256, 128, 256, 32), (50, 200, 64, 256, 32), (33, 500, 256, 512, 32),
                                                  (48, 2048, 256, 2048, 32)])
def test_qk_softmax_matches_oracle(gpu, oracle, M, N, D, max_keys, flags):
    qb, _ = oracle.to_bf16(oracle.normal((M, D), 5))
    kb, _ = oracle.to_bf16(oracle.normal((N, D), 6))
    scale = np.float32(1.0 / np.sqrt(D))
    got = _run_qk(gpu, qb, kb, scale, max_keys, flags)
    want = oracle.qk_softmax(qb, kb, scale)
    # the bf16-GEMM tolerance governs: inputs are identical bf16 values, the
    # logits differ only by fp32 summation order
    assert np.max(np.abs(got - want) / want) < 1e-2
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5)


# More than sixteen column blocks per row: a wavefront collects the row's statistics in passes of sixteen
# entries.  Widths that are whole passes, one block more, and a ragged last block; the exchange memory bounds
# M x N (1024 rows at 65536 keys), and more is refused.
@pytest.mark.parametrize("M,N,max_keys", [(520, 8192, 8192), (300, 4352, 8192), (257, 10000, 10240), (100, 16384, 16384),
                                          (40, 65536, 65536)])
def test_qk_softmax_tile_kernel_on_rows_wider_than_4096_keys(gpu, oracle, M, N, max_keys):
    import torch
    D = 64
    qb, _ = oracle.to_bf16(oracle.normal((M, D), 50 + M))
    kb, _ = oracle.to_bf16(oracle.normal((N, D), 60 + M))
    scale = np.float32(1.0 / np.sqrt(D))
    p = gpu.QKSoftmax(D, max_keys)
    assert "view_score_tile" in p.source
    S = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, scale)
    torch.cuda.synchronize()
    assert p.faults() == 0
    got = S.cpu().numpy()
    rows = sorted({0, 1, M // 2, M - 1, min(M - 1, 255), min(M - 1, 256)})
    want = oracle.qk_softmax(qb[rows], kb, scale)
    assert np.max(np.abs(got[rows] - want) / want) < 1e-2, (M, N)
    assert not np.isnan(got).any()
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-4)
    if N == 65536:
        big = torch.zeros((1025, D), dtype=torch.int16, device="cuda")
        with pytest.raises(gpu.GernError, match="GERN_QK_SCRATCH_BYTES"):
            p(big, _dev(kb.view(np.int16)), torch.zeros((1025, N), device="cuda"), scale)
        with pytest.raises(gpu.GernError, match="4096"):
            gpu.QKSoftmax(96, 8192)  # the row-block kernel keeps whole rows in registers


@pytest.mark.parametrize("M,N", [(4096, 4096), (8192, 4096), (300, 2560), (2100, 1000)])
def test_qk_softmax_tile_kernel_either_workgroup_order_gives_the_same_bits(gpu, oracle, M, N):
    # Rows of up to 4096 keys: by default every row block's tiles run on one XCD (XCD x takes row blocks x, x + 8,
    # ...; launch numbers past the last whole group of eight row blocks keep their tiles); with NO_XCD_REMAP tiles
    # are taken in launch order.  Which workgroup computes a tile changes nothing in it.
    import torch
    D = 128
    qb, _ = oracle.to_bf16(oracle.normal((M, D), 81))
    kb, _ = oracle.to_bf16(oracle.normal((N, D), 82))
    scale = np.float32(1.0 / np.sqrt(D))
    by_rows, in_order = gpu.QKSoftmax(D, 4096), gpu.QKSoftmax(D, 4096, flags=gpu.NO_XCD_REMAP)
    assert "gern_band" in by_rows.source and "gern_band" not in in_order.source
    results = []
    for p in (by_rows, in_order):
        S = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, scale)
        torch.cuda.synchronize()
        assert p.faults() == 0
        results.append(S.cpu().numpy())
    assert np.array_equal(results[0], results[1])
    rows = sorted({0, 255, 256, M // 2, M - 1})
    want = oracle.qk_softmax(qb[rows], kb, scale)
    assert np.max(np.abs(results[0][rows] - want) / want) < 1e-2
    # wider rows keep the launch order: their row blocks would lie too many launch numbers apart
    assert "gern_band" not in gpu.QKSoftmax(D, 8192).source


def test_qk_softmax_tile_kernel_over_changing_shapes_and_scales(gpu, oracle):
    # One pipeline, one exchange memory: every launch tags its entries with its
    # own number, so shapes may change from run to run (entries left by a wider
    # or taller run are never mistaken for this run's), the scale may be
    # negative (the largest product is then the smallest logit) or zero
    # (a uniform row), and a graph of launches needs nothing from the host.
    import torch
    D = 128
    p = gpu.QKSoftmax(D, 4096)
    assert "view_score_tile" in p.source
    for n, (M, N, scale) in enumerate([(600, 4096, 0.088), (100, 300, 0.088), (600, 4096, -0.05), (257, 1025, 0.0),
                                       (1024, 2048, 0.088), (16, 256, 0.3), (600, 4096, 0.088)]):
        qb, _ = oracle.to_bf16(oracle.normal((M, D), 30 + n))
        kb, _ = oracle.to_bf16(oracle.normal((N, D), 50 + n))
        S = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        for _ in range(3):  # back-to-back launches of one shape, then the next shape
            p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, np.float32(scale))
        torch.cuda.synchronize()
        got = S.cpu().numpy()
        want = oracle.qk_softmax(qb, kb, np.float32(scale))
        assert np.max(np.abs(got - want) / want) < 1e-2, (M, N, scale)
        assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5), (M, N, scale)
    assert p.faults() == 0


# More workgroups than the GPU holds at once: 512 and 1024 tiles of 256 x 256 on 256 compute units, one
# workgroup each.  The workgroups of a row block wait for one another, so this only works if a row block's
# workgroups are dispatched together and ahead of the next row block's; nobody may give up waiting.
@pytest.mark.parametrize("M", [8192, 16384])
def test_qk_softmax_tile_kernel_with_more_workgroups_than_compute_units(gpu, oracle, M):
    import torch
    N, D = 4096, 128
    qb, _ = oracle.to_bf16(oracle.normal((M, D), 81))
    kb, _ = oracle.to_bf16(oracle.normal((N, D), 82))
    scale = np.float32(1.0 / np.sqrt(D))
    p = gpu.QKSoftmax(D, N)
    assert "view_score_tile" in p.source
    S = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, scale)
    torch.cuda.synchronize()
    assert p.faults() == 0
    assert int(torch.isnan(S).sum()) == 0
    assert float((S.sum(dim=1, dtype=torch.float64) - 1).abs().max()) < 1e-5
    for r0 in (0, M // 2 + 250, M - 16):  # first, last, and across a seam of row blocks in the second half of the launch
        got = S[r0:r0 + 16].cpu().numpy()
        want = oracle.qk_softmax(qb, kb, scale, rows=(r0, r0 + 16))[r0:r0 + 16]
        assert np.max(np.abs(got - want) / want) < 1e-2, r0


def test_qk_softmax_tile_kernel_launch_number_wraps_around(gpu, oracle, monkeypatch):
    # A tag is the launch number; when the number wraps around, the last
    # workgroup of that launch clears every entry, so the entries that a tall
    # launch left behind one period ago are not taken for those of the current
    # one.  The period is 65535 launches; this pipeline is built with 1000.
    import torch
    D = 64
    monkeypatch.setenv("GERN_EXPERIMENTS", "1")
    monkeypatch.setenv("GERN_PIPELINE_EXTRA_OPTIONS", "-DGERN_QK_TAG_PERIOD=1000u")
    p = gpu.QKSoftmax(D, 512)
    monkeypatch.delenv("GERN_PIPELINE_EXTRA_OPTIONS")
    monkeypatch.delenv("GERN_EXPERIMENTS")
    big = (oracle.to_bf16(oracle.normal((600, D), 71))[0], oracle.to_bf16(oracle.normal((512, D), 72))[0])
    small = (oracle.to_bf16(oracle.normal((8, D), 73))[0], oracle.to_bf16(oracle.normal((256, D), 74))[0])
    scale = np.float32(0.125)

    def run(qb, kb, times):
        S = torch.full((qb.shape[0], kb.shape[0]), float("nan"), dtype=torch.float32, device="cuda")
        dq, dk = _dev(qb.view(np.int16)), _dev(kb.view(np.int16))
        for _ in range(times):
            p(dq, dk, S, scale)
        torch.cuda.synchronize()
        return S.cpu().numpy()

    want_big = oracle.qk_softmax(big[0], big[1], scale)
    assert np.max(np.abs(run(*big, 3) - want_big) / want_big) < 1e-2          # launches 0-2: tags 1-3 in 768 x 2 entries
    want_small = oracle.qk_softmax(small[0], small[1], scale)
    assert np.max(np.abs(run(*small, 1000) - want_small) / want_small) < 1e-2  # past the wrap: launch number 3 again
    for times in (1, 1, 1, 995, 3):                                            # launch numbers 3, 4, 5, ..., across the next wrap
        assert np.max(np.abs(run(*big, times) - want_big) / want_big) < 1e-2
    assert p.faults() == 0
    # the library's own exchange memory is shared by pipelines that all wrap at the default period: this one may not use it
    S = torch.zeros((8, 256), dtype=torch.float32, device="cuda")
    with pytest.raises(gpu.GernError, match="GERN_QK_TAG_PERIOD"):
        p(_dev(small[0].view(np.int16)), _dev(small[1].view(np.int16)), S, scale, no_alloc=True)


# The second shape splits a row block over two rounds of dispatch: 30 row blocks of 10 tiles are 300
# workgroups on 256 compute units, so six tiles of the 26th row block start with the launch and its other four
# only when a compute unit is free again.  With the normal limit the six wait for the four; with no polls
# allowed they are certain to give up.
@pytest.mark.parametrize("M,N,must_give_up", [(1024, 4096, False), (7680, 2560, True)])
def test_qk_softmax_tile_kernel_gives_up_waiting_without_hanging(gpu, oracle, monkeypatch, M, N, must_give_up):
    # With no polls allowed, a wavefront that does not find the statistics of
    # the whole row block at its first look gives up and stores NaN in its
    # rows: the launch still finishes, every row is either right or NaN, and
    # the next launch (with the normal limit) is right everywhere.
    import torch
    D = 128
    qb, qv = oracle.to_bf16(oracle.normal((M, D), 5))
    kb, kv = oracle.to_bf16(oracle.normal((N, D), 6))
    scale = np.float32(1.0 / np.sqrt(D))
    if M <= 1024:
        want = oracle.qk_softmax(qb, kb, scale)
    else:  # fp64 of the same bf16 values (the kernel is within 1e-5 of it, the oracle within 1e-2)
        logits = (qv.astype(np.float64) @ kv.T.astype(np.float64)) * float(scale)
        e = np.exp(logits - logits.max(axis=1, keepdims=True))
        want = (e / e.sum(axis=1, keepdims=True)).astype(np.float32)
        del logits, e
    p = gpu.QKSoftmax(D, 4096)
    dq, dk = _dev(qb.view(np.int16)), _dev(kb.view(np.int16))
    S = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    monkeypatch.setenv("GERN_QK_SPIN_LIMIT", "0")
    p(dq, dk, S, scale)
    torch.cuda.synchronize()
    got = S.cpu().numpy()
    bad = np.isnan(got)
    assert np.all(np.abs(got[~bad] - want[~bad]) / want[~bad] < 1e-2)
    # NaNs come as whole 256-column pieces of rows (one wavefront's rows of one tile)
    assert np.array_equal(bad, np.repeat(bad[:, ::256], 256, axis=1))
    # the host learns of it without scanning S: one count per wavefront that gave up (32 rows x 256 columns
    # each), read and cleared by the query
    gave_up = int(bad[::32, ::256].sum())
    assert p.faults() == gave_up
    assert p.faults() == 0
    assert gave_up > 0 or not must_give_up
    # a limit that is not a whole number in range is refused, not read as 0
    for garbage in ("-1", "many", "12x", "99999999999"):
        monkeypatch.setenv("GERN_QK_SPIN_LIMIT", garbage)
        with pytest.raises(gpu.GernError, match="GERN_QK_SPIN_LIMIT"):
            p(dq, dk, S, scale)
    monkeypatch.delenv("GERN_QK_SPIN_LIMIT")
    p(dq, dk, S, scale)
    torch.cuda.synchronize()
    got = S.cpu().numpy()
    assert np.max(np.abs(got - want) / want) < 1e-2
    assert p.faults() == 0


def test_qk_softmax_tile_kernel_reports_logits_that_do_not_fit(gpu, oracle):
    # A row statistic travels as a sixteen-bit shift: logits beyond 32767 in log2 units (or not a number)
    # cannot be exchanged, their rows come back NaN, and the pipeline counts the (row, block of 256 keys)
    # pairs; rows that fit are untouched.
    import torch
    M, N, D = 64, 512, 64
    q = oracle.normal((M, D), 91)
    k = oracle.normal((N, D), 92)
    q[5, :] = 256.0          # row 5 against key 7: 64 * 256 * 256 * scale, far beyond the range
    k[7, :] = 256.0
    k[300, 3] = np.nan       # one key that poisons every row's second block of 256 keys
    qb, _ = oracle.to_bf16(q)
    kb, _ = oracle.to_bf16(k)
    p = gpu.QKSoftmax(D, N)
    S = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, np.float32(1.0))
    torch.cuda.synchronize()
    got = S.cpu().numpy()
    assert np.all(np.isnan(got))  # the NaN key reaches every row's sum
    assert p.faults() == M + 1    # every row's second block, and row 5's first
    assert p.faults() == 0
    kb[300, 3] = 0
    p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, np.float32(1.0))
    torch.cuda.synchronize()
    got = S.cpu().numpy()
    assert np.all(np.isnan(got[5])) and not np.any(np.isnan(np.delete(got, 5, axis=0)))
    assert p.faults() == 1


def test_qk_softmax_full_size(gpu, oracle):
    M = N = 4096
    D = 128
    qb, qv = oracle.to_bf16(oracle.normal((M, D), 5))
    kb, kv = oracle.to_bf16(oracle.normal((N, D), 6))
    scale = np.float32(1.0 / np.sqrt(D))
    got = _run_qk(gpu, qb, kb, scale, 4096)
    # against the oracle (the CPU pipeline: sequential fp32 sums, expf): first and last row blocks, a seam
    for r0 in (0, 2049, 4096 - 16):
        want = oracle.qk_softmax(qb, kb, scale, rows=(r0, r0 + 16))[r0:r0 + 16]
        assert np.max(np.abs(got[r0:r0 + 16] - want) / want) < 1e-2
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5)
    # EVERY row against the exact result: softmax in fp64 of the fp64 product of
    # the same bf16 values.  The kernel differs from it by the fp32 summation
    # of 128 exact products per logit, one v_exp_f32 and one fp32 row sum, so
    # the bound is the softmax stage's 1e-5, not the bf16 GEMM's 1e-2.
    worst = 0.0
    for r0 in range(0, M, 512):
        logits = (qv[r0:r0 + 512].astype(np.float64) @ kv.T.astype(np.float64)) * float(scale)
        e = np.exp(logits - logits.max(axis=1, keepdims=True))
        exact = e / e.sum(axis=1, keepdims=True)
        worst = max(worst, float(np.max(np.abs(got[r0:r0 + 512] - exact) / exact)))
    print("qk softmax 4096x4096x128: max relative error against fp64 = %.3g" % worst)
    assert worst < 1e-5


def test_qk_softmax_wide_logit_spread(gpu, oracle):
    # With scale 2 the logits of a row spread over more than 200, so many
    # probabilities fall below 2^-126.  The kernel computes exp as v_exp_f32 of
    # logits held in log2 units, which returns 0 where expf on the CPU returns
    # a subnormal number: there the two differ by at most the smallest normal
    # number, everywhere else by the usual relative bound.
    M, N, D = 64, 2048, 128
    qb, _ = oracle.to_bf16(oracle.normal((M, D), 15))
    kb, _ = oracle.to_bf16(oracle.normal((N, D), 16))
    scale = np.float32(2.0)
    got = _run_qk(gpu, qb, kb, scale, 2048)
    want = oracle.qk_softmax(qb, kb, scale)
    assert np.any((want > 0) & (want < 2.0 ** -126)) and np.any(want > 0.5)
    assert np.all(np.isfinite(got)) and np.all(got >= 0)
    assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-2 * want.astype(np.float64) + 2.0 ** -126)
    assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5)


def test_qk_softmax_argument_errors(gpu):
    import torch
    p = gpu.QKSoftmax(64, 512)
    q = torch.zeros((16, 64), dtype=torch.int16, device="cuda")
    k = torch.zeros((1024, 64), dtype=torch.int16, device="cuda")
    with pytest.raises(gpu.GernError, match="max_keys"):
        p(q, k, torch.zeros((16, 1024), device="cuda"), 1.0)
    buf = torch.zeros(16 * 64 + 8, dtype=torch.int16, device="cuda")
    with pytest.raises(gpu.GernError, match="aligned"):
        p(buf[1:1 + 16 * 64].view(16, 64), k[:512], torch.zeros((16, 512), device="cuda"), 1.0)


# ------------------------------------------------- code-object cache ----
def test_kernel_loaded_from_the_code_object_cache_runs(gpu, tmp_path, monkeypatch):
    import ctypes as C
    import torch
    monkeypatch.setenv("GERN_HIP_CACHE_DIR", str(tmp_path))
    hip = gpu.hip_lib()
    src = b"template<int N> __global__ void scale(float *p) { p[threadIdx.x] = p[threadIdx.x] * N + 1.0f; }\n"
    names = (C.c_char_p * 1)(b"scale<3>")
    x = torch.arange(64, dtype=torch.float32, device="cuda")
    expect = x.cpu().numpy()
    for attempt in range(2):  # the first compiles and stores, the second loads the stored code object
        mod, k = C.c_void_p(), C.c_void_p()
        assert hip.gern_hip_compile(src, names, 1, None, 0, None, C.byref(mod)) == 0
        assert len(list(tmp_path.iterdir())) == 1
        assert hip.gern_hip_get_kernel(mod, b"scale<3>", C.byref(k)) == 0
        grid, block = (C.c_uint32 * 3)(1, 1, 1), (C.c_uint32 * 3)(64, 1, 1)
        ptr = C.c_void_p(x.data_ptr())
        params = (C.c_void_p * 1)(C.cast(C.pointer(ptr), C.c_void_p))
        assert hip.gern_hip_launch(k, grid, block, 0, params, None) == 0
        torch.cuda.synchronize()
        expect = expect * 3 + 1
        assert np.array_equal(x.cpu().numpy(), expect), attempt


def test_destroying_pipelines_frees_their_code_objects(gpu, oracle):
    # a server that creates and destroys pipelines must not pile up loaded
    # modules: destroy waits for the device and unloads them
    import gc
    import torch
    x = oracle.normal((8, 1024), 3, 0.0, 2.0)
    dx = _dev(x)
    want = oracle.softmax_rows(x)

    def once():
        sm = gpu.Softmax(1024)
        out = torch.empty_like(dx)
        sm(dx, out)          # still in flight when the pipeline goes away
        del sm
        gc.collect()
        torch.cuda.synchronize()
        assert np.max(np.abs(out.cpu().numpy() - want) / want) < 1e-5

    for _ in range(3):
        once()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(40):
        once()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_before - free_after < 32 * 2 ** 20, (free_before, free_after)


# ------------------------------------------------------------- LDS allocator ----
def test_lds_allocator_is_a_stack_that_takes_releases_in_any_order(gpu):
    # gernels/lds_alloc.h: blocks come from the top of a stack; a block released out of order gives its
    # space back when the blocks above it are released too; requests that do not fit are counted.
    import ctypes as C
    import os
    import torch
    src = rb"""
#include "gernels/lds_alloc.h"
extern "C" __global__ void __launch_bounds__(256) lds_alloc_sequence(unsigned int *out, long long bytes) {
    using namespace gernels;
    lds_init(bytes);
    unsigned char *base = gern_lds;
    auto note = [&](int slot, unsigned int v) { if (threadIdx.x == 5) out[slot] = v; };
    void *a = lds_alloc(1000);   // 1008 bytes after the 128-byte table
    void *b = lds_alloc(64);
    void *c = lds_alloc(16);
    note(0, (unsigned int)((unsigned char *)a - base));
    note(1, (unsigned int)((unsigned char *)b - base));
    note(2, (unsigned int)((unsigned char *)c - base));
    __syncthreads();
    note(3, lds_in_use());
    lds_free(b);                 // out of order: c is still above it
    void *d = lds_alloc(32);     // goes above c, not into the hole
    note(4, (unsigned int)((unsigned char *)d - base));
    lds_free(d);
    lds_free(c);                 // now b's hole is at the top too: the stack falls back to the end of a
    void *e = lds_alloc(48);
    note(5, (unsigned int)((unsigned char *)e - base));
    lds_free(a);                 // a lies below e: stays until e goes
    lds_free(e);
    void *f = lds_alloc(4096);   // the whole heap again
    note(6, (unsigned int)((unsigned char *)f - base));
    note(7, lds_overflowed() ? 1u : 0u);
    lds_free(f);
    void *g = lds_alloc(bytes);  // cannot fit (the table takes 128 bytes): start of the heap, counted
    note(8, (unsigned int)((unsigned char *)g - base));
    __syncthreads();
    note(9, lds_overflowed() ? 1u : 0u);
    note(10, gern_lds_overflows);
}
"""
    hip = gpu.hip_lib()
    opts = (C.c_char_p * 1)(("-I" + os.path.dirname(os.path.abspath(gpu.__file__))).encode())
    names = (C.c_char_p * 1)(b"lds_alloc_sequence")
    mod, k = C.c_void_p(), C.c_void_p()
    assert hip.gern_hip_compile(src, names, 1, opts, 1, None, C.byref(mod)) == 0, gpu._hip_error()
    assert hip.gern_hip_get_kernel(mod, b"lds_alloc_sequence", C.byref(k)) == 0
    out = torch.zeros(16, dtype=torch.int32, device="cuda")
    lds = 8192
    ptr, nbytes = C.c_void_p(out.data_ptr()), C.c_longlong(lds)
    params = (C.c_void_p * 2)(C.cast(C.pointer(ptr), C.c_void_p), C.cast(C.pointer(nbytes), C.c_void_p))
    grid, block = (C.c_uint32 * 3)(1, 1, 1), (C.c_uint32 * 3)(256, 1, 1)
    assert hip.gern_hip_launch(k, grid, block, lds, params, None) == 0, gpu._hip_error()
    torch.cuda.synchronize()
    got = out.cpu().numpy().tolist()
    assert got[0:3] == [128, 128 + 1008, 128 + 1008 + 64]
    assert got[3] == 1008 + 64 + 16
    assert got[4] == 128 + 1008 + 64 + 16          # above c
    assert got[5] == 128 + 1008                    # b's and c's space is back
    assert got[6] == 128 and got[7] == 0           # everything released: the heap starts over
    assert got[8] == 128 and got[9] == 1 and got[10] == 1
