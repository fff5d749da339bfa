"""Seeded random shapes and schedules for every pipeline, against the CPU
oracle: the fixed cases of test_gpu_parity.py were chosen by hand, these were
not.  Same tolerances as there."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch
    import gern_amd
    if gern_amd.device_count() < 1 or not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests must run on an MI355X box")
    return gern_amd


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_blur_random_shapes_patterns_and_tiles(gpu, oracle):
    import torch
    rng = np.random.RandomState(101)
    for case in range(20):
        pattern = "".join(rng.choice(["x", "y"]) for _ in range(rng.randint(1, 5)))
        nx, ny = pattern.count("x"), pattern.count("y")
        rows = int(rng.randint(2 * ny + 1, 260))
        cols = int(rng.randint(2 * nx + 1, 700))
        tile_rows = int(rng.randint(1, 10))
        max_cols = (256 - 2 * nx) // 4 * 4
        tile_cols = int(rng.randint(1, max_cols // 4 + 1)) * 4
        if case % 2 == 1:
            # whole 128-byte lines per tile: windows moved to line boundaries where the halo leaves room
            tile_cols = int(rng.randint(1, max_cols // 32 + 1)) * 32
        waves = int(rng.choice([1, 1, 2, 4]))
        img = oracle.uniform((rows, cols), 200 + case) - np.float32(0.5 if case % 3 == 0 else 0.0)
        if case % 4 == 1:
            img[rng.randint(0, rows), :] = 0.0          # a row of zeros: the exact-division path
        p = gpu.BlurChain(pattern, tile_rows=tile_rows, tile_cols=tile_cols, waves_per_block=waves)
        out = torch.full(p.out_shape(rows, cols), float("nan"), dtype=torch.float32, device="cuda")
        p(_dev(img), out)
        torch.cuda.synchronize()
        want = oracle.blur_chain(img, pattern)
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32)), \
            (case, pattern, rows, cols, tile_rows, tile_cols, waves)


def test_softmax_random_widths_and_rows(gpu, oracle):
    import torch
    rng = np.random.RandomState(102)
    widths = [int(rng.randint(1, 3000)) for _ in range(6)] + [512, 1024, 1280, 1536, 2048, 2560, 3072, 5120, 7168, 8192]
    # rows wider than one wavefront holds: cut into 4, 8 or 16 pieces, evenly or not
    widths += [int(rng.randint(8193, 16385)), int(rng.randint(16385, 32769)), int(rng.randint(32769, 65537)), 24576]
    for case, ncol in enumerate(widths):
        rows = int(rng.randint(1, 70))
        per_wave_chunks = 32
        rpw = int(rng.choice([1, 1, 2, 3]))
        chunks = (ncol + 255) // 256
        if rpw * chunks > per_wave_chunks and not (ncol >= 1024 and ncol % 512 == 0):
            rpw = 1
        if ncol > 8192:
            rpw = 1
        x = oracle.normal((rows, ncol), 300 + case, 0.0, 3.0)
        sm = gpu.Softmax(ncol, rows_per_wave=rpw)
        out = torch.full((rows, ncol), float("nan"), dtype=torch.float32, device="cuda")
        sm(_dev(x), out)
        torch.cuda.synchronize()
        got, want = out.cpu().numpy(), oracle.softmax_rows(x)
        # The oracle sums a row left to right in fp32, as the reference's CPU
        # path does; over thousands of columns that sum itself strays from the
        # exact one by more than the 1e-5 bar in some rows.  So: the kernel is
        # held to 1e-5 against the exact (fp64) result, and to the oracle within
        # 1e-5 plus the oracle's own distance from the exact result.
        x64 = x.astype(np.float64)
        e = np.exp(x64 - x64.max(axis=1, keepdims=True))
        exact = e / e.sum(axis=1, keepdims=True)
        ok = exact > 1e-30
        rel = lambda a, b: np.max(np.abs(a[ok] - b[ok]) / b[ok])  # noqa: E731
        assert rel(got, exact) < 1e-5, (case, rows, ncol, rpw)
        assert rel(got, want) < 1e-5 + rel(want, exact), (case, rows, ncol, rpw)
        assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5), (case, rows, ncol, rpw)


@pytest.mark.parametrize("variant", ["f32", "bf16"])
def test_gemm_random_shapes(gpu, oracle, variant):
    import torch
    rng = np.random.RandomState(103 if variant == "f32" else 104)
    for case in range(10):
        M = int(rng.randint(1, 600))
        N = int(rng.randint(1, 600))
        K = int(rng.randint(1, 700))
        if variant == "bf16":
            N = max(2, N // 2 * 2)
            K = max(8, K // 8 * 8)
            if case % 2 == 0:                 # whole K stages and 16-byte rows of B
                K = max(64, K // 64 * 64)
                N = max(8, N // 8 * 8)
        overwrite = bool(case % 3 == 0)
        ai = rng.randint(-3, 4, size=(M, K)).astype(np.float32)   # exact in any summation order
        bi = rng.randint(-3, 4, size=(K, N)).astype(np.float32)
        c0 = rng.randint(-9, 10, size=(M, N)).astype(np.float32)
        g = gpu.Gemm(variant, overwrite=overwrite)
        dC = _dev(c0)
        if variant == "bf16":
            a_dev = _dev(oracle.to_bf16(ai)[0].view(np.int16))
            b_dev = _dev(oracle.to_bf16(bi)[0].view(np.int16))
        else:
            a_dev, b_dev = _dev(ai), _dev(bi)
        g(a_dev, b_dev, dC)
        torch.cuda.synchronize()
        want = ai.astype(np.float64) @ bi.astype(np.float64) + (0 if overwrite else c0)
        assert np.array_equal(dC.cpu().numpy().astype(np.float64), want), (case, M, N, K, overwrite, g.kernel_name)


def test_qk_softmax_random_shapes(gpu, oracle):
    import torch
    rng = np.random.RandomState(105)
    for case in range(12):
        D = int(rng.choice([32, 64, 96, 128, 160, 256]))
        max_keys = int(rng.choice([256, 512, 1024, 2048]))
        N = int(rng.randint(1, max_keys + 1))
        M = int(rng.randint(1, 80)) if case < 8 else int(rng.randint(200, 800))  # the last four: several row blocks
        qb, _ = oracle.to_bf16(oracle.normal((M, D), 400 + case))
        kb, _ = oracle.to_bf16(oracle.normal((N, D), 500 + case))
        scale = np.float32(1.0 / np.sqrt(D))
        p = gpu.QKSoftmax(D, max_keys)
        S = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        p(_dev(qb.view(np.int16)), _dev(kb.view(np.int16)), S, scale)
        torch.cuda.synchronize()
        got, want = S.cpu().numpy(), oracle.qk_softmax(qb, kb, scale)
        assert np.max(np.abs(got - want) / want) < 1e-2, (case, M, N, D, max_keys)
        assert np.all(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0) < 1e-5), (case, M, N, D, max_keys)
