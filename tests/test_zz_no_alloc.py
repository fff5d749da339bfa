"""gern_qk_softmax_run_no_alloc: the QK^T softmax with its exchange memory in a
device array of the library.  Checked through the C ABI against
gern_qk_softmax_run on the same inputs (both run the same kernel, so every bit
agrees), on two calls in a row, the second with a smaller input; then against
the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_no_alloc_entry_point_matches_the_allocating_one(oracle):
    import torch
    import gern_amd
    if gern_amd.device_count() < 1 or not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests must run on an MI355X box")
    D = 128
    p = gern_amd.QKSoftmax(D, 4096)
    assert "view_score_tile" in p.source  # the kernel that uses exchange memory
    scale = np.float32(1.0 / np.sqrt(D))
    # No set-up call: gern_qk_softmax_create has looked the device array up (the runtime loads the library's
    # code object then), so already the FIRST run through the entry point takes no device memory.
    for (M, N) in ((1000, 4096), (300, 700)):  # the second call is smaller: entries of the first stay behind
        qb, _ = oracle.to_bf16(oracle.normal((M, D), 11 + M))
        kb, _ = oracle.to_bf16(oracle.normal((N, D), 12 + N))
        dq = torch.from_numpy(qb.view(np.int16)).cuda()
        dk = torch.from_numpy(kb.view(np.int16)).cuda()
        a = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        b = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info()
        p(dq, dk, a, scale, no_alloc=True)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_before - free_after < 2 ** 20, (free_before, free_after)  # the call took no device memory
        p(dq, dk, b, scale)
        torch.cuda.synchronize()
        got, ref = a.cpu().numpy(), b.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (M, N)
        want = oracle.qk_softmax(qb, kb, scale)
        assert np.max(np.abs(got - want) / want) < 1e-2, (M, N)
    assert p.faults() == 0  # reads the counters of the pipeline's own memory and of the library's
    # sizes beyond the array are refused, not truncated
    big_q = torch.zeros((16385, D), dtype=torch.int16, device="cuda")
    big_k = torch.zeros((4096, D), dtype=torch.int16, device="cuda")
    out = torch.zeros((16385, 4096), dtype=torch.float32, device="cuda")
    with pytest.raises(gern_amd.GernError, match="GERN_QK_SCRATCH_BYTES"):
        p(big_q, big_k, out, scale, no_alloc=True)
    # a pipeline whose kernel exchanges nothing (sixteen whole rows per workgroup) takes the same call
    q = gern_amd.QKSoftmax(96, 512)
    qb, _ = oracle.to_bf16(oracle.normal((40, 96), 3))
    kb, _ = oracle.to_bf16(oracle.normal((500, 96), 4))
    s = torch.full((40, 500), float("nan"), dtype=torch.float32, device="cuda")
    q(torch.from_numpy(qb.view(np.int16)).cuda(), torch.from_numpy(kb.view(np.int16)).cuda(), s, np.float32(0.1), no_alloc=True)
    torch.cuda.synchronize()
    want = oracle.qk_softmax(qb, kb, np.float32(0.1))
    assert np.max(np.abs(s.cpu().numpy() - want) / want) < 1e-2
