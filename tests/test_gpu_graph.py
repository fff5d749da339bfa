"""Pipelines recorded into a HIP graph: a run is one kernel launch on the
caller's stream (no allocation, no synchronisation, no memset), so it can be
captured and replayed.  Every replay is checked against the oracle, with eager
work and synchronisations between the replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_pipelines_replay_from_a_hip_graph(oracle):
    import torch
    import gern_amd as gpu
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests must run on an MI355X box")

    blur = gpu.BlurChain("xyx", tile_rows=6)
    sm = gpu.Softmax(1024)
    gemm = gpu.Gemm("bf16", overwrite=True)
    # the 256 x 256 tile kernel: two row blocks x two column blocks exchange row statistics through device
    # memory; its launch number lives there too, so a replay is a launch like any other
    qk = gpu.QKSoftmax(128, 512)
    m_q, n_k, d_h = 300, 512, 128
    shape_img, shape_x, n = (200, 520), (48, 1024), 256
    d_img = torch.zeros(shape_img, device="cuda")
    d_blur = torch.zeros(blur.out_shape(*shape_img), device="cuda")
    d_x = torch.zeros(shape_x, device="cuda")
    d_y = torch.zeros(shape_x, device="cuda")
    d_a = torch.zeros((n, n), dtype=torch.int16, device="cuda")
    d_b = torch.zeros((n, n), dtype=torch.int16, device="cuda")
    d_c = torch.zeros((n, n), device="cuda")
    d_q = torch.zeros((m_q, d_h), dtype=torch.int16, device="cuda")
    d_k = torch.zeros((n_k, d_h), dtype=torch.int16, device="cuda")
    d_s = torch.zeros((m_q, n_k), device="cuda")
    scale = np.float32(1.0 / np.sqrt(d_h))

    side = torch.cuda.Stream()  # default priority

    def record():
        h = side.cuda_stream
        blur(d_img, d_blur, stream=h)
        sm(d_x, d_y, stream=h)
        gemm(d_a, d_b, d_c, stream=h)
        qk(d_q, d_k, d_s, scale, stream=h)

    # everything that loads code or queries the device happens before capture
    with torch.cuda.stream(side):
        record()
    side.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        record()

    for rep in range(3):
        img = oracle.uniform(shape_img, 100 + rep)
        x = oracle.normal(shape_x, 200 + rep, 0.0, 2.0)
        ai = np.random.RandomState(300 + rep).randint(-3, 4, size=(n, n)).astype(np.float32)
        bi = np.random.RandomState(400 + rep).randint(-3, 4, size=(n, n)).astype(np.float32)
        ab, _ = oracle.to_bf16(ai)
        bb, _ = oracle.to_bf16(bi)
        # eager work between replays: new inputs, poisoned outputs
        d_img.copy_(torch.from_numpy(img))
        d_x.copy_(torch.from_numpy(x))
        d_a.copy_(torch.from_numpy(ab.view(np.int16)))
        d_b.copy_(torch.from_numpy(bb.view(np.int16)))
        qb, _ = oracle.to_bf16(oracle.normal((m_q, d_h), 500 + rep))
        kb, _ = oracle.to_bf16(oracle.normal((n_k, d_h), 600 + rep))
        d_q.copy_(torch.from_numpy(qb.view(np.int16)))
        d_k.copy_(torch.from_numpy(kb.view(np.int16)))
        for out in (d_blur, d_y, d_c, d_s):
            out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(d_blur.cpu().numpy(), oracle.blur_chain(img, "xyx")), rep
        want = oracle.softmax_rows(x)
        assert np.max(np.abs(d_y.cpu().numpy() - want) / want) < 1e-5, rep
        assert np.array_equal(d_c.cpu().numpy(), ai @ bi), rep
        want = oracle.qk_softmax(qb, kb, scale)
        got = d_s.cpu().numpy()
        assert np.all(np.isfinite(got)), rep
        assert np.max(np.abs(got - want) / want) < 1e-2, rep
