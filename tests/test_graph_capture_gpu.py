"""GPU: the enqueue-only entry points can be captured into a HIP graph and
replayed (a decode step is a fixed sequence of launches): every replay is
checked against the eager result for the inputs it ran on."""
import numpy as np
import pytest

from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu


def test_gemv_sequence_replays(cuda):
    import torch
    from rocmforge_amd import ops
    n, k = 512, 2048
    fmts = [Q.Q4_K, Q.Q8_0, Q.MXFP4, Q.Q6_K]
    ws = [torch.from_numpy(Q.make_weights(f, n, k, seed=40 + f)).to(cuda) for f in fmts]
    x = torch.zeros(k, device=cuda)
    xb = torch.zeros((4, k), device=cuda)
    ys = [torch.empty((1, n), device=cuda) for _ in fmts]
    yb = torch.empty((4, n), device=cuda)

    def step():
        for f, w, y in zip(fmts, ws, ys):
            ops.gemv(f, w, x, n, k, out=y)
        ops.gemv(Q.Q8_0, ws[1], xb, n, k, out=yb)          # the batched matrix-core kernel (uses the kept temporary)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()                                             # first use on this stream allocates the kept temporary
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    gen = torch.Generator(device="cpu").manual_seed(5)
    for _ in range(3):
        x.copy_(torch.randn(k, generator=gen))
        xb.copy_(torch.randn(4, k, generator=gen))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [y.clone() for y in ys] + [yb.clone()]
        step()                                             # eager, same inputs
        torch.cuda.synchronize()
        want = ys + [yb]
        for g, w_ in zip(got, want):
            assert torch.equal(g, w_)


def test_prefill_gemms_replay(cuda):
    import torch
    from rocmforge_amd import _lib, ops
    m, n, k = 96, 256, 512
    w = torch.from_numpy(Q.make_weights(Q.Q4_K, n, k, seed=3)).to(cuda)
    a = torch.zeros((m, k), dtype=torch.float16, device=cuda)
    out = torch.empty((m, n), dtype=torch.float16, device=cuda)
    rng = np.random.default_rng(4)
    gauss = lambda r, std: (rng.standard_normal((r, k), dtype=np.float32) * np.float32(std))
    A = ops.MxOperand(Q.MXFP4, torch.from_numpy(Q.pack_mxfp4(gauss(m, 1.0))).to(cuda), m, k)
    W = ops.MxOperand(Q.MXFP4, torch.from_numpy(Q.pack_mxfp4(gauss(n, 0.02))).to(cuda), n, k)
    out_mx = torch.empty((m, n), dtype=torch.bfloat16, device=cuda)

    def step():
        ops.gemm_f16(Q.Q4_K, w, a, n, k, out_dtype=torch.float16, out=out)
        ops.gemm_mx(A, W, out_dtype=torch.bfloat16, out=out_mx)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()                                             # the temporary is kept per stream: warm this one too
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    for seed in (1, 2, 3):
        a.copy_(torch.from_numpy(np.random.default_rng(seed).standard_normal((m, k)).astype(np.float16)))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got, got_mx = out.clone(), out_mx.clone()
        step()
        torch.cuda.synchronize()
        assert torch.equal(got, out) and torch.equal(got_mx, out_mx)


def test_capture_refuses_to_allocate_temporaries(cuda):
    """A stream that has never run the call has no kept temporary: under capture the call must fail with
    RFQ_E_UNSUPPORTED instead of allocating (or growing, which would free memory an earlier graph holds)."""
    import torch
    from rocmforge_amd import _lib, ops
    m, n, k = 64, 128, 512
    w = torch.from_numpy(Q.make_weights(Q.Q4_K, n, k, seed=8)).to(cuda)
    a = torch.zeros((m, k), dtype=torch.float16, device=cuda)
    a2 = torch.zeros((4 * m, k), dtype=torch.float16, device=cuda)
    out = torch.empty((m, n), dtype=torch.float16, device=cuda)
    out2 = torch.empty((4 * m, n), dtype=torch.float16, device=cuda)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        ops.gemm_f16(Q.Q4_K, w, a, n, k, out=out)          # the stream now keeps a temporary for m = 64
        torch.cuda.synchronize()
        refused = None
        with torch.cuda.graph(graph, stream=side):
            ops.gemm_f16(Q.Q4_K, w, a, n, k, out=out)      # fits: captured
            try:
                ops.gemm_f16(Q.Q4_K, w, a2, n, k, out=out2)  # four times the rows: would have to grow
            except _lib.RfqError as e:
                refused = e
    assert refused is not None and refused.status == _lib.E_UNSUPPORTED and "captur" in refused.message
    a.copy_(torch.from_numpy(np.random.default_rng(9).standard_normal((m, k)).astype(np.float16)))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    got = out.clone()
    # growing afterwards (eagerly) must leave the captured graph's buffer alive: replay again and compare
    with torch.cuda.stream(side):
        ops.gemm_f16(Q.Q4_K, w, a2, n, k, out=out2)
        torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, got)
    want = ops.gemm_f16(Q.Q4_K, w, a, n, k)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
