"""GPU: rfq_gemm_f16_static, the entry point that allocates nothing, against rfq_gemm_f16: same kernels, so the
outputs must be bit-identical; two calls in a row on the library's static device array, the second smaller (the
array keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest

from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fmt", [Q.Q4_K, Q.GGUF_Q4_K, Q.Q8_0])
def test_static_scratch_gemm_matches_the_allocating_entry_point(fmt, cuda):
    import torch
    from rocmforge_amd import _lib, ops
    for (m, n, k) in [(300, 384, 1024), (70, 130, 512)]:       # second call: smaller in every dimension, ragged m and n
        w = torch.from_numpy(Q.make_weights(fmt, n, k, seed=900 + fmt + m)).to(cuda)
        a = torch.from_numpy(np.random.default_rng(901 + m).standard_normal((m, k)).astype(np.float16)).to(cuda)
        for out_dtype in (torch.float16, torch.float32):
            want = ops.gemm_f16(fmt, w, a, n, k, out_dtype=out_dtype)
            got = torch.full((m, n), float("nan"), dtype=out_dtype, device=cuda)
            ops.gemm_f16_static(fmt, w, a, n, k, out=got, out_dtype=out_dtype)
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"{Q.NAMES[fmt]} {m}x{n}x{k} {out_dtype}"


def test_static_scratch_limit_is_reported(cuda):
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    m, n, k = 4096, 32, 4096                                   # 32 MiB of arranged activations: beyond the 16 MiB array
    w = torch.zeros(n * k // 256 * 256, dtype=torch.uint8, device=cuda)
    a = torch.zeros((m, k), dtype=torch.float16, device=cuda)
    out = torch.zeros((m, n), dtype=torch.float16, device=cuda)
    rc = L.rfq_gemm_f16_static(Q.Q4_K, C.c_void_p(w.data_ptr()), w.numel(), C.c_void_p(a.data_ptr()),
                               C.c_void_p(out.data_ptr()), _lib.F16, m, n, k, None)
    assert rc == _lib.E_SIZE and b"static buffer" in L.rfq_last_error()
    torch.cuda.synchronize()


def test_static_scratch_call_allocates_nothing(cuda):
    """The property the entry point exists for.  On a stream the library has never seen, rfq_gemm_f16 has to allocate
    its kept temporary (so under capture it refuses), while rfq_gemm_f16_static must neither change the device's free
    memory nor refuse to be captured; the captured call replays to the eager result."""
    import torch
    from rocmforge_amd import _lib, ops
    L = _lib.lib()
    fmt, m, n, k = Q.GGUF_Q4_K, 512, 256, 2048
    w = torch.from_numpy(Q.make_weights(fmt, n, k, seed=77)).to(cuda)
    a = torch.zeros((m, k), dtype=torch.float16, device=cuda)
    out = torch.empty((m, n), dtype=torch.float16, device=cuda)
    ops.gemm_f16_static(fmt, w, a, n, k, out=out)               # resolves the array's address: outside capture, once per device
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    args = (fmt, C.c_void_p(w.data_ptr()), w.numel(), C.c_void_p(a.data_ptr()), C.c_void_p(out.data_ptr()), _lib.F16, m, n, k,
            C.c_void_p(side.cuda_stream))
    free_before = torch.cuda.mem_get_info()[0]
    assert L.rfq_gemm_f16_static(*args) == _lib.OK
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before           # 2.1 MiB of temporaries would show
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            # the allocating entry point has no buffer on this stream and may not create one now
            assert L.rfq_gemm_f16(*args) == _lib.E_UNSUPPORTED
            assert L.rfq_gemm_f16_static(*args) == _lib.OK
    gen = torch.Generator(device="cpu").manual_seed(6)
    for _ in range(3):
        a.copy_(torch.randn(m, k, generator=gen).to(torch.float16))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = ops.gemm_f16(fmt, w, a, n, k)                     # eager, current stream, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got, want)
