"""GPU: rfq_upload (host bytes -> device through the pinned staging ring) delivers every byte, for
sizes around the 8 MiB slot and the 4-slot ring, on two streams, and after the ring was released;
rfq_dequant_upload and rfq_matmul_host_weights, which upload through it, still match the oracle."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bit_exact, assert_close
from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu
SLOT = 8 << 20


def pattern(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(0, 256, size=n, dtype=np.uint8)


@pytest.mark.parametrize("n", [0, 1, 4097, SLOT - 1, SLOT, SLOT + 1, 2 * SLOT + 12345, 4 * SLOT, 9 * SLOT + 7])
def test_every_byte_arrives(n, cuda):
    import torch
    from rocmforge_amd import ops
    src = pattern(n, n % 1000)
    out = ops.upload(src, torch.zeros(n, dtype=torch.uint8, device=cuda))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), src)


def test_source_may_be_overwritten_after_return_and_streams_alternate(cuda):
    import torch
    from rocmforge_amd import ops
    n = 3 * SLOT + 999
    streams = [torch.cuda.Stream(device=cuda), torch.cuda.Stream(device=cuda)]
    outs, wants = [], []
    src = pattern(n, 1)
    for i in range(4):
        with torch.cuda.stream(streams[i % 2]):
            wants.append(src.copy())
            outs.append(ops.upload(src))
        src[:] = pattern(n, 2 + i)                                       # the call has taken its copy
    torch.cuda.synchronize()
    for out, want in zip(outs, wants):
        assert np.array_equal(out.cpu().numpy(), want)


def test_ring_is_rebuilt_after_release(cuda):
    import torch
    from rocmforge_amd import _lib, ops
    src = pattern(SLOT + 5, 3)
    a = ops.upload(src)
    torch.cuda.synchronize()
    assert _lib.lib().rfq_release_temporaries() == _lib.OK
    b = ops.upload(src)
    torch.cuda.synchronize()
    assert np.array_equal(a.cpu().numpy(), src) and np.array_equal(b.cpu().numpy(), src)


def test_rejects_null_pointers(cuda):
    from rocmforge_amd import _lib
    L = _lib.lib()
    assert L.rfq_upload(None, 16, C.c_void_p(16), None) == _lib.E_BADARG
    assert L.rfq_upload(C.c_void_p(16), 16, None, None) == _lib.E_BADARG
    assert L.rfq_upload(None, 0, None, None) == _lib.OK


def test_dequant_upload_and_host_weight_matmul_through_the_ring(oracle, cuda):
    """20 MiB of packed Q4_K weights: several slots per call."""
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    fmt, n, k = Q.Q4_K, 5120, 4096
    w = Q.make_weights(fmt, n, k, seed=77)
    out = torch.empty(n * k, dtype=torch.float32, device=cuda)
    _lib.check(L.rfq_dequant_upload(fmt, C.c_void_p(w.ctypes.data), w.size, C.c_void_p(out.data_ptr()), n * k, None))
    assert_bit_exact(out.cpu().numpy(), oracle.dequantize(fmt, w, n * k), "dequant_upload")
    x = np.random.Generator(np.random.PCG64(78)).standard_normal(k, dtype=np.float32)
    dx, dy = torch.from_numpy(x).to(cuda), torch.empty(n, dtype=torch.float32, device=cuda)
    _lib.check(L.rfq_matmul_host_weights(fmt, C.c_void_p(w.ctypes.data), w.size, C.c_void_p(dx.data_ptr()), n, k,
                                         C.c_void_p(dy.data_ptr()), None))
    assert_close(dy.cpu().numpy(), oracle.qmatmul_nk(fmt, w, x, 1, n, k)[0], "matmul_host_weights")
