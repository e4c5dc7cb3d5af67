"""GPU parity: rfq_dequant* against the CPU oracle, bit for bit."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bit_exact
from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu

FORMATS = [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3, Q.MXFP6_E3M2]


def gpu_dequant(fmt, data, n, cuda):
    import torch
    from rocmforge_amd import ops
    d = torch.from_numpy(np.ascontiguousarray(data)).to(cuda)
    out = ops.dequant(fmt, d, n)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("fmt", FORMATS)
def test_random_blocks_all_codes(fmt, oracle, cuda):
    rng = np.random.default_rng(1000 + fmt)
    nb = 4099                                     # odd block count, several workgroups
    data = Q.random_blocks(fmt, nb, rng, exp_range=(-128, 127))
    n = nb * Q.BLOCK_ELEMS[fmt]
    assert_bit_exact(gpu_dequant(fmt, data, n, cuda), oracle.dequantize(fmt, data, n), Q.NAMES[fmt])


@pytest.mark.parametrize("fmt", FORMATS)
def test_ragged_element_count_and_short_input(fmt, oracle, cuda):
    rng = np.random.default_rng(2000 + fmt)
    be, bb = Q.BLOCK_ELEMS[fmt], Q.BLOCK_BYTES[fmt]
    data = Q.random_blocks(fmt, 9, rng, exp_range=(-6, 6))
    for n in (1, 3, be - 1, be + 1, 5 * be + 7, 9 * be - 3, 9 * be):
        assert_bit_exact(gpu_dequant(fmt, data, n, cuda), oracle.dequantize(fmt, data, n), f"{Q.NAMES[fmt]} n={n}")
    n = 9 * be
    for cut in (0, 1, 3, 4, 5, bb - 1, bb, bb + 1, bb + 4, bb + 9, 4 * bb + bb // 2, 9 * bb - 1):
        got = gpu_dequant(fmt, data[:cut], n, cuda)
        want = oracle.dequantize(fmt, data[:cut], n)
        assert_bit_exact(got, want, f"{Q.NAMES[fmt]} bytes={cut}")


def test_reference_vectors_on_gpu(cuda):
    # byte patterns of src/kernels/quant/q4_0.rs:338-362, q8_0.rs:99-120 and the
    # GPU parity recipes of tests/q_dequant_tests.rs
    d = np.zeros(20, np.uint8); d[0:4] = np.frombuffer(np.float32(2.0).tobytes(), np.uint8)
    d[4:] = [(((i + 1) << 4) | i) & 0xFF for i in range(16)]
    r = gpu_dequant(Q.Q4_0, d, 32, cuda)
    assert r[0] == -16.0 and r[1] == -14.0 and r[30] == 14.0 and r[31] == -16.0
    d = np.zeros(36, np.uint8); d[0:4] = np.frombuffer(np.float32(2.0).tobytes(), np.uint8)
    d[4:] = 120 + np.arange(32)
    r = gpu_dequant(Q.Q8_0, d, 32, cuda)
    assert r[0] == -16.0 and r[15] == 14.0 and r[31] == 46.0
    d = np.zeros(256, np.uint8)
    d[0:16] = np.full(8, 1.0, np.float16).view(np.uint8); d[32:] = 0x88
    assert np.all(gpu_dequant(Q.Q4_K, d, 100, cuda) == 8.0)
    d = np.zeros(256, np.uint8)
    d[0:32] = np.full(16, 1.0, np.float16).view(np.uint8); d[32:224] = 0xFF
    assert np.all(gpu_dequant(Q.Q6_K, d, 256, cuda) == -1.0)
    d = np.zeros(17, np.uint8); d[0] = 1; d[1:] = 0x11              # 2^1 * code 1 (1.0)
    assert np.all(gpu_dequant(Q.MXFP4, d, 32, cuda) == 2.0)


def test_exhaustive_small_domains(oracle, cuda):
    rng = np.random.default_rng(77)
    # MXFP4: 256 exponents x 16 codes; MXFP6: 256 exponents x random payload
    b = np.zeros((256, 17), np.uint8); b[:, 0] = np.arange(256)
    codes = np.tile(np.arange(16, dtype=np.uint8), 2)
    b[:, 1:] = (codes[0::2] << 4) | codes[1::2]
    assert_bit_exact(gpu_dequant(Q.MXFP4, b.ravel(), 8192, cuda), oracle.dequantize(Q.MXFP4, b.ravel(), 8192), "mxfp4")
    b = rng.integers(0, 256, (256 * 16, 25), dtype=np.uint8); b[:, 0] = np.arange(256 * 16) % 256
    assert_bit_exact(gpu_dequant(Q.MXFP6_E2M3, b.ravel(), b.shape[0] * 32, cuda),
                     oracle.dequantize(Q.MXFP6_E2M3, b.ravel(), b.shape[0] * 32), "mxfp6")
    # Q4_K / Q6_K: every finite f16 bit pattern as a scale (NaN payloads are
    # compared as NaN-ness only)
    for fmt, nsc in ((Q.Q4_K, 8), (Q.Q6_K, 16)):
        nb = 65536 // nsc
        b = rng.integers(0, 256, (nb, 256), dtype=np.uint8)
        b[:, 0:2 * nsc] = np.arange(65536, dtype=np.uint16).view(np.uint8).reshape(nb, 2 * nsc)
        got = gpu_dequant(fmt, b.ravel(), nb * 256, cuda)
        want = oracle.dequantize(fmt, b.ravel(), nb * 256)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert_bit_exact(got[~nan], want[~nan], Q.NAMES[fmt])
    # Q4_0 / Q8_0: special scales
    specials = np.array([0.0, -0.0, 1e-45, -1e-40, 3.4e38, np.inf, -np.inf, 1.17549435e-38], np.float32)
    for fmt, bb in ((Q.Q4_0, 20), (Q.Q8_0, 36)):
        b = rng.integers(0, 256, (8, bb), dtype=np.uint8)
        b[:, 0:4] = specials.view(np.uint8).reshape(8, 4)
        got, want = gpu_dequant(fmt, b.ravel(), 256, cuda), oracle.dequantize(fmt, b.ravel(), 256)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert_bit_exact(got[~nan], want[~nan], Q.NAMES[fmt])


@pytest.mark.parametrize("fmt,n,k", [(Q.Q4_0, 4864, 896), (Q.Q8_0, 4096, 4096), (Q.Q4_K, 14336, 4096),
                                     (Q.Q6_K, 14336, 4096), (Q.MXFP4, 2048, 8192), (Q.MXFP6_E2M3, 2048, 8192)])
def test_full_size_tensors(fmt, n, k, oracle, cuda):
    data = Q.make_weights(fmt, n, k, seed=20260000 + fmt)
    got = gpu_dequant(fmt, data, n * k, cuda)
    want = oracle.dequantize(fmt, data, n * k)
    assert_bit_exact(got, want, f"{Q.NAMES[fmt]} {n}x{k}")


def test_unaligned_output_and_input(oracle, cuda):
    import torch
    from rocmforge_amd import ops
    rng = np.random.default_rng(31)
    for fmt in (Q.Q4_0, Q.Q4_K, Q.MXFP4):
        data = Q.random_blocks(fmt, 33, rng, exp_range=(-4, 4))
        n = 33 * Q.BLOCK_ELEMS[fmt]
        base_in = torch.zeros(data.size + 3, dtype=torch.uint8, device=cuda)
        base_in[3:] = torch.from_numpy(data).to(cuda)                # input at a 3-byte offset
        base_out = torch.zeros(n + 1, dtype=torch.float32, device=cuda)
        ops.dequant(fmt, base_in[3:], n, out=base_out[1:])           # output 4-byte aligned only
        torch.cuda.synchronize()
        assert_bit_exact(base_out[1:].cpu().numpy(), oracle.dequantize(fmt, data, n), Q.NAMES[fmt])
        assert base_out[0].item() == 0.0


@pytest.mark.parametrize("fmt", [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3])
def test_host_entry_points(fmt, oracle, cuda):
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(41 + fmt)
    data = Q.random_blocks(fmt, 70, rng, exp_range=(-5, 5))
    n = 70 * Q.BLOCK_ELEMS[fmt] - 5
    want = oracle.dequantize(fmt, data, n)
    out = np.full(n, 7.0, np.float32)
    _lib.check(L.rfq_dequant_host(fmt, data.ctypes.data_as(C.c_void_p), data.size, out.ctypes.data_as(C.c_void_p), n))
    assert_bit_exact(out, want, "rfq_dequant_host")
    d_out = torch.full((n,), 7.0, dtype=torch.float32, device=cuda)
    _lib.check(L.rfq_dequant_upload(fmt, data.ctypes.data_as(C.c_void_p), data.size, C.c_void_p(d_out.data_ptr()), n, None))
    assert_bit_exact(d_out.cpu().numpy(), want, "rfq_dequant_upload")
    short = data[: data.size // 2]
    _lib.check(L.rfq_dequant_host(fmt, short.ctypes.data_as(C.c_void_p), short.size, out.ctypes.data_as(C.c_void_p), n))
    assert_bit_exact(out, oracle.dequantize(fmt, short, n), "rfq_dequant_host short")
