"""GPU parity for the matmul module's own decoders (RFQ_MM_Q8_0 / MM_Q4_K / MM_Q6_K:
src/kernels/matmul/quantized/q8_0.rs:18-56, q4_k.rs:90-148, q6_k.rs:90-148) and for the orientation the
reference's matmuls compute, y[j] = sum_l x[l] * Wd[l * n + j] (rfq_gemv_kn: kernels/q4_0_matmul.hip:207,
quantized/q4_0.rs:274-311 + src/tensor/matmul.rs:219-233), against the CPU oracle."""
import ctypes as C
import struct

import numpy as np
import pytest

from helpers import assert_bit_exact, assert_close
from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu

MM = [Q.MM_Q8_0, Q.MM_Q4_K, Q.MM_Q6_K]
KN_FORMATS = [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3, Q.GGUF_Q4_0, Q.GGUF_Q8_0, Q.GGUF_Q4_K, Q.GGUF_Q6_K] + MM


def dev(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


@pytest.mark.parametrize("fmt", MM)
def test_mm_dequant_bit_exact(fmt, oracle, cuda):
    import torch
    from rocmforge_amd import ops
    rng = np.random.default_rng(100 + fmt)
    be, bb = Q.BLOCK_ELEMS[fmt], Q.BLOCK_BYTES[fmt]
    nb = 4099
    blocks = Q.random_blocks(fmt, nb, rng).reshape(nb, bb).copy()
    if fmt != Q.MM_Q8_0:                                      # every f16 exponent field in the scales, 0 and 31 too
        blocks[:64, 0:16] = rng.integers(0, 256, (64, 16), dtype=np.uint8)
    blocks = blocks.ravel()
    got = ops.dequant(fmt, dev(blocks, cuda), nb * be).cpu().numpy()
    assert_bit_exact(got, oracle.dequantize(fmt, blocks, nb * be), Q.NAMES[fmt])
    # ragged element counts and short inputs follow the CPU loops' early exits
    for n, length in [(2 * be + 7, 3 * bb), (3 * be, 2 * bb + bb // 2), (3 * be, 2 * bb + 33), (3 * be, 2 * bb + 3),
                      (be, 5), (2 * be, bb + 34), (10, bb)]:
        d = dev(blocks[:length], cuda)
        got = ops.dequant(fmt, d, n).cpu().numpy()
        assert_bit_exact(got, oracle.dequantize(fmt, blocks[:length], n), f"{Q.NAMES[fmt]} n={n} len={length}")
    torch.cuda.synchronize()


@pytest.mark.parametrize("fmt", MM)
@pytest.mark.parametrize("m,n,k", [(1, 130, 4096), (3, 77, 768), (8, 40, 512), (1, 3000, 4096), (1, 700, 2048), (1, 515, 8192),
                                   (1, 33, 14336), (1, 60, 768)])
def test_mm_gemv_rows_of_k(fmt, m, n, k, oracle, cuda):
    from rocmforge_amd import ops
    w = Q.make_weights(fmt, n, k, seed=7000 + fmt + n)
    x = np.random.default_rng(7100 + k).standard_normal((m, k)).astype(np.float32)
    got = ops.gemv(fmt, dev(w, cuda), dev(x, cuda), n, k).cpu().numpy()
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, m, n, k), f"{Q.NAMES[fmt]} m={m} n={n} k={k}")


@pytest.mark.parametrize("fmt", [Q.MM_Q4_K, Q.MM_Q6_K])
def test_mm_gemv_every_scale_exponent_field(fmt, oracle, cuda):
    """Scales decode the module's own way, +-2^(field - 15) * (1 + (bits & 7) / 1024) for every exponent field, 0 and 31
    included: the decode GEMV's kernels must widen them as the dequantiser does."""
    from rocmforge_amd import ops
    n, k = 512, 4096
    rng = np.random.default_rng(7300 + fmt)
    w = Q.random_blocks(fmt, n * k // 256, rng).reshape(-1, 256).copy()
    nsc = 16 if fmt == Q.MM_Q4_K else 32                     # bytes of f16 scales at the head of a block
    x = rng.standard_normal((1, k)).astype(np.float32)
    for what, fields in (("every field", np.arange(32)), ("fields 0 and 1", np.array([0, 1]))):
        sc = rng.integers(0, 65536, (w.shape[0], nsc // 2)).astype(np.uint16) & np.uint16(0x83FF)
        sc |= (rng.choice(fields, size=sc.shape).astype(np.uint16) << np.uint16(10))
        wv = w.copy()
        wv[:, :nsc] = sc.view(np.uint8).reshape(w.shape[0], nsc)
        if fmt == Q.MM_Q4_K:
            wv[:, 16:24] = 0                                 # no minimum term: the scales carry the result
        wv = wv.ravel()
        got = ops.gemv(fmt, dev(wv, cuda), dev(x, cuda), n, k).cpu().numpy()
        want = oracle.qmatmul_nk(fmt, wv, x, 1, n, k)
        assert np.all(np.isfinite(want)) and float(np.abs(want).max()) > 0
        assert_close(got, want, f"{Q.NAMES[fmt]} scales with {what}")


@pytest.mark.parametrize("fmt", [Q.MM_Q4_K, Q.MM_Q6_K])
def test_mm_scale_widening_hand_values(fmt, cuda):
    """f16_to_f32_cpu (quantized/common.rs:47) shifts the mantissa in 16 bits: 0x3E00 (IEEE 1.5) widens to 1.0 and
    0x2E66 (IEEE 0.1) to 0.0628662109375.  Checked without the oracle, on the dequantiser and on the decode GEMV."""
    from rocmforge_amd import ops
    rng = np.random.default_rng(7400 + fmt)
    k, n = 1024, 64
    base = Q.random_blocks(fmt, n * k // 256, rng).reshape(-1, 256).copy()
    nsc = 8 if fmt == Q.MM_Q4_K else 16
    if fmt == Q.MM_Q4_K:
        base[:, 16:24] = 0
    x = rng.standard_normal((1, k)).astype(np.float32)
    res = {}
    for bits in (0x3C00, 0x3E00, 0x3FF8, 0x2C00, 0x2E66, 0x2C06):
        w = base.copy()
        w[:, :2 * nsc] = np.full((w.shape[0], nsc), bits, "<u2").view(np.uint8)
        res[bits] = (ops.dequant(fmt, dev(w.ravel(), cuda), n * k).cpu().numpy(),
                     ops.gemv(fmt, dev(w.ravel(), cuda), dev(x, cuda), n, k).cpu().numpy())
    for a, b in ((0x3E00, 0x3C00), (0x3FF8, 0x3C00), (0x2E66, 0x2C06)):      # same low three mantissa bits: same numbers
        assert_bit_exact(res[a][0], res[b][0], f"{Q.NAMES[fmt]} {a:#x} reads as {b:#x}")
        assert np.array_equal(res[a][1], res[b][1])
    d1, d2 = res[0x3C00][0], res[0x2E66][0]
    assert np.all(d1 == np.round(d1)) and np.abs(d1).max() >= 15                # scale 1.0: the codes themselves
    assert np.array_equal(d2, (d1 * np.float32(0.0628662109375)).astype(np.float32))


def test_kn_recipe_of_the_reference_gpu_test(oracle, cuda):
    # src/kernels/matmul/quantized/q4_0.rs:343-435
    from rocmforge_amd import ops
    m, n, k = 2, 4, 8
    a = (np.arange(m * k, dtype=np.float32) * np.float32(0.1)).reshape(m, k)
    w = np.zeros(20, np.uint8)
    w[0:4] = np.frombuffer(struct.pack("<f", 1.0), np.uint8)
    for i in range(16):
        w[4 + i] = ((i % 16) << 4) | (i % 16)
    got = ops.gemv_kn(Q.Q4_0, dev(w, cuda), dev(a, cuda), n, k).cpu().numpy()
    want = oracle.qmatmul_kn(Q.Q4_0, w, a, m, n, k)
    assert np.max(np.abs(got - want)) < 1e-5                 # (the reference's own test allows 0.1)


# n a multiple of 4 (a thread owns four columns) or not (one column); one split and many; n smaller and larger
# than a block, so that blocks straddle the rows of Wd.
@pytest.mark.parametrize("fmt", KN_FORMATS)
@pytest.mark.parametrize("n,k", [(256, 64), (96, 64), (1024, 512), (24, 2048), (250, 128), (3, 256), (4864, 896)])
def test_kn_against_the_oracle(fmt, n, k, oracle, cuda):
    from rocmforge_amd import ops
    be = Q.BLOCK_ELEMS[fmt]
    if (n * k) % be:
        pytest.skip("n * k must be whole blocks")
    rng = np.random.default_rng(7200 + fmt + n)
    w = Q.random_blocks(fmt, n * k // be, rng, exp_range=(-9, 3))
    x = rng.standard_normal(k).astype(np.float32)
    got = ops.gemv_kn(fmt, dev(w, cuda), dev(x, cuda), n, k).cpu().numpy()
    want = oracle.qmatmul_kn(fmt, w, x, 1, n, k)[0]
    assert_close(got, want, f"{Q.NAMES[fmt]} kn n={n} k={k}")


def test_kn_headline_shape_and_host_weights(oracle, cuda):
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    n, k = 14336, 4096                                         # config 3 in the orientation the reference computes
    w = Q.make_weights(Q.Q4_K, n, k, seed=20260003)
    x = np.random.default_rng(20260103).standard_normal(k).astype(np.float32)
    dx = dev(x, cuda)
    want = oracle.qmatmul_kn(Q.Q4_K, w, x, 1, n, k)[0]
    y = torch.empty(n, dtype=torch.float32, device=cuda)
    _lib.check(L.rfq_matmul_host_weights_kn(Q.Q4_K, C.c_void_p(w.ctypes.data), w.size, C.c_void_p(dx.data_ptr()), n, k,
                                            C.c_void_p(y.data_ptr()), None))
    e = assert_close(y.cpu().numpy(), want, "host weights, kn")
    print(f"Q4_K 14336x4096 kn: max rel err {e:.2e}")
    # the same bytes read as rows of k give other numbers
    from rocmforge_amd import ops
    other = ops.gemv(Q.Q4_K, dev(w, cuda), dx, n, k).cpu().numpy()
    assert np.max(np.abs(other - want)) > 1e-2 * np.sqrt(np.mean(want.astype(np.float64) ** 2))


def test_kn_validation(cuda):
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    one = C.c_void_p(16)
    assert L.rfq_gemv_kn(2, one, 20, one, one, 1, 3, 8, None) == _lib.E_SIZE          # 24 elements: not whole blocks
    assert L.rfq_gemv_kn(2, one, 21, one, one, 1, 4, 8, None) == _lib.E_SIZE          # byte count
    assert L.rfq_gemv_kn(10, one, 256, one, one, 1, 16, 16, None) == _lib.E_UNSUPPORTED
    assert L.rfq_get_rows(208, one, 36, 1, 32, one, 1, one, None, None) == _lib.E_UNSUPPORTED
    assert L.rfq_gemm_f16(212, one, 256, one, one, 1, 1, 1, 256, None) == _lib.E_UNSUPPORTED
