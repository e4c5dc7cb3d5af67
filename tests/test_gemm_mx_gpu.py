"""GPU parity: MXFP4 / MXFP6 prefill GEMM on the scaled matrix instruction
against the CPU oracle (dequantise both operands as the reference does, then
its sequential fp32 matmul)."""
import numpy as np
import pytest

from helpers import assert_close, error_report
from rocmforge_amd import _lib, quantize as Q

pytestmark = pytest.mark.gpu

MXFP4, MXFP6 = Q.MXFP4, Q.MXFP6_E2M3


def gauss(rows, k, seed, std):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal((rows, k), dtype=np.float32) * np.float32(std)


def packed(fmt, x):
    return Q.pack_mxfp4(x) if fmt == MXFP4 else Q.pack_mxfp6(x)


def run_gemm(a_fmt, a_raw, w_fmt, w_raw, m, n, k, cuda, out_dtype=None, a_kind=_lib.MX_AUTO, w_kind=_lib.MX_AUTO):
    import torch
    from rocmforge_amd import ops
    A = ops.MxOperand(a_fmt, torch.from_numpy(np.ascontiguousarray(a_raw)).to(cuda), m, k, a_kind)
    W = ops.MxOperand(w_fmt, torch.from_numpy(np.ascontiguousarray(w_raw)).to(cuda), n, k, w_kind)
    out = ops.gemm_mx(A, W, out_dtype or torch.float32)
    torch.cuda.synchronize()
    return out, A.kind, W.kind


def oracle_gemm(oracle, a_fmt, a_raw, w_fmt, w_raw, m, n, k, rows=None, cols=None):
    a = oracle.dequantize(a_fmt, a_raw, m * k).reshape(m, k)
    if rows is not None:
        a = np.ascontiguousarray(a[rows])
    return oracle.qmatmul_nk(w_fmt, w_raw, a, a.shape[0], n, k, rows=cols)


@pytest.mark.parametrize("m,n,k", [(32, 32, 128), (64, 96, 256), (70, 300, 384), (256, 256, 512), (300, 520, 1024)])
def test_fp4_operands_from_the_reference_packer(m, n, k, oracle, cuda):
    a_raw, w_raw = packed(MXFP4, gauss(m, k, 1, 1.0)), packed(MXFP4, gauss(n, k, 2, 0.02))
    out, ka, kw = run_gemm(MXFP4, a_raw, MXFP4, w_raw, m, n, k, cuda)
    assert ka == _lib.MX_FP4 and kw == _lib.MX_FP4      # what pack_mxfp4 emits always fits 4 bits
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a_raw, MXFP4, w_raw, m, n, k), f"fp4 {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k", [(32, 64, 128), (96, 160, 640)])
def test_random_codes_take_the_fp8_encoding(m, n, k, oracle, cuda):
    rng = np.random.default_rng(5)
    a_raw = Q.random_blocks(MXFP4, m * k // 32, rng, exp_range=(-6, 5))   # every code; clamp active
    w_raw = Q.random_blocks(MXFP4, n * k // 32, rng, exp_range=(-9, 2))
    out, ka, kw = run_gemm(MXFP4, a_raw, MXFP4, w_raw, m, n, k, cuda)
    assert ka == _lib.MX_FP8 and kw == _lib.MX_FP8
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a_raw, MXFP4, w_raw, m, n, k), "fp8 x fp8")


representable_blocks = Q.mxfp4_window_blocks


@pytest.mark.parametrize("exp_a,exp_w", [((-6, 1), (-9, -2)), ((-128, -120), (118, 127)), ((0, 6), (-4, 4))])
def test_fp4_reencoding_of_every_code_window(exp_a, exp_w, oracle, cuda):
    """The integer re-encoder against the oracle on blocks that use every code,
    at exponents where the +-8 clamp merges codes and at both ends of the range;
    the unchecked request writes the same bytes without the read-back."""
    import torch
    from rocmforge_amd import ops
    m, n, k = 96, 160, 512
    rng = np.random.default_rng(21)
    a_raw, w_raw = representable_blocks(rng, m * k // 32, exp_a), representable_blocks(rng, n * k // 32, exp_w)
    out, ka, kw = run_gemm(MXFP4, a_raw, MXFP4, w_raw, m, n, k, cuda)
    assert ka == _lib.MX_FP4 and kw == _lib.MX_FP4
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a_raw, MXFP4, w_raw, m, n, k), f"windows {exp_a} {exp_w}")
    checked = ops.MxOperand(MXFP4, torch.from_numpy(a_raw).to(cuda), m, k, _lib.MX_FP4)
    unchecked = ops.MxOperand(MXFP4, torch.from_numpy(a_raw).to(cuda), m, k, _lib.MX_FP4_UNCHECKED)
    torch.cuda.synchronize()
    # (the last 16 bytes are the status words, which an unchecked request neither clears nor reads)
    assert unchecked.kind == _lib.MX_FP4 and torch.equal(checked.buf[:-16], unchecked.buf[:-16])


def test_mixed_kinds_and_mxfp6_weights(oracle, cuda):
    rng = np.random.default_rng(6)
    m, n, k = 96, 224, 512
    a4 = packed(MXFP4, gauss(m, k, 3, 1.0))
    w6 = packed(MXFP6, gauss(n, k, 4, 0.02))
    out, ka, kw = run_gemm(MXFP4, a4, MXFP6, w6, m, n, k, cuda)
    assert ka == _lib.MX_FP4 and kw == _lib.MX_FP8
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a4, MXFP6, w6, m, n, k), "fp4 x mxfp6")
    # MXFP6 payload as the loader sees arbitrary bytes (its extraction differs from the packer's)
    w6r = Q.random_blocks(MXFP6, n * k // 32, rng, exp_range=(-8, 3))
    out, _, _ = run_gemm(MXFP4, a4, MXFP6, w6r, m, n, k, cuda)
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a4, MXFP6, w6r, m, n, k), "fp4 x random mxfp6")
    # 8-bit activations x 4-bit weights, and MXFP6 on both sides
    a_r = Q.random_blocks(MXFP4, m * k // 32, rng, exp_range=(-3, 3))
    w4 = packed(MXFP4, gauss(n, k, 7, 0.02))
    out, ka, kw = run_gemm(MXFP4, a_r, MXFP4, w4, m, n, k, cuda)
    assert ka == _lib.MX_FP8 and kw == _lib.MX_FP4
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a_r, MXFP4, w4, m, n, k), "fp8 x fp4")
    a6 = packed(MXFP6, gauss(m, k, 8, 1.0))
    out, _, _ = run_gemm(MXFP6, a6, MXFP6, w6, m, n, k, cuda)
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP6, a6, MXFP6, w6, m, n, k), "mxfp6 x mxfp6")


def test_forced_kinds(oracle, cuda):
    import torch
    from rocmforge_amd import ops
    m, n, k = 64, 64, 256
    a4, w4 = packed(MXFP4, gauss(m, k, 9, 1.0)), packed(MXFP4, gauss(n, k, 10, 0.02))
    want = oracle_gemm(oracle, MXFP4, a4, MXFP4, w4, m, n, k)
    out, ka, kw = run_gemm(MXFP4, a4, MXFP4, w4, m, n, k, cuda, a_kind=_lib.MX_FP8, w_kind=_lib.MX_FP8)
    assert ka == _lib.MX_FP8 and kw == _lib.MX_FP8
    assert_close(out.cpu().numpy(), want, "forced fp8")
    bad = Q.random_blocks(MXFP4, m * k // 32, np.random.default_rng(11), exp_range=(-2, 2))
    with pytest.raises(_lib.RfqError) as e:
        ops.MxOperand(MXFP4, torch.from_numpy(bad).to(cuda), m, k, _lib.MX_FP4)
    assert e.value.status == _lib.E_UNSUPPORTED
    # MXFP6 has no 4-bit re-encoding: it cannot even be sized
    assert _lib.lib().rfq_mx_prepared_bytes(MXFP6, _lib.MX_FP4, m, k) == 0
    raw6 = torch.from_numpy(packed(MXFP6, gauss(m, k, 12, 1.0))).to(cuda)
    buf = torch.empty(_lib.lib().rfq_mx_prepared_bytes(MXFP6, _lib.MX_FP8, m, k), dtype=torch.uint8, device=cuda)
    import ctypes as C
    rc = _lib.lib().rfq_mx_prepare(MXFP6, _lib.MX_FP4, C.c_void_p(raw6.data_ptr()), raw6.numel(), m, k,
                                   C.c_void_p(buf.data_ptr()), buf.numel(), None, None)
    assert rc == _lib.E_UNSUPPORTED


def test_extreme_exponents(oracle, cuda):
    # scale bytes at both ends of the i8 range: products far outside 1.0
    m, n, k = 32, 32, 256
    rng = np.random.default_rng(13)
    a = Q.random_blocks(MXFP4, m * k // 32, rng, exp_range=(-60, -50))
    w = Q.random_blocks(MXFP4, n * k // 32, rng, exp_range=(20, 30))
    out, _, _ = run_gemm(MXFP4, a, MXFP4, w, m, n, k, cuda)
    assert_close(out.cpu().numpy(), oracle_gemm(oracle, MXFP4, a, MXFP4, w, m, n, k), "extreme exponents")


def test_bf16_output_is_the_rounded_fp32_output(cuda):
    import torch
    m, n, k = 128, 384, 512
    a4, w4 = packed(MXFP4, gauss(m, k, 14, 1.0)), packed(MXFP4, gauss(n, k, 15, 0.02))
    f32, _, _ = run_gemm(MXFP4, a4, MXFP4, w4, m, n, k, cuda)
    b16, _, _ = run_gemm(MXFP4, a4, MXFP4, w4, m, n, k, cuda, out_dtype=torch.bfloat16)
    assert torch.equal(b16, f32.to(torch.bfloat16))      # same accumulation, round-to-nearest-even cast


@pytest.mark.timeout(900)
@pytest.mark.parametrize("w_fmt", [MXFP4, MXFP6])
def test_full_size_sampled(w_fmt, oracle, cuda):
    """M=2048, K=8192, N=28672 (bf16 out), W ~ N(0, 0.02) over all 28672 rows (seven independently seeded slabs of
    4096 rows, packed one at a time to bound host memory): sampled rows/columns against the oracle, and a checksum
    over every output: sum_n out[m, n] = A[m, :] . sum_n W[n, :]."""
    import torch
    m, n, k = 2048, 28672, 8192
    a_raw = packed(MXFP4, gauss(m, k, 20260005, 1.0))
    slabs = [packed(w_fmt, gauss(4096, k, 20260015 + w_fmt + 100 * i, 0.02)) for i in range(7)]
    w_raw = np.concatenate(slabs)
    out, ka, kw = run_gemm(MXFP4, a_raw, w_fmt, w_raw, m, n, k, cuda, out_dtype=torch.bfloat16)
    assert ka == _lib.MX_FP4 and kw == (_lib.MX_FP4 if w_fmt == MXFP4 else _lib.MX_FP8)
    rows = np.array([0, 1, 31, 32, 255, 256, 1000, 2047])
    cols = np.array([0, 1, 33, 255, 256, 4095, 4096, 5000, 8191, 8192, 14000, 16383, 20000, 24576, 28671])
    want = oracle_gemm(oracle, MXFP4, a_raw, w_fmt, w_raw, m, n, k, rows=rows, cols=cols)
    got = out[torch.from_numpy(rows).to(cuda)][:, torch.from_numpy(cols).to(cuda)].float().cpu().numpy()
    # bf16 keeps 8 significant bits: one rounding of up to 2^-8 relative on top of the fp32 tolerance
    assert_close(got, want, "sampled", tol=1e-3 + 2.0 ** -8)
    f32, _, _ = run_gemm(MXFP4, a_raw, w_fmt, w_raw, m, n, k, cuda)
    assert torch.equal(out, f32.to(torch.bfloat16))       # the bf16 result is the rounded fp32 result
    got = f32[torch.from_numpy(rows).to(cuda)][:, torch.from_numpy(cols).to(cuda)].cpu().numpy()
    assert_close(got, want, "sampled fp32")
    print(f"MXFP4 x {'MXFP4' if w_fmt == MXFP4 else 'MXFP6'} 2048x28672x8192, {rows.size} x {cols.size} samples, fp32 out: "
          f"{error_report(got, want)}")
    a = oracle.dequantize(MXFP4, a_raw, m * k).reshape(m, k).astype(np.float64)
    wsum = np.zeros(k, np.float64)
    for slab in slabs:
        wsum += oracle.dequantize(w_fmt, slab, 4096 * k).reshape(4096, k).astype(np.float64).sum(axis=0)
    check = f32.double().sum(dim=1).cpu().numpy()
    assert_close(check, a @ wsum, "row checksums", tol=1e-4)
