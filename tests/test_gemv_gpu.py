"""GPU parity: fused dequant + GEMV against the CPU oracle (dequantise, then
the reference's sequential fp32 matmul)."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_close, error_report
from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu

FORMATS = [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3]


def gpu_gemv(fmt, w, x, n, k, cuda):
    import torch
    from rocmforge_amd import ops
    dw = torch.from_numpy(np.ascontiguousarray(w)).to(cuda)
    dx = torch.from_numpy(np.ascontiguousarray(x)).to(cuda)
    y = ops.gemv(fmt, dw, dx, n, k)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def x_for(m, k, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    x = rng.standard_normal((m, k), dtype=np.float32)
    return x[0] if m == 1 else x


# k = 256 and 512 take the one-row-per-wavefront kernel, 768 ... 14336 the
# register-resident one at 1, 2, 2x2 and 2x4 units per lane x wavefronts per
# row, 32768 falls back again; n values exercise ragged teams.
@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("n,k", [(5, 256), (40, 512), (77, 768), (33, 1024), (64, 2048), (1001, 2048), (130, 4096), (257, 8192),
                                 (19, 14336), (9, 32768), (2048, 1536), (21, 16384), (300, 12288)])
def test_gemv_m1_shapes(fmt, n, k, oracle, cuda):
    w = Q.make_weights(fmt, n, k, seed=3000 + fmt + n)
    x = x_for(1, k, 4000 + k)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    want = oracle.qmatmul_nk(fmt, w, x, 1, n, k)[0]
    assert_close(got, want, f"{Q.NAMES[fmt]} n={n} k={k}")


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m", [2, 3, 5, 8])
def test_gemv_small_batches(fmt, m, oracle, cuda):
    n, k = 301, 2048
    w = Q.make_weights(fmt, n, k, seed=5000 + fmt)
    x = x_for(m, k, 6000 + m)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert got.shape == (m, n)
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, m, n, k), f"{Q.NAMES[fmt]} m={m}")


# Batches of a format or row length without a batch kernel go out as one decode launch per vector once the matrix has
# eight million weights (below that the one-row-per-wavefront kernel takes the whole batch).
@pytest.mark.parametrize("fmt,n,k", [(Q.Q6_K, 2100, 4096), (Q.MXFP4, 2100, 4096), (Q.MXFP6_E2M3, 2049, 4096),
                                     (Q.Q4_K, 700, 12288), (Q.Q4_0, 513, 16384), (Q.Q6_K, 1100, 8192)])
@pytest.mark.parametrize("m", [2, 5, 8])
def test_gemv_batches_as_decode_launches(fmt, n, k, m, oracle, cuda):
    w = Q.make_weights(fmt, n, k, seed=5100 + fmt + n)
    x = x_for(m, k, 6100 + m)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert got.shape == (m, n)
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, m, n, k), f"{Q.NAMES[fmt]} {n}x{k} m={m}")


# Q8_0 batches run on the matrix cores: 16 rows per workgroup, 16 wavefronts
# that take every 16th unit, eight units at a time: odd unit counts, more than
# one trip, fewer units than wavefronts, a ragged last row tile.
@pytest.mark.parametrize("fmt", [Q.Q8_0, Q.GGUF_Q8_0])
@pytest.mark.parametrize("m,n,k", [(2, 16, 96), (4, 50, 8224), (8, 33, 4096), (7, 1, 32)])
def test_q8_0_batches_on_the_matrix_cores(fmt, m, n, k, oracle, cuda):
    w = Q.make_weights(fmt, n, k, seed=5100 + n)
    x = x_for(m, k, 6100 + m)
    x[0, ::7] *= 1000.0                                                   # outliers: per-unit scaling
    x[m - 1, 5:40] = 0.0                                                  # an all-zero unit
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, m, n, k), f"{Q.NAMES[fmt]} m={m} n={n} k={k}")


@pytest.mark.parametrize("fmt", [Q.Q4_0, Q.Q4_K])
@pytest.mark.parametrize("m,k", [(8, 4096), (8, 8192), (5, 8192), (3, 8192)])
def test_batches_whose_prepared_vectors_exceed_lds(fmt, m, k, oracle, cuda):
    """Eight prepared vectors of k = 8192 need 229 KB of LDS: the batch goes out as launches of four."""
    n = 150
    w = Q.make_weights(fmt, n, k, seed=5200 + fmt)
    x = x_for(m, k, 6200 + m)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, m, n, k), f"{Q.NAMES[fmt]} m={m} k={k}")


@pytest.mark.parametrize("fmt", [Q.MXFP4, Q.MXFP6_E2M3])
def test_gemv_mx_random_codes_and_clamp(fmt, oracle, cuda):
    # every code, exponents up to +6 so the +-8 / +-7.5 clamp is active
    rng = np.random.default_rng(70 + fmt)
    n, k = 96, 4096
    w = Q.random_blocks(fmt, n * k // 32, rng, exp_range=(-9, 6))
    x = x_for(1, k, 71)
    assert_close(gpu_gemv(fmt, w, x, n, k, cuda), oracle.qmatmul_nk(fmt, w, x, 1, n, k)[0], Q.NAMES[fmt])


@pytest.mark.parametrize("fmt", [Q.MXFP4, Q.MXFP6_E2M3])
@pytest.mark.parametrize("n,k", [(96, 4096), (2100, 4096), (14336, 4096), (300, 12288)])
def test_gemv_mx_extreme_exponents(fmt, n, k, oracle, cuda):
    """Exponent bytes -128 (the reference's scale is 0 there) and 127 (every non-zero code clamps to +-8) among ordinary
    and clamping ones, at shapes where MXFP4 takes the integer-dot kernel (96, 14336 and 300 rows) and the float one (2100)."""
    rng = np.random.default_rng(7700 + n + fmt)
    w = Q.random_blocks(fmt, n * k // 32, rng, exp_range=(-9, 3)).copy()
    blocks = w.reshape(-1, Q.BLOCK_BYTES[fmt])
    blocks[rng.random(blocks.shape[0]) < 0.02, 0] = 0x80
    blocks[rng.random(blocks.shape[0]) < 0.02, 0] = 0x7F
    x = x_for(1, k, 7701)
    x[64:96] = 0.0
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert np.isfinite(got).all()
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, 1, n, k)[0], f"{Q.NAMES[fmt]} n={n} k={k} with exponents -128 and 127")


# The benchmark configurations: Q4_0 4864x896; Q8_0 4096x4096 at m = 1 and 8; Q4_K and Q6_K 14336x4096.
@pytest.mark.parametrize("fmt,n,k,m,cfg", [(Q.Q4_0, 4864, 896, 1, 1), (Q.Q8_0, 4096, 4096, 1, 2),
                                           (Q.Q8_0, 4096, 4096, 8, 2), (Q.Q4_K, 14336, 4096, 1, 3),
                                           (Q.Q6_K, 14336, 4096, 1, 3)])
def test_gemv_baseline_configs(fmt, n, k, m, cfg, oracle, cuda):
    w = Q.make_weights(fmt, n, k, seed=20260000 + cfg)
    x = x_for(m, k, 20260100 + cfg)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    want = oracle.qmatmul_nk(fmt, w, x, m, n, k)
    assert_close(got.reshape(m, n), want, f"config {cfg} {Q.NAMES[fmt]} m={m}")
    print(f"config {cfg} {Q.NAMES[fmt]} m={m}: {error_report(got.reshape(m, n), want)}")


# The vocabulary projection (LM head), the largest GEMV of a decode step: 128256 x 4096 (525 MB as Q4_K).  Sampled
# rows against the oracle (first and last rows of the matrix, of a team's and a workgroup's range, and random ones)
# and a checksum over every output: sum_n y[n] = x . sum_n W[n, :], the column sums taken from the oracle's dequantisation.
@pytest.mark.timeout(600)
@pytest.mark.parametrize("fmt", [Q.Q4_K, Q.GGUF_Q4_K, Q.Q6_K, Q.GGUF_Q6_K, Q.Q8_0, Q.MXFP4])
def test_lm_head_shape_sampled(fmt, oracle, cuda):
    n, k = 128256, 4096
    rng = np.random.default_rng(20260200 + fmt)
    w = Q.random_blocks(fmt, n * k // Q.BLOCK_ELEMS[fmt], rng)
    x = x_for(1, k, 20260201)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    # (a team walks its rows in groups of 5..8 with loads running on from group to group: whole teams' ranges)
    rows = np.unique(np.concatenate([np.arange(0, 140), np.arange(n - 140, n), np.arange(62600, 62740),
                                     rng.integers(0, n, 400)]))
    want = oracle.qmatmul_nk(fmt, w, x, 1, n, k, rows=rows)[0]
    assert_close(got[rows], want, f"{Q.NAMES[fmt]} LM head, {rows.size} sampled rows")
    print(f"{Q.NAMES[fmt]} 128256x4096, {rows.size} rows: {error_report(got[rows], want)}")
    rb = Q.BLOCK_BYTES[fmt] * k // Q.BLOCK_ELEMS[fmt]
    colsum = np.zeros(k, np.float64)
    step = 8016                                               # 16 chunks of rows
    for r0 in range(0, n, step):
        r1 = min(n, r0 + step)
        colsum += oracle.dequantize(fmt, w[r0 * rb:r1 * rb], (r1 - r0) * k).reshape(-1, k).astype(np.float64).sum(axis=0)
    total, want_total = float(got.astype(np.float64).sum()), float(x.astype(np.float64) @ colsum)
    scale = float(np.sqrt(n) * np.sqrt(np.mean(got.astype(np.float64) ** 2)))   # size of a sum of n outputs
    assert abs(total - want_total) <= 1e-4 * scale, (total, want_total, scale)


def test_q4_k_onesided_real_data(oracle, cuda):
    rng = np.random.default_rng(81)
    n, k = 512, 4096
    w = Q.quantize_q4_k_onesided(np.abs(rng.standard_normal((n, k)) * 0.02).astype(np.float32), rng)
    x = x_for(1, k, 82)
    assert_close(gpu_gemv(Q.Q4_K, w, x, n, k, cuda), oracle.qmatmul_nk(Q.Q4_K, w, x, 1, n, k)[0], "q4_k onesided")


def test_linearity_at_full_size(cuda):
    # size-independent property at the headline shape: W(a*x1 + x2) == a*W(x1) + W(x2)
    n, k = 14336, 4096
    w = Q.make_weights(Q.Q4_K, n, k, seed=91)
    x1, x2 = x_for(1, k, 92), x_for(1, k, 93)
    y1, y2 = gpu_gemv(Q.Q4_K, w, x1, n, k, cuda), gpu_gemv(Q.Q4_K, w, x2, n, k, cuda)
    y = gpu_gemv(Q.Q4_K, w, (np.float32(0.5) * x1 + x2).astype(np.float32), n, k, cuda)
    assert_close(y, 0.5 * y1.astype(np.float64) + y2, "linearity", tol=1e-4)


def test_reference_signatures(oracle, cuda):
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    n, k = 256, 1024
    x = x_for(1, k, 101)
    dx = torch.from_numpy(x).to(cuda)
    for fmt, fn in ((Q.Q4_0, L.rfq_matmul_q4_0), (Q.Q8_0, L.rfq_matmul_q8_0), (Q.Q4_K, L.rfq_matmul_q4_k),
                    (Q.Q6_K, L.rfq_matmul_q6_k)):
        w = Q.make_weights(fmt, n, k, seed=102 + fmt)
        want = oracle.qmatmul_nk(fmt, w, x, 1, n, k)[0]
        dw = torch.from_numpy(w).to(cuda)
        out = torch.zeros(n, dtype=torch.float32, device=cuda)
        # (activations, weights, output, m, n, k), as matmul_q4_0_gpu
        _lib.check(fn(C.c_void_p(dx.data_ptr()), C.c_void_p(dw.data_ptr()), C.c_void_p(out.data_ptr()), 1, n, k, None))
        torch.cuda.synchronize()
        assert_close(out.cpu().numpy(), want, f"raw {Q.NAMES[fmt]}")
        # host weights, device input/output, as matmul_q4_0(backend, &[u8], &HipBuffer, rows, cols, &HipBuffer)
        out.zero_()
        torch.cuda.synchronize()
        _lib.check(L.rfq_matmul_host_weights(fmt, w.ctypes.data_as(C.c_void_p), w.size, C.c_void_p(dx.data_ptr()),
                                             n, k, C.c_void_p(out.data_ptr()), None))
        assert_close(out.cpu().numpy(), want, f"host weights {Q.NAMES[fmt]}")
    # the all-0x88 Q4_0 weights of tests/q_dequant_tests.rs:396-489 give exactly zero
    w = np.zeros((n * k // 32, 20), np.uint8); w[:, 0:4] = np.frombuffer(np.float32(1.0).tobytes(), np.uint8); w[:, 4:] = 0x88
    assert np.all(np.abs(gpu_gemv(Q.Q4_0, w.ravel(), x, n, k, cuda)) < 1e-4)


def test_gemv_more_than_eight_rows(oracle, cuda):
    # eight rows of x per launch, any m
    fmt, n, k, m = Q.Q4_K, 130, 2048, 19
    w = Q.make_weights(fmt, n, k, seed=9100)
    x = x_for(m, k, 9101)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert got.shape == (m, n)
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, m, n, k), "m=19")


@pytest.mark.parametrize("fmt", [Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3, Q.Q4_0, Q.Q8_0, Q.GGUF_Q4_0, Q.GGUF_Q8_0])
@pytest.mark.parametrize("n,k", [(14336, 4096), (14413, 4096), (15001, 2304), (20000, 2560), (14337, 3840), (8192, 4096), (8201, 2304), (11008, 4096),
                                 (50000, 4096), (51203, 2304)])
def test_long_matrices_one_unit_per_lane(fmt, n, k, oracle, cuda):
    """Q4_K and the float-path formats with rows of 65..128 units and at least seven rows per team run with one
    unit per lane and two wavefronts per row: ragged row counts, rows that end inside the second wavefront; at 50000 rows
    a team walks several groups of five rows with its loads carrying on from group to group."""
    w = Q.make_weights(fmt, n, k, seed=5300 + n + fmt)
    x = x_for(1, k, 6300 + k)
    got = gpu_gemv(fmt, w, x, n, k, cuda)
    assert_close(got, oracle.qmatmul_nk(fmt, w, x, 1, n, k), f"{Q.NAMES[fmt]} {n}x{k}")


# The 17-, 25-, 18-, 34- and 210-byte layouts are read in place at whatever alignment their blocks have, through
# aligned windows of whole dwords (the GGUF ones when the tensor starts on a multiple of 4, byte-exactly otherwise):
# weights at odd device addresses, and tensors whose byte count is not a multiple of 4, must agree with the oracle.
@pytest.mark.parametrize("fmt", [Q.MXFP4, Q.MXFP6_E2M3, Q.GGUF_Q4_0, Q.GGUF_Q8_0, Q.GGUF_Q6_K])
def test_gemv_windowed_layouts_at_any_address(fmt, oracle, cuda):
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    be = Q.BLOCK_ELEMS[fmt]
    for (m, n, k) in [(1, 130, 4096), (1, 3, 3 * be), (4, 33, 2048), (1, 5, 5 * be)]:
        rng = np.random.default_rng(9000 + fmt + n)
        w = Q.random_blocks(fmt, n * k // be, rng, exp_range=(-9, 3))
        x = rng.standard_normal((m, k)).astype(np.float32)
        want = oracle.qmatmul_nk(fmt, w, x, m, n, k)
        dx = torch.from_numpy(x).to(cuda)
        for off in (0, 1, 2, 3):
            buf = torch.zeros(w.size + 8, dtype=torch.uint8, device=cuda)
            buf[off:off + w.size] = torch.from_numpy(w).to(cuda)
            y = torch.empty((m, n), dtype=torch.float32, device=cuda)
            _lib.check(L.rfq_gemv(fmt, C.c_void_p(buf.data_ptr() + off), w.size, C.c_void_p(dx.data_ptr()),
                                  C.c_void_p(y.data_ptr()), m, n, k, None))
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), want, f"{Q.NAMES[fmt]} m={m} n={n} k={k} offset {off}")


@pytest.mark.parametrize("fmt", [Q.Q4_K, Q.MXFP4, Q.GGUF_Q4_K])
def test_timeline_build_computes_the_same_and_stamps_in_order(fmt, oracle, cuda):
    """rfq_bench_gemv_timeline launches the build of the decode kernel that stamps a clock at 20 points per wavefront:
    its output must be the ordinary kernel's, every wavefront's stamps must not go backwards, and a shape whose
    kernel has no such build reports zero wavefronts."""
    import torch
    from rocmforge_amd import _lib
    L = _lib.lib()
    n, k = 14336, 4096
    w = Q.make_weights(fmt, n, k, seed=8800 + fmt)
    x = x_for(1, k, 8801)
    want = gpu_gemv(fmt, w, x, n, k, cuda)
    dw = torch.from_numpy(w).to(cuda)
    dx = torch.from_numpy(x).to(cuda)
    y = torch.zeros((1, n), dtype=torch.float32, device=cuda)
    cap = 8192
    trace = torch.zeros((cap, 20), dtype=torch.int64, device=cuda)
    ptrs = (C.c_void_p * 1)(dw.data_ptr())
    waves, stamps = C.c_int(-1), C.c_int(-1)
    _lib.check(L.rfq_bench_gemv_timeline(fmt, ptrs, 1, w.size, C.c_void_p(dx.data_ptr()), C.c_void_p(y.data_ptr()), n, k, 2, None,
                                         C.c_void_p(trace.data_ptr()), cap, C.byref(waves), C.byref(stamps)))
    torch.cuda.synchronize()
    assert stamps.value == 20 and waves.value in (2048, 4096), (stamps.value, waves.value)
    np.testing.assert_array_equal(y.cpu().numpy().reshape(-1), np.asarray(want).reshape(-1))
    t = trace[:waves.value].cpu().numpy()
    assert (t[:, 0] > 0).all() and (np.diff(t, axis=1) >= 0).all()
    assert (t[:, 19] - t[:, 0]).max() < 100 * 1000                  # (100 MHz ticks: under a millisecond)
    # a shape whose kernel has no such build: ordinary launch, nothing written
    n2, k2 = 256, 1024
    w2 = Q.make_weights(fmt, n2, k2, seed=8802)
    dw2 = torch.from_numpy(w2).to(cuda)
    x2 = x_for(1, k2, 8803)
    dx2 = torch.from_numpy(x2).to(cuda)
    y2 = torch.zeros((1, n2), dtype=torch.float32, device=cuda)
    ptrs2 = (C.c_void_p * 1)(dw2.data_ptr())
    _lib.check(L.rfq_bench_gemv_timeline(fmt, ptrs2, 1, w2.size, C.c_void_p(dx2.data_ptr()), C.c_void_p(y2.data_ptr()), n2, k2, 1, None,
                                         C.c_void_p(trace.data_ptr()), cap, C.byref(waves), C.byref(stamps)))
    torch.cuda.synchronize()
    assert waves.value == 0
    assert_close(y2.cpu().numpy(), oracle.qmatmul_nk(fmt, w2, x2, 1, n2, k2), f"{Q.NAMES[fmt]} untraced shape")
