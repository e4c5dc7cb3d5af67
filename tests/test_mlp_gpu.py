"""GPU parity: the neighbours of the quantised matmul in a decoder layer
(RMSNorm, SwiGLU, RMSNorm over packed rows, RMSNorm -> GEMV, the SwiGLU MLP)
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from helpers import assert_close
from rocmforge_amd import quantize as Q

pytestmark = pytest.mark.gpu

FORMATS = [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3]
# The reference's own comparisons allow 1e-4 on small and 2e-3 on large inputs
# (src/mlp/rms_norm_tests.rs:15-16, src/mlp/swiglu_tests.rs:15-16); the elementwise
# operators here are held to 1e-5 relative, the matmul chains to the 1e-3 of the GEMV.
ELEMENTWISE_TOL = 1e-5


def dev(a, cuda):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.cpu().numpy()


def gauss(shape, seed, std=1.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def norm_weight(hidden, seed):
    return (1.0 + 0.2 * gauss((hidden,), seed)).astype(np.float32)


@pytest.mark.parametrize("rows,hidden", [(4, 8), (32, 128), (1, 4096), (7, 5120), (3, 12)])
def test_rms_norm(rows, hidden, oracle, cuda):
    from rocmforge_amd import ops
    if (rows, hidden) == (4, 8):      # src/mlp/rms_norm_tests.rs:79-88
        x = (np.arange(32, dtype=np.float32) * np.float32(0.1)).reshape(4, 8)
        w = np.float32(1.0) + np.arange(8, dtype=np.float32) * np.float32(0.1)
    elif (rows, hidden) == (32, 128):  # :148-157
        x = (np.arange(4096, dtype=np.float32) * np.float32(0.01)).reshape(32, 128)
        w = np.float32(0.5) + np.arange(128, dtype=np.float32) * np.float32(0.01)
    else:
        x, w = gauss((rows, hidden), 100 + hidden, 3.0), norm_weight(hidden, 200 + hidden)
    got = host(ops.rms_norm(dev(x, cuda), dev(w, cuda), 1e-6))
    assert_close(got, oracle.rms_norm(x, w, 1e-6), f"rms_norm {rows}x{hidden}", tol=ELEMENTWISE_TOL)


def test_rms_norm_properties(cuda):
    # src/mlp/rms_norm_tests.rs:211-251
    from rocmforge_amd import ops
    one = dev(np.ones(4, np.float32), cuda)
    assert not host(ops.rms_norm(dev(np.zeros((1, 4), np.float32), cuda), one, 1e-6)).any()
    assert np.all(np.abs(host(ops.rms_norm(dev(np.full((1, 4), 2.0, np.float32), cuda), one, 1e-6)) - 1.0) < 0.01)
    assert np.array_equal(host(ops.rms_norm(dev(np.full((1, 16), 3.0, np.float32), cuda),
                                            dev(np.ones(16, np.float32), cuda), 7.0)), np.full((1, 16), 0.75, np.float32))


@pytest.mark.parametrize("case", ["4x8", "32x32", "8x64", "large", "random", "ragged"])
def test_swiglu(case, oracle, cuda):
    from rocmforge_amd import ops
    if case == "4x8":        # src/mlp/swiglu_tests.rs:71-78
        g = np.arange(32, dtype=np.float32) * np.float32(0.1); u = g + np.float32(1.0); shape = (4, 8)
    elif case == "32x32":    # :141-147
        g = np.arange(1024, dtype=np.float32) * np.float32(0.01); u = g - np.float32(1.0); shape = (32, 32)
    elif case == "8x64":     # :202-208
        g = np.arange(512, dtype=np.float32) * np.float32(0.05); u = g - np.float32(2.0); shape = (8, 64)
    elif case == "large":    # :263-310
        g = np.arange(16, dtype=np.float32) * 100 - 50; u = np.arange(16, dtype=np.float32) * 50 - 25; shape = (2, 8)
    elif case == "random":
        g, u, shape = gauss((5 * 14336,), 31, 2.0), gauss((5 * 14336,), 32, 4.0), (5, 14336)
    else:
        g, u, shape = gauss((3 * 37,), 33), gauss((3 * 37,), 34), (3, 37)
    got = host(ops.swiglu(dev(g.reshape(shape), cuda), dev(u.reshape(shape), cuda)))
    want = oracle.swiglu(g, u).reshape(shape)
    assert np.all(np.isfinite(got))
    assert_close(got, want, f"swiglu {case}", tol=ELEMENTWISE_TOL)


def test_swiglu_properties(cuda):
    # src/mlp/swiglu_tests.rs:329-372
    from rocmforge_amd import ops
    z = host(ops.swiglu(dev(np.array([[1, 2, 3]], np.float32), cuda), dev(np.zeros((1, 3), np.float32), cuda)))
    assert np.all(np.abs(z) < 1e-6)
    big = host(ops.swiglu(dev(np.ones((1, 3), np.float32), cuda), dev(np.array([[10, 20, 30]], np.float32), cuda)))
    assert np.all(np.abs(big - [10, 20, 30]) < 0.1)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("rows,hidden", [(1, 256), (5, 1024), (64, 4096)])
def test_dequant_rms_norm(fmt, rows, hidden, oracle, cuda):
    from rocmforge_amd import ops
    packed = Q.make_weights(fmt, rows, hidden, seed=700 + fmt + rows)
    w = norm_weight(hidden, 710 + hidden)
    got = host(ops.dequant_rms_norm(fmt, dev(packed, cuda), dev(w, cuda), rows, hidden, 1e-5))
    assert_close(got, oracle.dequant_rms_norm(fmt, packed, w, rows, hidden, 1e-5), f"{Q.NAMES[fmt]} {rows}x{hidden}",
                 tol=ELEMENTWISE_TOL)


# k = 768 ... 14336: the one-launch kernels at every units-per-lane x wavefronts-per-row
# shape; 512 and 32768 have no such kernel and run norm, then GEMV.
@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("n,k", [(40, 512), (77, 768), (64, 2048), (1001, 2048), (130, 4096), (257, 8192), (19, 14336),
                                 (9, 32768), (2048, 1536)])
def test_rms_norm_gemv_m1(fmt, n, k, oracle, cuda):
    from rocmforge_amd import ops
    w = Q.make_weights(fmt, n, k, seed=800 + fmt + n)
    x, nw = gauss((k,), 810 + k, 2.5), norm_weight(k, 820 + k)
    got = host(ops.rms_norm_gemv(fmt, dev(w, cuda), dev(x, cuda), dev(nw, cuda), 1e-5, n, k))
    want = oracle.qmatmul_nk(fmt, w, oracle.rms_norm(x[None, :], nw, 1e-5), 1, n, k)[0]
    assert_close(got, want, f"{Q.NAMES[fmt]} n={n} k={k}")


def test_rms_norm_gemv_one_launch_needs_no_scratch(oracle, cuda):
    from rocmforge_amd import _lib, ops
    n, k = 64, 4096
    w = Q.make_weights(Q.Q4_K, n, k, seed=830)
    x, nw = gauss((k,), 831), norm_weight(k, 832)
    got = host(ops.rms_norm_gemv(Q.Q4_K, dev(w, cuda), dev(x, cuda), dev(nw, cuda), 1e-5, n, k, scratch=False))
    assert_close(got, oracle.qmatmul_nk(Q.Q4_K, w, oracle.rms_norm(x[None, :], nw, 1e-5), 1, n, k)[0], "no scratch")
    with pytest.raises(_lib.RfqError) as e:     # a batch has no one-launch kernel
        ops.rms_norm_gemv(Q.Q4_K, dev(w, cuda), dev(gauss((2, k), 833), cuda), dev(nw, cuda), 1e-5, n, k, scratch=False)
    assert e.value.status == _lib.E_BADARG


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m", [2, 8])
def test_rms_norm_gemv_batches(fmt, m, oracle, cuda):
    from rocmforge_amd import ops
    n, k = 301, 2048
    w = Q.make_weights(fmt, n, k, seed=840 + fmt)
    x, nw = gauss((m, k), 850 + m, 0.5), norm_weight(k, 860)
    got = host(ops.rms_norm_gemv(fmt, dev(w, cuda), dev(x, cuda), dev(nw, cuda), 1e-6, n, k))
    assert_close(got, oracle.qmatmul_nk(fmt, w, oracle.rms_norm(x, nw, 1e-6), m, n, k), f"{Q.NAMES[fmt]} m={m}")


def mlp_case(fmt_gu, fmt_d, m, hidden, inter, with_norm, seed, oracle, cuda):
    from rocmforge_amd import ops
    wg = Q.make_weights(fmt_gu, inter, hidden, seed=seed)
    wu = Q.make_weights(fmt_gu, inter, hidden, seed=seed + 1)
    wd = Q.make_weights(fmt_d, hidden, inter, seed=seed + 2)
    x = gauss((m, hidden), seed + 3)
    nw = norm_weight(hidden, seed + 4) if with_norm else None
    xin = dev(x[0] if m == 1 else x, cuda)
    got = host(ops.mlp_swiglu(fmt_gu, dev(wg, cuda), dev(wu, cuda), fmt_d, dev(wd, cuda), xin,
                              dev(nw, cuda) if with_norm else None, 1e-5, hidden, inter)).reshape(m, hidden)
    want = oracle.mlp_swiglu_q(fmt_gu, wg, wu, fmt_d, wd, x, nw, 1e-5, m, hidden, inter)
    return assert_close(got, want, f"mlp {Q.NAMES[fmt_gu]}/{Q.NAMES[fmt_d]} m={m} {hidden}x{inter} norm={with_norm}")


# inter values give odd and even row groups per team, ragged last teams, and
# every wavefronts-per-row shape for the gate/up pass (hidden) and the down pass (inter)
@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("hidden,inter", [(768, 1024), (2048, 5632), (4096, 1536), (1024, 14336), (8192, 1280)])
@pytest.mark.parametrize("with_norm", [False, True])
def test_mlp_swiglu_m1(fmt, hidden, inter, with_norm, oracle, cuda):
    mlp_case(fmt, fmt, 1, hidden, inter, with_norm, 900 + fmt + hidden, oracle, cuda)


@pytest.mark.parametrize("inter", [1280, 3, 7, 64, 1000])
def test_mlp_swiglu_m1_row_counts(inter, oracle, cuda):
    # few and odd numbers of gate/up pairs; the down projection then has a short or ragged k
    inter_k = (inter + 31) // 32 * 32
    mlp_case(Q.Q4_0, Q.Q8_0, 1, 1024, inter_k, True, 950 + inter, oracle, cuda)


def test_mlp_swiglu_mixed_formats(oracle, cuda):
    mlp_case(Q.Q4_K, Q.Q6_K, 1, 2048, 2816, True, 960, oracle, cuda)
    mlp_case(Q.MXFP4, Q.Q8_0, 1, 2048, 2816, False, 961, oracle, cuda)


@pytest.mark.parametrize("fmt", [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K])
@pytest.mark.parametrize("m", [2, 8])
def test_mlp_swiglu_batches(fmt, m, oracle, cuda):
    mlp_case(fmt, fmt, m, 1024, 1536, True, 970 + fmt + m, oracle, cuda)


def test_mlp_swiglu_at_the_llama_shape(oracle, cuda):
    # hidden 4096, intermediate 14336, Q4_K: the shape the GEMV headline is quoted on
    e = mlp_case(Q.Q4_K, Q.Q4_K, 1, 4096, 14336, True, 980, oracle, cuda)
    assert e < 1e-3


def test_mlp_rejects_bad_arguments(cuda):
    import torch
    from rocmforge_amd import _lib, ops
    hidden, inter = 1024, 1536
    wg = dev(Q.make_weights(Q.Q4_0, inter, hidden, seed=1), cuda)
    wd = dev(Q.make_weights(Q.Q4_0, hidden, inter, seed=2), cuda)
    x = dev(gauss((hidden,), 3), cuda)
    with pytest.raises(_lib.RfqError) as e:   # scratch too small
        ops.mlp_swiglu(Q.Q4_0, wg, wg, Q.Q4_0, wd, x, None, 1e-5, hidden, inter,
                       scratch=torch.empty(64, dtype=torch.uint8, device=cuda))
    assert e.value.status == _lib.E_SIZE
    with pytest.raises(_lib.RfqError) as e:   # down matrix of the wrong size
        ops.mlp_swiglu(Q.Q4_0, wg, wg, Q.Q4_0, wd[:-20], x, None, 1e-5, hidden, inter)
    assert e.value.status == _lib.E_SIZE
    with pytest.raises(_lib.RfqError) as e:   # more rows than the decode kernels take
        ops.mlp_swiglu(Q.Q4_0, wg, wg, Q.Q4_0, wd, dev(gauss((9, hidden), 4), cuda), None, 1e-5, hidden, inter)
    assert e.value.status == _lib.E_UNSUPPORTED
