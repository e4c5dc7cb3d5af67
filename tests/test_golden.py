"""Committed golden vectors (tests/golden/vectors.npz, written by
tests/golden/make_golden.py): the oracle must still reproduce them, and the
GPU path must match them without the oracle being present."""
import os

import numpy as np
import pytest

from helpers import assert_bit_exact, assert_close
from rocmforge_amd import quantize as Q

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz")
FORMATS = [Q.Q4_0, Q.Q8_0, Q.Q4_K, Q.Q6_K, Q.MXFP4, Q.MXFP6_E2M3, Q.GGUF_Q4_0, Q.GGUF_Q8_0, Q.GGUF_Q4_K, Q.GGUF_Q6_K]
MLP_FORMATS = [Q.Q4_0, Q.GGUF_Q4_K]
HIDDEN, INTER = 768, 256
N, K, M = 16, 256, 2


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)            # plain arrays only (allow_pickle stays False)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("tag", ["gen", "raw"])
def test_oracle_reproduces_the_golden_vectors(fmt, tag, golden, oracle):
    name = Q.NAMES[fmt]
    blob = golden[f"{name}.{tag}.bytes"]
    assert blob.size == Q.packed_bytes(fmt, N * K)
    assert_bit_exact(oracle.dequantize(fmt, blob, N * K), golden[f"{name}.{tag}.dequant"], f"{name} {tag} dequant")
    y = oracle.qmatmul_nk(fmt, blob, golden[f"{name}.x"], M, N, K)
    assert_bit_exact(y, golden[f"{name}.{tag}.gemv"], f"{name} {tag} gemv")


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("tag", ["gen", "raw"])
def test_gpu_matches_the_golden_vectors(fmt, tag, golden, cuda):
    import torch
    from rocmforge_amd import ops
    name = Q.NAMES[fmt]
    blob = torch.from_numpy(golden[f"{name}.{tag}.bytes"]).to(cuda)
    got = ops.dequant(fmt, blob, N * K).cpu().numpy()
    assert_bit_exact(got, golden[f"{name}.{tag}.dequant"], f"{name} {tag} dequant on the GPU")
    x = torch.from_numpy(golden[f"{name}.x"]).to(cuda)
    y = ops.gemv(fmt, blob, x, N, K).cpu().numpy()
    assert_close(y, golden[f"{name}.{tag}.gemv"], f"{name} {tag} gemv on the GPU")


def test_oracle_reproduces_the_golden_mlp_vectors(golden, oracle):
    x, nw = golden["mlp.x"], golden["mlp.norm_weight"]
    assert_bit_exact(oracle.rms_norm(x, nw, 1e-5), golden["rms_norm.out"], "rms_norm")
    assert_bit_exact(oracle.swiglu(golden["swiglu.gate"], golden["swiglu.up"]), golden["swiglu.out"], "swiglu")
    for fmt in MLP_FORMATS:
        n = Q.NAMES[fmt]
        y = oracle.mlp_swiglu_q(fmt, golden[f"mlp.{n}.gate"], golden[f"mlp.{n}.up"], fmt, golden[f"mlp.{n}.down"], x, nw, 1e-5,
                                M, HIDDEN, INTER)
        assert_bit_exact(y, golden[f"mlp.{n}.out"], f"mlp {n}")


@pytest.mark.gpu
def test_gpu_matches_the_golden_mlp_vectors(golden, cuda):
    import torch
    from rocmforge_amd import ops
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    x, nw = t(golden["mlp.x"]), t(golden["mlp.norm_weight"])
    assert_close(ops.rms_norm(x, nw, 1e-5).cpu().numpy(), golden["rms_norm.out"], "rms_norm on the GPU", tol=1e-5)
    assert_close(ops.swiglu(t(golden["swiglu.gate"]), t(golden["swiglu.up"])).cpu().numpy(), golden["swiglu.out"],
                 "swiglu on the GPU", tol=1e-5)
    for fmt in MLP_FORMATS:
        n = Q.NAMES[fmt]
        for rows in (1, M):                      # the two-launch form and the separate-launch form
            xin = x[0].contiguous() if rows == 1 else x
            y = ops.mlp_swiglu(fmt, t(golden[f"mlp.{n}.gate"]), t(golden[f"mlp.{n}.up"]), fmt, t(golden[f"mlp.{n}.down"]), xin, nw,
                               1e-5, HIDDEN, INTER).cpu().numpy().reshape(rows, HIDDEN)
            assert_close(y, golden[f"mlp.{n}.out"][:rows], f"mlp {n} m={rows} on the GPU")
