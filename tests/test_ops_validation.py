"""The torch wrappers refuse tensors that would become out-of-bounds device accesses: wrong device, dtype, layout
or shape raise ValueError before any library call."""
import numpy as np
import pytest
import torch

from rocmforge_amd import ops, quantize as Q


def test_host_tensors_are_refused():
    w = torch.zeros(20, dtype=torch.uint8)
    x = torch.zeros(32, dtype=torch.float32)
    with pytest.raises(ValueError):
        ops.gemv(Q.Q4_0, w, x, 1, 32)
    with pytest.raises(ValueError):
        ops.gemv_kn(Q.Q4_0, w, x, 1, 32)
    with pytest.raises(ValueError):
        ops.dequant(Q.Q4_0, w, 32)
    with pytest.raises(ValueError):
        ops.get_rows(Q.Q4_0, w, torch.zeros(1, dtype=torch.int32), 1, 32)
    with pytest.raises(ValueError):
        ops.rms_norm(x, x, 1e-5)
    with pytest.raises(ValueError):
        ops.gemm_f16(Q.Q4_0, w, torch.zeros((1, 32), dtype=torch.float16), 1, 32)


@pytest.mark.gpu
def test_mismatched_shapes_and_buffers_are_refused(cuda):
    n, k = 8, 64
    w = torch.from_numpy(Q.make_weights(Q.Q4_0, n, k, seed=1)).to(cuda)
    x = torch.zeros((2, k), dtype=torch.float32, device=cuda)
    assert ops.gemv(Q.Q4_0, w, x, n, k).shape == (2, n)
    with pytest.raises(ValueError):
        ops.gemv(Q.Q4_0, w, x[:, :32].contiguous(), n, k)                     # x has 32 columns, k = 64
    with pytest.raises(ValueError):
        ops.gemv(Q.Q4_0, w, x, n, k, out=torch.empty((2, n - 1), dtype=torch.float32, device=cuda))
    with pytest.raises(ValueError):
        ops.gemv(Q.Q4_0, w, x, n, k, out=torch.empty((2, n), dtype=torch.float16, device=cuda))
    with pytest.raises(ValueError):
        ops.gemv(Q.Q4_0, w, x.double(), n, k)
    with pytest.raises(ValueError):
        ops.dequant(Q.Q4_0, w, n * k, out=torch.empty(n * k - 1, dtype=torch.float32, device=cuda))
    tok = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(ValueError):
        ops.get_rows(Q.Q4_0, w, tok, n, k)                                    # token ids on the host
    with pytest.raises(ValueError):
        ops.get_rows(Q.Q4_0, w, tok.to(cuda), n, k, status=torch.zeros(1, dtype=torch.int32))
    a = torch.zeros((4, k), dtype=torch.float16, device=cuda)
    with pytest.raises(ValueError):
        ops.gemm_f16(Q.Q4_0, w, a[:, :32].contiguous(), n, k)
    with pytest.raises(ValueError):
        ops.gemm_f16(Q.Q4_0, w, a, n, k, out=torch.empty((4, n), dtype=torch.float32, device=cuda))   # fp16 out asked
    with pytest.raises(ValueError):
        ops.rms_norm(x, torch.ones(k - 1, dtype=torch.float32, device=cuda), 1e-5)
    with pytest.raises(ValueError):
        ops.rms_norm_gemv(Q.Q4_0, w, x, torch.ones(k + 1, dtype=torch.float32, device=cuda), 1e-5, n, k)
    # a prepared operand used with a larger shape than it was prepared for
    raw = torch.from_numpy(Q.pack_mxfp4(np.ones((32, 128), dtype=np.float32))).to(cuda)
    A = ops.MxOperand(Q.MXFP4, raw, 32, 128)
    W = ops.MxOperand(Q.MXFP4, raw, 32, 128)
    assert ops.gemm_mx(A, W, torch.float32).shape == (32, 32)
    A.rows = 64
    with pytest.raises(RuntimeError):
        ops.gemm_mx(A, W, torch.float32)
