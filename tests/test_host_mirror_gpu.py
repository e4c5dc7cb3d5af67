"""Runs the C++ host tests of include/rocmforge_rfq.hpp (the mirror of the
reference's operator surface) on the GPU: tests/host/test_host_mirror.cpp,
built by `make -C tests/host` (also done by __graft_entry__.build())."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "host", "build", "test_host_mirror")


@pytest.mark.gpu
def test_cpp_host_mirror(cuda):
    assert os.path.exists(BINARY), f"{BINARY} is missing: run make -C tests/host"
    p = subprocess.run([BINARY], capture_output=True, text=True, timeout=120)
    print(p.stdout)
    print(p.stderr)
    assert p.returncode == 0, p.stdout[-4000:]
    assert "0 test(s) failed" in p.stdout


def test_mirror_header_names_the_reference_surface():
    """CPU-side check: the header declares every function and type the
    reference's benches and tests use on this path."""
    text = open(os.path.join(os.path.dirname(HERE), "include", "rocmforge_rfq.hpp")).read()
    for name in ("GgufTensorType", "TensorShape", "GgufTensor", "dequant_q4_0", "dequant_q8_0", "dequant_q4_k",
                 "dequant_q6_k", "dequant_mxfp4", "dequant_mxfp6", "dequantize", "HipBuffer", "HipBackend",
                 "matmul_q4_0", "matmul_q8_0", "matmul_q4_k", "matmul_q6_k", "matmul_q4_0_gpu",
                 "dequantize_q4_0_kernel_cached", "dequantize_q4_k_gpu_kernel", "dequantize_q6_k_gpu_kernel",
                 "QuantFormat", "QuantizedMatmulOp", "validate_matmul_q4_0", "validate_matmul_q8_0", "get_rows",
                 "validate_token_ids", "rms_norm_gpu_kernel", "swiglu_gpu_kernel", "fused_q4_0_rmsnorm", "DeviceTensor",
                 "mlp_swiglu", "execute_matmul_quantized", "MatMulQ4_K", "MatMulMxfp4", "BatchQuantizedMatmul",
                 "BatchMatmulResult"):
        assert name in text, name
