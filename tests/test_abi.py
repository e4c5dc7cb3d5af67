"""The C-ABI library loads without a GPU and exports every symbol that
include/rfq.h declares; host-side argument validation works without a device."""
import ctypes as C
import os
import re

import rocmforge_amd
from rocmforge_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = "".join(open(os.path.join(ROOT, "include", f)).read() for f in sorted(os.listdir(os.path.join(ROOT, "include")))
                   if f.endswith(".h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"RFQ_API\s+[\w\s\*]+?\b(rfq_\w+)\s*\(", text)))


def test_header_symbols_exported():
    names = declared_symbols()
    assert len(names) >= 18, names
    L = C.CDLL(rocmforge_amd.lib_path())
    for n in names:
        assert hasattr(L, n), f"{n} declared in rfq.h but not exported"
    assert set(names) == set(_lib._SIGNATURES), "binding and header disagree"


def test_sizes_and_version():
    L = rocmforge_amd.lib()
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "rfq.h")).read()
    crate = open(os.path.join(os.path.dirname(__file__), "..", "rust", "rocmforge-mi355-sys", "src", "lib.rs")).read()
    declared = int(re.search(r"#define\s+RFQ_VERSION\s+(\d+)", header).group(1))
    assert L.rfq_version() == declared == int(re.search(r"RFQ_VERSION: c_int = (\d+);", crate).group(1))
    assert declared >= 102
    assert [L.rfq_block_bytes(f) for f in (2, 8, 12, 14, 20, 21, 22)] == [20, 36, 256, 256, 17, 25, 25]
    assert [L.rfq_block_elems(f) for f in (2, 8, 12, 14, 20, 21, 22)] == [32, 32, 256, 256, 32, 32, 32]
    assert L.rfq_block_bytes(3) == 0 and L.rfq_block_elems(99) == 0
    assert L.rfq_packed_bytes(2, 4864 * 896) == 2723840           # Q4_0 4864 x 896
    assert L.rfq_packed_bytes(8, 4096 * 4096) == 18874368
    assert L.rfq_packed_bytes(12, 14336 * 4096) == 58720256
    assert L.rfq_packed_bytes(20, 28672 * 8192) == 124780544
    assert L.rfq_packed_bytes(21, 28672 * 8192) == 183500800
    assert L.rfq_packed_bytes(12, 100) == 256 and L.rfq_packed_bytes(2, 33) == 40


def test_validation_needs_no_device():
    L = rocmforge_amd.lib()
    one = C.c_void_p(16)  # never dereferenced: every call below fails validation first
    assert L.rfq_dequant(99, one, 20, one, 32, None) == _lib.E_BADARG
    assert b"unknown format" in L.rfq_last_error()
    assert L.rfq_dequant(2, one, 20, None, 32, None) == _lib.E_BADARG
    assert L.rfq_dequant(2, None, 0, None, 0, None) == _lib.OK            # nothing to do
    assert L.rfq_gemv(2, None, 0, one, one, 1, 4, 32, None) == _lib.E_BADARG
    assert L.rfq_gemv(2, one, 80, one, one, 0, 4, 32, None) == _lib.E_BADARG   # m = 0
    assert L.rfq_gemv(2, one, 80, one, one, 1, 4, 33, None) == _lib.E_SIZE     # k % 32
    assert L.rfq_gemv(12, one, 1024, one, one, 1, 4, 128, None) == _lib.E_SIZE  # k % 256
    assert L.rfq_gemv(2, one, 81, one, one, 1, 4, 32, None) == _lib.E_SIZE     # byte count
    assert b"needs 80" in L.rfq_last_error()
    assert L.rfq_matmul_q4_0(one, one, one, 9, 4, 32, None) == _lib.E_UNSUPPORTED   # the raw launch takes m <= 8
    assert L.rfq_mlp_swiglu(2, one, one, 80, 2, one, 80, one, None, 0.0, one, 9, 32, 4, one, 1 << 20, None) == _lib.E_SIZE
    assert L.rfq_matmul_q4_0(one, one, one, 1, 0, 32, None) == _lib.E_BADARG
    assert L.rfq_matmul_host_weights(2, one, 80, one, 0, 32, one, None) == _lib.E_BADARG
    assert L.rfq_gemm_f16(12, one, 256, one, one, 2, 1, 1, 256, None) == _lib.E_BADARG  # bf16 out
    assert L.rfq_mx_prepare(12, 0, one, 17, 1, 128, one, 64, None, None) == _lib.E_BADARG
    assert L.rfq_mx_prepare(20, 0, one, 68, 1, 100, one, 64, None, None) == _lib.E_SIZE
    pb = L.rfq_mx_prepared_bytes(20, 4, 32, 128)
    assert L.rfq_gemm_mx(one, pb, 4, one, pb, 4, one, 1, 32, 32, 128, None) == _lib.E_BADARG     # f16 out
    assert L.rfq_gemm_mx(one, pb, 5, one, pb, 4, one, 0, 32, 32, 128, None) == _lib.E_BADARG
    assert L.rfq_gemm_mx(one, pb, 4, one, pb, 4, one, 0, 64, 32, 128, None) == _lib.E_SIZE       # A was prepared for 32 rows
    assert b"prepared A" in L.rfq_last_error()
    assert L.rfq_gemm_mx(one, pb, 4, one, pb - 16, 4, one, 0, 32, 32, 128, None) == _lib.E_SIZE
    assert b"prepared W" in L.rfq_last_error()


def test_empty_inputs_are_accepted_without_touching_the_device():
    """Zero elements / zero tokens: the reference's loops run zero times (dequantize_q4_0_cpu with n = 0 returns an
    empty vector, src/kernels/quant/q4_0.rs:266-310); here the calls return before any device work."""
    L = _lib.lib()
    for fmt in (2, 8, 12, 14, 20, 21, 102, 112, 208, 212):
        assert L.rfq_dequant(fmt, None, 0, None, 0, None) == _lib.OK
        assert L.rfq_dequant_host(fmt, None, 0, None, 0) == _lib.OK
        assert L.rfq_dequant_upload(fmt, None, 0, None, 0, None) == _lib.OK
    assert L.rfq_get_rows(12, None, 256 * 16, 1, 4096, None, 0, None, None, None) == _lib.OK
    assert L.rfq_upload(None, 0, None, None) == _lib.OK
    assert L.rfq_packed_bytes(12, 0) == 0
