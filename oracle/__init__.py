"""ctypes front-end to the CPU oracle (``rf_oracle.c``).

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the bench's
``cpu_baseline`` leg import this module; the shipped package never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librf_oracle.so")

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, MXFP4, MXFP6_E2M3, MXFP6_E3M2 = 0, 1, 2, 8, 12, 14, 20, 21, 22
# the decoders of src/kernels/matmul/quantized/ (q8_0.rs:18-56, q4_k.rs:90-148, q6_k.rs:90-148)
MM_Q8_0, MM_Q4_K, MM_Q6_K = 208, 212, 214


def build(force: bool = False) -> str:
    """Compile rf_oracle.c with gcc (see oracle/Makefile)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        u8p, f32p, sz = C.c_void_p, C.c_void_p, C.c_size_t
        for name in ("q4_0", "q8_0", "q4_k", "q6_k", "mxfp4", "mxfp6", "mm_q8_0", "mm_q4_k", "mm_q6_k"):
            fn = getattr(L, "rf_dequant_" + name)
            fn.argtypes = [u8p, sz, sz, f32p]
            fn.restype = None
        L.rf_dequantize.argtypes = [C.c_int, u8p, sz, sz, f32p]
        L.rf_dequantize.restype = C.c_int
        L.rf_f16_to_f32.argtypes = [C.c_uint16]
        L.rf_f16_to_f32.restype = C.c_float
        L.rf_f16_to_f32_mm.argtypes = [C.c_uint16]
        L.rf_f16_to_f32_mm.restype = C.c_float
        L.rf_qmatmul_kn.argtypes = [C.c_int, u8p, sz, f32p, sz, sz, sz, f32p, f32p]
        L.rf_qmatmul_kn.restype = C.c_int
        L.rf_powi_f32.argtypes = [C.c_float, C.c_int]
        L.rf_powi_f32.restype = C.c_float
        for name in ("rf_decode_e2m1", "rf_decode_e2m3"):
            getattr(L, name).argtypes = [C.c_uint8]
            getattr(L, name).restype = C.c_float
        for name in ("rf_encode_e2m1", "rf_encode_e2m3"):
            getattr(L, name).argtypes = [C.c_float]
            getattr(L, name).restype = C.c_uint8
        L.rf_e8m0_from_f32.argtypes = [C.c_float]
        L.rf_e8m0_from_f32.restype = C.c_int8
        L.rf_e8m0_to_f32.argtypes = [C.c_int8]
        L.rf_e8m0_to_f32.restype = C.c_float
        L.rf_pack_6bit.argtypes = [u8p, sz, u8p]
        L.rf_unpack_6bit.argtypes = [u8p, sz, sz, u8p]
        L.rf_pack_mxfp4.argtypes = [f32p, sz, u8p]
        L.rf_pack_mxfp6.argtypes = [f32p, sz, u8p]
        L.rf_unpack_mxfp4.argtypes = [u8p, f32p]
        L.rf_unpack_mxfp6.argtypes = [u8p, f32p]
        L.rf_data_size.argtypes = [C.c_int, sz]
        L.rf_data_size.restype = sz
        L.rf_block_bytes.argtypes = [C.c_int]
        L.rf_block_bytes.restype = sz
        L.rf_cpu_matmul_f32.argtypes = [f32p, f32p, sz, sz, sz, f32p]
        L.rf_matmul_nk_f32.argtypes = [f32p, f32p, sz, sz, sz, f32p]
        L.rf_qmatmul_nk.argtypes = [C.c_int, u8p, sz, f32p, sz, sz, sz, C.c_void_p, sz, f32p]
        L.rf_qmatmul_nk.restype = C.c_int
        L.rf_rms_norm.argtypes = [f32p, f32p, sz, sz, C.c_float, f32p]
        L.rf_swiglu.argtypes = [f32p, f32p, sz, f32p]
        L.rf_dequant_rms_norm.argtypes = [C.c_int, u8p, sz, f32p, sz, sz, C.c_float, f32p]
        L.rf_mlp_swiglu_q.argtypes = [C.c_int, u8p, u8p, sz, C.c_int, u8p, sz, f32p, f32p, C.c_float, sz, sz, sz,
                                      f32p, f32p]
        L.rf_qmatmul_nk_staged.argtypes = [C.c_int, u8p, sz, f32p, sz, sz, sz, f32p, f32p]
        L.rf_qmatmul_nk_staged.restype = C.c_int
        _lib = L
    return _lib


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(np.frombuffer(bytes(a), dtype=np.uint8) if not isinstance(a, np.ndarray) else a, dtype=np.uint8)


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def block_elems(fmt: int) -> int:
    return 256 if fmt in (10, 11, Q4_K, 13, Q6_K, 112, 114, MM_Q4_K, MM_Q6_K) else 32


def block_bytes(fmt: int) -> int:
    return int(lib().rf_block_bytes(fmt))


def dequantize(fmt: int, data, n: int) -> np.ndarray:
    """loader::dequantize on raw bytes -> float32[n]."""
    d = _u8(data)
    out = np.empty(n, dtype=np.float32)
    rc = lib().rf_dequantize(fmt, _p(d), d.size, n, _p(out))
    if rc != 0:
        raise ValueError(f"format {fmt} is not on the oracle's path")
    return out


def cpu_matmul_f32(a: np.ndarray, b: np.ndarray, m: int, n: int, k: int) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    assert a.size == m * k and b.size == k * n
    c = np.empty(m * n, dtype=np.float32)
    lib().rf_cpu_matmul_f32(_p(a), _p(b), m, n, k, _p(c))
    return c.reshape(m, n)


def matmul_nk_f32(a: np.ndarray, w: np.ndarray, m: int, n: int, k: int) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    assert a.size == m * k and w.size == n * k
    c = np.empty(m * n, dtype=np.float32)
    lib().rf_matmul_nk_f32(_p(a), _p(w), m, n, k, _p(c))
    return c.reshape(m, n)


def qmatmul_nk(fmt: int, w_bytes, a: np.ndarray, m: int, n: int, k: int, rows=None) -> np.ndarray:
    """y[m, n] = a[m,k] . dequant(W[n,k])^T, fp32 sequential in k.  ``rows``
    restricts the computed output columns (returns [m, len(rows)])."""
    w = _u8(w_bytes)
    a = np.ascontiguousarray(a, dtype=np.float32)
    assert a.size == m * k
    if rows is None:
        c = np.empty((m, n), dtype=np.float32)
        rc = lib().rf_qmatmul_nk(fmt, _p(w), w.size, _p(a), m, n, k, None, 0, _p(c))
    else:
        r = np.ascontiguousarray(rows, dtype=np.int64)
        c = np.empty((m, r.size), dtype=np.float32)
        rc = lib().rf_qmatmul_nk(fmt, _p(w), w.size, _p(a), m, n, k, _p(r), r.size, _p(c))
    if rc != 0:
        raise ValueError(f"rf_qmatmul_nk failed rc={rc}")
    return c


def qmatmul_kn(fmt: int, w_bytes, a: np.ndarray, m: int, n: int, k: int) -> np.ndarray:
    """c[m, n] = a[m, k] . Wd[k, n] where Wd is the packed stream dequantised as one flat array of n * k
    elements and read as b[l * n + j]: what matmul_q4_0_cpu_fallback and the fused kernel compute
    (src/kernels/matmul/quantized/q4_0.rs:274-311, src/tensor/matmul.rs:219-233)."""
    w = _u8(w_bytes)
    a = np.ascontiguousarray(a, dtype=np.float32)
    assert a.size == m * k
    wd = np.empty(n * k, dtype=np.float32)
    c = np.empty((m, n), dtype=np.float32)
    rc = lib().rf_qmatmul_kn(fmt, _p(w), w.size, _p(a), m, n, k, _p(wd), _p(c))
    if rc != 0:
        raise ValueError(f"rf_qmatmul_kn failed rc={rc}")
    return c


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """RMSNorm over the last axis of x[rows, hidden] (src/mlp/rms_norm_tests.rs:44-73)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    rows, hidden = x.reshape(-1, x.shape[-1]).shape
    assert w.size == hidden
    out = np.empty_like(x)
    lib().rf_rms_norm(_p(x), _p(w), rows, hidden, eps, _p(out))
    return out


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """gate * (up * sigmoid(up)), the reference's definition (src/mlp/swiglu_tests.rs:43-66)."""
    g = np.ascontiguousarray(gate, dtype=np.float32)
    u = np.ascontiguousarray(up, dtype=np.float32)
    assert g.shape == u.shape
    out = np.empty_like(g)
    lib().rf_swiglu(_p(g), _p(u), g.size, _p(out))
    return out


def dequant_rms_norm(fmt: int, packed, weight: np.ndarray, rows: int, hidden: int, eps: float) -> np.ndarray:
    """Dequantise packed[rows, hidden], then RMSNorm each row (src/ggml/hip_backend/ops/fused_ops.rs:149-160)."""
    d = _u8(packed)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    assert w.size == hidden
    out = np.empty((rows, hidden), dtype=np.float32)
    rc = lib().rf_dequant_rms_norm(fmt, _p(d), d.size, _p(w), rows, hidden, eps, _p(out))
    if rc != 0:
        raise ValueError(f"rf_dequant_rms_norm failed rc={rc}")
    return out


def mlp_swiglu_q(fmt_gu: int, wg, wu, fmt_d: int, wd, x: np.ndarray, norm_weight, eps: float, m: int, hidden: int,
                 inter: int) -> np.ndarray:
    """out[m, hidden] = swiglu(xn.Wg^T, xn.Wu^T).Wd^T with xn = rms_norm(x) when norm_weight is given, else x
    (src/backend/hip_backend/backend.rs:1153-1278 over quantised [outputs, k] matrices)."""
    wg, wu, wd = _u8(wg), _u8(wu), _u8(wd)
    assert wg.size == wu.size
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size == m * hidden
    nw = None if norm_weight is None else np.ascontiguousarray(norm_weight, dtype=np.float32)
    scratch = np.empty(m * (hidden + 3 * inter), dtype=np.float32)
    out = np.empty((m, hidden), dtype=np.float32)
    rc = lib().rf_mlp_swiglu_q(fmt_gu, _p(wg), _p(wu), wg.size, fmt_d, _p(wd), wd.size, _p(x),
                               None if nw is None else _p(nw), eps, m, hidden, inter, _p(scratch), _p(out))
    if rc != 0:
        raise ValueError(f"rf_mlp_swiglu_q failed rc={rc}")
    return out


def get_rows(fmt: int, table, tokens, n_vocab: int, n_embd: int):
    """get_rows (src/ggml/hip_backend/ops/get_rows.rs:6-53, RowMajor) over a
    table that is dequantised first (fmt != 0) or already f32 (fmt == 0):
    out[i, :] = table[tokens[i], :].  Returns (out, bad) where bad is None or
    the index of the first token id >= n_vocab; the reference stops with an
    error there (:18-23), rows from that index on are returned as zero."""
    tokens = np.asarray(tokens, dtype=np.int64)
    if fmt == 0:
        tab = np.ascontiguousarray(table, dtype=np.float32).reshape(n_vocab, n_embd)
    else:
        tab = None
        d = _u8(table)
        row_bytes = n_embd // block_elems(fmt) * block_bytes(fmt)
    out = np.zeros((tokens.size, n_embd), dtype=np.float32)
    bad = None
    for i, t in enumerate(tokens):
        if t >= n_vocab or t < 0:
            if bad is None:
                bad = i
            continue
        out[i] = tab[t] if tab is not None else dequantize(fmt, d[t * row_bytes:(t + 1) * row_bytes], n_embd)
    return out, bad


def pack_mxfp4(values: np.ndarray) -> np.ndarray:
    """MxfpBlock::pack_mxfp4 over consecutive 32-element blocks -> bytes."""
    v = np.ascontiguousarray(values, dtype=np.float32).ravel()
    nb = (v.size + 31) // 32
    out = np.zeros(nb * 17, dtype=np.uint8)
    L = lib()
    for b in range(nb):
        chunk = np.ascontiguousarray(v[b * 32:(b + 1) * 32])
        L.rf_pack_mxfp4(_p(chunk), chunk.size, C.c_void_p(out.ctypes.data + b * 17))
    return out


def pack_mxfp6(values: np.ndarray) -> np.ndarray:
    v = np.ascontiguousarray(values, dtype=np.float32).ravel()
    nb = (v.size + 31) // 32
    out = np.zeros(nb * 25, dtype=np.uint8)
    L = lib()
    for b in range(nb):
        chunk = np.ascontiguousarray(v[b * 32:(b + 1) * 32])
        L.rf_pack_mxfp6(_p(chunk), chunk.size, C.c_void_p(out.ctypes.data + b * 25))
    return out


def unpack_mxfp4(block17) -> np.ndarray:
    b = _u8(block17)
    out = np.empty(32, dtype=np.float32)
    lib().rf_unpack_mxfp4(_p(b), _p(out))
    return out


def unpack_mxfp6(block25) -> np.ndarray:
    b = _u8(block25)
    out = np.empty(32, dtype=np.float32)
    lib().rf_unpack_mxfp6(_p(b), _p(out))
    return out


def pack_6bit(values) -> np.ndarray:
    v = _u8(np.asarray(values, dtype=np.uint8))
    out = np.zeros((v.size * 6 + 7) // 8, dtype=np.uint8)
    lib().rf_pack_6bit(_p(v), v.size, _p(out))
    return out


def unpack_6bit(packed, count: int) -> np.ndarray:
    p = _u8(packed)
    out = np.zeros(count, dtype=np.uint8)
    lib().rf_unpack_6bit(_p(p), p.size, count, _p(out))
    return out
