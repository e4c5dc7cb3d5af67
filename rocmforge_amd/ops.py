"""Device-side operators over torch tensors (torch is only the allocator and
the stream here; every computation is a librfq call).

Mirrors the raw-pointer layer of ROCmForge's kernel wrappers:
``matmul_q4_0_gpu`` and twins (src/kernels/matmul/quantized/q4_0.rs:209-260)
and the dequant launches (src/kernels/quant/q4_0.rs:107-153).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib
from .quantize import BLOCK_BYTES, BLOCK_ELEMS


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: torch.Tensor) -> C.c_void_p:
    return C.c_void_p(t.data_ptr())


def _dev_u8(t: torch.Tensor) -> torch.Tensor:
    if not (t.is_cuda and t.dtype == torch.uint8 and t.is_contiguous()):
        raise ValueError("packed weights must be a contiguous uint8 device tensor")
    return t


def _f32(t: torch.Tensor, what: str) -> torch.Tensor:
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise ValueError(f"{what} must be a contiguous float32 device tensor")
    return t


def _rows_of(x: torch.Tensor, k: int, what: str) -> int:
    """Rows of x[m, k] (or of a single vector x[k]); the last axis must be k."""
    if x.dim() not in (1, 2) or x.shape[-1] != k:
        raise ValueError(f"{what} has shape {tuple(x.shape)}, expected [m, {k}] or [{k}]")
    return 1 if x.dim() == 1 else x.shape[0]


def _out(out: torch.Tensor | None, shape, dtype, like: torch.Tensor) -> torch.Tensor:
    """The caller's output buffer, checked, or a new one on the device of `like`."""
    if out is None:
        return torch.empty(shape, dtype=dtype, device=like.device)
    n = 1
    for d in shape:
        n *= d
    if not (out.is_cuda and out.device == like.device and out.dtype == dtype and out.is_contiguous() and out.numel() == n):
        raise ValueError(f"out must be a contiguous {dtype} tensor of {n} elements on {like.device}")
    return out


def upload(host: "np.ndarray | bytes | memoryview", out: torch.Tensor | None = None) -> torch.Tensor:
    """Host bytes -> a device uint8 tensor through the library's pinned staging ring (rfq_upload)."""
    import numpy as np
    h = np.frombuffer(host, dtype=np.uint8) if not isinstance(host, np.ndarray) else np.ascontiguousarray(host).view(np.uint8).reshape(-1)
    if out is None:
        out = torch.empty(h.size, dtype=torch.uint8, device="cuda")
    if out.numel() != h.size or out.dtype != torch.uint8 or not out.is_contiguous():
        raise ValueError("upload: out must be a contiguous uint8 device tensor of the source's size")
    check(lib().rfq_upload(C.c_void_p(h.ctypes.data), h.size, _ptr(out), _stream()))
    return out


def dequant(fmt: int, packed: torch.Tensor, n_elems: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """Packed device bytes -> f32 device tensor of n_elems."""
    packed = _dev_u8(packed)
    if n_elems < 0:
        raise ValueError("n_elems is negative")
    out = _out(out, (n_elems,), torch.float32, packed)
    check(lib().rfq_dequant(fmt, _ptr(packed), packed.numel(), _ptr(out), n_elems, _stream()))
    return out


def gemv(fmt: int, w: torch.Tensor, x: torch.Tensor, n: int, k: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """y[m, n] = x[m, k] . dequant(W)[n, k]^T (m <= 8), fp32."""
    w, x = _dev_u8(w), _f32(x, "x")
    m = _rows_of(x, k, "x")
    out = _out(out, (m, n), torch.float32, x)
    check(lib().rfq_gemv(fmt, _ptr(w), w.numel(), _ptr(x), _ptr(out), m, n, k, _stream()))
    return out if x.dim() > 1 else out.view(n)


def gemv_kn(fmt: int, w: torch.Tensor, x: torch.Tensor, n: int, k: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """y[m, n] = x[m, k] . Wd[k, n] with Wd[l, j] = element l * n + j of the packed stream decoded as one flat
    array: the orientation the reference's kernel and CPU fallback compute (kernels/q4_0_matmul.hip:207,
    src/kernels/matmul/quantized/q4_0.rs:274-311)."""
    w, x = _dev_u8(w), _f32(x, "x")
    m = _rows_of(x, k, "x")
    out = _out(out, (m, n), torch.float32, x)
    check(lib().rfq_gemv_kn(fmt, _ptr(w), w.numel(), _ptr(x), _ptr(out), m, n, k, _stream()))
    return out if x.dim() > 1 else out.view(n)


def get_rows(fmt: int, table: torch.Tensor, tokens: torch.Tensor, n_vocab: int, n_embd: int,
             status: torch.Tensor | None = None) -> torch.Tensor:
    """out[i, :] = dequantised (fmt = block format) or copied (fmt = 0, f32 table) row tokens[i] of the table."""
    if fmt == 0:
        table = _f32(table, "an f32 table")
        nbytes = table.numel() * 4
    else:
        table = _dev_u8(table)
        nbytes = table.numel()
    if not (tokens.is_cuda and tokens.device == table.device and tokens.dtype in (torch.int32, torch.uint32)
            and tokens.is_contiguous()):
        raise ValueError("tokens must be a contiguous int32/uint32 tensor on the table's device")
    if status is not None and not (status.is_cuda and status.device == table.device and status.dtype == torch.int32
                                   and status.numel() >= 1):
        raise ValueError("status must be an int32 tensor on the table's device")
    out = torch.empty((tokens.numel(), n_embd), dtype=torch.float32, device=table.device)
    check(lib().rfq_get_rows(fmt, _ptr(table), nbytes, n_vocab, n_embd, _ptr(tokens), tokens.numel(), _ptr(out),
                             _ptr(status) if status is not None else None, _stream()))
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm over the last axis of x[seq_len, hidden] (src/mlp/kernels.rs:261-330)."""
    x, weight = _f32(x, "x"), _f32(weight, "weight")
    hidden = x.shape[-1]
    if weight.numel() != hidden:
        raise ValueError(f"weight has {weight.numel()} elements, hidden = {hidden}")
    out = torch.empty_like(x)
    check(lib().rfq_rms_norm(_ptr(x), _ptr(weight), _ptr(out), x.numel() // hidden, hidden, eps, _stream()))
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """gate * (up * sigmoid(up)) elementwise (src/mlp/kernels.rs:177-240)."""
    gate, up = _f32(gate, "gate"), _f32(up, "up")
    if gate.shape != up.shape:
        raise ValueError("gate and up differ in shape")
    inter = gate.shape[-1] if gate.dim() else 1
    out = torch.empty_like(gate)
    check(lib().rfq_swiglu(_ptr(gate), _ptr(up), _ptr(out), gate.numel() // max(inter, 1), inter, _stream()))
    return out


def dequant_rms_norm(fmt: int, packed: torch.Tensor, weight: torch.Tensor, seq_len: int, hidden: int,
                     eps: float) -> torch.Tensor:
    """RMSNorm of packed rows, decoded on the fly (src/ggml/hip_backend/ops/fused_ops.rs:149-160)."""
    packed, weight = _dev_u8(packed), _f32(weight, "weight")
    if weight.numel() != hidden:
        raise ValueError(f"weight has {weight.numel()} elements, hidden = {hidden}")
    out = torch.empty((seq_len, hidden), dtype=torch.float32, device=packed.device)
    check(lib().rfq_dequant_rms_norm(fmt, _ptr(packed), packed.numel(), _ptr(weight), _ptr(out), seq_len, hidden, eps,
                                     _stream()))
    return out


def rms_norm_gemv(fmt: int, w: torch.Tensor, x: torch.Tensor, norm_weight: torch.Tensor, eps: float, n: int,
                  k: int, scratch: bool = True) -> torch.Tensor:
    """y[m, n] = RMSNorm(x[m, k]) . dequant(W)[n, k]^T in one call."""
    w, x, norm_weight = _dev_u8(w), _f32(x, "x"), _f32(norm_weight, "norm_weight")
    m = _rows_of(x, k, "x")
    if norm_weight.numel() != k:
        raise ValueError(f"norm_weight has {norm_weight.numel()} elements, k = {k}")
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    tmp = torch.empty((m, k), dtype=torch.float32, device=x.device) if scratch else None
    check(lib().rfq_rms_norm_gemv(fmt, _ptr(w), w.numel(), _ptr(x), _ptr(norm_weight), eps, _ptr(out), m, n, k,
                                  _ptr(tmp) if tmp is not None else None, _stream()))
    return out if x.dim() > 1 else out.view(n)


def mlp_swiglu(fmt_gate_up: int, gate_w: torch.Tensor, up_w: torch.Tensor, fmt_down: int, down_w: torch.Tensor,
               x: torch.Tensor, norm_weight: torch.Tensor | None, eps: float, hidden: int, inter: int,
               scratch: torch.Tensor | None = None) -> torch.Tensor:
    """out[m, hidden] = swiglu(xn . gate^T, xn . up^T) . down^T over quantised weights
    (src/backend/hip_backend/backend.rs:1153-1278); xn = RMSNorm(x) when norm_weight is given."""
    gate_w, up_w, down_w, x = _dev_u8(gate_w), _dev_u8(up_w), _dev_u8(down_w), _f32(x, "x")
    if gate_w.numel() != up_w.numel():
        raise ValueError("gate and up weights differ in size")
    m = _rows_of(x, hidden, "x")
    if norm_weight is not None and _f32(norm_weight, "norm_weight").numel() != hidden:
        raise ValueError(f"norm_weight has {norm_weight.numel()} elements, hidden = {hidden}")
    need = lib().rfq_mlp_scratch_bytes(m, hidden, inter)
    if scratch is None:
        scratch = torch.empty(need, dtype=torch.uint8, device=x.device)
    elif not (scratch.is_cuda and scratch.device == x.device and scratch.dtype == torch.uint8 and scratch.is_contiguous()):
        raise ValueError("scratch must be a contiguous uint8 tensor on x's device")
    out = torch.empty((m, hidden), dtype=torch.float32, device=x.device)
    check(lib().rfq_mlp_swiglu(fmt_gate_up, _ptr(gate_w), _ptr(up_w), gate_w.numel(), fmt_down, _ptr(down_w),
                               down_w.numel(), _ptr(x), _ptr(_f32(norm_weight, "norm_weight")) if norm_weight is not None else None,
                               eps, _ptr(out), m, hidden, inter, _ptr(scratch), scratch.numel(), _stream()))
    return out if x.dim() > 1 else out.view(hidden)


def gemm_f16(fmt: int, w: torch.Tensor, a: torch.Tensor, n: int, k: int, out_dtype=torch.float16,
             out: torch.Tensor | None = None, one_plane: bool = False) -> torch.Tensor:
    """out[m, n] = a[m, k] (fp16) . dequant(W)[n, k]^T on the fp16 matrix cores.  one_plane: every weight as a single
    fp16 operand (relative 2^-12 per weight, about half the time) instead of the pair hi + lo."""
    w = _dev_u8(w)
    if not (a.is_cuda and a.dtype == torch.float16 and a.is_contiguous() and a.dim() == 2 and a.shape[1] == k):
        raise ValueError(f"a must be a contiguous [m, {k}] float16 device tensor")
    m = a.shape[0]
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16}[out_dtype] | (_lib.GEMM_ONE_PLANE if one_plane else 0)
    out = _out(out, (m, n), out_dtype, a)
    check(lib().rfq_gemm_f16(fmt, _ptr(w), w.numel(), _ptr(a), _ptr(out), code, m, n, k, _stream()))
    return out


def gemm_f16_static(fmt: int, w: torch.Tensor, a: torch.Tensor, n: int, k: int, out: torch.Tensor,
                    out_dtype=torch.float16) -> torch.Tensor:
    """rfq_gemm_f16 with its temporaries in the library's static device array: the call allocates nothing, so the
    caller passes ``out``."""
    w = _dev_u8(w)
    if not (a.is_cuda and a.dtype == torch.float16 and a.is_contiguous() and a.dim() == 2 and a.shape[1] == k):
        raise ValueError("a must be a contiguous [m, k] float16 device tensor")
    m = a.shape[0]
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16}[out_dtype]
    out = _out(out, (m, n), out_dtype, a)
    check(lib().rfq_gemm_f16_static(fmt, _ptr(w), w.numel(), _ptr(a), _ptr(out), code, m, n, k, _stream()))
    return out


class ArrangedA:
    """Activations a[m, k] (fp16) in matrix-operand order, written once for several gemm_f16_arranged calls."""

    def __init__(self, a: torch.Tensor):
        if not (a.is_cuda and a.dtype == torch.float16 and a.is_contiguous() and a.dim() == 2):
            raise ValueError("a must be a contiguous [m, k] float16 device tensor")
        self.m, self.k = a.shape
        nbytes = lib().rfq_gemm_f16_arranged_bytes(self.m, self.k)
        if nbytes == 0:
            raise ValueError(f"cannot arrange activations of shape {tuple(a.shape)} (k must be a multiple of 8)")
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device=a.device)
        check(lib().rfq_gemm_f16_arrange(_ptr(a), self.m, self.k, _ptr(self.buf), nbytes, _stream()))


def gemm_f16_arranged(fmt: int, w: torch.Tensor, a: ArrangedA, n: int, out_dtype=torch.float16,
                      out: torch.Tensor | None = None) -> torch.Tensor:
    """out[m, n] = a . dequant(W)[n, k]^T with activations arranged beforehand (bit-identical to gemm_f16)."""
    w = _dev_u8(w)
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16}[out_dtype]
    out = _out(out, (a.m, n), out_dtype, a.buf)
    check(lib().rfq_gemm_f16_arranged(fmt, _ptr(w), w.numel(), _ptr(a.buf), a.buf.numel(), _ptr(out), code, a.m, n, a.k,
                                      _stream()))
    return out


class MxOperand:
    """A [rows, k] MXFP matrix re-encoded for the block-scaled matrix core."""

    def __init__(self, fmt: int, raw: torch.Tensor, rows: int, k: int, kind: int = _lib.MX_AUTO):
        raw = _dev_u8(raw)
        nbytes = lib().rfq_mx_prepared_bytes(fmt, _lib.MX_FP4 if kind == _lib.MX_FP4_UNCHECKED else kind, rows, k)
        if nbytes == 0:
            raise ValueError(f"cannot size a prepared operand for fmt={fmt} rows={rows} k={k}")
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device=raw.device)
        got = C.c_int(0)
        check(lib().rfq_mx_prepare(fmt, kind, _ptr(raw), raw.numel(), rows, k, _ptr(self.buf), nbytes,
                                   C.byref(got), _stream()))
        self.kind, self.rows, self.k, self.fmt = got.value, rows, k, fmt


def gemm_mx(a: MxOperand, w: MxOperand, out_dtype=torch.bfloat16, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[m, n] = A[m, k] . W[n, k]^T on the scaled f8f6f4 matrix core."""
    if a.k != w.k:
        raise ValueError("inner dimensions differ")
    code = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}[out_dtype]
    out = _out(out, (a.rows, w.rows), out_dtype, a.buf)
    check(lib().rfq_gemm_mx(_ptr(a.buf), a.buf.numel(), a.kind, _ptr(w.buf), w.buf.numel(), w.kind, _ptr(out), code, a.rows, w.rows,
                            a.k, _stream()))
    return out


def row_bytes(fmt: int, k: int) -> int:
    return (k // BLOCK_ELEMS[fmt]) * BLOCK_BYTES[fmt]
