"""Prefill GEMM lines of the bench (imported by bench.py; also runnable alone).

MXFP4 GEMM at M=2048, K=8192, N=28672 (bf16 out) and the MXFP6-weight variant,
plus the Q4_K fp16 GEMM at M=512, K=4096, N=14336 when that kernel is built.
FLOPs = 2*M*N*K; peaks: 10.1 PFLOP/s (FP4 scaled MFMA), 5.0 (FP8), 2.5 (fp16).

Each configuration runs `warmup` untimed launches first (20 to 30 ms): the
launches of the first tens of milliseconds after an idle period run 5-15 %
slower than the steady state (the part's clocks ramp), and the timed launches
should not include that.
"""
from __future__ import annotations

import ctypes as C
import json
import sys

import numpy as np


def _gauss(rows, k, seed, std):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal((rows, k), dtype=np.float32) * np.float32(std)


def mx_gemm(torch, w_fmt, m=2048, n=28672, k=8192, steps=50, warmup=150):
    from rocmforge_amd import _lib, ops, quantize as Q
    dev = torch.device("cuda:0")
    a_raw = Q.pack_mxfp4(_gauss(m, k, 20260005, 1.0))
    slab_rows = 4096
    pack = Q.pack_mxfp4 if w_fmt == Q.MXFP4 else Q.pack_mxfp6
    w_raw = np.tile(pack(_gauss(slab_rows, k, 20260015 + w_fmt, 0.02)), n // slab_rows)
    a_dev, w_dev = torch.from_numpy(a_raw).to(dev), torch.from_numpy(w_raw).to(dev)
    A = ops.MxOperand(Q.MXFP4, a_dev, m, k)
    W = ops.MxOperand(w_fmt, w_dev, n, k)

    def prepare_us(fmt, raw, rows, kind):
        # re-encoding into the matrix core's operand order, reported beside the GEMM, never inside it:
        # device time of back-to-back calls that do not synchronise (8-bit kinds, and the 4-bit kind
        # requested unchecked, which is how activations are prepared per prefill)
        req = _lib.MX_FP4_UNCHECKED if kind == _lib.MX_FP4 else kind
        ops.MxOperand(fmt, raw, rows, k, req)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(10):
            ops.MxOperand(fmt, raw, rows, k, req)
        e1.record()
        torch.cuda.synchronize()
        return round(e0.elapsed_time(e1) / 10 * 1e3, 1)

    prep = {"prepare_a_us": prepare_us(Q.MXFP4, a_dev, m, A.kind), "prepare_w_us": prepare_us(w_fmt, w_dev, n, W.kind)}
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ms = C.c_float(0)
    L = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = (C.c_void_p(A.buf.data_ptr()), A.kind, C.c_void_p(W.buf.data_ptr()), W.kind, C.c_void_p(out.data_ptr()),
            _lib.BF16, m, n, k)
    _lib.check(L.rfq_bench_gemm_mx(*args, 0, warmup, stream, C.byref(ms)))
    _lib.check(L.rfq_bench_gemm_mx(*args, 0, steps, stream, C.byref(ms)))
    t = ms.value / 1e3 / steps
    flops = 2.0 * m * n * k
    peak = 10.1e15 if (A.kind == _lib.MX_FP4 and W.kind == _lib.MX_FP4) else 5.0e15
    return {"TFLOP/s": round(flops / t / 1e12, 1), "us": round(t * 1e6, 1), "mfma_frac": round(flops / t / peak, 4),
            "peak_TFLOP/s": peak / 1e12, "kinds": [A.kind, W.kind], **prep}


def kq_gemm(torch, fmt, m=512, n=14336, k=4096, steps=100, warmup=300):
    """Q4_K / Q6_K prefill GEMM on the fp16 matrix cores, fp16 in and out."""
    from rocmforge_amd import _lib, quantize as Q
    dev = torch.device("cuda:0")
    w = torch.from_numpy(Q.make_weights(fmt, n, k, seed=20260004)).to(dev)
    a = torch.from_numpy(_gauss(m, k, 20260014, 1.0).astype(np.float16)).to(dev)
    out = torch.empty((m, n), dtype=torch.float16, device=dev)
    ms = C.c_float(0)
    L = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = (fmt, C.c_void_p(w.data_ptr()), w.numel(), C.c_void_p(a.data_ptr()), C.c_void_p(out.data_ptr()), _lib.F16,
            m, n, k)
    _lib.check(L.rfq_bench_gemm_f16(*args, 0, warmup, stream, C.byref(ms)))
    _lib.check(L.rfq_bench_gemm_f16(*args, 0, steps, stream, C.byref(ms)))
    t = ms.value / 1e3 / steps
    flops = 2.0 * m * n * k
    return {"TFLOP/s": round(flops / t / 1e12, 1), "us": round(t * 1e6, 1), "mfma_frac": round(flops / t / 2.5e15, 4),
            "peak_TFLOP/s": 2500.0}


def run(torch):
    from rocmforge_amd import quantize as Q
    res = {}
    res["Q4_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.Q4_K)
    res["Q6_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.Q6_K)
    res["GGUF_Q4_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.GGUF_Q4_K)
    res["GGUF_Q6_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.GGUF_Q6_K)
    res["MXFP4 gemm 2048x8192x28672 bf16"] = mx_gemm(torch, Q.MXFP4)
    res["MXFP6-weight gemm 2048x8192x28672 bf16"] = mx_gemm(torch, Q.MXFP6_E2M3)
    return res


if __name__ == "__main__":
    import argparse
    import os
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", choices=["mxfp4", "mxfp6", "q4_k", "gguf_q4_k"], help="one configuration (for profiling runs)")
    ap.add_argument("--steps", type=int, default=50)
    a = ap.parse_args()
    import torch
    from rocmforge_amd import quantize as Q
    if a.only in ("q4_k", "gguf_q4_k"):
        print(json.dumps(kq_gemm(torch, Q.Q4_K if a.only == "q4_k" else Q.GGUF_Q4_K, steps=a.steps)))
    elif a.only:
        print(json.dumps(mx_gemm(torch, Q.MXFP4 if a.only == "mxfp4" else Q.MXFP6_E2M3, steps=a.steps)))
    else:
        print(json.dumps(run(torch)))
