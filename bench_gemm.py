"""Prefill GEMM lines of the bench (imported by bench.py; also runnable alone).

MXFP4 GEMM at M=2048, K=8192, N=28672 (bf16 out) and the MXFP6-weight variant,
plus the Q4_K fp16 GEMM at M=512, K=4096, N=14336 when that kernel is built.
FLOPs = 2*M*N*K; peaks: 10.1 PFLOP/s (FP4 scaled MFMA), 5.0 (FP8), 2.5 (fp16).

The launches of the first tens of milliseconds after an idle period run 5-15 % slower than the steady state (the
part's clocks ramp).  The MXFP4 configurations run 40 untimed launches (7 ms), then 200 timed ones, and report the
average over all timed launches, ramp included; the fp16 K-quant configurations run 300 untimed launches (20 ms)
and 300 timed ones (`warmup_launches` / `timed_launches` in each line say which).  The MXFP4 GEMM
is reported three ways: on operands from the reference's packer (which emits only codes {0, 1, 8, 9}), on
full-entropy operands (every code of a four-octave window, both signs), and as a prefill step that re-encodes
the raw activations for the matrix core before every GEMM.
"""
from __future__ import annotations

import ctypes as C
import json
import sys

import numpy as np


def _gauss(rows, k, seed, std):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal((rows, k), dtype=np.float32) * np.float32(std)


def mx_gemm(torch, w_fmt, m=2048, n=28672, k=8192, steps=200, warmup=200, data="packer"):
    """`warmup` untimed launches (200 = 36 ms, the same preheat as the GEMV lines of bench.py: the part's clocks ramp for
    the first tens of milliseconds out of idle), then `steps` timed ones; the figure after 40 warm-up launches, taken
    first, is reported beside it."""
    from rocmforge_amd import _lib, ops, quantize as Q
    dev = torch.device("cuda:0")
    slab_rows = 4096
    if data == "packer":
        a_raw = Q.pack_mxfp4(_gauss(m, k, 20260005, 1.0))
        pack = Q.pack_mxfp4 if w_fmt == Q.MXFP4 else Q.pack_mxfp6
        w_raw = np.tile(pack(_gauss(slab_rows, k, 20260015 + w_fmt, 0.02)), n // slab_rows)
    else:                                                     # every code of a four-octave window, random exponents
        rng = np.random.Generator(np.random.PCG64(20260065))
        a_raw = Q.mxfp4_window_blocks(rng, m * k // 32, (-3, 3), zero_blocks=0.0)
        w_raw = Q.mxfp4_window_blocks(rng, n * k // 32, (-9, -3), zero_blocks=0.0)
    a_dev, w_dev = torch.from_numpy(a_raw).to(dev), torch.from_numpy(w_raw).to(dev)
    A = ops.MxOperand(Q.MXFP4, a_dev, m, k)
    W = ops.MxOperand(w_fmt, w_dev, n, k)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ms = C.c_float(0)
    L = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def prepare_us(fmt, raw, rows, kind, reps=20):
        # re-encoding into the matrix core's operand order: device time of back-to-back rfq_mx_prepare calls into one
        # buffer that do not synchronise (8-bit kinds, and the 4-bit kind requested unchecked, which is how
        # activations are prepared per prefill)
        req = _lib.MX_FP4_UNCHECKED if kind == _lib.MX_FP4 else kind
        nbytes = L.rfq_mx_prepared_bytes(fmt, kind, rows, k)
        buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        got = C.c_int(0)
        call = lambda: _lib.check(L.rfq_mx_prepare(fmt, req, C.c_void_p(raw.data_ptr()), raw.numel(), rows, k,
                                                   C.c_void_p(buf.data_ptr()), nbytes, C.byref(got), stream))
        call()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            call()
        e1.record()
        torch.cuda.synchronize()
        return round(e0.elapsed_time(e1) / reps * 1e3, 1)

    prep = {"prepare_a_us": prepare_us(Q.MXFP4, a_dev, m, A.kind), "prepare_w_us": prepare_us(w_fmt, w_dev, n, W.kind, reps=5)}
    args = (C.c_void_p(A.buf.data_ptr()), A.buf.numel(), A.kind, C.c_void_p(W.buf.data_ptr()), W.buf.numel(), W.kind,
            C.c_void_p(out.data_ptr()), _lib.BF16, m, n, k)
    flops = 2.0 * m * n * k
    peak = 10.1e15 if (A.kind == _lib.MX_FP4 and W.kind == _lib.MX_FP4) else 5.0e15
    _lib.check(L.rfq_bench_gemm_mx(*args, min(warmup, 40), steps, stream, C.byref(ms)))
    t40 = ms.value / 1e3 / steps
    _lib.check(L.rfq_bench_gemm_mx(*args, warmup, steps, stream, C.byref(ms)))
    t = ms.value / 1e3 / steps
    res = {"TFLOP/s": round(flops / t / 1e12, 1), "us": round(t * 1e6, 1), "mfma_frac": round(flops / t / peak, 4),
           "peak_TFLOP/s": peak / 1e12, "kinds": [A.kind, W.kind], "warmup_launches": warmup, "timed_launches": steps,
           "after_40_warmup_launches_out_of_idle": {"us": round(t40 * 1e6, 1), "mfma_frac": round(flops / t40 / peak, 4)},
           "operands": "reference packer (codes 0, 1, 8, 9)" if data == "packer" else "every code of a four-octave window", **prep}
    if A.kind == _lib.MX_FP4 and data == "packer":
        # the prefill step end to end: raw MXFP4 activations re-encoded before every GEMM
        _lib.check(L.rfq_bench_gemm_mx_prefill(C.c_void_p(a_dev.data_ptr()), a_dev.numel(), C.c_void_p(A.buf.data_ptr()),
                                               A.buf.numel(), C.c_void_p(W.buf.data_ptr()), W.buf.numel(), W.kind, C.c_void_p(out.data_ptr()),
                                               _lib.BF16, m, n, k, warmup, steps, stream, C.byref(ms)))
        te = ms.value / 1e3 / steps
        res["prefill_step"] = {"us": round(te * 1e6, 1), "TFLOP/s": round(flops / te / 1e12, 1), "mfma_frac": round(flops / te / peak, 4),
                               "what": "rfq_mx_prepare(A, unchecked) + rfq_gemm_mx per step"}
    return res


def kq_gemm(torch, fmt, m=512, n=14336, k=4096, steps=300, warmup=600, arranged=False, one_plane=False):
    """Q4_K / Q6_K prefill GEMM on the fp16 matrix cores, fp16 in and out.  one_plane: RFQ_GEMM_ONE_PLANE (every weight
    as one fp16 operand) beside the default two (hi + lo)."""
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
    _lib.check(L.rfq_bench_gemm_f16(*args, warmup, steps, stream, C.byref(ms)))
    t = ms.value / 1e3 / steps
    flops = 2.0 * m * n * k
    res = {"TFLOP/s": round(flops / t / 1e12, 1), "us": round(t * 1e6, 1), "mfma_frac": round(flops / t / 2.5e15, 4),
           "peak_TFLOP/s": 2500.0, "warmup_launches": warmup, "timed_launches": steps,
           "fp16_operands_per_weight": 1 if fmt in (Q.Q4_K, Q.GGUF_Q4_K) else 2}
    if fmt == Q.GGUF_Q4_K:
        res["what"] = "exact in one pass: integer operands sc*q, d and dmin applied in f32 per super-block"
    if one_plane and fmt != Q.Q4_K:
        args1 = args[:5] + (_lib.F16 | _lib.GEMM_ONE_PLANE,) + args[6:]
        _lib.check(L.rfq_bench_gemm_f16(*args1, warmup, steps, stream, C.byref(ms)))
        t1 = ms.value / 1e3 / steps
        res["one_fp16_operand_per_weight"] = {"us": round(t1 * 1e6, 1), "TFLOP/s": round(flops / t1 / 1e12, 1),
                                              "mfma_frac": round(flops / t1 / 2.5e15, 4),
                                              "what": "RFQ_GEMM_ONE_PLANE: weights rounded once to fp16 (8e-4 of rms(out) from the reference)"}
    if arranged:
        # the same GEMM on activations arranged once (the second and third projection of one input)
        from rocmforge_amd import ops
        A = ops.ArrangedA(a)
        _lib.check(L.rfq_bench_gemm_f16_arranged(fmt, C.c_void_p(w.data_ptr()), w.numel(), C.c_void_p(A.buf.data_ptr()), A.buf.numel(),
                                                 C.c_void_p(out.data_ptr()), _lib.F16, m, n, k, warmup, steps, stream, C.byref(ms)))
        ta = ms.value / 1e3 / steps
        res["activations_arranged_once"] = {"us": round(ta * 1e6, 1), "TFLOP/s": round(flops / ta / 1e12, 1),
                                            "mfma_frac": round(flops / ta / 2.5e15, 4),
                                            "what": "rfq_gemm_f16_arranged per step, rfq_gemm_f16_arrange before the loop"}
    return res


def mfma_probe(torch, only_variant=None):
    """What the fp16 matrix pipe delivers alone and beside a fused kernel's operand traffic (rfq_bench_mfma_f16_probe):
    instruction shape x (VALU, LDS fragment reads, global fragment loads per round) x workgroups x wavefronts per SIMD x
    operand data, each launched for about 20 ms before the timed launch."""
    import ctypes as C
    from rocmforge_amd import _lib
    L = _lib.lib()
    torch.zeros(1, device="cuda")
    rows = []
    mixes = {0: [(0, 0, 0), (2, 0, 0), (4, 0, 0), (0, 4, 0), (0, 8, 0), (0, 0, 2), (0, 0, 4), (0, 4, 2), (2, 4, 2), (3, 4, 2), (3, 6, 0)],
             1: [(0, 0, 0), (1, 0, 0), (2, 0, 0), (0, 7, 0), (0, 0, 4), (0, 7, 4), (1, 7, 4), (2, 7, 4)]}
    if only_variant is not None:
        mixes = {only_variant: mixes[only_variant]}
    for variant, name in ((0, "32x32x16_f16"), (1, "16x16x32_f16")):
        for valu, ldsr, gld in mixes.get(variant, []):
            for wgs, waves in ((128, 4), (224, 4), (256, 4), (224, 8), (256, 8)):
                for rnd in (1, 0):
                    if (not rnd) and (valu or ldsr or gld or wgs != 256):
                        continue
                    if wgs == 128 and (valu or ldsr or gld):
                        continue
                    us, cpm, ghz, tf = C.c_float(), C.c_float(), C.c_float(), C.c_float()
                    iters = (4000 if variant == 0 else 2288) // (waves // 4)     # about 0.5 ms per launch
                    _lib.check(L.rfq_bench_mfma_f16_probe(variant, valu, ldsr, gld, wgs, waves, rnd, iters, 30, None,
                                                          C.byref(us), C.byref(cpm), C.byref(ghz), C.byref(tf)))
                    rows.append({"instruction": name, "valu_per_mfma": valu, "lds_reads_per_round": ldsr, "global_loads_per_round": gld,
                                 "workgroups": wgs, "waves_per_simd": waves // 4, "operands": "random" if rnd else "zero",
                                 "launch_us": round(us.value, 1),
                                 "clocks_per_mfma_and_simd": round(us.value * ghz.value * 1e3 / (iters * (8 if variant == 0 else 28) * (waves // 4)), 2),
                                 "clocks_per_mfma_in_loop": round(cpm.value, 2),
                                 "shader_ghz": round(ghz.value, 3), "tflops": round(tf.value, 1),
                                 "frac_of_2500": round(tf.value / 2500.0, 3)})
                    print(json.dumps(rows[-1]), flush=True)
    return rows


def run(torch):
    from rocmforge_amd import quantize as Q
    res = {}
    res["Q4_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.Q4_K, arranged=True)
    res["Q6_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.Q6_K, one_plane=True)
    res["GGUF_Q4_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.GGUF_Q4_K, one_plane=True)
    res["GGUF_Q6_K gemm 512x4096x14336 fp16"] = kq_gemm(torch, Q.GGUF_Q6_K, one_plane=True)
    # the down projection of the same layer: 64 output tiles, split along k in four parts (rfq_gemm_f16_k_parts)
    for fmt in (Q.Q4_K, Q.GGUF_Q4_K):
        r = kq_gemm(torch, fmt, n=4096, k=14336, steps=200, warmup=400, arranged=True)
        r["k_parts"] = 4
        r["activations_arranged_once"]["what"] += " (a single pass over k: that entry point has no temporary for parts)"
        res[f"{Q.NAMES[fmt]} gemm 512x14336x4096 fp16 (down projection)"] = r
    res["MXFP4 gemm 2048x8192x28672 bf16"] = mx_gemm(torch, Q.MXFP4)
    res["MXFP4 gemm 2048x8192x28672 bf16, full-entropy operands"] = mx_gemm(torch, Q.MXFP4, data="window")
    res["MXFP6-weight gemm 2048x8192x28672 bf16"] = mx_gemm(torch, Q.MXFP6_E2M3)
    return res


if __name__ == "__main__":
    import argparse
    import os
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", choices=["mxfp4", "mxfp6", "q4_k", "gguf_q4_k"], help="one configuration (for profiling runs)")
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--probe-mfma", action="store_true", help="the fp16 matrix pipe alone and beside a fused kernel's operand traffic")
    ap.add_argument("--probe-variant", type=int, choices=[0, 1], help="only v_mfma_f32_32x32x16_f16 (0) or v_mfma_f32_16x16x32_f16 (1)")
    ap.add_argument("--data", choices=["packer", "window"], default="packer", help="MXFP4 operands: the reference packer's, or full-entropy")
    ap.add_argument("--down", action="store_true", help="with --only q4_k / gguf_q4_k: the down projection 512 x 14336 -> 4096 (split along k)")
    a = ap.parse_args()
    import torch
    from rocmforge_amd import quantize as Q
    if a.probe_mfma:
        mfma_probe(torch, a.probe_variant)
    elif a.only in ("q4_k", "gguf_q4_k"):
        shape = dict(n=4096, k=14336) if a.down else {}
        print(json.dumps(kq_gemm(torch, Q.Q4_K if a.only == "q4_k" else Q.GGUF_Q4_K, steps=a.steps, arranged=not a.down, **shape)))
    elif a.only:
        print(json.dumps(mx_gemm(torch, Q.MXFP4 if a.only == "mxfp4" else Q.MXFP6_E2M3, steps=a.steps, data=a.data)))
    else:
        print(json.dumps(run(torch)))
