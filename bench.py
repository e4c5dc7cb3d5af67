#!/usr/bin/env python3
"""Headline bench: Q4_K decode GEMV, W [14336 x 4096], x fp32 [4096], batch 1.

One step = one rfq_gemv call (one token's FFN projection).  The packed weights
are resident in HBM before the timed region; the step loop rotates through
enough distinct weight copies that the 256 MB last-level cache cannot hold
them, so every step streams its 58.7 MB from HBM ("cold").  The metric is
algorithmic bytes (packed W as stored + x + y) per second.

Prints ONE JSON line.  `value` and `roofline.achieved` come from one clock: HIP
events recorded on the launch stream around the K timed launches (the host's
wall clock around the same region, which adds the final synchronisation's
wake-up -- tens of microseconds, as much as the work itself at K = 20 -- is
reported as `wall_ms_per_step`).  Extra keys: `roofline` (with the name of the
kernel the dispatch took, read back from the library, and the time of a kernel
that only reads the same bytes), `cpu_baseline` (the CPU oracle timed on this
host), `also` (the other configurations, one short run each).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
N, K = 14336, 4096
CACHE_BYTES = 256 << 20
# HBM bytes one launch of the headline kernel moves, from FETCH_SIZE / WRITE_SIZE profiler counters scaled by a copy
# kernel of known size: read from the committed summary of those runs, so that the figure cannot outlive its source.
TRAFFIC_SOURCE = "profiles/gemv_q4k_14336x4096_hbm_counters.txt"


def measured_traffic_bytes():
    """(bytes per launch, kernel the counters belong to) from the line 'traffic per launch = ... = N bytes' and the
    kernel named in the per-dispatch table of TRAFFIC_SOURCE; (None, None) when the file or the line is missing."""
    import re
    try:
        text = open(os.path.join(ROOT, TRAFFIC_SOURCE)).read()
    except OSError:
        return None, None
    m = re.search(r"traffic per launch\s*=.*?=\s*([\d,]+)\s*bytes", text)
    kern = re.search(r"^\s*(gemv_\w+<[^>]*>).*FETCH_SIZE", text, re.M)
    return (int(m.group(1).replace(",", "")) if m else None), (kern.group(1) if kern else None)
# launch shapes of the read-only kernel that the floor is taken over (workgroups, threads, loads in flight, non-temporal)
PREHEAT_MS = 30.0
READ_FLOOR_SHAPES = ((256, 512, 4, 1), (256, 768, 4, 1), (256, 1024, 8, 1), (512, 512, 8, 1), (256, 512, 4, 0))


def algorithmic_bytes(fmt, n, k, m, Q):
    return Q.packed_bytes(fmt, n * k) + 4 * m * k + 4 * m * n


class GemvRun:
    """Weights (rotating copies), x and y of one GEMV configuration on the device, and the native timing loop over them."""

    def __init__(self, torch, fmt, n, k, m, copies, Q, seed):
        import ctypes as C

        import numpy as np
        self.torch, self.C = torch, C
        dev = torch.device("cuda:0")
        slab = 4008 if n > 32768 and n % 4008 == 0 else n   # a vocabulary-sized matrix: quantise a slab, repeat it down the rows
        w = Q.make_weights(fmt, slab, k, seed=seed)
        if slab != n:
            w = np.tile(w, n // slab)
        rng = np.random.Generator(np.random.PCG64(seed + 1))
        self.w, self.x = w, rng.standard_normal((m, k), dtype=np.float32)
        self.dws = [torch.from_numpy(w).to(dev) for _ in range(copies)]
        self.ptrs = (C.c_void_p * copies)(*[t.data_ptr() for t in self.dws])
        self.dx = torch.from_numpy(self.x).to(dev)
        self.y = torch.empty((m, n), dtype=torch.float32, device=dev)
        self.args = (fmt, self.ptrs, copies, w.size, C.c_void_p(self.dx.data_ptr()), C.c_void_p(self.y.data_ptr()), m, n, k)

    def run(self, warmup, steps):
        """(wall seconds, device seconds) of `steps` rfq_gemv calls issued back to back by the library's native loop on
        torch's current stream, after `warmup` untimed ones in the same loop: the rotation through the weight copies
        continues across the boundary, so the first timed steps do not meet copies the warm-up touched last."""
        from rocmforge_amd import _lib
        C, torch = self.C, self.torch
        ms = C.c_float(0)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _lib.check(_lib.lib().rfq_bench_gemv(*self.args, max(warmup, 1), steps, stream, C.byref(ms)))
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * steps / (steps + max(warmup, 1))
        return wall, ms.value / 1e3


TIMELINE_POINTS = ["wavefront started", "x and first rows requested, x arrived", "x converted (before the barrier)", "past the barrier",
                   "prepared x of its units in registers"] + \
                  [t for i in range(7) for t in (f"row {i} in registers", f"row {i} reduced")] + ["results stored"]


def gemv_timeline(torch, fmt, n, k, copies, warmup, Q, seed):
    """One launch of the decode GEMV with every wavefront stamping the constant 100 MHz clock at fixed points
    (rfq_bench_gemv_timeline), after `warmup` ordinary launches over the rotating weight copies.  Returns the kernel
    name and the stamps in microseconds after the first wavefront's start, shape [wavefronts, points], or None when
    the kernel this shape takes has no such build."""
    import ctypes as C

    import numpy as np
    from rocmforge_amd import _lib
    g = GemvRun(torch, fmt, n, k, 1, copies, Q, seed)
    cap = 1 << 16
    trace = torch.zeros((cap, 20), dtype=torch.int64, device="cuda:0")
    waves, stamps = C.c_int(0), C.c_int(0)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    _lib.check(_lib.lib().rfq_bench_gemv_timeline(fmt, g.ptrs, copies, g.w.size, C.c_void_p(g.dx.data_ptr()), C.c_void_p(g.y.data_ptr()),
                                                  n, k, warmup, stream, C.c_void_p(trace.data_ptr()), cap, C.byref(waves), C.byref(stamps)))
    torch.cuda.synchronize()
    kern = _lib.lib().rfq_bench_last_gemv_kernel().decode()
    if waves.value == 0:
        return kern, None
    assert stamps.value == 20
    t = trace[:waves.value].cpu().numpy().astype(np.float64)
    return kern, (t - t[:, 0].min()) / 100.0                # 100 MHz ticks -> microseconds


def print_timeline(name, n, k, kern, us, warmup):
    import numpy as np
    print(f"# {name} decode GEMV {n} x {k}: one launch of {kern} after {warmup} ordinary launches; {us.shape[0]} wavefronts;")
    print("# microseconds after the first wavefront's start (constant 100 MHz clock, 10 ns a tick): the point was reached by")
    print(f"# {'point':42s} {'first':>7s} {'10 %':>7s} {'median':>7s} {'90 %':>7s} {'last':>7s}")
    for i, label in enumerate(TIMELINE_POINTS):
        c = us[:, i]
        print(f"  {label:42s} {c.min():7.2f} {np.percentile(c, 10):7.2f} {np.median(c):7.2f} {np.percentile(c, 90):7.2f} {c.max():7.2f}")
    d = lambda a, b: np.median(us[:, a] - us[:, b])
    print("# median over wavefronts of the time between points:")
    print(f"  start -> requests issued and x arrived {d(1, 0):.2f}; conversion {d(2, 1):.2f}; wait at the barrier {d(3, 2):.2f}; prepared x {d(4, 3):.2f};")
    print("  row i: wait for its bytes / dot products and reduction: " +
          "  ".join(f"{d(5 + 2 * i, 4 + 2 * i):.2f} / {d(6 + 2 * i, 5 + 2 * i):.2f}" for i in range(7)))
    print(f"  store {d(19, 18):.2f}; a wavefront's life {np.median(us[:, 19] - us[:, 0]):.2f}; first start to last store {us[:, 19].max():.2f}")


def time_gemv(torch, fmt, n, k, m, copies, steps, warmup, Q, seed):
    """Returns (wall seconds, device seconds, w, x, y) for `steps` rfq_gemv calls."""
    g = GemvRun(torch, fmt, n, k, m, copies, Q, seed)
    # like the headline: PREHEAT_MS of untimed launches first (uploading a configuration's weight copies leaves the
    # part idle, and the launches of the first milliseconds after that run on ramping clocks)
    probe_steps = min(steps, 100)
    _, probe_s = g.run(warmup, probe_steps)
    g.run(1, max(1, int(PREHEAT_MS * 1e-3 / max(probe_s / probe_steps, 2e-6))))
    wall, dev_s = g.run(warmup, steps)
    return wall, dev_s, g.w, g.x, g.y.cpu().numpy()


def read_floor(torch, nbytes, copies, steps, warmup):
    """Device seconds per launch of a kernel that only reads `nbytes` (rotating copies, back-to-back launches like
    the GEMV): the floor of a one-launch step over the same bytes.  The best of a few launch shapes."""
    import ctypes as C

    from rocmforge_amd import _lib
    dev = torch.device("cuda:0")
    bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(copies)]
    ptrs = (C.c_void_p * copies)(*[b.data_ptr() for b in bufs])
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ms, best = C.c_float(0), None
    for blocks, threads, depth, nt in READ_FLOOR_SHAPES:
        _lib.check(_lib.lib().rfq_bench_read_floor(ptrs, copies, nbytes, blocks, threads, nt, depth, warmup, steps, stream,
                                                   C.byref(ms)))
        t = ms.value / 1e3 / steps
        if best is None or t < best[0]:
            best = (t, f"{blocks} x {threads} threads, {depth} loads in flight, {'non-temporal' if nt else 'plain'}")
    return best


def time_dequant(torch, fmt, n, k, steps, warmup, Q, seed):
    """Device seconds per rfq_dequant call of an [n, k] matrix; bytes moved = packed in + 4 per element out."""
    import ctypes as C

    from rocmforge_amd import _lib
    dev = torch.device("cuda:0")
    import numpy as np
    slab = min(n, 4096)                                  # quantise a slab once, repeat it down the rows
    w = np.tile(Q.make_weights(fmt, slab, k, seed=seed), n // slab) if n % slab == 0 else Q.make_weights(fmt, n, k, seed=seed)
    copies = 4
    dws = [torch.from_numpy(w).to(dev) for _ in range(copies)]
    ptrs = (C.c_void_p * copies)(*[t.data_ptr() for t in dws])
    # enough output buffers that a step's output lines are not the last step's, still in the last-level cache
    out_copies = max(1, -(-int(2.5 * CACHE_BYTES) // (4 * n * k)))
    out = torch.empty(out_copies * n * k, dtype=torch.float32, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ms = C.c_float(0)
    L = _lib.lib()
    _lib.check(L.rfq_bench_dequant(fmt, ptrs, copies, w.size, C.c_void_p(out.data_ptr()), n * k, out_copies, 0, warmup, stream,
                                   C.byref(ms)))
    # PREHEAT_MS of untimed calls, as for the GEMV lines (out of idle the first milliseconds run on ramping clocks)
    preheat = max(1, int(PREHEAT_MS / max(ms.value / warmup, 2e-3)))
    _lib.check(L.rfq_bench_dequant(fmt, ptrs, copies, w.size, C.c_void_p(out.data_ptr()), n * k, out_copies, 0, preheat, stream,
                                   C.byref(ms)))
    _lib.check(L.rfq_bench_dequant(fmt, ptrs, copies, w.size, C.c_void_p(out.data_ptr()), n * k, out_copies, 0, steps, stream,
                                   C.byref(ms)))
    return ms.value / 1e3 / steps, w.size + 4 * n * k


def time_get_rows(torch, fmt, n_vocab, n_embd, n_tokens, Q):
    """Embedding gather: n_tokens rows of a packed [n_vocab, n_embd] table, token ids on the device."""
    import numpy as np

    from rocmforge_amd import ops
    dev = torch.device("cuda:0")
    slab = 4008
    tab = torch.from_numpy(np.tile(Q.make_weights(fmt, slab, n_embd, seed=20260033), n_vocab // slab)).to(dev)
    rng = np.random.Generator(np.random.PCG64(20260034))
    tok = torch.from_numpy(rng.integers(0, n_vocab, size=n_tokens).astype(np.int32)).to(dev)
    import ctypes as C

    from rocmforge_amd import _lib
    out_copies = 32                                            # 268 MB of outputs: none is rewritten while still cached
    out = torch.empty((out_copies, n_tokens, n_embd), dtype=torch.float32, device=dev)
    ms = C.c_float(0)
    _lib.check(_lib.lib().rfq_bench_get_rows(fmt, C.c_void_p(tab.data_ptr()), tab.numel(), n_vocab, n_embd,
                                             C.c_void_p(tok.data_ptr()), n_tokens, C.c_void_p(out.data_ptr()), out_copies, 20, 200,
                                             C.c_void_p(torch.cuda.current_stream().cuda_stream), C.byref(ms)))
    t = ms.value / 200 * 1e-3
    b = n_tokens * (n_embd * 4 + Q.packed_bytes(fmt, n_embd))
    return {"us": round(t * 1e6, 2), "GB/s": round(b / t / 1e9, 1), "rows/s": round(n_tokens / t)}


def time_gemv_kn(torch, fmt, n, k, Q, copies=6, reps=10):
    """The reference's own orientation (y[j] = sum_l x[l] * Wd[l * n + j] over the flat dequantised stream) on the
    same bytes as the headline, rotating weight copies."""
    import numpy as np

    from rocmforge_amd import ops
    dev = torch.device("cuda:0")
    w = torch.from_numpy(Q.make_weights(fmt, n, k, seed=20260003)).to(dev)
    ws = [w.clone() for _ in range(copies)]
    rng = np.random.Generator(np.random.PCG64(20260036))
    x = torch.from_numpy(rng.standard_normal(k, dtype=np.float32)).to(dev)
    out = torch.empty((1, n), dtype=torch.float32, device=dev)
    for wc in ws:
        ops.gemv_kn(fmt, wc, x, n, k, out=out)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        for wc in ws:
            ops.gemv_kn(fmt, wc, x, n, k, out=out)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) / (reps * copies) * 1e-3
    b = algorithmic_bytes(fmt, n, k, 1, Q)
    return {"us": round(t * 1e6, 2), "GB/s": round(b / t / 1e9, 1), "hbm_frac": round(b / t / 1e9 / HBM_PEAK_GBS, 4)}


def time_mlp(torch, fmt, hidden, inter, Q, steps=300, warmup=60):
    """The SwiGLU MLP of one decode step (RMSNorm, gate and up projections, activation, down projection) over
    rotating weight sets: rfq_mlp_swiglu (two launches) and the same arithmetic as five separate calls."""
    import ctypes as C

    import numpy as np

    from rocmforge_amd import _lib
    dev = torch.device("cuda:0")
    L = _lib.lib()
    gu_bytes, d_bytes = Q.packed_bytes(fmt, inter * hidden), Q.packed_bytes(fmt, hidden * inter)
    copies = -(-int(2.5 * CACHE_BYTES) // (2 * gu_bytes + d_bytes))
    slab = 1024                                                    # quantise a slab of rows, repeat it down the matrix
    mats = []
    for c in range(copies):
        g = np.tile(Q.make_weights(fmt, slab, hidden, seed=20260040 + 3 * c), inter // slab)
        u = np.tile(Q.make_weights(fmt, slab, hidden, seed=20260041 + 3 * c), inter // slab)
        d = np.tile(Q.make_weights(fmt, slab, inter, seed=20260042 + 3 * c), hidden // slab)
        mats.append(tuple(torch.from_numpy(a).to(dev) for a in (g, u, d)))
    arr = [(C.c_void_p * copies)(*[m[i].data_ptr() for m in mats]) for i in range(3)]
    rng = np.random.Generator(np.random.PCG64(20260049))
    x = torch.from_numpy(rng.standard_normal(hidden, dtype=np.float32)).to(dev)
    nw = torch.from_numpy(1.0 + 0.1 * rng.standard_normal(hidden, dtype=np.float32)).to(dev)
    out = torch.empty(hidden, dtype=torch.float32, device=dev)
    nscr = L.rfq_mlp_scratch_bytes(1, hidden, inter)
    scratch = torch.empty(nscr, dtype=torch.uint8, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = {}
    for key, one_call in (("us", 1), ("five_calls_us", 0)):
        ms = C.c_float(0)
        for w_, s_ in ((warmup, 1), (0, steps)):
            _lib.check(L.rfq_bench_mlp_swiglu(fmt, arr[0], arr[1], gu_bytes, fmt, arr[2], d_bytes, copies,
                                              C.c_void_p(x.data_ptr()), C.c_void_p(nw.data_ptr()), 1e-5,
                                              C.c_void_p(out.data_ptr()), 1, hidden, inter, C.c_void_p(scratch.data_ptr()),
                                              nscr, one_call, w_, s_, stream, C.byref(ms)))
        res[key] = round(ms.value / steps * 1e3, 2)
    b = 2 * gu_bytes + d_bytes + 4 * (3 * hidden)                  # the three matrices, x, the norm weight, the output
    res["GB/s"] = round(b / res["us"] / 1e3, 1)
    res["hbm_frac"] = round(b / res["us"] / 1e3 / HBM_PEAK_GBS, 4)
    return res


def time_host_path(torch, fmt, w, x, n, k):
    """The boundary with host-resident weights, as the reference's matmul_q4_k has it (the weights
    cross the host link on every call): rfq_upload of the packed weights from pageable memory beside
    the runtime's own pageable copy and a copy from pinned memory, and the whole rfq_matmul_host_weights."""
    import ctypes as C
    import numpy as np
    from rocmforge_amd import _lib
    L, dev = _lib.lib(), torch.device("cuda:0")
    nb = int(w.size)
    dst = torch.empty(nb, dtype=torch.uint8, device=dev)
    pin = torch.empty(nb, dtype=torch.uint8, pin_memory=True)
    pin.numpy()[:] = w
    dx = torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    dy = torch.empty(n, dtype=torch.float32, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def best(f, reps=5):
        f()
        torch.cuda.synchronize()
        t = 1e9
        for _ in range(reps):
            t0 = time.perf_counter()
            f()
            torch.cuda.synchronize()
            t = min(t, time.perf_counter() - t0)
        return t

    t_up = best(lambda: _lib.check(L.rfq_upload(C.c_void_p(w.ctypes.data), nb, C.c_void_p(dst.data_ptr()), stream)))
    t_page = best(lambda: dst.copy_(torch.from_numpy(w)))
    t_pin = best(lambda: dst.copy_(pin, non_blocking=True))
    t_mm = best(lambda: _lib.check(L.rfq_matmul_host_weights(fmt, C.c_void_p(w.ctypes.data), nb, C.c_void_p(dx.data_ptr()), n, k,
                                                             C.c_void_p(dy.data_ptr()), stream)))
    return {"MB": round(nb / 1e6, 1), "rfq_upload_GB/s": round(nb / t_up / 1e9, 1), "pageable_copy_GB/s": round(nb / t_page / 1e9, 1),
            "pinned_copy_GB/s": round(nb / t_pin / 1e9, 1), "matmul_host_weights_ms": round(t_mm * 1e3, 3)}


def _omp_threads(nthreads):
    import ctypes as C
    C.CDLL("libgomp.so.1").omp_set_num_threads(int(nthreads))


def cpu_baseline(fmt, w, x, n, k, budget_s=8.0):
    """The CPU oracle (dequantise everything, then the sequential fp32 matmul)
    on one host thread, repeated until ~budget_s of CPU work."""
    import ctypes as C

    import numpy as np

    import oracle
    L = oracle.lib()
    _omp_threads(1)
    wd = np.empty(n * k, np.float32)
    c = np.empty(n, np.float32)
    reps, spent = 0, 0.0
    while spent < budget_s and reps < 64:
        t = time.perf_counter()
        rc = L.rf_qmatmul_nk_staged(fmt, w.ctypes.data_as(C.c_void_p), w.size, x.ctypes.data_as(C.c_void_p), 1, n, k,
                                    wd.ctypes.data_as(C.c_void_p), c.ctypes.data_as(C.c_void_p))
        assert rc == 0
        spent += time.perf_counter() - t
        reps += 1
    _omp_threads(os.cpu_count() or 1)
    return spent / reps, reps, c


def cpu_baseline_more(Q, fmt, w, x, n, k, threads):
    """The other legs of the CPU baseline, each a few repetitions (about 10 s together):
      * the headline GEMV with `threads` OpenMP threads (rows spread over threads, each row dequantised and
        multiplied by its thread; the reference itself is single-threaded);
      * dequantisation alone of a 4096 x 4096 tensor in Q4_0 and Q8_0, one thread, beside the figures the reference
        publishes for exactly that (benchmarks/baselines/rdna3-baseline.json:187-237: 12.8 ms and 15.2 ms);
      * the Q4_0 and Q8_0 decode configurations (4864 x 896; 4096 x 4096 at m = 1 and 8) in full, one thread;
      * the two prefill GEMMs at M = 1 and M = 4 rows (dequantise all of W once, then the sequential fp32 matmul
        per row, one thread), with the linear extrapolation to their full M labelled as such."""
    import ctypes as C

    import numpy as np

    import oracle
    L = oracle.lib()
    p = lambda a: a.ctypes.data_as(C.c_void_p)

    def best_of(f, reps):
        t = 1e30
        for _ in range(reps):
            t0 = time.perf_counter()
            f()
            t = min(t, time.perf_counter() - t0)
        return t

    out = {}
    _omp_threads(threads)
    y = np.empty(n, np.float32)
    t = best_of(lambda: L.rf_qmatmul_nk(fmt, p(w), w.size, p(x), 1, n, k, None, 0, p(y)), 5)
    out["gemv_all_threads"] = {"threads": threads, "ms_per_step": round(t * 1e3, 2),
                               "GB/s": round((w.size + 4 * k + 4 * n) / t / 1e9, 2),
                               "what": "the same GEMV, rows spread over OpenMP threads (per-row dequantise + dot)"}
    _omp_threads(1)
    for name, f, ref_ms in (("Q4_0", Q.Q4_0, 12.8), ("Q8_0", Q.Q8_0, 15.2)):
        wq = Q.make_weights(f, 4096, 4096, seed=20260021)
        dst = np.empty(4096 * 4096, np.float32)
        t = best_of(lambda: L.rf_dequantize(f, p(wq), wq.size, dst.size, p(dst)), 5)
        out[f"dequant_{name}_4096x4096"] = {"ms": round(t * 1e3, 2), "Gelem/s": round(dst.size / t / 1e9, 2), "threads": 1,
                                            "reference_published_ms": ref_ms}
    # the two other decode configurations, measured in full: dequantise all weights, then the sequential matmul
    rng = np.random.Generator(np.random.PCG64(20260061))
    for name, f, gm, gn, gk in (("Q4_0_gemv_4864x896_m1", Q.Q4_0, 1, 4864, 896), ("Q8_0_gemv_4096x4096_m1", Q.Q8_0, 1, 4096, 4096),
                                ("Q8_0_gemv_4096x4096_m8", Q.Q8_0, 8, 4096, 4096)):
        wq = Q.make_weights(f, gn, gk, seed=20260063)
        wd = np.empty(gn * gk, np.float32)
        a = rng.standard_normal((gm, gk), dtype=np.float32)
        c = np.empty(gm * gn, np.float32)
        t = best_of(lambda: L.rf_qmatmul_nk_staged(f, p(wq), wq.size, p(a), gm, gn, gk, p(wd), p(c)), 3)
        out[name] = {"ms": round(t * 1e3, 2), "GB/s": round((wq.size + 4 * gm * gk + 4 * gm * gn) / t / 1e9, 3), "threads": 1}
    for name, f, gm, gn, gk in (("Q4_K_gemm_512x4096x14336", Q.Q4_K, 512, 14336, 4096),
                                ("MXFP4_gemm_2048x8192x28672", Q.MXFP4, 2048, 28672, 8192)):
        slab = Q.make_weights(f, 4096 if gn % 4096 == 0 else gn, gk, seed=20260062)
        wq = np.tile(slab, gn // 4096) if gn % 4096 == 0 else slab
        wd = np.empty(gn * gk, np.float32)
        res = {}
        for m in (1, 4):
            a = rng.standard_normal((m, gk), dtype=np.float32)
            c = np.empty(m * gn, np.float32)
            t = best_of(lambda: L.rf_qmatmul_nk_staged(f, p(wq), wq.size, p(a), m, gn, gk, p(wd), p(c)), 1 if gn > 20000 else 2)
            res[f"m{m}_ms"] = round(t * 1e3, 1)
        per_row = (res["m4_ms"] - res["m1_ms"]) / 3.0
        fixed = res["m1_ms"] - per_row
        res["extrapolated_full_m_ms"] = round(fixed + per_row * gm, 1)
        res["extrapolation"] = f"linear in M from M = 1 and M = 4 (dequantise once + {gm} rows of the fp32 matmul), not measured"
        res["extrapolated_GFLOP/s"] = round(2.0 * gm * gn * gk / (res["extrapolated_full_m_ms"] * 1e-3) / 1e9, 2)
        res["threads"] = 1
        out[name] = res
    _omp_threads(os.cpu_count() or 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-also", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--no-warm", action="store_true", help="skip the cache-resident variant (profiling runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain elementwise copy of 256 MiB five times (for scaling HBM byte counters "
                         "of a profiler against a kernel of known traffic)")
    ap.add_argument("--only-mlp", action="store_true", help="only the SwiGLU MLP line (profiling runs)")
    ap.add_argument("--mlp-steps", type=int, default=300)
    ap.add_argument("--only-gguf", action="store_true", help="only the GGUF-layout Q4_K GEMV line (profiling runs)")
    ap.add_argument("--only-dequant", action="store_true", help="only the dequantisation lines (profiling runs)")
    ap.add_argument("--only-gemv", metavar="FMT:NxK:M", help="only one decode GEMV, e.g. MXFP4:14336x4096:1 (profiling runs)")
    ap.add_argument("--timeline", metavar="FMT:NxK", help="where one decode GEMV launch spends its time, from clock readings "
                    "inside the kernel, e.g. Q4_K:14336x4096 (text, not JSON)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is single-GPU (one MI355X per box); run with --gpus 1. "
                 "The path shards by output rows with no exchange during compute.")

    import numpy as np
    import torch

    from rocmforge_amd import quantize as Q
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import rocmforge_amd
    rocmforge_amd.lib()  # fail loudly if librfq.so is missing

    if args.only_mlp:
        print(json.dumps({"Q4_K mlp_swiglu 4096x14336 m1": time_mlp(torch, Q.Q4_K, 4096, 14336, Q, steps=args.mlp_steps)}))
        return

    if args.only_dequant:
        res = {}
        for name, f, n, k, seed in (("Q4_K dequant 14336x4096", Q.Q4_K, N, K, 20260023),
                                    ("MXFP4 dequant 28672x8192", Q.MXFP4, 28672, 8192, 20260025)):
            t, b = time_dequant(torch, f, n, k, min(args.steps, 50), min(args.warmup, 5), Q, seed)
            res[name] = {"GB/s": round(b / t / 1e9, 1), "us": round(t * 1e6, 2), "hbm_frac": round(b / t / 1e9 / HBM_PEAK_GBS, 4),
                         "algorithmic_bytes": b}
        print(json.dumps(res))
        return

    if args.timeline:
        name, shape = args.timeline.split(":")
        f = {v: k_ for k_, v in Q.NAMES.items()}[name]
        n_, k_ = (int(t) for t in shape.split("x"))
        c = min(-(-int(2.5 * CACHE_BYTES) // Q.packed_bytes(f, n_ * k_)), 64)
        kern, us = gemv_timeline(torch, f, n_, k_, c, args.warmup, Q, 20260061)
        if us is None:
            print(f"{kern}: no build of this kernel stamps its timeline")
        else:
            print_timeline(name, n_, k_, kern, us, args.warmup)
        return

    if args.only_gemv:
        name, shape, mm = args.only_gemv.split(":")
        f = {v: k_ for k_, v in Q.NAMES.items()}[name]
        n_, k_ = (int(t) for t in shape.split("x"))
        m_ = int(mm)
        c = min(-(-int(2.5 * CACHE_BYTES) // Q.packed_bytes(f, n_ * k_)), 64)
        _, d, *_ = time_gemv(torch, f, n_, k_, m_, c, args.steps, args.warmup, Q, 20260060)
        b = algorithmic_bytes(f, n_, k_, m_, Q)
        from rocmforge_amd import _lib
        kern = _lib.lib().rfq_bench_last_gemv_kernel().decode()
        # the floor for these bytes: a kernel that only reads them, launched the same way
        floor_s, floor_shape = read_floor(torch, Q.packed_bytes(f, n_ * k_), c, min(args.steps, 500), min(args.warmup, 50))
        print(json.dumps({f"{name} gemv {n_}x{k_} m{m_}": {
            "GB/s": round(b / (d / args.steps) / 1e9, 1), "us": round(d / args.steps * 1e6, 2),
            "hbm_frac": round(b / (d / args.steps) / 1e9 / HBM_PEAK_GBS, 4), "algorithmic_bytes": b, "weight_copies": c,
            "kernel": kern, "read_only_kernel_us": round(floor_s * 1e6, 2), "read_only_kernel": floor_shape,
            "over_read_only_kernel": round(d / args.steps / floor_s - 1.0, 4)}}))
        return

    if args.only_gguf:
        f = Q.GGUF_Q4_K
        c = min(-(-int(2.5 * CACHE_BYTES) // Q.packed_bytes(f, N * K)), 64)
        _, d, *_ = time_gemv(torch, f, N, K, 1, c, args.steps, args.warmup, Q, 20260051)
        b = algorithmic_bytes(f, N, K, 1, Q)
        print(json.dumps({"GGUF_Q4_K gemv 14336x4096": {"GB/s": round(b / (d / args.steps) / 1e9, 1), "us": round(d / args.steps * 1e6, 2),
                                                        "hbm_frac": round(b / (d / args.steps) / 1e9 / HBM_PEAK_GBS, 4),
                                                        "algorithmic_bytes": b, "weight_copies": c}}))
        return

    fmt = Q.Q4_K
    wbytes = Q.packed_bytes(fmt, N * K)
    copies = -(-int(2.5 * CACHE_BYTES) // wbytes)          # 11 copies, 646 MB > 2.5x the last-level cache
    abytes = algorithmic_bytes(fmt, N, K, 1, Q)
    # Three runs of the same loop over the same buffers: straight out of idle (the launches of the first tens of
    # milliseconds after an idle period run about 5 % slower: the part's clocks ramp), then PREHEAT_MS of untimed
    # launches, then the measurement proper (W warm-up launches, K timed ones), which is what `value` reports.
    head = GemvRun(torch, fmt, N, K, 1, copies, Q, 20260003)
    _, idle_s = head.run(args.warmup, args.steps)
    per_launch = max(idle_s / args.steps, 5e-6)
    head.run(1, max(1, int(PREHEAT_MS * 1e-3 / per_launch)))
    wall, dev_s = head.run(args.warmup, args.steps)
    w, x, y = head.w, head.x, head.y.cpu().numpy()
    from rocmforge_amd import _lib
    kernel_name = _lib.lib().rfq_bench_last_gemv_kernel().decode()
    ms_per_step = dev_s / args.steps * 1e3
    achieved = abytes / (dev_s / args.steps) / 1e9
    value = achieved
    floor_s, floor_shape = read_floor(torch, wbytes, copies, min(args.steps, 500), min(args.warmup, 50))

    # warm variant (one copy, cache-resident) for the record
    dev_w = None
    if not args.no_warm:
        _, dev_w, *_ = time_gemv(torch, fmt, N, K, 1, 1, args.steps, args.warmup, Q, 20260003)

    # the counters of the committed profile belong to one kernel: report them only while the dispatcher still takes it
    import re
    traffic, traffic_kernel = measured_traffic_bytes()
    def _shape(name):                                      # "gemv_idot_kernel<12, 1, 2, 7, false>" / "...<Q4_K,1,2,7>" -> (name, [1, 2, 7])
        m_ = re.match(r"(\w+)<([^>]*)>", name or "")
        return (m_.group(1), [t.strip() for t in m_.group(2).split(",")][1:4]) if m_ else None
    if _shape(traffic_kernel) != _shape(kernel_name):
        traffic = None

    out = {
        "metric": "Q4_K decode GEMV GB/s (% HBM peak); quant prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "wall_ms_per_step": round(wall / args.steps * 1e3, 6),
        "value_clock": "HIP events on the launch stream around the timed launches (roofline.achieved is the same figure)",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Q4_K decode GEMV W[14336x4096] (256-byte super-blocks), x fp32[4096], batch 1, "
                               f"{copies} rotating weight copies (cold HBM)",
                   "algorithmic_bytes_per_step": abytes, "weight_copies": copies,
                   "preheat_ms": PREHEAT_MS, "preheat": "untimed launches of the same loop before the W warm-up and K timed "
                   "launches, so that the part has left its idle clocks; the same K launches straight out of idle are "
                   "roofline.avg_launch_us_from_idle"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": TRAFFIC_SOURCE, "traffic_kernel": traffic_kernel,
                     "kernel": kernel_name, "avg_launch_us": round(dev_s / args.steps * 1e6, 3),
                     "avg_launch_us_from_idle": round(idle_s / args.steps * 1e6, 3),
                     "read_only_kernel_us": round(floor_s * 1e6, 3), "read_only_kernel": floor_shape,
                     "over_read_only_kernel": round(dev_s / args.steps / floor_s - 1.0, 4),
                     "warm_cache_gbs": round(abytes / (dev_w / args.steps) / 1e9, 1) if dev_w else None},
    }

    if args.calibrate_copy:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.add(src, 0.0, out=dst)                   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        out["config"]["calibration_copy"] = "5 x torch.add(src, 0, out=dst), 2^26 floats each way"

    if not args.no_also:
        also = {}
        for name, f, n, k, m, seed in (("Q6_K gemv 14336x4096", Q.Q6_K, N, K, 1, 20260013),
                                       ("Q8_0 gemv 4096x4096 m1", Q.Q8_0, 4096, 4096, 1, 20260002),
                                       ("Q8_0 gemv 4096x4096 m8", Q.Q8_0, 4096, 4096, 8, 20260002),
                                       ("Q4_0 gemv 4864x896", Q.Q4_0, 4864, 896, 1, 20260001),
                                       ("MXFP4 gemv 14336x4096", Q.MXFP4, N, K, 1, 20260041),
                                       ("MXFP6 gemv 14336x4096", Q.MXFP6_E2M3, N, K, 1, 20260042),
                                       # the matmul module's own decoders (nibble stride 20; bytes as int8)
                                       ("MM_Q4_K gemv 14336x4096", Q.MM_Q4_K, N, K, 1, 20260043),
                                       ("MM_Q8_0 gemv 4096x4096 m1", Q.MM_Q8_0, 4096, 4096, 1, 20260044)):
            c = -(-int(2.5 * CACHE_BYTES) // Q.packed_bytes(f, n * k))
            c = min(c, 64)
            _, d, *_ = time_gemv(torch, f, n, k, m, c, 500, 50, Q, seed)
            b = algorithmic_bytes(f, n, k, m, Q)
            also[name] = {"GB/s": round(b / (d / 500) / 1e9, 1), "us": round(d / 500 * 1e6, 2),
                          "hbm_frac": round(b / (d / 500) / 1e9 / HBM_PEAK_GBS, 4)}
        # the vocabulary projection, the largest GEMV of a decode step (525 MB: cold by size, one copy)
        _, d, *_ = time_gemv(torch, Q.Q4_K, 128256, 4096, 1, 1, 50, 5, Q, 20260031)
        b = algorithmic_bytes(Q.Q4_K, 128256, 4096, 1, Q)
        also["Q4_K gemv 128256x4096 (LM head)"] = {"GB/s": round(b / (d / 50) / 1e9, 1), "us": round(d / 50 * 1e6, 2),
                                                   "hbm_frac": round(b / (d / 50) / 1e9 / HBM_PEAK_GBS, 4)}
        # the block layouts of GGUF model files (no counterpart in the reference: reported beside, never as its parity)
        for name, f, n, k, m, seed in (("GGUF_Q4_K gemv 14336x4096", Q.GGUF_Q4_K, N, K, 1, 20260051),
                                       ("GGUF_Q6_K gemv 14336x4096", Q.GGUF_Q6_K, N, K, 1, 20260052),
                                       ("GGUF_Q8_0 gemv 4096x4096 m1", Q.GGUF_Q8_0, 4096, 4096, 1, 20260053),
                                       ("GGUF_Q8_0 gemv 4096x4096 m8", Q.GGUF_Q8_0, 4096, 4096, 8, 20260053),
                                       ("GGUF_Q4_0 gemv 4864x896", Q.GGUF_Q4_0, 4864, 896, 1, 20260054)):
            c = min(-(-int(2.5 * CACHE_BYTES) // Q.packed_bytes(f, n * k)), 64)
            _, d, *_ = time_gemv(torch, f, n, k, m, c, 500, 50, Q, seed)
            b = algorithmic_bytes(f, n, k, m, Q)
            also[name] = {"GB/s": round(b / (d / 500) / 1e9, 1), "us": round(d / 500 * 1e6, 2),
                          "hbm_frac": round(b / (d / 500) / 1e9 / HBM_PEAK_GBS, 4)}
        also["Q4_K gemv_kn n=14336 k=4096 (the orientation the reference computes)"] = time_gemv_kn(torch, Q.Q4_K, N, K, Q)
        also["Q4_K mlp_swiglu 4096x14336 m1"] = time_mlp(torch, Q.Q4_K, 4096, 14336, Q)
        also["Q4_K get_rows 512 of 128256x4096"] = time_get_rows(torch, Q.Q4_K, 128256, 4096, 512, Q)
        for name, f, n, k, seed in (("Q4_0 dequant 4096x4096", Q.Q4_0, 4096, 4096, 20260021),
                                    ("Q4_K dequant 14336x4096", Q.Q4_K, N, K, 20260023),
                                    ("MXFP4 dequant 28672x8192", Q.MXFP4, 28672, 8192, 20260025)):
            t, b = time_dequant(torch, f, n, k, 50, 5, Q, seed)
            also[name] = {"GB/s": round(b / t / 1e9, 1), "us": round(t * 1e6, 2), "hbm_frac": round(b / t / 1e9 / HBM_PEAK_GBS, 4),
                          "Gelem/s": round(n * k / t / 1e9, 1)}
        also["Q4_K 14336x4096 weights from host memory"] = time_host_path(torch, fmt, w, x[0], N, K)
        try:
            import bench_gemm
            also.update(bench_gemm.run(torch))
        except ImportError:
            pass
        out["also"] = also
        out["also_preheat_ms"] = PREHEAT_MS   # every GEMV line above was timed after that many ms of untimed launches, like `value`

    if not args.no_cpu:
        t_cpu, reps, c = cpu_baseline(fmt, w, x[0], N, K)
        ref = c.astype(np.float64)
        rms = float(np.sqrt(np.mean(ref * ref)))
        err = float(np.max(np.abs(y[0] - ref) / np.maximum(np.abs(ref), rms)))
        threads = min(os.cpu_count() or 1, 16)
        out["cpu_baseline"] = {"value": round(abytes / t_cpu / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"the full 14336x4096 GEMV (dequantise all weights to f32, then the sequential "
                                         f"fp32 matmul), {reps} repetitions on one host thread",
                               "ms_per_step": round(t_cpu * 1e3, 2), "gpu_vs_cpu_max_rel_err": float(f"{err:.3e}"),
                               "host_cpus": os.cpu_count(), "compiler_flags": "gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp",
                               "more": cpu_baseline_more(Q, fmt, w, x[0], N, K, threads)}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
