"""CPU model of the arithmetic of the one-pass GGUF_Q4_K GEMM kernel (integer operands sc * q, accumulators in units of
the running super-block's d, mins as fp16 pairs against the activations' group sums): the scheme itself, in numpy with
the kernel's roundings, must give the float64 contraction of the decoded weights to fp32 level - for ordinary data and
for super-block scales of any size.  (The kernel is compared with the oracle on the GPU in test_gemm_f16_gpu.py.)"""
import numpy as np

from rocmforge_amd import quantize as Q

f32, f16 = np.float32, np.float16


def unpack(w, n, k):
    b = np.frombuffer(bytes(w), np.uint8).reshape(n, k // 256, 144)
    d = b[..., 0:2].copy().view("<f2")[..., 0].astype(f32)
    dmin = b[..., 2:4].copy().view("<f2")[..., 0].astype(f32)
    s = b[..., 4:16].astype(np.uint32)
    sc = np.concatenate([s[..., 0:4] & 63, (s[..., 8:12] & 15) | ((s[..., 0:4] >> 6) << 4)], axis=-1)
    mn = np.concatenate([s[..., 4:8] & 63, (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)], axis=-1)
    qs = b[..., 16:].reshape(n, k // 256, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, k // 256, 8, 32)
    return d, dmin, sc.astype(f32), mn.astype(f32), q.astype(f32)


def exponent_field(x):
    return (np.float32(x).view(np.uint32) >> 23) & 255


def one_pass_model(w, a, n, k):
    """out[m, n] as the kernel forms it; every product below is exact in float64 and sums are rounded to f32 per k-step of
    16 (the matrix instruction's own order inside a k-step is not modelled: it moves the result by fp32 rounding only)."""
    d, dmin, sc, mn, q = unpack(w, n, k)
    m = a.shape[0]
    a64 = a.astype(np.float64).reshape(m, k // 256, 8, 32)
    S = a.astype(f32).reshape(m, k // 256, 8, 32).sum(axis=3, dtype=f32)          # group sums, f32
    S_hi = S.astype(f16)
    S_lo = (S - S_hi.astype(f32)).astype(f16)
    out = np.zeros((m, n), f32)
    for r in range(n):
        acc = np.zeros(m, f32)
        unit = f32(1.0)
        for blk in range(k // 256):
            dv, dm = d[r, blk], dmin[r, blk]
            j = int(np.clip(int(exponent_field(dm)) - int(exponent_field(dv)) - 8, 0, 24))
            nxt = f32(dv * f32(2.0 ** j)) if dv != 0 else (f32(abs(dm)) if dm != 0 else unit)
            inv = f32(1.0) / nxt
            ratio = f32(1.0) if nxt == unit else f32(unit * inv)
            unit = nxt
            acc = (acc * ratio).astype(f32)
            v = (f32(-1.0) * (dm * mn[r, blk]).astype(f32) * inv).astype(f32)     # -(dmin * m) / unit, per sub-block
            hi = v.astype(f16)
            lo = (v - hi.astype(f32)).astype(f16)
            mins = (hi.astype(np.float64) * (S_hi[:, blk].astype(np.float64) + S_lo[:, blk].astype(np.float64))).sum(axis=1)
            acc = (acc + mins.astype(f32)).astype(f32)
            acc = (acc + (lo.astype(np.float64) * S_hi[:, blk].astype(np.float64)).sum(axis=1).astype(f32)).astype(f32)
            down = f32(2.0 ** -j) if dv != 0 else f32(0.0)
            s = (sc[r, blk] * down).astype(f16)                                  # exact
            assert np.array_equal(s.astype(f32), sc[r, blk] * down)
            op = (s.astype(np.float64)[:, None] * q[r, blk].astype(np.float64))   # sc * q * 2^-j
            assert np.array_equal(op.astype(f16).astype(np.float64), op)          # an fp16 number: exact operand
            prod = a64[:, blk] * op[None]                                         # [m, 8, 32]
            for step in range(16):                                                # k-steps of 16
                sb, half = step // 2, step % 2
                acc = (acc + prod[:, sb, 16 * half:16 * half + 16].sum(axis=1).astype(f32)).astype(f32)
        out[:, r] = acc * unit
    return out


def exact(w, a, n, k):
    d, dmin, sc, mn, q = unpack(w, n, k)
    w64 = (d.astype(np.float64)[..., None, None] * sc.astype(np.float64)[..., None] * q.astype(np.float64)
           - (dmin.astype(np.float64) * 1.0)[..., None, None] * mn.astype(np.float64)[..., None])
    return a.astype(np.float64) @ w64.reshape(n, k).T


def check(w, a, n, k, what):
    got, want = one_pass_model(w, a, n, k), exact(w, a, n, k)
    for r in range(n):
        rms = np.sqrt(np.mean(want[:, r] ** 2))
        err = np.max(np.abs(got[:, r] - want[:, r])) / (rms if rms > 0 else 1.0)
        assert err <= 4e-6, (what, r, err)


def acts(m, k, seed):
    return np.random.Generator(np.random.PCG64(seed)).standard_normal((m, k), dtype=f32).astype(f16)


def test_quantised_gaussian_weights():
    n, k = 12, 2048
    check(Q.make_weights(Q.GGUF_Q4_K, n, k, seed=5), acts(6, k, 6), n, k, "N(0, 0.02) weights")


def test_super_block_scales_of_any_size():
    n, k = 12, 2048
    w = Q.make_weights(Q.GGUF_Q4_K, n, k, seed=7).copy()
    blocks = w.reshape(n, k // 256, 144)
    d = blocks[:, :, 0:2].copy().view("<f2")[..., 0]
    dmin = blocks[:, :, 2:4].copy().view("<f2")[..., 0]
    d[0, :] = 0.0
    d[1, 0] = 0.0
    d[2, 7] = 0.0
    d[3, 3] = -0.0
    d[4, :] = -d[4, :]
    d[5, 1::2] *= f16(256.0)
    d[6, 1::2] /= f16(256.0)                      # the mins leave the fp16 range against this d: the unit is d * 2^j
    d[7, 2] *= f16(-64.0)
    dmin[8, 2] = 0.0
    dmin[9, :] = -dmin[9, :]
    d[10, :] = 0.0
    dmin[10, :] = 0.0                             # a row of zeros
    blocks[:, :, 0:2] = d.astype("<f2")[..., None].view(np.uint8)
    blocks[:, :, 2:4] = dmin.astype("<f2")[..., None].view(np.uint8)
    check(w, acts(5, k, 8), n, k, "special scales")
