"""Seeded block generators / quantisers for the byte layouts ROCmForge decodes.

ROCmForge ships no quantiser for Q4_0 / Q8_0 / Q4_K / Q6_K (only decoders), so
these produce *inputs*: both the HIP path and the CPU check consume the same
bytes.  The MXFP packers restate ``MxfpBlock::pack_mxfp4`` / ``pack_mxfp6``
(src/loader/mxfp.rs:77-117, 142-174) vectorised over blocks.

Layouts (all little-endian, blocks run along the last axis):
  Q4_0   20 B / 32 elts : f32 scale, 16 nibble bytes, element 2i = low nibble
                          of byte i, 2i+1 = high nibble; value = scale*(q-8)
                          (src/kernels/quant/q4_0.rs:266-310)
  Q8_0   36 B / 32 elts : f32 scale, 32 offset-binary bytes; (b-128)*scale
                          (src/kernels/quant/q8_0.rs:23-71)
  Q4_K  256 B / 256 elts: 8 f16 scales @0, 8 i8 mins @16, nibbles @32 with a
                          28-byte stride per 32-element sub-block (16 used);
                          value = min + q*scale (src/kernels/quant/q4_k.rs:201-273)
  Q6_K  256 B / 256 elts: 16 f16 scales @0, 192 B LSB-first 6-bit stream @32,
                          32 B padding; signed6*scale (src/kernels/quant/q6_k.rs:201-266)
  MXFP4  17 B / 32 elts : i8 exponent, 16 nibble bytes, element 2j = HIGH nibble
                          (src/loader/dequant.rs:41-82)
  MXFP6  25 B / 32 elts : i8 exponent, 24 packed bytes (src/loader/dequant.rs:85-132)
"""
from __future__ import annotations

import numpy as np

Q4_0, Q8_0, Q4_K, Q6_K, MXFP4, MXFP6_E2M3, MXFP6_E3M2 = 2, 8, 12, 14, 20, 21, 22
# the loader's other K types (src/loader/dequant.rs:150-420): dequantisation only
Q2_K, Q3_K, Q5_K = 10, 11, 13
DEQUANT_ONLY_FORMATS = (Q2_K, Q3_K, Q5_K)
# the block layouts of GGUF model files (ggml), which ROCmForge does not decode: 100 + the ggml type id
GGUF_Q4_0, GGUF_Q8_0, GGUF_Q4_K, GGUF_Q6_K = 102, 108, 112, 114
GGUF_FORMATS = (GGUF_Q4_0, GGUF_Q8_0, GGUF_Q4_K, GGUF_Q6_K)
# what the decoders of src/kernels/matmul/quantized/ read (q8_0.rs:18-56: int8 bytes; q4_k.rs:90-148: nibbles at
# 32 + 20 * sub-block; q6_k.rs:90-148: the canonical stream; the K scales through common.rs:44-60): 200 + the id
# of the format they are a variant of
MM_Q8_0, MM_Q4_K, MM_Q6_K = 208, 212, 214
MM_FORMATS = (MM_Q8_0, MM_Q4_K, MM_Q6_K)

BLOCK_ELEMS = {Q2_K: 256, Q3_K: 256, Q5_K: 256, Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, MXFP4: 32, MXFP6_E2M3: 32, MXFP6_E3M2: 32,
               GGUF_Q4_0: 32, GGUF_Q8_0: 32, GGUF_Q4_K: 256, GGUF_Q6_K: 256, MM_Q8_0: 32, MM_Q4_K: 256, MM_Q6_K: 256}
BLOCK_BYTES = {Q2_K: 256, Q3_K: 256, Q5_K: 256, Q4_0: 20, Q8_0: 36, Q4_K: 256, Q6_K: 256, MXFP4: 17, MXFP6_E2M3: 25, MXFP6_E3M2: 25,
               GGUF_Q4_0: 18, GGUF_Q8_0: 34, GGUF_Q4_K: 144, GGUF_Q6_K: 210, MM_Q8_0: 36, MM_Q4_K: 256, MM_Q6_K: 256}
NAMES = {Q2_K: "Q2_K", Q3_K: "Q3_K", Q5_K: "Q5_K", Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", MXFP4: "MXFP4",
         MXFP6_E2M3: "MXFP6_E2M3", MXFP6_E3M2: "MXFP6_E3M2",
         GGUF_Q4_0: "GGUF_Q4_0", GGUF_Q8_0: "GGUF_Q8_0", GGUF_Q4_K: "GGUF_Q4_K", GGUF_Q6_K: "GGUF_Q6_K",
         MM_Q8_0: "MM_Q8_0", MM_Q4_K: "MM_Q4_K", MM_Q6_K: "MM_Q6_K"}


def packed_bytes(fmt: int, n_elems: int) -> int:
    be = BLOCK_ELEMS[fmt]
    return ((n_elems + be - 1) // be) * BLOCK_BYTES[fmt]


def _blocks(w: np.ndarray, be: int) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.float32).ravel()
    if w.size % be:
        w = np.concatenate([w, np.zeros(be - w.size % be, np.float32)])
    return w.reshape(-1, be)


def _f16_round(x: np.ndarray) -> np.ndarray:
    return x.astype(np.float16).astype(np.float32)


def quantize_q4_0(w: np.ndarray) -> np.ndarray:
    """ggml-style Q4_0 decision rule (d = signed-absmax / -8, rounded through
    f16 as a GGUF file would hold it), stored in ROCmForge's 20-byte layout."""
    b = _blocks(w, 32)
    idx = np.argmax(np.abs(b), axis=1)
    mx = b[np.arange(b.shape[0]), idx]
    d = _f16_round(mx / -8.0)
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.floor(b * inv[:, None] + 8.5), 0, 15).astype(np.uint8)
    out = np.zeros((b.shape[0], 20), np.uint8)
    out[:, 0:4] = d.astype("<f4").view(np.uint8).reshape(-1, 4)
    out[:, 4:20] = q[:, 0::2] | (q[:, 1::2] << 4)
    return out.ravel()


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    """d = absmax/127 (f16-rounded), byte = round(x/d) + 128 (offset binary)."""
    b = _blocks(w, 32)
    amax = np.abs(b).max(axis=1)
    d = _f16_round(amax / 127.0)
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.rint(b * inv[:, None]), -127, 127).astype(np.int32) + 128
    out = np.zeros((b.shape[0], 36), np.uint8)
    out[:, 0:4] = d.astype("<f4").view(np.uint8).reshape(-1, 4)
    out[:, 4:36] = q.astype(np.uint8)
    return out.ravel()


def quantize_mm_q8_0(w: np.ndarray) -> np.ndarray:
    """The same decision rule with the bytes as two's-complement int8, which is how
    src/kernels/matmul/quantized/q8_0.rs:18-56 reads them."""
    out = quantize_q8_0(w).reshape(-1, 36).copy()
    out[:, 4:36] ^= 0x80                                  # offset binary -> two's complement
    return out.ravel()


def synth_mm_q4_k(n_superblocks: int, rng: np.random.Generator) -> np.ndarray:
    """Random super-blocks for the stride-20 reading (src/kernels/matmul/quantized/q4_k.rs:90-148): the same
    scales and mins as synth_q4_k; every other byte is random, so the nibble bytes are random wherever they
    are taken from."""
    return synth_q4_k(n_superblocks, rng)


def pack6_lsb(codes: np.ndarray) -> np.ndarray:
    """[..., 4g] 6-bit codes -> [..., 3g] bytes, LSB-first bit stream."""
    c = codes.astype(np.uint32).reshape(*codes.shape[:-1], -1, 4)
    word = c[..., 0] | (c[..., 1] << 6) | (c[..., 2] << 12) | (c[..., 3] << 18)
    out = np.stack([word & 0xFF, (word >> 8) & 0xFF, (word >> 16) & 0xFF], axis=-1).astype(np.uint8)
    return out.reshape(*codes.shape[:-1], -1)


def quantize_q6_k(w: np.ndarray, rng: np.random.Generator | None = None) -> np.ndarray:
    """Per 16-element group: scale = f16(absmax/31), q = round(x/scale) as a
    6-bit two's-complement code.  The 32 padding bytes get random content when
    ``rng`` is given (they must be ignored by every decoder)."""
    b = _blocks(w, 256)
    g = b.reshape(-1, 16, 16)
    amax = np.abs(g).max(axis=2)
    sc16 = (amax / 31.0).astype(np.float16)
    sc = sc16.astype(np.float32)
    inv = np.where(sc != 0, 1.0 / np.where(sc != 0, sc, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.rint(g * inv[:, :, None]), -32, 31).astype(np.int32) & 63
    out = np.zeros((b.shape[0], 256), np.uint8)
    out[:, 0:32] = sc16.view(np.uint8).reshape(-1, 32)
    out[:, 32:224] = pack6_lsb(q.reshape(-1, 256))
    if rng is not None:
        out[:, 224:256] = rng.integers(0, 256, (b.shape[0], 32), dtype=np.uint8)
    return out.ravel()


def synth_q4_k(n_superblocks: int, rng: np.random.Generator) -> np.ndarray:
    """Valid random Q4_K super-blocks.  The layout cannot hold a zero-mean
    Gaussian (integer ``min``, one-sided ``q*scale``), so blocks are drawn
    directly: scale = +-U[2^-8, 2^-5] as f16, min in {-2..2}, uniform nibbles,
    and random bytes in every position the decoder never reads."""
    n = n_superblocks
    out = rng.integers(0, 256, (n, 256), dtype=np.uint8)
    mag = rng.uniform(2.0 ** -8, 2.0 ** -5, (n, 8)).astype(np.float32)
    sign = rng.choice(np.array([-1.0, 1.0], np.float32), (n, 8))
    out[:, 0:16] = (mag * sign).astype(np.float16).view(np.uint8).reshape(n, 16)
    out[:, 16:24] = rng.integers(-2, 3, (n, 8)).astype(np.int8).view(np.uint8)
    return out.ravel()


def quantize_q4_k_onesided(w: np.ndarray, rng: np.random.Generator | None = None) -> np.ndarray:
    """Nearest representable Q4_K block for real data: per sub-block
    min = round(lowest value) (an integer), scale = f16((max-min)/15),
    q = round((x-min)/scale).  Coarse for small weights; used as a second,
    data-derived input family."""
    b = _blocks(w, 256)
    n = b.shape[0]
    s = b.reshape(n, 8, 32)
    mn = np.clip(np.rint(s.min(axis=2)), -128, 127).astype(np.float32)
    span = s.max(axis=2) - mn
    sc16 = (span / 15.0).astype(np.float16)
    sc = sc16.astype(np.float32)
    inv = np.where(sc != 0, 1.0 / np.where(sc != 0, sc, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.rint((s - mn[:, :, None]) * inv[:, :, None]), 0, 15).astype(np.uint8)
    out = (rng.integers(0, 256, (n, 256), dtype=np.uint8) if rng is not None
           else np.zeros((n, 256), np.uint8))
    out[:, 0:16] = sc16.view(np.uint8).reshape(n, 16)
    out[:, 16:24] = mn.astype(np.int8).view(np.uint8)
    nib = q[:, :, 0::2] | (q[:, :, 1::2] << 4)  # element 2i low nibble, 2i+1 high
    for sb in range(8):
        out[:, 32 + 28 * sb: 32 + 28 * sb + 16] = nib[:, sb, :]
    return out.ravel()


# ---------------------------------------------------------------- MXFP

_E2M1_MAG = np.array([0.5, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0, 8.0], np.float32)   # code 0..7 (mxfp.rs:216-221)
_E2M3_MAG = np.array([(1.0 + m / 8.0) * 2.0 ** (e - 1) for e in range(4) for m in range(8)], np.float32)


def _round_half_away(x: np.ndarray) -> np.ndarray:
    return np.sign(x) * np.floor(np.abs(x) + np.float32(0.5))


def _e8m0_exponents(b: np.ndarray) -> np.ndarray:
    """E8M0::from_f32 on the block absmax (mxfp.rs:29-43); zero block -> 0."""
    amax = np.abs(b).max(axis=1)
    with np.errstate(divide="ignore"):
        l = np.log2(amax.astype(np.float32)).astype(np.float32)
    e = _round_half_away(np.clip(l, -127.0, 127.0))
    e = np.where(amax == 0, 0, e)
    e = np.where(np.isinf(amax), 127, e)
    return e.astype(np.int8)


def _pow2(e: np.ndarray) -> np.ndarray:
    return np.ldexp(np.float32(1.0), e.astype(np.int32)).astype(np.float32)


def _encode(norm: np.ndarray, table: np.ndarray, hi: float, sign_bit: int) -> np.ndarray:
    """Nearest table entry to clamp(|v|, 0.5, hi), the first (lowest code) on a
    tie -- the outcome of the reference's exhaustive strict-'<' search
    (mxfp.rs:212-228, 261-277), evaluated with midpoint thresholds: for a value
    between two neighbouring table entries both error terms are exact in f32,
    so comparing against the midpoint decides identically."""
    vals, first = np.unique(table, return_index=True)       # ascending distinct magnitudes
    mid = ((vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2).astype(np.float32)
    a = np.abs(norm)
    cl = np.minimum(np.maximum(a, np.float32(0.5)), np.float32(hi))
    code = first[np.searchsorted(mid, cl, side="left")].astype(np.uint8)
    code = code | np.where(norm < 0, sign_bit, 0).astype(np.uint8)
    return np.where(norm == 0, 0, code).astype(np.uint8)


def pack_mxfp4(values: np.ndarray) -> np.ndarray:
    b = _blocks(values, 32)
    e = _e8m0_exponents(b)
    norm = (b / _pow2(e)[:, None]).astype(np.float32)
    code = _encode(norm, _E2M1_MAG, 8.0, 0x08)
    out = np.zeros((b.shape[0], 17), np.uint8)
    out[:, 0] = e.view(np.uint8)
    out[:, 1:] = (code[:, 0::2] << 4) | (code[:, 1::2] & 0x0F)
    return out.ravel()


def pack_mxfp6(values: np.ndarray) -> np.ndarray:
    b = _blocks(values, 32)
    e = _e8m0_exponents(b)
    norm = (b / _pow2(e)[:, None]).astype(np.float32)
    code = _encode(norm, _E2M3_MAG, 7.5, 0x20)
    out = np.zeros((b.shape[0], 25), np.uint8)
    out[:, 0] = e.view(np.uint8)
    out[:, 1:] = pack6_lsb(code)
    return out.ravel()


# ---- GGUF file layouts (public ggml block definitions) ---------------------------------
#   GGUF_Q4_0  18 B / 32 : f16 d, 16 bytes; element j = low nibble of byte j, j + 16 = high nibble; d * (q - 8)
#   GGUF_Q8_0  34 B / 32 : f16 d, 32 int8; d * q
#   GGUF_Q4_K 144 B / 256: f16 d, f16 dmin, 12 bytes of 6-bit scales and mins (8 each), 128 nibble bytes; per
#                          64 elements: low nibbles then high nibbles of 32 bytes; d * sc * q - dmin * m
#   GGUF_Q6_K 210 B / 256: 128 bytes of low nibbles, 64 bytes of high bit pairs, 16 int8 scales, f16 d;
#                          d * sc * (q - 32)
# The quantisers below are simple decision rules (no search); they exist to produce valid inputs whose
# dequantised values approximate w, not to match ggml's quantiser bit for bit.

def _f16_bytes(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x, dtype="<f2").view(np.uint8)


def quantize_gguf_q4_0(w: np.ndarray) -> np.ndarray:
    b = _blocks(w, 32)
    idx = np.argmax(np.abs(b), axis=1)
    mx = b[np.arange(b.shape[0]), idx]
    d = _f16_round(mx / -8.0)
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.floor(b * inv[:, None] + 8.5), 0, 15).astype(np.uint8)
    out = np.zeros((b.shape[0], 18), np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:] = q[:, :16] | (q[:, 16:] << 4)
    return out.ravel()


def quantize_gguf_q8_0(w: np.ndarray) -> np.ndarray:
    b = _blocks(w, 32)
    d = _f16_round(np.abs(b).max(axis=1) / 127.0)
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.rint(b * inv[:, None]), -127, 127).astype(np.int8)
    out = np.zeros((b.shape[0], 34), np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.ravel()


def pack_scale_min_k4(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Eight 6-bit scales and eight 6-bit mins per block -> the 12 bytes get_scale_min_k4 reads."""
    sc, mn = sc.astype(np.uint8), mn.astype(np.uint8)
    out = np.zeros((sc.shape[0], 12), np.uint8)
    out[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    out[:, 4:8] = (mn[:, 0:4] & 63) | ((mn[:, 4:8] >> 4) << 6)
    out[:, 8:12] = (sc[:, 4:8] & 15) | ((mn[:, 4:8] & 15) << 4)
    return out


def quantize_gguf_q4_k(w: np.ndarray) -> np.ndarray:
    b = _blocks(w, 256).reshape(-1, 8, 32)                        # sub-blocks of 32
    lo = np.minimum(b.min(axis=2), 0.0)                           # value = scale * q - min, min >= 0
    scale = (b.max(axis=2) - lo) / 15.0
    d = _f16_round(scale.max(axis=1) / 63.0)
    dmin = _f16_round((-lo).max(axis=1) / 63.0)
    inv_d = np.where(d != 0, 1.0 / np.where(d != 0, d, 1.0), 0.0).astype(np.float32)
    inv_m = np.where(dmin != 0, 1.0 / np.where(dmin != 0, dmin, 1.0), 0.0).astype(np.float32)
    sc = np.clip(np.rint(scale * inv_d[:, None]), 0, 63)
    mn = np.clip(np.rint(-lo * inv_m[:, None]), 0, 63)
    eff_s = (d[:, None] * sc).astype(np.float32)
    eff_m = (dmin[:, None] * mn).astype(np.float32)
    inv_s = np.where(eff_s != 0, 1.0 / np.where(eff_s != 0, eff_s, 1.0), 0.0).astype(np.float32)
    q = np.clip(np.rint((b + eff_m[:, :, None]) * inv_s[:, :, None]), 0, 15).astype(np.uint8)
    out = np.zeros((b.shape[0], 144), np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:4] = _f16_bytes(dmin).reshape(-1, 2)
    out[:, 4:16] = pack_scale_min_k4(sc, mn)
    q = q.reshape(-1, 4, 2, 32)                                   # chunk of 64: low nibbles, then high nibbles
    out[:, 16:] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(-1, 128)
    return out.ravel()


def quantize_gguf_q6_k(w: np.ndarray) -> np.ndarray:
    b = _blocks(w, 256).reshape(-1, 16, 16)                       # groups of 16
    amax = np.abs(b).max(axis=2)
    scale = amax / 31.0
    d = _f16_round(scale.max(axis=1) / 127.0)
    inv_d = np.where(d != 0, 1.0 / np.where(d != 0, d, 1.0), 0.0).astype(np.float32)
    sc = np.clip(np.rint(scale * inv_d[:, None]), 0, 127).astype(np.int8)
    eff = (d[:, None] * sc).astype(np.float32)
    inv = np.where(eff != 0, 1.0 / np.where(eff != 0, eff, 1.0), 0.0).astype(np.float32)
    q = (np.clip(np.rint(b * inv[:, :, None]), -32, 31) + 32).astype(np.uint8).reshape(-1, 2, 4, 32)   # half, quarter, l
    out = np.zeros((b.shape[0], 210), np.uint8)
    lo, hi = q & 15, q >> 4
    ql = np.zeros((b.shape[0], 2, 64), np.uint8)
    ql[:, :, 0:32] = lo[:, :, 0, :] | (lo[:, :, 2, :] << 4)
    ql[:, :, 32:64] = lo[:, :, 1, :] | (lo[:, :, 3, :] << 4)
    qh = hi[:, :, 0, :] | (hi[:, :, 1, :] << 2) | (hi[:, :, 2, :] << 4) | (hi[:, :, 3, :] << 6)
    out[:, 0:128] = ql.reshape(-1, 128)
    out[:, 128:192] = qh.reshape(-1, 64)
    out[:, 192:208] = sc.view(np.uint8)
    out[:, 208:210] = _f16_bytes(d).reshape(-1, 2)
    return out.ravel()


def mxfp4_window_blocks(rng: np.random.Generator, nblk: int, exp_range=(-6, 1), zero_blocks: float = 0.05) -> np.ndarray:
    """Random MXFP4 blocks whose values span at most the four octaves a 4-bit matrix-core operand holds: every
    code of a window of exponents -1..2 or 0..3, zeros, both signs (the reference's packer only ever produces codes
    {0, 1, 8, 9} of the second window).  Full-entropy input for the 4-bit path of the prefill GEMM."""
    p_of_m = np.array([-1, 0, 0, 1, 1, 2, 2, 3])
    raw = np.zeros((nblk, 17), dtype=np.uint8)
    raw[:, 0] = rng.integers(exp_range[0], exp_range[1] + 1, size=nblk).astype(np.int8).view(np.uint8)
    codes = rng.integers(0, 16, size=(nblk, 32))
    lo = rng.integers(-1, 1, size=nblk)[:, None]
    p = p_of_m[codes & 7]
    codes = np.where((codes != 0) & ((p < lo) | (p > lo + 3)), 0, codes)
    if zero_blocks > 0:
        codes[rng.random(nblk) < zero_blocks] = 0                              # some all-zero blocks
    raw[:, 1:] = ((codes[:, 0::2] << 4) | codes[:, 1::2]).astype(np.uint8)     # element 2j in the high nibble
    return raw.reshape(-1)


def random_blocks(fmt: int, n_blocks: int, rng: np.random.Generator, exp_range=(-20, 12)) -> np.ndarray:
    """Uniformly random payload bytes with sane scales, covering every code."""
    bb = BLOCK_BYTES[fmt]
    out = rng.integers(0, 256, (n_blocks, bb), dtype=np.uint8)
    if fmt in GGUF_FORMATS:
        d = (rng.standard_normal((n_blocks, 2)) * 0.01).astype("<f2").view(np.uint8).reshape(-1, 4)
        if fmt in (GGUF_Q4_0, GGUF_Q8_0):
            out[:, 0:2] = d[:, 0:2]
        elif fmt == GGUF_Q4_K:
            out[:, 0:4] = d
        else:
            out[:, 208:210] = d[:, 0:2]
        return out.ravel()
    if fmt in (Q4_0, Q8_0, MM_Q8_0):
        s = (rng.standard_normal(n_blocks) * 0.01).astype("<f4")
        out[:, 0:4] = s.view(np.uint8).reshape(-1, 4)
    elif fmt in (Q4_K, MM_Q4_K):
        return synth_q4_k(n_blocks, rng)
    elif fmt in (Q6_K, Q3_K, Q5_K, MM_Q6_K):
        s = (rng.standard_normal((n_blocks, 16)) * 0.01).astype(np.float16)
        out[:, 0:32] = s.view(np.uint8).reshape(-1, 32)
    elif fmt == Q2_K:                                     # f16 scales, then f16 mins
        s = (rng.standard_normal((n_blocks, 32)) * 0.01).astype(np.float16)
        out[:, 0:64] = s.view(np.uint8).reshape(-1, 64)
    else:
        out[:, 0] = rng.integers(exp_range[0], exp_range[1] + 1, n_blocks).astype(np.int8).view(np.uint8)
    return out.ravel()


def make_weights(fmt: int, n: int, k: int, seed: int, std: float = 0.02) -> np.ndarray:
    """Seeded W[n,k] ~ N(0, std) quantised to ``fmt`` (Q4_K: synthetic blocks)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    if fmt in (Q4_K, MM_Q4_K):
        return synth_q4_k(n * k // 256, rng)
    w = (rng.standard_normal((n, k), dtype=np.float32) * np.float32(std))
    if fmt == MM_Q8_0:
        return quantize_mm_q8_0(w)
    if fmt == MM_Q6_K:
        return quantize_q6_k(w, rng)
    if fmt == Q4_0:
        return quantize_q4_0(w)
    if fmt == Q8_0:
        return quantize_q8_0(w)
    if fmt == Q6_K:
        return quantize_q6_k(w, rng)
    if fmt in GGUF_FORMATS:
        return {GGUF_Q4_0: quantize_gguf_q4_0, GGUF_Q8_0: quantize_gguf_q8_0, GGUF_Q4_K: quantize_gguf_q4_k,
                GGUF_Q6_K: quantize_gguf_q6_k}[fmt](w)
    if fmt == MXFP4:
        return pack_mxfp4(w)
    return pack_mxfp6(w)
