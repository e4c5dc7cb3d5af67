"""Pins the oracle's restatements of the decoders the matmul module carries beside the loader's
(src/kernels/matmul/quantized/: q8_0.rs:18-56, q4_k.rs:90-148, q6_k.rs:90-148, common.rs:44-60) and of the
orientation its matmuls compute (q4_0.rs:274-311 with src/tensor/matmul.rs:219-233).  CPU only.

What pins what:
  * the reference's own vector for the int8 decoder (quantized/q8_0.rs:113-131) and the recipe of its GPU test
    (quantized/q4_0.rs:343-435: shapes and byte pattern), evaluated independently in float64;
  * f16_to_f32_cpu on all 65 536 patterns against a statement of it in numpy integers of Rust's widths (its mantissa
    shift runs in u16 and keeps mantissa bits 0..2 only), a closed form, and hand values;
  * whole-array numpy statements of the three layouts written from the Rust, compared bit for bit on random blocks
    (a wrong stride, nibble order, sign extension or operand order fails them);
  * the canonical decoders wherever the two families must agree (normal scales whose mantissa bits 3..9 are clear, the
    only ones both widenings read alike: Q6_K as a whole; sub-block 0 of Q4_K, whose nibbles start at byte 32 under
    either stride), and that they part ways on any other scale.
The reference holds no vector for f16_to_f32_cpu itself; what is checked is its arithmetic as written, branch
included (the branch for zero and subnormals can never be taken: the exponent it tests is field + 112)."""
import struct

import numpy as np
import pytest

from rocmforge_amd import quantize as Q

MM_Q8_0, MM_Q4_K, MM_Q6_K = 208, 212, 214


def f32le(v):
    return np.frombuffer(struct.pack("<f", v), np.uint8)


def mm_f16_numpy(bits):
    """f16_to_f32_cpu (quantized/common.rs:44-60) with every intermediate in the integer width Rust gives it:
    `bits` is u16, so `(bits & 0x03FF) << 13` is a 16-bit shift whose high bits fall off before `as u32`."""
    bits = np.asarray(bits).astype(np.uint16)
    sign = np.where((bits & np.uint16(0x8000)) != 0, np.uint32(1 << 31), np.uint32(0)).astype(np.uint32)
    exp = ((bits & np.uint16(0x7C00)) >> np.uint16(10)).astype(np.int32) - 15 + 127
    mant16 = (bits & np.uint16(0x03FF)) << np.uint16(13)
    assert mant16.dtype == np.uint16                                  # the shift stayed in 16 bits
    mant = mant16.astype(np.uint32)
    normal = (sign | (exp.astype(np.uint32) << np.uint32(23)) | mant).astype(np.uint32).view(np.float32)
    zero = sign.view(np.float32)
    return np.where(exp <= 0, np.where((bits & np.uint16(0x7FFF)) == 0, zero, np.float32(0.0)), normal).astype(np.float32)


def test_f16_mm_all_patterns(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = np.array([L.rf_f16_to_f32_mm(int(b)) for b in bits], dtype=np.float32)
    want = mm_f16_numpy(bits)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # closed form: +-2^(field - 15) * (1 + (bits & 7) / 1024) -- mantissa bits 3..9 never arrive
    b = bits.astype(np.int64)
    closed = np.where(b & 0x8000, -1.0, 1.0) * 2.0 ** (((b >> 10) & 31) - 15.0) * (1.0 + (b & 7) / 1024.0)
    assert np.array_equal(got.astype(np.float64), closed)
    # it equals IEEE widening exactly where mantissa bits 3..9 are clear and the number is normal (1/128 of them), and by
    # coincidence on the subnormal +-0x0200 = 2^-15, which this routine reads as 2^-15 * (1 + 0)
    ieee = bits.view(np.float16).astype(np.float32)
    field = (bits >> 10) & 31
    same = got.view(np.uint32) == ieee.view(np.uint32)
    assert np.array_equal(same, ((field >= 1) & (field <= 30) & ((bits & 0x03F8) == 0)) | ((bits & 0x7FFF) == 0x0200))
    assert same.sum() == 2 * 30 * 8 + 2


def test_f16_mm_hand_values(oracle):
    L = oracle.lib()
    assert L.rf_f16_to_f32_mm(0x3C00) == np.float32(1.0)               # the powers of two the reference's tests use
    assert L.rf_f16_to_f32_mm(0x4000) == np.float32(2.0)
    assert L.rf_f16_to_f32_mm(0x3E00) == np.float32(1.0)               # IEEE 1.5: mantissa bit 9 is shifted out
    assert L.rf_f16_to_f32_mm(0x2E66) == np.float32(0.0625 * (1.0 + 6.0 / 1024.0))   # IEEE 0.1 -> 0.062866...
    assert abs(L.rf_f16_to_f32_mm(0x2E66) - 0.0628662109375) == 0.0
    assert L.rf_f16_to_f32_mm(0xC007) == np.float32(-2.0 * (1.0 + 7.0 / 1024.0))
    assert L.rf_f16_to_f32_mm(0) == np.float32(2.0 ** -15)             # not 0.0: the zero branch is dead code
    assert L.rf_f16_to_f32_mm(0x8000) == np.float32(-(2.0 ** -15))
    assert L.rf_f16_to_f32_mm(0x7C00) == np.float32(65536.0)           # not inf
    assert L.rf_f16_to_f32_mm(0x03FF) == np.float32(2.0 ** -15 * (1.0 + 7.0 / 1024.0))


def test_mm_q8_0_reference_vector(oracle):
    # quantized/q8_0.rs:113-131: scale 1.0, bytes (i - 16) as u8 -> i - 16
    d = np.zeros(36, np.uint8)
    d[0:4] = f32le(1.0)
    d[4:36] = (np.arange(32) - 16).astype(np.int8).view(np.uint8)
    r = oracle.dequantize(MM_Q8_0, d, 32)
    assert np.array_equal(r, (np.arange(32) - 16).astype(np.float32))
    # the loader's decoder reads the same bytes as offset binary: different numbers
    assert oracle.dequantize(Q.Q8_0, d, 32)[0] == np.float32(240.0 - 128.0)


def test_mm_q8_0_numpy_statement(oracle):
    rng = np.random.default_rng(11)
    nb = 300
    blocks = Q.random_blocks(MM_Q8_0, nb, rng).reshape(nb, 36)
    scale = blocks[:, 0:4].copy().view("<f4")                       # [nb, 1]
    want = (scale * blocks[:, 4:].view(np.int8).astype(np.float32)).astype(np.float32)
    got = oracle.dequantize(MM_Q8_0, blocks.ravel(), nb * 32).reshape(nb, 32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def mm_q4_k_numpy(blocks):
    nb = blocks.shape[0]
    scale = mm_f16_numpy(blocks[:, 0:16].copy().view("<u2"))        # [nb, 8]
    mn = blocks[:, 16:24].view(np.int8).astype(np.float32)          # [nb, 8]
    out = np.empty((nb, 8, 32), np.float32)
    for sb in range(8):
        nib = blocks[:, 32 + 20 * sb: 32 + 20 * sb + 16]
        q = np.empty((nb, 32), np.float32)
        q[:, 0::2] = nib & 15
        q[:, 1::2] = nib >> 4
        prod = (q * scale[:, sb:sb + 1]).astype(np.float32)
        out[:, sb, :] = (mn[:, sb:sb + 1] + prod).astype(np.float32)
    return out.reshape(nb, 256)


def test_mm_q4_k_numpy_statement(oracle):
    rng = np.random.default_rng(12)
    nb = 200
    blocks = Q.random_blocks(MM_Q4_K, nb, rng).reshape(nb, 256).copy()
    blocks[0:40, 0:16] = rng.integers(0, 256, (40, 16), dtype=np.uint8)   # any scale pattern, zero and inf fields too
    blocks[0, 0:2] = 0
    got = oracle.dequantize(MM_Q4_K, blocks.ravel(), nb * 256).reshape(nb, 256)
    want = mm_q4_k_numpy(blocks)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_mm_q4_k_agrees_with_the_canonical_decoder_where_it_must(oracle):
    # sub-block 0 reads bytes 32..47 under either stride; both widenings agree on normal scales with mantissa bits 3..9 clear
    rng = np.random.default_rng(13)
    nb = 64
    full = Q.synth_q4_k(nb, rng)
    blocks = full.reshape(nb, 256).copy()
    blocks[:, 0:16] = (blocks[:, 0:16].copy().view("<u2") & np.uint16(0xFC07)).view(np.uint8)
    blocks = blocks.ravel()
    # with the generator's own scales (all ten mantissa bits in use) even sub-block 0 differs
    assert not np.array_equal(oracle.dequantize(MM_Q4_K, full, nb * 256).reshape(nb, 8, 32)[:, 0],
                              oracle.dequantize(Q.Q4_K, full, nb * 256).reshape(nb, 8, 32)[:, 0])
    a = oracle.dequantize(MM_Q4_K, blocks, nb * 256).reshape(nb, 8, 32)
    b = oracle.dequantize(Q.Q4_K, blocks, nb * 256).reshape(nb, 8, 32)
    assert np.array_equal(a[:, 0].view(np.uint32), b[:, 0].view(np.uint32))
    assert not np.array_equal(a[:, 1], b[:, 1])                     # sub-block 1: bytes 52.. against 60..
    # and the stride: moving the canonical bytes of sub-block sb to 32 + 20 * sb reproduces the canonical values
    moved = blocks.reshape(nb, 256).copy()
    src = blocks.reshape(nb, 256)
    for sb in range(8):
        moved[:, 32 + 20 * sb: 32 + 20 * sb + 16] = src[:, 32 + 28 * sb: 32 + 28 * sb + 16]
    c = oracle.dequantize(MM_Q4_K, moved.ravel(), nb * 256).reshape(nb, 8, 32)
    assert np.array_equal(c.view(np.uint32), b.view(np.uint32))


def test_mm_q6_k_is_the_canonical_decoder_where_the_widenings_agree(oracle):
    rng = np.random.default_rng(14)
    w = (rng.standard_normal((8, 1024)) * 0.02).astype(np.float32)
    full = Q.quantize_q6_k(w, rng)
    nb = w.size // 256
    blocks = full.reshape(nb, 256).copy()
    blocks[:, 0:32] = (blocks[:, 0:32].copy().view("<u2") & np.uint16(0xFC07)).view(np.uint8)
    blocks = blocks.ravel()
    a = oracle.dequantize(MM_Q6_K, blocks, w.size)
    b = oracle.dequantize(Q.Q6_K, blocks, w.size)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # a real quantiser's scales use every mantissa bit: there this decoder returns other numbers
    a, b = oracle.dequantize(MM_Q6_K, full, w.size), oracle.dequantize(Q.Q6_K, full, w.size)
    assert not np.array_equal(a, b)
    scale = mm_f16_numpy(full.reshape(nb, 256)[:, 0:32].copy().view("<u2"))          # [nb, 16]
    codes = np.where(b.reshape(nb, 16, 16) != 0, 1, 0)                                # same zero pattern: the codes are shared
    assert np.array_equal(np.where(a.reshape(nb, 16, 16) != 0, 1, 0), codes)
    ieee = full.reshape(nb, 256)[:, 0:32].copy().view("<f2").astype(np.float32)
    ratio = (scale / ieee)[:, :, None]                                                # this widening never exceeds IEEE's
    assert np.all(ratio <= 1.0) and np.all(ratio > 0.5)
    assert np.allclose(a.reshape(nb, 16, 16), b.reshape(nb, 16, 16) * ratio, rtol=1e-6, atol=0)
    # a subnormal scale: the canonical decoder widens 0x0201 to 513 * 2^-24, this one reads 2^-15 * (1 + 1 / 1024)
    blk = full[:256].copy()
    blk[0:2] = np.array([0x0201], "<u2").view(np.uint8)
    a, b = oracle.dequantize(MM_Q6_K, blk, 256), oracle.dequantize(Q.Q6_K, blk, 256)
    nz = b[:16] != 0
    assert nz.any()
    q = (b[:16] / np.float32(513 * 2.0 ** -24)).astype(np.float32)                    # the signed codes
    assert np.array_equal(a[:16], (q * np.float32(2.0 ** -15 * (1 + 1 / 1024))).astype(np.float32))


# The loops of the three decoders, element by element, with the Rust's early exits.
def rust_loop(fmt, data, n):
    data = bytes(data)
    out = [0.0] * n
    f32 = lambda o: struct.unpack("<f", data[o:o + 4])[0]
    f16 = lambda o: float(mm_f16_numpy(np.array([data[o] | (data[o + 1] << 8)], np.uint16))[0])
    if fmt == MM_Q8_0:
        for b in range((n + 31) // 32):
            off = b * 36
            if off + 4 > len(data):
                break
            for i in range(32):
                if off + 4 + i >= len(data):
                    break
                if b * 32 + i < n:
                    v = data[off + 4 + i]
                    out[b * 32 + i] = np.float32(f32(off)) * np.float32(v - 256 if v > 127 else v)
    elif fmt == MM_Q4_K:
        for s in range((n + 255) // 256):
            so = s * 256
            if so + 32 > len(data):
                break
            for sb in range(8):
                scale = np.float32(f16(so + 2 * sb))
                m = data[so + 16 + sb]
                mn = np.float32(m - 256 if m > 127 else m)
                for i in range(32):
                    e = s * 256 + sb * 32 + i
                    if e >= n:
                        break
                    qi = so + 32 + sb * 20 + i // 2
                    if qi + 1 >= len(data):
                        break
                    q = (data[qi] >> 4) if i & 1 else (data[qi] & 15)
                    out[e] = mn + np.float32(q) * scale
    else:
        for b in range((n + 255) // 256):
            bo = b * 256
            if bo + 32 > len(data):
                break
            for i in range(256):
                e = b * 256 + i
                if e >= n:
                    break
                scale = np.float32(f16(bo + 2 * (i // 16)))
                qi = bo + 32 + (i * 6) // 8
                if qi + 1 >= len(data):
                    break
                q = ((data[qi] | (data[qi + 1] << 8)) >> ((i * 6) % 8)) & 63
                out[e] = np.float32(q - 64 if q >= 32 else q) * scale
    return np.array(out, dtype=np.float32)


@pytest.mark.parametrize("fmt", [MM_Q8_0, MM_Q4_K, MM_Q6_K])
def test_mm_short_and_ragged_inputs(fmt, oracle):
    rng = np.random.default_rng(15 + fmt)
    be, bb = Q.BLOCK_ELEMS[fmt], Q.BLOCK_BYTES[fmt]
    blocks = Q.random_blocks(fmt, 3, rng)
    for n, length in [(3 * be, 3 * bb), (2 * be + 7, 3 * bb), (3 * be, 2 * bb + bb // 2), (3 * be, 2 * bb + 33),
                      (3 * be, 2 * bb + 3), (be, 5), (2 * be, bb + 34), (10, bb), (0, 0)]:
        got = oracle.dequantize(fmt, blocks[:length], n)
        want = rust_loop(fmt, blocks[:length], n)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (fmt, n, length)


def test_kn_recipe_of_the_reference_gpu_test(oracle):
    # quantized/q4_0.rs:343-435: m = 2, n = 4, k = 8; activations i * 0.1; one Q4_0 block, scale 1.0,
    # byte i = (i % 16) << 4 | (i % 16).  Wd is the flat decode read as [k, n].
    m, n, k = 2, 4, 8
    a = (np.arange(m * k, dtype=np.float32) * np.float32(0.1)).reshape(m, k)
    w = np.zeros(20, np.uint8)
    w[0:4] = f32le(1.0)
    for i in range(16):
        w[4 + i] = ((i % 16) << 4) | (i % 16)
    got = oracle.qmatmul_kn(Q.Q4_0, w, a, m, n, k)
    wd = np.repeat(np.arange(16) - 8, 2).astype(np.float64)            # element 2i and 2i+1 = i - 8
    want = a.astype(np.float64) @ wd.reshape(k, n)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    # not the row-major [n, k] product
    assert not np.allclose(got, a.astype(np.float64) @ wd.reshape(n, k).T, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("fmt", [Q.Q4_0, MM_Q8_0, MM_Q4_K, MM_Q6_K, Q.Q4_K, Q.MXFP4])
def test_kn_is_the_f32_matmul_over_the_flat_decode(fmt, oracle):
    rng = np.random.default_rng(16 + fmt)
    m, n, k = 3, 96, 64                                                # n * k = 6144 elements: whole blocks
    w = Q.random_blocks(fmt, n * k // Q.BLOCK_ELEMS[fmt], rng)
    a = rng.standard_normal((m, k)).astype(np.float32)
    got = oracle.qmatmul_kn(fmt, w, a, m, n, k)
    wd = oracle.dequantize(fmt, w, n * k)
    want = oracle.cpu_matmul_f32(a, wd, m, n, k)                       # cpu_matmul_f32 with b[l * n + j]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref64 = a.astype(np.float64) @ wd.astype(np.float64).reshape(k, n)
    assert np.max(np.abs(got - ref64)) <= 1e-5 * np.max(np.abs(ref64)) + 1e-6
