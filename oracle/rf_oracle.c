/*
 * rf_oracle.c -- CPU restatement of ROCmForge's quantized dequant / matmul path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists only so that the
 * HIP kernels can be checked against the arithmetic the reference performs on
 * the CPU.  Only tests, the smoke check and the bench's cpu_baseline leg may
 * link or call it; nothing in the shipped library does.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the ROCmForge tree).  The reference is Rust; there is no Rust toolchain to
 * build it here, so each function is pinned by the reference's own unit-test
 * vectors and by independent closed-form / brute-force checks in tests/.
 *
 * Parity status per function:
 *   pinned   : rf_dequant_q4_0, rf_dequant_q8_0, rf_dequant_q4_k,
 *              rf_dequant_q6_k, rf_dequant_q2_k, rf_dequant_q3_k, rf_dequant_q5_k, rf_dequant_mxfp4, rf_dequant_mxfp6,
 *              rf_decode_e2m1, rf_decode_e2m3, rf_encode_e2m1, rf_encode_e2m3,
 *              rf_pack_6bit, rf_unpack_6bit, rf_pack_mxfp4, rf_pack_mxfp6,
 *              rf_unpack_mxfp4, rf_unpack_mxfp6, rf_cpu_matmul_f32,
 *              rf_f16_to_f32, rf_data_size, rf_rms_norm, rf_swiglu (the
 *              reference's test properties and an independent float64
 *              evaluation), rf_dequant_rms_norm, rf_mlp_swiglu_q (compositions
 *              of pinned parts, checked against float64)
 *   pinned   : rf_dequant_mm_q8_0 (the reference's vector at
 *              src/kernels/matmul/quantized/q8_0.rs:113-131 and an independent
 *              numpy statement), rf_dequant_mm_q4_k, rf_dequant_mm_q6_k
 *              (independent whole-array numpy statements on random blocks; the
 *              canonical decoders on the inputs where the two must agree),
 *              rf_f16_to_f32_mm for all 65 536 patterns (an independent
 *              statement in 16-bit numpy integers of the shift the reference
 *              performs in u16, and hand values), rf_qmatmul_kn
 *              (rf_cpu_matmul_f32 on the flat dequantised stream; the recipe of
 *              quantized/q4_0.rs:343-435)
 *   parity unpinned (no reference vector; follows from reading the code):
 *              that the `exp <= 0` branch of f16_to_f32_cpu is dead (exponent
 *              fields 0 and 31 of rf_f16_to_f32_mm take the same closed form as
 *              every other field)
 *   parity unpinned (no counterpart in the reference; public ggml layouts):
 *              rf_dequant_gguf_q4_0 / q8_0 / q4_k / q6_k
 *   parity unpinned (no reference vector, reasoned from compiler-rt source):
 *              rf_powi_f32 for exponent -128 only (returns 0.0), hence the
 *              MXFP scale byte 0x80; rf_e8m0_from_f32 when log2 lands on an
 *              exact .5 tie (affects generated inputs only, never compute).
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC
 * (no FMA contraction: Rust never fuses a*b+c).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define RF_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* scalar helpers                                                      */
/* ------------------------------------------------------------------ */

/* IEEE binary16 -> binary32 widening, exact (subnormals, inf, nan kept).
 * Stands for half::f16::from_bits(b).to_f32() (crate half 2.7.1) used at
 * src/kernels/quant/q4_k.rs:236 and q6_k.rs:236. */
RF_API float rf_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* f32::powi lowers to llvm.powi.f32 -> compiler-rt __powisf2: repeated
 * squaring on |b|, reciprocal at the end for negative b.  Used by
 * E8M0::to_f32 (src/loader/mxfp.rs:23-25) and decode_e2m1/e2m3
 * (mxfp.rs:243,292).  For b = -128 the squaring overflows to +inf and the
 * reciprocal gives 0.0. */
RF_API float rf_powi_f32(float a, int b)
{
    const int recip = b < 0;
    float r = 1.0f;
    for (;;) {
        if (b & 1) r *= a;
        b /= 2;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0f / r : r;
}

static float clampf(float v, float lo, float hi)
{
    /* f32::clamp: if v < lo -> lo; if v > hi -> hi; else v (NaN stays) */
    if (v < lo) return lo;
    if (v > hi) return hi;
    return v;
}

/* src/loader/mxfp.rs:234-244 */
RF_API float rf_decode_e2m1(uint8_t bits)
{
    if (bits == 0) return 0.0f;
    float sign = (bits & 0x08) ? -1.0f : 1.0f;
    int exp = (int)((bits >> 1) & 0x03) - 1;
    float mant = (float)(bits & 0x01);
    return sign * (1.0f + mant) * rf_powi_f32(2.0f, exp);
}

/* src/loader/mxfp.rs:283-293 */
RF_API float rf_decode_e2m3(uint8_t bits)
{
    if (bits == 0) return 0.0f;
    float sign = (bits & 0x20) ? -1.0f : 1.0f;
    int exp = (int)((bits >> 3) & 0x03) - 1;
    float mant = (float)(bits & 0x07) / 8.0f;
    return sign * (1.0f + mant) * rf_powi_f32(2.0f, exp);
}

/* src/loader/mxfp.rs:200-231 */
RF_API uint8_t rf_encode_e2m1(float value)
{
    if (value == 0.0f) return 0;
    uint8_t sign = (value < 0.0f) ? 0x08 : 0x00;
    float a = fabsf(value);
    float clamped = fminf(fmaxf(a, 0.5f), 8.0f);
    uint8_t best = 0;
    float best_err = 3.40282347e+38f;
    for (int e = 0; e < 4; e++) {
        for (int m = 0; m < 2; m++) {
            float decoded = (1.0f + (float)m) * rf_powi_f32(2.0f, e - 1);
            float err = fabsf(clamped - decoded);
            if (err < best_err) {
                best_err = err;
                best = (uint8_t)((e << 1) | m);
            }
        }
    }
    return sign | best;
}

/* src/loader/mxfp.rs:249-280 */
RF_API uint8_t rf_encode_e2m3(float value)
{
    if (value == 0.0f) return 0;
    uint8_t sign = (value < 0.0f) ? 0x20 : 0x00;
    float a = fabsf(value);
    float clamped = fminf(fmaxf(a, 0.5f), 7.5f);
    uint8_t best = 0;
    float best_err = 3.40282347e+38f;
    for (int e = 0; e < 4; e++) {
        for (int m = 0; m < 8; m++) {
            float mant = (float)m / 8.0f;
            float decoded = (1.0f + mant) * rf_powi_f32(2.0f, e - 1);
            float err = fabsf(clamped - decoded);
            if (err < best_err) {
                best_err = err;
                best = (uint8_t)((e << 3) | m);
            }
        }
    }
    return sign | best;
}

/* E8M0::from_f32, src/loader/mxfp.rs:29-43.  Returns the signed exponent. */
RF_API int8_t rf_e8m0_from_f32(float value)
{
    if (value == 0.0f || isnan(value)) return 0;
    if (isinf(value)) return 127;
    float l = log2f(fabsf(value));
    l = clampf(l, -127.0f, 127.0f);
    return (int8_t)roundf(l); /* f32::round = half away from zero */
}

/* E8M0::to_f32, src/loader/mxfp.rs:23-25 */
RF_API float rf_e8m0_to_f32(int8_t e) { return rf_powi_f32(2.0f, (int)e); }

/* src/loader/mxfp.rs:297-320 (LSB-first bit stream) */
RF_API void rf_pack_6bit(const uint8_t *values, size_t count, uint8_t *packed /* ceil(count*6/8), pre-zeroed by us */)
{
    size_t nbytes = (count * 6 + 7) / 8;
    memset(packed, 0, nbytes);
    for (size_t i = 0; i < count; i++) {
        size_t bit_pos = i * 6;
        size_t byte_idx = bit_pos / 8;
        unsigned bit_offset = (unsigned)(bit_pos % 8);
        uint8_t v = values[i] & 0x3F;
        if (bit_offset <= 2) {
            packed[byte_idx] |= (uint8_t)(v << bit_offset);
        } else {
            unsigned first = 8 - bit_offset;
            packed[byte_idx] |= (uint8_t)(v << bit_offset);
            packed[byte_idx + 1] |= (uint8_t)(v >> first);
        }
    }
}

/* src/loader/mxfp.rs:324-353 */
RF_API void rf_unpack_6bit(const uint8_t *packed, size_t packed_len, size_t count, uint8_t *values)
{
    for (size_t i = 0; i < count; i++) {
        size_t bit_pos = i * 6;
        size_t byte_idx = bit_pos / 8;
        unsigned bit_offset = (unsigned)(bit_pos % 8);
        values[i] = 0;
        if (byte_idx < packed_len) {
            if (bit_offset <= 2) {
                values[i] = (packed[byte_idx] >> bit_offset) & 0x3F;
            } else {
                unsigned first = 8 - bit_offset;
                unsigned second = 6 - first;
                uint8_t p1 = (packed[byte_idx] >> bit_offset) & (uint8_t)((1u << first) - 1);
                uint8_t p2 = (byte_idx + 1 < packed_len)
                                 ? (packed[byte_idx + 1] & (uint8_t)((1u << second) - 1))
                                 : 0;
                values[i] = p1 | (uint8_t)(p2 << first);
            }
        }
    }
}

static float block_absmax(const float *v, size_t n)
{
    float m = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float a = fabsf(v[i]);
        /* f32::max ignores a NaN operand */
        if (a > m || isnan(m)) m = a;
    }
    return m;
}

/* MxfpBlock::pack_mxfp4, src/loader/mxfp.rs:77-117.  values: up to 32 floats
 * (n_values <= 32); out: 17 bytes = exponent byte + 16 nibble bytes, element
 * 2j in the HIGH nibble of byte j. */
RF_API void rf_pack_mxfp4(const float *values, size_t n_values, uint8_t *out17)
{
    float max_val = block_absmax(values, n_values);
    int8_t e = (max_val == 0.0f) ? 0 : rf_e8m0_from_f32(max_val);
    float scale = rf_e8m0_to_f32(e);
    memset(out17, 0, 17);
    out17[0] = (uint8_t)e;
    size_t n = n_values < 32 ? n_values : 32;
    for (size_t i = 0; i < n; i++) {
        float normalized = (scale > 0.0f) ? values[i] / scale : values[i];
        uint8_t enc = rf_encode_e2m1(normalized);
        if ((i & 1) == 0) out17[1 + i / 2] |= (uint8_t)(enc << 4);
        else out17[1 + i / 2] |= (uint8_t)(enc & 0x0F);
    }
}

/* MxfpBlock::pack_mxfp6, src/loader/mxfp.rs:142-174. out: 25 bytes. */
RF_API void rf_pack_mxfp6(const float *values, size_t n_values, uint8_t *out25)
{
    float max_val = block_absmax(values, n_values);
    int8_t e = (max_val == 0.0f) ? 0 : rf_e8m0_from_f32(max_val);
    float scale = rf_e8m0_to_f32(e);
    uint8_t codes[32];
    size_t n = n_values < 32 ? n_values : 32;
    for (size_t i = 0; i < n; i++) {
        float normalized = (scale > 0.0f) ? values[i] / scale : values[i];
        codes[i] = rf_encode_e2m3(normalized);
    }
    memset(out25, 0, 25);
    out25[0] = (uint8_t)e;
    rf_pack_6bit(codes, n, out25 + 1);
}

/* MxfpBlock::unpack_mxfp4, src/loader/mxfp.rs:120-139 */
RF_API void rf_unpack_mxfp4(const uint8_t *blk17, float *out32)
{
    float scale = rf_e8m0_to_f32((int8_t)blk17[0]);
    for (int i = 0; i < 32; i++) {
        uint8_t b = blk17[1 + i / 2];
        uint8_t nib = (i % 2 == 0) ? ((b >> 4) & 0x0F) : (b & 0x0F);
        out32[i] = clampf(scale * rf_decode_e2m1(nib), -8.0f, 8.0f);
    }
}

/* MxfpBlock::unpack_mxfp6, src/loader/mxfp.rs:177-190 (LSB-first unpack; note
 * this is NOT the extraction the loader's dequant_mxfp6 uses). */
RF_API void rf_unpack_mxfp6(const uint8_t *blk25, float *out32)
{
    uint8_t codes[32];
    rf_unpack_6bit(blk25 + 1, 24, 32, codes);
    float scale = rf_e8m0_to_f32((int8_t)blk25[0]);
    for (int i = 0; i < 32; i++)
        out32[i] = clampf(scale * rf_decode_e2m3(codes[i]), -7.5f, 7.5f);
}

/* ------------------------------------------------------------------ */
/* canonical dequantisers (what rocmforge::loader::dequant_* resolve to) */
/* ------------------------------------------------------------------ */

static float rd_f32le(const uint8_t *p)
{
    uint32_t u = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* dequantize_q4_0_cpu, src/kernels/quant/q4_0.rs:266-310 */
RF_API void rf_dequant_q4_0(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t n_blocks = (n + 31) / 32;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        size_t off = b * 20;
        if (off + 4 > len) break;
        float scale = rd_f32le(data + off);
        size_t ds = off + 4, base = b * 32;
        for (size_t i = 0; i < 16; i++) {
            if (ds + i >= len) break;
            uint8_t packed = data[ds + i];
            int low = (int)(packed & 0x0F) - 8;
            if (base + i * 2 < n) out[base + i * 2] = scale * (float)low;
            int high = (int)((packed >> 4) & 0x0F) - 8;
            if (base + i * 2 + 1 < n) out[base + i * 2 + 1] = scale * (float)high;
        }
    }
}

/* dequantize_q8_0, src/kernels/quant/q8_0.rs:23-71 (block order is
 * irrelevant: every block writes a disjoint slice) */
RF_API void rf_dequant_q8_0(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t blocks = (n + 31) / 32;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        size_t start = b * 36;
        if (start + 4 > len) continue;
        float scale = rd_f32le(data + start);
        size_t qs = start + 4;
        size_t qe = qs + 32 < len ? qs + 32 : len;
        for (size_t i = 0; qs + i < qe; i++) {
            size_t idx = b * 32 + i;
            if (idx < n) out[idx] = ((float)data[qs + i] - 128.0f) * scale;
        }
    }
}

/* dequantize_q4_k_cpu, src/kernels/quant/q4_k.rs:201-273 */
RF_API void rf_dequant_q4_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t nsb = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t s = 0; s < nsb; s++) {
        size_t so = s * 256;
        if (so + 256 > len) break;
        size_t scales_start = so, mins_start = so + 16, quants_start = so + 32;
        for (size_t sub = 0; sub < 8; sub++) {
            size_t sub_start = s * 256 + sub * 32;
            if (sub_start >= n) break;
            size_t sc_off = scales_start + sub * 2;
            float scale = 1.0f;
            if (sc_off + 2 <= len)
                scale = rf_f16_to_f32((uint16_t)(data[sc_off] | (data[sc_off + 1] << 8)));
            size_t mn_off = mins_start + sub;
            float mn = 0.0f;
            if (mn_off < len) mn = (float)(int8_t)data[mn_off];
            for (size_t i = 0; i < 32; i++) {
                size_t idx = sub_start + i;
                if (idx >= n) break;
                size_t bit_pos = i * 4;
                size_t byte_idx = bit_pos / 8;
                unsigned bit_offset = (unsigned)(bit_pos % 8);
                size_t qo = quants_start + sub * 28 + byte_idx;
                if (qo + 1 < len) {
                    uint16_t combined = (uint16_t)(((uint16_t)data[qo + 1] << 8) | data[qo]);
                    uint8_t q = (uint8_t)((combined >> bit_offset) & 0x0F);
                    out[idx] = mn + (float)q * scale;
                }
            }
        }
    }
}

/* dequantize_q6_k_cpu, src/kernels/quant/q6_k.rs:201-266 */
RF_API void rf_dequant_q6_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t nb = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        size_t bs = b * 256;
        if (bs + 256 > len) break;
        size_t scales_start = bs, quants_start = bs + 32;
        for (size_t i = 0; i < 256; i++) {
            size_t idx = b * 256 + i;
            if (idx >= n) break;
            size_t sc_off = scales_start + (i / 16) * 2;
            float scale = 1.0f;
            if (sc_off + 2 <= len)
                scale = rf_f16_to_f32((uint16_t)(data[sc_off] | (data[sc_off + 1] << 8)));
            unsigned bit_offset = (unsigned)((i * 6) % 8);
            size_t byte_idx = (i * 6) / 8;
            if (quants_start + byte_idx + 1 < len) {
                uint16_t combined = (uint16_t)(((uint16_t)data[quants_start + byte_idx + 1] << 8) |
                                               data[quants_start + byte_idx]);
                uint8_t q = (uint8_t)((combined >> bit_offset) & 0x3F);
                float sv = (q >= 32) ? (float)(int8_t)((int8_t)q - 64) : (float)q;
                out[idx] = sv * scale;
            }
        }
    }
}

/* dequant_mxfp4, src/loader/dequant.rs:41-82 */
RF_API void rf_dequant_mxfp4(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t blocks = (n + 31) / 32;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        size_t bs = b * 17;
        if (bs + 1 > len) break;
        float scale = rf_powi_f32(2.0f, (int)(int8_t)data[bs]);
        size_t ds = bs + 1;
        size_t de = ds + 16 < len ? ds + 16 : len;
        for (size_t bo = 0; ds + bo < de; bo++) {
            uint8_t packed = data[ds + bo];
            for (int j = 0; j < 2; j++) {
                size_t idx = b * 32 + bo * 2 + (size_t)j;
                if (idx < n) {
                    uint8_t bits = (j == 0) ? ((packed >> 4) & 0x0F) : (packed & 0x0F);
                    float val = scale * rf_decode_e2m1(bits);
                    out[idx] = clampf(val, -8.0f, 8.0f);
                }
            }
        }
    }
}

/* dequant_mxfp6, src/loader/dequant.rs:85-132.  Used for both Mxfp6E2m3 and
 * Mxfp6E3m2 (dequant.rs:693).  Note the ">> (10 - bit_offset)" extraction and
 * that element 31 of a block is never written. */
RF_API void rf_dequant_mxfp6(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t blocks = (n + 31) / 32;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        size_t bs = b * 25;
        if (bs + 1 > len) break;
        float scale = rf_powi_f32(2.0f, (int)(int8_t)data[bs]);
        size_t ds = bs + 1;
        size_t de = ds + 24 < len ? ds + 24 : len;
        const uint8_t *pd = data + ds;
        size_t plen = de - ds;
        for (size_t i = 0; i < 32; i++) {
            size_t idx = b * 32 + i;
            if (idx >= n) break;
            unsigned bit_offset = (unsigned)((i * 6) % 8);
            size_t byte_idx = (i * 6) / 8;
            if (byte_idx + 1 < plen) {
                uint16_t combined = (uint16_t)(((uint16_t)pd[byte_idx + 1] << 8) | pd[byte_idx]);
                uint8_t bits = (uint8_t)((combined >> (10 - bit_offset)) & 0x3F);
                float val = scale * rf_decode_e2m3(bits);
                out[idx] = clampf(val, -7.5f, 7.5f);
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* the matmul module's own decoders (src/kernels/matmul/quantized/):    */
/* what matmul_q8_0 and the *_cpu_fallback paths really compute.  They   */
/* differ from the canonical decoders above in layout or arithmetic.     */
/* ------------------------------------------------------------------ */

/* f16_to_f32_cpu, src/kernels/matmul/quantized/common.rs:44-60, token by
 * token with Rust's integer widths.  Two things make it differ from IEEE
 * widening:
 *  - line 47 is `((bits & 0x03FF) << 13) as u32` with `bits: u16`: the shift
 *    happens in 16 bits (a shift count below the width never panics, the bits
 *    shifted out are dropped) and only then is the result widened, so mantissa
 *    bits 3..9 are lost and the mantissa term is `(bits & 7) << 13`;
 *  - `exp` already carries the f32 bias (field + 112 >= 112), so the
 *    `exp <= 0` branch meant for zero and subnormals is never taken.
 * Every pattern therefore decodes as sign | (field + 112) << 23 | (bits & 7) << 13
 * = +-2^(field - 15) * (1 + (bits & 7) / 1024): 0x3E00 (1.5) reads 1.0, 0x2E66
 * (0.1) reads 0.062866..., 0x0000 reads 2^-15.  Only patterns whose mantissa
 * bits 3..9 are zero (powers of two among them: 0x3C00 -> 1.0, 0x4000 -> 2.0)
 * come out as IEEE.  The branch is kept as written. */
RF_API float rf_f16_to_f32_mm(uint16_t bits)
{
    uint32_t sign = (bits & 0x8000u) != 0 ? (1u << 31) : 0u;
    int32_t exp = (int32_t)((bits & 0x7C00u) >> 10) - 15 + 127;
    uint16_t mant16 = (uint16_t)((bits & 0x03FFu) << 13);   /* u16 << 13: Rust shifts before `as u32` */
    uint32_t mant = (uint32_t)mant16;
    uint32_t out;
    if (exp <= 0) {
        if ((bits & 0x7FFFu) == 0) out = sign;
        else return 0.0f;
    } else {
        out = sign | ((uint32_t)exp << 23) | mant;
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

/* dequantize_q8_0, src/kernels/matmul/quantized/q8_0.rs:18-56: the bytes are
 * two's-complement int8, value = scale * (byte as i8). */
RF_API void rf_dequant_mm_q8_0(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t n_blocks = (n + 31) / 32;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        size_t off = b * 36;
        if (off + 4 > len) break;
        float scale = rd_f32le(data + off);
        size_t ds = off + 4, base = b * 32;
        for (size_t i = 0; i < 32; i++) {
            size_t idx = ds + i;
            if (idx >= len) break;
            size_t e = base + i;
            if (e < n) out[e] = scale * (float)(int8_t)data[idx];
        }
    }
}

/* dequantize_q4_k, src/kernels/matmul/quantized/q4_k.rs:90-148: the nibbles of
 * sub-block sb start at 32 + 20 * sb (the canonical decoder strides 28), the
 * scale goes through rf_f16_to_f32_mm, a super-block needs only its first 32
 * bytes to be present. */
RF_API void rf_dequant_mm_q4_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t nsb = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t s = 0; s < nsb; s++) {
        size_t so = s * 256;
        if (so + 32 > len) break;
        for (size_t sub = 0; sub < 8; sub++) {
            size_t base = s * 256 + sub * 32;
            size_t sc_off = so + sub * 2;
            if (sc_off + 2 > len) break;
            float scale = rf_f16_to_f32_mm((uint16_t)(data[sc_off] | (data[sc_off + 1] << 8)));
            size_t mn_off = so + 16 + sub;
            if (mn_off >= len) break;
            float mn = (float)(int8_t)data[mn_off];
            size_t qb = so + 32 + sub * 20;
            for (size_t i = 0; i < 32; i++) {
                size_t e = base + i;
                if (e >= n) break;
                size_t bit_pos = i * 4, byte_idx = bit_pos / 8;
                unsigned bit_offset = (unsigned)(bit_pos % 8);
                size_t qi = qb + byte_idx;
                if (qi + 1 >= len) break;
                uint16_t combined = (uint16_t)(((uint16_t)data[qi + 1] << 8) | data[qi]);
                float quant = (float)((combined >> bit_offset) & 0x0F);
                out[e] = mn + (quant * scale);
            }
        }
    }
}

/* dequantize_q6_k, src/kernels/matmul/quantized/q6_k.rs:90-148: the canonical
 * bit stream, but the scale goes through rf_f16_to_f32_mm and a block needs
 * only its first 32 bytes to be present. */
RF_API void rf_dequant_mm_q6_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t nb = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        size_t bo = b * 256;
        if (bo + 32 > len) break;
        for (size_t i = 0; i < 256; i++) {
            size_t e = b * 256 + i;
            if (e >= n) break;
            size_t sc_off = bo + (i / 16) * 2;
            if (sc_off + 2 > len) break;
            float scale = rf_f16_to_f32_mm((uint16_t)(data[sc_off] | (data[sc_off + 1] << 8)));
            size_t bit_pos = i * 6, byte_idx = bit_pos / 8;
            unsigned bit_offset = (unsigned)(bit_pos % 8);
            size_t qi = bo + 32 + byte_idx;
            if (qi + 1 >= len) break;
            uint16_t combined = (uint16_t)(((uint16_t)data[qi + 1] << 8) | data[qi]);
            int quant = (int)((combined >> bit_offset) & 0x3F);
            int sv = quant >= 32 ? quant - 64 : quant;
            out[e] = (float)sv * scale;
        }
    }
}

/* ------------------------------------------------------------------ */
/* block layouts of GGUF model files (ggml)                            */
/* ------------------------------------------------------------------ */
/* PARITY UNPINNED against ROCmForge: nothing in the reference decodes these
 * layouts (its Q4_0 / Q8_0 / Q4_K / Q6_K are the 20 / 36 / 256-byte layouts
 * above).  They follow the public ggml definitions -- block_q4_0 {f16 d;
 * u8 qs[16]}, block_q8_0 {f16 d; i8 qs[32]}, block_q4_K {f16 d, dmin;
 * u8 scales[12]; u8 qs[128]}, block_q6_K {u8 ql[128]; u8 qh[64]; i8 scales[16];
 * f16 d} and dequantize_row_q4_0 / q8_0 / q4_K / q6_K of ggml-quants.c -- in
 * ggml's evaluation order, unfused.  They are pinned only by that published
 * arithmetic: an independent numpy statement, hand-made blocks, and
 * quantise -> dequantise error bounds in tests/.  Whole blocks only: decoding
 * stops at the first block the input does not hold, the tail stays 0.0. */

static float rd_f16le(const uint8_t *p) { return rf_f16_to_f32((uint16_t)(p[0] | (p[1] << 8))); }

RF_API void rf_dequant_gguf_q4_0(const uint8_t *data, size_t len, size_t n, float *out)
{
    memset(out, 0, n * sizeof(float));
    for (size_t b = 0; b * 32 + 32 <= n && b * 18 + 18 <= len; b++) {
        const uint8_t *blk = data + b * 18;
        float d = rd_f16le(blk);
        for (int j = 0; j < 16; j++) {
            int x0 = (blk[2 + j] & 0x0F) - 8, x1 = (blk[2 + j] >> 4) - 8;
            out[b * 32 + j] = (float)x0 * d;
            out[b * 32 + j + 16] = (float)x1 * d;
        }
    }
}

RF_API void rf_dequant_gguf_q8_0(const uint8_t *data, size_t len, size_t n, float *out)
{
    memset(out, 0, n * sizeof(float));
    for (size_t b = 0; b * 32 + 32 <= n && b * 34 + 34 <= len; b++) {
        const uint8_t *blk = data + b * 34;
        float d = rd_f16le(blk);
        for (int j = 0; j < 32; j++) out[b * 32 + j] = (float)(int8_t)blk[2 + j] * d;
    }
}

/* get_scale_min_k4 of ggml-quants.c: 6-bit scale and min number j of 8, packed in 12 bytes */
static void gguf_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m)
{
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

RF_API void rf_dequant_gguf_q4_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    memset(out, 0, n * sizeof(float));
    for (size_t b = 0; b * 256 + 256 <= n && b * 144 + 144 <= len; b++) {
        const uint8_t *blk = data + b * 144;
        float d = rd_f16le(blk), dmin = rd_f16le(blk + 2);
        const uint8_t *scales = blk + 4, *q = blk + 16;
        float *y = out + b * 256;
        int is = 0;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc, m;
            gguf_scale_min_k4(is + 0, scales, &sc, &m);
            float d1 = d * (float)sc, m1 = dmin * (float)m;
            gguf_scale_min_k4(is + 1, scales, &sc, &m);
            float d2 = d * (float)sc, m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) *y++ = d1 * (float)(q[l] & 0x0F) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

RF_API void rf_dequant_gguf_q6_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    memset(out, 0, n * sizeof(float));
    for (size_t b = 0; b * 256 + 256 <= n && b * 210 + 210 <= len; b++) {
        const uint8_t *ql = data + b * 210, *qh = ql + 128;
        const int8_t *sc = (const int8_t *)(ql + 192);
        float d = rd_f16le(ql + 208);
        float *y = out + b * 256;
        for (int half = 0; half < 2; half++) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int8_t)((ql[l] & 0x0F) | (((qh[l] >> 0) & 3) << 4)) - 32;
                int q2 = (int8_t)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l] = d * (float)sc[is + 0] * (float)q1;
                y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
            y += 128; ql += 64; qh += 32; sc += 8;
        }
    }
}

/* The loader's other K-type decoders (src/loader/dequant.rs): ROCmForge's own 256-byte
 * layouts of 16 sub-blocks x 16 elements, f16 scale at 2 * sub.  A block the input
 * does not hold completely ends the loop; elements past n are not written. */
static inline uint32_t rd_u16le(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

/* dequant_q5_k, src/loader/dequant.rs:150-225: i8 min at 32 + sub, 5-bit codes LSB first
 * at 48 + 10 * sub, read through a 16-bit window; min + q * scale */
RF_API void rf_dequant_q5_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t blocks = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        size_t bs = b * 256;
        if (bs + 256 > len) break;
        for (size_t sub = 0; sub < 16; sub++) {
            float scale = rf_f16_to_f32((uint16_t)rd_u16le(data + bs + sub * 2));
            float mn = (float)(int8_t)data[bs + 32 + sub];
            for (size_t i = 0; i < 16; i++) {
                size_t idx = b * 256 + sub * 16 + i;
                if (idx >= n) break;
                size_t bit = i * 5, off = bs + 48 + sub * 10 + bit / 8;
                uint32_t q = 0;
                if (off + 2 <= len) q = (rd_u16le(data + off) >> (bit % 8)) & 31u;
                out[idx] = mn + (float)q * scale;
            }
        }
    }
}

/* dequant_q3_k, src/loader/dequant.rs:243-320: two high bits per sub-block at 32 + sub / 4
 * (shift 2 * (sub % 4)), 3-bit codes LSB first at 36 + 6 * sub; bit i of the pair is bit 3
 * of element i for i < 8 (so only elements 0 and 1 can carry one); (q - 4) * scale */
RF_API void rf_dequant_q3_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t blocks = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        size_t bs = b * 256;
        if (bs + 256 > len) break;
        for (size_t sub = 0; sub < 16; sub++) {
            float scale = rf_f16_to_f32((uint16_t)rd_u16le(data + bs + sub * 2));
            uint32_t qh = (data[bs + 32 + sub / 4] >> ((sub % 4) * 2)) & 3u;
            for (size_t i = 0; i < 16; i++) {
                size_t idx = b * 256 + sub * 16 + i;
                if (idx >= n) break;
                size_t bit = i * 3, off = bs + 36 + sub * 6 + bit / 8;
                float q = 0.0f;
                if (off + 1 < len) {
                    uint32_t low = (rd_u16le(data + off) >> (bit % 8)) & 7u;
                    uint32_t high = i < 8 ? (qh >> i) & 1u : 0u;
                    q = (float)(int8_t)(low | (high << 3)) - 4.0f;
                }
                out[idx] = q * scale;
            }
        }
    }
}

/* dequant_q2_k, src/loader/dequant.rs:326-420: f16 min at 32 + 2 * sub, one high bit per
 * sub-block at 64 + sub / 8 (shift sub % 8), 2-bit codes LSB first at 68 + 4 * sub; the
 * high bit is bit 2 of element 0 only; min + q * scale */
RF_API void rf_dequant_q2_k(const uint8_t *data, size_t len, size_t n, float *out)
{
    size_t blocks = (n + 255) / 256;
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        size_t bs = b * 256;
        if (bs + 256 > len) break;
        for (size_t sub = 0; sub < 16; sub++) {
            float scale = rf_f16_to_f32((uint16_t)rd_u16le(data + bs + sub * 2));
            float mn = rf_f16_to_f32((uint16_t)rd_u16le(data + bs + 32 + sub * 2));
            uint32_t qh = (data[bs + 64 + sub / 8] >> (sub % 8)) & 1u;
            for (size_t i = 0; i < 16; i++) {
                size_t idx = b * 256 + sub * 16 + i;
                if (idx >= n) break;
                size_t bit = i * 2, off = bs + 68 + sub * 4 + bit / 8;
                float q = 0.0f;
                if (off + 1 < len) {
                    uint32_t low = (rd_u16le(data + off) >> (bit % 8)) & 3u;
                    uint32_t high = i < 8 ? (qh >> i) & 1u : 0u;
                    q = (float)(int8_t)(low | (high << 2));
                }
                out[idx] = mn + q * scale;
            }
        }
    }
}

/* GgufTensorType ids, src/loader/tensor_type.rs:16-32 */
enum { RF_F32 = 0, RF_F16 = 1, RF_Q4_0 = 2, RF_Q8_0 = 8, RF_Q2_K = 10, RF_Q3_K = 11, RF_Q4_K = 12, RF_Q5_K = 13, RF_Q6_K = 14,
       RF_MXFP4 = 20, RF_MXFP6_E2M3 = 21, RF_MXFP6_E3M2 = 22,
       /* GGUF file layouts: 100 + the ggml type id */
       RF_GGUF_Q4_0 = 102, RF_GGUF_Q8_0 = 108, RF_GGUF_Q4_K = 112, RF_GGUF_Q6_K = 114,
       /* the matmul module's decoders: 200 + the id of the format they are a variant of */
       RF_MM_Q8_0 = 208, RF_MM_Q4_K = 212, RF_MM_Q6_K = 214 };

/* GgufTensor::data_size, src/loader/gguf_tensor.rs:41-75 (Q4_0 is sized
 * 36 bytes per block there although the decoder strides 20). */
RF_API size_t rf_data_size(int type, size_t n)
{
    switch (type) {
    case RF_F32: return n * 4;
    case RF_F16: return n * 2;
    case RF_Q4_0: return ((n + 31) / 32) * 36;
    case RF_Q8_0: return ((n + 31) / 32) * 36;
    case RF_Q2_K: case RF_Q3_K: case RF_Q4_K: case RF_Q5_K: case RF_Q6_K: return ((n + 255) / 256) * 256;
    case RF_MXFP4: return ((n + 31) / 32) * 17;
    case RF_MXFP6_E2M3: case RF_MXFP6_E3M2: return ((n + 31) / 32) * 25;
    default: return 0;
    }
}

/* Bytes per block that the DECODERS stride by (q4_0.rs:269, q8_0.rs:33,
 * q4_k.rs:206, q6_k.rs:206, dequant.rs:47,91). */
RF_API size_t rf_block_bytes(int type)
{
    switch (type) {
    case RF_Q4_0: return 20;
    case RF_Q8_0: return 36;
    case RF_Q2_K: case RF_Q3_K: case RF_Q4_K: case RF_Q5_K: case RF_Q6_K: return 256;
    case RF_MXFP4: return 17;
    case RF_MXFP6_E2M3: case RF_MXFP6_E3M2: return 25;
    case RF_GGUF_Q4_0: return 18;
    case RF_GGUF_Q8_0: return 34;
    case RF_GGUF_Q4_K: return 144;
    case RF_GGUF_Q6_K: return 210;
    case RF_MM_Q8_0: return 36;
    case RF_MM_Q4_K: case RF_MM_Q6_K: return 256;
    default: return 0;
    }
}

/* loader::dequantize dispatcher, src/loader/dequant.rs:673-700 (the formats
 * on this path).  Returns 0 on success, -1 for a type outside the path. */
RF_API int rf_dequantize(int type, const uint8_t *data, size_t len, size_t n, float *out)
{
    switch (type) {
    case RF_F32:
        for (size_t i = 0; i < n && i * 4 + 4 <= len; i++) out[i] = rd_f32le(data + 4 * i);
        return 0;
    case RF_F16:
        for (size_t i = 0; i < n && i * 2 + 2 <= len; i++)
            out[i] = rf_f16_to_f32((uint16_t)(data[2 * i] | (data[2 * i + 1] << 8)));
        return 0;
    case RF_Q4_0: rf_dequant_q4_0(data, len, n, out); return 0;
    case RF_Q8_0: rf_dequant_q8_0(data, len, n, out); return 0;
    case RF_Q4_K: rf_dequant_q4_k(data, len, n, out); return 0;
    case RF_Q6_K: rf_dequant_q6_k(data, len, n, out); return 0;
    case RF_Q2_K: rf_dequant_q2_k(data, len, n, out); return 0;
    case RF_Q3_K: rf_dequant_q3_k(data, len, n, out); return 0;
    case RF_Q5_K: rf_dequant_q5_k(data, len, n, out); return 0;
    case RF_MXFP4: rf_dequant_mxfp4(data, len, n, out); return 0;
    case RF_MXFP6_E2M3:
    case RF_MXFP6_E3M2: rf_dequant_mxfp6(data, len, n, out); return 0;
    case RF_GGUF_Q4_0: rf_dequant_gguf_q4_0(data, len, n, out); return 0;
    case RF_GGUF_Q8_0: rf_dequant_gguf_q8_0(data, len, n, out); return 0;
    case RF_GGUF_Q4_K: rf_dequant_gguf_q4_k(data, len, n, out); return 0;
    case RF_GGUF_Q6_K: rf_dequant_gguf_q6_k(data, len, n, out); return 0;
    case RF_MM_Q8_0: rf_dequant_mm_q8_0(data, len, n, out); return 0;
    case RF_MM_Q4_K: rf_dequant_mm_q4_k(data, len, n, out); return 0;
    case RF_MM_Q6_K: rf_dequant_mm_q6_k(data, len, n, out); return 0;
    default: return -1;
    }
}

/* ------------------------------------------------------------------ */
/* matmul                                                              */
/* ------------------------------------------------------------------ */

/* cpu_matmul_f32, src/tensor/matmul.rs:219-233: a[m,k] . b[k,n], each output
 * a sequential fp32 sum over l ascending, product rounded before the add. */
RF_API void rf_cpu_matmul_f32(const float *a, const float *b, size_t m, size_t n, size_t k, float *c)
{
    for (size_t i = 0; i < m; i++) {
        for (size_t j = 0; j < n; j++) {
            float sum = 0.0f;
            for (size_t l = 0; l < k; l++) sum += a[i * k + l] * b[l * n + j];
            c[i * n + j] = sum;
        }
    }
}

/* Same arithmetic with the weight matrix stored [n,k] (rows of K, the layout
 * matmul_q4_0's doc comment states, src/kernels/matmul/quantized/q4_0.rs:139-148):
 * c[i,j] = sum_{l ascending} a[i,l] * w[j,l].  Per-output summation order and
 * rounding are identical to rf_cpu_matmul_f32 on w transposed; rows of the
 * output are spread over OpenMP threads, which does not change any value. */
RF_API void rf_matmul_nk_f32(const float *a, const float *w, size_t m, size_t n, size_t k, float *c)
{
#pragma omp parallel for schedule(static)
    for (long j = 0; j < (long)n; j++) {
        const float *wr = w + (size_t)j * k;
        for (size_t i = 0; i < m; i++) {
            const float *ar = a + i * k;
            float sum = 0.0f;
            for (size_t l = 0; l < k; l++) sum += ar[l] * wr[l];
            c[i * n + (size_t)j] = sum;
        }
    }
}

/* Quantised matmul as the reference's CPU path composes it
 * (matmul_q4_0_cpu_fallback, src/kernels/matmul/quantized/q4_0.rs:274-311;
 * benches/matmul_bench.rs:360-365): dequantise every weight to f32, then the
 * naive matmul.  Weights [n,k] row-major, blocks along k, row r starting at
 * byte r * (k / block_elems) * block_bytes.  scratch_row: k floats per thread
 * are allocated internally.  rows_sel (optional): only these output columns
 * are computed (c is then [m, n_sel]); pass NULL for all. */
RF_API int rf_qmatmul_nk(int type, const uint8_t *w, size_t w_len, const float *a, size_t m, size_t n,
                         size_t k, const int64_t *rows_sel, size_t n_sel, float *c)
{
    size_t bb = rf_block_bytes(type);
    size_t be = (type == RF_Q4_K || type == RF_Q6_K || type == RF_GGUF_Q4_K || type == RF_GGUF_Q6_K || type == RF_MM_Q4_K ||
                 type == RF_MM_Q6_K) ? 256 : 32;
    if (bb == 0 || k % be != 0) return -1;
    size_t row_bytes = (k / be) * bb;
    if (w_len < row_bytes * n) return -2;
    size_t nout = rows_sel ? n_sel : n;
    int rc = 0;
#pragma omp parallel
    {
        float *wr = (float *)__builtin_malloc(k * sizeof(float));
#pragma omp for schedule(static)
        for (long jj = 0; jj < (long)nout; jj++) {
            size_t j = rows_sel ? (size_t)rows_sel[jj] : (size_t)jj;
            if (!wr || j >= n) { rc = -3; continue; }
            rf_dequantize(type, w + j * row_bytes, row_bytes, k, wr);
            for (size_t i = 0; i < m; i++) {
                const float *ar = a + i * k;
                float sum = 0.0f;
                for (size_t l = 0; l < k; l++) sum += ar[l] * wr[l];
                c[i * nout + (size_t)jj] = sum;
            }
        }
        __builtin_free(wr);
    }
    return rc;
}

/* Single-threaded twin of the above used for the timed CPU baseline: full
 * dequantise of the weight tensor into wd[n*k] (as dequantize_q4_0 does in
 * the reference), then rf_matmul_nk_f32 restricted to one thread by the
 * caller (omp_set_num_threads).  Kept separate so the baseline times exactly
 * the two reference stages. */
RF_API int rf_qmatmul_nk_staged(int type, const uint8_t *w, size_t w_len, const float *a, size_t m,
                                size_t n, size_t k, float *wd, float *c)
{
    int r = rf_dequantize(type, w, w_len, n * k, wd);
    if (r) return r;
    rf_matmul_nk_f32(a, wd, m, n, k, c);
    return 0;
}

/* What the reference's quantised matmuls compute on the bytes they are given
 * (matmul_q4_0_cpu_fallback, src/kernels/matmul/quantized/q4_0.rs:274-311, and
 * matmul_q8_0, q8_0.rs:69-106; the fused kernel indexes the same way,
 * kernels/q4_0_matmul.hip: weight_linear_idx = k_idx * n + col): the packed
 * stream is dequantised as ONE flat array of n * k elements, and that array is
 * handed to the f32 matmul as b[k, n] (cpu_matmul_f32, src/tensor/matmul.rs:219-233,
 * b[l * n + j]):  c[i, j] = sum_{l ascending} a[i, l] * Wd[l * n + j].
 * The blocks therefore run along j.  Each output is the same sequential fp32
 * sum as rf_cpu_matmul_f32 (the loops are reordered i-l-j for the cache; every
 * c[i, j] still adds its l terms in ascending order, product rounded first).
 * wd: n * k floats of scratch. */
RF_API int rf_qmatmul_kn(int type, const uint8_t *w, size_t w_len, const float *a, size_t m, size_t n, size_t k,
                         float *wd, float *c)
{
    int r = rf_dequantize(type, w, w_len, n * k, wd);
    if (r) return r;
    for (size_t i = 0; i < m; i++) {
        float *ci = c + i * n;
        for (size_t j = 0; j < n; j++) ci[j] = 0.0f;
        for (size_t l = 0; l < k; l++) {
            const float al = a[i * k + l];
            const float *row = wd + l * n;
            for (size_t j = 0; j < n; j++) ci[j] += al * row[j];
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* neighbours of the quantised matmul in a decode step                 */
/* ------------------------------------------------------------------ */

/* RMSNorm as the reference's CPU check states it
 * (rms_norm_cpu_reference, src/mlp/rms_norm_tests.rs:44-73; the GPU kernel
 * kernels/rms_norm.hip:40-84 multiplies by rsqrtf instead of dividing):
 * per row, sum of squares in ascending order, mean = sum / hidden,
 * rms = sqrt(mean + eps), out = (x / rms) * weight.  */
RF_API void rf_rms_norm(const float *x, const float *weight, size_t rows, size_t hidden, float eps, float *out)
{
    for (size_t r = 0; r < rows; r++) {
        const float *row = x + r * hidden;
        float sum_sq = 0.0f;
        for (size_t j = 0; j < hidden; j++) sum_sq += row[j] * row[j];
        float mean_sq = sum_sq / (float)hidden;
        float rms = sqrtf(mean_sq + eps);
        for (size_t j = 0; j < hidden; j++) out[r * hidden + j] = (row[j] / rms) * weight[j];
    }
}

/* SwiGLU as the reference defines it: the activation is applied to the UP
 * projection, out = gate * (up * (1 / (1 + exp(-up))))
 * (swiglu_cpu_reference, src/mlp/swiglu_tests.rs:43-66; kernels/swiglu.hip:40-62). */
RF_API void rf_swiglu(const float *gate, const float *up, size_t total, float *out)
{
    for (size_t i = 0; i < total; i++) {
        float u = up[i];
        float sigmoid_up = 1.0f / (1.0f + expf(-u));
        float swish_up = u * sigmoid_up;
        out[i] = gate[i] * swish_up;
    }
}

/* Dequantise rows of a packed [rows, hidden] tensor, then RMSNorm them: the
 * arithmetic of fused_q4_0_rmsnorm (src/ggml/hip_backend/ops/fused_ops.rs:149-160,
 * kernels/fused_dequant_rmsnorm.hip:87-163) composed from its two unfused
 * stages, for any format of the path.  */
RF_API int rf_dequant_rms_norm(int type, const uint8_t *packed, size_t len, const float *weight, size_t rows,
                               size_t hidden, float eps, float *out)
{
    float *tmp = (float *)__builtin_malloc(rows * hidden * sizeof(float));
    if (!tmp) return -3;
    int r = rf_dequantize(type, packed, len, rows * hidden, tmp);
    if (r == 0) rf_rms_norm(tmp, weight, rows, hidden, eps, out);
    __builtin_free(tmp);
    return r;
}

/* The SwiGLU MLP of HipBackend::mlp_swiglu (src/backend/hip_backend/backend.rs:1153-1278:
 * gate = x.Wg, up = x.Wu, h = swiglu(gate, up), out = h.Wd) with the three
 * matrices quantised and stored [outputs, k] as the quantised matmuls take
 * them (matmul_q4_0, src/kernels/matmul/quantized/q4_0.rs:139-148), each
 * product being dequantise + naive matmul as in rf_qmatmul_nk.  norm_weight
 * (optional) applies rf_rms_norm to x first, the step that precedes the MLP in
 * a decoder layer.  scratch: m * (hidden + 3 * inter) floats.  */
RF_API int rf_mlp_swiglu_q(int type_gu, const uint8_t *wg, const uint8_t *wu, size_t gu_len, int type_d,
                           const uint8_t *wd, size_t d_len, const float *x, const float *norm_weight, float eps,
                           size_t m, size_t hidden, size_t inter, float *scratch, float *out)
{
    float *xn = scratch, *g = xn + m * hidden, *u = g + m * inter, *h = u + m * inter;
    const float *xin = x;
    if (norm_weight) {
        rf_rms_norm(x, norm_weight, m, hidden, eps, xn);
        xin = xn;
    }
    int r = rf_qmatmul_nk(type_gu, wg, gu_len, xin, m, inter, hidden, NULL, 0, g);
    if (r) return r;
    r = rf_qmatmul_nk(type_gu, wu, gu_len, xin, m, inter, hidden, NULL, 0, u);
    if (r) return r;
    rf_swiglu(g, u, m * inter, h);
    return rf_qmatmul_nk(type_d, wd, d_len, h, m, hidden, inter, NULL, 0, out);
}
