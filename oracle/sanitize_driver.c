/*
 * sanitize_driver.c -- runs every function of rf_oracle.c under
 * -fsanitize=address,undefined (CPU only; `make -C oracle asan`).
 *
 * TEST INFRASTRUCTURE, like the oracle itself.  The restatement follows Rust
 * source whose integer widths (u8/u16 shifts, `as i8`, usize arithmetic) decide
 * results; this driver feeds each function heap buffers of exactly the stated
 * size -- whole, ragged and empty inputs, every scale pattern -- so that a read
 * or write past an end, a shift beyond a type's width or a signed overflow in
 * the restatement stops the run.  It prints one FNV-1a checksum over all
 * results; the same driver built without the sanitizers must print the same
 * number (tests/test_oracle_sanitized.py compares them).
 */
#include <stdio.h>
#include <stdlib.h>

#include "rf_oracle.c"

static uint64_t g_hash = 1469598103934665603ull;
static void mix(const void *p, size_t bytes)
{
    const uint8_t *b = (const uint8_t *)p;
    for (size_t i = 0; i < bytes; i++) {
        g_hash ^= b[i];
        g_hash *= 1099511628211ull;
    }
}

static uint64_t g_rng = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void)
{
    g_rng ^= g_rng << 13;
    g_rng ^= g_rng >> 7;
    g_rng ^= g_rng << 17;
    return (uint32_t)(g_rng >> 16);
}

/* exact-size heap copies: the sanitizer's red zones sit right behind them */
static uint8_t *bytes_exact(size_t n)
{
    uint8_t *p = (uint8_t *)malloc(n ? n : 1);
    if (!p) abort();
    for (size_t i = 0; i < n; i++) p[i] = (uint8_t)rnd();
    return p;
}

static float *floats_exact(size_t n, float scale)
{
    float *p = (float *)malloc((n ? n : 1) * sizeof(float));
    if (!p) abort();
    for (size_t i = 0; i < n; i++) p[i] = scale * ((float)(int32_t)(rnd() & 0xFFFF) - 32768.0f) / 8192.0f;
    return p;
}

static const int kTypes[] = {RF_F32, RF_F16, RF_Q4_0, RF_Q8_0, RF_Q2_K, RF_Q3_K, RF_Q4_K, RF_Q5_K, RF_Q6_K, RF_MXFP4,
                             RF_MXFP6_E2M3, RF_MXFP6_E3M2, RF_GGUF_Q4_0, RF_GGUF_Q8_0, RF_GGUF_Q4_K, RF_GGUF_Q6_K,
                             RF_MM_Q8_0, RF_MM_Q4_K, RF_MM_Q6_K};

static size_t block_elems(int t)
{
    switch (t) {
    case RF_F32: case RF_F16: return 1;
    case RF_Q4_0: case RF_Q8_0: case RF_MXFP4: case RF_MXFP6_E2M3: case RF_MXFP6_E3M2: case RF_GGUF_Q4_0:
    case RF_GGUF_Q8_0: case RF_MM_Q8_0: return 32;
    default: return 256;
    }
}

static size_t block_bytes_of(int t) { return t == RF_F32 ? 4 : t == RF_F16 ? 2 : rf_block_bytes(t); }

/* finite f32 scales in the formats that store one, so that checksums do not depend on NaN payloads */
static void tame_scales(int t, uint8_t *d, size_t len)
{
    if (t == RF_Q4_0 || t == RF_Q8_0 || t == RF_MM_Q8_0) {
        size_t bb = rf_block_bytes(t);
        for (size_t o = 0; o + 4 <= len; o += bb) {
            float s = ((float)(rnd() & 1023) - 512.0f) / 4096.0f;
            memcpy(d + o, &s, 4);
        }
    }
    if (t == RF_F32)
        for (size_t o = 0; o + 4 <= len; o += 4) {
            float s = (float)(int32_t)(rnd() & 0xFFFF) / 7.0f;
            memcpy(d + o, &s, 4);
        }
}

static void run_dequant(int t, size_t n, size_t len)
{
    uint8_t *d = bytes_exact(len);
    tame_scales(t, d, len);
    float *out = (float *)malloc((n ? n : 1) * sizeof(float));
    if (!out) abort();
    for (size_t i = 0; i < n; i++) out[i] = 0.0f; /* rf_dequantize leaves F32/F16 tails alone */
    if (rf_dequantize(t, d, len, n, out) != 0) abort();
    /* NaN payloads of f16 scales differ in nothing the checks read; hash them as one value */
    for (size_t i = 0; i < n; i++) {
        if (out[i] != out[i]) {
            uint32_t q = 0x7FC00000u;
            mix(&q, 4);
        } else {
            mix(&out[i], 4);
        }
    }
    free(out);
    free(d);
}

int main(void)
{
    /* scalar helpers over their whole domains */
    for (uint32_t b = 0; b < 65536; b++) {
        float a = rf_f16_to_f32((uint16_t)b), c = rf_f16_to_f32_mm((uint16_t)b);
        if (a == a) mix(&a, 4);
        mix(&c, 4);
    }
    for (int e = -128; e <= 127; e++) {
        float p = rf_powi_f32(2.0f, e), q = rf_e8m0_to_f32((int8_t)e);
        mix(&p, 4);
        mix(&q, 4);
    }
    for (int c = 0; c < 256; c++) {
        float a = rf_decode_e2m1((uint8_t)c), b = rf_decode_e2m3((uint8_t)c);
        mix(&a, 4);
        mix(&b, 4);
    }
    {
        const float probes[] = {0.0f, -0.0f, 1e-30f, 0.25f, 0.5f, 0.74f, 0.75f, 0.76f, 1.0f, 1.49f, 1.5f, 2.9f, 3.0f, 5.9f, 6.0f,
                                7.5f, 8.0f, 9.0f, 1e30f, -0.3f, -1.0f, -7.9f, -1e30f, 3.40282347e+38f, 1.17549435e-38f, 1e-45f};
        for (size_t i = 0; i < sizeof(probes) / sizeof(probes[0]); i++) {
            uint8_t a = rf_encode_e2m1(probes[i]), b = rf_encode_e2m3(probes[i]);
            int8_t e = rf_e8m0_from_f32(probes[i]);
            mix(&a, 1);
            mix(&b, 1);
            mix(&e, 1);
        }
        float inf = 1.0f / 0.0f, nan = inf - inf;
        int8_t e1 = rf_e8m0_from_f32(inf), e2 = rf_e8m0_from_f32(nan), e3 = rf_e8m0_from_f32(-inf);
        mix(&e1, 1);
        mix(&e2, 1);
        mix(&e3, 1);
    }
    /* 6-bit packer: every count up to 40 values, buffers of exactly ceil(6 n / 8) bytes */
    for (size_t n = 0; n <= 40; n++) {
        size_t nb = (n * 6 + 7) / 8;
        uint8_t *vals = bytes_exact(n), *packed = bytes_exact(nb), *back = bytes_exact(n);
        rf_pack_6bit(vals, n, packed);
        rf_unpack_6bit(packed, nb, n, back);
        for (size_t i = 0; i < n; i++)
            if (back[i] != (vals[i] & 0x3F)) abort();
        if (nb > 1) rf_unpack_6bit(packed, nb - 1, n, back); /* a short stream: the last values read zero bits */
        mix(packed, nb);
        mix(back, n);
        free(vals);
        free(packed);
        free(back);
    }
    /* MXFP block packers: 0..32 values, all-zero, huge and tiny blocks */
    for (int rep = 0; rep < 200; rep++) {
        size_t n = rep < 33 ? (size_t)rep : 32;
        float scale = rep % 5 == 0 ? 0.0f : rep % 5 == 1 ? 1e30f : rep % 5 == 2 ? 1e-30f : 0.02f;
        float *v = floats_exact(n, scale);
        uint8_t *b4 = bytes_exact(17), *b6 = bytes_exact(25);
        float *o = (float *)malloc(32 * sizeof(float));
        rf_pack_mxfp4(v, n, b4);
        rf_pack_mxfp6(v, n, b6);
        mix(b4, 17);
        mix(b6, 25);
        rf_unpack_mxfp4(b4, o);
        mix(o, 128);
        rf_unpack_mxfp6(b6, o);
        mix(o, 128);
        free(o);
        free(v);
        free(b4);
        free(b6);
    }
    /* every decoder: whole blocks, ragged element counts, inputs cut at every kind of place, empty */
    for (size_t ti = 0; ti < sizeof(kTypes) / sizeof(kTypes[0]); ti++) {
        int t = kTypes[ti];
        size_t be = block_elems(t), bb = block_bytes_of(t);
        const size_t counts[] = {0, 1, be - 1 ? be - 1 : 1, be, be + 1, 3 * be, 3 * be + 7, 5 * be};
        for (size_t ci = 0; ci < sizeof(counts) / sizeof(counts[0]); ci++) {
            size_t n = counts[ci], full = ((n + be - 1) / be) * bb;
            const size_t cuts[] = {full, full + 5, 0, 1, 3, 4, 5, bb / 2, bb - 1, bb + 1, bb + 4, bb + 33 < full ? bb + 33 : full,
                                   full > 1 ? full - 1 : 0, full > 3 ? full - 3 : 0, 2 * bb + 3, 2 * bb + 32, 2 * bb + 34};
            for (size_t k = 0; k < sizeof(cuts) / sizeof(cuts[0]); k++) run_dequant(t, n, cuts[k]);
        }
        if (rf_data_size(t, 1000) == 0 && t < 100) abort();
    }
    if (rf_dequantize(3, NULL, 0, 0, NULL) != -1) abort();
    /* matmuls, norm, SwiGLU, MLP on small shapes */
    {
        const size_t m = 3, n = 40, k = 512;
        float *a = floats_exact(m * k, 1.0f), *c = (float *)malloc(m * n * sizeof(float)), *wd = (float *)malloc(n * k * sizeof(float));
        const int mm[] = {RF_Q4_0, RF_Q8_0, RF_Q4_K, RF_Q6_K, RF_MXFP4, RF_MXFP6_E2M3, RF_GGUF_Q4_0, RF_GGUF_Q8_0, RF_GGUF_Q4_K,
                          RF_GGUF_Q6_K, RF_MM_Q8_0, RF_MM_Q4_K, RF_MM_Q6_K};
        for (size_t ti = 0; ti < sizeof(mm) / sizeof(mm[0]); ti++) {
            int t = mm[ti];
            size_t len = n * (k / block_elems(t)) * rf_block_bytes(t);
            uint8_t *w = bytes_exact(len);
            tame_scales(t, w, len);
            /* keep f16 scale fields finite: clear the top exponent bit of every second byte pair at block heads */
            if (t == RF_Q4_K || t == RF_Q6_K || t == RF_MM_Q4_K || t == RF_MM_Q6_K)
                for (size_t o = 0; o < len; o += 256)
                    for (size_t s = 0; s < 32; s += 2) w[o + s + 1] &= 0xBF;
            if (t == RF_GGUF_Q4_0 || t == RF_GGUF_Q8_0)
                for (size_t o = 0; o < len; o += rf_block_bytes(t)) w[o + 1] &= 0xBF;
            if (t == RF_GGUF_Q4_K)
                for (size_t o = 0; o < len; o += 144) { w[o + 1] &= 0xBF; w[o + 3] &= 0xBF; }
            if (t == RF_GGUF_Q6_K)
                for (size_t o = 0; o < len; o += 210) w[o + 209] &= 0xBF;
            if (t == RF_MXFP4 || t == RF_MXFP6_E2M3)
                for (size_t o = 0; o < len; o += rf_block_bytes(t)) w[o] = (uint8_t)(int8_t)((int)(rnd() % 12) - 9);
            if (rf_qmatmul_nk(t, w, len, a, m, n, k, NULL, 0, c) != 0) abort();
            mix(c, m * n * 4);
            const int64_t sel[3] = {0, 17, 39};
            if (rf_qmatmul_nk(t, w, len, a, m, n, k, sel, 3, c) != 0) abort();
            mix(c, m * 3 * 4);
            if (rf_qmatmul_nk_staged(t, w, len, a, m, n, k, wd, c) != 0) abort();
            mix(c, m * n * 4);
            if (rf_qmatmul_kn(t, w, len, a, m, n, k, wd, c) != 0) abort();
            mix(c, m * n * 4);
            free(w);
        }
        float *b = floats_exact(k * n, 0.02f);
        rf_cpu_matmul_f32(a, b, m, n, k, c);
        mix(c, m * n * 4);
        rf_matmul_nk_f32(a, b, m, n, k, c);
        mix(c, m * n * 4);
        float *nw = floats_exact(k, 1.0f), *o = (float *)malloc(m * k * sizeof(float));
        rf_rms_norm(a, nw, m, k, 1e-6f, o);
        mix(o, m * k * 4);
        rf_swiglu(a, o, m * k, o);
        mix(o, m * k * 4);
        {
            size_t len = m * (k / 32) * 20;
            uint8_t *w = bytes_exact(len);
            tame_scales(RF_Q4_0, w, len);
            if (rf_dequant_rms_norm(RF_Q4_0, w, len, nw, m, k, 1e-6f, o) != 0) abort();
            mix(o, m * k * 4);
            free(w);
        }
        {
            const size_t hidden = 256, inter = 512, mm_rows = 2;
            size_t gl = inter * (hidden / 32) * 36, dl = hidden * (inter / 32) * 20;
            uint8_t *wg = bytes_exact(gl), *wu = bytes_exact(gl), *wdn = bytes_exact(dl);
            tame_scales(RF_Q8_0, wg, gl);
            tame_scales(RF_Q8_0, wu, gl);
            tame_scales(RF_Q4_0, wdn, dl);
            float *x = floats_exact(mm_rows * hidden, 1.0f), *nrm = floats_exact(hidden, 1.0f);
            float *scratch = (float *)malloc(mm_rows * (hidden + 3 * inter) * sizeof(float)), *y = (float *)malloc(mm_rows * hidden * sizeof(float));
            if (rf_mlp_swiglu_q(RF_Q8_0, wg, wu, gl, RF_Q4_0, wdn, dl, x, nrm, 1e-5f, mm_rows, hidden, inter, scratch, y) != 0) abort();
            mix(y, mm_rows * hidden * 4);
            if (rf_mlp_swiglu_q(RF_Q8_0, wg, wu, gl, RF_Q4_0, wdn, dl, x, NULL, 0.0f, mm_rows, hidden, inter, scratch, y) != 0) abort();
            mix(y, mm_rows * hidden * 4);
            free(wg); free(wu); free(wdn); free(x); free(nrm); free(scratch); free(y);
        }
        free(a); free(b); free(c); free(wd); free(nw); free(o);
    }
    printf("%016llx\n", (unsigned long long)g_hash);
    return 0;
}
