// Host tests of the C++ mirror (include/rocmforge_rfq.hpp): the reference's own
// unit-test vectors for this path, run through the mirrored entry points -- so
// every value comes from the GPU kernels.  Vectors and names follow
//   src/kernels/quant/q4_0.rs:317-438, q8_0.rs:78-183, q4_k.rs:280-368, q6_k.rs:273-399,
//   src/loader/mxfp_tests.rs:97-187 and 424-464, src/loader/dequant.rs:440-470,
//   src/kernels/matmul/quantized/q4_0.rs:318-338, src/ggml/hip_backend/op_dispatch.rs:951-1014,
//   src/ggml/hip_backend/ops/get_rows.rs:6-65.
// Prints one line per test; exit status 0 only if all passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "rocmforge_rfq.hpp"

using namespace rocmforge;
using bytes = std::vector<uint8_t>;

static int failures = 0;
#define EXPECT(cond)                                                                 \
    do {                                                                             \
        if (!(cond)) { std::printf("    FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); failures++; } \
    } while (0)

static void put_f32(bytes &d, size_t off, float v) { std::memcpy(d.data() + off, &v, 4); }
static void put_f16(bytes &d, size_t off, uint16_t bits) { std::memcpy(d.data() + off, &bits, 2); }
static bool all_eq(const std::vector<float> &v, size_t a, size_t b, float want)
{
    for (size_t i = a; i < b; i++) if (v[i] != want) return false;
    return true;
}

// ---- Q4_0 ---------------------------------------------------------------------
static void test_dequantize_q4_0_zeros()
{
    bytes d(20, 0x88);
    put_f32(d, 0, 1.0f);
    auto r = loader::dequant_q4_0(d, 32);
    EXPECT(r.size() == 32 && all_eq(r, 0, 32, 0.0f));
}
static void test_dequantize_q4_0_positive()
{
    bytes d(20, 0);
    put_f32(d, 0, 2.0f);
    for (int i = 0; i < 16; i++) d[4 + i] = (uint8_t)(((i + 1) << 4) | i);
    auto r = loader::dequant_q4_0(d, 32);
    EXPECT(r[0] == -16.0f && r[1] == -14.0f && r[30] == 14.0f && r[31] == -16.0f);
}
static void test_dequantize_q4_0_partial_and_multiple_blocks()
{
    bytes d(20, 0x88);
    put_f32(d, 0, 1.0f);
    auto r = loader::dequant_q4_0(d, 10);
    EXPECT(r.size() == 10 && all_eq(r, 0, 10, 0.0f));
    bytes d2(40, 0x88);
    put_f32(d2, 0, 1.0f);
    put_f32(d2, 20, 2.0f);
    for (int i = 24; i < 40; i++) d2[i] = 0xCC;
    r = loader::dequant_q4_0(d2, 64);
    EXPECT(all_eq(r, 0, 32, 0.0f) && all_eq(r, 32, 64, 8.0f));
    // short input: the blocks that are missing stay 0.0
    r = loader::dequant_q4_0(d2, 96);
    EXPECT(r.size() == 96 && all_eq(r, 64, 96, 0.0f));
}

// ---- Q8_0 ---------------------------------------------------------------------
static void test_dequantize_q8_0_vectors()
{
    bytes d(36, 128);
    put_f32(d, 0, 1.0f);
    EXPECT(all_eq(loader::dequant_q8_0(d, 32), 0, 32, 0.0f));
    put_f32(d, 0, 2.0f);
    for (int i = 0; i < 32; i++) d[4 + i] = (uint8_t)(120 + i);
    auto r = loader::dequant_q8_0(d, 32);
    EXPECT(r[0] == -16.0f && r[15] == 14.0f && r[31] == 46.0f);
    bytes d2(72, 128);
    put_f32(d2, 0, 1.0f);
    put_f32(d2, 36, 0.5f);
    for (int i = 40; i < 72; i++) d2[i] = 138;
    r = loader::dequant_q8_0(d2, 64);
    EXPECT(all_eq(r, 0, 32, 0.0f) && all_eq(r, 32, 64, 5.0f));
}

// ---- Q4_K ---------------------------------------------------------------------
static void test_dequantize_q4_k_single_block()
{
    bytes d(256, 0);
    for (int i = 0; i < 8; i++) put_f16(d, 2 * i, 0x3C00); // 1.0
    for (int i = 0; i < 224; i++) d[32 + i] = (uint8_t)(((i % 16) << 4) | (i % 16));
    auto r = loader::dequant_q4_k(d, 256);
    bool ok = true;
    for (int i = 0; i < 256; i++) {
        int sb = i / 32, e = i % 32, qo = sb * 28 + (e * 4) / 8;
        unsigned combined = ((unsigned)d[32 + qo + 1] << 8) | d[32 + qo];
        if (r[i] != (float)((combined >> ((e * 4) % 8)) & 15u)) ok = false;
    }
    EXPECT(ok);
}
static void test_dequantize_q4_k_partial_block_and_mins()
{
    bytes d(256, 0x88);
    for (int i = 0; i < 32; i++) d[i] = 0;
    for (int i = 0; i < 8; i++) put_f16(d, 2 * i, 0x3C00);
    auto r = loader::dequant_q4_k(d, 100);
    EXPECT(r.size() == 100 && all_eq(r, 0, 100, 8.0f));
    d[16 + 1] = (uint8_t)(int8_t)-3; // min of sub-block 1
    r = loader::dequant_q4_k(d, 256);
    EXPECT(all_eq(r, 0, 32, 8.0f) && all_eq(r, 32, 64, 5.0f));
}

// ---- Q6_K ---------------------------------------------------------------------
static void test_dequantize_q6_k_vectors()
{
    bytes d(256, 0);
    for (int i = 0; i < 16; i++) put_f16(d, 2 * i, 0x4000); // 2.0
    EXPECT(all_eq(loader::dequant_q6_k(d, 100), 0, 100, 0.0f));
    for (int i = 0; i < 16; i++) put_f16(d, 2 * i, 0x3C00);
    for (int i = 32; i < 224; i++) d[i] = 0xFF;                // every 6-bit field = 63 = -1
    EXPECT(all_eq(loader::dequant_q6_k(d, 256), 0, 256, -1.0f));
    for (int i = 0; i < 192; i++) d[32 + i] = (uint8_t)((i % 64) * 4);
    auto r = loader::dequant_q6_k(d, 256);
    bool finite = true;
    for (float v : r) if (!std::isfinite(v)) finite = false;
    EXPECT(finite);
}

// ---- MXFP ---------------------------------------------------------------------
static GgufTensor mx_tensor(GgufTensorType t, size_t n, bytes data)
{
    GgufTensor g("w", TensorShape::from_dims({n}), t, 0);
    g.data = std::move(data);
    return g;
}
static void test_mxfp4_block_of_twos_and_clamp()
{
    // exponent byte 1 (scale 2.0), every nibble 0b0001 (decodes to 1.0): 2.0 each
    bytes d(17, 0x11);
    d[0] = 1;
    auto r = loader::dequant_mxfp4(mx_tensor(GgufTensorType::Mxfp4, 32, d));
    EXPECT(r.ok && r.value.size() == 32 && all_eq(r.value, 0, 32, 2.0f));
    // code 7 decodes to 8.0; scale 4.0: clamped to +8; code 15 to -8
    bytes c(17, 0x7F);
    c[0] = 2;
    r = loader::dequant_mxfp4(mx_tensor(GgufTensorType::Mxfp4, 32, c));
    EXPECT(r.ok && r.value[0] == 8.0f && r.value[1] == -8.0f); // element 2j = HIGH nibble
    GgufTensor t = mx_tensor(GgufTensorType::Mxfp4, 64, d);
    EXPECT(t.data_size() == 34);
}
static void test_mxfp6_block_size_clamp_and_last_element()
{
    bytes d(25, 0xFF);
    d[0] = 3; // scale 8: every code 0b111111 = -7.5 * 8 -> clamped to -7.5
    auto r = loader::dequant_mxfp6(mx_tensor(GgufTensorType::Mxfp6E2m3, 32, d));
    EXPECT(r.ok && r.value.size() == 32 && all_eq(r.value, 0, 31, -7.5f));
    EXPECT(r.value[31] == 0.0f); // the loader never reaches the last element of a block
    auto r2 = loader::dequantize(mx_tensor(GgufTensorType::Mxfp6E3m2, 32, d)); // decoded like E2M3
    EXPECT(r2.ok && r2.value == r.value);
    EXPECT(mx_tensor(GgufTensorType::Mxfp6E2m3, 32, d).data_size() == 25);
}

// ---- types ----------------------------------------------------------------------
static void test_tensor_types_and_sizes()
{
    EXPECT(tensor_type_from_u32(20).ok && tensor_type_from_u32(20).value == GgufTensorType::Mxfp4);
    EXPECT(tensor_type_from_u32(21).value == GgufTensorType::Mxfp6E2m3 && tensor_type_from_u32(22).value == GgufTensorType::Mxfp6E3m2);
    EXPECT(!tensor_type_from_u32(3).ok && !tensor_type_from_u32(6).ok && !tensor_type_from_u32(7).ok && !tensor_type_from_u32(99).ok);
    EXPECT(element_size(GgufTensorType::Mxfp4) == 32 && element_size(GgufTensorType::Q4_K) == 256 && element_size(GgufTensorType::F16) == 2);
    EXPECT(block_size(GgufTensorType::Q8_0) == 32 && block_size(GgufTensorType::Q6_K) == 256 && block_size(GgufTensorType::F32) == 1);
    EXPECT(std::string(to_string(GgufTensorType::Q4_K)) == "Q4_K" && std::string(to_string(GgufTensorType::F32)) == "FP32");
    TensorShape s = TensorShape::from_dims({4, 8, 16});
    EXPECT(s.total_elements() == 512 && s.strides()[0] == 128 && s.strides()[1] == 16 && s.strides()[2] == 1);
    GgufTensor q4("t", TensorShape::from_dims({2, 32}), GgufTensorType::Q4_0, 0);
    EXPECT(q4.data_size() == 2 * 36);            // as the reference counts it (the decoder strides by 20)
    GgufTensor qk("t", TensorShape::from_dims({300}), GgufTensorType::Q4_K, 0);
    EXPECT(qk.data_size() == 512 && qk.quant_type == "Q4_K");
}
static void test_dequantize_dispatch_f32_f16()
{
    GgufTensor f("f", TensorShape::from_dims({2}), GgufTensorType::F32, 0);
    f.data.resize(9);                             // one trailing byte is dropped
    float a = 1.5f, b = -2.25f;
    std::memcpy(f.data.data(), &a, 4);
    std::memcpy(f.data.data() + 4, &b, 4);
    auto r = loader::dequantize(f);
    EXPECT(r.ok && r.value.size() == 2 && r.value[0] == 1.5f && r.value[1] == -2.25f);
    GgufTensor h("h", TensorShape::from_dims({4}), GgufTensorType::F16, 0);
    h.data.resize(8);
    put_f16(h.data, 0, 0x3C00); put_f16(h.data, 2, 0x4000); put_f16(h.data, 4, 0xC000); put_f16(h.data, 6, 0x0001);
    r = loader::dequantize(h);
    EXPECT(r.ok && r.value[0] == 1.0f && r.value[1] == 2.0f && r.value[2] == -2.0f && r.value[3] == std::ldexp(1.0f, -24));
}
// src/loader/dequant.rs:440-665 (Q5_K, Q3_K, Q2_K through the dispatcher)
static void test_dequantize_other_k_types()
{
    auto one_block = [](GgufTensorType t, size_t n) {
        GgufTensor g("q", TensorShape::from_dims({n}), t, 0);
        g.data.assign(256, 0);
        put_f16(g.data, 0, 0x3C00);               // sub-block 0: scale 1.0
        return g;
    };
    GgufTensor q5 = one_block(GgufTensorType::Q5_K, 256);
    q5.data[48] = 0x01;
    auto r = loader::dequantize(q5);
    EXPECT(r.ok && r.value.size() == 256 && r.value[0] == 1.0f && r.value[1] == 0.0f && r.value[15] == 0.0f);
    GgufTensor q5p = one_block(GgufTensorType::Q5_K, 100);
    r = loader::dequant_q5_k(q5p);
    EXPECT(r.ok && r.value.size() == 100 && r.value[0] == 0.0f && r.value[99] == 0.0f);
    GgufTensor q5m("q", TensorShape::from_dims({512}), GgufTensorType::Q5_K, 0);
    q5m.data.assign(512, 0);
    put_f16(q5m.data, 0, 0x3C00); put_f16(q5m.data, 256, 0x4000);
    q5m.data[256 + 48] = 0xFF; q5m.data[256 + 49] = 0x80;
    r = loader::dequantize(q5m);
    EXPECT(r.ok && r.value[0] == 0.0f && r.value[255] == 0.0f && r.value[256] == 62.0f);
    GgufTensor q3 = one_block(GgufTensorType::Q3_K, 256);
    r = loader::dequantize(q3);
    EXPECT(r.ok && r.value[0] == -4.0f && r.value[15] == -4.0f);
    q3.data[36] = 0x01;
    r = loader::dequant_q3_k(q3);
    EXPECT(r.ok && r.value[0] == -3.0f && r.value[1] == -4.0f);
    GgufTensor q2 = one_block(GgufTensorType::Q2_K, 256);
    r = loader::dequantize(q2);
    EXPECT(r.ok && r.value[0] == 0.0f && r.value[15] == 0.0f);
    q2.data[68] = 0x01;
    r = loader::dequant_q2_k(q2);
    EXPECT(r.ok && r.value[0] == 1.0f);
    GgufTensor q2p = one_block(GgufTensorType::Q2_K, 100);
    r = loader::dequantize(q2p);
    EXPECT(r.ok && r.value.size() == 100 && r.value[0] == 0.0f);
}

// ---- device buffers and matmul ------------------------------------------------------
static void test_dequantize_q4_0_kernel_cached_and_twins()
{
    auto be = HipBackend::create();
    EXPECT(be.ok);
    bytes d(40, 0x88);
    put_f32(d, 0, 1.0f);
    put_f32(d, 20, 2.0f);
    for (int i = 24; i < 40; i++) d[i] = 0xCC;
    auto out = HipBuffer::create(64 * sizeof(float));
    EXPECT(out.ok);
    EXPECT(dequantize_q4_0_kernel_cached(be.value, d, out.value, 64).ok);
    std::vector<float> h(64);
    EXPECT(out.value.copy_to_host(h).ok && all_eq(h, 0, 32, 0.0f) && all_eq(h, 32, 64, 8.0f));
    auto small = HipBuffer::create(16);
    EXPECT(!dequantize_q4_0_kernel_cached(be.value, d, small.value, 64).ok);   // output too small
    bytes k(256, 0x88);
    for (int i = 0; i < 32; i++) k[i] = 0;
    for (int i = 0; i < 8; i++) put_f16(k, 2 * i, 0x3C00);
    auto outk = HipBuffer::create(256 * sizeof(float));
    EXPECT(dequantize_q4_k_gpu_kernel(be.value, k, outk.value, 256).ok);
    std::vector<float> hk(256);
    EXPECT(outk.value.copy_to_host(hk).ok && all_eq(hk, 0, 256, 8.0f));
}
static void test_matmul_q4_0_against_dequantized_weights()
{
    // weights [n_rows=8, n_cols=64], input [64]: out = deq(W) . x, as q4_0.rs:318-338 checks it
    const size_t n_rows = 8, n_cols = 64;
    bytes w(n_rows * (n_cols / 32) * 20);
    for (size_t b = 0; b < w.size() / 20; b++) {
        put_f32(w, b * 20, 0.25f * (float)(b % 5 + 1));
        for (int i = 0; i < 16; i++) w[b * 20 + 4 + i] = (uint8_t)((b * 37 + i * 11) & 0xFF);
    }
    std::vector<float> x(n_cols);
    for (size_t i = 0; i < n_cols; i++) x[i] = 0.125f * (float)((int)(i % 9) - 4);
    auto be = HipBackend::create();
    auto in = HipBuffer::create(n_cols * 4), out = HipBuffer::create(n_rows * 4);
    EXPECT(in.value.copy_from_host(x).ok);
    EXPECT(matmul_q4_0(be.value, w, in.value, n_rows, n_cols, out.value).ok);
    std::vector<float> y(n_rows), deq = loader::dequant_q4_0(w, n_rows * n_cols);
    EXPECT(out.value.copy_to_host(y).ok);
    bool close = true;
    for (size_t r = 0; r < n_rows; r++) {
        float s = 0.0f;
        for (size_t c = 0; c < n_cols; c++) s += x[c] * deq[r * n_cols + c];   // cpu_matmul_f32 order
        if (std::fabs(y[r] - s) > 1e-3f * std::fmax(std::fabs(s), 1.0f)) close = false;
    }
    EXPECT(close);
    // the batch description type runs the same operation
    QuantizedMatmulOp op(w, n_rows, n_cols, QuantFormat::Q4_0);
    auto out2 = HipBuffer::create(n_rows * 4);
    EXPECT(op.m == 1 && op.execute(be.value, in.value, out2.value).ok);
    std::vector<float> y2(n_rows);
    EXPECT(out2.value.copy_to_host(y2).ok && y2 == y);
    // raw device pointers
    auto dw = HipBuffer::create(w.size());
    EXPECT(dw.value.copy_from_host(w).ok);
    EXPECT(matmul_q4_0_gpu(be.value, (const float *)in.value.as_ptr(), (const uint8_t *)dw.value.as_ptr(),
                           (float *)out2.value.as_ptr(), 1, n_rows, n_cols).ok);
    EXPECT(be.value.synchronize().ok && out2.value.copy_to_host(y2).ok && y2 == y);
    // wrong byte count is an error, not a crash
    bytes shorter(w.begin(), w.end() - 20);
    EXPECT(!matmul_q4_0(be.value, shorter, in.value, n_rows, n_cols, out.value).ok);
}
// What the reference computes on the bytes (src/kernels/matmul/quantized/q4_0.rs:274-311 + src/tensor/matmul.rs:219-233,
// kernels/q4_0_matmul.hip:207): the flat dequantised array read as b[k, n], and the module's own int8 decoder
// (quantized/q8_0.rs:18-56; its unit-test vector :113-131).
static void test_matmul_as_the_reference_computes_it()
{
    const size_t n_rows = 8, n_cols = 64;
    bytes w(n_rows * n_cols / 32 * 20);
    for (size_t b = 0; b < w.size() / 20; b++) {
        put_f32(w, b * 20, 0.25f * (float)(b % 5 + 1));
        for (int i = 0; i < 16; i++) w[b * 20 + 4 + i] = (uint8_t)((b * 37 + i * 11) & 0xFF);
    }
    std::vector<float> x(n_cols);
    for (size_t i = 0; i < n_cols; i++) x[i] = 0.125f * (float)((int)(i % 9) - 4);
    auto be = HipBackend::create();
    auto in = HipBuffer::create(n_cols * 4), out = HipBuffer::create(n_rows * 4), out2 = HipBuffer::create(n_rows * 4);
    EXPECT(in.value.copy_from_host(x).ok);
    EXPECT(matmul_q4_0_cpu_fallback(be.value, w, in.value, n_rows, n_cols, out.value).ok);
    std::vector<float> y(n_rows), y2(n_rows), deq = matmul_quantized::dequantize_q4_0(w, n_rows * n_cols);
    EXPECT(out.value.copy_to_host(y).ok);
    bool close = true, differs = false;
    for (size_t j = 0; j < n_rows; j++) {
        float s = 0.0f, s_rows = 0.0f;
        for (size_t l = 0; l < n_cols; l++) s += x[l] * deq[l * n_rows + j];          // cpu_matmul_f32: b[l * n + j]
        for (size_t l = 0; l < n_cols; l++) s_rows += x[l] * deq[j * n_cols + l];
        if (std::fabs(y[j] - s) > 1e-3f * std::fmax(std::fabs(s), 1.0f)) close = false;
        if (std::fabs(s - s_rows) > 1e-2f) differs = true;
    }
    EXPECT(close);
    EXPECT(differs);                                                                   // the two readings are different numbers
    auto dw = HipBuffer::create(w.size());
    EXPECT(dw.value.copy_from_host(w).ok);
    EXPECT(matmul_q4_0_gpu(be.value, (const float *)in.value.as_ptr(), (const uint8_t *)dw.value.as_ptr(),
                           (float *)out2.value.as_ptr(), 1, n_rows, n_cols, WeightLayout::FlatKN).ok);
    EXPECT(be.value.synchronize().ok && out2.value.copy_to_host(y2).ok && y2 == y);
    // int8 decoder: scale 1.0, bytes (i - 16) as u8 -> i - 16
    bytes q8(36);
    put_f32(q8, 0, 1.0f);
    for (int i = 0; i < 32; i++) q8[4 + i] = (uint8_t)(int8_t)(i - 16);
    auto v = matmul_quantized::dequantize_q8_0(q8, 32);
    bool exact = true;
    for (int i = 0; i < 32; i++) if (v[i] != (float)(i - 16)) exact = false;
    EXPECT(exact);
    // matmul_q8_0 as its body computes it: 32 rows x 1 column of that block, x = 1 -> the sum of the 32 values... over l:
    // n_rows = 1, n_cols = 32: out[0] = sum_l x[l] * deq[l]
    std::vector<float> ones(32, 1.0f);
    auto in8 = HipBuffer::create(32 * 4), out8 = HipBuffer::create(4);
    EXPECT(in8.value.copy_from_host(ones).ok);
    EXPECT(matmul_q8_0_as_computed(be.value, q8, in8.value, 1, 32, out8.value).ok);
    std::vector<float> y8(1);
    EXPECT(out8.value.copy_to_host(y8).ok && y8[0] == -16.0f);                          // sum of -16 .. 15
    // the K decoders of the module: a scale whose mantissa bits 3..9 are clear decodes like the loader's Q6_K; Q4_K reads
    // other bytes
    bytes k6(256, 0);
    for (int g = 0; g < 16; g++) put_f16(k6, 2 * g, 0x3C00);                           // 1.0
    for (int i = 32; i < 224; i++) k6[i] = (uint8_t)(i * 7);
    EXPECT(matmul_quantized::dequantize_q6_k(k6, 256) == loader::dequant_q6_k(k6, 256));
    // f16_to_f32_cpu (quantized/common.rs:47) shifts the mantissa within 16 bits: 0x3E00 (1.5) widens to 1.0 there
    bytes k6b = k6;
    for (int g = 0; g < 16; g++) put_f16(k6b, 2 * g, 0x3E00);
    EXPECT(matmul_quantized::dequantize_q6_k(k6b, 256) == matmul_quantized::dequantize_q6_k(k6, 256));
    EXPECT(loader::dequant_q6_k(k6b, 256) != loader::dequant_q6_k(k6, 256));
    bytes k4(256, 0);
    for (int sb = 0; sb < 8; sb++) put_f16(k4, 2 * sb, 0x3C00);
    for (int i = 32; i < 256; i++) k4[i] = (uint8_t)(i * 5 + 1);
    auto a4 = matmul_quantized::dequantize_q4_k(k4, 256), c4 = loader::dequant_q4_k(k4, 256);
    bool sb0_same = true, rest_differs = false;
    for (int i = 0; i < 32; i++) if (a4[i] != c4[i]) sb0_same = false;
    for (int i = 32; i < 256; i++) if (a4[i] != c4[i]) rest_differs = true;
    EXPECT(sb0_same && rest_differs);
    EXPECT(a4[32] == (float)(k4[32 + 20] & 15));                                      // sub-block 1 starts at byte 52
}

static void test_matmul_validation_like_op_dispatch()
{
    EXPECT(validate_matmul_q4_0({8, 64}, 8 * 2 * 20, {1, 64}).ok);
    EXPECT(!validate_matmul_q4_0({8, 64}, 8 * 2 * 20 - 1, {1, 64}).ok);          // weights size mismatch
    EXPECT(!validate_matmul_q4_0({8, 64}, 8 * 2 * 20, {1, 32}).ok);              // k != weights_k
    EXPECT(!validate_matmul_q4_0({8, 64, 1}, 8 * 2 * 20, {1, 64}).ok);           // expects 2D tensors
    EXPECT(validate_matmul_q8_0({4, 32}, 4 * 36, {8, 32}).ok);
    EXPECT(bytes_per_element(QuantFormat::Q8_0) == 36.0f / 32.0f && std::string(name(QuantFormat::Q6_K)) == "Q6_K");
}

// get_rows.rs:6-65: rows are copied by token id; an id outside the vocabulary is an error
static void test_get_rows_f32_and_packed_tables()
{
    auto be = HipBackend::create();
    EXPECT(be.ok);
    const size_t n_vocab = 5, n_embd = 32;
    std::vector<float> table(n_vocab * n_embd);
    for (size_t i = 0; i < table.size(); i++) table[i] = (float)i * 0.5f;
    auto tab = HipBuffer::create(table.size() * 4), out = HipBuffer::create(3 * n_embd * 4);
    EXPECT(tab.ok && out.ok && tab.value.copy_from_host(table).ok);
    EXPECT(get_rows(be.value, tab.value, {4, 0, 4}, n_embd, n_vocab, RFQ_TABLE_F32, out.value).ok);
    std::vector<float> got(3 * n_embd);
    EXPECT(out.value.copy_to_host(got).ok);
    for (size_t j = 0; j < n_embd; j++)
        EXPECT(got[j] == table[4 * n_embd + j] && got[n_embd + j] == table[j] && got[2 * n_embd + j] == got[j]);
    Status bad = get_rows(be.value, tab.value, {1, 5}, n_embd, n_vocab, RFQ_TABLE_F32, out.value);
    EXPECT(!bad.ok && bad.error == "Token ID 5 exceeds vocab size 5");
    // a Q4_0 table: row r = one block with scale r + 1 and every nibble 9 -> (9 - 8) * (r + 1)
    bytes packed(n_vocab * 20);
    for (size_t r = 0; r < n_vocab; r++) {
        put_f32(packed, r * 20, (float)(r + 1));
        for (size_t j = 0; j < 16; j++) packed[r * 20 + 4 + j] = 0x99;
    }
    auto ptab = HipBuffer::create(packed.size());
    EXPECT(ptab.ok && ptab.value.copy_from_host(packed).ok);
    EXPECT(get_rows(be.value, ptab.value, {2, 0, 3}, n_embd, n_vocab, RFQ_Q4_0, out.value).ok);
    EXPECT(out.value.copy_to_host(got).ok);
    EXPECT(all_eq(got, 0, 32, 3.0f) && all_eq(got, 32, 64, 1.0f) && all_eq(got, 64, 96, 4.0f));
}

// src/mlp/rms_norm_tests.rs:211-251, src/mlp/swiglu_tests.rs:329-372, and an MLP whose result is known in closed form
static void test_norm_swiglu_and_mlp()
{
    auto be = HipBackend::create();
    EXPECT(be.ok);
    const size_t hidden = 1024, inter = 512;
    auto x = HipBuffer::create(hidden * 4), w = HipBuffer::create(hidden * 4), o = HipBuffer::create(hidden * 4);
    EXPECT(x.ok && w.ok && o.ok);
    std::vector<float> twos(hidden, 2.0f), ones(hidden, 1.0f), got(hidden);
    EXPECT(x.value.copy_from_host(twos).ok && w.value.copy_from_host(ones).ok);
    EXPECT(rms_norm_gpu_kernel(be.value, (const float *)x.value.as_ptr(), (const float *)w.value.as_ptr(),
                               (float *)o.value.as_ptr(), 1, hidden, 1e-6f).ok && be.value.synchronize().ok);
    EXPECT(o.value.copy_to_host(got).ok);
    for (float v : got) EXPECT(std::fabs(v - 1.0f) < 0.01f);            // constant positive input -> ~1
    std::vector<float> zeros(hidden, 0.0f);
    EXPECT(x.value.copy_from_host(zeros).ok);
    EXPECT(swiglu_gpu_kernel(be.value, (const float *)w.value.as_ptr(), (const float *)x.value.as_ptr(),
                             (float *)o.value.as_ptr(), 1, hidden).ok && be.value.synchronize().ok);
    EXPECT(o.value.copy_to_host(got).ok && all_eq(got, 0, hidden, 0.0f)); // up = 0 -> 0

    // fused_q4_0_rmsnorm: one row of blocks with scale 2 and every nibble 9 decodes to 2.0 everywhere -> ~1 * weight
    bytes row(hidden / 32 * 20);
    for (size_t blk = 0; blk < hidden / 32; blk++) {
        put_f32(row, blk * 20, 2.0f);
        for (size_t j = 0; j < 16; j++) row[blk * 20 + 4 + j] = 0x99;
    }
    auto packed = HipBuffer::create(row.size());
    EXPECT(packed.ok && packed.value.copy_from_host(row).ok);
    std::vector<float> threes(hidden, 3.0f);
    EXPECT(w.value.copy_from_host(threes).ok);
    EXPECT(fused_q4_0_rmsnorm(be.value, (const uint8_t *)packed.value.as_ptr(), (const float *)w.value.as_ptr(),
                              (float *)o.value.as_ptr(), 1, hidden, 1e-6f).ok && be.value.synchronize().ok);
    EXPECT(o.value.copy_to_host(got).ok);
    for (float v : got) EXPECT(std::fabs(v - 3.0f) < 0.01f);

    // MLP with constant matrices: gate weights 1/64, up weights 1/32, down weights 1/8 (Q4_0: scale * (9 - 8)),
    // x = 1: gate = 16, up = 32, h = 16 * 32 * sigmoid(32) = 512, out = 512 * 512 / 8 = 32768
    auto constant = [&](size_t rows, size_t k, float value) {
        bytes m(rows * (k / 32) * 20);
        for (size_t blk = 0; blk < rows * (k / 32); blk++) {
            put_f32(m, blk * 20, value);
            for (size_t j = 0; j < 16; j++) m[blk * 20 + 4 + j] = 0x99;
        }
        DeviceTensor t;
        auto buf = HipBuffer::create(m.size());
        EXPECT(buf.ok && buf.value.copy_from_host(m).ok);
        t.buffer = buf.value;
        t.shape = TensorShape::from_dims({rows, k});
        t.format = RFQ_Q4_0;
        return t;
    };
    DeviceTensor gate = constant(inter, hidden, 1.0f / 64), up = constant(inter, hidden, 1.0f / 32),
                 down = constant(hidden, inter, 1.0f / 8), hs, out;
    EXPECT(x.value.copy_from_host(ones).ok);
    hs.buffer = x.value; hs.shape = TensorShape::from_dims({1, hidden});
    out.buffer = o.value; out.shape = TensorShape::from_dims({1, hidden});
    Status st = mlp_swiglu(be.value, hs, gate, up, down, out);
    EXPECT(st.ok);
    EXPECT(o.value.copy_to_host(got).ok);
    for (float v : got) EXPECT(std::fabs(v - 32768.0f) < 1.0f);
    // the reference's shape checks
    DeviceTensor bad = down;
    bad.shape = TensorShape::from_dims({hidden, inter + 32});
    Status e = mlp_swiglu(be.value, hs, gate, up, bad, out);
    EXPECT(!e.ok && e.error == "All intermediate dimensions must match");
    hs.shape = TensorShape::from_dims({hidden});
    e = mlp_swiglu(be.value, hs, gate, up, down, out);
    EXPECT(!e.ok && e.error == "hidden_states must be 2D [seq_len, hidden_size]");
}

// op_dispatch.rs:951-1083 without the round trip of the weights through the host: constant matrices, 11 input rows
static void test_execute_matmul_quantized_ops()
{
    auto be = HipBackend::create();
    EXPECT(be.ok);
    const size_t n = 48, k = 512, m = 11;
    struct Case { Op op; size_t block_elems, block_bytes; float weight; };
    // every block decodes to one constant: Q4_0 scale 0.5, nibbles 9 -> 0.5; Q8_0 scale 0.25, bytes 130 -> 0.5;
    // Q4_K scales 0.5 (f16 0x3800), mins 0, nibbles 1 -> 0.5; MXFP4 exponent 0, codes 2 -> 1.0
    const Case cases[] = {{Op::MatMulQ4_0, 32, 20, 0.5f}, {Op::MatMulQ8_0, 32, 36, 0.5f}, {Op::MatMulQ4_K, 256, 256, 0.5f},
                          {Op::MatMulMxfp4, 32, 17, 1.0f}};
    std::vector<float> x(m * k);
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < k; j++) x[i * k + j] = (float)(i + 1) * ((j & 1) ? 0.25f : 0.5f);   // row sum = (i + 1) * 192
    DeviceTensor in, out;
    auto xb = HipBuffer::create(x.size() * 4), ob = HipBuffer::create(m * n * 4);
    EXPECT(xb.ok && ob.ok && xb.value.copy_from_host(x).ok);
    in.buffer = xb.value; in.shape = TensorShape::from_dims({m, k});
    out.buffer = ob.value; out.shape = TensorShape::from_dims({m, n});
    for (const Case &c : cases) {
        bytes w(n * k / c.block_elems * c.block_bytes);
        for (size_t blk = 0; blk < w.size() / c.block_bytes; blk++) {
            uint8_t *p = w.data() + blk * c.block_bytes;
            switch (c.op) {
            case Op::MatMulQ4_0: put_f32(w, blk * 20, 0.5f); std::memset(p + 4, 0x99, 16); break;
            case Op::MatMulQ8_0: put_f32(w, blk * 36, 0.25f); std::memset(p + 4, 130, 32); break;
            case Op::MatMulQ4_K:
                for (int sb = 0; sb < 8; sb++) put_f16(w, blk * 256 + 2 * sb, 0x3800);
                std::memset(p + 16, 0, 16);
                std::memset(p + 32, 0x11, 224);
                break;
            default: p[0] = 0; std::memset(p + 1, 0x22, 16); break;
            }
        }
        DeviceTensor wt;
        auto wb = HipBuffer::create(w.size());
        EXPECT(wb.ok && wb.value.copy_from_host(w).ok);
        wt.buffer = wb.value; wt.shape = TensorShape::from_dims({n, k});
        Status st = execute_matmul_quantized(be.value, c.op, wt, in, out);
        EXPECT(st.ok && be.value.synchronize().ok);
        std::vector<float> got(m * n);
        EXPECT(ob.value.copy_to_host(got).ok);
        for (size_t i = 0; i < m; i++)
            for (size_t j = 0; j < n; j++) EXPECT(std::fabs(got[i * n + j] - (float)(i + 1) * 192.0f * c.weight) < 1e-3f * (i + 1) * 192.0f);
        // the reference's checks
        DeviceTensor short_in = in;
        short_in.shape = TensorShape::from_dims({m, k - 32});
        Status e = execute_matmul_quantized(be.value, c.op, wt, short_in, out);
        EXPECT(!e.ok && e.error == std::string(name(c.op)) + " dimension mismatch: k=" + std::to_string(k - 32) +
                                       " weights_k=" + std::to_string(k));
        wt.shape = TensorShape::from_dims({n + 1, k});
        e = execute_matmul_quantized(be.value, c.op, wt, in, out);
        EXPECT(!e.ok && e.error.find("weights size mismatch") != std::string::npos);
    }
}

// batch_quantized.rs:139-190: ops sharing one input, one output buffer each
static void test_batch_quantized_matmul()
{
    auto be = HipBackend::create();
    EXPECT(be.ok);
    const size_t k = 256;
    std::vector<float> x(k, 1.0f);
    auto xb = HipBuffer::create(k * 4);
    EXPECT(xb.ok && xb.value.copy_from_host(x).ok);
    std::vector<QuantizedMatmulOp> ops;
    for (size_t n : {4u, 9u}) {                      // Q4_0 rows of scale (r + 1), nibbles 9: row sum = 256 * (r + 1)
        bytes w(n * (k / 32) * 20);
        for (size_t r = 0; r < n; r++)
            for (size_t blk = 0; blk < k / 32; blk++) {
                put_f32(w, (r * (k / 32) + blk) * 20, (float)(r + 1));
                std::memset(w.data() + (r * (k / 32) + blk) * 20 + 4, 0x99, 16);
            }
        ops.emplace_back(w, n, k, QuantFormat::Q4_0);
    }
    BatchQuantizedMatmul batch(be.value);
    auto res = batch.process_batch(xb.value, ops);
    EXPECT(res.ok && res.value.size() == 2);
    for (size_t i = 0; res.ok && i < 2; i++) {
        std::vector<float> got(ops[i].n);
        EXPECT(res.value[i].copy_to_host(got).ok);
        for (size_t r = 0; r < ops[i].n; r++) EXPECT(got[r] == 256.0f * (float)(r + 1));
    }
    auto prof = batch.with_profiling().process_batch_profiled(xb.value, ops);
    EXPECT(prof.ok && prof.value.outputs.size() == 2 && prof.value.timings_ms.size() == 2 && prof.value.total_time_ms > 0.0f);
}

int main()
{
    struct T { const char *name; std::function<void()> fn; };
    const T tests[] = {
        {"test_dequantize_q4_0_zeros", test_dequantize_q4_0_zeros},
        {"test_dequantize_q4_0_positive", test_dequantize_q4_0_positive},
        {"test_dequantize_q4_0_partial_and_multiple_blocks", test_dequantize_q4_0_partial_and_multiple_blocks},
        {"test_dequantize_q8_0_vectors", test_dequantize_q8_0_vectors},
        {"test_dequantize_q4_k_single_block", test_dequantize_q4_k_single_block},
        {"test_dequantize_q4_k_partial_block_and_mins", test_dequantize_q4_k_partial_block_and_mins},
        {"test_dequantize_q6_k_vectors", test_dequantize_q6_k_vectors},
        {"test_dequantize_other_k_types", test_dequantize_other_k_types},
        {"test_mxfp4_block_of_twos_and_clamp", test_mxfp4_block_of_twos_and_clamp},
        {"test_mxfp6_block_size_clamp_and_last_element", test_mxfp6_block_size_clamp_and_last_element},
        {"test_tensor_types_and_sizes", test_tensor_types_and_sizes},
        {"test_dequantize_dispatch_f32_f16", test_dequantize_dispatch_f32_f16},
        {"test_dequantize_q4_0_kernel_cached_and_twins", test_dequantize_q4_0_kernel_cached_and_twins},
        {"test_matmul_q4_0_against_dequantized_weights", test_matmul_q4_0_against_dequantized_weights},
        {"test_matmul_as_the_reference_computes_it", test_matmul_as_the_reference_computes_it},
        {"test_matmul_validation_like_op_dispatch", test_matmul_validation_like_op_dispatch},
        {"test_get_rows_f32_and_packed_tables", test_get_rows_f32_and_packed_tables},
        {"test_norm_swiglu_and_mlp", test_norm_swiglu_and_mlp},
        {"test_execute_matmul_quantized_ops", test_execute_matmul_quantized_ops},
        {"test_batch_quantized_matmul", test_batch_quantized_matmul},
    };
    for (const T &t : tests) {
        int before = failures;
        std::printf("%s ...\n", t.name);
        std::fflush(stdout);
        t.fn();
        std::printf("%s %s\n", t.name, failures == before ? "ok" : "FAILED");
        std::fflush(stdout);
    }
    std::printf("%d test(s) failed\n", failures);
    return failures ? 1 : 0;
}
