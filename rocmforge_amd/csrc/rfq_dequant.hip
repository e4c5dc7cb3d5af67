// Block dequantisation kernels, bit-exact with ROCmForge's CPU decoders.
//
// These kernels are bound by the f32 write stream (4 B out for 0.53-1.13 B in),
// so the mapping is chosen for the stores: one thread decodes 4 consecutive
// elements and issues one 16-byte store; a wavefront writes 1 KiB contiguous.
// Whole blocks go through the fast kernel; anything ragged (element count not
// a multiple of the block, or fewer bytes than the shape needs) goes through a
// bounds-checked per-element kernel that follows the CPU loops' early exits.
//
// Compiled with -ffp-contract=off so no multiply-add is fused (the reference
// never fuses).
#include "rfq_common.hpp"

namespace rfq {
namespace {

// ---- 4 consecutive elements e0..e0+3 (e0 % 4 == 0) of one whole block -------

template <int FMT> __device__ __forceinline__ float4 decode_quad(const uint8_t *blk, int e0);

// src/kernels/quant/q4_0.rs:289-306
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q4_0>(const uint8_t *blk, int e0)
{
    float scale = ld<float>(blk);
    uint32_t w = ld<uint16_t>(blk + 4 + (e0 >> 1));
    float4 r;
    r.x = scale * (float)((int)(w & 15u) - 8);
    r.y = scale * (float)((int)((w >> 4) & 15u) - 8);
    r.z = scale * (float)((int)((w >> 8) & 15u) - 8);
    r.w = scale * (float)((int)((w >> 12) & 15u) - 8);
    return r;
}

// src/kernels/quant/q8_0.rs:55-59
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q8_0>(const uint8_t *blk, int e0)
{
    float scale = ld<float>(blk);
    uint32_t w = ld<uint32_t>(blk + 4 + e0);
    float4 r;
    r.x = ((float)(w & 255u) - 128.0f) * scale;
    r.y = ((float)((w >> 8) & 255u) - 128.0f) * scale;
    r.z = ((float)((w >> 16) & 255u) - 128.0f) * scale;
    r.w = ((float)(w >> 24) - 128.0f) * scale;
    return r;
}

// src/kernels/quant/q4_k.rs:222-268
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q4_K>(const uint8_t *blk, int e0)
{
    int sb = e0 >> 5, i = e0 & 31;
    float scale = f16_bits_to_f32(ld<uint16_t>(blk + 2 * sb));
    float mn = (float)(int8_t)blk[16 + sb];
    uint32_t w = ld<uint16_t>(blk + 32 + 28 * sb + (i >> 1));
    float4 r;
    r.x = mn + (float)(w & 15u) * scale;
    r.y = mn + (float)((w >> 4) & 15u) * scale;
    r.z = mn + (float)((w >> 8) & 15u) * scale;
    r.w = mn + (float)((w >> 12) & 15u) * scale;
    return r;
}

// src/kernels/quant/q6_k.rs:221-261: element i sits at bit 6*i of the stream
// at +32, so four elements starting at a multiple of 4 are exactly 3 bytes.
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q6_K>(const uint8_t *blk, int e0)
{
    float scale = f16_bits_to_f32(ld<uint16_t>(blk + 2 * (e0 >> 4)));
    const uint8_t *p = blk + 32 + 3 * (e0 >> 2);
    uint32_t w = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
    float4 r;
    r.x = (float)sbfe6(w, 0) * scale;
    r.y = (float)sbfe6(w, 6) * scale;
    r.z = (float)sbfe6(w, 12) * scale;
    r.w = (float)sbfe6(w, 18) * scale;
    return r;
}

// src/loader/dequant.rs:53-77: element 2j is the HIGH nibble of byte j.
template <> __device__ __forceinline__ float4 decode_quad<RFQ_MXFP4>(const uint8_t *blk, int e0)
{
    float scale = mx_scale((int)(int8_t)blk[0]);
    uint32_t w = ld<uint16_t>(blk + 1 + (e0 >> 1));
    float4 r;
    r.x = clampf(scale * decode_e2m1((w >> 4) & 15u), -8.0f, 8.0f);
    r.y = clampf(scale * decode_e2m1(w & 15u), -8.0f, 8.0f);
    r.z = clampf(scale * decode_e2m1((w >> 12) & 15u), -8.0f, 8.0f);
    r.w = clampf(scale * decode_e2m1((w >> 8) & 15u), -8.0f, 8.0f);
    return r;
}

// src/loader/dequant.rs:107-127.  With b = the 24 packed bytes and j = e0/4,
// "(u16le[b + (6i)/8] >> (10 - (6i)%8)) & 63" reduces to
//   i=4j  : b[3j+1] >> 2
//   i=4j+1: (b[3j] >> 4) | ((b[3j+1] & 3) << 4)
//   i=4j+2: (b[3j+1] >> 6) | ((b[3j+2] & 15) << 2)
//   i=4j+3: b[3j+3] & 63, which needs byte 24 for j = 7: the reference skips
//           that element, it stays 0.0.
template <> __device__ __forceinline__ float4 decode_quad<RFQ_MXFP6_E2M3>(const uint8_t *blk, int e0)
{
    float scale = mx_scale((int)(int8_t)blk[0]);
    int j = e0 >> 2;
    const uint8_t *b = blk + 1 + 3 * j;
    uint32_t b0 = b[0], b1 = b[1], b2 = b[2];
    float4 r;
    r.x = clampf(scale * decode_e2m3(b1 >> 2), -7.5f, 7.5f);
    r.y = clampf(scale * decode_e2m3((b0 >> 4) | ((b1 & 3u) << 4)), -7.5f, 7.5f);
    r.z = clampf(scale * decode_e2m3((b1 >> 6) | ((b2 & 15u) << 2)), -7.5f, 7.5f);
    r.w = 0.0f;
    if (j < 7) r.w = clampf(scale * decode_e2m3((uint32_t)b[3] & 63u), -7.5f, 7.5f);
    return r;
}

// ---- GGUF file layouts (ggml-quants.c dequantize_row_q4_0 / q8_0 / q4_K / q6_K) ----
// Blocks are only 2-byte aligned; the loads below are byte-exact copies.

template <> __device__ __forceinline__ float4 decode_quad<RFQ_GGUF_Q4_0>(const uint8_t *blk, int e0)
{
    float d = f16_bits_to_f32(ld<uint16_t>(blk));
    uint32_t w = ld<uint32_t>(blk + 2 + (e0 & 15));      // elements j and j + 16 share byte j
    if (e0 & 16) w >>= 4;
    float4 r;
    r.x = (float)((int)(w & 15u) - 8) * d;
    r.y = (float)((int)((w >> 8) & 15u) - 8) * d;
    r.z = (float)((int)((w >> 16) & 15u) - 8) * d;
    r.w = (float)((int)((w >> 24) & 15u) - 8) * d;
    return r;
}

template <> __device__ __forceinline__ float4 decode_quad<RFQ_GGUF_Q8_0>(const uint8_t *blk, int e0)
{
    float d = f16_bits_to_f32(ld<uint16_t>(blk));
    uint32_t w = ld<uint32_t>(blk + 2 + e0);
    float4 r;
    r.x = (float)(int8_t)(w & 255u) * d;
    r.y = (float)(int8_t)((w >> 8) & 255u) * d;
    r.z = (float)(int8_t)((w >> 16) & 255u) * d;
    r.w = (float)(int8_t)(w >> 24) * d;
    return r;
}

template <> __device__ __forceinline__ float4 decode_quad<RFQ_GGUF_Q4_K>(const uint8_t *blk, int e0)
{
    const float d = f16_bits_to_f32(ld<uint16_t>(blk)), dmin = f16_bits_to_f32(ld<uint16_t>(blk + 2));
    const int c = e0 >> 6, h = (e0 >> 5) & 1, l = e0 & 31;   // chunk of 64, nibble half, byte
    const uint32_t sm = gguf_scale_min_k4(2 * c + h, ld<uint32_t>(blk + 4), ld<uint32_t>(blk + 8), ld<uint32_t>(blk + 12));
    const float d1 = d * (float)(sm & 255u), m1 = dmin * (float)(sm >> 8);
    uint32_t w = ld<uint32_t>(blk + 16 + 32 * c + l) >> (4 * h);
    float4 r;
    r.x = d1 * (float)(w & 15u) - m1;
    r.y = d1 * (float)((w >> 8) & 15u) - m1;
    r.z = d1 * (float)((w >> 16) & 15u) - m1;
    r.w = d1 * (float)((w >> 24) & 15u) - m1;
    return r;
}

template <> __device__ __forceinline__ float4 decode_quad<RFQ_GGUF_Q6_K>(const uint8_t *blk, int e0)
{
    const int half = e0 >> 7, t = (e0 >> 5) & 3, l = e0 & 31;   // 128-element half, quarter, byte
    const float d = f16_bits_to_f32(ld<uint16_t>(blk + 208));
    const float sc = (float)(int8_t)blk[192 + 8 * half + 2 * t + (l >> 4)];
    const uint32_t lo = (ld<uint32_t>(blk + 64 * half + 32 * (t & 1) + l) >> (4 * (t >> 1))) & 0x0F0F0F0Fu;
    const uint32_t hi = (ld<uint32_t>(blk + 128 + 32 * half + l) >> (2 * t)) & 0x03030303u;
    const uint32_t q = lo | (hi << 4);
    const float ds = d * sc;
    float4 r;
    r.x = ds * (float)((int)(q & 255u) - 32);
    r.y = ds * (float)((int)((q >> 8) & 255u) - 32);
    r.z = ds * (float)((int)((q >> 16) & 255u) - 32);
    r.w = ds * (float)((int)(q >> 24) - 32);
    return r;
}

// ---- the matmul module's own decoders (src/kernels/matmul/quantized/) -------------

// quantized/q8_0.rs:34-52: two's-complement bytes, scale * q
template <> __device__ __forceinline__ float4 decode_quad<RFQ_MM_Q8_0>(const uint8_t *blk, int e0)
{
    float scale = ld<float>(blk);
    uint32_t w = ld<uint32_t>(blk + 4 + e0);
    float4 r;
    r.x = scale * (float)(int8_t)(w & 255u);
    r.y = scale * (float)(int8_t)((w >> 8) & 255u);
    r.z = scale * (float)(int8_t)((w >> 16) & 255u);
    r.w = scale * (float)(int8_t)(w >> 24);
    return r;
}

// quantized/q4_k.rs:101-143: nibbles of sub-block sb at 32 + 20 * sb, scale through f16_to_f32_cpu
template <> __device__ __forceinline__ float4 decode_quad<RFQ_MM_Q4_K>(const uint8_t *blk, int e0)
{
    int sb = e0 >> 5, i = e0 & 31;
    float scale = f16_bits_to_f32_mm(ld<uint16_t>(blk + 2 * sb));
    float mn = (float)(int8_t)blk[16 + sb];
    uint32_t w = ld<uint16_t>(blk + 32 + 20 * sb + (i >> 1));
    float4 r;
    r.x = mn + (float)(w & 15u) * scale;
    r.y = mn + (float)((w >> 4) & 15u) * scale;
    r.z = mn + (float)((w >> 8) & 15u) * scale;
    r.w = mn + (float)((w >> 12) & 15u) * scale;
    return r;
}

// quantized/q6_k.rs:101-143: the canonical stream, scale through f16_to_f32_cpu
template <> __device__ __forceinline__ float4 decode_quad<RFQ_MM_Q6_K>(const uint8_t *blk, int e0)
{
    float scale = f16_bits_to_f32_mm(ld<uint16_t>(blk + 2 * (e0 >> 4)));
    const uint8_t *p = blk + 32 + 3 * (e0 >> 2);
    uint32_t w = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
    float4 r;
    r.x = (float)sbfe6(w, 0) * scale;
    r.y = (float)sbfe6(w, 6) * scale;
    r.z = (float)sbfe6(w, 12) * scale;
    r.w = (float)sbfe6(w, 18) * scale;
    return r;
}

// The loader's other K types (src/loader/dequant.rs): 256-byte blocks of 16 sub-blocks x 16
// elements, f16 scale at 2 * sub; the codes of a sub-block are an LSB-first bit stream that the
// reference reads through 16-bit windows.  Four consecutive elements never leave a sub-block.

// dequant_q5_k, src/loader/dequant.rs:150-225: i8 min at 32 + sub, 5-bit codes at 48 + 10 * sub
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q5_K>(const uint8_t *blk, int e0)
{
    const int sub = e0 >> 4, bit = (e0 & 15) * 5;
    const float scale = f16_bits_to_f32(ld<uint16_t>(blk + 2 * sub));
    const float mn = (float)(int8_t)blk[32 + sub];
    const uint32_t w = ld<uint32_t>(blk + 48 + 10 * sub + (bit >> 3)) >> (bit & 7);   // 20 bits from bit 0 or 4
    float4 r;
    r.x = mn + (float)(w & 31u) * scale;
    r.y = mn + (float)((w >> 5) & 31u) * scale;
    r.z = mn + (float)((w >> 10) & 31u) * scale;
    r.w = mn + (float)((w >> 15) & 31u) * scale;
    return r;
}

// dequant_q3_k, src/loader/dequant.rs:243-320: two high bits per sub-block at 32 + sub / 4, 3-bit
// codes at 36 + 6 * sub; high bit i is bit 3 of element i (elements 0 and 1 only); (q - 4) * scale
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q3_K>(const uint8_t *blk, int e0)
{
    const int sub = e0 >> 4, i0 = e0 & 15, bit = i0 * 3;
    const float scale = f16_bits_to_f32(ld<uint16_t>(blk + 2 * sub));
    const uint32_t qh = i0 == 0 ? ((uint32_t)blk[32 + (sub >> 2)] >> ((sub & 3) * 2)) & 3u : 0u;
    const uint32_t w = ld<uint16_t>(blk + 36 + 6 * sub + (bit >> 3)) >> (bit & 7);    // 12 bits from bit 0 or 4
    float4 r;
    r.x = ((float)(int)((w & 7u) | ((qh & 1u) << 3)) - 4.0f) * scale;
    r.y = ((float)(int)(((w >> 3) & 7u) | ((qh >> 1) << 3)) - 4.0f) * scale;
    r.z = ((float)(int)((w >> 6) & 7u) - 4.0f) * scale;
    r.w = ((float)(int)((w >> 9) & 7u) - 4.0f) * scale;
    return r;
}

// dequant_q2_k, src/loader/dequant.rs:326-420: f16 min at 32 + 2 * sub, one high bit per sub-block at
// 64 + sub / 8 (bit 2 of element 0 only), 2-bit codes at 68 + 4 * sub; min + q * scale
template <> __device__ __forceinline__ float4 decode_quad<RFQ_Q2_K>(const uint8_t *blk, int e0)
{
    const int sub = e0 >> 4, i0 = e0 & 15;
    const float scale = f16_bits_to_f32(ld<uint16_t>(blk + 2 * sub));
    const float mn = f16_bits_to_f32(ld<uint16_t>(blk + 32 + 2 * sub));
    const uint32_t qh = i0 == 0 ? ((uint32_t)blk[64 + (sub >> 3)] >> (sub & 7)) & 1u : 0u;
    const uint32_t w = blk[68 + 4 * sub + (i0 >> 2)];
    float4 r;
    r.x = mn + (float)((w & 3u) | (qh << 2)) * scale;
    r.y = mn + (float)((w >> 2) & 3u) * scale;
    r.z = mn + (float)((w >> 4) & 3u) * scale;
    r.w = mn + (float)(w >> 6) * scale;
    return r;
}

// 16-byte store of decoded values.  The f32 output is four to eight times the packed input and is
// written once: non-temporal stores keep it from displacing the input stream in the caches
// (Q4_K 14336x4096: 53.7 -> 40.7 us, MXFP4 28672x8192: 232 -> 213 us).
__device__ __forceinline__ void store_quad(float *o, const float4 &v)
{
    typedef float v4f_nt __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(v4f_nt{v.x, v.y, v.z, v.w}, reinterpret_cast<v4f_nt *>(o));
}

template <int FMT, bool ALIGNED16>
__global__ void __launch_bounds__(256)
dequant_blocks_kernel(const uint8_t *__restrict__ in, float *__restrict__ out, size_t n_quads)
{
    constexpr int QPB = Fmt<FMT>::BE / 4;
    size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_quads) return;
    size_t b = t / QPB;
    int e0 = (int)(t % QPB) * 4;
    float4 v = decode_quad<FMT>(in + b * Fmt<FMT>::BB, e0);
    float *o = out + t * 4;
    if (ALIGNED16) {
        store_quad(o, v);
    } else {
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
}

// MXFP4 spends more instructions on decoding a code (zero test, sign, exponent)
// than the store stream leaves room for, so the two values of a code byte come
// from a 256-entry table in LDS, built once per workgroup: entry b holds
// (decode(b >> 4), decode(b & 15)), element 2j being the HIGH nibble of byte j
// (src/loader/dequant.rs:53-77).  What remains per element is the multiply by
// the block's power of two and the clamp.  A workgroup walks MX_LUT_TRIPS
// consecutive chunks of 256 quads so the table is built once per 12 KiB written.
constexpr int MX_LUT_TRIPS = 3;   // measured 1..8, 16 at 28672x8192: 214, 181, 171, 186, 201, 201, 200, 203, 212 us

__device__ __forceinline__ float4 mxfp4_quad_from_table(const float2 *lut, int exponent, uint32_t w)
{
    const float scale = mx_scale(exponent);
    const float2 a = lut[w & 255u], b = lut[w >> 8];
    float4 r;
    r.x = __builtin_amdgcn_fmed3f(scale * a.x, -8.0f, 8.0f);   // (no NaN can arise: clamp == median)
    r.y = __builtin_amdgcn_fmed3f(scale * a.y, -8.0f, 8.0f);
    r.z = __builtin_amdgcn_fmed3f(scale * b.x, -8.0f, 8.0f);
    r.w = __builtin_amdgcn_fmed3f(scale * b.y, -8.0f, 8.0f);
    return r;
}

__global__ void __launch_bounds__(256)
dequant_mxfp4_lut_kernel(const uint8_t *__restrict__ in, float *__restrict__ out, size_t n_quads)
{
    __shared__ float2 lut[256];
    lut[threadIdx.x] = make_float2(decode_e2m1(threadIdx.x >> 4), decode_e2m1(threadIdx.x & 15u));
    __syncthreads();
    // quad t = first + 256 * trip: block (t >> 3) = 32 * MX_LUT_TRIPS * blockIdx.x + (threadIdx.x >> 3) + 32 * trip
    const size_t wg_first = (size_t)blockIdx.x * (256 * MX_LUT_TRIPS);
    const uint8_t *blk0 = in + (wg_first >> 3) * 17 + (threadIdx.x >> 3) * 17;
    const uint32_t code_off = 1u + ((threadIdx.x & 7u) << 1);
    float *o = out + (wg_first + threadIdx.x) * 4;
    if (wg_first + 256 * MX_LUT_TRIPS <= n_quads) {
        // Every load first (constant offsets from one address), then table, scale, clamp, store.
        // One dword per lane and trip: lane j of a block's eight reads bytes 2j .. 2j+3 (its two code
        // bytes are bytes 1 and 2 of the dword; the last lane starts one byte earlier so as not to
        // read past the block), and lane 0's byte 0 is the block's exponent, handed to the other
        // seven through the LDS crossbar -- half the load instructions of a byte and a halfword each.
        const int j = threadIdx.x & 7, last = j == 7;
        const uint8_t *dw_ptr = blk0 + 2 * j - last;
        const int code_shift = 8 + 8 * last;
        const int from_lane0 = (int)((threadIdx.x & 63u & ~7u) << 2);
        uint32_t dw[MX_LUT_TRIPS];
#pragma unroll
        for (int trip = 0; trip < MX_LUT_TRIPS; trip++) dw[trip] = ld<uint32_t>(dw_ptr + trip * 32 * 17);
#pragma unroll
        for (int trip = 0; trip < MX_LUT_TRIPS; trip++) {
            const int ex = (int)(int8_t)(__builtin_amdgcn_ds_bpermute(from_lane0, (int)dw[trip]) & 255);
            store_quad(o + (size_t)trip * 1024, mxfp4_quad_from_table(lut, ex, (dw[trip] >> code_shift) & 0xFFFFu));
        }
    } else {
        for (int trip = 0; trip < MX_LUT_TRIPS; trip++) {
            if (wg_first + threadIdx.x + (size_t)trip * 256 < n_quads) {
                const uint8_t *blk = blk0 + trip * 32 * 17;
                *reinterpret_cast<float4 *>(o + (size_t)trip * 1024) =
                    mxfp4_quad_from_table(lut, (int)(int8_t)blk[0], ld<uint16_t>(blk + code_off));
            }
        }
    }
}

// ---- one element with the CPU loops' bounds behaviour ------------------------

template <int FMT> __device__ float decode_checked(const uint8_t *in, size_t len, size_t idx);

template <> __device__ float decode_checked<RFQ_Q4_0>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 32) * 20;
    if (off + 4 > len) return 0.0f;             // q4_0.rs:273-275
    size_t e = idx % 32, p = off + 4 + e / 2;
    if (p >= len) return 0.0f;                  // q4_0.rs:290-292
    uint32_t q = (e & 1) ? (in[p] >> 4) : (in[p] & 15u);
    return ld<float>(in + off) * (float)((int)q - 8);
}

template <> __device__ float decode_checked<RFQ_Q8_0>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 32) * 36;
    if (off + 4 > len) return 0.0f;             // q8_0.rs:35-37
    size_t p = off + 4 + idx % 32;
    if (p >= len) return 0.0f;                  // q8_0.rs:50-51
    return ((float)in[p] - 128.0f) * ld<float>(in + off);
}

template <> __device__ float decode_checked<RFQ_Q4_K>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 256) * 256;
    if (off + 256 > len) return 0.0f;           // q4_k.rs:208-210
    float4 v = decode_quad<RFQ_Q4_K>(in + off, (int)(idx % 256) & ~3);
    int l = (int)(idx & 3);
    return l == 0 ? v.x : l == 1 ? v.y : l == 2 ? v.z : v.w;
}

template <> __device__ float decode_checked<RFQ_Q6_K>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 256) * 256;
    if (off + 256 > len) return 0.0f;           // q6_k.rs:208-210
    float4 v = decode_quad<RFQ_Q6_K>(in + off, (int)(idx % 256) & ~3);
    int l = (int)(idx & 3);
    return l == 0 ? v.x : l == 1 ? v.y : l == 2 ? v.z : v.w;
}

// (src/loader/dequant.rs:158-160, 251-253, 334-336: a block the input does not hold completely ends the loop)
template <int FMT> __device__ float decode_checked_k256(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 256) * 256;
    if (off + 256 > len) return 0.0f;
    float4 v = decode_quad<FMT>(in + off, (int)(idx % 256) & ~3);
    int l = (int)(idx & 3);
    return l == 0 ? v.x : l == 1 ? v.y : l == 2 ? v.z : v.w;
}
template <> __device__ float decode_checked<RFQ_Q2_K>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_k256<RFQ_Q2_K>(in, len, idx); }
template <> __device__ float decode_checked<RFQ_Q3_K>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_k256<RFQ_Q3_K>(in, len, idx); }
template <> __device__ float decode_checked<RFQ_Q5_K>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_k256<RFQ_Q5_K>(in, len, idx); }

template <> __device__ float decode_checked<RFQ_MXFP4>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 32) * 17;
    if (off + 1 > len) return 0.0f;             // dequant.rs:49-51
    size_t e = idx % 32, p = off + 1 + e / 2;
    if (p >= len) return 0.0f;                  // dequant.rs:59-61
    uint32_t q = (e & 1) ? (in[p] & 15u) : (in[p] >> 4);
    return clampf(mx_scale((int)(int8_t)in[off]) * decode_e2m1(q), -8.0f, 8.0f);
}

template <> __device__ float decode_checked<RFQ_MXFP6_E2M3>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 32) * 25;
    if (off + 1 > len) return 0.0f;             // dequant.rs:93-95
    size_t avail = len - (off + 1);
    size_t plen = avail < 24 ? avail : 24;      // dequant.rs:102-104
    size_t i = idx % 32;
    uint32_t bit_offset = (uint32_t)((i * 6) % 8);
    size_t bi = (i * 6) / 8;
    if (bi + 1 >= plen) return 0.0f;            // dequant.rs:117
    const uint8_t *pd = in + off + 1;
    uint32_t combined = ((uint32_t)pd[bi + 1] << 8) | pd[bi];
    uint32_t q = (combined >> (10u - bit_offset)) & 63u;
    return clampf(mx_scale((int)(int8_t)in[off]) * decode_e2m3(q), -7.5f, 7.5f);
}

// The matmul module's decoders reach into an incomplete last block as far as its bytes go.
template <> __device__ float decode_checked<RFQ_MM_Q8_0>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 32) * 36;
    if (off + 4 > len) return 0.0f;             // quantized/q8_0.rs:24-26
    size_t p = off + 4 + idx % 32;
    if (p >= len) return 0.0f;                  // q8_0.rs:42-44
    return ld<float>(in + off) * (float)(int8_t)in[p];
}

template <> __device__ float decode_checked<RFQ_MM_Q4_K>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 256) * 256;
    if (off + 32 > len) return 0.0f;            // quantized/q4_k.rs:96-98 (scales and mins are then present)
    int e = (int)(idx % 256), sb = e >> 5, i = e & 31;
    size_t qi = off + 32 + 20 * sb + (i >> 1);
    if (qi + 1 >= len) return 0.0f;             // q4_k.rs:135-137
    uint32_t q = (i & 1) ? (in[qi] >> 4) : (in[qi] & 15u);
    float scale = f16_bits_to_f32_mm(ld<uint16_t>(in + off + 2 * sb));
    return (float)(int8_t)in[off + 16 + sb] + (float)q * scale;
}

template <> __device__ float decode_checked<RFQ_MM_Q6_K>(const uint8_t *in, size_t len, size_t idx)
{
    size_t off = (idx / 256) * 256;
    if (off + 32 > len) return 0.0f;            // quantized/q6_k.rs:96-98
    int i = (int)(idx % 256);
    size_t qi = off + 32 + (size_t)(i * 6) / 8;
    if (qi + 1 >= len) return 0.0f;             // q6_k.rs:128-130
    uint32_t combined = (uint32_t)in[qi] | ((uint32_t)in[qi + 1] << 8);
    int q = (int)((combined >> ((i * 6) % 8)) & 63u);
    float scale = f16_bits_to_f32_mm(ld<uint16_t>(in + off + 2 * (i >> 4)));
    return (float)(q >= 32 ? q - 64 : q) * scale;
}

// GGUF layouts: a block the input does not hold completely decodes to 0.0.
template <int FMT> __device__ float decode_checked_whole_blocks(const uint8_t *in, size_t len, size_t idx)
{
    const size_t b = idx / Fmt<FMT>::BE;
    if ((b + 1) * Fmt<FMT>::BB > len) return 0.0f;
    const int e = (int)(idx % Fmt<FMT>::BE);
    const float4 q = decode_quad<FMT>(in + b * Fmt<FMT>::BB, e & ~3);
    return (e & 3) == 0 ? q.x : ((e & 3) == 1 ? q.y : ((e & 3) == 2 ? q.z : q.w));
}
template <> __device__ float decode_checked<RFQ_GGUF_Q4_0>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_whole_blocks<RFQ_GGUF_Q4_0>(in, len, idx); }
template <> __device__ float decode_checked<RFQ_GGUF_Q8_0>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_whole_blocks<RFQ_GGUF_Q8_0>(in, len, idx); }
template <> __device__ float decode_checked<RFQ_GGUF_Q4_K>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_whole_blocks<RFQ_GGUF_Q4_K>(in, len, idx); }
template <> __device__ float decode_checked<RFQ_GGUF_Q6_K>(const uint8_t *in, size_t len, size_t idx) { return decode_checked_whole_blocks<RFQ_GGUF_Q6_K>(in, len, idx); }

template <int FMT>
__global__ void __launch_bounds__(256)
dequant_checked_kernel(const uint8_t *__restrict__ in, size_t len, float *__restrict__ out, size_t first, size_t n)
{
    size_t idx = first + (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx < n) out[idx] = decode_checked<FMT>(in, len, idx);
}

// ---- GetRows: out[i, :] = dequant(row tokens[i]) -----------------------------
//
// The reference gathers embedding rows from an f32 table with one device copy
// per token after copying the token ids to the host
// (src/ggml/hip_backend/ops/get_rows.rs:6-53, op_dispatch.rs:70-100).  Here the
// ids are read on the device and the table may stay packed: thread t decodes
// quad t % (n_embd/4) of output row t / (n_embd/4).  An id outside the table
// leaves its row zero and records 1 + the row's index in *status (the smallest
// such index wins), where the reference returns "Token ID exceeds vocab size".
template <int FMT>
__global__ void __launch_bounds__(256)
get_rows_kernel(const uint8_t *__restrict__ table, const uint32_t *__restrict__ tokens, float *__restrict__ out,
                int n_vocab, int quads_per_row, size_t n_quads, int *status)
{
    constexpr int QPB = Fmt<FMT>::BE / 4;
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_quads) return;
    const size_t i = t / quads_per_row;
    const int qd = (int)(t % quads_per_row);
    const uint32_t id = tokens[i];
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (id < (uint32_t)n_vocab) {
        const size_t blk = (size_t)id * (quads_per_row / QPB) + qd / QPB;
        v = decode_quad<FMT>(table + blk * Fmt<FMT>::BB, (qd % QPB) * 4);
    } else if (status != nullptr && qd == 0) {
        atomicMin(reinterpret_cast<unsigned *>(status), (unsigned)i + 1u);
    }
    *reinterpret_cast<float4 *>(out + t * 4) = v;
}

__global__ void __launch_bounds__(256)
get_rows_f32_kernel(const float *__restrict__ table, const uint32_t *__restrict__ tokens, float *__restrict__ out,
                    int n_vocab, int quads_per_row, size_t n_quads, int *status)
{
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_quads) return;
    const size_t i = t / quads_per_row;
    const int qd = (int)(t % quads_per_row);
    const uint32_t id = tokens[i];
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (id < (uint32_t)n_vocab) {
        v = *reinterpret_cast<const float4 *>(table + ((size_t)id * quads_per_row + qd) * 4);
    } else if (status != nullptr && qd == 0) {
        atomicMin(reinterpret_cast<unsigned *>(status), (unsigned)i + 1u);
    }
    *reinterpret_cast<float4 *>(out + t * 4) = v;
}

// *status = "no bad id yet" (all ones), folded to 0 after the gather.
__global__ void get_rows_status_kernel(int *status, int phase)
{
    if (phase == 0) *status = -1;
    else if (*status == -1) *status = 0;
}

template <int FMT>
int run_get_rows(const uint8_t *table, const uint32_t *tokens, float *out, int n_vocab, int n_embd, int n_tokens,
                 int *status, hipStream_t s)
{
    const size_t n_quads = (size_t)n_tokens * (n_embd / 4);
    const size_t grid = (n_quads + 255) / 256;
    if (grid > 0x7fffffffu) return fail(RFQ_E_SIZE, "rfq_get_rows: %d rows of %d exceed one launch", n_tokens, n_embd);
    hipLaunchKernelGGL((get_rows_kernel<FMT>), dim3((unsigned)grid), dim3(256), 0, s, table, tokens, out, n_vocab,
                       n_embd / 4, n_quads, status);
    RFQ_LAUNCH_CHECK("get_rows_kernel");
    return RFQ_OK;
}

template <int FMT>
int run(const uint8_t *d_in, size_t in_bytes, float *d_out, size_t n, hipStream_t s)
{
    constexpr size_t BE = Fmt<FMT>::BE, BB = Fmt<FMT>::BB;
    size_t full = n / BE;
    if (in_bytes / BB < full) full = in_bytes / BB;
    size_t n_quads = full * (BE / 4);
    if (n_quads) {
        size_t grid = (n_quads + 255) / 256;
        if (grid > 0x7fffffffu) return fail(RFQ_E_SIZE, "rfq_dequant: %zu elements exceed one launch", n);
        if (FMT == RFQ_MXFP4 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0)
            hipLaunchKernelGGL(dequant_mxfp4_lut_kernel, dim3((unsigned)((grid + MX_LUT_TRIPS - 1) / MX_LUT_TRIPS)), dim3(256), 0,
                               s, d_in, d_out, n_quads);
        else if ((reinterpret_cast<uintptr_t>(d_out) & 15u) == 0)
            hipLaunchKernelGGL((dequant_blocks_kernel<FMT, true>), dim3((unsigned)grid), dim3(256), 0, s, d_in, d_out, n_quads);
        else
            hipLaunchKernelGGL((dequant_blocks_kernel<FMT, false>), dim3((unsigned)grid), dim3(256), 0, s, d_in, d_out, n_quads);
        RFQ_LAUNCH_CHECK("dequant_blocks_kernel");
    }
    size_t first = full * BE;
    if (first < n) {
        size_t grid = (n - first + 255) / 256;
        if (grid > 0x7fffffffu) return fail(RFQ_E_SIZE, "rfq_dequant: ragged tail of %zu elements exceeds one launch", n - first);
        // (GGUF layouts decode whole blocks only: everything past the last whole block is 0.0)
        const size_t reach = (FMT >= RFQ_GGUF_Q4_0 && FMT < RFQ_MM_Q8_0) ? full * BB : in_bytes;
        hipLaunchKernelGGL((dequant_checked_kernel<FMT>), dim3((unsigned)grid), dim3(256), 0, s, d_in, reach, d_out, first, n);
        RFQ_LAUNCH_CHECK("dequant_checked_kernel");
    }
    return RFQ_OK;
}

// ---- the orientation the reference computes: y[j] = sum_l x[l] * Wd[l * n + j] -----------
//
// Wd is the packed stream decoded as one flat array of n * k elements (blocks run along j):
// kernels/q4_0_matmul.hip:207 (weight_linear_idx = k_idx * n + col) and
// matmul_q4_0_cpu_fallback + cpu_matmul_f32 (src/kernels/matmul/quantized/q4_0.rs:274-311,
// src/tensor/matmul.rs:219-233).  A thread owns VEC consecutive columns (4 when n is a multiple of 4: a
// decoded quad never straddles two rows of Wd then; else 1) and walks the rows l of its split, so a
// wavefront reads consecutive bytes of one row of Wd per step and the stream is read once.  The k rows are
// split over blockIdx.y; split s writes its partial sums to part[s * n + j], and a second kernel adds the
// splits in ascending order (fixed summation order: the result does not change from run to run).
template <int FMT, int VEC>
__global__ void __launch_bounds__(256)
gemv_kn_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ part, int n, int k,
               int rows_per_split)
{
    constexpr size_t BE = Fmt<FMT>::BE, BB = Fmt<FMT>::BB;
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int groups = VEC == 4 ? n / 4 : n;
    if (c >= groups) return;
    const int l0 = blockIdx.y * rows_per_split;
    int l1 = l0 + rows_per_split;
    if (l1 > k) l1 = k;
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    size_t e = (size_t)l0 * n + (size_t)c * VEC;
#pragma unroll 4
    for (int l = l0; l < l1; l++, e += n) {
        const int eo = (int)(e % BE);
        const float4 v = decode_quad<FMT>(w + (e / BE) * BB, eo & ~3);
        const float xl = x[l];
        if (VEC == 4) {
            acc.x = __builtin_fmaf(xl, v.x, acc.x);
            acc.y = __builtin_fmaf(xl, v.y, acc.y);
            acc.z = __builtin_fmaf(xl, v.z, acc.z);
            acc.w = __builtin_fmaf(xl, v.w, acc.w);
        } else {
            const int r = eo & 3;
            acc.x = __builtin_fmaf(xl, r == 0 ? v.x : (r == 1 ? v.y : (r == 2 ? v.z : v.w)), acc.x);
        }
    }
    float *o = part + (size_t)blockIdx.y * n + (size_t)c * VEC;
    o[0] = acc.x;
    if (VEC == 4) { o[1] = acc.y; o[2] = acc.z; o[3] = acc.w; }
}

// The same contraction for the reference's own four layouts when n is a multiple of 32: a lane owns one unit of 32
// consecutive columns and fetches it with one wide load per row of Wd (16 to 32 bytes plus the scale) instead of
// eight quads of two or three small loads each; what the 32 values of a unit share (a minimum, a code offset) is
// summed once per row instead of per value.  The four
// wavefronts of a workgroup take the rows l0 + w, l0 + w + 4, ... of the split and add their 32 sums per lane
// through LDS in a fixed order.
template <int FMT> struct KnUnit;

// add(xl, acc, off): acc[i] += xl * (the part of value i that varies with i); off collects what all 32 values of the
// unit share (the Q4_K minimum, the -8 and -128 of the code offsets), times xl; finish() puts it back.
template <> struct KnUnit<RFQ_Q4_0> {                   // src/kernels/quant/q4_0.rs:289-306: scale * (nibble - 8)
    float scale; uint4 q;
    __device__ __forceinline__ void load(const uint8_t *w, size_t u)
    {
        const uint8_t *blk = w + u * 20;
        scale = ld<float>(blk);
        q = ld<uint4>(blk + 4);
    }
    __device__ __forceinline__ void add(float xl, float (&acc)[32], float &off) const
    {
        const float xs = xl * scale;
        off = __builtin_fmaf(-8.0f, xs, off);
        // nibbles 0, 2, 4, 6 of a dword become the bytes of one register, 1, 3, 5, 7 of another: a byte converts to
        // float in one instruction
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t lo = (&q.x)[d] & 0x0F0F0F0Fu, hi = ((&q.x)[d] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                acc[8 * d + 2 * b] = __builtin_fmaf((float)((lo >> (8 * b)) & 255u), xs, acc[8 * d + 2 * b]);
                acc[8 * d + 2 * b + 1] = __builtin_fmaf((float)((hi >> (8 * b)) & 255u), xs, acc[8 * d + 2 * b + 1]);
            }
        }
    }
};

template <> struct KnUnit<RFQ_Q8_0> {                   // src/kernels/quant/q8_0.rs:55-59: (byte - 128) * scale
    float scale; uint4 q0, q1;
    __device__ __forceinline__ void load(const uint8_t *w, size_t u)
    {
        const uint8_t *blk = w + u * 36;
        scale = ld<float>(blk);
        q0 = ld<uint4>(blk + 4);
        q1 = ld<uint4>(blk + 20);
    }
    __device__ __forceinline__ void add(float xl, float (&acc)[32], float &off) const
    {
        const float xs = xl * scale;
        off = __builtin_fmaf(-128.0f, xs, off);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const uint32_t d = i < 16 ? (&q0.x)[i >> 2] : (&q1.x)[(i - 16) >> 2];
            acc[i] = __builtin_fmaf((float)((d >> (8 * (i & 3))) & 255u), xs, acc[i]);
        }
    }
};

template <> struct KnUnit<RFQ_Q4_K> {                   // src/kernels/quant/q4_k.rs:222-268: min + nibble * scale
    float scale, mn; uint4 q;
    __device__ __forceinline__ void load(const uint8_t *w, size_t u)
    {
        const uint8_t *blk = w + (u >> 3) * 256;
        const int sb = (int)(u & 7);
        scale = f16_bits_to_f32(ld<uint16_t>(blk + 2 * sb));
        mn = (float)(int8_t)blk[16 + sb];
        q = ld<uint4>(blk + 32 + 28 * sb);
    }
    __device__ __forceinline__ void add(float xl, float (&acc)[32], float &off) const
    {
        const float xs = xl * scale;
        off = __builtin_fmaf(xl, mn, off);
        // nibbles 0, 2, 4, 6 of a dword become the bytes of one register, 1, 3, 5, 7 of another: a byte converts to
        // float in one instruction
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t lo = (&q.x)[d] & 0x0F0F0F0Fu, hi = ((&q.x)[d] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                acc[8 * d + 2 * b] = __builtin_fmaf((float)((lo >> (8 * b)) & 255u), xs, acc[8 * d + 2 * b]);
                acc[8 * d + 2 * b + 1] = __builtin_fmaf((float)((hi >> (8 * b)) & 255u), xs, acc[8 * d + 2 * b + 1]);
            }
        }
    }
};

template <> struct KnUnit<RFQ_Q6_K> {                   // src/kernels/quant/q6_k.rs:221-261: signed 6-bit code * scale of its 16
    uint32_t sc2; uint32_t q[6];
    __device__ __forceinline__ void load(const uint8_t *w, size_t u)
    {
        const uint8_t *blk = w + (u >> 3) * 256;
        const int g = (int)(u & 7);
        sc2 = ld<uint32_t>(blk + 4 * g);
        const uint2 a = ld<uint2>(blk + 32 + 24 * g);
        const uint4 b = ld<uint4>(blk + 32 + 24 * g + 8);
        q[0] = a.x; q[1] = a.y; q[2] = b.x; q[3] = b.y; q[4] = b.z; q[5] = b.w;
    }
    __device__ __forceinline__ void add(float xl, float (&acc)[32], float &) const
    {
        const float xs0 = xl * f16_bits_to_f32((uint16_t)(sc2 & 0xFFFFu)), xs1 = xl * f16_bits_to_f32((uint16_t)(sc2 >> 16));
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const int bit = 6 * i, d = bit >> 5, sh = bit & 31;
            const uint32_t lo = q[d] >> sh;
            const uint32_t v = sh > 26 ? (lo | (q[d + 1] << (32 - sh))) : lo;     // a code that straddles two dwords
            acc[i] = __builtin_fmaf((float)sbfe6(v, 0), i < 16 ? xs0 : xs1, acc[i]);
        }
    }
};

template <int FMT>
__global__ void __launch_bounds__(256)
gemv_kn_unit_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ part, int n, int k,
                    int rows_per_split)
{
    __shared__ float red[4 * 32 * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int units_per_row = n >> 5;
    const int c = blockIdx.x * 64 + lane;
    const bool live = c < units_per_row;
    const int cc = live ? c : units_per_row - 1;
    const int l0 = blockIdx.y * rows_per_split;
    int l1 = l0 + rows_per_split;
    if (l1 > k) l1 = k;
    float acc[32], off = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) acc[i] = 0.0f;
    // eight rows per trip: every load of the trip is issued before the first value is used (rows past the split's
    // end repeat its last row with x taken as 0)
    for (int lb = l0 + wave; lb < l1; lb += 32) {
        KnUnit<FMT> un[8];
        float xl[8];
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const int l = lb + 4 * r, lc = l < l1 ? l : l1 - 1;
            un[r].load(w, (size_t)lc * units_per_row + cc);
            xl[r] = l < l1 ? x[lc] : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < 8; r++) un[r].add(xl[r], acc, off);
    }
#pragma unroll
    for (int i = 0; i < 32; i++) red[(wave * 32 + i) * 64 + lane] = acc[i] + off;
    __syncthreads();
    if (wave == 0 && live) {
        float *o = part + (size_t)blockIdx.y * n + (size_t)c * 32;
#pragma unroll
        for (int i = 0; i < 32; i++)
            o[i] = ((red[i * 64 + lane] + red[(32 + i) * 64 + lane]) + red[(64 + i) * 64 + lane]) + red[(96 + i) * 64 + lane];
    }
}

// 64 columns per workgroup; wavefront g adds the splits g, g + 4, ... in ascending order and the four sums are
// added in a fixed order: the result does not depend on timing.
__global__ void __launch_bounds__(256)
gemv_kn_reduce_kernel(const float *__restrict__ part, float *__restrict__ y, int n, int splits)
{
    __shared__ float red[4][64];
    const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int j = blockIdx.x * 64 + lane;
    float sum = 0.0f;
    if (j < n) {
#pragma unroll 8
        for (int s = g; s < splits; s += 4) sum += part[(size_t)s * n + j];
    }
    red[g][lane] = sum;
    __syncthreads();
    if (g == 0 && j < n) y[j] = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
}

constexpr size_t KN_PART_MAX = (size_t)8 << 20;   // bytes of partial sums at most

template <int FMT> struct HasKnUnit { static constexpr bool value = FMT == RFQ_Q4_0 || FMT == RFQ_Q8_0 || FMT == RFQ_Q4_K || FMT == RFQ_Q6_K; };

template <int FMT>
int run_gemv_kn_units(const uint8_t *w, const float *x, float *y, int n, int k, hipStream_t s)
{
    const int bx = (n / 32 + 63) / 64;
    // about four workgroups per CU, at least 16 rows per split (four per wavefront), partial sums within KN_PART_MAX
    int splits = (4 * device_cu_count() + bx - 1) / bx;
    if (splits > k / 16) splits = k / 16;
    const size_t by_bytes = KN_PART_MAX / ((size_t)n * 4);
    if ((size_t)splits > by_bytes) splits = (int)by_bytes;
    if (splits < 1) splits = 1;
    if (splits > 65535) splits = 65535;
    const int rows_per_split = (k + splits - 1) / splits;
    splits = (k + rows_per_split - 1) / rows_per_split;
    float *part = y;
    if (splits > 1) {
        uint8_t *tmp = nullptr;
        bool transient = false;
        if (int rc = workspace(s, (size_t)splits * n * 4, &tmp, &transient)) return rc;   // (never transient: <= 8 MiB)
        part = reinterpret_cast<float *>(tmp);
    }
    hipLaunchKernelGGL((gemv_kn_unit_kernel<FMT>), dim3(bx, splits), dim3(256), 0, s, w, x, part, n, k, rows_per_split);
    RFQ_LAUNCH_CHECK("gemv_kn_unit_kernel");
    if (splits > 1) {
        hipLaunchKernelGGL(gemv_kn_reduce_kernel, dim3((n + 63) / 64), dim3(256), 0, s, part, y, n, splits);
        RFQ_LAUNCH_CHECK("gemv_kn_reduce_kernel");
    }
    return RFQ_OK;
}

template <int FMT>
int run_gemv_kn(const uint8_t *w, const float *x, float *y, int n, int k, hipStream_t s)
{
    if constexpr (HasKnUnit<FMT>::value) {
        if (n % 32 == 0 && (reinterpret_cast<uintptr_t>(w) & 3u) == 0) return run_gemv_kn_units<FMT>(w, x, y, n, k, s);
    }
    const bool vec = n % 4 == 0;
    const int groups = vec ? n / 4 : n;
    const int bx = (groups + 255) / 256;
    // about four workgroups per CU, at least 16 rows per split, partial sums within KN_PART_MAX
    int splits = (4 * device_cu_count() + bx - 1) / bx;
    if (splits > k / 16) splits = k / 16;
    const size_t by_bytes = KN_PART_MAX / ((size_t)n * 4);
    if ((size_t)splits > by_bytes) splits = (int)by_bytes;
    if (splits < 1) splits = 1;
    if (splits > 65535) splits = 65535;
    const int rows_per_split = (k + splits - 1) / splits;
    splits = (k + rows_per_split - 1) / rows_per_split;
    float *part = y;
    if (splits > 1) {
        uint8_t *tmp = nullptr;
        bool transient = false;
        if (int rc = workspace(s, (size_t)splits * n * 4, &tmp, &transient)) return rc;   // (never transient: <= 8 MiB)
        part = reinterpret_cast<float *>(tmp);
    }
    if (vec) hipLaunchKernelGGL((gemv_kn_kernel<FMT, 4>), dim3(bx, splits), dim3(256), 0, s, w, x, part, n, k, rows_per_split);
    else hipLaunchKernelGGL((gemv_kn_kernel<FMT, 1>), dim3(bx, splits), dim3(256), 0, s, w, x, part, n, k, rows_per_split);
    RFQ_LAUNCH_CHECK("gemv_kn_kernel");
    if (splits > 1) {
        hipLaunchKernelGGL(gemv_kn_reduce_kernel, dim3((n + 63) / 64), dim3(256), 0, s, part, y, n, splits);
        RFQ_LAUNCH_CHECK("gemv_kn_reduce_kernel");
    }
    return RFQ_OK;
}

// ---- neighbours of the matmul in a decoder layer --------------------------------
//
// RMSNorm (kernels/rms_norm.hip:40-84; CPU statement src/mlp/rms_norm_tests.rs:44-73):
// out[r, j] = (x[r, j] / sqrt(mean_j x[r, j]^2 + eps)) * weight[j].  One workgroup
// per row; the row is read twice (the second read is served by the cache).
// SRC_FMT != 0 decodes the row from packed blocks instead of reading f32
// (fused_q4_0_rmsnorm, src/ggml/hip_backend/ops/fused_ops.rs:149-160, for every format).

__device__ __forceinline__ float block_sum_256(float v, float *lds4)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
    __syncthreads();
    return (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
}

template <int SRC_FMT> __device__ __forceinline__ float4 norm_src_quad(const void *row, int q)
{
    if constexpr (SRC_FMT == RFQ_TABLE_F32) {
        return *(reinterpret_cast<const float4 *>(row) + q);
    } else {
        constexpr int QPB = Fmt<SRC_FMT>::BE / 4;
        return decode_quad<SRC_FMT>(static_cast<const uint8_t *>(row) + (size_t)(q / QPB) * Fmt<SRC_FMT>::BB, (q % QPB) * 4);
    }
}

template <int SRC_FMT>
__global__ void __launch_bounds__(256)
rms_norm_kernel(const void *__restrict__ x, size_t row_stride_bytes, const float *__restrict__ weight,
                float *__restrict__ out, int hidden, float eps)
{
    __shared__ float red[4];
    const void *row = static_cast<const uint8_t *>(x) + (size_t)blockIdx.x * row_stride_bytes;
    float *o = out + (size_t)blockIdx.x * hidden;
    const int quads = hidden >> 2;
    float ss = 0.0f;
    for (int q = threadIdx.x; q < quads; q += 256) {
        float4 v = norm_src_quad<SRC_FMT>(row, q);
        ss += v.x * v.x; ss += v.y * v.y; ss += v.z * v.z; ss += v.w * v.w;
    }
    const float total = block_sum_256(ss, red);
    const float rms = sqrtf(total / (float)hidden + eps);
    for (int q = threadIdx.x; q < quads; q += 256) {
        float4 v = norm_src_quad<SRC_FMT>(row, q);
        float4 w = *(reinterpret_cast<const float4 *>(weight) + q);
        float4 r;
        r.x = (v.x / rms) * w.x; r.y = (v.y / rms) * w.y; r.z = (v.z / rms) * w.z; r.w = (v.w / rms) * w.w;
        *(reinterpret_cast<float4 *>(o) + q) = r;
    }
}

// SwiGLU as the reference defines it (kernels/swiglu.hip:40-62): the activation
// is applied to the UP projection, out = gate * (up * 1 / (1 + exp(-up))).
__global__ void __launch_bounds__(256)
swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up, float *__restrict__ out, size_t total)
{
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float u = up[i];
    float sigmoid_up = 1.0f / (1.0f + expf(-u));
    out[i] = gate[i] * (u * sigmoid_up);
}

template <int SRC_FMT>
int run_rms_norm(const void *x, size_t row_stride_bytes, const float *weight, float *out, int rows, int hidden, float eps,
                 hipStream_t s)
{
    hipLaunchKernelGGL((rms_norm_kernel<SRC_FMT>), dim3((unsigned)rows), dim3(256), 0, s, x, row_stride_bytes, weight, out,
                       hidden, eps);
    RFQ_LAUNCH_CHECK("rms_norm_kernel");
    return RFQ_OK;
}

} // namespace

int launch_rms_norm(int src_fmt, const void *d_x, const float *d_weight, float *d_out, int rows, int hidden, float eps,
                    hipStream_t s)
{
    if (rows == 0) return RFQ_OK;
    const int be = src_fmt == RFQ_TABLE_F32 ? 4 : fmt_block_elems(src_fmt);
    const size_t stride = src_fmt == RFQ_TABLE_F32 ? (size_t)hidden * 4 : (size_t)(hidden / be) * fmt_block_bytes(src_fmt);
    switch (canonical_format(src_fmt)) {
    case RFQ_TABLE_F32: return run_rms_norm<RFQ_TABLE_F32>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_Q4_0: return run_rms_norm<RFQ_Q4_0>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_Q8_0: return run_rms_norm<RFQ_Q8_0>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_Q4_K: return run_rms_norm<RFQ_Q4_K>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_Q6_K: return run_rms_norm<RFQ_Q6_K>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_MXFP4: return run_rms_norm<RFQ_MXFP4>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_MXFP6_E2M3: return run_rms_norm<RFQ_MXFP6_E2M3>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_GGUF_Q4_0: return run_rms_norm<RFQ_GGUF_Q4_0>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_GGUF_Q8_0: return run_rms_norm<RFQ_GGUF_Q8_0>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_GGUF_Q4_K: return run_rms_norm<RFQ_GGUF_Q4_K>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    case RFQ_GGUF_Q6_K: return run_rms_norm<RFQ_GGUF_Q6_K>(d_x, stride, d_weight, d_out, rows, hidden, eps, s);
    default: return fail(RFQ_E_BADARG, "rms_norm: unknown source format %d", src_fmt);
    }
}

int launch_swiglu(const float *d_gate, const float *d_up, float *d_out, size_t total, hipStream_t s)
{
    if (total == 0) return RFQ_OK;
    const size_t grid = (total + 255) / 256;
    if (grid > 0x7fffffffu) return fail(RFQ_E_SIZE, "rfq_swiglu: %zu elements exceed one launch", total);
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)grid), dim3(256), 0, s, d_gate, d_up, d_out, total);
    RFQ_LAUNCH_CHECK("swiglu_kernel");
    return RFQ_OK;
}

int launch_dequant(int fmt, const uint8_t *d_in, size_t in_bytes, float *d_out, size_t n, hipStream_t s)
{
    switch (canonical_format(fmt)) {
    case RFQ_Q4_0: return run<RFQ_Q4_0>(d_in, in_bytes, d_out, n, s);
    case RFQ_Q8_0: return run<RFQ_Q8_0>(d_in, in_bytes, d_out, n, s);
    case RFQ_Q4_K: return run<RFQ_Q4_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_Q6_K: return run<RFQ_Q6_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_Q2_K: return run<RFQ_Q2_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_Q3_K: return run<RFQ_Q3_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_Q5_K: return run<RFQ_Q5_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_MXFP4: return run<RFQ_MXFP4>(d_in, in_bytes, d_out, n, s);
    case RFQ_MXFP6_E2M3: return run<RFQ_MXFP6_E2M3>(d_in, in_bytes, d_out, n, s);
    case RFQ_GGUF_Q4_0: return run<RFQ_GGUF_Q4_0>(d_in, in_bytes, d_out, n, s);
    case RFQ_GGUF_Q8_0: return run<RFQ_GGUF_Q8_0>(d_in, in_bytes, d_out, n, s);
    case RFQ_GGUF_Q4_K: return run<RFQ_GGUF_Q4_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_GGUF_Q6_K: return run<RFQ_GGUF_Q6_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_MM_Q8_0: return run<RFQ_MM_Q8_0>(d_in, in_bytes, d_out, n, s);
    case RFQ_MM_Q4_K: return run<RFQ_MM_Q4_K>(d_in, in_bytes, d_out, n, s);
    case RFQ_MM_Q6_K: return run<RFQ_MM_Q6_K>(d_in, in_bytes, d_out, n, s);
    default: return fail(RFQ_E_BADARG, "rfq_dequant: unknown format %d", fmt);
    }
}

int launch_gemv_kn(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int n, int k, hipStream_t s)
{
    switch (canonical_format(fmt)) {
    case RFQ_Q4_0: return run_gemv_kn<RFQ_Q4_0>(d_w, d_x, d_y, n, k, s);
    case RFQ_Q8_0: return run_gemv_kn<RFQ_Q8_0>(d_w, d_x, d_y, n, k, s);
    case RFQ_Q4_K: return run_gemv_kn<RFQ_Q4_K>(d_w, d_x, d_y, n, k, s);
    case RFQ_Q6_K: return run_gemv_kn<RFQ_Q6_K>(d_w, d_x, d_y, n, k, s);
    case RFQ_MXFP4: return run_gemv_kn<RFQ_MXFP4>(d_w, d_x, d_y, n, k, s);
    case RFQ_MXFP6_E2M3: return run_gemv_kn<RFQ_MXFP6_E2M3>(d_w, d_x, d_y, n, k, s);
    case RFQ_GGUF_Q4_0: return run_gemv_kn<RFQ_GGUF_Q4_0>(d_w, d_x, d_y, n, k, s);
    case RFQ_GGUF_Q8_0: return run_gemv_kn<RFQ_GGUF_Q8_0>(d_w, d_x, d_y, n, k, s);
    case RFQ_GGUF_Q4_K: return run_gemv_kn<RFQ_GGUF_Q4_K>(d_w, d_x, d_y, n, k, s);
    case RFQ_GGUF_Q6_K: return run_gemv_kn<RFQ_GGUF_Q6_K>(d_w, d_x, d_y, n, k, s);
    case RFQ_MM_Q8_0: return run_gemv_kn<RFQ_MM_Q8_0>(d_w, d_x, d_y, n, k, s);
    case RFQ_MM_Q4_K: return run_gemv_kn<RFQ_MM_Q4_K>(d_w, d_x, d_y, n, k, s);
    case RFQ_MM_Q6_K: return run_gemv_kn<RFQ_MM_Q6_K>(d_w, d_x, d_y, n, k, s);
    default: return fail(RFQ_E_BADARG, "rfq_gemv_kn: unknown format %d", fmt);
    }
}

int launch_get_rows(int fmt, const void *d_table, int n_vocab, int n_embd, const uint32_t *d_tokens, int n_tokens,
                    float *d_out, int *d_status, hipStream_t s)
{
    if (d_status) {
        hipLaunchKernelGGL(get_rows_status_kernel, dim3(1), dim3(1), 0, s, d_status, 0);
        RFQ_LAUNCH_CHECK("get_rows_status_kernel");
    }
    int rc;
    const uint8_t *table = static_cast<const uint8_t *>(d_table);
    switch (fmt) {
    case RFQ_TABLE_F32: {
        const size_t n_quads = (size_t)n_tokens * (n_embd / 4);
        const size_t grid = (n_quads + 255) / 256;
        if (grid > 0x7fffffffu) return fail(RFQ_E_SIZE, "rfq_get_rows: %d rows of %d exceed one launch", n_tokens, n_embd);
        hipLaunchKernelGGL(get_rows_f32_kernel, dim3((unsigned)grid), dim3(256), 0, s, static_cast<const float *>(d_table),
                           d_tokens, d_out, n_vocab, n_embd / 4, n_quads, d_status);
        hipError_t e = hipGetLastError();
        rc = e == hipSuccess ? RFQ_OK : hip_fail(e, "get_rows_f32_kernel");
        break;
    }
    case RFQ_Q4_0: rc = run_get_rows<RFQ_Q4_0>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_Q8_0: rc = run_get_rows<RFQ_Q8_0>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_Q4_K: rc = run_get_rows<RFQ_Q4_K>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_Q6_K: rc = run_get_rows<RFQ_Q6_K>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_MXFP4: rc = run_get_rows<RFQ_MXFP4>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_MXFP6_E2M3: case RFQ_MXFP6_E3M2:
        rc = run_get_rows<RFQ_MXFP6_E2M3>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_GGUF_Q4_0: rc = run_get_rows<RFQ_GGUF_Q4_0>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_GGUF_Q8_0: rc = run_get_rows<RFQ_GGUF_Q8_0>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_GGUF_Q4_K: rc = run_get_rows<RFQ_GGUF_Q4_K>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    case RFQ_GGUF_Q6_K: rc = run_get_rows<RFQ_GGUF_Q6_K>(table, d_tokens, d_out, n_vocab, n_embd, n_tokens, d_status, s); break;
    default: return fail(RFQ_E_BADARG, "rfq_get_rows: unknown format %d", fmt);
    }
    if (rc != RFQ_OK) return rc;
    if (d_status) {
        hipLaunchKernelGGL(get_rows_status_kernel, dim3(1), dim3(1), 0, s, d_status, 1);
        RFQ_LAUNCH_CHECK("get_rows_status_kernel");
    }
    return RFQ_OK;
}

} // namespace rfq
