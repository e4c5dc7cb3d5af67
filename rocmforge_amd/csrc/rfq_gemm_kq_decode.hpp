// For the fp16 matrix-core GEMM kernel of the block formats with f16/f32 scales (rfq_gemm_kq.hip): vector types, the LDS hand-over barrier, and per format the raw bytes of one 32-element
// group of a weight row with its decode to fp16 (Raw32<FMT>).
#pragma once
#include <type_traits>

#include "rfq_common.hpp"

namespace rfq {
// RFQ_GGUF_Q4_K bytes decoded to the integer operand sc * q (Raw32<KQ_GGUF_Q4_K_INT> below): a name inside this
// library, not a format of the C ABI.
constexpr int KQ_GGUF_Q4_K_INT = 0x1000 + RFQ_GGUF_Q4_K;
template <> struct Fmt<KQ_GGUF_Q4_K_INT> { static constexpr int BE = 256, BB = 144; };
namespace kq {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4))); // 16 bytes in flight (a builtin vector: plain loads and stores)
template <int N> struct IC { static constexpr int value = N; };

// Workgroup barrier for LDS hand-over that leaves global loads in flight
// (__syncthreads would wait for the prefetches issued just before it): this
// wavefront's LDS writes are complete (lgkmcnt), then everyone meets.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0); vmcnt and expcnt unconstrained
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// ---- raw bytes of one 32-element group g of a row, and its f32 values --------
template <int FMT> struct Raw32;

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef __amdgpu_buffer_rsrc_t Rsrc;

// Where element e (0..7) of an 8-element k chunk sits in the chunk as both
// operands store it: [k0 k4 k1 k5 k2 k6 k3 k7].  Nibble pairs (k, k+4) of a
// dword of packed 4-bit weights come out of one mask operation in that order;
// the activations are arranged to match (any assignment of k to the matrix
// instruction's k slots works as long as both operands use it).
__device__ __forceinline__ constexpr int chunk_pos(int e) { return ((e & 3) << 1) | (e >> 2); }

// The fp16 operands a decoded weight v (f32) is contracted as: hi = fp16(v) (round to nearest even) and, when the
// kernel runs two planes, lo = fp16(v - hi), so that hi + lo = v to 2^-22 of v.
// v goes through an opaque statement first when both are wanted: the compiler otherwise folds the multiplication that
// produced v into ONE of the two conversions it emits (v_fma_mixlo_f16 rounds the exact product, v_cvt_f16_f32 the
// f32-rounded one), and where the f32 value is a tie of the fp16 grid the stored hi and the hi that lo was formed
// against then differ by an fp16 ulp.
__device__ __forceinline__ void fp16_pair(float v, _Float16 &hi, _Float16 &lo)
{
    asm("" : "+v"(v));
    hi = (_Float16)v;
    float back = (float)hi;
    asm("" : "+v"(back));
    lo = (_Float16)(v - back);
}
template <bool BOTH> __device__ __forceinline__ void fp16_parts(float v, _Float16 &hi, _Float16 &lo)
{
    if constexpr (BOTH) fp16_pair(v, hi, lo);
    else hi = (_Float16)v;
}

// Every format decodes a 32-element group in 12 steps (chunk c = T/3 of 8
// elements, three steps each) so that the work can be spread evenly between
// matrix instructions.  load() reads group 2*st + wh of the row at lane
// offset row_off through a buffer descriptor of the weight tile: the stage
// part of the address is scalar, the lane part a 32-bit offset.

// src/kernels/quant/q4_0.rs:289-306: 20-byte block = f32 scale + 16 nibble bytes
template <> struct Raw32<RFQ_Q4_0> {
    static constexpr int ND = 5;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        const uint32_t v = row_off + 20u * wh;
        d[0] = __builtin_amdgcn_raw_buffer_load_b32(w, v, st * 40, 0);
        v4u q = __builtin_amdgcn_raw_buffer_load_b128(w, v + 4, st * 40, 0);
        d[1] = q[0]; d[2] = q[1]; d[3] = q[2]; d[4] = q[3];
    }
    __device__ __forceinline__ void zero() { d[0] = 0; d[1] = d[2] = d[3] = d[4] = 0x88888888u; } // nibble 8 is 0.0
    __device__ __forceinline__ void settle(int, uint32_t, int) {}
    __device__ __forceinline__ float value(int e) const            // element 2i = low nibble of byte i
    {
        uint32_t q = (d[1 + (e >> 3)] >> (4 * (e & 7))) & 15u;
        // scale * (q - 8) as a fused multiply-add of q: 8 * scale is exact, so the one rounding is the product's
        return __builtin_fmaf(__uint_as_float(d[0]), (float)q, -8.0f * __uint_as_float(d[0]));
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

// src/kernels/quant/q8_0.rs:55-59: 36-byte block = f32 scale + 32 offset-binary bytes
template <> struct Raw32<RFQ_Q8_0> {
    static constexpr int ND = 9;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        const uint32_t v = row_off + 36u * wh;
        d[0] = __builtin_amdgcn_raw_buffer_load_b32(w, v, st * 72, 0);
        v4u q0 = __builtin_amdgcn_raw_buffer_load_b128(w, v + 4, st * 72, 0);
        v4u q1 = __builtin_amdgcn_raw_buffer_load_b128(w, v + 20, st * 72, 0);
        d[1] = q0[0]; d[2] = q0[1]; d[3] = q0[2]; d[4] = q0[3];
        d[5] = q1[0]; d[6] = q1[1]; d[7] = q1[2]; d[8] = q1[3];
    }
    __device__ __forceinline__ void zero()
    {
        d[0] = 0;
#pragma unroll
        for (int i = 1; i < ND; i++) d[i] = 0x80808080u;
    }
    __device__ __forceinline__ void settle(int, uint32_t, int) {}
    __device__ __forceinline__ float value(int e) const
    {
        uint32_t b = (d[1 + (e >> 2)] >> (8 * (e & 3))) & 255u;
        // (b - 128) * scale as a fused multiply-add of b: 128 * scale is exact, so the one rounding is the product's
        return __builtin_fmaf(__uint_as_float(d[0]), (float)b, -128.0f * __uint_as_float(d[0]));
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

// src/kernels/quant/q4_k.rs:222-268: sub-block sb of a 256-byte super-block:
// f16 scale at 2*sb, i8 min at 16+sb, 16 nibble bytes at 32+28*sb
template <> struct Raw32<RFQ_Q4_K> {
    static constexpr int ND = 5;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        // (the scale comes with the super-block's header)
        v4u q = __builtin_amdgcn_raw_buffer_load_b128(w, row_off + 28u * wh + 32, (st >> 2) * 256 + 56 * (st & 3), 0);
        d[1] = q[0]; d[2] = q[1]; d[3] = q[2]; d[4] = q[3];
    }
    __device__ __forceinline__ void zero() { d[0] = d[1] = d[2] = d[3] = d[4] = 0; }
    // d[0] becomes the f16 scale in both halves; `pair` is the header dword
    // that holds the scales of sub-blocks g & ~1 and g | 1.
    __device__ __forceinline__ void settle(int g, uint32_t pair, int) { d[0] = ((pair >> (16 * (g & 1))) & 0xFFFFu) * 0x10001u; }
    // q * scale only: the min is contracted separately.  The product of the
    // integer q and the f16 scale is exact in f32, so rounding it to fp16 is
    // what a single fp16 multiplication returns: two weights per instruction.
    // A dword holds nibbles k0..k7 of a chunk; 0x6400 | q reads 1024 + q and
    // 0x5400 | (q << 4) reads 64 + q, so one and-or per pair (k0,k4), (k1,k5),
    // and of the dword shifted by 8, (k2,k6), (k3,k7); then subtract the
    // offset (exact) and multiply by the scale (one rounding).
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&)[4], v2h (&t)[4]) const
    {
        const int c = T / 3, ph = T % 3;
        if (ph == 0) {
            uint32_t m_lo = 0x000F000Fu, m_hi = 0x00F000F0u, g_lo = 0x64006400u, g_hi = 0x54005400u;
            asm("" : "+s"(m_lo));                                  // (register operands: and + or in one instruction)
            asm("" : "+s"(m_hi));
            asm("" : "+v"(g_lo));
            asm("" : "+v"(g_hi));
            const uint32_t x = d[1 + c], y = x >> 8;
            const uint32_t b[4] = {(x & m_lo) | g_lo, (x & m_hi) | g_hi, (y & m_lo) | g_lo, (y & m_hi) | g_hi};
#pragma unroll
            for (int q = 0; q < 4; q++) __builtin_memcpy(&t[q], &b[q], 4);
        } else if (ph == 1) {
            const v2h b_lo = {(_Float16)-1024.0f, (_Float16)-1024.0f}, b_hi = {(_Float16)-64.0f, (_Float16)-64.0f};
#pragma unroll
            for (int q = 0; q < 4; q++) t[q] = t[q] + ((q & 1) ? b_hi : b_lo);
        } else {
            v2h s2;
            __builtin_memcpy(&s2, &d[0], 4);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const v2h v = t[q] * s2;
                h[c][2 * q] = v[0];
                h[c][2 * q + 1] = v[1];
            }
        }
    }
};

// src/kernels/quant/q6_k.rs:221-261: element i of a 256-byte block: f16 scale
// 2*(i/16), signed 6-bit field at bit 6*i of the stream at +32.  32 elements =
// two scales + 24 stream bytes.
template <> struct Raw32<RFQ_Q6_K> {
    static constexpr int ND = 7;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        const int blk = (st >> 2) * 256;
        d[0] = __builtin_amdgcn_raw_buffer_load_b32(w, row_off + 4u * wh, blk + 8 * (st & 3), 0);
        const uint32_t v = row_off + 24u * wh + 32;
        v4u q = __builtin_amdgcn_raw_buffer_load_b128(w, v, blk + 48 * (st & 3), 0);
        v2u r = __builtin_amdgcn_raw_buffer_load_b64(w, v + 16, blk + 48 * (st & 3), 0);
        d[1] = q[0]; d[2] = q[1]; d[3] = q[2]; d[4] = q[3]; d[5] = r[0]; d[6] = r[1];
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    __device__ __forceinline__ void settle(int, uint32_t, int) {}
    __device__ __forceinline__ float value(int e) const
    {
        const float scale = f16_bits_to_f32((uint16_t)((d[0] >> (16 * (e >> 4))) & 0xFFFFu));
        const int bit = 6 * e, w = bit >> 5, o = bit & 31;
        uint64_t two = (uint64_t)d[1 + w] | ((uint64_t)d[1 + (w < 5 ? w + 1 : w)] << 32);
        return (float)sbfe6((uint32_t)(two >> o), 0) * scale;
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

// ---- the block layouts of GGUF model files (ggml-common.h, ggml-quants.c) --------
// Blocks are 2-byte aligned only: the loads below land on any byte address.
// Each format decodes with the generic step (f32 value, one rounding to fp16).

// block_q4_0: f16 d, 16 bytes; low nibbles = elements 0..15, high = 16..31; d * (q - 8)
template <> struct Raw32<RFQ_GGUF_Q4_0> {
    static constexpr int ND = 5;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        const uint32_t v = row_off + 18u * wh;
        d[0] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(w, v, st * 36, 0);
        v4u q = __builtin_amdgcn_raw_buffer_load_b128(w, v + 2, st * 36, 0);
        d[1] = q[0]; d[2] = q[1]; d[3] = q[2]; d[4] = q[3];
    }
    __device__ __forceinline__ void zero() { d[0] = 0; d[1] = d[2] = d[3] = d[4] = 0x88888888u; }
    // d[0] becomes the f32 scale
    __device__ __forceinline__ void settle(int, uint32_t, int) { d[0] = __float_as_uint(f16_bits_to_f32((uint16_t)d[0])); }
    // d * (q - 8) as a fused multiply-add of q (8 * d is exact: the same single rounding)
    __device__ __forceinline__ float value(int e) const
    {
        uint32_t q = (d[1 + ((e & 15) >> 2)] >> (8 * (e & 3) + 4 * (e >> 4))) & 15u;
        const float sc = __uint_as_float(d[0]);
        return __builtin_fmaf(sc, (float)q, -8.0f * sc);
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

// block_q8_0: f16 d, 32 int8; d * q
template <> struct Raw32<RFQ_GGUF_Q8_0> {
    static constexpr int ND = 9;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        const uint32_t v = row_off + 34u * wh;
        d[0] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(w, v, st * 68, 0);
        v4u q0 = __builtin_amdgcn_raw_buffer_load_b128(w, v + 2, st * 68, 0);
        v4u q1 = __builtin_amdgcn_raw_buffer_load_b128(w, v + 18, st * 68, 0);
        d[1] = q0[0]; d[2] = q0[1]; d[3] = q0[2]; d[4] = q0[3];
        d[5] = q1[0]; d[6] = q1[1]; d[7] = q1[2]; d[8] = q1[3];
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    __device__ __forceinline__ void settle(int, uint32_t, int) { d[0] = __float_as_uint(f16_bits_to_f32((uint16_t)d[0])); }
    __device__ __forceinline__ float value(int e) const
    {
        const int b = (int)(int8_t)((d[1 + (e >> 2)] >> (8 * (e & 3))) & 255u);
        return (float)b * __uint_as_float(d[0]);
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

// block_q4_K (144 bytes): f16 d, f16 dmin, 12 bytes of 6-bit scales and mins, 128
// nibble bytes.  Sub-block sb = 32 elements: chunk sb >> 1 of 32 bytes, low
// (even sb) or high (odd sb) nibbles; value = (d * sc) * q - dmin * m.  The two
// threads of a row read the same 32 bytes of a stage and take a nibble half each.
// Unlike the 256-byte layout's integer mins, d * sc * q and dmin * m have the
// same magnitude here (a real min/max quantisation), so the rounded fp16 value
// of the whole expression carries the usual 2^-12 relative error.
template <> struct Raw32<RFQ_GGUF_Q4_K> {
    static constexpr int ND = 12;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int)
    {
        const int blk = (st >> 2) * 144;
        v4u h = __builtin_amdgcn_raw_buffer_load_b128(w, row_off, blk, 0);
        v4u q0 = __builtin_amdgcn_raw_buffer_load_b128(w, row_off + 16, blk + 32 * (st & 3), 0);
        v4u q1 = __builtin_amdgcn_raw_buffer_load_b128(w, row_off + 32, blk + 32 * (st & 3), 0);
        d[0] = h[0]; d[1] = h[1]; d[2] = h[2]; d[3] = h[3];
        d[4] = q0[0]; d[5] = q0[1]; d[6] = q0[2]; d[7] = q0[3];
        d[8] = q1[0]; d[9] = q1[1]; d[10] = q1[2]; d[11] = q1[3];
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    // d[0] = d * sc, d[1] = -(dmin * m) (f32); the nibbles of this half become bytes.
    // The stage's number c within its super-block (its 64-element chunk) is a
    // compile-time constant where this is called, wh the thread's nibble half.
    __device__ __forceinline__ void settle(int wh, uint32_t, int c)
    {
        const int sub = 2 * c + wh;
        const uint32_t sm = gguf_scale_min_k4(sub, d[1], d[2], d[3]);
        const float d1 = f16_bits_to_f32((uint16_t)(d[0] & 0xFFFFu)) * (float)(sm & 255u);
        const float m1 = f16_bits_to_f32((uint16_t)(d[0] >> 16)) * (float)(sm >> 8);
        d[0] = __float_as_uint(d1);
        d[1] = __float_as_uint(-m1);
        const int sh = 4 * (sub & 1);
#pragma unroll
        for (int i = 4; i < ND; i++) d[i] = (d[i] >> sh) & 0x0F0F0F0Fu;
    }
    __device__ __forceinline__ float value(int e) const
    {
        // one fused multiply-add (what ggml's own GPU and -march=native CPU builds compute); against the
        // two roundings of the plain C expression the f32 value differs by at most one ulp, far below
        // the fp16 rounding that follows
        const uint32_t q = (d[4 + (e >> 2)] >> (8 * (e & 3))) & 255u;
        return __builtin_fmaf(__uint_as_float(d[0]), (float)q, __uint_as_float(d[1]));
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

// block_q4_K contracted exactly in one pass: the operand is the integer sc * q (at most 63 * 15 = 945, exact in
// fp16), summed over a super-block by the matrix cores; d multiplies that sum in f32 and -(dmin * m) goes through
// the sub-block sums of the activations (the kernel does both).
template <> struct Raw32<KQ_GGUF_Q4_K_INT> {
    static constexpr int ND = 12;
    uint32_t d[ND];
    // Stage number C within its super-block (the ring slot): only a super-block's first stage fetches the header.
    template <int C> __device__ __forceinline__ void load_slot(Rsrc w, uint32_t row_off, int st)
    {
        const int blk = (st >> 2) * 144;
        if constexpr (C == 0) {
            v4u h = __builtin_amdgcn_raw_buffer_load_b128(w, row_off, blk, 0);
            d[0] = h[0]; d[1] = h[1]; d[2] = h[2]; d[3] = h[3];
        }
        v4u q0 = __builtin_amdgcn_raw_buffer_load_b128(w, row_off + 16, blk + 32 * (st & 3), 0);
        v4u q1 = __builtin_amdgcn_raw_buffer_load_b128(w, row_off + 32, blk + 32 * (st & 3), 0);
        d[4] = q0[0]; d[5] = q0[1]; d[6] = q0[2]; d[7] = q0[3];
        d[8] = q1[0]; d[9] = q1[1]; d[10] = q1[2]; d[11] = q1[3];
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    // The unit a super-block's sums are kept in is d * 2^j: j > 0 only where -(dmin * m) / d would leave the fp16 range
    // (data far from zero against its spread: |dmin| * 64 >= 2^15 * |d|); the operand is then sc * q * 2^-j, still exact
    // (945 * 2^-24 is an fp16 number).  j from the f32 exponent fields: |dmin * 63 / d| < 2^(e_dmin - e_d + 7).
    static __device__ __forceinline__ int unit_shift(float dv, float dmin)
    {
        const int j = (int)((__float_as_uint(dmin) >> 23) & 255u) - (int)((__float_as_uint(dv) >> 23) & 255u) - 8;
        return j < 0 ? 0 : (j > 24 ? 24 : j);
    }
    // Before settle().  `unit` comes in as the unit the accumulators are in and leaves as this super-block's;
    // ratio = old / new.  A super-block with d = 0 has no q term (settle() clears its sc) and takes |dmin| as its
    // unit, or the old one when dmin is 0 too.  For the thread's four sub-blocks 4*wh .. 4*wh+3,
    // v = -(dmin * m) / unit (dmin * m is exact in f32: 11 x 6 bits) as the fp16 pairs (hi, hi) and (lo, 0) with
    // hi + lo = v: contracted with the activations' group sums (S_hi, S_lo) they give hi * S_hi + hi * S_lo + lo * S_hi.
    // s2 / o2: for the thread's sub-block 2c + wh of each stage c = 0..3 of the super-block, s = sc * 2^-j (0 where d
    // is 0: no q term) and -(offset * s) as fp16, two per dword: what settle_packed() spreads into a stage's registers.
    // The work is cut into eight phases so that the kernel can lay them between matrix instructions: 0 = units and
    // ratio, 1-2 = the scales, 3-6 = the mins, (7 = the kernel's LDS writes).  header() runs them all.
    struct Header {
        float ratio, dmin, inv, down;
        v8h m_hi, m_lo;
    };
    template <int PH>
    __device__ __forceinline__ void header_phase(int wh, float &unit, uint32_t (&s2)[2], uint32_t (&o2)[2], Header &h) const
    {
        if constexpr (PH == 0) {
            const float dv = f16_bits_to_f32((uint16_t)(d[0] & 0xFFFFu));
            h.dmin = f16_bits_to_f32((uint16_t)(d[0] >> 16));
            const int j = unit_shift(dv, h.dmin);
            const float scaled = dv * __uint_as_float((uint32_t)(127 + j) << 23);
            h.down = dv != 0.0f ? __uint_as_float((uint32_t)(127 - j) << 23) : 0.0f;
            const float next = dv != 0.0f ? scaled : (h.dmin != 0.0f ? __builtin_fabsf(h.dmin) : unit);
            h.inv = 1.0f / next;
            h.ratio = next == unit ? 1.0f : unit * h.inv;
            unit = next;
        } else if constexpr (PH <= 2) {
            constexpr int p = PH - 1;
            v2h sv, ov;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int c = 2 * p + e;
                const uint32_t s0 = gguf_scale_min_k4(2 * c, d[1], d[2], d[3]) & 255u, s1 = gguf_scale_min_k4(2 * c + 1, d[1], d[2], d[3]) & 255u;
                const float sc = (float)(wh ? s1 : s0) * h.down;
                sv[e] = (_Float16)sc;                                             // exact (sc < 64, j <= 24)
                ov[e] = (_Float16)(-(wh ? 64.0f : 1024.0f) * sc);                 // exact
            }
            __builtin_memcpy(&s2[p], &sv, 4);
            __builtin_memcpy(&o2[p], &ov, 4);
        } else if constexpr (PH <= 6) {
            constexpr int q = PH - 3;
            // (both halves unpacked with compile-time sub-block numbers, the thread's half chosen after)
            const uint32_t m0 = gguf_scale_min_k4(q, d[1], d[2], d[3]) >> 8, m1 = gguf_scale_min_k4(4 + q, d[1], d[2], d[3]) >> 8;
            const float v = -(h.dmin * (float)(wh ? m1 : m0)) * h.inv;
            _Float16 hi, lo;
            fp16_pair(v, hi, lo);
            h.m_hi[2 * q] = hi;
            h.m_hi[2 * q + 1] = hi;
            h.m_lo[2 * q] = lo;
            h.m_lo[2 * q + 1] = (_Float16)0.0f;
        }
    }
    __device__ __forceinline__ void header(int wh, float &unit, uint32_t (&s2)[2], uint32_t (&o2)[2], Header &h) const
    {
        header_phase<0>(wh, unit, s2, o2, h);
        header_phase<1>(wh, unit, s2, o2, h);
        header_phase<2>(wh, unit, s2, o2, h);
        header_phase<3>(wh, unit, s2, o2, h);
        header_phase<4>(wh, unit, s2, o2, h);
        header_phase<5>(wh, unit, s2, o2, h);
        header_phase<6>(wh, unit, s2, o2, h);
    }
    // d[0] = (s, s) as fp16, d[1] = -(offset * s) twice (both from header(), by the stage's number c within its
    // super-block, a compile-time constant at the call), d[2] = the nibble mask of the thread's half wh, d[3] = the fp16
    // bits the nibbles are or-ed into: low nibbles read 1024 + q (0x6400 | q), high nibbles 64 + q (0x5400 | q << 4).
    __device__ __forceinline__ void settle_packed(int wh, const uint32_t (&s2)[2], const uint32_t (&o2)[2], int c)
    {
        const uint32_t sel = (c & 1) ? 0x03020302u : 0x01000100u;
        d[0] = __builtin_amdgcn_perm(s2[c >> 1], s2[c >> 1], sel);
        d[1] = __builtin_amdgcn_perm(o2[c >> 1], o2[c >> 1], sel);
        d[2] = wh ? 0x00F000F0u : 0x000F000Fu;
        d[3] = wh ? 0x54005400u : 0x64006400u;
    }
    __device__ __forceinline__ void settle(int, uint32_t, int) {}
    __device__ __forceinline__ void load(Rsrc, uint32_t, int, int) {}
    // Chunk c = elements 8c .. 8c+7 of the sub-block = bytes 8c .. 8c+7 of the stage's 32: dwords x0 (k0..k3) and x1
    // (k4..k7).  Their low halves side by side are the bytes (k0 k1 k4 k5): one and-or gives the pair (k0, k4), the same
    // on the dword shifted by 8 (k1, k5); the high halves (k2, k6) and (k3, k7) - the order the activations are in.
    // (offset + q) * sc - offset * sc as one fp16 fused multiply-add: sc * q, exact.
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&)[4], v2h (&t)[4]) const
    {
        const int c = T / 3, ph = T % 3;
        if (ph == 0) {
            const uint32_t u0 = __builtin_amdgcn_perm(d[5 + 2 * c], d[4 + 2 * c], 0x05040100u);
            const uint32_t u1 = __builtin_amdgcn_perm(d[5 + 2 * c], d[4 + 2 * c], 0x07060302u);
            const uint32_t b0 = (u0 & d[2]) | d[3], b1 = ((u0 >> 8) & d[2]) | d[3];
            __builtin_memcpy(&t[0], &b0, 4);
            __builtin_memcpy(&t[1], &b1, 4);
            __builtin_memcpy(&t[2], &u1, 4);
        } else if (ph == 1) {
            uint32_t u1;
            __builtin_memcpy(&u1, &t[2], 4);
            const uint32_t b2 = (u1 & d[2]) | d[3], b3 = ((u1 >> 8) & d[2]) | d[3];
            __builtin_memcpy(&t[2], &b2, 4);
            __builtin_memcpy(&t[3], &b3, 4);
        } else {
            v2h s2, o2;
            __builtin_memcpy(&s2, &d[0], 4);
            __builtin_memcpy(&o2, &d[1], 4);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const v2h v = __builtin_elementwise_fma(t[q], s2, o2);
                h[c][2 * q] = v[0];
                h[c][2 * q + 1] = v[1];
            }
        }
    }
};

// block_q6_K (210 bytes): ql[128], qh[64], i8 scales[16], f16 d.  Sub-block sb =
// 32 elements: half n = sb >> 2 of 128 elements, quarter t = sb & 3: low nibbles
// from ql[64 n + 32 (t & 1) + l] (>> 4 for t >= 2), bits 4-5 from qh[32 n + l] >> 2 t,
// scales sc[8 n + 2 t + l / 16]; value = (d * sc) * (q - 32).
template <> struct Raw32<RFQ_GGUF_Q6_K> {
    static constexpr int ND = 17;
    uint32_t d[ND];
    __device__ __forceinline__ void load(Rsrc w, uint32_t row_off, int st, int wh)
    {
        const int blk = (st >> 2) * 210, half = (st & 3) >> 1, odd = st & 1;
        const uint32_t vq = row_off + 32u * wh;
        v4u l0 = __builtin_amdgcn_raw_buffer_load_b128(w, vq, blk + 64 * half, 0);
        v4u l1 = __builtin_amdgcn_raw_buffer_load_b128(w, vq + 16, blk + 64 * half, 0);
        v4u h0 = __builtin_amdgcn_raw_buffer_load_b128(w, row_off, blk + 128 + 32 * half, 0);
        v4u h1 = __builtin_amdgcn_raw_buffer_load_b128(w, row_off + 16, blk + 128 + 32 * half, 0);
        const uint32_t sc = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(w, row_off + 2u * wh, blk + 192 + 8 * half + 4 * odd, 0);
        const uint32_t dd = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(w, row_off, blk + 208, 0);
        d[0] = l0[0]; d[1] = l0[1]; d[2] = l0[2]; d[3] = l0[3]; d[4] = l1[0]; d[5] = l1[1]; d[6] = l1[2]; d[7] = l1[3];
        d[8] = h0[0]; d[9] = h0[1]; d[10] = h0[2]; d[11] = h0[3]; d[12] = h1[0]; d[13] = h1[1]; d[14] = h1[2]; d[15] = h1[3];
        d[16] = sc | (dd << 16);
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    // d[0..7] = the 6-bit codes as bytes, d[8] / d[9] = d * sc of the two 16-element halves (f32), d[10] / d[11] = -32 times those;
    // c = the stage's number within its super-block (a compile-time constant at the call), wh = the thread's group
    __device__ __forceinline__ void settle(int wh, uint32_t, int c)
    {
        const int t = 2 * (c & 1) + wh, shl = 4 * (c & 1), shh = 2 * t;
#pragma unroll
        for (int i = 0; i < 8; i++) d[i] = ((d[i] >> shl) & 0x0F0F0F0Fu) | (((d[8 + i] >> shh) & 0x03030303u) << 4);
        const float dv = f16_bits_to_f32((uint16_t)(d[16] >> 16));
        const float s0 = dv * (float)(int)(int8_t)(d[16] & 255u), s1 = dv * (float)(int)(int8_t)((d[16] >> 8) & 255u);
        d[8] = __float_as_uint(s0);
        d[9] = __float_as_uint(s1);
        d[10] = __float_as_uint(-32.0f * s0);
        d[11] = __float_as_uint(-32.0f * s1);
    }
    // (d * sc) * (q - 32) as one fused multiply-add of q: 32 * (d * sc) is exact, so the
    // single rounding of q * (d * sc) - 32 * (d * sc) is the rounding of the product.
    __device__ __forceinline__ float value(int e) const
    {
        const uint32_t q = (d[e >> 2] >> (8 * (e & 3))) & 255u;
        return __builtin_fmaf(__uint_as_float(d[8 + (e >> 4)]), (float)q, __uint_as_float(d[10 + (e >> 4)]));
    }
    template <bool BOTH> __device__ __forceinline__ void step(int T, v8h (&h)[4], v8h (&l)[4], v2h (&)[4]) const
    {
        const int c = T / 3, e0 = 3 * (T % 3), e1 = e0 + 3 < 8 ? e0 + 3 : 8;
#pragma unroll
        for (int e = e0; e < e1; e++) {
            _Float16 hi, lo = (_Float16)0.0f;
            fp16_parts<BOTH>(value(8 * c + e), hi, lo);
            h[c][chunk_pos(e)] = hi;
            if constexpr (BOTH) l[c][chunk_pos(e)] = lo;
        }
    }
};

} // namespace kq

} // namespace rfq
