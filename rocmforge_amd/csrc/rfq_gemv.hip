// Fused dequantise + GEMV for decode:  y[m, n] = x[m, k] . dequant(W)[n, k]^T.
//
// Bandwidth-bound: every packed weight byte is read from HBM exactly once and
// nothing else of size is touched.  No matrix cores.  The work quantum is a
// "unit" of 32 consecutive k (one block of the 32-element formats, one
// sub-block of Q4_K, two scale groups of Q6_K), fetched by one lane with
// 16-byte loads; a wavefront's 64 lanes fetch 64 neighbouring units, i.e. one
// contiguous span of the row.
//
// Two kernels:
//   gemv_xreg    (m == 1): a team of WPR wavefronts owns a fixed set of k
//                positions and walks down the rows; each lane keeps the x
//                values of its units in registers for the whole kernel, so x is
//                read once per team instead of once per row and the only
//                traffic in the loop is the weight stream (next row prefetched
//                while the current one is reduced).
//   gemv_generic (any m <= 8, any k): one row per wavefront, lanes stride over
//                the units and read x through the L1/L2 caches.
// Reduction: DPP butterflies inside each row of 16 lanes, v_readlane across
// the four rows; an LDS hop only when a row is split over several wavefronts.
#include <stdio.h>

#include <mutex>

#include "rfq_common.hpp"

// This file is compiled RFQ_GEMV_PARTS times, -DRFQ_GEMV_PART=0 .. RFQ_GEMV_PARTS-1: every part holds the kernels of
// some of the formats (gemv_part_of) behind launch_gemv_part<N> / launch_gemv_fused_part<N>, and part 0 holds the entry
// points that hand a call to its format's part, so the formats compile side by side.  -DRFQ_GEMV_ONLY=<format> builds
// part 0 with that format alone (a quick build while working on one format's kernel).
#ifndef RFQ_GEMV_PART
#error "compile with -DRFQ_GEMV_PART=0 .. 3 (see the Makefile)"
#endif

namespace rfq {

constexpr int gemv_part_of(int canonical)
{
#ifdef RFQ_GEMV_ONLY
    return canonical == RFQ_GEMV_ONLY ? 0 : -1;
#else
    switch (canonical) {
    case RFQ_Q4_K: case RFQ_Q4_0: case RFQ_MM_Q4_K: return 0;
    case RFQ_Q8_0: case RFQ_GGUF_Q8_0: case RFQ_MM_Q8_0: return 1;
    case RFQ_Q6_K: case RFQ_MM_Q6_K: case RFQ_MXFP4: case RFQ_MXFP6_E2M3: return 2;
    case RFQ_GGUF_Q4_0: case RFQ_GGUF_Q4_K: case RFQ_GGUF_Q6_K: return 3;
    default: return -1;
    }
#endif
}

#if RFQ_GEMV_PART == 0
thread_local GemvLastKernel g_gemv_last_kernel = {"", 0, 0, 0, 0};
thread_local GemvTraceRequest g_gemv_trace_request = {nullptr, 0, 0};
#endif

namespace {

// Which kernel the last GEMV launch of this thread took (name and template arguments), for the benchmark
// driver's report: plain stores on the launch path, formatted only when asked for.
inline void note_kernel(const char *name, int fmt, int a, int b, int c) { g_gemv_last_kernel = GemvLastKernel{name, fmt, a, b, c}; }

// ---- wavefront reduction -----------------------------------------------------

template <int CTRL> __device__ __forceinline__ float dpp_add(float v)
{
    int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
    return v + __int_as_float(o);
}

// Sum over the 64 lanes; the result is valid in every lane.
__device__ __forceinline__ float wave_sum(float v)
{
    v = dpp_add<0xB1>(v);  // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v); // row_half_mirror
    v = dpp_add<0x140>(v); // row_mirror: every lane holds its 16-lane row sum
    int b = __float_as_int(v);
    float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// Sums of M values per lane over the 16 lanes of each row, M = 2, 4 or 8: instead of M separate reductions, lanes that
// differ in one bit exchange half of what they hold (the lane keeps the value whose index has that bit like its own
// number and adds the partner's copy of it), so after log2(M) steps a lane holds a single partial sum, of value number
// lane % M, and the remaining steps are one addition each.  Afterwards lane l holds the sum of value l % M over its
// row of 16 lanes.  25 instructions for M = 8 where eight wave_sum take about 90.
template <int CTRL> __device__ __forceinline__ float dpp_get(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// the value of lane ^ 4: lanes 4..7 and 12..15 of a row take it from four lanes down, the others from four lanes up
__device__ __forceinline__ float dpp_xor4(float v)
{
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x114, 0xF, 0xA, false);          // row_shr:4 into banks 1, 3
    r = __builtin_amdgcn_update_dpp(r, __float_as_int(v), 0x104, 0xF, 0x5, false);              // row_shl:4 into banks 0, 2
    return __int_as_float(r);
}
template <int M> __device__ __forceinline__ float rows16_sum_of(const float (&a)[M], int lane)
{
    static_assert(M == 2 || M == 4 || M == 8, "two, four or eight values");
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4;
    float w[M / 2];
#pragma unroll
    for (int p = 0; p < M / 2; p++) w[p] = (b0 ? a[2 * p + 1] : a[2 * p]) + dpp_get<0xB1>(b0 ? a[2 * p] : a[2 * p + 1]);
    float f;
    if constexpr (M == 2) {
        f = w[0] + dpp_get<0x4E>(w[0]);
        f += dpp_xor4(f);
    } else {
        float z[M / 4];
#pragma unroll
        for (int q = 0; q < M / 4; q++) z[q] = (b1 ? w[2 * q + 1] : w[2 * q]) + dpp_get<0x4E>(b1 ? w[2 * q] : w[2 * q + 1]);
        if constexpr (M == 4) {
            f = z[0] + dpp_xor4(z[0]);
        } else {
            f = (b2 ? z[1] : z[0]) + dpp_xor4(b2 ? z[0] : z[1]);
        }
    }
    return f + dpp_get<0x128>(f);                                                              // row_ror:8
}

// The value of the neighbouring lane (lane ^ 1).
__device__ __forceinline__ float dpp_xor1_f(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
}

// ---- units: 32 consecutive k of one row -------------------------------------
//
// Unit<FMT>::load(row, u)  fetches unit u of the row starting at `row`.
// Unit<FMT>::dot(x, xsum)  returns sum_i w[i] * x[i] over the unit's 32 weights;
//                          xsum = sum_i x[i] lets offset formats (q-8, b-128,
//                          min + ...) fold their constant into one multiply.

__device__ __forceinline__ float ub(uint32_t w, int b) { return (float)((w >> (8 * b)) & 255u); }

struct U4 { uint32_t v[4]; };
struct U6 { uint32_t v[6]; };
struct U8 { uint32_t v[8]; };

// Sum of nibble[i] * x[i] for 16 bytes where element 2i is the LOW nibble of
// byte i (Q4_0 and Q4_K order).
__device__ __forceinline__ float nib_dot_lo_first(const U4 &q, const float (&x)[32])
{
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        uint32_t lo = q.v[d] & 0x0F0F0F0Fu, hi = (q.v[d] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            s0 = __builtin_fmaf(ub(lo, b), x[8 * d + 2 * b], s0);
            s1 = __builtin_fmaf(ub(hi, b), x[8 * d + 2 * b + 1], s1);
        }
    }
    return s0 + s1;
}

template <int FMT> struct Unit;

// ---- pieces that do not start on a multiple of 4 ------------------------------------------
// A 16-byte load from an address that is not a multiple of 4 runs at a fraction of the aligned rate on this part
// (17-byte blocks streamed as stored, a byte and 16 bytes per lane: 9.2 us for 31 MB; through aligned windows of whole
// dwords: 6.8 us).  The units of the layouts whose blocks start at odd or 2-byte offsets (MXFP4 17 bytes, MXFP6 25,
// GGUF_Q4_0 18, GGUF_Q8_0 34, GGUF_Q6_K 210) are therefore fetched as the aligned dwords that hold them and moved
// into place with byte permutes, the lane's byte offset in the selector: 14336 x 4096 MXFP6 14.2 -> 13.4 us, GGUF_Q8_0
// 15.0 -> 13.1 us; 128256 x 4096 MXFP6 108 -> 93 us, GGUF_Q4_0 75 -> 57 us, GGUF_Q8_0 138 -> 101 us (GGUF_Q4_0 14336 x
// 4096 alone measured 3 % slower, 9.5 -> 9.7 us).
template <int NW> __device__ __forceinline__ void load_dwords_a4(const uint8_t *a, uint32_t (&d)[NW])
{
    typedef uint32_t v4a4 __attribute__((ext_vector_type(4), aligned(4)));
    int i = 0;
#pragma unroll
    for (; i + 4 <= NW; i += 4) {
        const v4a4 v = *reinterpret_cast<const v4a4 *>(a + 4 * i);
        d[i] = v[0]; d[i + 1] = v[1]; d[i + 2] = v[2]; d[i + 3] = v[3];
    }
#pragma unroll
    for (; i < NW; i++) d[i] = *reinterpret_cast<const uint32_t *>(a + 4 * i);
}

// A piece of 4 * NQ bytes that starts SKIP bytes (a header: an exponent byte, an f16 scale) behind p, at any byte
// address: the NQ + 1 dwords from the multiple of 4 at or before p are fetched, and the piece is moved into place with
// byte permutes only where it is used -- permutes issued with the loads would make a wavefront wait for every row it
// has in flight before it can touch the first.  With SKIP >= 1 every dword read holds a byte of the block; with
// SKIP = 0 the last one can lie behind the piece (inside the block for the pieces this is used on).  The bytes read
// before p stay inside the tensor when the tensor starts on a multiple of 4.
template <int NQ> struct Window {
    uint32_t d[NQ + 1], o;                               // o: the byte offset of p in d[0]
    __device__ __forceinline__ void load(const uint8_t *p)
    {
        // (stepping back from p rather than building a pointer from the masked integer: the loads stay global loads
        // instead of flat ones, which also count against the LDS counter)
        o = (uint32_t)(reinterpret_cast<uintptr_t>(p) & 3u);
        load_dwords_a4<NQ + 1>(p - o, d);
    }
    // The same content from byte-exact loads (a tensor at an address the windows cannot take).
    template <uint32_t SKIP> __device__ __forceinline__ void load_bytes(const uint8_t *p)
    {
        static_assert(SKIP <= 2, "no header, a byte or two bytes");
        struct Piece { uint32_t v[NQ]; };
        const Piece q = ld<Piece>(p + SKIP);
        if constexpr (SKIP == 0) {
            o = 0;
#pragma unroll
            for (int i = 0; i < NQ; i++) d[i] = q.v[i];
            d[NQ] = 0;
        } else {
            o = 4u - SKIP;
            d[0] = (SKIP == 1 ? (uint32_t)p[0] : (uint32_t)ld<uint16_t>(p)) << (8u * o);
#pragma unroll
            for (int i = 0; i < NQ; i++) d[i + 1] = q.v[i];
        }
    }
    template <uint32_t SKIP> __device__ __forceinline__ void piece(uint32_t (&q)[NQ]) const
    {
        // o + SKIP <= 4: bytes of a dword pair.  (o in all four bytes by a byte permute: a 32-bit multiply runs at a
        // quarter of the rate)
        const uint32_t sel = (0x03020100u + 0x01010101u * SKIP) + __builtin_amdgcn_perm(0u, o, 0u);
#pragma unroll
        for (int i = 0; i < NQ; i++) q[i] = __builtin_amdgcn_perm(d[i + 1], d[i], sel);
    }
    __device__ __forceinline__ uint32_t head() const { return d[0] >> (8u * o); }   // the block's first bytes (4 - o of them)
};

template <int FMT> struct NeedsAlignedTensor { static constexpr bool value = false; };
template <> struct NeedsAlignedTensor<RFQ_GGUF_Q6_K> { static constexpr bool value = true; };
template <> struct NeedsAlignedTensor<RFQ_GGUF_Q4_0> { static constexpr bool value = true; };   // (blocks at even offsets
template <> struct NeedsAlignedTensor<RFQ_GGUF_Q8_0> { static constexpr bool value = true; };   // of the window's first dword)

template <> struct Unit<RFQ_Q4_0> {
    static constexpr bool NEEDS_XSUM = true;
    float scale; U4 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *p = row + (size_t)u * 20;
        scale = ld<float>(p);
        q = ld<U4>(p + 4);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        return scale * __builtin_fmaf(-8.0f, xsum, nib_dot_lo_first(q, x));
    }
};

template <> struct Unit<RFQ_Q8_0> {
    static constexpr bool NEEDS_XSUM = true;
    float scale; U8 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *p = row + (size_t)u * 36;
        scale = ld<float>(p);
        q = ld<U8>(p + 4);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int d = 0; d < 8; d++) {
            s0 = __builtin_fmaf(ub(q.v[d], 0), x[4 * d], s0);
            s1 = __builtin_fmaf(ub(q.v[d], 1), x[4 * d + 1], s1);
            s0 = __builtin_fmaf(ub(q.v[d], 2), x[4 * d + 2], s0);
            s1 = __builtin_fmaf(ub(q.v[d], 3), x[4 * d + 3], s1);
        }
        return scale * __builtin_fmaf(-128.0f, xsum, s0 + s1);
    }
};

template <> struct Unit<RFQ_Q4_K> {
    static constexpr bool NEEDS_XSUM = true;
    uint16_t sc; int8_t mn; U4 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *blk = row + (size_t)(u >> 3) * 256;
        int sb = u & 7;
        sc = ld<uint16_t>(blk + 2 * sb);
        mn = (int8_t)blk[16 + sb];
        q = ld_once<U4>(blk + 32 + 28 * sb);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        return __builtin_fmaf(f16_bits_to_f32(sc), nib_dot_lo_first(q, x), (float)mn * xsum);
    }
};

template <> struct Unit<RFQ_Q6_K> {
    static constexpr bool NEEDS_XSUM = false;
    uint32_t sc2; U6 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *blk = row + (size_t)(u >> 3) * 256;
        int g = u & 7;
        sc2 = ld<uint32_t>(blk + 4 * g);          // scales of groups 2g, 2g+1
        q = ld<U6>(blk + 32 + 24 * g);            // 32 six-bit codes, LSB first
    }
    // 16 codes in three dwords; code j starts at bit 6j.
    static __device__ __forceinline__ float dot16(uint32_t a, uint32_t b, uint32_t c, const float *x)
    {
        float s0 = 0.f, s1 = 0.f;
        uint32_t ab = __builtin_amdgcn_alignbit(b, a, 30); // bits 30.. of a:b -> code 5 at bit 0
        uint32_t bc = __builtin_amdgcn_alignbit(c, b, 28); // bits 60.. -> code 10 at bit 0
        s0 = __builtin_fmaf((float)sbfe6(a, 0), x[0], s0);
        s1 = __builtin_fmaf((float)sbfe6(a, 6), x[1], s1);
        s0 = __builtin_fmaf((float)sbfe6(a, 12), x[2], s0);
        s1 = __builtin_fmaf((float)sbfe6(a, 18), x[3], s1);
        s0 = __builtin_fmaf((float)sbfe6(a, 24), x[4], s0);
        s1 = __builtin_fmaf((float)sbfe6(ab, 0), x[5], s1);
        s0 = __builtin_fmaf((float)sbfe6(b, 4), x[6], s0);
        s1 = __builtin_fmaf((float)sbfe6(b, 10), x[7], s1);
        s0 = __builtin_fmaf((float)sbfe6(b, 16), x[8], s0);
        s1 = __builtin_fmaf((float)sbfe6(b, 22), x[9], s1);
        s0 = __builtin_fmaf((float)sbfe6(bc, 0), x[10], s0);
        s1 = __builtin_fmaf((float)sbfe6(c, 2), x[11], s1);
        s0 = __builtin_fmaf((float)sbfe6(c, 8), x[12], s0);
        s1 = __builtin_fmaf((float)sbfe6(c, 14), x[13], s1);
        s0 = __builtin_fmaf((float)sbfe6(c, 20), x[14], s0);
        s1 = __builtin_fmaf((float)sbfe6(c, 26), x[15], s1);
        return s0 + s1;
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        float a = dot16(q.v[0], q.v[1], q.v[2], &x[0]);
        float b = dot16(q.v[3], q.v[4], q.v[5], &x[16]);
        return __builtin_fmaf(f16_bits_to_f32((uint16_t)(sc2 & 0xFFFFu)), a, f16_bits_to_f32((uint16_t)(sc2 >> 16)) * b);
    }
};

// clamp(scale * v, +-L) == scale * clamp(v, +-L/scale) for a power-of-two
// scale, so the clamp is applied to the decoded code and the scale once per
// unit.  The bound only bites for exponents >= 1 (|code value| <= 8).
// MXFP4: decoding a code (zero test, sign, exponent) costs more than its multiply-add, so the
// two values of a code byte come from a 256-entry table in LDS, entry b = (decode(b >> 4),
// decode(b & 15)); the kernels that dot MXFP4 units fill it first (unit_tables_init).
__device__ __forceinline__ float2 *mxfp4_lut()
{
    __shared__ float2 lut[256];
    return lut;
}

// MXFP6 likewise: 64 decoded codes.
__device__ __forceinline__ float *mxfp6_lut()
{
    __shared__ float lut[64];
    return lut;
}

template <int FMT> __device__ __forceinline__ void unit_tables_init()
{
    if constexpr (FMT == RFQ_MXFP4) {
        float2 *lut = mxfp4_lut();
        for (int i = threadIdx.x; i < 256; i += blockDim.x)
            lut[i] = make_float2(decode_e2m1((uint32_t)i >> 4), decode_e2m1((uint32_t)i & 15u));
        __syncthreads();
    }
    if constexpr (FMT == RFQ_MXFP6_E2M3) {
        float *lut = mxfp6_lut();
        if (threadIdx.x < 64) lut[threadIdx.x] = decode_e2m3(threadIdx.x);
        __syncthreads();
    }
}

// Opened<FMT>: the fields of a unit that was fetched as windows (Unit<FMT>::open), with the unit's arithmetic.
template <int FMT> struct Opened;

template <> struct Opened<RFQ_MXFP4> {
    int e; U4 q;
    template <bool CLAMP> __device__ __forceinline__ float dot_as(const float (&x)[32]) const
    {
        // bound on |code value|: 8 / 2^e when e >= 1 (exact, 2^(3-e)), else 8.
        float bound = e >= 1 ? __uint_as_float((uint32_t)(130 - e) << 23) : 8.0f;
        const float2 *lut = mxfp4_lut();
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int d = 0; d < 4; d++) {
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float2 v = lut[(q.v[d] >> (8 * b)) & 255u];                // element 2j = high nibble
                const float hi = CLAMP ? __builtin_amdgcn_fmed3f(v.x, -bound, bound) : v.x;
                const float lo = CLAMP ? __builtin_amdgcn_fmed3f(v.y, -bound, bound) : v.y;
                s0 = __builtin_fmaf(hi, x[8 * d + 2 * b], s0);
                s1 = __builtin_fmaf(lo, x[8 * d + 2 * b + 1], s1);
            }
        }
        return mx_scale(e) * (s0 + s1);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        // (the clamp only bites for exponents >= 1, which weights below 1 never have: a wavefront without such a
        // unit skips the 32 clamps)
        return __builtin_amdgcn_ballot_w64(e >= 1) != 0 ? dot_as<true>(x) : dot_as<false>(x);
    }
};
template <> struct Unit<RFQ_MXFP4> {
    static constexpr bool NEEDS_XSUM = false;
    Window<4> w;
    __device__ __forceinline__ void load(const uint8_t *row, int u) { w.load(row + (size_t)u * 17); }
    __device__ __forceinline__ Opened<RFQ_MXFP4> open() const
    {
        Opened<RFQ_MXFP4> r;
        r.e = __builtin_amdgcn_sbfe((int)w.d[0], 8u * w.o, 8u);
        w.piece<1>(r.q.v);
        return r;
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const { return open().dot(x, xsum); }
};

template <> struct Opened<RFQ_MXFP6_E2M3> {
    int e; U6 q;
    template <bool CLAMP> __device__ __forceinline__ float dot_as(const float (&x)[32]) const
    {
        // 7.5 * 2^-e for e >= 1: 7.5 = 0x40F00000 (biased exponent 129).
        float bound = e >= 1 ? __uint_as_float(0x40F00000u - ((uint32_t)e << 23)) : 7.5f;
        const float *lut = mxfp6_lut();
        float s0 = 0.f, s1 = 0.f;
        // group j: bytes b[3j..3j+3]; see the extraction table in rfq_dequant.hip.
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // bytes 3j..3j+3 as one word w (byte 3j in bits 0-7)
            int bit = 24 * j, d = bit >> 5, sh = bit & 31;
            uint32_t w = (sh == 0) ? q.v[d]
                                   : __builtin_amdgcn_alignbit(d + 1 < 6 ? q.v[d + 1] : 0u, q.v[d], sh);
            uint32_t b0 = w & 255u, b1 = (w >> 8) & 255u, b2 = (w >> 16) & 255u, b3 = w >> 24;
            float v0 = lut[b1 >> 2];
            float v1 = lut[(b0 >> 4) | ((b1 & 3u) << 4)];
            float v2 = lut[(b1 >> 6) | ((b2 & 15u) << 2)];
            if (CLAMP) {
                v0 = __builtin_amdgcn_fmed3f(v0, -bound, bound);
                v1 = __builtin_amdgcn_fmed3f(v1, -bound, bound);
                v2 = __builtin_amdgcn_fmed3f(v2, -bound, bound);
            }
            s0 = __builtin_fmaf(v0, x[4 * j], s0);
            s1 = __builtin_fmaf(v1, x[4 * j + 1], s1);
            s0 = __builtin_fmaf(v2, x[4 * j + 2], s0);
            if (j < 7) { // element 31 is never written by the reference: weight 0
                float v3 = lut[b3 & 63u];
                if (CLAMP) v3 = __builtin_amdgcn_fmed3f(v3, -bound, bound);
                s1 = __builtin_fmaf(v3, x[4 * j + 3], s1);
            }
        }
        return mx_scale(e) * (s0 + s1);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        return __builtin_amdgcn_ballot_w64(e >= 1) != 0 ? dot_as<true>(x) : dot_as<false>(x);
    }
};
template <> struct Unit<RFQ_MXFP6_E2M3> {
    static constexpr bool NEEDS_XSUM = false;
    Window<6> w;
    __device__ __forceinline__ void load(const uint8_t *row, int u) { w.load(row + (size_t)u * 25); }
    __device__ __forceinline__ Opened<RFQ_MXFP6_E2M3> open() const
    {
        Opened<RFQ_MXFP6_E2M3> r;
        r.e = __builtin_amdgcn_sbfe((int)w.d[0], 8u * w.o, 8u);
        w.piece<1>(r.q.v);
        return r;
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const { return open().dot(x, xsum); }
};

// ---- GGUF file layouts (ggml block_q4_0 / q8_0 / q4_K / q6_K) -----------------
// Blocks are 2-byte aligned only; loads are byte-exact copies.

template <> struct Opened<RFQ_GGUF_Q4_0> {
    uint16_t d; U4 q;
    // element j = low nibble of byte j, element 16 + j = high nibble
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            uint32_t lo = q.v[w] & 0x0F0F0F0Fu, hi = (q.v[w] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                s0 = __builtin_fmaf(ub(lo, b), x[4 * w + b], s0);
                s1 = __builtin_fmaf(ub(hi, b), x[16 + 4 * w + b], s1);
            }
        }
        return f16_bits_to_f32(d) * __builtin_fmaf(-8.0f, xsum, s0 + s1);
    }
};
// (blocks at even addresses, see NeedsAlignedTensor: o = 0 or 2 and the f16 scale lies inside the first dword)
template <> struct Unit<RFQ_GGUF_Q4_0> {
    static constexpr bool NEEDS_XSUM = true;
    Window<4> w;
    __device__ __forceinline__ void load(const uint8_t *row, int u) { w.load(row + (size_t)u * 18); }
    __device__ __forceinline__ void load_bytes(const uint8_t *row, int u) { w.load_bytes<2>(row + (size_t)u * 18); }
    __device__ __forceinline__ Opened<RFQ_GGUF_Q4_0> open() const
    {
        Opened<RFQ_GGUF_Q4_0> r;
        r.d = (uint16_t)w.head();
        w.piece<2>(r.q.v);
        return r;
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const { return open().dot(x, xsum); }
};

template <> struct Opened<RFQ_GGUF_Q8_0> {
    uint16_t d; U8 q;
    // int8 q = (q ^ 0x80) - 128 with the left term read as an unsigned byte
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            uint32_t v = q.v[w] ^ 0x80808080u;
            s0 = __builtin_fmaf(ub(v, 0), x[4 * w], s0);
            s1 = __builtin_fmaf(ub(v, 1), x[4 * w + 1], s1);
            s0 = __builtin_fmaf(ub(v, 2), x[4 * w + 2], s0);
            s1 = __builtin_fmaf(ub(v, 3), x[4 * w + 3], s1);
        }
        return f16_bits_to_f32(d) * __builtin_fmaf(-128.0f, xsum, s0 + s1);
    }
};
template <> struct Unit<RFQ_GGUF_Q8_0> {
    static constexpr bool NEEDS_XSUM = true;
    Window<8> w;
    __device__ __forceinline__ void load(const uint8_t *row, int u) { w.load(row + (size_t)u * 34); }
    __device__ __forceinline__ void load_bytes(const uint8_t *row, int u) { w.load_bytes<2>(row + (size_t)u * 34); }
    __device__ __forceinline__ Opened<RFQ_GGUF_Q8_0> open() const
    {
        Opened<RFQ_GGUF_Q8_0> r;
        r.d = (uint16_t)w.head();
        w.piece<2>(r.q.v);
        return r;
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const { return open().dot(x, xsum); }
};

// Unit u of a 144-byte super-block: chunk c = u >> 1 of 64 elements, half h = u & 1
// (low or high nibbles of the chunk's 32 bytes); value = d * sc * q - dmin * m.
template <> struct Unit<RFQ_GGUF_Q4_K> {
    static constexpr bool NEEDS_XSUM = true;
    uint32_t dd, s0, s1, s2; U8 q; int sub;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *blk = row + (size_t)(u >> 3) * 144;
        sub = u & 7;
        dd = ld<uint32_t>(blk);
        s0 = ld<uint32_t>(blk + 4); s1 = ld<uint32_t>(blk + 8); s2 = ld<uint32_t>(blk + 12);
        q = ld<U8>(blk + 16 + 32 * (sub >> 1));
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        const uint32_t sm = gguf_scale_min_k4(sub, s0, s1, s2);
        const int sh = 4 * (sub & 1);
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            uint32_t v = (q.v[w] >> sh) & 0x0F0F0F0Fu;
            a0 = __builtin_fmaf(ub(v, 0), x[4 * w], a0);
            a1 = __builtin_fmaf(ub(v, 1), x[4 * w + 1], a1);
            a0 = __builtin_fmaf(ub(v, 2), x[4 * w + 2], a0);
            a1 = __builtin_fmaf(ub(v, 3), x[4 * w + 3], a1);
        }
        const float d1 = f16_bits_to_f32((uint16_t)(dd & 0xFFFFu)) * (float)(sm & 255u);
        const float m1 = f16_bits_to_f32((uint16_t)(dd >> 16)) * (float)(sm >> 8);
        return __builtin_fmaf(d1, a0 + a1, -m1 * xsum);
    }
};

// Unit u of a 210-byte super-block: half n = (u >> 2) & 1 of 128 elements, quarter t = u & 3:
// low nibbles from ql[64 n + 32 (t & 1) + l] (>> 4 for t >= 2), bits 4-5 from qh[32 n + l] >> 2 t,
// scales sc[8 n + 2 t + l / 16]; value = d * sc * (q - 32).
template <> struct Opened<RFQ_GGUF_Q6_K> {
    U8 ql, qh; uint16_t sc2, d; int t;
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        const int shl = 4 * (t >> 1), shh = 2 * t;
        float a[2] = {0.f, 0.f}, xs0 = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const uint32_t lo = (ql.v[w] >> shl) & 0x0F0F0F0Fu, hi = (qh.v[w] >> shh) & 0x03030303u;
            const uint32_t v = lo | (hi << 4);
            float s = a[w >> 2];
            s = __builtin_fmaf(ub(v, 0), x[4 * w], s);
            s = __builtin_fmaf(ub(v, 1), x[4 * w + 1], s);
            s = __builtin_fmaf(ub(v, 2), x[4 * w + 2], s);
            s = __builtin_fmaf(ub(v, 3), x[4 * w + 3], s);
            a[w >> 2] = s;
            if (w < 4) xs0 += (x[4 * w] + x[4 * w + 1]) + (x[4 * w + 2] + x[4 * w + 3]);
        }
        const float g0 = __builtin_fmaf(-32.0f, xs0, a[0]), g1 = __builtin_fmaf(-32.0f, xsum - xs0, a[1]);
        const float c0 = (float)(int8_t)(sc2 & 255u), c1 = (float)(int8_t)(sc2 >> 8);
        return f16_bits_to_f32(d) * __builtin_fmaf(c0, g0, c1 * g1);
    }
};
template <> struct Unit<RFQ_GGUF_Q6_K> {
    static constexpr bool NEEDS_XSUM = true;
    Window<8> wl, wh; uint16_t sc2, sc2b, d; int t;
    template <bool BYTES> __device__ __forceinline__ void load_as(const uint8_t *row, int u)
    {
        const uint8_t *blk = row + (size_t)(u >> 3) * 210;
        const int half = (u >> 2) & 1;
        t = u & 3;
        // (the scales of quarter t | 2, which shares this unit's bytes: what the paired form multiplies as well)
        sc2b = ld<uint16_t>(blk + 192 + 8 * half + 2 * (t | 2));
        if constexpr (BYTES) {
            wl.load_bytes<0>(blk + 64 * half + 32 * (t & 1));
            wh.load_bytes<0>(blk + 128 + 32 * half);
        } else {
            wl.load(blk + 64 * half + 32 * (t & 1));
            wh.load(blk + 128 + 32 * half);
        }
        sc2 = ld<uint16_t>(blk + 192 + 8 * half + 2 * t);
        d = ld<uint16_t>(blk + 208);
    }
    __device__ __forceinline__ void load(const uint8_t *row, int u) { load_as<false>(row, u); }
    __device__ __forceinline__ void load_bytes(const uint8_t *row, int u) { load_as<true>(row, u); }
    __device__ __forceinline__ Opened<RFQ_GGUF_Q6_K> open() const
    {
        Opened<RFQ_GGUF_Q6_K> r;
        wl.piece<0>(r.ql.v);
        wh.piece<0>(r.qh.v);
        r.sc2 = sc2; r.d = d; r.t = t;
        return r;
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const { return open().dot(x, xsum); }
};

// ---- the matmul module's own decoders (src/kernels/matmul/quantized/) -------------
// Multiplied by the one-row-per-wavefront kernel only (the reference multiplies them in the other orientation,
// see gemv_kn_kernel).

template <> struct Unit<RFQ_MM_Q8_0> {                 // quantized/q8_0.rs:34-52: scale * (byte as i8)
    static constexpr bool NEEDS_XSUM = false;
    float scale; U8 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *p = row + (size_t)u * 36;
        scale = ld<float>(p);
        q = ld<U8>(p + 4);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int d = 0; d < 8; d++) {
            s0 = __builtin_fmaf((float)(int8_t)(q.v[d] & 255u), x[4 * d], s0);
            s1 = __builtin_fmaf((float)(int8_t)((q.v[d] >> 8) & 255u), x[4 * d + 1], s1);
            s0 = __builtin_fmaf((float)(int8_t)((q.v[d] >> 16) & 255u), x[4 * d + 2], s0);
            s1 = __builtin_fmaf((float)(int8_t)(q.v[d] >> 24), x[4 * d + 3], s1);
        }
        return scale * (s0 + s1);
    }
};

template <> struct Unit<RFQ_MM_Q4_K> {                 // quantized/q4_k.rs:101-143: nibbles at 32 + 20 * sb
    static constexpr bool NEEDS_XSUM = true;
    uint16_t sc; int8_t mn; U4 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *blk = row + (size_t)(u >> 3) * 256;
        int sb = u & 7;
        sc = ld<uint16_t>(blk + 2 * sb);
        mn = (int8_t)blk[16 + sb];
        q = ld_once<U4>(blk + 32 + 20 * sb);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float xsum) const
    {
        return __builtin_fmaf(f16_bits_to_f32_mm(sc), nib_dot_lo_first(q, x), (float)mn * xsum);
    }
};

template <> struct Unit<RFQ_MM_Q6_K> : Unit<RFQ_Q6_K> { // quantized/q6_k.rs:101-143: scales through f16_to_f32_cpu
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        float a = dot16(q.v[0], q.v[1], q.v[2], &x[0]);
        float b = dot16(q.v[3], q.v[4], q.v[5], &x[16]);
        return __builtin_fmaf(f16_bits_to_f32_mm((uint16_t)(sc2 & 0xFFFFu)), a, f16_bits_to_f32_mm((uint16_t)(sc2 >> 16)) * b);
    }
};

template <int FMT> __host__ __device__ constexpr size_t row_bytes(int k)
{
    return (size_t)(k / Fmt<FMT>::BE) * Fmt<FMT>::BB;
}

__device__ __forceinline__ void load_x32(const float *p, float (&x)[32])
{
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float4 v = ld<float4>(reinterpret_cast<const uint8_t *>(p + 4 * i));
        x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
    }
}

__device__ __forceinline__ float sum32(const float (&x)[32])
{
    float a = 0.f, b = 0.f, c = 0.f, d = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i += 4) { a += x[i]; b += x[i + 1]; c += x[i + 2]; d += x[i + 3]; }
    return (a + b) + (c + d);
}

// ---- optional fusion around the m == 1 kernels -------------------------------
//
// FUSE kernels take two run-time options.  norm_w != nullptr: the vector that
// is multiplied is RMSNorm(x) * norm_w (kernels/rms_norm.hip:40-84) instead
// of x; since the normalisation is one factor 1 / sqrt(mean(x^2) + eps) for the
// whole vector, x * norm_w goes through the dot products and the factor is
// applied to each result.  glu != 0: the n rows are an interleaving of two
// matrices (row 2j = row j of w, row 2j+1 = row j of w2: gate and up
// projections sharing x) and y[j] = swiglu(row 2j, row 2j+1) as the reference
// defines it (kernels/swiglu.hip:40-62): gate * (up * sigmoid(up)).
struct GemvFuse {
    const uint8_t *w2;
    const float *norm_w;
    float eps;
    int glu;
};

__device__ __forceinline__ float swiglu_ref(float gate, float up)
{
    return gate * (up * (1.0f / (1.0f + expf(-up))));
}

// Row r of the (possibly interleaved) matrix.
template <bool FUSE>
__device__ __forceinline__ const uint8_t *fused_row(const uint8_t *w, const GemvFuse &f, int r, size_t rb)
{
    if constexpr (FUSE) {
        if (f.glu) return ((r & 1) ? f.w2 : w) + (size_t)(r >> 1) * rb;
    }
    return w + (size_t)r * rb;
}

// Results of one group of R rows (res[i] valid in every lane of each of the
// team's WPR wavefronts) go to y.  `part` is [R][WAVES] floats of LDS; with
// WPR > 1 every wavefront of the block must call this the same number of times.
// ONE_BARRIER: the caller alternates between two `part` arrays from group to group, so a group's partial sums cannot
// be overwritten before they are read and the second barrier is not needed.
template <int R, int WPR, bool FUSE, int WAVES = 4, bool ONE_BARRIER = false>
__device__ __forceinline__ void store_group(const float (&res)[R], float (*part)[WAVES], float *__restrict__ y, int row_first,
                                            int row_end, int lane, int wave, const GemvFuse &f, float rinv)
{
    const int team = wave / WPR, wit = wave % WPR;
    if (WPR == 1) {
        if (lane == 0) {
            if (FUSE && f.glu) {
#pragma unroll
                for (int i = 0; i + 1 < R; i += 2) {
                    int r = row_first + i;
                    if (r < row_end) y[r >> 1] = swiglu_ref(res[i] * rinv, res[i + 1] * rinv);
                }
            } else {
#pragma unroll
                for (int i = 0; i < R; i++) {
                    int r = row_first + i;
                    if (r < row_end) y[r] = FUSE ? res[i] * rinv : res[i];
                }
            }
        }
    } else {
        if (lane == 0) {
#pragma unroll
            for (int i = 0; i < R; i++) part[i][wave] = res[i];
        }
        __syncthreads();
        if (wit == 0) {
            const int li = lane < R ? lane : R - 1;
            int r = row_first + li;
            float t = 0.f;
#pragma unroll
            for (int q = 0; q < WPR; q++) t += part[li][team * WPR + q];
            if (FUSE) {
                t *= rinv;
                float other = dpp_xor1_f(t);           // the up row's result sits in the odd neighbour lane
                if (f.glu) {
                    if (lane < R && (lane & 1) == 0 && r < row_end) y[r >> 1] = swiglu_ref(t, other);
                } else if (lane < R && r < row_end) {
                    y[r] = t;
                }
            } else if (lane < R && r < row_end) {
                y[r] = t;
            }
        }
        if constexpr (!ONE_BARRIER) __syncthreads();
    }
}

// The plain GEMV of the integer-dot kernel reduces the R rows of a group together: every lane keeps its partial sum of
// each row until the group is done, rows16_sum_of leaves lane l with the sum of row l % 8 over its 16-lane row (25
// instructions where R wavefront sums took 11 each), and the four lane rows of each of the team's wavefronts meet in
// LDS: part[row][4 * wavefront + lane row].  The caller alternates between two `part` arrays from group to group, so a
// group's partial sums cannot be overwritten before they are read and one barrier per group is enough (none for a team
// of one wavefront, whose LDS operations complete in order).
constexpr int JOINT_ROWS = 8;
template <int FMT> struct JointRows { static constexpr bool value = false; };
template <> struct JointRows<RFQ_Q4_0> { static constexpr bool value = true; };
template <> struct JointRows<RFQ_Q6_K> { static constexpr bool value = true; };
template <> struct JointRows<RFQ_GGUF_Q4_0> { static constexpr bool value = true; };
template <> struct JointRows<RFQ_GGUF_Q8_0> { static constexpr bool value = true; };
template <> struct JointRows<RFQ_GGUF_Q6_K> { static constexpr bool value = true; };
template <int R, int WPR, int WAVES>
__device__ __forceinline__ void store_group_joint(const float (&acc)[R], float (*part)[WAVES * 4], float *__restrict__ y,
                                                  int row_first, int row_end, int lane, int wave)
{
    static_assert(R <= JOINT_ROWS, "at most eight rows per group");
    constexpr int M = R <= 2 ? 2 : (R <= 4 ? 4 : 8);
    float a[M];
#pragma unroll
    for (int i = 0; i < M; i++) a[i] = i < R ? acc[i] : 0.f;
    const float f = rows16_sum_of<M>(a, lane);
    const int team = wave / WPR, wit = wave % WPR;
    if ((lane & 15) < R) part[lane & 15][wave * 4 + (lane >> 4)] = f;   // (lanes 8..15 of a row repeat 0..7: same value, same slot)
    if (WPR > 1) __syncthreads();
    if (wit == 0 && lane < R) {
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < 4 * WPR; q++) t += part[lane][team * WPR * 4 + q];
        const int r = row_first + lane;
        if (r < row_end) y[r] = t;
    }
}

// ---- m == 1, x resident in registers ----------------------------------------
//
// Block = 4 wavefronts = 4 / WPR teams.  Lane `tl` of a team (0 .. 64*WPR-1)
// owns units tl + j * 64 * WPR, j < UPL, of EVERY row the team visits.  A team
// walks `groups * R` consecutive rows, R (a compile-time constant) at a time,
// with a rolling prefetch: three rows are in flight per lane, and as soon as a
// row has been consumed its slot takes the row three further on, so loads and
// arithmetic overlap.  Rows past the end
// re-read the team's last valid row (same addresses, served by the cache) and
// their result is dropped; lanes past the end of a row do the same with the
// row's last unit.  HBM latency, not bandwidth, bounds a wavefront that has a
// single row in flight, hence the depth.
template <int FMT, int UPL, int WPR, int R, bool FUSE>
__global__ void __launch_bounds__(256)
gemv_xreg_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y, int n, int k,
                 int groups, GemvFuse f, int xstage)
{
    constexpr int TEAMS = 4 / WPR, TL = 64 * WPR;
    // rows in flight per lane: three, or five in the form with one unit per lane and two wavefronts per row
    // (Q6_K 14336 x 4096 in that form: 14.6 us with three, 13.8 us with five)
    // (MXFP4 in that form, whose look-ups go through LDS: three -- 32000 x 4096 16.3 -> 15.2 us, level at 8192 rows;
    // MXFP6 with three: 32000 x 4096 23.1 -> 24.7)
    // (MXFP6 with two units per lane: two -- 4096 x 8192 9.36 -> 8.69 us, 8192 x 8192 13.5 -> 12.8, 4096 x 5120 8.05 -> 7.57,
    // 4096 x 14336 14.6 -> 14.0, 28672 x 8192 38.0 -> 37.8; MXFP4 28672 x 8192 with two 28.0 -> 29.0, Q6_K mixed)
    // (groups of up to four rows, any format: two -- Q6_K 4096 x 8192 8.40 -> 7.76 us, 4096 x 5120 6.85 -> 6.34,
    // 4096 x 6144 7.31 -> 6.83, MXFP4 4096 x 5120 6.60 -> 6.44; with longer groups Q6_K and MXFP4 measured mixed)
    constexpr int DW = (UPL == 1 && WPR == 2) ? (FMT == RFQ_MXFP4 ? 3 : 5) : ((FMT == RFQ_MXFP6_E2M3 || R <= 4) ? 2 : 3);
    constexpr int D = R < DW ? R : DW;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int team = wave / WPR, wit = wave % WPR;
    const int tl = wit * 64 + lane;
    const int ku = k >> 5;
    const size_t rb = row_bytes<FMT>(k);

    float xs[UPL][32], xsum[UPL];
    bool live[UPL];
    int unit[UPL];
#pragma unroll
    for (int j = 0; j < UPL; j++) {
        int u = tl + j * TL;
        live[j] = u < ku;
        unit[j] = live[j] ? u : ku - 1;
    }
    const bool norm = FUSE && f.norm_w != nullptr;

    // x reaches the lanes through LDS (xstage != 0: the launcher gave the block k floats of dynamic LDS): the block
    // fetches it once with consecutive lanes on consecutive 16-byte pieces, and a lane then reads its units from
    // LDS.  Every lane fetching its own 128-byte unit from memory instead costs a wavefront eight load
    // instructions that each touch 64 different cache lines -- with sixteen short-lived wavefronts per CU that
    // address traffic, not the weight stream, set the kernel's time (Q6_K 14336 x 4096: 6.4 us of 13.9).
    // LDS layout: 16-byte piece q (0..7) of unit u at ((q * ku + u) * 16), so consecutive lanes read consecutive pieces.
    extern __shared__ __attribute__((aligned(16))) float xstage_lds[];
    // pieces a thread requests before the first rows' weights: all of x for the rows this form takes, up to the 8192
    // values that are staged this way (a piece requested behind the weights would be served behind them, and the
    // barrier below would hold every wavefront's first dot until then)
    constexpr int XQ = 2 * UPL * WPR < 8 ? (2 * UPL * WPR < 4 ? 4 : 2 * UPL * WPR) : 8;
    const int pieces = ku * 8;
    float4 xq[XQ], nq[FUSE ? XQ : 1];
    if (xstage) {
#pragma unroll
        for (int i = 0; i < XQ; i++) {
            const int p = threadIdx.x + 256 * i;
            if (p < pieces) {
                xq[i] = ld<float4>(reinterpret_cast<const uint8_t *>(x + (size_t)p * 4));
                if constexpr (FUSE) {
                    if (norm) nq[i] = ld<float4>(reinterpret_cast<const uint8_t *>(f.norm_w + (size_t)p * 4));
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < UPL; j++) load_x32(x + (size_t)unit[j] * 32, xs[j]);
    }
    float nws[(FUSE ? UPL : 1)][32];
    if (norm && !xstage) {
#pragma unroll
        for (int j = 0; j < UPL; j++) load_x32(f.norm_w + (size_t)unit[j] * 32, nws[FUSE ? j : 0]);
    }

    unit_tables_init<FMT>();
    __shared__ float part[R][4];
    // (the plain GEMV reduces a group's rows together, see store_group_joint: MXFP6 11008 x 4096 10.9 -> 10.6 us, 32000 x
    // 4096 24.0 -> 23.1; Q6_K 32000 x 4096 24.9 -> 24.2; level elsewhere)
    constexpr bool XJOINT = !FUSE;
    __shared__ float partj[XJOINT ? 2 : 1][JOINT_ROWS][XJOINT ? 16 : 1];
    (void)partj;
    const int rows_per_team = groups * R;
    const int row0 = (blockIdx.x * TEAMS + team) * rows_per_team;
    int row_end = row0 + rows_per_team;
    if (row_end > n) row_end = n;
    const int row_last = row_end > row0 ? row_end - 1 : (n - 1);

    Unit<FMT> buf[D][UPL];
    auto load_row = [&](int slot, int i) {
        int r = row0 + i;
        if (r > row_last) r = row_last;
        const uint8_t *row = fused_row<FUSE>(w, f, r, rb);
#pragma unroll
        for (int j = 0; j < UPL; j++) buf[slot][j].load(row, unit[j]);
    };
    // x first, then the first rows, and only then the first use of x: the
    // weight loads are already in flight while x is staged and its sums are formed.
#pragma unroll
    for (int d = 0; d < D; d++) load_row(d, d);
    float rinv = 1.0f;
    if (xstage) {
        float ssq = 0.f;
        auto put = [&](int p, float4 v, float4 nv) {
            if constexpr (FUSE) {
                if (norm) {
                    ssq = __builtin_fmaf(v.x, v.x, ssq); ssq = __builtin_fmaf(v.y, v.y, ssq);
                    ssq = __builtin_fmaf(v.z, v.z, ssq); ssq = __builtin_fmaf(v.w, v.w, ssq);
                    v.x *= nv.x; v.y *= nv.y; v.z *= nv.z; v.w *= nv.w;
                }
            }
            *reinterpret_cast<float4 *>(xstage_lds + ((size_t)(p & 7) * ku + (p >> 3)) * 4) = v;
        };
#pragma unroll
        for (int i = 0; i < XQ; i++) {
            const int p = threadIdx.x + 256 * i;
            if (p < pieces) put(p, xq[i], nq[FUSE ? i : 0]);
        }
        for (int p = threadIdx.x + 256 * XQ; p < pieces; p += 256) {  // (longer rows: the rest, behind the first rows' loads)
            float4 v = ld<float4>(reinterpret_cast<const uint8_t *>(x + (size_t)p * 4)), nv = v;
            if constexpr (FUSE) {
                if (norm) nv = ld<float4>(reinterpret_cast<const uint8_t *>(f.norm_w + (size_t)p * 4));
            }
            put(p, v, nv);
        }
        if constexpr (FUSE) {
            if (norm) {
                ssq = wave_sum(ssq);
                if (lane == 0) part[0][wave] = ssq;
            }
        }
        __syncthreads();
        if constexpr (FUSE) {
            if (norm) rinv = 1.0f / sqrtf(((part[0][0] + part[0][1]) + (part[0][2] + part[0][3])) / (float)k + f.eps);
        }
#pragma unroll
        for (int j = 0; j < UPL; j++) {
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const float4 v = *reinterpret_cast<const float4 *>(xstage_lds + ((size_t)q * ku + unit[j]) * 4);
                xs[j][4 * q] = v.x; xs[j][4 * q + 1] = v.y; xs[j][4 * q + 2] = v.z; xs[j][4 * q + 3] = v.w;
            }
        }
        if constexpr (FUSE) {
            if (norm) __syncthreads();                            // part[0] is reused by the first group's results
        }
    } else if (norm) {
        // every team holds all of x: its own sum of squares, no exchange between teams
        float ssq = 0.f;
#pragma unroll
        for (int j = 0; j < UPL; j++) {
            float sj = 0.f;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                sj = __builtin_fmaf(xs[j][i], xs[j][i], sj);
                xs[j][i] *= nws[FUSE ? j : 0][i];
            }
            ssq += live[j] ? sj : 0.f;
        }
        ssq = wave_sum(ssq);
        if (WPR > 1) {
            if (lane == 0) part[0][wave] = ssq;
            __syncthreads();
            ssq = 0.f;
#pragma unroll
            for (int q = 0; q < WPR; q++) ssq += part[0][team * WPR + q];
            __syncthreads();
        }
        rinv = 1.0f / sqrtf(ssq / (float)k + f.eps);
    }
#pragma unroll
    for (int j = 0; j < UPL; j++) xsum[j] = Unit<FMT>::NEEDS_XSUM ? sum32(xs[j]) : 0.f;

    for (int g = 0; g < groups; g++) {
        const int base = g * R;
        if (g > 0) {
#pragma unroll
            for (int d = 0; d < D; d++) load_row(d, base + d);
        }
        float res[R];
#pragma unroll
        for (int i = 0; i < R; i++) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < UPL; j++) {
                float t = buf[i % D][j].dot(xs[j], xsum[j]);
                acc += live[j] ? t : 0.f;
            }
            if (i + D < R) load_row(i % D, base + i + D); // the slot just consumed takes the row D further on
            if constexpr (XJOINT) res[i] = acc;
            else res[i] = wave_sum(acc);
        }
        // (`groups` is uniform over the block: every wavefront stores the same number of groups)
        if constexpr (XJOINT) store_group_joint<R, WPR, 4>(res, partj[g & 1], y, row0 + base, row_end, lane, wave);
        else store_group<R, WPR, FUSE>(res, part, y, row0 + base, row_end, lane, wave, f, rinv);
    }
}

// ---- m == 1, integer dot products ---------------------------------------------
//
// The float kernel above spends ~3 VALU instructions per weight (convert,
// multiply-add, unpack) and is bound by them, not by HBM.  Here x is turned,
// once per workgroup, into block-fixed-point: per unit of 32 values a power of
// two s and 22-bit integers X_i = round(x_i / s), |X_i| < 2^22, split into
// three byte limbs (X = top * 65536 + mid * 256 + low; top signed, mid and low
// unsigned) and packed four elements to a dword in the order the weight bytes
// unpack to.  The weights stay integers too, so a unit's 32 products are
// 4-way byte dot products (v_dot4) with exact int32 sums:
//     sum_i q_i x_i  =  s * (65536 * sum q.top + 256 * sum q.mid + sum q.low)
// about 1.1 instructions per weight, and more accurate than an fp32
// running sum (the only roundings: x to 22 bits relative to the unit's largest
// value, and the final scaling).  A non-finite x value poisons its unit's s
// with NaN, as it would poison the float sum.
//
// LDS holds, per unit, 24 limb dwords + s + sum(x) + the sums of its two halves (stride 28 dwords).

struct XPrep { uint32_t l[24]; float s, xsum, xh0, xh1; };   // xh0, xh1: sums of elements 0..15 and 16..31

// Byte-transpose four 24-bit integers into (low, mid, top) limb dwords.
__device__ __forceinline__ void limbs4(uint32_t x0, uint32_t x1, uint32_t x2, uint32_t x3, uint32_t *out3)
{
    uint32_t t01l = __builtin_amdgcn_perm(x1, x0, 0x05010400u); // b0x0 b0x1 b1x0 b1x1
    uint32_t t23l = __builtin_amdgcn_perm(x3, x2, 0x05010400u);
    uint32_t t01h = __builtin_amdgcn_perm(x1, x0, 0x0C0C0602u); // b2x0 b2x1 0 0
    uint32_t t23h = __builtin_amdgcn_perm(x3, x2, 0x0C0C0602u);
    out3[0] = __builtin_amdgcn_perm(t23l, t01l, 0x05040100u);
    out3[1] = __builtin_amdgcn_perm(t23l, t01l, 0x07060302u);
    out3[2] = __builtin_amdgcn_perm(t23h, t01h, 0x05040100u);
}

// One thread converts half a unit (16 consecutive x) and writes 12 limb
// dwords; the two threads of a unit are neighbouring lanes.
// NIBBLE: groups are elements 8d+{0,2,4,6} then 8d+{1,3,5,7} (low nibbles,
// then high nibbles of four consecutive bytes); otherwise 4g+{0,1,2,3}.
// TOPOFF: added to every integer before the split (2^22 makes the top limb
// unsigned, 0..127, for formats whose weight bytes exceed 127).
__device__ __forceinline__ void prep_load(const float *xp, float (&xv)[16])
{
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float4 v = ld<float4>(reinterpret_cast<const uint8_t *>(xp + 4 * i));
        xv[4 * i] = v.x; xv[4 * i + 1] = v.y; xv[4 * i + 2] = v.z; xv[4 * i + 3] = v.w;
    }
}

template <bool NIBBLE, uint32_t TOPOFF>
__device__ __forceinline__ void prep_convert(const float (&xv)[16], int half, uint32_t *lds_unit)
{
    float m = 0.f, sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) { m = fmaxf(m, fabsf(xv[i])); sum += xv[i]; }
    bool bad = false;
#pragma unroll
    for (int i = 0; i < 16; i++) bad |= !(fabsf(xv[i]) <= 3.40282347e+38f);
    const float half_sum = sum;
    m = fmaxf(m, dpp_xor1_f(m));
    sum += dpp_xor1_f(sum);
    bad |= __builtin_amdgcn_update_dpp(0, (int)bad, 0xB1, 0xF, 0xF, true) != 0;
    int e = (int)(__float_as_uint(m) >> 23);          // biased exponent of the largest |x|
    int ie = 275 - e;                                 // 1/s = 2^(21 - (e - 127))
    if (ie > 254) ie = 254;
    float inv_s = __uint_as_float((uint32_t)ie << 23);
    float sc = ie == 254 ? __uint_as_float(0x00400000u) : __uint_as_float((uint32_t)(254 - ie) << 23);
    if (bad) sc = __uint_as_float(0x7FC00000u);
    uint32_t X[16];
#pragma unroll
    for (int i = 0; i < 16; i++)
        X[i] = __float_as_uint(__builtin_fmaf(xv[i], inv_s, 12582912.0f)) - 0x4B400000u + TOPOFF;
    uint32_t *o = lds_unit + half * 12;
    if (NIBBLE) {
#pragma unroll
        for (int d = 0; d < 2; d++) {
            limbs4(X[8 * d], X[8 * d + 2], X[8 * d + 4], X[8 * d + 6], o + (2 * d) * 3);
            limbs4(X[8 * d + 1], X[8 * d + 3], X[8 * d + 5], X[8 * d + 7], o + (2 * d + 1) * 3);
        }
    } else {
#pragma unroll
        for (int g = 0; g < 4; g++) limbs4(X[4 * g], X[4 * g + 1], X[4 * g + 2], X[4 * g + 3], o + g * 3);
    }
    if (half == 0) {
        lds_unit[24] = __float_as_uint(sc);
        lds_unit[25] = __float_as_uint(sum);
    }
    lds_unit[26 + half] = __float_as_uint(half_sum);
}

// The same conversion with four threads per unit (neighbouring lanes), eight consecutive x each:
// a quarter is two limb groups in either order, so thread q of a unit writes limb dwords 6q .. 6q+5.
__device__ __forceinline__ float dpp_xor2_f(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
}

__device__ __forceinline__ void prep_load8(const float *xp, float (&xv)[8])
{
#pragma unroll
    for (int i = 0; i < 2; i++) {
        float4 v = ld<float4>(reinterpret_cast<const uint8_t *>(xp + 4 * i));
        xv[4 * i] = v.x; xv[4 * i + 1] = v.y; xv[4 * i + 2] = v.z; xv[4 * i + 3] = v.w;
    }
}

// QSUM: the slot of the first half's sum holds s * sum(X) instead, the sum of the unit's values as rounded to block
// fixed point.  A format that subtracts an offset times the sum of x from its byte dot products (MXFP4: 16) takes it:
// the offset then cancels exactly, where the sum of the unrounded x would leave offset * s * (sum of the 32 rounding
// errors) in every row alike.
template <bool NIBBLE, uint32_t TOPOFF, bool QSUM = false>
__device__ __forceinline__ void prep_convert_quarter(const float (&xv)[8], int quarter, uint32_t *lds_unit)
{
    float m = 0.f, sum = 0.f;
    uint32_t top = 0;                                 // largest |x| bit pattern: at or above 0x7F800000 means inf or NaN
#pragma unroll
    for (int i = 0; i < 8; i++) {
        m = fmaxf(m, fabsf(xv[i]));
        sum += xv[i];
        const uint32_t a = __float_as_uint(xv[i]) & 0x7FFFFFFFu;
        top = a > top ? a : top;
    }
    bool bad = top >= 0x7F800000u;
    m = fmaxf(m, dpp_xor1_f(m));
    sum += dpp_xor1_f(sum);
    bad |= __builtin_amdgcn_update_dpp(0, (int)bad, 0xB1, 0xF, 0xF, true) != 0;
    const float half_sum = sum;
    m = fmaxf(m, dpp_xor2_f(m));
    sum += dpp_xor2_f(sum);
    bad |= __builtin_amdgcn_update_dpp(0, (int)bad, 0x4E, 0xF, 0xF, true) != 0;
    int e = (int)(__float_as_uint(m) >> 23);          // biased exponent of the largest |x|
    int ie = 275 - e;                                 // 1/s = 2^(21 - (e - 127))
    if (ie > 254) ie = 254;
    float inv_s = __uint_as_float((uint32_t)ie << 23);
    float sc = ie == 254 ? __uint_as_float(0x00400000u) : __uint_as_float((uint32_t)(254 - ie) << 23);
    if (bad) sc = __uint_as_float(0x7FC00000u);
    uint32_t X[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
        X[i] = __float_as_uint(__builtin_fmaf(xv[i], inv_s, 12582912.0f)) - 0x4B400000u + TOPOFF;
    if constexpr (QSUM) {
        int isum = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) isum += (int)(X[i] - TOPOFF);
        isum += __builtin_amdgcn_update_dpp(0, isum, 0xB1, 0xF, 0xF, true);
        isum += __builtin_amdgcn_update_dpp(0, isum, 0x4E, 0xF, 0xF, true);
        if (quarter == 0) lds_unit[26] = __float_as_uint((float)isum * sc);
    }
    uint32_t *o = lds_unit + quarter * 6;
    if (NIBBLE) {
        limbs4(X[0], X[2], X[4], X[6], o);
        limbs4(X[1], X[3], X[5], X[7], o + 3);
    } else {
        limbs4(X[0], X[1], X[2], X[3], o);
        limbs4(X[4], X[5], X[6], X[7], o + 3);
    }
    if (quarter == 0) {
        lds_unit[24] = __float_as_uint(sc);
        lds_unit[25] = __float_as_uint(sum);
    }
    if constexpr (!QSUM) {
        if ((quarter & 1) == 0) lds_unit[26 + (quarter >> 1)] = __float_as_uint(half_sum);
    }
}

// sum_i nibble_i * X_i for 16 weight bytes in low-nibble-first order.
__device__ __forceinline__ float nib_idot(const U4 &q, const XPrep &xp)
{
    uint32_t alo = 0, amid = 0;
    int atop = 0;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        uint32_t lo = q.v[d] & 0x0F0F0F0Fu, hi = (q.v[d] >> 4) & 0x0F0F0F0Fu;
        const uint32_t *L = &xp.l[(2 * d) * 3], *H = &xp.l[(2 * d + 1) * 3];
        alo = __builtin_amdgcn_udot4(lo, L[0], alo, false);
        amid = __builtin_amdgcn_udot4(lo, L[1], amid, false);
        atop = __builtin_amdgcn_sdot4((int)lo, (int)L[2], atop, false);
        alo = __builtin_amdgcn_udot4(hi, H[0], alo, false);
        amid = __builtin_amdgcn_udot4(hi, H[1], amid, false);
        atop = __builtin_amdgcn_sdot4((int)hi, (int)H[2], atop, false);
    }
    return __builtin_fmaf((float)atop, 65536.0f, __builtin_fmaf((float)amid, 256.0f, (float)alo));
}

template <int FMT> struct IUnit;
template <int FMT> struct WantsQSum { static constexpr bool value = false; };
template <> struct WantsQSum<RFQ_MXFP4> { static constexpr bool value = true; };

template <> struct IUnit<RFQ_Q4_K> : Unit<RFQ_Q4_K> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = true;
    static constexpr uint32_t TOPOFF = 0;
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        return __builtin_fmaf(f16_bits_to_f32(sc) * xp.s, nib_idot(q, xp), (float)mn * xp.xsum);
    }
};

template <> struct IUnit<RFQ_Q4_0> : Unit<RFQ_Q4_0> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = true;
    static constexpr uint32_t TOPOFF = 0;
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        return scale * __builtin_fmaf(xp.s, nib_idot(q, xp), -8.0f * xp.xsum);
    }
};

template <> struct IUnit<RFQ_Q8_0> : Unit<RFQ_Q8_0> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0x400000u; // weight bytes reach 255: keep every limb unsigned
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        uint32_t alo = 0, amid = 0, atop = 0, bsum = 0;
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const uint32_t *L = &xp.l[g * 3];
            alo = __builtin_amdgcn_udot4(q.v[g], L[0], alo, false);
            amid = __builtin_amdgcn_udot4(q.v[g], L[1], amid, false);
            atop = __builtin_amdgcn_udot4(q.v[g], L[2], atop, false);
            bsum = __builtin_amdgcn_udot4(q.v[g], 0x01010101u, bsum, false);
        }
        // top limbs carry +64: sum b*(top+64) - 64*sum b
        float S = __builtin_fmaf((float)((int)atop - 64 * (int)bsum), 65536.0f,
                                 __builtin_fmaf((float)amid, 256.0f, (float)alo));
        return scale * __builtin_fmaf(xp.s, S, -128.0f * xp.xsum);
    }
};

// The matmul module's variants of the two integer formats: the same sums, the f16 scale widened the module's own
// way (Q4_K), the bytes read as int8 (Q8_0: one XOR per dword makes them the offset-binary bytes of the sum above).
template <> struct IUnit<RFQ_MM_Q4_K> : Unit<RFQ_MM_Q4_K> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = true;
    static constexpr uint32_t TOPOFF = 0;
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        return __builtin_fmaf(f16_bits_to_f32_mm(sc) * xp.s, nib_idot(q, xp), (float)mn * xp.xsum);
    }
};

template <> struct IUnit<RFQ_MM_Q8_0> : Unit<RFQ_MM_Q8_0> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0x400000u;
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        uint32_t alo = 0, amid = 0, atop = 0, bsum = 0;
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const uint32_t *L = &xp.l[g * 3];
            const uint32_t b = q.v[g] ^ 0x80808080u;               // int8 + 128
            alo = __builtin_amdgcn_udot4(b, L[0], alo, false);
            amid = __builtin_amdgcn_udot4(b, L[1], amid, false);
            atop = __builtin_amdgcn_udot4(b, L[2], atop, false);
            bsum = __builtin_amdgcn_udot4(b, 0x01010101u, bsum, false);
        }
        float S = __builtin_fmaf((float)((int)atop - 64 * (int)bsum), 65536.0f,
                                 __builtin_fmaf((float)amid, 256.0f, (float)alo));
        return scale * __builtin_fmaf(xp.s, S, -128.0f * xp.xsum);
    }
};

// GGUF layouts: x limbs in plain order (group g = elements 4g .. 4g+3).

template <> struct IUnit<RFQ_GGUF_Q4_0> : Unit<RFQ_GGUF_Q4_0> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0;
    // low nibbles of dword w are elements 4w .. 4w+3 (group w), high nibbles elements 16+4w .. (group 4+w)
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        const Opened<RFQ_GGUF_Q4_0> b = open();
        const U4 &q = b.q;
        const uint16_t d = b.d;
        uint32_t alo = 0, amid = 0;
        int atop = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            uint32_t lo = q.v[w] & 0x0F0F0F0Fu, hi = (q.v[w] >> 4) & 0x0F0F0F0Fu;
            const uint32_t *L = &xp.l[w * 3], *H = &xp.l[(4 + w) * 3];
            alo = __builtin_amdgcn_udot4(lo, L[0], alo, false);
            amid = __builtin_amdgcn_udot4(lo, L[1], amid, false);
            atop = __builtin_amdgcn_sdot4((int)lo, (int)L[2], atop, false);
            alo = __builtin_amdgcn_udot4(hi, H[0], alo, false);
            amid = __builtin_amdgcn_udot4(hi, H[1], amid, false);
            atop = __builtin_amdgcn_sdot4((int)hi, (int)H[2], atop, false);
        }
        float S = __builtin_fmaf((float)atop, 65536.0f, __builtin_fmaf((float)amid, 256.0f, (float)alo));
        return f16_bits_to_f32(d) * __builtin_fmaf(xp.s, S, -8.0f * xp.xsum);
    }
};

template <> struct IUnit<RFQ_GGUF_Q8_0> : Unit<RFQ_GGUF_Q8_0> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0x400000u; // offset-binary weight bytes reach 255: keep every limb unsigned
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        const Opened<RFQ_GGUF_Q8_0> b = open();
        const U8 &q = b.q;
        const uint16_t d = b.d;
        uint32_t alo = 0, amid = 0, atop = 0, bsum = 0;
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const uint32_t v = q.v[g] ^ 0x80808080u;   // int8 q -> q + 128
            const uint32_t *L = &xp.l[g * 3];
            alo = __builtin_amdgcn_udot4(v, L[0], alo, false);
            amid = __builtin_amdgcn_udot4(v, L[1], amid, false);
            atop = __builtin_amdgcn_udot4(v, L[2], atop, false);
            bsum = __builtin_amdgcn_udot4(v, 0x01010101u, bsum, false);
        }
        // top limbs carry +64: sum b*(top+64) - 64*sum b
        float S = __builtin_fmaf((float)((int)atop - 64 * (int)bsum), 65536.0f,
                                 __builtin_fmaf((float)amid, 256.0f, (float)alo));
        return f16_bits_to_f32(d) * __builtin_fmaf(xp.s, S, -128.0f * xp.xsum);
    }
};

template <> struct IUnit<RFQ_GGUF_Q4_K> : Unit<RFQ_GGUF_Q4_K> {
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0;
    static constexpr bool PAIR = true;            // units 2p and 2p+1 read the same bytes: give both to one lane
    static __device__ __forceinline__ int pair_first(int p) { return 2 * p; }
    static __device__ __forceinline__ int pair_second(int p) { return 2 * p + 1; }
    // byte l of the chunk holds element l of this unit in its low (even unit) or high (odd unit) nibble
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        const uint32_t sm = gguf_scale_min_k4(sub, s0, s1, s2);
        const int sh = 4 * (sub & 1);
        uint32_t alo = 0, amid = 0;
        int atop = 0;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const uint32_t v = (q.v[w] >> sh) & 0x0F0F0F0Fu;
            const uint32_t *L = &xp.l[w * 3];
            alo = __builtin_amdgcn_udot4(v, L[0], alo, false);
            amid = __builtin_amdgcn_udot4(v, L[1], amid, false);
            atop = __builtin_amdgcn_sdot4((int)v, (int)L[2], atop, false);
        }
        const float S = __builtin_fmaf((float)atop, 65536.0f, __builtin_fmaf((float)amid, 256.0f, (float)alo));
        const float d1 = f16_bits_to_f32((uint16_t)(dd & 0xFFFFu)) * (float)(sm & 255u);
        const float m1 = f16_bits_to_f32((uint16_t)(dd >> 16)) * (float)(sm >> 8);
        return __builtin_fmaf(d1 * xp.s, S, -m1 * xp.xsum);
    }
    // Both units of a chunk (this one is the even one) from one fetch: low nibbles against
    // xe, high nibbles against xo, the chunk's two scales and mins unpacked together.
    __device__ __forceinline__ float idot_pair(const XPrep &xe, const XPrep &xo) const
    {
        const int c = sub >> 1, sh = 16 * (c & 1);
        const uint32_t a = (s0 >> sh) & 0xFFFFu, b = (s1 >> sh) & 0xFFFFu, cc = (s2 >> sh) & 0xFFFFu;
        const uint32_t sc2 = c < 2 ? (a & 0x3F3Fu) : ((cc & 0x0F0Fu) | ((a >> 2) & 0x3030u));
        const uint32_t mn2 = c < 2 ? (b & 0x3F3Fu) : (((cc >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u));
        uint32_t elo = 0, emid = 0, olo = 0, omid = 0;
        int etop = 0, otop = 0;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const uint32_t lo = q.v[w] & 0x0F0F0F0Fu, hi = (q.v[w] >> 4) & 0x0F0F0F0Fu;
            const uint32_t *E = &xe.l[w * 3], *O = &xo.l[w * 3];
            elo = __builtin_amdgcn_udot4(lo, E[0], elo, false);
            emid = __builtin_amdgcn_udot4(lo, E[1], emid, false);
            etop = __builtin_amdgcn_sdot4((int)lo, (int)E[2], etop, false);
            olo = __builtin_amdgcn_udot4(hi, O[0], olo, false);
            omid = __builtin_amdgcn_udot4(hi, O[1], omid, false);
            otop = __builtin_amdgcn_sdot4((int)hi, (int)O[2], otop, false);
        }
        const float Se = __builtin_fmaf((float)etop, 65536.0f, __builtin_fmaf((float)emid, 256.0f, (float)elo));
        const float So = __builtin_fmaf((float)otop, 65536.0f, __builtin_fmaf((float)omid, 256.0f, (float)olo));
        const float dv = f16_bits_to_f32((uint16_t)(dd & 0xFFFFu)), dm = f16_bits_to_f32((uint16_t)(dd >> 16));
        const float pos = __builtin_fmaf((float)(sc2 & 255u) * xe.s, Se, (float)(sc2 >> 8) * xo.s * So);
        const float neg = __builtin_fmaf((float)(mn2 & 255u), xe.xsum, (float)(mn2 >> 8) * xo.xsum);
        return __builtin_fmaf(dv, pos, -dm * neg);
    }
};

// A 6-bit code is a byte once its nibble and its bit pair are joined (five instructions per
// four weights), which is what the byte dot products take; the two int8 scales of the unit
// get a sum each, and the offset of 32 goes through the sums of x over the two halves.
template <> struct IUnit<RFQ_GGUF_Q6_K> : Unit<RFQ_GGUF_Q6_K> {
    // Quarters t and t + 2 of a half read the same 32 ql bytes (low and high nibbles) and the same 32 qh bytes: one lane
    // takes both from one fetch (units 4h + t and 4h + t + 2, t < 2), which halves the loads and the window moves per weight.
    static constexpr bool PAIR = true;
    static __device__ __forceinline__ int pair_first(int p) { return ((p >> 1) << 2) | (p & 1); }
    static __device__ __forceinline__ int pair_second(int p) { return pair_first(p) + 2; }
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0;
    __device__ __forceinline__ float idot_pair(const XPrep &xa, const XPrep &xb) const    // this unit (t < 2) and the one two on
    {
        U8 ql, qh;
        wl.piece<0>(ql.v);
        wh.piece<0>(qh.v);
        const int shr = 2 * t;
        uint32_t alo[2] = {0, 0}, amid[2] = {0, 0}, blo[2] = {0, 0}, bmid[2] = {0, 0};
        int atop[2] = {0, 0}, btop[2] = {0, 0};
#pragma unroll
        for (int w = 0; w < 8; w++) {
            // bits 4-5 of a code: the bit pair at 2t (this unit) or 2t + 4 (the other) of its qh byte; what a shift drags in
            // from the neighbouring byte is masked away
            const uint32_t r = qh.v[w] >> shr;
            const uint32_t va = ((r << 4) & 0x30303030u) | (ql.v[w] & 0x0F0F0F0Fu);
            const uint32_t vb = (r & 0x30303030u) | ((ql.v[w] >> 4) & 0x0F0F0F0Fu);
            const uint32_t *A = &xa.l[w * 3], *B = &xb.l[w * 3];
            alo[w >> 2] = __builtin_amdgcn_udot4(va, A[0], alo[w >> 2], false);
            amid[w >> 2] = __builtin_amdgcn_udot4(va, A[1], amid[w >> 2], false);
            atop[w >> 2] = __builtin_amdgcn_sdot4((int)va, (int)A[2], atop[w >> 2], false);
            blo[w >> 2] = __builtin_amdgcn_udot4(vb, B[0], blo[w >> 2], false);
            bmid[w >> 2] = __builtin_amdgcn_udot4(vb, B[1], bmid[w >> 2], false);
            btop[w >> 2] = __builtin_amdgcn_sdot4((int)vb, (int)B[2], btop[w >> 2], false);
        }
        const float SA0 = __builtin_fmaf((float)atop[0], 65536.0f, __builtin_fmaf((float)amid[0], 256.0f, (float)alo[0]));
        const float SA1 = __builtin_fmaf((float)atop[1], 65536.0f, __builtin_fmaf((float)amid[1], 256.0f, (float)alo[1]));
        const float SB0 = __builtin_fmaf((float)btop[0], 65536.0f, __builtin_fmaf((float)bmid[0], 256.0f, (float)blo[0]));
        const float SB1 = __builtin_fmaf((float)btop[1], 65536.0f, __builtin_fmaf((float)bmid[1], 256.0f, (float)blo[1]));
        const float a0 = (float)(int)(int8_t)(sc2 & 255u), a1 = (float)(int)(int8_t)(sc2 >> 8);
        const float b0 = (float)(int)(int8_t)(sc2b & 255u), b1 = (float)(int)(int8_t)(sc2b >> 8);
        const float ha0 = __builtin_fmaf(xa.s, SA0, -32.0f * xa.xh0), ha1 = __builtin_fmaf(xa.s, SA1, -32.0f * xa.xh1);
        const float hb0 = __builtin_fmaf(xb.s, SB0, -32.0f * xb.xh0), hb1 = __builtin_fmaf(xb.s, SB1, -32.0f * xb.xh1);
        return f16_bits_to_f32(d) * (__builtin_fmaf(a0, ha0, a1 * ha1) + __builtin_fmaf(b0, hb0, b1 * hb1));
    }
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        // bits 4-5 of a code: the bit pair at 2t of its qh byte, brought to bits 4-5 by one rotation (what it drags in
        // from the neighbouring bytes is masked away)
        U8 ql, qh;
        wl.piece<0>(ql.v);
        wh.piece<0>(qh.v);
        const int shl = 4 * (t >> 1), rot = (2 * t + 28) & 31;
        uint32_t alo[2] = {0, 0}, amid[2] = {0, 0};
        int atop[2] = {0, 0};
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const uint32_t h4 = __builtin_amdgcn_alignbit(qh.v[w], qh.v[w], rot);
            const uint32_t v = (h4 & 0x30303030u) | ((ql.v[w] >> shl) & 0x0F0F0F0Fu);
            const uint32_t *L = &xp.l[w * 3];
            alo[w >> 2] = __builtin_amdgcn_udot4(v, L[0], alo[w >> 2], false);
            amid[w >> 2] = __builtin_amdgcn_udot4(v, L[1], amid[w >> 2], false);
            atop[w >> 2] = __builtin_amdgcn_sdot4((int)v, (int)L[2], atop[w >> 2], false);
        }
        const float S0 = __builtin_fmaf((float)atop[0], 65536.0f, __builtin_fmaf((float)amid[0], 256.0f, (float)alo[0]));
        const float S1 = __builtin_fmaf((float)atop[1], 65536.0f, __builtin_fmaf((float)amid[1], 256.0f, (float)alo[1]));
        const float sc0 = (float)(int)(int8_t)(sc2 & 255u), sc1 = (float)(int)(int8_t)(sc2 >> 8);
        const float h0 = __builtin_fmaf(xp.s, S0, -32.0f * xp.xh0), h1 = __builtin_fmaf(xp.s, S1, -32.0f * xp.xh1);
        return f16_bits_to_f32(d) * __builtin_fmaf(sc0, h0, sc1 * h1);
    }
};

// The 256-byte Q6_K layout: a unit is 24 stream bytes = 32 two's-complement 6-bit codes, LSB first, and two f16 scales
// (src/kernels/quant/q6_k.rs:221-261).  Four codes are three bytes: the 24-bit window of a group is spread over the
// four bytes of a dword by three shifts that each write one byte (sub-dword destination select), one mask clears what
// the shifts dragged in, and code ^ 32 = value + 32 is an unsigned byte for the byte dot products; the offset goes
// through the sums of x over the unit's two halves, which have a scale each.
template <> struct IUnit<RFQ_Q6_K> : Unit<RFQ_Q6_K> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = false;
    static constexpr uint32_t TOPOFF = 0;
    static __device__ __forceinline__ uint32_t bytes_of(uint32_t t)    // t: four 6-bit codes in bits 0..23 (anything above)
    {
        uint32_t v = t;
        asm("v_lshrrev_b32_sdwa %0, %2, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(v) : "v"(t), "i"(6));
        asm("v_lshrrev_b32_sdwa %0, %2, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(v) : "v"(t), "i"(12));
        asm("v_lshrrev_b32_sdwa %0, %2, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(v) : "v"(t), "i"(18));
        return (v & 0x3F3F3F3Fu) ^ 0x20202020u;
    }
    __device__ __forceinline__ float idot(const XPrep &xp) const
    {
        uint32_t alo[2] = {0, 0}, amid[2] = {0, 0};
        int atop[2] = {0, 0};
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const int b = 3 * (g & 3), d = 3 * (g >> 2);               // window at byte b of dwords d .. d + 2
            const uint32_t t = b == 0 ? q.v[d] : b == 9 ? q.v[d + 2] >> 8 : __builtin_amdgcn_alignbit(q.v[d + b / 4 + 1], q.v[d + b / 4], 8 * (b & 3));
            const uint32_t v = bytes_of(t);
            const uint32_t *L = &xp.l[g * 3];
            alo[g >> 2] = __builtin_amdgcn_udot4(v, L[0], alo[g >> 2], false);
            amid[g >> 2] = __builtin_amdgcn_udot4(v, L[1], amid[g >> 2], false);
            atop[g >> 2] = __builtin_amdgcn_sdot4((int)v, (int)L[2], atop[g >> 2], false);
        }
        const float S0 = __builtin_fmaf((float)atop[0], 65536.0f, __builtin_fmaf((float)amid[0], 256.0f, (float)alo[0]));
        const float S1 = __builtin_fmaf((float)atop[1], 65536.0f, __builtin_fmaf((float)amid[1], 256.0f, (float)alo[1]));
        const float h0 = __builtin_fmaf(xp.s, S0, -32.0f * xp.xh0), h1 = __builtin_fmaf(xp.s, S1, -32.0f * xp.xh1);
        return __builtin_fmaf(f16_bits_to_f32((uint16_t)(sc2 & 0xFFFFu)), h0, f16_bits_to_f32((uint16_t)(sc2 >> 16)) * h1);
    }
};

// MXFP4 (src/loader/dequant.rs:41-82, mxfp.rs:234-244): the code values doubled are small integers,
// {0, 2, 2, 4, 4, 8, 8, 16} for codes 0..7 and {-1, -2, -2, -4, -4, -8, -8, -16} for 8..15, so a unit is a byte dot product
// like the others once codes are bytes: two 8-entry byte tables (v_perm_b32 looks four codes up at once) hold the
// values + 16 for either sign, the sign bit of each code becomes a byte mask by the same instruction's sign-fill
// selectors, and the offset of 16 goes through the sum of the unit's fixed-point x (exactly: the scales are all
// positive, so a residue common to all rows would add up over a column of outputs).  Element 2j is the HIGH nibble of byte j.  The +-8 clamp
// of the reference bites only for exponents >= 1, where it is a bound 2^(4 - e) on the doubled value (from e = 4 on
// every value but 0 sits at the bound and the unit's scale is 8): such units rebuild their tables with that bound.
// MXFP4.  The codes 0..7 decode to {0, 1, 1, 2, 2, 4, 4, 8} and 8..15 to -{1/2, 1, 1, 2, 2, 4, 4, 8}
// (MxfpBlock::decode_e2m1, src/loader/mxfp.rs:234-244: 0 for code 0, otherwise sign * (1 + mant) * 2^(exp - 1)), so
// 16 + 2 * value is a byte.  A weight byte holds two
// codes (elements 2i in the high, 2i+1 in the low nibble) and is translated to its two value bytes by ONE 16-bit
// load from a 256-entry table in LDS; two look-ups, joined by a shift-or, make the four bytes that v_dot4 multiplies
// with four consecutive elements of x (the loads that write only one half of a register are of no use here: with
// ECC on the register file they clear the other half).  The table is replicated per lane (entry stride 256 bytes =
// 64 lanes x 4) so that no two lanes of a look-up meet in a bank, and the address is entry * 256 + lane * 4: one
// v_perm_b32 per look-up.  16 address + 16 LDS + 8 join + 24 dot instructions per 32 weights, where spreading the
// codes with v_perm_b32 tables in registers took 56 + 24.
// The reference clamps value * scale to +-8 (mxfp.rs:196-203), which changes a value only when the exponent is >= 1;
// a wavefront that holds such a unit (one ballot) takes the slower path that builds clamped tables in registers.
constexpr size_t MX4_LUT_BYTES = 256 * 256;

// 16 + 2 * decode_e2m1(code)
__device__ __forceinline__ uint32_t mx4_value_byte(uint32_t code)
{
    const uint32_t t = code == 0u ? 0u : 1u << (((code & 7u) + 1u) >> 1);
    return (code & 8u) ? 16u - t : 16u + t;
}

// Fills the block's table: entry b, replicated over the 64 lane slots, holds the value bytes of b's high nibble (low
// byte) and low nibble (next byte).
template <int THREADS> __device__ __forceinline__ void mx4_fill_lut(uint32_t *lut, int tid)
{
    static_assert(THREADS == 512, "eight 16-byte pieces (four lane slots of one entry) per thread");
    // piece tid + 512 j belongs to entry b = (tid >> 4) + 32 j: its low nibble is the thread's own, its high nibble
    // 2 j + (tid >> 8), one of two neighbouring bytes of the value bytes of the sixteen codes
    constexpr uint64_t POS = 0x2018181414121210ull, NEG = 0x0008080C0C0E0E0Full;
    const uint32_t second = mx4_value_byte(((uint32_t)tid >> 4) & 15u) << 8;
    const uint32_t odd = ((uint32_t)tid >> 8) * 8u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t two = (uint32_t)(((j < 4 ? POS : NEG) >> (16 * (j & 3))) & 0xFFFFu);
        const uint32_t v = second | __builtin_amdgcn_ubfe(two, odd, 8u);
        reinterpret_cast<uint4 *>(lut)[tid + THREADS * j] = make_uint4(v, v, v, v);
    }
}

template <> struct IUnit<RFQ_MXFP4> : Unit<RFQ_MXFP4> {
    static constexpr bool PAIR = false;
    static constexpr bool NIBBLE = false;                                // x limbs in plain element order
    static constexpr uint32_t TOPOFF = 0;
    static __device__ __forceinline__ uint32_t pack4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) { return a | (b << 8) | (c << 16) | (d << 24); }
    static __device__ __forceinline__ void dot3(uint32_t r, const uint32_t *L, uint32_t &alo, uint32_t &amid, int &atop)
    {
        alo = __builtin_amdgcn_udot4(r, L[0], alo, false);
        amid = __builtin_amdgcn_udot4(r, L[1], amid, false);
        atop = __builtin_amdgcn_sdot4((int)r, (int)L[2], atop, false);
    }
    // The two value bytes of the weight byte whose table slot is at LDS address a.
    static __device__ __forceinline__ uint32_t lut_at(uint32_t a)
    {
        return *reinterpret_cast<const uint16_t __attribute__((address_space(3))) *>((uintptr_t)a);
    }
    // slot: the LDS address of this lane's slot of entry 0 of the block's table (mx4_fill_lut), the table at a
    // multiple of 64 KiB: entry b's slot is then `slot` with b as its second byte.
    __device__ __forceinline__ float idot_lut(const XPrep &xp, uint32_t slot) const
    {
        const Opened<RFQ_MXFP4> b = open();
        const U4 &q = b.q;
        const int e = b.e;
        uint32_t alo = 0, amid = 0;
        int atop = 0;
        int ee = e;
        // (e + 127 as unsigned: 0 .. 127 for the plain exponents -127 .. 0, beyond for e >= 1 and for -128)
        if (__builtin_amdgcn_ballot_w64((uint32_t)(e + 127) > 127u) == 0) {
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t x = q.v[d];
                const uint32_t t0 = lut_at(__builtin_amdgcn_perm(x, slot, 0x03020400u)), t1 = lut_at(__builtin_amdgcn_perm(x, slot, 0x03020500u));
                const uint32_t t2 = lut_at(__builtin_amdgcn_perm(x, slot, 0x03020600u)), t3 = lut_at(__builtin_amdgcn_perm(x, slot, 0x03020700u));
                dot3(t0 | (t1 << 16), &xp.l[(2 * d) * 3], alo, amid, atop);
                dot3(t2 | (t3 << 16), &xp.l[(2 * d + 1) * 3], alo, amid, atop);
            }
        } else {                                                         // (weights below 1 never have such a unit)
            // magnitudes capped at 8 / 2^e in units of 1/2: tables 16 + {0, 2, 2, 4 | 4, 8, 8, 16}, 16 - {1, 2, 2, 4 | 4, 8, 8, 16}
            int es = e;
            asm volatile("" : "+v"(es));                                 // (keeps this path's set-up out of the common one)
            const uint32_t b = es <= 0 ? 16u : (es >= 4 ? 1u : (16u >> es));
            auto lim = [&](uint32_t m) { return m < b ? m : b; };
            const uint32_t plo = pack4(16u, 16u + lim(2), 16u + lim(2), 16u + lim(4));
            const uint32_t phi = pack4(16u + lim(4), 16u + lim(8), 16u + lim(8), 16u + lim(16));
            const uint32_t nlo = pack4(16u - lim(1), 16u - lim(2), 16u - lim(2), 16u - lim(4));
            const uint32_t nhi = pack4(16u - lim(4), 16u - lim(8), 16u - lim(8), 16u - lim(16));
            ee = es > 4 ? 4 : (es == -128 ? -300 : es);
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t x = q.v[d];
                const uint32_t sl = x & 0x07070707u, sh = (x >> 4) & 0x07070707u;
                const uint32_t ml = __builtin_amdgcn_perm(x << 4, x << 12, 0x0B090A08u);   // 0xFF where the low code's sign bit is set
                const uint32_t mh = __builtin_amdgcn_perm(x, x << 8, 0x0B090A08u);         // likewise for the high code
                const uint32_t pl = __builtin_amdgcn_perm(phi, plo, sl), nl = __builtin_amdgcn_perm(nhi, nlo, sl);
                const uint32_t ph = __builtin_amdgcn_perm(phi, plo, sh), nh = __builtin_amdgcn_perm(nhi, nlo, sh);
                const uint32_t rl = (ml & nl) | (~ml & pl), rh = (mh & nh) | (~mh & ph);   // odd / even elements of 8d .. 8d+7
                dot3(__builtin_amdgcn_perm(rl, rh, 0x05010400u), &xp.l[(2 * d) * 3], alo, amid, atop);
                dot3(__builtin_amdgcn_perm(rl, rh, 0x07030602u), &xp.l[(2 * d + 1) * 3], alo, amid, atop);
            }
        }
        const float S = __builtin_fmaf((float)atop, 65536.0f, __builtin_fmaf((float)amid, 256.0f, (float)alo));
        // xh0: s * sum(X), see prep_convert_quarter; the scale of exponent -128 is 0 (mx_scale)
        const float v = __builtin_fmaf(0.5f * xp.s, S, -8.0f * xp.xh0);
        return __builtin_ldexpf(v, ee);                                  // (-300 for the exponent -128: scale 0)
    }
};

// The formats without paired units never call idot_pair.
template <typename IU>
__device__ __forceinline__ float idot_pair_of(const IU &u, const XPrep &xe, const XPrep &xo)
{
    if constexpr (IU::PAIR) return u.idot_pair(xe, xo);
    else return 0.0f;
}

// Block = 4 wavefronts = 4 / WPR teams.  Lane `tl` of a team owns units
// tl + j*64*WPR, j < UPL, of every row the team visits.  A team walks
// `groups` groups of R consecutive rows; R is a compile-time constant so a
// group is straight-line code: D rows are requested up front, then row i is
// reduced and row i+D requested, so D rows (D * UPL unit loads per lane) stay in
// flight while the matrix streams in and the hardware load counters release
// each row exactly when it has arrived.  Deeper prefetch does not help: a CU
// accepts only so many outstanding requests and later loads just block issue.
// Rows past the end re-read the team's last valid row (a cache hit) and their
// result is dropped; so do lanes past the end of a row with the last unit.
// Wavefronts per block of the integer-dot kernel: one block per CU, so that x is converted once per CU and
// each thread converts a quarter unit.
constexpr int IDOT_WAVES = 8;

// Rows in flight per lane in the form with one unit per lane and two wavefronts per row.
constexpr int idot_rows_in_flight_12(int fmt)
{
    return fmt == RFQ_MXFP4 ? 2 : (fmt == RFQ_Q6_K || fmt == RFQ_MM_Q6_K) ? 3 : 5;
}

// ---- a timeline from inside the kernel (rfq_bench_gemv_timeline) ------------------------------------------------
// gemv_idot_kernel<..., TRACE = true> has every wavefront read the constant 100 MHz clock (s_memrealtime) at the
// points below and write the readings, lane 0, to g_gemv_trace[wavefront][TRACE_STAMPS] when it ends.  A reading is
// ordered behind the data it marks the arrival of by an empty asm that consumes the register.  Only a few
// configurations are compiled with the flag (TraceCompiled); a launch takes the flagged kernel when the calling
// thread has asked for it (g_gemv_trace_request).
//   0 entry   1 x in registers (behind the requests for x and the first rows, which block while the CU's memory
//   pipeline is full)   2 x converted (before the barrier)   3 after the barrier   4 prepared x in registers
//   5 + 2 i  row i of the first group in registers   6 + 2 i  row i reduced   (i < 7)
//   19 group stored (end)
constexpr int TRACE_STAMPS = 20;
__device__ unsigned long long *g_gemv_trace;

// (a register that the unit's loads fill, for the formats whose kernels are compiled with the trace)
__device__ __forceinline__ uint32_t first_word_of(const Unit<RFQ_Q4_K> &u) { return u.q.v[3]; }
__device__ __forceinline__ uint32_t first_word_of(const Unit<RFQ_GGUF_Q4_K> &u) { return u.q.v[7]; }
__device__ __forceinline__ uint32_t first_word_of(const Unit<RFQ_MXFP4> &u) { return u.w.d[4]; }
template <int FMT> __device__ __forceinline__ uint32_t first_word_of(const Unit<FMT> &) { return 0; }

template <bool ON> struct WaveTrace {
    __device__ __forceinline__ void stamp(int) {}
    __device__ __forceinline__ void stamp_after(int, uint32_t) {}
    __device__ __forceinline__ void flush(int, int, int) {}
};
template <> struct WaveTrace<true> {
    unsigned long long t[TRACE_STAMPS];
    __device__ __forceinline__ void stamp(int i)
    {
        unsigned long long now;
        asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(now) :: "memory");
        t[i] = now;
    }
    __device__ __forceinline__ void stamp_after(int i, uint32_t arrived)
    {
        asm volatile("" :: "v"(arrived) : "memory");
        stamp(i);
    }
    __device__ __forceinline__ void flush(int block_wave, int lane, int waves_total)
    {
        (void)waves_total;
        if (lane == 0) {
            unsigned long long *o = g_gemv_trace + (size_t)block_wave * TRACE_STAMPS;
#pragma unroll
            for (int i = 0; i < TRACE_STAMPS; i++) o[i] = t[i];
        }
    }
};
template <int FMT, int UPL, int WPR, int R, bool FUSE> struct TraceCompiled {
    static constexpr bool value = !FUSE && R == 7 && ((FMT == RFQ_Q4_K && UPL == 1 && WPR == 2) ||
                                                      (FMT == RFQ_MXFP4 && UPL == 1 && WPR == 2) ||
                                                      (FMT == RFQ_GGUF_Q4_K && UPL == 2 && WPR == 1));
};

template <int FMT, int UPL, int WPR, int R, bool FUSE, bool TRACE = false>
__global__ void __launch_bounds__(64 * IDOT_WAVES)
gemv_idot_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y, int n, int k,
                 int groups, GemvFuse f)
{
    using IU = IUnit<FMT>;
    constexpr int WAVES = IDOT_WAVES, TEAMS = WAVES / WPR, TL = 64 * WPR, THREADS = 64 * WAVES;
    // rows in flight per lane: three, or five in the form with one unit per lane (its registers allow it;
    // measured 3..7 there at 14336 x 4096: 11.58, 11.41, 11.30, 11.72, 11.95 us)
    // (GGUF_Q6_K in its paired form, one fetch per two units: four -- 14336 x 4096 with 3, 4, 5 in flight: 13.8, 13.2, 13.8 us)
    // (MXFP4 and Q6_K, bound by their instructions, want fewer in that form, 14336 x 4096 with 5 / 3 / 2 in flight:
    // MXFP4 8.93 / 8.51 / 8.29 us (9.87 with one; 11008 rows 8.27 -> 7.70), Q6_K 11.62 / 11.52 / 11.87; Q4_K, bound by
    // its bytes, 10.43 with 5, 10.67 with 4, 10.86 with 3; GGUF_Q4_0 and GGUF_Q8_0 gain 1-2 % there with three but
    // lose the ring of five rows on long walks: 50000 x 4096 22.2 -> 25.1 and 39.2 -> 40.4 us)
    constexpr int DW12 = idot_rows_in_flight_12(FMT);
    constexpr int DW = (UPL == 1 && WPR == 2) ? DW12 : (FMT == RFQ_GGUF_Q6_K && UPL == 2) ? 4 : 3;
    constexpr int D = R < DW ? R : DW;
    extern __shared__ __attribute__((aligned(16))) uint32_t idot_lds[]; // (MXFP4: the code table,) [units][28]
    constexpr size_t LUT_DWORDS = FMT == RFQ_MXFP4 ? MX4_LUT_BYTES / 4 : 0;
    uint32_t *const xlds = idot_lds + LUT_DWORDS;
    WaveTrace<TRACE> trace;
    trace.stamp(0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;   // (made uniform with readfirstlane the headline kernel measured 2 % slower)
    const int team = wave / WPR, wit = wave % WPR;
    const int tl = wit * 64 + lane;
    const int ku = k >> 5;
    const size_t rb = row_bytes<FMT>(k);

    bool live[UPL];
    int unit[UPL];
    if constexpr (IU::PAIR && UPL == 2) {
        // lane p owns the two units of pair p (the unit count of such a format is a multiple of eight: both live or
        // both past the end)
        const bool in = 2 * tl < ku;
        const int p = in ? tl : (ku >> 1) - 1;
        live[0] = live[1] = in;
        unit[0] = IU::pair_first(p);
        unit[1] = IU::pair_second(p);
    } else {
#pragma unroll
        for (int j = 0; j < UPL; j++) {
            int u = tl + j * TL;
            live[j] = u < ku;
            unit[j] = live[j] ? u : ku - 1;
        }
    }
    const int rows_per_team = groups * R;
    const int row0 = (blockIdx.x * TEAMS + team) * rows_per_team;
    int row_end = row0 + rows_per_team;
    if (row_end > n) row_end = n;
    const int row_last = row_end > row0 ? row_end - 1 : (n - 1);

    // x goes first so that it also returns first: all of it, NX quarter units (eight values each) per thread for the
    // longest row this form takes.  A CU serves its loads in the order they were issued, so a piece of x requested
    // behind the first rows' weights would hold the barrier below, and with it every wavefront's first dot, until
    // those rows had arrived (Q4_K 4096 x 14336: 12.2 -> 11.5 us, 8192 x 8192: 14.0 -> 12.8 us).
    constexpr int NX = (4 * 64 * WPR * UPL + THREADS - 1) / THREADS;
    const int xthread = threadIdx.x;
    float xv[NX][8], nv[FUSE ? NX : 1][8];
    bool prep[NX];
    const bool norm = FUSE && f.norm_w != nullptr;
#pragma unroll
    for (int i = 0; i < NX; i++) {
        const int h = xthread + i * THREADS;
        prep[i] = h < 4 * ku;
        if (prep[i]) prep_load8(x + (size_t)h * 8, xv[i]);
        if constexpr (FUSE) {
            if (norm && prep[i]) prep_load8(f.norm_w + (size_t)h * 8, nv[i]);
        }
    }

    IU buf[D][UPL];
    auto load_row = [&](int slot, int i) {
        int r = row0 + i;
        if (r > row_last) r = row_last;
        const uint8_t *row = fused_row<FUSE>(w, f, r, rb);
        if constexpr (IU::PAIR && UPL == 2) {
            buf[slot][0].load(row, unit[0]);          // one fetch serves both units of the pair
        } else {
#pragma unroll
            for (int j = 0; j < UPL; j++) buf[slot][j].load(row, unit[j]);
        }
    };
#pragma unroll
    for (int d = 0; d < D; d++) load_row(d, d);

    if constexpr (FMT == RFQ_MXFP4) mx4_fill_lut<THREADS>(idot_lds, threadIdx.x);

    if constexpr (TRACE) trace.stamp_after(1, __float_as_uint(xv[0][0]));

    // Cooperative conversion of x: 4*ku quarter-units (eight values each) over the block's threads.
    float ssq = 0.f;
#pragma unroll
    for (int c = 0; c < NX; c++) {
        const int h = xthread + c * THREADS;
        if constexpr (FUSE) {
            if (norm && prep[c]) {
#pragma unroll
                for (int i = 0; i < 8; i++) { ssq = __builtin_fmaf(xv[c][i], xv[c][i], ssq); xv[c][i] *= nv[c][i]; }
            }
        }
        if (prep[c]) prep_convert_quarter<IU::NIBBLE, IU::TOPOFF, WantsQSum<FMT>::value>(xv[c], h & 3, xlds + (size_t)(h >> 2) * 28);
    }
    // With the table the block keeps no static LDS (the table then starts at LDS address 0 and a look-up address
    // needs no base added): the partial sums follow the prepared x in the dynamic part.
    // (the fused forms keep one reduction per row, and so do the formats and forms where the joint one measured level
    // or slower, 14336 x 4096: Q4_K 10.47 -> 10.53 us, GGUF_Q4_K 7.7 -> 9.2, MXFP4 9.4 -> 10.6, Q8_0 level; taken by
    // GGUF_Q4_0 8.44 -> 7.86, GGUF_Q6_K 14.2 -> 13.1, Q6_K 12.1 -> 11.7, Q4_0 8.19 -> 7.88, GGUF_Q8_0 12.3 -> 12.0)
    constexpr bool JOINT = !FUSE && JointRows<FMT>::value && WPR <= 2;
    float *ssq_part = nullptr;
    float (*part)[R][WAVES] = nullptr;
    float (*partj)[JOINT_ROWS][WAVES * 4] = nullptr;
    if constexpr (LUT_DWORDS != 0) {
        // (two workgroups with the table fit a CU's 160 KiB only with the small arrays: such a format reduces row by row)
        static_assert(!JOINT, "the dynamic part of LDS is sized for one reduction per row");
        part = reinterpret_cast<float (*)[R][WAVES]>(xlds + (size_t)ku * 28);
        ssq_part = reinterpret_cast<float *>(part + 2);
    } else if constexpr (JOINT) {
        __shared__ float partj_static[2][JOINT_ROWS][WAVES * 4];
        partj = partj_static;
    } else {
        __shared__ float ssq_part_static[WAVES];
        __shared__ float part_static[2][R][WAVES];
        ssq_part = ssq_part_static;
        part = part_static;
    }
    (void)part; (void)partj; (void)ssq_part;
    if constexpr (FUSE) {
        if (norm) {
            ssq = wave_sum(ssq);
            if (lane == 0) ssq_part[wave] = ssq;
        }
    }
    trace.stamp(2);
    __syncthreads();
    trace.stamp(3);
    float rinv = 1.0f;
    if constexpr (FUSE) {
        if (norm) {
            float total = 0.0f;
#pragma unroll
            for (int q = 0; q < WAVES; q++) total += ssq_part[q];
            rinv = 1.0f / sqrtf(total / (float)k + f.eps);
        }
    }
    XPrep xp[UPL];
#pragma unroll
    for (int j = 0; j < UPL; j++) {
        const uint32_t *src = xlds + (size_t)unit[j] * 28;
#pragma unroll
        for (int i = 0; i < 24; i += 4) {
            uint4 v = *reinterpret_cast<const uint4 *>(src + i);
            xp[j].l[i] = v.x; xp[j].l[i + 1] = v.y; xp[j].l[i + 2] = v.z; xp[j].l[i + 3] = v.w;
        }
        xp[j].s = __uint_as_float(src[24]);
        xp[j].xsum = __uint_as_float(src[25]);
        xp[j].xh0 = __uint_as_float(src[26]);
        xp[j].xh1 = __uint_as_float(src[27]);
    }

    if constexpr (TRACE) trace.stamp_after(4, xp[0].l[0] ^ xp[UPL - 1].l[23]);

    // With R = D a row's slot is the same in every group, and the ring of rows in flight runs on across the groups:
    // the slot a row leaves takes the same row of the next group (past the last group: the team's last row again,
    // a cache hit whose result is never used).  Otherwise a group starts by requesting its first D rows with nothing
    // in flight.  The ring's loads are unconditional: a load under a condition makes the compiler wait for every
    // load in flight behind it.  Only the group size that long walks choose is compiled this way (the same ring
    // measured on the other forms and on the float kernel gained 0..2 % or lost).
    constexpr bool RING = R == 5 && D == 5;
    // (a kernel with the table has no static LDS, which launch_idot checks: the table starts at LDS address 0)
    const uint32_t lut_slot = (uint32_t)(uintptr_t)idot_lds + 4u * (uint32_t)lane;
    (void)lut_slot;
    for (int g = 0; g < groups; g++) {
        const int base = g * R;
        if (!RING && g > 0) {
#pragma unroll
            for (int d = 0; d < D; d++) load_row(d, base + d);
        }
        float res[R];
#pragma unroll
        for (int i = 0; i < R; i++) {
            float acc = 0.f;
            if constexpr (TRACE) {
                if (g == 0) trace.stamp_after(5 + 2 * i, first_word_of(buf[i % D][0]));
            }
            if constexpr (IU::PAIR && UPL == 2) {
                const float t = idot_pair_of(buf[i % D][0], xp[0], xp[1]);
                acc = live[0] ? t : 0.f;
            } else {
#pragma unroll
                for (int j = 0; j < UPL; j++) {
                    float t;
                    if constexpr (FMT == RFQ_MXFP4) t = buf[i % D][j].idot_lut(xp[j], lut_slot);
                    else t = buf[i % D][j].idot(xp[j]);
                    acc += live[j] ? t : 0.f;
                }
            }
            if (i + D < R) load_row(i % D, base + i + D);
            else if (RING) load_row(i % D, base + i + D);
            if constexpr (JOINT) res[i] = acc;
            else res[i] = wave_sum(acc);
            if constexpr (TRACE) {
                if (g == 0) trace.stamp_after(6 + 2 * i, __float_as_uint(res[i]));
            }
        }
        // (`groups` is uniform over the block: every wavefront stores the same number of groups)
        if constexpr (JOINT) store_group_joint<R, WPR, WAVES>(res, partj[g & 1], y, row0 + base, row_end, lane, wave);
        else store_group<R, WPR, FUSE, WAVES, true>(res, part[g & 1], y, row0 + base, row_end, lane, wave, f, rinv);
        if constexpr (TRACE) {
            if (g == 0) trace.stamp(19);
        }
    }
    trace.flush(blockIdx.x * WAVES + wave, lane, gridDim.x * WAVES);
}

// ---- 2 <= m <= 8: the same integer-dot scheme with M activation vectors ----------
//
// Every weight unit is loaded once and dotted against the M prepared vectors,
// whose limbs stay in registers (26 per unit and vector: one unit per lane,
// WPR = ceil(units / 64) wavefronts per row).  Vectors past m_valid repeat the
// last one and are not stored.  LDS holds the M prepared vectors.
template <int FMT, int WPR, int R, int M>
__global__ void __launch_bounds__(256)
gemv_idot_batch_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y, int n, int k,
                       int groups, int m_valid)
{
    using IU = IUnit<FMT>;
    constexpr int TEAMS = 4 / WPR, TL = 64 * WPR;
    // (two rows in flight: with three, Q8_0 4096 x 4096 m = 2 6.83 -> 6.50 us, m = 4 9.15 -> 8.92, Q4_K 14336 x 4096 m = 4
    // 17.7 -> 17.3; with four 7.58, 10.16 and 18.7)
    constexpr int D = R < 2 ? R : 2;
    static_assert(R * M <= 64, "one lane per (row, vector) in the cross-wavefront sum");
    extern __shared__ __attribute__((aligned(16))) uint32_t xlds[]; // [M][units][28]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int team = wave / WPR, wit = wave % WPR;
    const int tl = wit * 64 + lane;
    const int ku = k >> 5;
    const size_t rb = row_bytes<FMT>(k);
    const bool live = tl < ku;
    const int unit = live ? tl : ku - 1;
    (void)TL;

    const int rows_per_team = groups * R;
    const int row0 = (blockIdx.x * TEAMS + team) * rows_per_team;
    int row_end = row0 + rows_per_team;
    if (row_end > n) row_end = n;
    const int row_last = row_end > row0 ? row_end - 1 : (n - 1);

    IU buf[D];
    auto load_row = [&](int slot, int i) {
        int r = row0 + i;
        if (r > row_last) r = row_last;
        buf[slot].load(w + (size_t)r * rb, unit);
    };
#pragma unroll
    for (int d = 0; d < D; d++) load_row(d, d);

    // Cooperative conversion of the M vectors: 2*ku half-units each.
    for (int h = threadIdx.x; h < 2 * ku * M; h += 256) {
        const int v = h / (2 * ku), hh = h - v * 2 * ku;
        const int vs = v < m_valid ? v : m_valid - 1;
        float xw[16];
        prep_load(x + (size_t)vs * k + (size_t)hh * 16, xw);
        prep_convert<IU::NIBBLE, IU::TOPOFF>(xw, hh & 1, xlds + ((size_t)v * ku + (hh >> 1)) * 28);
    }
    __syncthreads();
    XPrep xp[M];
#pragma unroll
    for (int v = 0; v < M; v++) {
        const uint32_t *src = xlds + ((size_t)v * ku + unit) * 28;
#pragma unroll
        for (int i = 0; i < 24; i += 4) {
            uint4 q = *reinterpret_cast<const uint4 *>(src + i);
            xp[v].l[i] = q.x; xp[v].l[i + 1] = q.y; xp[v].l[i + 2] = q.z; xp[v].l[i + 3] = q.w;
        }
        xp[v].s = __uint_as_float(src[24]);
        xp[v].xsum = __uint_as_float(src[25]);
        xp[v].xh0 = __uint_as_float(src[26]);
        xp[v].xh1 = __uint_as_float(src[27]);
    }

    // The M sums of a row are reduced together (rows16_sum_of) and the four 16-lane rows of each of the team's
    // wavefronts meet in LDS: part[row * M + vector][4 * wavefront + lane row].
    __shared__ float part[R * M][16];
    for (int g = 0; g < groups; g++) {
        const int base = g * R;
        if (g > 0) {
#pragma unroll
            for (int d = 0; d < D; d++) load_row(d, base + d);
        }
#pragma unroll
        for (int i = 0; i < R; i++) {
            float acc[M];
#pragma unroll
            for (int v = 0; v < M; v++) {
                float t = buf[i % D].idot(xp[v]);
                acc[v] = live ? t : 0.f;
            }
            if (i + D < R) load_row(i % D, base + i + D);
            const float f = rows16_sum_of<M>(acc, lane);
            if ((lane & 15) < M) part[i * M + (lane & 15)][wave * 4 + (lane >> 4)] = f;
        }
        // `groups` is uniform over the block, so every wavefront reaches both barriers the same number of times
        // (a team of one wavefront reads back what it wrote itself: its LDS operations complete in order).
        if (WPR > 1) __syncthreads();
        if (wit == 0 && lane < R * M) {
            const int i = lane / M, v = lane % M;
            const int r = row0 + base + i;
            float t = 0.f;
#pragma unroll
            for (int q = 0; q < 4 * WPR; q++) t += part[lane][team * WPR * 4 + q];
            if (r < row_end && v < m_valid) y[(size_t)v * n + r] = t;
        }
        if (WPR > 1) __syncthreads();
    }
}

// ---- 2 <= m <= 8, Q8_0: the batch through the matrix cores ----------------------
//
// With M vectors in registers the integer-dot kernel above needs more than 250
// registers per lane, one wavefront per SIMD, and cannot keep enough loads in
// flight to stream the matrix.  Here the M vectors are the rows of a matrix
// operand instead: v_mfma_f32_16x16x32_f16 multiplies a 16 x 32 tile of
// activations (one unit of k; rows 0..7 are the high parts of the eight
// vectors, rows 8..15 their low parts, see below) with a 32 x 16 tile of
// weights (one unit of 16 rows).
//
// Exactness is kept as in the integer-dot scheme.  A small kernel first turns x
// into block-fixed-point per unit and vector: a power of two s and integers
// X_i = round(x_i / s), |X_i| <= 2^22, split as X = 2048 * hi + lo with
// |hi| <= 2048 and 0 <= lo < 2048, both exact in fp16; the weights b - 128 are
// exact in fp16 too, so every product and every 32-term sum is an exact
// integer below 2^24 in the fp32 accumulator:
//     sum_i (b_i - 128) x_i  =  s * (2048 * sum (b-128).hi + sum (b-128).lo).
// Operand layout of the instruction: lane l holds row/column l % 16 and the
// eight k values 8 * (l / 16) ..+8; the result's lane l holds column l % 16
// (a weight row: the lane that loaded its bytes and its scale) and rows
// 4 * (l / 16) ..+4 (vectors).
//
// A workgroup owns 16 weight rows; its 8 wavefronts take the units
// w, w + 8, ... of those rows, sixteen at a time with all their loads issued up
// front (64 KiB of weights in flight per CU), and add their partial results
// through LDS.

typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));
typedef _Float16 v2h_t __attribute__((ext_vector_type(2)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef uint32_t v2u_t __attribute__((ext_vector_type(2)));
typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));

// parts: [unit][k octet 0..3][row 0..15][8 fp16] (1 KiB per unit; row i < 8 is
// the high part of vector i, row i >= 8 the low part of vector i - 8; operand lane
// 16 * q + i reads octet q, row i); sx: [unit][8] f32.  One workgroup per unit;
// thread t: vector t / 32, element t % 32.
__global__ void __launch_bounds__(256)
gemv_mfma_prep_kernel(const float *__restrict__ x, _Float16 *__restrict__ parts, float *__restrict__ sx, int m, int k)
{
    const int u = blockIdx.x, v = threadIdx.x >> 5, kk = threadIdx.x & 31, lane = threadIdx.x & 63;
    const float xv = v < m ? x[(size_t)v * k + u * 32 + kk] : 0.0f;
    float mx = fabsf(xv);
    const bool bad = !(mx <= 3.40282347e+38f);
    const unsigned long long bad_mask = __ballot(bad);
    const bool any_bad = ((bad_mask >> (lane & 32)) & 0xFFFFFFFFull) != 0;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 32));
    const int e = (int)(__float_as_uint(mx) >> 23);   // biased exponent of the largest |x|
    int ie = 275 - e;                                 // 1/s = 2^(21 - (e - 127))
    if (ie > 254) ie = 254;
    const float inv_s = __uint_as_float((uint32_t)ie << 23);
    float sc = ie == 254 ? __uint_as_float(0x00400000u) : __uint_as_float((uint32_t)(254 - ie) << 23);
    if (any_bad) sc = __uint_as_float(0x7FC00000u);   // a non-finite x poisons its unit, as it would a float sum
    const int X = any_bad ? 0 : (int)(__float_as_uint(__builtin_fmaf(xv, inv_s, 12582912.0f)) - 0x4B400000u);
    const int hi = X >> 11, lo = X & 2047;
    const size_t at = ((size_t)u * 64 + (kk >> 3) * 16 + v) * 8 + (kk & 7);
    parts[at] = (_Float16)(float)hi;
    parts[at + 8 * 8] = (_Float16)(float)lo;
    if (kk == 0) sx[u * 8 + v] = sc;
}

constexpr int MFMA_NB = 16;                           // units of a wavefront in flight together
constexpr int MFMA_WAVES = 8;

// FMT: RFQ_Q8_0 (36-byte blocks: f32 scale, offset-binary bytes) or RFQ_GGUF_Q8_0 (34-byte
// blocks: f16 scale, int8 bytes, flipped to offset binary with one XOR per dword).
template <int FMT>
__global__ void __launch_bounds__(64 * MFMA_WAVES)
gemv_mfma_q8_0_kernel(const uint8_t *__restrict__ w, const _Float16 *__restrict__ parts, const float *__restrict__ sx,
                      float *__restrict__ y, int m, int n, int k)
{
    constexpr int BB = Fmt<FMT>::BB, DOFF = FMT == RFQ_Q8_0 ? 4 : 2;
    constexpr uint32_t FLIP = FMT == RFQ_Q8_0 ? 0u : 0x80808080u;
    __shared__ float red[MFMA_WAVES * 2 * 16 * 8];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, q = lane >> 4;
    const int units = k / 32, n0 = blockIdx.x * 16;

    const int row = n0 + j < n ? n0 + j : n - 1;
    const uint8_t *row_ptr = w + (size_t)row * units * BB;
    // The weight bytes are fetched by four neighbouring lanes per row (32
    // consecutive bytes: one request instead of four) and handed to the lane
    // that holds them as an operand, lane 16 * q + j <- lane 4 * j + q.
    const int row_c = n0 + (lane >> 2) < n ? n0 + (lane >> 2) : n - 1;
    const uint8_t *row_ptr_c = w + (size_t)row_c * units * BB + DOFF + 8 * (lane & 3);
    const int from_lane4 = 4 * (4 * j + q);
    const v4u_t *parts_l = reinterpret_cast<const v4u_t *>(parts) + lane;     // (octet q, row j: 16 bytes per lane)
    const v2h_t bias = {(_Float16)-1152.0f, (_Float16)-1152.0f};
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int base = wave; base < units; base += MFMA_WAVES * MFMA_NB) {
        v2u_t wq[MFMA_NB];
        float ws[MFMA_NB];
        v4u_t xa[MFMA_NB];
        v4f_t s4[MFMA_NB / 2];                          // (the x scales follow half a batch behind: registers)
        auto load_s4 = [&](int b) {
            const int u = base + MFMA_WAVES * b, uc = u < units ? u : units - 1;
            s4[b % (MFMA_NB / 2)] = *reinterpret_cast<const v4f_t *>(sx + uc * 8 + 4 * (q & 1));
        };
#pragma unroll
        for (int b = 0; b < MFMA_NB; b++) {
            const int u = base + MFMA_WAVES * b, uc = u < units ? u : units - 1; // (past the end: a valid unit, weight scale 0)
            const uint8_t *blk = row_ptr + (size_t)uc * BB;
            wq[b] = ld<v2u_t>(row_ptr_c + (size_t)uc * BB);
            ws[b] = FMT == RFQ_Q8_0 ? ld<float>(blk) : f16_bits_to_f32(ld<uint16_t>(blk));                    // (no branch around a load: it would wait for the others)
            xa[b] = parts_l[(size_t)uc * 64];
            if (b < MFMA_NB / 2) load_s4(b);
        }
        __builtin_amdgcn_sched_barrier(0);             // (every load of the batch is out before the first is used)
#pragma unroll
        for (int b = 0; b < MFMA_NB; b++) {
            // bytes b0..b3 of a dword -> fp16 pairs (b0, b1), (b2, b3): 0x6400 | b reads 1024 + b
            v4u_t wb;
#pragma unroll
            for (int d = 0; d < 2; d++) {
                const uint32_t wd = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)wq[b][d]) ^ FLIP;
                const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, wd, 0x04010400u);
                const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, wd, 0x04030402u);
                v2h_t h0, h1;
                __builtin_memcpy(&h0, &p0, 4);
                __builtin_memcpy(&h1, &p1, 4);
                h0 = h0 + bias;                        // 1024 + b - 1152 = b - 128
                h1 = h1 + bias;
                uint32_t o0, o1;
                __builtin_memcpy(&o0, &h0, 4);
                __builtin_memcpy(&o1, &h1, 4);
                wb[2 * d] = o0;
                wb[2 * d + 1] = o1;
            }
            v8h_t wf, ax;
            __builtin_memcpy(&wf, &wb, 16);
            __builtin_memcpy(&ax, &xa[b], 16);
            const v4f_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
            // this lane's four results: weight row j times the high (q < 2) or low parts of vectors 4 (q & 1) ..+4
            const v4f_t sp = __builtin_amdgcn_mfma_f32_16x16x32_f16(ax, wf, zero, 0, 0, 0);
            const float wsc = base + MFMA_WAVES * b < units ? ws[b] : 0.0f;
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = __builtin_fmaf(wsc * s4[b % (MFMA_NB / 2)][r], sp[r], acc[r]);
            if (b + MFMA_NB / 2 < MFMA_NB) load_s4(b + MFMA_NB / 2);
        }
    }
    // red[wavefront][part: 0 high, 1 low][weight row][vector]
#pragma unroll
    for (int r = 0; r < 4; r++) red[((wave * 2 + (q >> 1)) * 16 + j) * 8 + 4 * (q & 1) + r] = acc[r];
    __syncthreads();
    if (tid < 128) {
        const int jj = tid >> 3, v = tid & 7;
        float hi = 0.0f, lo = 0.0f;
#pragma unroll
        for (int wv = 0; wv < MFMA_WAVES; wv++) {
            hi += red[((wv * 2 + 0) * 16 + jj) * 8 + v];
            lo += red[((wv * 2 + 1) * 16 + jj) * 8 + v];
        }
        if (v < m && n0 + jj < n) y[(size_t)v * n + n0 + jj] = __builtin_fmaf(hi, 2048.0f, lo);
    }
}

// ---- any m <= 8, any k: one row per wavefront ---------------------------------
// BYTES: fetch blocks byte-exactly (a tensor that does not start on a multiple of 4, see load32_a2).
template <int FMT, int M, bool BYTES = false>
__global__ void __launch_bounds__(256)
gemv_generic_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y, int n, int k)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ku = k >> 5;
    const size_t rb = row_bytes<FMT>(k);
    const int waves_total = gridDim.x * 4;
    unit_tables_init<FMT>();
    for (int r = blockIdx.x * 4 + wave; r < n; r += waves_total) {
        const uint8_t *row = w + (size_t)r * rb;
        float acc[M];
#pragma unroll
        for (int mi = 0; mi < M; mi++) acc[mi] = 0.f;
        for (int u = lane; u < ku; u += 64) {
            Unit<FMT> un;
            if constexpr (BYTES) un.load_bytes(row, u);            // (only instantiated for units that have it)
            else un.load(row, u);
#pragma unroll
            for (int mi = 0; mi < M; mi++) {
                float xv[32];
                load_x32(x + (size_t)mi * k + (size_t)u * 32, xv);
                float xsum = Unit<FMT>::NEEDS_XSUM ? sum32(xv) : 0.f;
                acc[mi] += un.dot(xv, xsum);
            }
        }
#pragma unroll
        for (int mi = 0; mi < M; mi++) {
            float t = wave_sum(acc[mi]);
            if (lane == 0) y[(size_t)mi * n + r] = t;
        }
    }
}

// `per_cu` resident blocks per CU, every team walking the same number of rows
// (a straggler is expensive on a ~10 us kernel).  Rows per team = groups * R
// with R from a small compiled set; the pair that wastes the fewest row slots
// wins, the larger R on a tie.
struct RowPlan { int r, groups, blocks; };
inline RowPlan plan_rows(int n, int teams, int per_cu, bool even_only = false)
{
    const int slots = device_cu_count() * per_cu;
    int want = (n + slots * teams - 1) / (slots * teams);
    if (want < 1) want = 1;
    static const int RS[6] = {2, 4, 5, 6, 7, 8};
    RowPlan best{8, 1, 0};
    long best_cost = -1;
    for (int idx = 0; idx < 6; idx++) {
        int r = RS[idx];
        if (even_only && (r & 1)) continue;
        int groups = (want + r - 1) / r;
        int blocks = (n + teams * r * groups - 1) / (teams * r * groups);
        long waves_of_blocks = (blocks + slots - 1) / slots;
        long cost = waves_of_blocks * r * groups;
        if (best_cost < 0 || cost < best_cost || (cost == best_cost && r > best.r)) {
            best_cost = cost;
            best = RowPlan{r, groups, blocks};
        }
    }
    return best;
}

template <int FMT, int UPL, int WPR, int R, bool FUSE>
int launch_xreg(const uint8_t *w, const float *x, float *y, int n, int k, const RowPlan &p, const GemvFuse &f,
                hipStream_t s)
{
    note_kernel(FUSE ? "gemv_xreg_kernel<%s,%d,%d,%d,fused>" : "gemv_xreg_kernel<%s,%d,%d,%d>", FMT, UPL, WPR, R);
    // x goes through k floats of LDS when that stays well inside the default limit beside the decode tables
    // (and its address is one 16-byte loads accept); longer rows fetch it per lane
    const size_t xbytes = (size_t)k * 4;
    const int xstage = xbytes <= 32 * 1024 && (reinterpret_cast<uintptr_t>(x) & 3u) == 0 ? 1 : 0;
    hipLaunchKernelGGL((gemv_xreg_kernel<FMT, UPL, WPR, R, FUSE>), dim3(p.blocks), dim3(256), xstage ? xbytes : 0, s, w, x, y,
                       n, k, p.groups, f, xstage);
    RFQ_LAUNCH_CHECK("gemv_xreg_kernel");
    return RFQ_OK;
}

// FUSE launches with f.glu set need an even R: the two rows of a pair are reduced together.
template <int FMT, int UPL, int WPR, bool FUSE>
int run_xreg(const uint8_t *w, const float *x, float *y, int n, int k, const GemvFuse &f, hipStream_t s)
{
    // two blocks of four wavefronts per CU (three fit for Q6_K in the two-units-per-lane form but run slower);
    // four in the form with one unit per lane and two wavefronts per row, which is light on registers
    const RowPlan p = plan_rows(n, 4 / WPR, (UPL == 1 && WPR == 2) ? 4 : 2, FUSE && f.glu);
    switch (p.r) {
    case 2: return launch_xreg<FMT, UPL, WPR, 2, FUSE>(w, x, y, n, k, p, f, s);
    case 4: return launch_xreg<FMT, UPL, WPR, 4, FUSE>(w, x, y, n, k, p, f, s);
    case 5: return launch_xreg<FMT, UPL, WPR, 5, FUSE>(w, x, y, n, k, p, f, s);
    case 6: return launch_xreg<FMT, UPL, WPR, 6, FUSE>(w, x, y, n, k, p, f, s);
    case 7: return launch_xreg<FMT, UPL, WPR, 7, FUSE>(w, x, y, n, k, p, f, s);
    default: return launch_xreg<FMT, UPL, WPR, 8, FUSE>(w, x, y, n, k, p, f, s);
    }
}

template <int FMT> struct HasIdot { static constexpr bool value = false; };
template <> struct HasIdot<RFQ_Q4_K> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_Q4_0> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_Q8_0> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_GGUF_Q4_0> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_GGUF_Q8_0> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_GGUF_Q4_K> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_GGUF_Q6_K> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_MM_Q4_K> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_MM_Q8_0> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_Q6_K> { static constexpr bool value = true; };
template <> struct HasIdot<RFQ_MXFP4> { static constexpr bool value = true; };
template <int FMT> struct HasIdotBatch { static constexpr bool value = HasIdot<FMT>::value; };
template <> struct HasIdotBatch<RFQ_Q6_K> { static constexpr bool value = false; };   // batches keep one decode launch per vector
template <> struct HasIdotBatch<RFQ_MXFP4> { static constexpr bool value = false; };

template <int FMT, int UPL, int WPR, int R, bool FUSE>
int launch_idot(const uint8_t *w, const float *x, float *y, int n, int k, int blocks, int groups, const GemvFuse &f,
                hipStream_t s)
{
    size_t lds = (size_t)(k / 32) * 28 * sizeof(uint32_t);
    if constexpr (FMT == RFQ_MXFP4) {
        lds += MX4_LUT_BYTES + (2 * R + 1) * IDOT_WAVES * sizeof(float);   // the table; partial sums (no static LDS)
        static std::once_flag once;
        static hipError_t attr_err = hipSuccess;
        static bool table_at_zero = false;
        std::call_once(once, [] {
            const void *kernel = reinterpret_cast<const void *>(&gemv_idot_kernel<FMT, UPL, WPR, R, FUSE>);
            hipFuncAttributes fa;
            attr_err = hipFuncGetAttributes(&fa, kernel);
            if (attr_err != hipSuccess) return;
            table_at_zero = fa.sharedSizeBytes == 0;                     // no static LDS in front of the table
            attr_err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 4096);
        });
        if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemv_idot_kernel)");
        if (!table_at_zero) return run_xreg<FMT, UPL, WPR, FUSE>(w, x, y, n, k, f, s);   // (not expected: the float kernel)
    }
    note_kernel(FUSE ? "gemv_idot_kernel<%s,%d,%d,%d,fused>" : "gemv_idot_kernel<%s,%d,%d,%d>", FMT, UPL, WPR, R);
    if constexpr (TraceCompiled<FMT, UPL, WPR, R, FUSE>::value) {
        if (g_gemv_trace_request.d_buf != nullptr && (size_t)blocks * IDOT_WAVES <= g_gemv_trace_request.capacity_waves) {
            if constexpr (FMT == RFQ_MXFP4) {
                const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_idot_kernel<FMT, UPL, WPR, R, FUSE, true>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 4096);
                if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(gemv_idot_kernel, traced)");
            }
            const hipError_t e = hipMemcpyToSymbol(HIP_SYMBOL(g_gemv_trace), &g_gemv_trace_request.d_buf, sizeof(g_gemv_trace_request.d_buf), 0,
                                                   hipMemcpyHostToDevice);    // (blocking: a tool of the benchmark driver)
            if (e != hipSuccess) return hip_fail(e, "hipMemcpyToSymbol(g_gemv_trace)");
            hipLaunchKernelGGL((gemv_idot_kernel<FMT, UPL, WPR, R, FUSE, true>), dim3(blocks), dim3(64 * IDOT_WAVES), lds, s, w, x, y, n,
                               k, groups, f);
            RFQ_LAUNCH_CHECK("gemv_idot_kernel (traced)");
            g_gemv_trace_request.waves_written = blocks * IDOT_WAVES;
            return RFQ_OK;
        }
    }
    hipLaunchKernelGGL((gemv_idot_kernel<FMT, UPL, WPR, R, FUSE>), dim3(blocks), dim3(64 * IDOT_WAVES), lds, s, w, x, y, n, k, groups,
                       f);
    RFQ_LAUNCH_CHECK("gemv_idot_kernel");
    return RFQ_OK;
}

// prefer_idot = false: a format that has both kernels takes the float one for this shape.
template <int FMT, int UPL, int WPR, bool FUSE>
int run_idot(const uint8_t *w, const float *x, float *y, int n, int k, const GemvFuse &f, hipStream_t s, bool prefer_idot = true)
{
    if constexpr (HasIdot<FMT>::value) {
        if (!prefer_idot) return run_xreg<FMT, UPL, WPR, FUSE>(w, x, y, n, k, f, s);
        constexpr int TEAMS = IDOT_WAVES / WPR;
        // Aim at eight resident wavefronts per CU, every team walking the same number
        // of rows (a straggler is expensive on a ~10 us kernel).  Rows per team
        // = groups * R with R from a small compiled set; take the pair that
        // wastes the fewest row slots, the larger R on a tie.  Where a team walks several groups, an R that lets the
        // ring of rows in flight run on across the groups (R = 5 in the form that keeps five rows in flight) is worth
        // 5 % more rows: measured at 128256 x 4096, 65 rows per team in groups of 5 against 63 in groups of 7, -2 %.
        // (the form with one unit per lane and two wavefronts per row is light on registers: two blocks per CU)
        const int slots = device_cu_count() * 8 / IDOT_WAVES * (UPL == 1 && WPR == 2 ? 2 : 1);
        int want = (n + slots * TEAMS - 1) / (slots * TEAMS);
        if (want < 1) want = 1;
        constexpr bool FIVE = UPL == 1 && WPR == 2 && !FUSE && idot_rows_in_flight_12(FMT) == 5;   // (groups of five ring on only with five in flight)
        static const int RS[5] = {2, 4, 5, 7, 8};
        int best_r = 8, best_groups = 1, best_blocks = 0;
        long best_cost = -1;
        // (one row per team where two would leave CUs without a workgroup -- a key/value projection of a long hidden
        // state: 1024 x 8192 4.38 -> 3.58 us, 1024 x 5120 3.50 -> 3.03, 512 x 8192 4.10 -> 3.11; teams of several
        // wavefronts, plain GEMV)
        constexpr bool ONE = UPL == 2 && WPR >= 2 && !FUSE;
        if (ONE && want == 1 && n <= slots * TEAMS) {
            const int blocks = (n + TEAMS - 1) / TEAMS;
            return launch_idot<FMT, UPL, WPR, ONE ? 1 : 2, FUSE>(w, x, y, n, k, blocks, 1, f, s);
        }
        for (int idx = 0; idx < 5; idx++) {
            int r = RS[idx];
            if (FUSE && f.glu && (r & 1)) continue;
            int groups = (want + r - 1) / r;
            if (r == 5 && !(FIVE && groups > 1)) continue;
            int blocks = (n + TEAMS * r * groups - 1) / (TEAMS * r * groups);
            long waves_of_blocks = (blocks + slots - 1) / slots;
            // (a group that starts with nothing in flight costs a team of several wavefronts per row about as much as
            // a row and a half: 5120 x 5120 in three groups of 2 rows 8.15 us, in one of 7 7.48 us; 13824 x 5120 in four
            // of 4 17.2 us, in two of 8 15.2 us)
            long cost = waves_of_blocks * (r * groups * (r == 5 && groups > 1 ? 19 : 20) + (UPL == 2 && WPR >= 2 ? 30 * (groups - 1) : 0));
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && r > best_r)) {
                best_cost = cost; best_r = r; best_groups = groups; best_blocks = blocks;
            }
        }
        switch (best_r) {
        case 2: return launch_idot<FMT, UPL, WPR, 2, FUSE>(w, x, y, n, k, best_blocks, best_groups, f, s);
        case 4: return launch_idot<FMT, UPL, WPR, 4, FUSE>(w, x, y, n, k, best_blocks, best_groups, f, s);
        case 5:
            if constexpr (FIVE) return launch_idot<FMT, UPL, WPR, 5, FUSE>(w, x, y, n, k, best_blocks, best_groups, f, s);
            return RFQ_E_UNSUPPORTED;                     // (not reached: 5 is only offered when FIVE)
        case 7: return launch_idot<FMT, UPL, WPR, 7, FUSE>(w, x, y, n, k, best_blocks, best_groups, f, s);
        default: return launch_idot<FMT, UPL, WPR, 8, FUSE>(w, x, y, n, k, best_blocks, best_groups, f, s);
        }
    } else {
        return run_xreg<FMT, UPL, WPR, FUSE>(w, x, y, n, k, f, s);
    }
}

template <int FMT, int WPR, int R, int M>
int launch_idot_batch(const uint8_t *w, const float *x, float *y, int m, int n, int k, int blocks, int groups,
                      hipStream_t s)
{
    const size_t lds = (size_t)M * (k / 32) * 28 * sizeof(uint32_t);
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_idot_batch_kernel<FMT, WPR, R, M>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 4096);
    });
    if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemv_idot_batch_kernel)");
    note_kernel("gemv_idot_batch_kernel<%s,%d,%d,%d>", FMT, WPR, R, M);
    hipLaunchKernelGGL((gemv_idot_batch_kernel<FMT, WPR, R, M>), dim3(blocks), dim3(256), lds, s, w, x, y, n, k, groups,
                       m);
    RFQ_LAUNCH_CHECK("gemv_idot_batch_kernel");
    return RFQ_OK;
}

template <int FMT, int WPR, int M>
int run_idot_batch(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    if constexpr (HasIdotBatch<FMT>::value) {
        constexpr int TEAMS = 4 / WPR;
        // one or two resident blocks per CU (LDS holds the M prepared vectors),
        // every team walking the same number of rows
        const size_t lds = (size_t)M * (k / 32) * 28 * sizeof(uint32_t);
        const int slots = device_cu_count() * (lds > 72 * 1024 ? 1 : 2);
        int want = (n + slots * TEAMS - 1) / (slots * TEAMS);
        if (want < 1) want = 1;
        constexpr int RMAX = 64 / M < 8 ? 64 / M : 8;
        int best_r = RMAX, best_groups = 1, best_blocks = 0;
        long best_cost = -1;
        for (int r : {4, RMAX}) {
            int groups = (want + r - 1) / r;
            int blocks = (n + TEAMS * r * groups - 1) / (TEAMS * r * groups);
            long waves_of_blocks = (blocks + slots - 1) / slots;
            long cost = waves_of_blocks * r * groups;
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && r > best_r)) {
                best_cost = cost; best_r = r; best_groups = groups; best_blocks = blocks;
            }
        }
        if (best_r == 4) return launch_idot_batch<FMT, WPR, 4, M>(w, x, y, m, n, k, best_blocks, best_groups, s);
        return launch_idot_batch<FMT, WPR, RMAX, M>(w, x, y, m, n, k, best_blocks, best_groups, s);
    } else {
        (void)w; (void)x; (void)y; (void)m; (void)n; (void)k; (void)s;
        return RFQ_E_UNSUPPORTED;
    }
}

template <int FMT, int M>
int run_idot_batch_k(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    const int ku = k / 32;
    if (ku <= 64) return run_idot_batch<FMT, 1, M>(w, x, y, m, n, k, s);
    if (ku <= 128) return run_idot_batch<FMT, 2, M>(w, x, y, m, n, k, s);
    return run_idot_batch<FMT, 4, M>(w, x, y, m, n, k, s);
}

// Windowed loads read whole dwords around a piece: the tensor must start on a multiple of 4.
template <int FMT> bool tensor_aligned(const uint8_t *w, int, int)
{
    return (reinterpret_cast<uintptr_t>(w) & 3u) == 0;
}

template <int FMT, int M>
int run_generic(const uint8_t *w, const float *x, float *y, int n, int k, hipStream_t s)
{
    int blocks = (n + 3) / 4;
    int cap = device_cu_count() * 8;
    if (blocks > cap) blocks = cap;
    if constexpr (NeedsAlignedTensor<FMT>::value) {
        if (!tensor_aligned<FMT>(w, n, k)) {
            note_kernel("gemv_generic_kernel<%s,%d,bytes>", FMT, M, 0, 0);
            hipLaunchKernelGGL((gemv_generic_kernel<FMT, M, true>), dim3(blocks), dim3(256), 0, s, w, x, y, n, k);
            RFQ_LAUNCH_CHECK("gemv_generic_kernel");
            return RFQ_OK;
        }
    }
    note_kernel("gemv_generic_kernel<%s,%d>", FMT, M, 0, 0);
    hipLaunchKernelGGL((gemv_generic_kernel<FMT, M>), dim3(blocks), dim3(256), 0, s, w, x, y, n, k);
    RFQ_LAUNCH_CHECK("gemv_generic_kernel");
    return RFQ_OK;
}

template <int FMT>
int run_mfma_q8_0(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    const int units = k / 32;
    const size_t parts_bytes = (size_t)units * 1024, sx_bytes = (size_t)units * 32;
    uint8_t *tmp = nullptr;
    bool transient = false;
    if (int rc = workspace(s, parts_bytes + sx_bytes, &tmp, &transient)) return rc;
    _Float16 *parts = reinterpret_cast<_Float16 *>(tmp);
    float *sx = reinterpret_cast<float *>(tmp + parts_bytes);
    note_kernel("gemv_mfma_prep_kernel + gemv_mfma_q8_0_kernel<%s>", FMT, 0, 0, 0);
    hipLaunchKernelGGL(gemv_mfma_prep_kernel, dim3(units), dim3(256), 0, s, x, parts, sx, m, k);
    hipLaunchKernelGGL(gemv_mfma_q8_0_kernel<FMT>, dim3((n + 15) / 16), dim3(64 * MFMA_WAVES), 0, s, w, parts, sx, y, m, n, k);
    hipError_t launch_err = hipGetLastError();
    if (transient) {
        hipError_t free_err = hipFreeAsync(tmp, s);
        if (launch_err == hipSuccess) launch_err = free_err;
    }
    if (launch_err != hipSuccess) return hip_fail(launch_err, "gemv_mfma_q8_0_kernel");
    return RFQ_OK;
}

// m == 1, 16 < k / 32 <= 512: the kernels that keep x per lane.
template <int FMT, bool FUSE>
int run_rows(const uint8_t *w, const float *x, float *y, int n, int k, const GemvFuse &f, hipStream_t s)
{
    const int ku = k / 32;
    // The 256-byte Q6_K layout has both kernels, a few per cent apart either way (measured on 14336, 11008, 4096 and
    // 32000 rows of 4096, 4096 rows of 8192 and of 14336): the integer-dot one where a team walks a single group of rows
    // of 65..128 units or rows longer than 256 units, the float one elsewhere and in the fused forms.
    // MXFP4 has both kernels too: the integer-dot one for rows longer than 256 units (4096 x 14336 11.6 -> 11.1 us)
    // and, with up to 128 units, for few rows (up to 16 per CU: 4096 x 4096 5.0 -> 4.6 us) and around 56 rows per CU
    // (14336 x 4096 9.8 -> 9.4 us); elsewhere the float one (code values from a table of floats in LDS) is level or
    // ahead (8192 x 8192 10.5 against 11.1 us, 32000 x 4096 16.8 against 18.8 us), and the fused forms keep it.
    if constexpr (FMT == RFQ_MXFP4) {
        const int cus = device_cu_count();
        if (FUSE || !(ku > 256 || (ku <= 128 && (n <= cus * 16 || (n >= cus * 52 && n <= cus * 64))))) {
            if (ku <= 64) return run_idot<FMT, 1, 1, FUSE>(w, x, y, n, k, f, s, false);
            if (!FUSE && ku <= 128 && (n > cus * 16 || n <= cus * 8)) return run_idot<FMT, 1, 2, FUSE>(w, x, y, n, k, f, s, false);
            if (ku <= 128) return run_idot<FMT, 2, 1, FUSE>(w, x, y, n, k, f, s, false);
            if (ku <= 256) return run_idot<FMT, 2, 2, FUSE>(w, x, y, n, k, f, s, false);
            return run_idot<FMT, 2, 4, FUSE>(w, x, y, n, k, f, s, false);
        }
    }
    if constexpr (FMT == RFQ_Q6_K) {
        const int cus = device_cu_count();
        if (FUSE || !((ku > 64 && ku <= 128 && n >= cus * 56 && n <= cus * 64) || ku > 256)) {
            if (ku <= 64) return run_idot<FMT, 1, 1, FUSE>(w, x, y, n, k, f, s, false);
            if (!FUSE && ku <= 128 && (n > cus * 16 || n <= cus * 8)) return run_idot<FMT, 1, 2, FUSE>(w, x, y, n, k, f, s, false);
            if (ku <= 128) return run_idot<FMT, 2, 1, FUSE>(w, x, y, n, k, f, s, false);
            if (ku <= 256) return run_idot<FMT, 2, 2, FUSE>(w, x, y, n, k, f, s, false);
            return run_idot<FMT, 2, 4, FUSE>(w, x, y, n, k, f, s, false);
        }
    }
    if (ku <= 64) return run_idot<FMT, 1, 1, FUSE>(w, x, y, n, k, f, s);
    // Rows of 65..128 units: one unit per lane and two wavefronts per row (sixteen wavefronts per CU) against two units
    // per lane and one wavefront per row (eight).  Measured per format on 1024, 4096, 6144, 11008, 14336, 32000 and
    // 128256 rows of 4096 with every group size either form offers:
    //  * up to eight rows per CU the first form puts twice as many CUs to work (1024 rows: Q4_K 3.87 -> 3.10 us, Q8_0
    //    3.42 -> 2.92, Q6_K 3.29 -> 2.83, MXFP4 4.24 -> 3.31, MXFP6 4.27 -> 3.57, GGUF_Q8_0 3.74 -> 2.94, GGUF_Q6_K 4.73 -> 3.39);
    //  * the float formats, bound by their instructions, take it from 16 rows per CU on (6144 rows: Q6_K 7.70 -> 6.53 us,
    //    MXFP4 6.84 -> 5.99, MXFP6 8.86 -> 7.26; 14336 rows: Q6_K 16.5 -> 13.8);
    //  * the integer-dot formats from 56 rows per CU on (Q4_K 14336 x 4096: 11.67 -> 11.30 us; at 11008 rows the second
    //    form is ahead, Q4_K 10.4 against 9.0 us), GGUF_Q4_0 and GGUF_Q8_0 between 16 and 32 rows per CU as well (6144
    //    rows: GGUF_Q4_0 5.69 -> 5.26 us, GGUF_Q8_0 7.24 -> 7.05);
    //  * GGUF_Q6_K up to 16 rows per CU only (4096 rows 6.16 -> 5.55 us; 14336 rows 13.4 against 14.9), and GGUF_Q4_K
    //    never: its two units per lane share their bytes.
    // (the plain GEMV only: the fused gate/up form measured slower this way, 22.5 -> 25 us)
    if constexpr (!FUSE && FMT != RFQ_GGUF_Q4_K) {
        if (ku > 64 && ku <= 128) {
            const int cus = device_cu_count();
            bool two_wavefronts_per_row = n <= cus * 8;
            if constexpr (!HasIdot<FMT>::value) two_wavefronts_per_row |= n > cus * 16;
            else if constexpr (FMT == RFQ_GGUF_Q6_K) two_wavefronts_per_row |= n <= cus * 16;
            else {
                two_wavefronts_per_row |= n >= cus * 56;
                if constexpr (FMT == RFQ_GGUF_Q4_0 || FMT == RFQ_GGUF_Q8_0)
                    two_wavefronts_per_row |= n > cus * 16 && n < cus * 32;
            }
            if (two_wavefronts_per_row) {
                if constexpr (HasIdot<FMT>::value) return run_idot<FMT, 1, 2, FUSE>(w, x, y, n, k, f, s);
                else return run_xreg<FMT, 1, 2, FUSE>(w, x, y, n, k, f, s);
            }
        }
    }
    if (ku <= 128) return run_idot<FMT, 2, 1, FUSE>(w, x, y, n, k, f, s);
    if (ku <= 256) return run_idot<FMT, 2, 2, FUSE>(w, x, y, n, k, f, s);
    return run_idot<FMT, 2, 4, FUSE>(w, x, y, n, k, f, s);
}

template <int FMT>
int run_generic_m(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    switch (m) {
    case 1: return run_generic<FMT, 1>(w, x, y, n, k, s);
    case 2: return run_generic<FMT, 2>(w, x, y, n, k, s);
    case 3: return run_generic<FMT, 3>(w, x, y, n, k, s);
    case 4: return run_generic<FMT, 4>(w, x, y, n, k, s);
    case 5: return run_generic<FMT, 5>(w, x, y, n, k, s);
    case 6: return run_generic<FMT, 6>(w, x, y, n, k, s);
    case 7: return run_generic<FMT, 7>(w, x, y, n, k, s);
    case 8: return run_generic<FMT, 8>(w, x, y, n, k, s);
    default: return fail(RFQ_E_BADARG, "rfq_gemv: m=%d outside 1..8", m);
    }
}

template <int FMT>
int run(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    const int ku = k / 32;
    if constexpr (NeedsAlignedTensor<FMT>::value) {
        if (!tensor_aligned<FMT>(w, n, k)) return run_generic_m<FMT>(w, x, y, m, n, k, s);
    }
    if (m == 1 && ku > 16 && ku <= 512)                        // (shorter rows leave most of a wavefront's lanes without a unit)
        return run_rows<FMT, false>(w, x, y, n, k, GemvFuse{nullptr, nullptr, 0.0f, 0}, s);
    if constexpr (FMT == RFQ_Q8_0 || FMT == RFQ_GGUF_Q8_0) {
        // (the matrix-core kernel costs the same for any m; up to four vectors the integer-dot batch kernel below is
        // faster where it applies -- 4096 x 4096: m = 2 7.1 against 11.8 us, m = 4 9.7 against 11.8, m = 8 14.3 against 11.8)
        const bool idot_batch_fits = ku > 32 && ku <= 256;
        if (m > (idot_batch_fits ? 4 : 1) && (reinterpret_cast<uintptr_t>(w) & (FMT == RFQ_Q8_0 ? 3u : 1u)) == 0)
            return run_mfma_q8_0<FMT>(w, x, y, m, n, k, s);
    }
    if (HasIdotBatch<FMT>::value && m > 1 && ku > 32 && ku <= 256) {
        // the prepared vectors of a launch live in LDS (112 bytes per unit and vector): a batch that
        // does not fit goes out as launches of four or two vectors
        const size_t lds_limit = 160 * 1024 - 4096;
        int mb = m <= 2 ? 2 : (m <= 4 ? 4 : 8);
        while (mb > 2 && (size_t)mb * ku * 112 > lds_limit) mb /= 2;
        for (int v0 = 0; v0 < m; v0 += mb) {
            const int mv = m - v0 < mb ? m - v0 : mb;
            const float *xv = x + (size_t)v0 * k;
            float *yv = y + (size_t)v0 * n;
            int rc;
            if (mb == 2) rc = run_idot_batch_k<FMT, 2>(w, xv, yv, mv, n, k, s);
            else if (mb == 4) rc = run_idot_batch_k<FMT, 4>(w, xv, yv, mv, n, k, s);
            else rc = run_idot_batch_k<FMT, 8>(w, xv, yv, mv, n, k, s);
            if (rc != RFQ_OK) return rc;
        }
        return RFQ_OK;
    }
    // No batch kernel for this format or row length (the float-path formats; integer formats beyond 256 units per
    // row): from eight million weights on, one decode launch per vector beats the one-row-per-wavefront kernel,
    // although it reads the weights m times (Q6_K, m = 8: 14336 x 4096 321 -> 91 us, 4096 x 4096 80 -> 37 us; at
    // 1024 x 2048 the single launch is the faster one, 11 against 22 us).
    if (m > 1 && ku > 16 && ku <= 512 && (size_t)n * (size_t)k >= ((size_t)1 << 23)) {
        for (int v = 0; v < m; v++) {
            const int rc = run_rows<FMT, false>(w, x + (size_t)v * k, y + (size_t)v * n, n, k, GemvFuse{nullptr, nullptr, 0.0f, 0}, s);
            if (rc != RFQ_OK) return rc;
        }
        return RFQ_OK;
    }
    return run_generic_m<FMT>(w, x, y, m, n, k, s);
}

// The matmul module's variants: the decode GEMV (m == 1) through the kernels of their canonical twins, batches
// and odd shapes through the one-row-per-wavefront kernel.
template <int FMT>
int run_mm(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    const int ku = k / 32;
    if (m == 1 && ku > 16 && ku <= 512) return run_rows<FMT, false>(w, x, y, n, k, GemvFuse{nullptr, nullptr, 0.0f, 0}, s);
    return run_generic_m<FMT>(w, x, y, m, n, k, s);
}

} // namespace

#define RFQ_GEMV_CAT2(a, b) a##b
#define RFQ_GEMV_CAT(a, b) RFQ_GEMV_CAT2(a, b)

// The formats of this part (the others' kernels are not instantiated here).
int RFQ_GEMV_CAT(launch_gemv_part, RFQ_GEMV_PART)(int canonical, const uint8_t *d_w, const float *d_x, float *d_y, int m, int n,
                                                  int k, hipStream_t s)
{
    constexpr int PART = RFQ_GEMV_PART;
    return [&](auto part) -> int {
        constexpr int P = decltype(part)::value;
#define RFQ_GEMV_CASE(F, RUN)                                                             \
    case F:                                                                              \
        if constexpr (gemv_part_of(F) == P) return RUN<F>(d_w, d_x, d_y, m, n, k, s);   \
        break;
        switch (canonical) {
            RFQ_GEMV_CASE(RFQ_Q4_0, run)
            RFQ_GEMV_CASE(RFQ_Q8_0, run)
            RFQ_GEMV_CASE(RFQ_Q4_K, run)
            RFQ_GEMV_CASE(RFQ_Q6_K, run)
            RFQ_GEMV_CASE(RFQ_MXFP4, run)
            RFQ_GEMV_CASE(RFQ_MXFP6_E2M3, run)
            RFQ_GEMV_CASE(RFQ_GGUF_Q4_0, run)
            RFQ_GEMV_CASE(RFQ_GGUF_Q8_0, run)
            RFQ_GEMV_CASE(RFQ_GGUF_Q4_K, run)
            RFQ_GEMV_CASE(RFQ_GGUF_Q6_K, run)
            RFQ_GEMV_CASE(RFQ_MM_Q8_0, run_mm)
            RFQ_GEMV_CASE(RFQ_MM_Q4_K, run_mm)
            RFQ_GEMV_CASE(RFQ_MM_Q6_K, run_mm)
        default: break;
        }
#undef RFQ_GEMV_CASE
        return fail(RFQ_E_UNSUPPORTED, "rfq_gemv: format %d is not in this part of the build", canonical);
    }(std::integral_constant<int, PART>{});
}

int RFQ_GEMV_CAT(launch_gemv_fused_part, RFQ_GEMV_PART)(int canonical, const uint8_t *d_w, const float *d_x, float *d_y, int rows,
                                                        int k, const void *fuse, hipStream_t s)
{
    constexpr int PART = RFQ_GEMV_PART;
    const GemvFuse &f = *static_cast<const GemvFuse *>(fuse);
    return [&](auto part) -> int {
        constexpr int P = decltype(part)::value;
#define RFQ_GEMV_CASE(F)                                                                             \
    case F:                                                                                          \
        if constexpr (gemv_part_of(F) == P) return run_rows<F, true>(d_w, d_x, d_y, rows, k, f, s); \
        break;
        switch (canonical) {
            RFQ_GEMV_CASE(RFQ_Q4_0)
            RFQ_GEMV_CASE(RFQ_Q8_0)
            RFQ_GEMV_CASE(RFQ_Q4_K)
            RFQ_GEMV_CASE(RFQ_Q6_K)
            RFQ_GEMV_CASE(RFQ_MXFP4)
            RFQ_GEMV_CASE(RFQ_MXFP6_E2M3)
            RFQ_GEMV_CASE(RFQ_GGUF_Q4_0)
            RFQ_GEMV_CASE(RFQ_GGUF_Q8_0)
            RFQ_GEMV_CASE(RFQ_GGUF_Q4_K)
            RFQ_GEMV_CASE(RFQ_GGUF_Q6_K)
        default: break;
        }
#undef RFQ_GEMV_CASE
        return fail(RFQ_E_UNSUPPORTED, "fused gemv: format %d is not in this part of the build", canonical);
    }(std::integral_constant<int, PART>{});
}

#if RFQ_GEMV_PART == 0

int launch_gemv(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int m, int n, int k, hipStream_t s)
{
    const int cf = canonical_format(fmt);
    switch (gemv_part_of(cf)) {
    case 0: return launch_gemv_part0(cf, d_w, d_x, d_y, m, n, k, s);
#ifndef RFQ_GEMV_ONLY
    case 1: return launch_gemv_part1(cf, d_w, d_x, d_y, m, n, k, s);
    case 2: return launch_gemv_part2(cf, d_w, d_x, d_y, m, n, k, s);
    case 3: return launch_gemv_part3(cf, d_w, d_x, d_y, m, n, k, s);
#endif
    default: return fail(RFQ_E_BADARG, "rfq_gemv: unknown format %d", fmt);
    }
}

// One launch for RMSNorm -> GEMV (norm_w != nullptr) and / or two GEMVs sharing
// x -> SwiGLU (w2 != nullptr: y[j] = swiglu(w row j . x, w2 row j . x), n counts
// the rows of each matrix).  m == 1 only; RFQ_E_UNSUPPORTED (without an error
// text) when the shape has no such kernel, so the caller can compose the steps.
int launch_gemv_fused(int fmt, const uint8_t *d_w, const uint8_t *d_w2, const float *d_x, const float *d_norm_w,
                      float eps, float *d_y, int n, int k, hipStream_t s)
{
    const int ku = k / 32;
    if (k % 32 != 0 || ku <= 16 || ku > 512 || (d_w2 != nullptr && n > 0x3fffffff)) return RFQ_E_UNSUPPORTED;
    if (k % fmt_block_elems(fmt) != 0) return RFQ_E_UNSUPPORTED;
    const GemvFuse f{d_w2, d_norm_w, eps, d_w2 != nullptr ? 1 : 0};
    const int rows = d_w2 != nullptr ? 2 * n : n;
    // (the 2-byte aligned GGUF blocks are fetched through aligned windows: both matrices must start on a multiple of
    // 4, else the caller composes the separate steps, which take the byte-exact kernel)
    const int cf = canonical_format(fmt);
    if ((cf == RFQ_GGUF_Q6_K || cf == RFQ_GGUF_Q4_0 || cf == RFQ_GGUF_Q8_0) &&
        ((reinterpret_cast<uintptr_t>(d_w) | (d_w2 ? reinterpret_cast<uintptr_t>(d_w2) : 0)) & 3u) != 0)
        return RFQ_E_UNSUPPORTED;
    if (cf == RFQ_MM_Q8_0 || cf == RFQ_MM_Q4_K || cf == RFQ_MM_Q6_K) return fail(RFQ_E_BADARG, "fused gemv: unknown format %d", fmt);
    switch (gemv_part_of(cf)) {
    case 0: return launch_gemv_fused_part0(cf, d_w, d_x, d_y, rows, k, &f, s);
#ifndef RFQ_GEMV_ONLY
    case 1: return launch_gemv_fused_part1(cf, d_w, d_x, d_y, rows, k, &f, s);
    case 2: return launch_gemv_fused_part2(cf, d_w, d_x, d_y, rows, k, &f, s);
    case 3: return launch_gemv_fused_part3(cf, d_w, d_x, d_y, rows, k, &f, s);
#endif
    default: return fail(RFQ_E_BADARG, "fused gemv: unknown format %d", fmt);
    }
}

// One m = 1 launch with the in-kernel timeline (see WaveTrace): the same dispatch as launch_gemv; *waves = 0 when the
// kernel it takes for this format and shape is not compiled with the trace.
int launch_gemv_traced(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int n, int k, unsigned long long *d_trace,
                       size_t capacity_waves, int *waves, hipStream_t s)
{
    g_gemv_trace_request = GemvTraceRequest{d_trace, capacity_waves, 0};
    const int rc = launch_gemv(fmt, d_w, d_x, d_y, 1, n, k, s);
    *waves = g_gemv_trace_request.waves_written;
    g_gemv_trace_request = GemvTraceRequest{nullptr, 0, 0};
    return rc;
}

#endif // part 0

} // namespace rfq

#if RFQ_GEMV_PART == 0
extern "C" RFQ_API const char *rfq_bench_last_gemv_kernel(void)
{
    static thread_local char text[128];
    const rfq::GemvLastKernel &k = rfq::g_gemv_last_kernel;
    const char *f = "?";
    switch (k.fmt) {
    case RFQ_Q4_0: f = "Q4_0"; break;
    case RFQ_Q8_0: f = "Q8_0"; break;
    case RFQ_Q4_K: f = "Q4_K"; break;
    case RFQ_Q6_K: f = "Q6_K"; break;
    case RFQ_MXFP4: f = "MXFP4"; break;
    case RFQ_MXFP6_E2M3: f = "MXFP6"; break;
    case RFQ_GGUF_Q4_0: f = "GGUF_Q4_0"; break;
    case RFQ_GGUF_Q8_0: f = "GGUF_Q8_0"; break;
    case RFQ_GGUF_Q4_K: f = "GGUF_Q4_K"; break;
    case RFQ_GGUF_Q6_K: f = "GGUF_Q6_K"; break;
    case RFQ_MM_Q8_0: f = "MM_Q8_0"; break;
    case RFQ_MM_Q4_K: f = "MM_Q4_K"; break;
    case RFQ_MM_Q6_K: f = "MM_Q6_K"; break;
    default: break;
    }
    snprintf(text, sizeof text, k.name, f, k.a, k.b, k.c);
    return text;
}
#endif // part 0
