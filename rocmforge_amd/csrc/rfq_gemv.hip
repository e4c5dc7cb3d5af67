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
#include "rfq_common.hpp"

namespace rfq {
namespace {

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
        q = ld<U4>(blk + 32 + 28 * sb);
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
template <> struct Unit<RFQ_MXFP4> {
    static constexpr bool NEEDS_XSUM = false;
    int e; U4 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *p = row + (size_t)u * 17;
        e = (int)(int8_t)p[0];
        q = ld<U4>(p + 1);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        // bound on |code value|: 8 / 2^e when e >= 1 (exact, 2^(3-e)), else 8.
        float bound = e >= 1 ? __uint_as_float((uint32_t)(130 - e) << 23) : 8.0f;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int d = 0; d < 4; d++) {
#pragma unroll
            for (int b = 0; b < 4; b++) {
                uint32_t byte = (q.v[d] >> (8 * b)) & 255u;
                float hi = decode_e2m1(byte >> 4), lo = decode_e2m1(byte & 15u); // element 2j = high nibble
                hi = __builtin_amdgcn_fmed3f(hi, -bound, bound);
                lo = __builtin_amdgcn_fmed3f(lo, -bound, bound);
                s0 = __builtin_fmaf(hi, x[8 * d + 2 * b], s0);
                s1 = __builtin_fmaf(lo, x[8 * d + 2 * b + 1], s1);
            }
        }
        return mx_scale(e) * (s0 + s1);
    }
};

template <> struct Unit<RFQ_MXFP6_E2M3> {
    static constexpr bool NEEDS_XSUM = false;
    int e; U6 q;
    __device__ __forceinline__ void load(const uint8_t *row, int u)
    {
        const uint8_t *p = row + (size_t)u * 25;
        e = (int)(int8_t)p[0];
        q = ld<U6>(p + 1);
    }
    __device__ __forceinline__ float dot(const float (&x)[32], float) const
    {
        // 7.5 * 2^-e for e >= 1: 7.5 = 0x40F00000 (biased exponent 129).
        float bound = e >= 1 ? __uint_as_float(0x40F00000u - ((uint32_t)e << 23)) : 7.5f;
        float s0 = 0.f, s1 = 0.f;
        // group j: bytes b[3j..3j+3]; see the extraction table in rfq_dequant.hip.
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // bytes 3j..3j+3 as one word w (byte 3j in bits 0-7)
            int bit = 24 * j, d = bit >> 5, sh = bit & 31;
            uint32_t w = (sh == 0) ? q.v[d]
                                   : __builtin_amdgcn_alignbit(d + 1 < 6 ? q.v[d + 1] : 0u, q.v[d], sh);
            uint32_t b0 = w & 255u, b1 = (w >> 8) & 255u, b2 = (w >> 16) & 255u, b3 = w >> 24;
            float v0 = decode_e2m3(b1 >> 2);
            float v1 = decode_e2m3((b0 >> 4) | ((b1 & 3u) << 4));
            float v2 = decode_e2m3((b1 >> 6) | ((b2 & 15u) << 2));
            v0 = __builtin_amdgcn_fmed3f(v0, -bound, bound);
            v1 = __builtin_amdgcn_fmed3f(v1, -bound, bound);
            v2 = __builtin_amdgcn_fmed3f(v2, -bound, bound);
            s0 = __builtin_fmaf(v0, x[4 * j], s0);
            s1 = __builtin_fmaf(v1, x[4 * j + 1], s1);
            s0 = __builtin_fmaf(v2, x[4 * j + 2], s0);
            if (j < 7) { // element 31 is never written by the reference: weight 0
                float v3 = __builtin_amdgcn_fmed3f(decode_e2m3(b3 & 63u), -bound, bound);
                s1 = __builtin_fmaf(v3, x[4 * j + 3], s1);
            }
        }
        return mx_scale(e) * (s0 + s1);
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

// ---- m == 1, x resident in registers ----------------------------------------
//
// Block = 4 wavefronts = 4 / WPR teams.  Lane `tl` of a team (0 .. 64*WPR-1)
// owns units tl + j * 64 * WPR, j < UPL, of EVERY row the team visits.
template <int FMT, int UPL, int WPR>
__global__ void __launch_bounds__(256)
gemv_xreg_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y, int n, int k,
                 int rows_per_team)
{
    constexpr int TEAMS = 4 / WPR, TL = 64 * WPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int team = wave / WPR, wit = wave % WPR;
    const int tl = wit * 64 + lane;
    const int ku = k >> 5;
    const size_t rb = row_bytes<FMT>(k);

    float xs[UPL][32], xsum[UPL];
    bool live[UPL];
#pragma unroll
    for (int j = 0; j < UPL; j++) {
        int u = tl + j * TL;
        live[j] = u < ku;
        if (live[j]) {
            load_x32(x + (size_t)u * 32, xs[j]);
        } else {
#pragma unroll
            for (int i = 0; i < 32; i++) xs[j][i] = 0.f;
        }
        xsum[j] = Unit<FMT>::NEEDS_XSUM ? sum32(xs[j]) : 0.f;
    }

    __shared__ float part[4];
    const int row0 = (blockIdx.x * TEAMS + team) * rows_per_team;

    Unit<FMT> cur[UPL], nxt[UPL];
    if (row0 < n) {
#pragma unroll
        for (int j = 0; j < UPL; j++)
            if (live[j]) cur[j].load(w + (size_t)row0 * rb, tl + j * TL);
    }
    for (int i = 0; i < rows_per_team; i++) {
        const int r = row0 + i;
        const bool have = r < n;
        const bool have_next = (i + 1 < rows_per_team) && (r + 1 < n);
        if (have_next) {
#pragma unroll
            for (int j = 0; j < UPL; j++)
                if (live[j]) nxt[j].load(w + (size_t)(r + 1) * rb, tl + j * TL);
        }
        float acc = 0.f;
        if (have) {
#pragma unroll
            for (int j = 0; j < UPL; j++)
                if (live[j]) acc += cur[j].dot(xs[j], xsum[j]);
        }
        acc = wave_sum(acc);
        if (WPR == 1) {
            if (have && lane == 0) y[r] = acc;
        } else {
            // rows_per_team and the loop bounds are uniform over the block, so
            // every wavefront reaches both barriers the same number of times.
            if (lane == 0) part[wave] = acc;
            __syncthreads();
            if (have && wit == 0 && lane == 0) {
                float t = 0.f;
#pragma unroll
                for (int q = 0; q < WPR; q++) t += part[team * WPR + q];
                y[r] = t;
            }
            __syncthreads();
        }
        if (have_next) {
#pragma unroll
            for (int j = 0; j < UPL; j++) cur[j] = nxt[j];
        }
    }
}

// ---- any m <= 8, any k: one row per wavefront ---------------------------------
template <int FMT, int M>
__global__ void __launch_bounds__(256)
gemv_generic_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y, int n, int k)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ku = k >> 5;
    const size_t rb = row_bytes<FMT>(k);
    const int waves_total = gridDim.x * 4;
    for (int r = blockIdx.x * 4 + wave; r < n; r += waves_total) {
        const uint8_t *row = w + (size_t)r * rb;
        float acc[M];
#pragma unroll
        for (int mi = 0; mi < M; mi++) acc[mi] = 0.f;
        for (int u = lane; u < ku; u += 64) {
            Unit<FMT> un;
            un.load(row, u);
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

template <int FMT, int UPL, int WPR>
int run_xreg(const uint8_t *w, const float *x, float *y, int n, int k, hipStream_t s)
{
    constexpr int TEAMS = 4 / WPR;
    // Two resident blocks per CU; then even out the rows so every team walks
    // the same number of them (no straggler tail on a ~10 us kernel).
    int cus = device_cu_count();
    int blocks = cus * 2;
    int rows_per_team = (n + blocks * TEAMS - 1) / (blocks * TEAMS);
    if (rows_per_team < 1) rows_per_team = 1;
    blocks = (n + rows_per_team * TEAMS - 1) / (rows_per_team * TEAMS);
    hipLaunchKernelGGL((gemv_xreg_kernel<FMT, UPL, WPR>), dim3(blocks), dim3(256), 0, s, w, x, y, n, k, rows_per_team);
    RFQ_LAUNCH_CHECK("gemv_xreg_kernel");
    return RFQ_OK;
}

template <int FMT, int M>
int run_generic(const uint8_t *w, const float *x, float *y, int n, int k, hipStream_t s)
{
    int blocks = (n + 3) / 4;
    int cap = device_cu_count() * 8;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((gemv_generic_kernel<FMT, M>), dim3(blocks), dim3(256), 0, s, w, x, y, n, k);
    RFQ_LAUNCH_CHECK("gemv_generic_kernel");
    return RFQ_OK;
}

template <int FMT>
int run(const uint8_t *w, const float *x, float *y, int m, int n, int k, hipStream_t s)
{
    const int ku = k / 32;
    if (m == 1 && ku > 32) {
        if (ku <= 64) return run_xreg<FMT, 1, 1>(w, x, y, n, k, s);
        if (ku <= 128) return run_xreg<FMT, 2, 1>(w, x, y, n, k, s);
        if (ku <= 256) return run_xreg<FMT, 2, 2>(w, x, y, n, k, s);
        if (ku <= 512) return run_xreg<FMT, 2, 4>(w, x, y, n, k, s);
    }
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

} // namespace

int launch_gemv(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int m, int n, int k, hipStream_t s)
{
    switch (canonical_format(fmt)) {
    case RFQ_Q4_0: return run<RFQ_Q4_0>(d_w, d_x, d_y, m, n, k, s);
    case RFQ_Q8_0: return run<RFQ_Q8_0>(d_w, d_x, d_y, m, n, k, s);
    case RFQ_Q4_K: return run<RFQ_Q4_K>(d_w, d_x, d_y, m, n, k, s);
    case RFQ_Q6_K: return run<RFQ_Q6_K>(d_w, d_x, d_y, m, n, k, s);
    case RFQ_MXFP4: return run<RFQ_MXFP4>(d_w, d_x, d_y, m, n, k, s);
    case RFQ_MXFP6_E2M3: return run<RFQ_MXFP6_E2M3>(d_w, d_x, d_y, m, n, k, s);
    default: return fail(RFQ_E_BADARG, "rfq_gemv: unknown format %d", fmt);
    }
}

} // namespace rfq
