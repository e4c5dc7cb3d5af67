// Prefill GEMM for the block formats with f16/f32 scales (Q4_0, Q8_0, Q4_K,
// Q6_K): out[m, n] = A[m, k] (fp16) . dequant(W)[n, k]^T on the fp16 matrix
// cores (v_mfma_f32_32x32x16_f16), fp32 accumulation.
//
// The weights are decoded with the reference's f32 arithmetic (the same
// formulas as the dequantisation kernels, cited there) and rounded ONCE to
// fp16 (round to nearest even) on their way into LDS; activations are fp16
// already, products are exact in the matrix core, sums are fp32.  The only
// error against the fp32 reference is that one rounding: relative 2^-12 per
// weight, independent across k.
//
// Q4_K values are min + q * scale with an integer min of up to +-128 next to a
// small q * scale: rounding the sum to fp16 would lose the small part's bits.
// The two parts are therefore contracted separately:
//   sum_k fp16(q_k * scale) * a_k  +  sum_sb min_sb * S_sb,   S_sb = sum of a over sub-block sb,
// the second as a short extra k loop over (min, S) pairs with S split into
// fp16 hi + lo (exact to 2^-22; min is exact in fp16).  S comes from a small
// pass over A into a stream-ordered temporary of M * K / 16 fp16 values.
//
// Workgroup tile 256 (m) x 128 (n), k advances 64 per stage, two LDS stages.
// Thread t decodes the 32 weights (row t/2, k-group t%2) of a stage: exactly
// one Q4_0/Q8_0 block or one Q4_K/Q6_K sub-block pair.  Four wavefronts in a
// 2 (n) x 2 (m) arrangement, each 64 n x 128 m = 2 x 4 instruction tiles.  The
// weight fragment is the instruction's first operand, so a lane ends up with
// 4 consecutive n of one output row: 8- or 16-byte stores without a transpose.
#include <mutex>

#include "rfq_common.hpp"

// -DRFQ_KQ_SKIP=<mask> (tuning builds, results are wrong on purpose): leave out
// 1 the A loads, 2 the W loads, 4 the LDS fragment reads, 8 the LDS writes,
// 16 the weight decoding, to see what a stage's time is made of.
#ifndef RFQ_KQ_SKIP
#define RFQ_KQ_SKIP 0
#endif

namespace rfq {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
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

constexpr int BM = 256, BN = 128, BK = 64;
constexpr int LDR = BK * 2 + 16;                 // bytes per LDS row: 64 fp16 + 16 pad (rows 36 dwords apart)
constexpr int A_BYTES = BM * LDR, W_BYTES = BN * LDR, STAGE_BYTES = A_BYTES + W_BYTES;

// ---- raw bytes of 32 consecutive weights of a row, and their f32 values -------
template <int FMT> struct Raw32;

// src/kernels/quant/q4_0.rs:289-306: 20-byte block = f32 scale + 16 nibble bytes
template <> struct Raw32<RFQ_Q4_0> {
    static constexpr int ND = 5;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g)
    {
        // few wide loads: every lane touches a different cache line, so the
        // address path pays per instruction, not per byte
        const uint8_t *p = row + (size_t)g * 20;
        d[0] = ld<uint32_t>(p);
        uint4 q = ld<uint4>(p + 4);
        d[1] = q.x; d[2] = q.y; d[3] = q.z; d[4] = q.w;
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
        d[1] = d[2] = d[3] = d[4] = 0x88888888u; // nibble 8 is 0.0
    }
    __device__ __forceinline__ float value(int e) const
    {
        float scale = __uint_as_float(d[0]);
        uint32_t q = (d[1 + (e >> 3)] >> (4 * (e & 7))) & 15u; // element 2i = low nibble of byte i
        return scale * (float)((int)q - 8);
    }
};

// src/kernels/quant/q8_0.rs:55-59: 36-byte block = f32 scale + 32 offset-binary bytes
template <> struct Raw32<RFQ_Q8_0> {
    static constexpr int ND = 9;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g)
    {
        const uint8_t *p = row + (size_t)g * 36;
        d[0] = ld<uint32_t>(p);
        uint4 q0 = ld<uint4>(p + 4), q1 = ld<uint4>(p + 20);
        d[1] = q0.x; d[2] = q0.y; d[3] = q0.z; d[4] = q0.w;
        d[5] = q1.x; d[6] = q1.y; d[7] = q1.z; d[8] = q1.w;
    }
    __device__ __forceinline__ void zero()
    {
        d[0] = 0;
#pragma unroll
        for (int i = 1; i < ND; i++) d[i] = 0x80808080u;
    }
    __device__ __forceinline__ float value(int e) const
    {
        float scale = __uint_as_float(d[0]);
        uint32_t b = (d[1 + (e >> 2)] >> (8 * (e & 3))) & 255u;
        return ((float)b - 128.0f) * scale;
    }
};

// src/kernels/quant/q4_k.rs:222-268: sub-block sb of a 256-byte super-block:
// f16 scale at 2*sb, i8 min at 16+sb, 16 nibble bytes at 32+28*sb
template <> struct Raw32<RFQ_Q4_K> {
    static constexpr int ND = 5;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g)
    {
        const uint8_t *blk = row + (size_t)(g >> 3) * 256;
        const int sb = g & 7;
        // the aligned dwords that hold scale sb and min sb, then the 16 nibble bytes
        uint32_t sc = ld<uint32_t>(blk + 2 * (sb & ~1)), mn = ld<uint32_t>(blk + 16 + (sb & ~3));
        d[0] = ((sc >> (16 * (sb & 1))) & 0xFFFFu) | (((mn >> (8 * (sb & 3))) & 0xFFu) << 16);
        uint4 q = ld<uint4>(blk + 32 + 28 * sb);
        d[1] = q.x; d[2] = q.y; d[3] = q.z; d[4] = q.w;
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    // q * scale only (exact in f32): the min is contracted separately
    __device__ __forceinline__ float value(int e) const
    {
        float scale = f16_bits_to_f32((uint16_t)(d[0] & 0xFFFFu));
        uint32_t q = (d[1 + (e >> 3)] >> (4 * (e & 7))) & 15u;
        return (float)q * scale;
    }
};

// src/kernels/quant/q6_k.rs:221-261: element i of a 256-byte block: f16 scale
// 2*(i/16), signed 6-bit field at bit 6*i of the stream at +32.  32 elements =
// 2 scales (one dword) + 24 stream bytes.
template <> struct Raw32<RFQ_Q6_K> {
    static constexpr int ND = 7;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g)
    {
        const uint8_t *blk = row + (size_t)(g >> 3) * 256;
        const int s = g & 7;
        d[0] = ld<uint32_t>(blk + 4 * s);
        uint4 q = ld<uint4>(blk + 32 + 24 * s);
        uint2 q2 = ld<uint2>(blk + 32 + 24 * s + 16);
        d[1] = q.x; d[2] = q.y; d[3] = q.z; d[4] = q.w; d[5] = q2.x; d[6] = q2.y;
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = 0;
    }
    __device__ __forceinline__ float value(int e) const
    {
        float scale = f16_bits_to_f32((uint16_t)(e < 16 ? d[0] & 0xFFFFu : d[0] >> 16));
        const int bit = 6 * e, w = bit >> 5, o = bit & 31;
        uint64_t two = (uint64_t)d[1 + w] | ((uint64_t)d[1 + (w < 5 ? w + 1 : w)] << 32);
        uint32_t f = (uint32_t)(two >> o);
        return (float)sbfe6(f, 0) * scale;
    }
};

// S[m, sb] = sum of the 32 activations of sub-block sb (fp32, in k order),
// stored as the fp16 pair (hi, lo) with hi + lo = S to 2^-22: [M][K/32][2].
__global__ void __launch_bounds__(256)
group_sums_kernel(const _Float16 *__restrict__ a, _Float16 *__restrict__ s2, int M, int K)
{
    const int groups = K / 32;
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= (size_t)M * groups) return;
    const uint4 *p = reinterpret_cast<const uint4 *>(a + t * 32);
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        uint4 v = p[c];
        v8h h;
        __builtin_memcpy(&h, &v, 16);
#pragma unroll
        for (int e = 0; e < 8; e++) sum += (float)h[e];
    }
    _Float16 hi = (_Float16)sum, lo = (_Float16)(sum - (float)hi);
    s2[2 * t] = hi;
    s2[2 * t + 1] = lo;
}

template <int FMT, bool OUT_F16>
__global__ void __launch_bounds__(256)
gemm_kq_kernel(const uint8_t *__restrict__ w, const _Float16 *__restrict__ a, const _Float16 *__restrict__ s2,
               void *__restrict__ outp, int M, int N, int K)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_n = wave & 1, wave_m = wave >> 1;
    const int tiles_m = (M + BM - 1) / BM;
    const int tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m; // the m tiles of one W tile are neighbours
    const int m0 = tm * BM, n0 = tn * BN;
    const int groups = K / 32;                                    // 32-element groups per row
    const size_t row_bytes = (size_t)(K / Fmt<FMT>::BE) * Fmt<FMT>::BB;
    const int nstages = (K + BK - 1) / BK;

    // this thread's share of a stage: weights (row wr, group wg); 8 A chunks of 16 bytes
    const int wr = tid >> 1, wg = tid & 1;
    const bool w_row_ok = n0 + wr < N;
    const uint8_t *w_row = w + (size_t)(w_row_ok ? n0 + wr : 0) * row_bytes;
    const int a_chunk = tid & 7, a_row0 = tid >> 3;               // rows a_row0 + 32*i

    // Global loads run three stages ahead of the arithmetic, through a ring of
    // three register sets (indices are compile-time: the loop is unrolled by 3).
    Raw32<FMT> raws[3];
    uint4 ras[3][8];
    // The loads are unconditional (clamped addresses): branches around them
    // would make the compiler wait for every outstanding load at each join.
    // Rows past M or N only feed outputs that are never stored; k past K is
    // cancelled by zero weights (selected after the load), whatever finite
    // activations the clamped address returns.
    auto fetch = [&](auto slotc, int st) {
        constexpr int S = decltype(slotc)::value;
        const int g = st * 2 + wg;
        if (!(RFQ_KQ_SKIP & 2)) raws[S].load(w_row, g < groups ? g : groups - 1);
        Raw32<FMT> z;
        z.zero();
#pragma unroll
        for (int i = 0; i < Raw32<FMT>::ND; i++) raws[S].d[i] = g < groups ? raws[S].d[i] : z.d[i];
        const int k = st * BK + a_chunk * 8, kc = k < K ? k : K - 8;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int m = m0 + a_row0 + 32 * i, mc = m < M ? m : M - 1;
            if (!(RFQ_KQ_SKIP & 1)) ras[S][i] = *reinterpret_cast<const uint4 *>(a + (size_t)mc * K + kc);
        }
    };
    // decode + round to fp16 (registers only: free to overlap the matrix instructions)
    auto convert = [&](auto slotc, v8h (&hw)[4]) {
        constexpr int S = decltype(slotc)::value;
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                if (RFQ_KQ_SKIP & 16) hw[c][e] = (_Float16)(float)(raws[S].d[0] & 1023u);
                else hw[c][e] = (_Float16)raws[S].value(8 * c + e); // round to nearest even
            }
    };
    auto stash = [&](auto slotc, const v8h (&hw)[4], int buf) {
        constexpr int S = decltype(slotc)::value;
        uint8_t *abase = lds + buf * STAGE_BYTES, *wbase = abase + A_BYTES;
        if (RFQ_KQ_SKIP & 8) {
            // keep the values alive without the writes (the test is never true for finite data)
            float keep = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) keep += __uint_as_float(ras[S][i].x ^ ras[S][i].y ^ ras[S][i].z ^ ras[S][i].w);
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) keep += (float)hw[c][e];
            if (keep == 1.2345e-30f) *reinterpret_cast<float *>(abase) = keep;
            return;
        }
#pragma unroll
        for (int i = 0; i < 8; i++)
            *reinterpret_cast<uint4 *>(abase + (a_row0 + 32 * i) * LDR + a_chunk * 16) = ras[S][i];
#pragma unroll
        for (int c = 0; c < 4; c++) *reinterpret_cast<v8h *>(wbase + wr * LDR + wg * 64 + c * 16) = hw[c];
    };

    v16f acc[2][4];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0.0f;

    const int fr = lane & 31, fh = lane >> 5;                     // fragment row, k half
    // Fragments of k-step ks+1 are read while the matrix instructions of k-step
    // ks run (two register sets), so LDS latency is paid once per stage.
    auto compute = [&](int buf) {
        const uint8_t *abase = lds + buf * STAGE_BYTES, *wbase = abase + A_BYTES;
        v8h fw[2][2], fa[2][4];
        auto load_frags = [&](int ks, int set) {
            if (RFQ_KQ_SKIP & 4) return;
#pragma unroll
            for (int j = 0; j < 2; j++)
                fw[set][j] = *reinterpret_cast<const v8h *>(wbase + (wave_n * 64 + j * 32 + fr) * LDR + ks * 32 + fh * 16);
#pragma unroll
            for (int i = 0; i < 4; i++)
                fa[set][i] = *reinterpret_cast<const v8h *>(abase + (wave_m * 128 + i * 32 + fr) * LDR + ks * 32 + fh * 16);
        };
        if (RFQ_KQ_SKIP & 4) {
#pragma unroll
            for (int set = 0; set < 2; set++) {
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 8; e++) fw[set][j][e] = (_Float16)(float)(lane + j + e);
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int e = 0; e < 8; e++) fa[set][i][e] = (_Float16)(float)(lane + i - e);
            }
        }
        load_frags(0, 0);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            if (ks + 1 < BK / 16) load_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[ks & 1][j], fa[ks & 1][i], acc[j][i], 0, 0, 0);
        }
    };

    // iteration st: stage st is in LDS; stage st+1 sits in register set NEXT
    // (loaded two iterations ago); set FREE (stage st, already in LDS) takes stage st+3
    auto iter = [&](auto nextc, auto freec, int st) {
        v8h hw[4];
        convert(nextc, hw);                    // (after the last stage this moves a stage nobody reads)
        compute(st & 1);
        stash(nextc, hw, (st + 1) & 1);
        fetch(freec, st + 3);
        lds_barrier();
    };
    {
        v8h hw[4];
        fetch(IC<0>{}, 0);
        fetch(IC<1>{}, 1);
        fetch(IC<2>{}, 2);
        convert(IC<0>{}, hw);
        stash(IC<0>{}, hw, 0);
        lds_barrier();
    }
    for (int st = 0; st < nstages; st += 3) {
        iter(IC<1>{}, IC<0>{}, st);
        if (st + 1 < nstages) iter(IC<2>{}, IC<1>{}, st + 1);
        if (st + 2 < nstages) iter(IC<0>{}, IC<2>{}, st + 2);
    }

    if (FMT == RFQ_Q4_K) {
        // The min term: "k" runs over (sub-block, hi/lo) pairs, K2 = K / 16 of
        // them; weight (n, 2*sb + t) = min[n, sb], activation (m, 2*sb + t) =
        // hi or lo of S[m, sb].  A stage of 64 covers 32 sub-blocks = 4
        // super-blocks; thread (wr, wg) expands the 16 mins of two of them.
        const int K2 = K / 16, nstages2 = (K2 + BK - 1) / BK;
        uint32_t mins[4];
        uint4 (&ra)[8] = ras[0];
        auto fetch2 = [&](int st) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int sblk = st * 4 + wg * 2 + h;             // super-block of this row
                if (w_row_ok && sblk < K / 256) {
                    mins[2 * h] = ld<uint32_t>(w_row + (size_t)sblk * 256 + 16);
                    mins[2 * h + 1] = ld<uint32_t>(w_row + (size_t)sblk * 256 + 20);
                } else {
                    mins[2 * h] = mins[2 * h + 1] = 0;
                }
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int m = m0 + a_row0 + 32 * i, k2 = st * BK + a_chunk * 8;
                if (m < M && k2 < K2) ra[i] = *reinterpret_cast<const uint4 *>(s2 + (size_t)m * K2 + k2);
                else ra[i] = make_uint4(0, 0, 0, 0);
            }
        };
        auto stash2 = [&](int buf) {
            uint8_t *abase = lds + buf * STAGE_BYTES, *wbase = abase + A_BYTES;
#pragma unroll
            for (int i = 0; i < 8; i++)
                *reinterpret_cast<uint4 *>(abase + (a_row0 + 32 * i) * LDR + a_chunk * 16) = ra[i];
#pragma unroll
            for (int c = 0; c < 4; c++) {                          // 4 mins -> 8 fp16 (each twice)
                v8h h;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    _Float16 v = (_Float16)(float)(int8_t)(mins[c] >> (8 * e));
                    h[2 * e] = v;
                    h[2 * e + 1] = v;
                }
                *reinterpret_cast<v8h *>(wbase + wr * LDR + wg * 64 + c * 16) = h;
            }
        };
        fetch2(0);
        stash2(0);
        lds_barrier();
        for (int st = 0; st < nstages2; st++) {
            const bool more = st + 1 < nstages2;
            if (more) fetch2(st + 1);
            compute(st & 1);
            if (more) stash2((st + 1) & 1);
            lds_barrier();
        }
    }

    // Register r of tile (j, i): n = 8*(r/4) + 4*(lane/32) + r%4 within the
    // tile (four consecutive n per r/4), m = lane%32.
    const bool vec_ok = (N % 4) == 0 && (reinterpret_cast<uintptr_t>(outp) & 15u) == 0;
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = m0 + wave_m * 128 + i * 32 + fr;
            if (m >= M) continue;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n = n0 + wave_n * 64 + j * 32 + 8 * g + 4 * fh;
                const size_t o = (size_t)m * N + n;
                if (vec_ok && n + 3 < N) {
                    if (OUT_F16) {
                        typedef _Float16 v4h __attribute__((ext_vector_type(4)));
                        v4h h = {(_Float16)acc[j][i][4 * g], (_Float16)acc[j][i][4 * g + 1],
                                 (_Float16)acc[j][i][4 * g + 2], (_Float16)acc[j][i][4 * g + 3]};
                        *reinterpret_cast<v4h *>(reinterpret_cast<_Float16 *>(outp) + o) = h;
                    } else {
                        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(outp) + o) =
                            make_float4(acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < N) {
                            if (OUT_F16) reinterpret_cast<_Float16 *>(outp)[o + e] = (_Float16)acc[j][i][4 * g + e];
                            else reinterpret_cast<float *>(outp)[o + e] = acc[j][i][4 * g + e];
                        }
                }
            }
        }
}

template <int FMT, bool OUT_F16>
int launch_cfg(const uint8_t *w, const void *a, void *out, int m, int n, int k, hipStream_t s)
{
    constexpr int LDS = 2 * STAGE_BYTES;
    static_assert(LDS <= 160 * 1024, "LDS budget");
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kq_kernel<FMT, OUT_F16>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    });
    if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemm_kq_kernel)");
    const int tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
    _Float16 *s2 = nullptr;
    if (FMT == RFQ_Q4_K) {
        // stream-ordered temporary: allocation and release are queued like the kernels
        RFQ_HIP(hipMallocAsync(reinterpret_cast<void **>(&s2), (size_t)m * (k / 16) * sizeof(_Float16), s));
        const size_t threads = (size_t)m * (k / 32);
        hipLaunchKernelGGL(group_sums_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                           reinterpret_cast<const _Float16 *>(a), s2, m, k);
    }
    hipLaunchKernelGGL((gemm_kq_kernel<FMT, OUT_F16>), dim3(tiles), dim3(256), LDS, s, w,
                       reinterpret_cast<const _Float16 *>(a), s2, out, m, n, k);
    hipError_t launch_err = hipGetLastError();
    if (s2) {
        hipError_t free_err = hipFreeAsync(s2, s);
        if (launch_err == hipSuccess) launch_err = free_err;
    }
    if (launch_err != hipSuccess) return hip_fail(launch_err, "gemm_kq_kernel");
    return RFQ_OK;
}

template <int FMT>
int launch_fmt(const uint8_t *w, const void *a, void *out, int out_dtype, int m, int n, int k, hipStream_t s)
{
    return out_dtype == RFQ_F16 ? launch_cfg<FMT, true>(w, a, out, m, n, k, s)
                                : launch_cfg<FMT, false>(w, a, out, m, n, k, s);
}

} // namespace

int launch_gemm_f16(int fmt, const uint8_t *d_w, const void *d_a, void *d_out, int out_dtype, int m, int n, int k,
                    hipStream_t s)
{
    if (out_dtype != RFQ_F16 && out_dtype != RFQ_F32)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16: out_dtype %d (want RFQ_F32 or RFQ_F16)", out_dtype);
    if ((reinterpret_cast<uintptr_t>(d_a) & 15u) != 0 || k % 8 != 0)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16: activations must be 16-byte aligned with k a multiple of 8");
    switch (fmt) {
    case RFQ_Q4_0: return launch_fmt<RFQ_Q4_0>(d_w, d_a, d_out, out_dtype, m, n, k, s);
    case RFQ_Q8_0: return launch_fmt<RFQ_Q8_0>(d_w, d_a, d_out, out_dtype, m, n, k, s);
    case RFQ_Q4_K: return launch_fmt<RFQ_Q4_K>(d_w, d_a, d_out, out_dtype, m, n, k, s);
    case RFQ_Q6_K: return launch_fmt<RFQ_Q6_K>(d_w, d_a, d_out, out_dtype, m, n, k, s);
    default: return fail(RFQ_E_UNSUPPORTED, "rfq_gemm_f16: no fp16 matrix-core kernel for format %d", fmt);
    }
}

} // namespace rfq
