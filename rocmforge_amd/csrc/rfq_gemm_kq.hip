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
// 512 threads; thread t decodes 16 weights of a stage (row t/4, 32-element
// group (t/2)%2, half t%2): half a Q4_0/Q8_0 block or half a Q4_K/Q6_K
// sub-block.  Eight wavefronts in a 2 (n) x 4 (m) arrangement, two per SIMD
// (one runs matrix instructions while the other decodes and moves data), each
// 64 n x 64 m = 2 x 2 instruction tiles.  The weight fragment is the
// instruction's first operand, so a lane ends up with 4 consecutive n of one
// output row: 8- or 16-byte stores without a transpose.
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

constexpr int BM = 256, BN = 128, BK = 64;
constexpr int LDR = BK * 2 + 16;                 // bytes per LDS row: 64 fp16 + 16 pad (rows 36 dwords apart)
constexpr int A_BYTES = BM * LDR, W_BYTES = BN * LDR, STAGE_BYTES = A_BYTES + W_BYTES;

// ---- raw bytes of 16 consecutive weights of a row (half `hf` of the 32-element
// group g), and their f32 values.  Few wide loads: every lane touches a
// different cache line, so the address path pays per instruction, not per byte.
template <int FMT> struct Raw16;

// src/kernels/quant/q4_0.rs:289-306: 20-byte block = f32 scale + 16 nibble bytes
template <> struct Raw16<RFQ_Q4_0> {
    static constexpr int ND = 3;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g, int hf)
    {
        const uint8_t *p = row + (size_t)g * 20;
        d[0] = ld<uint32_t>(p);
        uint2 q = ld<uint2>(p + 4 + 8 * hf);
        d[1] = q.x; d[2] = q.y;
    }
    __device__ __forceinline__ void zero() { d[0] = 0; d[1] = d[2] = 0x88888888u; } // nibble 8 is 0.0
    __device__ __forceinline__ float value(int e) const
    {
        float scale = __uint_as_float(d[0]);
        uint32_t q = (d[1 + (e >> 3)] >> (4 * (e & 7))) & 15u; // element 2i = low nibble of byte i
        return scale * (float)((int)q - 8);
    }
};

// src/kernels/quant/q8_0.rs:55-59: 36-byte block = f32 scale + 32 offset-binary bytes
template <> struct Raw16<RFQ_Q8_0> {
    static constexpr int ND = 5;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g, int hf)
    {
        const uint8_t *p = row + (size_t)g * 36;
        d[0] = ld<uint32_t>(p);
        uint4 q = ld<uint4>(p + 4 + 16 * hf);
        d[1] = q.x; d[2] = q.y; d[3] = q.z; d[4] = q.w;
    }
    __device__ __forceinline__ void zero() { d[0] = 0; d[1] = d[2] = d[3] = d[4] = 0x80808080u; }
    __device__ __forceinline__ float value(int e) const
    {
        float scale = __uint_as_float(d[0]);
        uint32_t b = (d[1 + (e >> 2)] >> (8 * (e & 3))) & 255u;
        return ((float)b - 128.0f) * scale;
    }
};

// src/kernels/quant/q4_k.rs:222-268: sub-block sb of a 256-byte super-block:
// f16 scale at 2*sb, i8 min at 16+sb, 16 nibble bytes at 32+28*sb
template <> struct Raw16<RFQ_Q4_K> {
    static constexpr int ND = 3;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g, int hf)
    {
        const uint8_t *blk = row + (size_t)(g >> 3) * 256;
        const int sb = g & 7;
        d[0] = ld<uint32_t>(blk + 2 * (sb & ~1)) >> (16 * (sb & 1)); // the aligned dword that holds scale sb
        uint2 q = ld<uint2>(blk + 32 + 28 * sb + 8 * hf);
        d[1] = q.x; d[2] = q.y;
    }
    __device__ __forceinline__ void zero() { d[0] = d[1] = d[2] = 0; }
    // q * scale only (exact in f32): the min is contracted separately
    __device__ __forceinline__ float value(int e) const
    {
        float scale = f16_bits_to_f32((uint16_t)(d[0] & 0xFFFFu));
        uint32_t q = (d[1 + (e >> 3)] >> (4 * (e & 7))) & 15u;
        return (float)q * scale;
    }
};

// src/kernels/quant/q6_k.rs:221-261: element i of a 256-byte block: f16 scale
// 2*(i/16), signed 6-bit field at bit 6*i of the stream at +32.  16 elements =
// one scale + 12 stream bytes.
template <> struct Raw16<RFQ_Q6_K> {
    static constexpr int ND = 4;
    uint32_t d[ND];
    __device__ __forceinline__ void load(const uint8_t *row, int g, int hf)
    {
        const uint8_t *blk = row + (size_t)(g >> 3) * 256;
        const int s = g & 7;
        d[0] = ld<uint32_t>(blk + 4 * s) >> (16 * hf);
        const uint8_t *p = blk + 32 + 24 * s + 12 * hf;
        uint2 q = ld<uint2>(p);
        d[1] = q.x; d[2] = q.y; d[3] = ld<uint32_t>(p + 8);
    }
    __device__ __forceinline__ void zero() { d[0] = d[1] = d[2] = d[3] = 0; }
    __device__ __forceinline__ float value(int e) const
    {
        float scale = f16_bits_to_f32((uint16_t)(d[0] & 0xFFFFu));
        const int bit = 6 * e, w = bit >> 5, o = bit & 31;
        uint64_t two = (uint64_t)d[1 + w] | ((uint64_t)d[1 + (w < 2 ? w + 1 : w)] << 32);
        return (float)sbfe6((uint32_t)(two >> o), 0) * scale;
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
__global__ void __launch_bounds__(512)
gemm_kq_kernel(const uint8_t *__restrict__ w, const _Float16 *__restrict__ a, const _Float16 *__restrict__ s2,
               void *__restrict__ outp, int M, int N, int K)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_n = wave & 1, wave_m = wave >> 1;               // 2 x 4 wavefronts
    const int tiles_m = (M + BM - 1) / BM;
    const int tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m; // the m tiles of one W tile are neighbours
    const int m0 = tm * BM, n0 = tn * BN;
    const int groups = K / 32;                                    // 32-element groups per row
    const size_t row_bytes = (size_t)(K / Fmt<FMT>::BE) * Fmt<FMT>::BB;
    const int nstages = (K + BK - 1) / BK;

    // this thread's share of a stage: 16 weights (row wr, group wg, half wh); 4 A chunks of 16 bytes
    const int wr = tid >> 2, wg = (tid >> 1) & 1, wh = tid & 1;
    const bool w_row_ok = n0 + wr < N;
    const uint8_t *w_row = w + (size_t)(w_row_ok ? n0 + wr : 0) * row_bytes;
    const int a_chunk = tid & 7, a_row0 = tid >> 3;               // rows a_row0 + 64*i

    // Global loads run four stages ahead of the arithmetic, through a ring of
    // four register sets (indices are compile-time: the loop is unrolled by 4).
    // (separate objects, not one array: nothing can then index the ring at run time)
    Raw16<FMT> raw0, raw1, raw2, raw3;
    v4u ra0[4], ra1[4], ra2[4], ra3[4];
    auto raw_of = [&](auto slotc) -> Raw16<FMT> & {
        constexpr int S = decltype(slotc)::value;
        if constexpr (S == 0) return raw0;
        else if constexpr (S == 1) return raw1;
        else if constexpr (S == 2) return raw2;
        else return raw3;
    };
    auto ra_of = [&](auto slotc) -> v4u (&)[4] {
        constexpr int S = decltype(slotc)::value;
        if constexpr (S == 0) return ra0;
        else if constexpr (S == 1) return ra1;
        else if constexpr (S == 2) return ra2;
        else return ra3;
    };
    // The loads are unconditional (clamped addresses): branches around them
    // would make the compiler wait for every outstanding load at each join.
    // Rows past M or N only feed outputs that are never stored; k past K is
    // cancelled by zero weights (selected after the load), whatever finite
    // activations the clamped address returns.
    auto fetch = [&](auto slotc, int st) __attribute__((always_inline)) {
        Raw16<FMT> &raw = raw_of(slotc);
        v4u (&ra)[4] = ra_of(slotc);
        const int g = st * 2 + wg;
        if (!(RFQ_KQ_SKIP & 2)) raw.load(w_row, g < groups ? g : groups - 1, wh);
        Raw16<FMT> z;
        z.zero();
#pragma unroll
        for (int i = 0; i < Raw16<FMT>::ND; i++) raw.d[i] = g < groups ? raw.d[i] : z.d[i];
        const int k = st * BK + a_chunk * 8, kc = k < K ? k : K - 8;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = m0 + a_row0 + 64 * i, mc = m < M ? m : M - 1;
            if (!(RFQ_KQ_SKIP & 1)) ra[i] = *reinterpret_cast<const v4u *>(a + (size_t)mc * K + kc);
        }
    };
    // decode + round to fp16 (registers only: free to overlap the matrix instructions)
    auto convert = [&](auto slotc, v8h (&hw)[2]) __attribute__((always_inline)) {
        Raw16<FMT> &raw = raw_of(slotc);
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                if (RFQ_KQ_SKIP & 16) hw[c][e] = (_Float16)(float)(raw.d[0] & 1023u);
                else hw[c][e] = (_Float16)raw.value(8 * c + e); // round to nearest even
            }
    };
    auto stash = [&](auto slotc, const v8h (&hw)[2], int buf) __attribute__((always_inline)) {
        v4u (&ra)[4] = ra_of(slotc);
        uint8_t *abase = lds + buf * STAGE_BYTES, *wbase = abase + A_BYTES;
        if (RFQ_KQ_SKIP & 8) {
            // keep the values alive without the writes (the test is never true for finite data)
            float keep = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) keep += __uint_as_float(ra[i][0] ^ ra[i][1] ^ ra[i][2] ^ ra[i][3]);
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) keep += (float)hw[c][e];
            if (keep == 1.2345e-30f) *reinterpret_cast<float *>(abase) = keep;
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            *reinterpret_cast<v4u *>(abase + (a_row0 + 64 * i) * LDR + a_chunk * 16) = ra[i];
#pragma unroll
        for (int c = 0; c < 2; c++) *reinterpret_cast<v8h *>(wbase + wr * LDR + wg * 64 + wh * 32 + c * 16) = hw[c];
    };

    v16f acc[2][2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0.0f;

    const int fr = lane & 31, fh = lane >> 5;                     // fragment row, k half
    // Fragments of k-step ks+1 are read while the matrix instructions of k-step
    // ks run (two register sets), so LDS latency is paid once per stage.
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const uint8_t *abase = lds + buf * STAGE_BYTES, *wbase = abase + A_BYTES;
        v8h fw[2][2], fa[2][2];
        auto load_frags = [&](int ks, int set) __attribute__((always_inline)) {
            if (RFQ_KQ_SKIP & 4) return;
#pragma unroll
            for (int j = 0; j < 2; j++)
                fw[set][j] = *reinterpret_cast<const v8h *>(wbase + (wave_n * 64 + j * 32 + fr) * LDR + ks * 32 + fh * 16);
#pragma unroll
            for (int i = 0; i < 2; i++)
                fa[set][i] = *reinterpret_cast<const v8h *>(abase + (wave_m * 64 + i * 32 + fr) * LDR + ks * 32 + fh * 16);
        };
        if (RFQ_KQ_SKIP & 4) {
#pragma unroll
            for (int set = 0; set < 2; set++) {
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 8; e++) fw[set][j][e] = (_Float16)(float)(lane + j + e);
#pragma unroll
                for (int i = 0; i < 2; i++)
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
                for (int i = 0; i < 2; i++)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[ks & 1][j], fa[ks & 1][i], acc[j][i], 0, 0, 0);
        }
    };

    // iteration st: stage st is in LDS; stage st+1 sits in register set NEXT
    // (loaded three iterations ago); set FREE (stage st, already in LDS) takes stage st+4
    auto iter = [&](auto nextc, auto freec, int st) __attribute__((always_inline)) {
        v8h hw[2];
        convert(nextc, hw);                    // (after the last stage this moves a stage nobody reads)
        compute(st & 1);
        stash(nextc, hw, (st + 1) & 1);
        fetch(freec, st + 4);
        lds_barrier();
    };
    {
        v8h hw[2];
        fetch(IC<0>{}, 0);
        fetch(IC<1>{}, 1);
        fetch(IC<2>{}, 2);
        fetch(IC<3>{}, 3);
        convert(IC<0>{}, hw);
        stash(IC<0>{}, hw, 0);
        lds_barrier();
    }
    // Whole trips through the ring only (no branch between the three bodies:
    // the compiler would merge their tails and index the ring at run time);
    // stages past the end multiply zero weights.
    for (int st = 0; st < nstages; st += 4) {
        iter(IC<1>{}, IC<0>{}, st);
        iter(IC<2>{}, IC<1>{}, st + 1);
        iter(IC<3>{}, IC<2>{}, st + 2);
        iter(IC<0>{}, IC<3>{}, st + 3);
    }

    if constexpr (FMT == RFQ_Q4_K) {
        // The min term: "k" runs over (sub-block, hi/lo) pairs, K2 = K / 16 of
        // them; weight (n, 2*sb + t) = min[n, sb], activation (m, 2*sb + t) =
        // hi or lo of S[m, sb].  A stage of 64 covers 32 sub-blocks = 4
        // super-blocks; thread (wr, wg, wh) expands the 8 mins of one of them.
        const int K2 = K / 16, nstages2 = (K2 + BK - 1) / BK;
        uint32_t mins[2];
        v4u (&ra)[4] = ra0;
        auto fetch2 = [&](int st) {
            const int sblk = st * 4 + wg * 2 + wh;                // super-block of this row
            if (w_row_ok && sblk < K / 256) {
                mins[0] = ld<uint32_t>(w_row + (size_t)sblk * 256 + 16);
                mins[1] = ld<uint32_t>(w_row + (size_t)sblk * 256 + 20);
            } else {
                mins[0] = mins[1] = 0;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int m = m0 + a_row0 + 64 * i, k2 = st * BK + a_chunk * 8;
                if (m < M && k2 < K2) ra[i] = *reinterpret_cast<const v4u *>(s2 + (size_t)m * K2 + k2);
                else ra[i] = v4u{0, 0, 0, 0};
            }
        };
        auto stash2 = [&](int buf) {
            uint8_t *abase = lds + buf * STAGE_BYTES, *wbase = abase + A_BYTES;
#pragma unroll
            for (int i = 0; i < 4; i++)
                *reinterpret_cast<v4u *>(abase + (a_row0 + 64 * i) * LDR + a_chunk * 16) = ra[i];
#pragma unroll
            for (int c = 0; c < 2; c++) {                          // 4 mins -> 8 fp16 (each twice)
                v8h h;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    _Float16 v = (_Float16)(float)(int8_t)(mins[c] >> (8 * e));
                    h[2 * e] = v;
                    h[2 * e + 1] = v;
                }
                *reinterpret_cast<v8h *>(wbase + wr * LDR + wg * 64 + wh * 32 + c * 16) = h;
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
        for (int i = 0; i < 2; i++) {
            const int m = m0 + wave_m * 64 + i * 32 + fr;
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
    hipLaunchKernelGGL((gemm_kq_kernel<FMT, OUT_F16>), dim3(tiles), dim3(512), LDS, s, w,
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
