// MXFP4 / MXFP6 prefill GEMM on the gfx950 block-scaled matrix instruction
// (v_mfma_scale_f32_32x32x64_f8f6f4), plus the one-time operand re-encoding.
//
//   out[m, n] = sum_k A[m, k] * W[n, k]          fp32 accumulation in the matrix core
//
// Why a re-encoding: ROCmForge stores a signed exponent byte and decodes its
// E2M1 / E2M3 codes with its own tables (code 1 -> 1.0, code 8 -> -0.5, ...,
// clamp to +-8 / +-7.5), the instruction wants a biased E8M0 scale and OCP
// element codes.  Every block is therefore decoded exactly as the reference
// does and re-expressed, value for value, as
//   FP4 kind: OCP E2M1 codes {0.5, 1, 2, 4} * 2^(E-127)   (only if the block's
//             non-zero magnitudes span at most a factor 8 -- always the case
//             for what the reference's own packer emits), or
//   FP8 kind: OCP E4M3 codes * 2^(E-127)                   (always possible).
// The operands keep the reference's values bit for bit, so the GEMM differs
// from the CPU path only in summation order.
//
// Prepared layout ("fragment-major"): rows are grouped in tiles of 32, k in
// steps of 64 (two MX blocks).  One (row-tile, k-step) page holds what the 64
// lanes of a wavefront feed into one matrix instruction: lane l = (kb << 5) | r
// owns row 32*rt + r and the scale of block 2*ks + kb.  FP4: the lane's 16
// bytes are that block's 32 codes, 1 KiB pages.  FP8: 32 bytes per lane as two
// 1 KiB half-pages, half-page b = elements 16*kb .. 16*kb+15 of block 2*ks + b
// (the instruction's 8-bit operand order).  So every global -> LDS ->
// register hop moves contiguous, 16-byte-per-lane, conflict-free data.
// Scales follow the data: per (row-tile, group of 4 k-steps) one dword per
// lane, byte b = scale of k-step 4*g + b (the instruction picks the byte).
#include <mutex>

#include "rfq_common.hpp"

// Tuning builds can switch parts of the GEMM off (-DRFQ_MX_ABLATE=bits: 1 no
// matrix instructions, 2 no global->LDS copies after the prologue, 4 no LDS
// fragment reads inside the loop, 8 no output stores); the library is built without it.
#ifndef RFQ_MX_ABLATE
#define RFQ_MX_ABLATE 0
#endif
// -DRFQ_MX_TRACE: wavefront 0 of every workgroup sums the shader-clock cycles
// it spends in each section of a stage and writes them to rfq_mx_trace.
#ifdef RFQ_MX_TRACE
__device__ unsigned long long *rfq_mx_trace;
#define RFQ_MX_T(n) unsigned long long t##n = __builtin_readcyclecounter()
#define RFQ_MX_ACC(slot, a, b) tacc[slot] += (b) - (a)
#else
#define RFQ_MX_T(n) do { } while (0)
#define RFQ_MX_ACC(slot, a, b) do { } while (0)
#endif

namespace rfq {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct MxLayout {
    int rows, k, rt, ks, ks4;
    size_t page_bytes, data_bytes, scale_bytes;
    __host__ __device__ size_t total() const { return data_bytes + scale_bytes + 16; } // +16: status words
};

__host__ __device__ inline MxLayout mx_layout(int kind, int rows, int k)
{
    MxLayout L;
    L.rows = rows; L.k = k;
    L.rt = (rows + 31) / 32;
    L.ks = k / 64;
    L.ks4 = (L.ks + 3) / 4;
    L.page_bytes = kind == RFQ_MX_FP4 ? 1024 : 2048;
    L.data_bytes = (size_t)L.rt * L.ks * L.page_bytes;
    L.scale_bytes = (size_t)L.rt * L.ks4 * 256;
    return L;
}

// ---- decode one raw block into the reference's 32 values ----------------------

template <int FMT> __device__ __forceinline__ void decode_block(const uint8_t *blk, float (&v)[32]);

template <> __device__ __forceinline__ void decode_block<RFQ_MXFP4>(const uint8_t *blk, float (&v)[32])
{
    float scale = mx_scale((int)(int8_t)blk[0]);
#pragma unroll
    for (int j = 0; j < 16; j++) {
        uint32_t b = blk[1 + j];
        v[2 * j] = clampf(scale * decode_e2m1(b >> 4), -8.0f, 8.0f);
        v[2 * j + 1] = clampf(scale * decode_e2m1(b & 15u), -8.0f, 8.0f);
    }
}

template <> __device__ __forceinline__ void decode_block<RFQ_MXFP6_E2M3>(const uint8_t *blk, float (&v)[32])
{
    float scale = mx_scale((int)(int8_t)blk[0]);
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint8_t *b = blk + 1 + 3 * j;
        uint32_t b0 = b[0], b1 = b[1], b2 = b[2];
        v[4 * j] = clampf(scale * decode_e2m3(b1 >> 2), -7.5f, 7.5f);
        v[4 * j + 1] = clampf(scale * decode_e2m3((b0 >> 4) | ((b1 & 3u) << 4)), -7.5f, 7.5f);
        v[4 * j + 2] = clampf(scale * decode_e2m3((b1 >> 6) | ((b2 & 15u) << 2)), -7.5f, 7.5f);
        v[4 * j + 3] = j < 7 ? clampf(scale * decode_e2m3((uint32_t)b[3] & 63u), -7.5f, 7.5f) : 0.0f;
    }
}

// Unbiased binary exponent of a finite non-zero float (subnormals included).
__device__ __forceinline__ int exponent_of(float a)
{
    float t = fabsf(a) * 18446744073709551616.0f; // 2^64: exact, lifts subnormals into the normal range
    return (int)((__float_as_uint(t) >> 23) & 255u) - 127 - 64;
}

// ---- re-encoding kernels --------------------------------------------------------
//
// One thread per (row, block).  Thread g: lane = g & 63, page = g >> 6.
// status[0] is set to 1 if an FP4 re-encoding met a block it cannot express.

template <int FMT, int KIND>
__global__ void __launch_bounds__(256)
mx_prepare_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ prep, MxLayout L)
{
    constexpr int BB = Fmt<FMT>::BB;
    size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t npages = (size_t)L.rt * L.ks;
    if (g >= npages * 64) return;
    int lane = (int)(g & 63);
    size_t page = g >> 6;
    int rt = (int)(page / L.ks), ks = (int)(page % L.ks);
    int row = rt * 32 + (lane & 31), kb = ks * 2 + (lane >> 5);
    uint32_t *status = reinterpret_cast<uint32_t *>(prep + L.data_bytes + L.scale_bytes);

    float v[32];
    if (row < L.rows) {
        decode_block<FMT>(raw + ((size_t)row * (L.k / 32) + kb) * BB, v);
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) v[i] = 0.0f;
    }
    float vmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) vmax = fmaxf(vmax, fabsf(v[i]));

    int E = 127; // biased E8M0 scale of the re-encoded block
    uint32_t out[8];
#pragma unroll
    for (int i = 0; i < 8; i++) out[i] = 0;

    if (KIND == RFQ_MX_FP4) {
        // codes 1, 2, 4, 6 are 0.5, 1, 2, 4; put the largest magnitude on 4 (or
        // lower if the scale exponent would leave the E8M0 range).
        bool ok = true;
        if (vmax > 0.0f) {
            E = exponent_of(vmax) - 2 + 127;
            if (E < 0) E = 0;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                uint32_t code = 0;
                if (v[i] != 0.0f) {
                    uint32_t bits = __float_as_uint(fabsf(v[i]) * 18446744073709551616.0f);
                    int kx = (int)((bits >> 23) & 255u) - 127 - 64 - (E - 127); // log2(|v| / scale)
                    bool pow2 = (bits & 0x7FFFFFu) == 0;
                    if (!pow2 || kx < -1 || kx > 2) ok = false;
                    code = kx == -1 ? 1u : kx == 0 ? 2u : kx == 1 ? 4u : 6u;
                    if (v[i] < 0.0f) code |= 8u;
                }
                out[i >> 3] |= code << (4 * (i & 7)); // element 2j in the low nibble of byte j
            }
        }
        if (!ok) status[0] = 1u;
        uint4 *dst = reinterpret_cast<uint4 *>(prep + page * 1024 + (size_t)lane * 16);
        *dst = make_uint4(out[0], out[1], out[2], out[3]);
    } else {
        // E4M3: sign, 4 exponent bits (bias 7), 3 mantissa bits.  Largest
        // magnitude scaled into [4, 8): every other value of the block is at
        // most 2^4 below it, inside the normal range.
        if (vmax > 0.0f) {
            E = exponent_of(vmax) - 2 + 127;
            if (E < 0) E = 0;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                uint32_t code = 0;
                if (v[i] != 0.0f) {
                    uint32_t bits = __float_as_uint(fabsf(v[i]) * 18446744073709551616.0f);
                    int p = (int)((bits >> 23) & 255u) - 127 - 64 - (E - 127); // exponent after scaling
                    uint32_t m3 = (bits >> 20) & 7u;
                    if (p >= -6) {
                        code = ((uint32_t)(p + 7) << 3) | m3;
                    } else if (p >= -9) {
                        code = (8u | m3) >> (-6 - p); // subnormal: (1.mmm) shifted into the 3 fraction bits
                    }
                    if (v[i] < 0.0f) code |= 0x80u;
                }
                out[i >> 2] |= code << (8 * (i & 3));
            }
        }
        // 8-bit operands: registers 0-3 of lane (r, h) carry elements 16h..16h+15
        // of the k-step's FIRST block, registers 4-7 the same elements of its
        // SECOND block (the scale of lane (r, h) still belongs to block h).
        // This thread owns block kb = lane >> 5: its low 16 codes go to lane
        // (r, 0), its high 16 to lane (r, 1), both in half-page kb.
        uint8_t *dst = prep + page * 2048 + (size_t)(lane >> 5) * 1024 + (size_t)(lane & 31) * 16;
        *reinterpret_cast<uint4 *>(dst) = make_uint4(out[0], out[1], out[2], out[3]);
        *reinterpret_cast<uint4 *>(dst + 512) = make_uint4(out[4], out[5], out[6], out[7]);
    }
    prep[L.data_bytes + ((size_t)rt * L.ks4 + (ks >> 2)) * 256 + (size_t)lane * 4 + (ks & 3)] = (uint8_t)E;
}

// Scale bytes of k-steps past the end (k not a multiple of 256) and the status words.
__global__ void mx_init_kernel(uint8_t *prep, MxLayout L)
{
    size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (g < L.scale_bytes) prep[L.data_bytes + g] = 127;
    if (g < 4) reinterpret_cast<uint32_t *>(prep + L.data_bytes + L.scale_bytes)[g] = 0;
}

// ---- GEMM ---------------------------------------------------------------------
//
// Workgroup = 4 wavefronts in a WM x WN arrangement, each owning TI x TJ
// instruction tiles (32 x 32) of the output: fp32 accumulators stay in
// registers for the whole k loop (TI*TJ*16 per lane, one wavefront per SIMD).
// k advances 128 per stage (two instruction k-steps).  A stage's operand pages
// and scale dwords are copied global -> LDS by direct-to-LDS loads (no
// registers in between) into a ring of NST slots; a slot is refilled NST
// stages ahead as soon as every wavefront has read it for the last time, so
// HBM / L2 latency is covered by more than NST-1 stages of matrix work.
// One barrier per stage, in the middle of it: after it every wavefront is done
// with the current slot and every wavefront's share of the next stage has
// landed.

template <int KIND> struct Pg { static constexpr int BYTES = KIND == RFQ_MX_FP4 ? 1024 : 2048; };
template <int KIND> struct Cbsz { static constexpr int V = KIND == RFQ_MX_FP4 ? 4 : 0; };

template <int KIND> __device__ __forceinline__ v8i read_frag(const uint8_t *page, int lane)
{
    v8i f;
    uint4 lo = *reinterpret_cast<const uint4 *>(page + lane * 16);
    f[0] = (int)lo.x; f[1] = (int)lo.y; f[2] = (int)lo.z; f[3] = (int)lo.w;
    if (KIND == RFQ_MX_FP4) {
        f[4] = 0; f[5] = 0; f[6] = 0; f[7] = 0;
    } else {
        uint4 hi = *reinterpret_cast<const uint4 *>(page + 1024 + lane * 16);
        f[4] = (int)hi.x; f[5] = (int)hi.y; f[6] = (int)hi.z; f[7] = (int)hi.w;
    }
    return f;
}

__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u); // NaN stays NaN
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);                  // round to nearest even
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding:
// vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]).
template <int N> __device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Direct global -> LDS copy, 64 lanes x 16 bytes: lane l's 16 bytes land at
// lds_addr + 16*l (lds_addr is wave-uniform and travels in M0).  Written as
// assembly on purpose: the compiler then keeps no book on these copies, so it
// does not drain them (vmcnt(0)) in front of every LDS read or barrier; the
// kernel waits for exactly the stage it needs with wait_vmcnt.  Loads the
// compiler cannot see only make its own waits longer, never shorter: the
// counter retires in order.
__device__ __forceinline__ void lds_dma16(const uint8_t *gsrc, uint32_t lds_addr)
{
    // M0 is read when the instruction issues; it is put back right after.
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\t"
                 "s_mov_b32 m0, %2\n\t"
                 "global_load_lds_dwordx4 %1, off\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(gsrc), "s"(lds_addr)
                 : "memory");
}

// Workgroup barrier without the memory-model fence of __syncthreads (which
// would drain every outstanding prefetch); the empty asm statements keep the
// compiler from moving LDS accesses across it.
__device__ __forceinline__ void barrier_no_drain()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int AK, int BK_, int WM, int WN, int TI, int TJ> struct GemmCfg {
    static constexpr int RTA = WM * TI, RTB = WN * TJ;          // row tiles per workgroup
    static constexpr int BM = RTA * 32, BN = RTB * 32;
    static constexpr int PA = Pg<AK>::BYTES, PB = Pg<BK_>::BYTES;
    static constexpr int A_STAGE = RTA * 2 * PA, B_STAGE = RTB * 2 * PB;
    static constexpr int SA_RT = (RTA + 3) / 4 * 4, SB_RT = (RTB + 3) / 4 * 4;
    static constexpr int S_STAGE = (SA_RT + SB_RT) * 256;
    static constexpr int STAGE = A_STAGE + B_STAGE + S_STAGE;
    static constexpr int A_WL = A_STAGE / 1024, B_WL = B_STAGE / 1024, S_WL = S_STAGE / 1024;
    static constexpr int WL = A_WL + B_WL + S_WL;               // 1 KiB wave-loads per stage
    static constexpr int WL_MIN = WL / 4, WL_MAX = (WL + 3) / 4; // per wavefront
    static constexpr int LDS_MAX = 160 * 1024;
    static constexpr int NST = LDS_MAX / STAGE >= 4 ? 4 : LDS_MAX / STAGE; // ring slots
    static_assert(NST >= 2, "a stage must fit LDS twice");
    static_assert((NST - 1) * WL_MIN < 64, "prefetch depth exceeds the load counter");
};

template <int AK, int BK_, bool OUT_BF16, int WM, int WN, int TI, int TJ>
__global__ void __launch_bounds__(256)
gemm_mx_kernel(const uint8_t *__restrict__ ap, const uint8_t *__restrict__ bp, void *__restrict__ outp, int M, int N,
               MxLayout LA, MxLayout LB)
{
    using C = GemmCfg<AK, BK_, WM, WN, TI, TJ>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform, and the compiler may know it
    const int wm = wave % WM, wn = wave / WM;
    // XCD-aware tile order: consecutive workgroup ids land on different XCDs
    // (round robin over 8).  Each XCD gets a contiguous run of tiles that walks
    // the M tiles of one N tile first, so a W tile is fetched into one L2 only.
    const int tiles_m = (M + C::BM - 1) / C::BM, tiles_n = (N + C::BN - 1) / C::BN;
    const int total = tiles_m * tiles_n;
    int bid = blockIdx.x;
    {
        int xcd = bid & 7, slot = bid >> 3;
        int per = (total + 7) / 8;
        int t = xcd * per + slot;
        if (slot >= per || t >= total) return; // uniform over the workgroup
        bid = t;
    }
    const int tn = bid / tiles_m, tmi = bid % tiles_m;
    const int rtA0 = tmi * C::RTA, rtB0 = tn * C::RTB;
    const uint8_t *a_scale = ap + LA.data_bytes, *b_scale = bp + LB.data_bytes;

    // Per-lane global source of each of this wavefront's wave-loads at stage 0;
    // a stage advances data pages by 2 pages and scales by 128 bytes... every
    // second stage (a scale dword covers 4 k-steps = 2 stages).
    const uint8_t *src[C::WL_MAX];
    int kind_of[C::WL_MAX]; // 0 = A data, 1 = B data, 2 = scales
#pragma unroll
    for (int i = 0; i < C::WL_MAX; i++) {
        int j = wave + 4 * i;
        src[i] = ap;
        kind_of[i] = 3;
        if (j < C::A_WL) {
            int off = j * 1024, rtl = off / (2 * C::PA), within = off % (2 * C::PA);
            int rt = rtA0 + rtl;
            if (rt >= LA.rt) rt = LA.rt - 1;
            src[i] = ap + (size_t)rt * LA.ks * C::PA + within + lane * 16;
            kind_of[i] = 0;
        } else if (j < C::A_WL + C::B_WL) {
            int off = (j - C::A_WL) * 1024, rtl = off / (2 * C::PB), within = off % (2 * C::PB);
            int rt = rtB0 + rtl;
            if (rt >= LB.rt) rt = LB.rt - 1;
            src[i] = bp + (size_t)rt * LB.ks * C::PB + within + lane * 16;
            kind_of[i] = 1;
        } else if (j < C::WL) {
            int q = j - C::A_WL - C::B_WL;           // 1 KiB = 4 row tiles x 256 bytes
            int rtl = q * 4 + (lane >> 4);
            bool isb = rtl >= C::SA_RT;
            int r = isb ? rtl - C::SA_RT : rtl;
            int rt = (isb ? rtB0 : rtA0) + r;
            int rtmax = isb ? LB.rt : LA.rt;
            if (rt >= rtmax) rt = rtmax - 1;
            src[i] = (isb ? b_scale : a_scale) + (size_t)rt * (isb ? LB.ks4 : LA.ks4) * 256 + (lane & 15) * 16;
            kind_of[i] = 2;
        }
    }
    // i-th copy of stage `st` by this wavefront into the ring slot at LDS address `slot`
    auto issue_piece = [&](int st, uint32_t slot, int i) {
        int j = wave + 4 * i;
        if (j < C::WL) {
            size_t adv = kind_of[i] == 0 ? (size_t)st * 2 * C::PA
                       : kind_of[i] == 1 ? (size_t)st * 2 * C::PB
                                         : (size_t)(st >> 1) * 256;
            lds_dma16(src[i] + adv, __builtin_amdgcn_readfirstlane(slot + j * 1024));
        }
    };
    auto issue = [&](int st) {
        // LDS byte address of the ring slot (the low 32 bits of a __shared__ pointer)
        uint32_t slot = (uint32_t)(uintptr_t)(lds + (st % C::NST) * C::STAGE);
        slot = __builtin_amdgcn_readfirstlane(slot);
#pragma unroll
        for (int i = 0; i < C::WL_MAX; i++) issue_piece(st, slot, i);
    };

    v16f acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int nstages = LA.ks / 2;
    // Ring prologue: NST stages requested, stage 0 awaited.
#pragma unroll
    for (int d = 0; d < C::NST; d++)
        if (d < nstages) issue(d);
    if (C::NST - 1 < nstages) wait_vmcnt<(C::NST - 1) * C::WL_MIN>();
    else wait_vmcnt<0>();
    barrier_no_drain();

    // One wavefront per SIMD owns the matrix core, so nothing but this
    // instruction stream can hide latency: fragment registers are
    // double-buffered by hand and every other piece of work of a stage (LDS
    // reads of the next k-step, the refill copies, the barrier) is slotted
    // between two matrix instructions (32 cycles each).  sched_barrier pins
    // that order against the compiler's instruction scheduler.
    constexpr int NMMA = TI * TJ, NFRAG = TI + TJ;
    constexpr int PPS = (C::WL_MAX + NMMA - 1) / NMMA;      // refill copies per matrix-instruction slot
    static_assert(NFRAG + 1 <= NMMA, "not enough matrix instructions to hide the fragment reads");
    v8i fa0[TI], fb0[TJ], fa1[TI], fb1[TJ];
    int sa[TI], sb[TJ], sa_n[TI], sb_n[TJ];
    auto read_piece = [&](const uint8_t *base, int ksl, int q, v8i (&fa)[TI], v8i (&fb)[TJ]) {
        if (q < TI) fa[q] = read_frag<AK>(base + ((wm * TI + q) * 2 + ksl) * C::PA, lane);
        else fb[q - TI] = read_frag<BK_>(base + C::A_STAGE + ((wn * TJ + (q - TI)) * 2 + ksl) * C::PB, lane);
    };
    // The stage uses scale bytes 2*(st&1) and 2*(st&1)+1 of its dwords: shift
    // them down so the instruction's byte selectors are constants.
    auto scale_piece = [&](const uint8_t *base, int st, int q, int (&xa)[TI], int (&xb)[TJ]) {
        const uint8_t *sA = base + C::A_STAGE + C::B_STAGE, *sB = sA + C::SA_RT * 256;
        const int sh = 16 * (st & 1);
        if (q < TI) xa[q] = (int)(*reinterpret_cast<const uint32_t *>(sA + ((wm * TI + q) * 64 + lane) * 4) >> sh);
        else xb[q - TI] = (int)(*reinterpret_cast<const uint32_t *>(sB + ((wn * TJ + (q - TI)) * 64 + lane) * 4) >> sh);
    };
#pragma unroll
    for (int q = 0; q < NFRAG; q++) {
        read_piece(lds, 0, q, fa0, fb0);
        scale_piece(lds, 0, q, sa, sb);
    }

#ifdef RFQ_MX_TRACE
    unsigned long long tacc[6] = {0, 0, 0, 0, 0, 0};
    unsigned long long t_begin = __builtin_readcyclecounter();
#endif
    for (int st = 0; st < nstages; st++) {
        RFQ_MX_T(0);
        const uint8_t *base = lds + (st % C::NST) * C::STAGE;
        const uint8_t *nbase = lds + ((st + 1) % C::NST) * C::STAGE;
        const bool more = st + 1 < nstages;
        const bool refill = st + C::NST < nstages;
        uint32_t slot = (uint32_t)(uintptr_t)(lds + (st % C::NST) * C::STAGE);
        slot = __builtin_amdgcn_readfirstlane(slot);

        // k-step 0 of the stage; its shadow: reads of k-step 1, then the hand-over.
#pragma unroll
        for (int q = 0; q < NMMA; q++) {
            if (!(RFQ_MX_ABLATE & 1))
                acc[q / TJ][q % TJ] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    fa0[q / TJ], fb0[q % TJ], acc[q / TJ][q % TJ], Cbsz<AK>::V, Cbsz<BK_>::V, 0, sa[q / TJ], 0,
                    sb[q % TJ]);
            __builtin_amdgcn_sched_barrier(0);
            if (q < NFRAG && !(RFQ_MX_ABLATE & 4)) read_piece(base, 1, q, fa1, fb1);
            if (q == NMMA - 2) {
                RFQ_MX_T(1);
                RFQ_MX_ACC(0, t0, t1);
                // Hand-over: this wavefront's last reads of the slot are
                // complete (lgkmcnt), the next stage has landed (vmcnt),
                // everyone agrees (barrier).  Afterwards the slot may be
                // refilled NST stages ahead.
                __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0) only
                RFQ_MX_T(2);
                RFQ_MX_ACC(1, t1, t2);
                if (more) {
                    if (st + C::NST - 1 < nstages) wait_vmcnt<(C::NST - 2) * C::WL_MIN>();
                    else wait_vmcnt<0>();
                }
                RFQ_MX_T(3);
                RFQ_MX_ACC(2, t2, t3);
                barrier_no_drain();
                RFQ_MX_T(4);
                RFQ_MX_ACC(3, t3, t4);
#ifdef RFQ_MX_TRACE
                tacc[5] = t4; // start of the second half
#endif
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // k-step 1; its shadow: refill copies, reads of the next stage's k-step 0 and scales.
#pragma unroll
        for (int q = 0; q < NMMA; q++) {
            if (!(RFQ_MX_ABLATE & 1))
                acc[q / TJ][q % TJ] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    fa1[q / TJ], fb1[q % TJ], acc[q / TJ][q % TJ], Cbsz<AK>::V, Cbsz<BK_>::V, 1, sa[q / TJ], 1,
                    sb[q % TJ]);
            __builtin_amdgcn_sched_barrier(0);
            if (refill && !(RFQ_MX_ABLATE & 2)) {
#pragma unroll
                for (int pp = 0; pp < PPS; pp++)
                    if (q * PPS + pp < C::WL_MAX) issue_piece(st + C::NST, slot, q * PPS + pp);
            }
            if (q < NFRAG && more) {
                if (!(RFQ_MX_ABLATE & 4)) read_piece(nbase, 0, q, fa0, fb0);
                scale_piece(nbase, st + 1, q, sa_n, sb_n);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (RFQ_MX_ABLATE & 1) {
#pragma unroll
            for (int i = 0; i < TI; i++) acc[i][0][0] += (float)(fa0[i][0] ^ fa1[i][1]);
#pragma unroll
            for (int j = 0; j < TJ; j++) acc[0][j][1] += (float)(fb0[j][0] ^ fb1[j][1]);
        }
#pragma unroll
        for (int i = 0; i < TI; i++) sa[i] = sa_n[i];
#pragma unroll
        for (int j = 0; j < TJ; j++) sb[j] = sb_n[j];
#ifdef RFQ_MX_TRACE
        {
            unsigned long long t9 = __builtin_readcyclecounter();
            tacc[4] += t9 - tacc[5];
        }
#endif
    }
#ifdef RFQ_MX_TRACE
    unsigned long long t_loop_end = __builtin_readcyclecounter();
#endif

    // Epilogue.  Accumulator register r of tile (i, j) is row
    // 8*(r/4) + 4*(lane/32) + r%4, column lane%32 of the tile: a lane owns
    // single elements scattered over rows.  Interior wavefront blocks go through
    // LDS (the ring is free now), one 32-row band at a time, and leave as whole
    // rows in 16-byte stores; ragged blocks fall back to element stores.
    constexpr int ES = OUT_BF16 ? 2 : 4;
    constexpr int ROW_BYTES = TJ * 32 * ES;                 // one band row of this wavefront
    constexpr int ROW_STRIDE = ROW_BYTES + 16;              // +4 dwords: the two half-waves (rows R, R+4) miss each other's banks
    constexpr int CPR = ROW_BYTES / 16;                     // 16-byte chunks per row
    static_assert(4 * 32 * ROW_STRIDE <= C::NST * C::STAGE, "epilogue staging exceeds the ring");
    const int m_base = tmi * C::BM + wm * TI * 32, n_base = tn * C::BN + wn * TJ * 32;
    const bool interior = m_base + TI * 32 <= M && n_base + TJ * 32 <= N && ((size_t)N * ES) % 16 == 0 &&
                          (reinterpret_cast<uintptr_t>(outp) & 15u) == 0 && !(RFQ_MX_ABLATE & 8);
    barrier_no_drain(); // every wavefront is past its last fragment read
    uint8_t *stage = lds + (size_t)wave * 32 * ROW_STRIDE;
    if (interior) {
#pragma unroll
        for (int i = 0; i < TI; i++) {
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int row = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    uint8_t *dst = stage + row * ROW_STRIDE + (32 * j + (lane & 31)) * ES;
                    if (OUT_BF16) *reinterpret_cast<uint16_t *>(dst) = f32_to_bf16(acc[i][j][r]);
                    else *reinterpret_cast<float *>(dst) = acc[i][j][r];
                }
            // LDS operations of one wavefront execute in order: no barrier needed
            // between its own writes and reads of its own staging area.
#pragma unroll
            for (int c0 = 0; c0 < 32 * CPR; c0 += 64) {
                int c = c0 + lane;
                if (c < 32 * CPR) {
                    int row = c / CPR, col16 = c % CPR;
                    uint4 v = *reinterpret_cast<const uint4 *>(stage + row * ROW_STRIDE + col16 * 16);
                    uint8_t *o = reinterpret_cast<uint8_t *>(outp) +
                                 ((size_t)(m_base + 32 * i + row) * N + n_base) * ES + col16 * 16;
                    *reinterpret_cast<uint4 *>(o) = v;
                }
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                int n = n_base + 32 * j + (lane & 31);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int m = m_base + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if ((RFQ_MX_ABLATE & 8) && (i | j | r)) continue;
                    if (m < M && n < N) {
                        if (OUT_BF16)
                            reinterpret_cast<uint16_t *>(outp)[(size_t)m * N + n] = f32_to_bf16(acc[i][j][r]);
                        else
                            reinterpret_cast<float *>(outp)[(size_t)m * N + n] = acc[i][j][r];
                    }
                }
            }
    }
#ifdef RFQ_MX_TRACE
    if (tid == 0 && rfq_mx_trace) {
        unsigned long long t_end = __builtin_readcyclecounter();
        unsigned long long *o = rfq_mx_trace + (size_t)blockIdx.x * 8;
        o[0] = tacc[0]; o[1] = tacc[1]; o[2] = tacc[2]; o[3] = tacc[3]; o[4] = tacc[4];
        o[5] = t_loop_end - t_begin; o[6] = t_end - t_loop_end; o[7] = t_begin;
    }
#endif
}

template <int AK, int BK_, bool OUT_BF16, int WM, int WN, int TI, int TJ>
int launch_gemm_cfg(const uint8_t *a, const uint8_t *b, void *out, int m, int n, int k, hipStream_t s)
{
    using C = GemmCfg<AK, BK_, WM, WN, TI, TJ>;
    MxLayout LA = mx_layout(AK, m, k), LB = mx_layout(BK_, n, k);
    constexpr size_t LDS = (size_t)C::NST * C::STAGE;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&gemm_mx_kernel<AK, BK_, OUT_BF16, WM, WN, TI, TJ>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
    });
    if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemm_mx_kernel)");
    int tiles = ((m + C::BM - 1) / C::BM) * ((n + C::BN - 1) / C::BN);
    int per = (tiles + 7) / 8;
    hipLaunchKernelGGL((gemm_mx_kernel<AK, BK_, OUT_BF16, WM, WN, TI, TJ>), dim3(per * 8), dim3(256), LDS, s, a, b,
                       out, m, n, LA, LB);
    RFQ_LAUNCH_CHECK("gemm_mx_kernel");
    return RFQ_OK;
}

// Two output tilings: 256 x 256 (2 x 2 wavefronts of 4 x 4 tiles) and 256 x 224
// (4 x 1 wavefronts of 2 x 7 tiles).  The one that leaves the last round of
// workgroups fuller wins (28672 = 128 * 224 fills 256 CUs exactly four times
// at M = 2048; 256-wide tiles would run 3.5 rounds).
template <int AK, int BK_, bool OUT_BF16>
int run_gemm(const uint8_t *a, const uint8_t *b, void *out, int m, int n, int k, hipStream_t s)
{
    const int cus = device_cu_count();
    auto rounds_cost = [&](int bm, int bn) {
        long tiles = (long)((m + bm - 1) / bm) * ((n + bn - 1) / bn);
        long rounds = (tiles + cus - 1) / cus;
        return (double)rounds * bm * bn; // time ~ rounds x tile area
    };
    if (rounds_cost(256, 224) < rounds_cost(256, 256))
        return launch_gemm_cfg<AK, BK_, OUT_BF16, 4, 1, 2, 7>(a, b, out, m, n, k, s);
    return launch_gemm_cfg<AK, BK_, OUT_BF16, 2, 2, 4, 4>(a, b, out, m, n, k, s);
}

template <int FMT, int KIND>
int run_prepare(const uint8_t *raw, uint8_t *prep, const MxLayout &L, hipStream_t s)
{
    size_t threads = (size_t)L.rt * L.ks * 64;
    size_t init = L.scale_bytes > 4 ? L.scale_bytes : 4;
    hipLaunchKernelGGL(mx_init_kernel, dim3((unsigned)((init + 255) / 256)), dim3(256), 0, s, prep, L);
    RFQ_LAUNCH_CHECK("mx_init_kernel");
    hipLaunchKernelGGL((mx_prepare_kernel<FMT, KIND>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, raw,
                       prep, L);
    RFQ_LAUNCH_CHECK("mx_prepare_kernel");
    return RFQ_OK;
}

} // namespace

size_t mx_prepared_bytes(int fmt, int kind, int rows, int k)
{
    if (fmt != RFQ_MXFP4 && fmt != RFQ_MXFP6_E2M3 && fmt != RFQ_MXFP6_E3M2) return 0;
    if (rows <= 0 || k <= 0 || k % 128 != 0) return 0;
    if (kind == RFQ_MX_AUTO) kind = RFQ_MX_FP8;
    if (kind != RFQ_MX_FP4 && kind != RFQ_MX_FP8) return 0;
    if (kind == RFQ_MX_FP4 && fmt != RFQ_MXFP4) return 0;
    return mx_layout(kind, rows, k).total();
}

int launch_mx_prepare(int fmt, int kind_req, const uint8_t *d_raw, int rows, int k, void *d_prep, size_t prep_bytes,
                      int *kind_out, hipStream_t s)
{
    const bool is4 = fmt == RFQ_MXFP4;
    if (kind_req == RFQ_MX_FP4 && !is4)
        return fail(RFQ_E_UNSUPPORTED, "rfq_mx_prepare: MXFP6 has no 4-bit re-encoding");
    uint8_t *prep = static_cast<uint8_t *>(d_prep);
    if ((reinterpret_cast<uintptr_t>(prep) & 15u) != 0)
        return fail(RFQ_E_BADARG, "rfq_mx_prepare: prepared buffer must be 16-byte aligned");

    if (is4 && kind_req != RFQ_MX_FP8) {
        MxLayout L = mx_layout(RFQ_MX_FP4, rows, k);
        size_t need = kind_req == RFQ_MX_AUTO ? mx_layout(RFQ_MX_FP8, rows, k).total() : L.total();
        if (prep_bytes < need)
            return fail(RFQ_E_SIZE, "rfq_mx_prepare: prepared buffer has %zu bytes, needs %zu", prep_bytes, need);
        int rc = run_prepare<RFQ_MXFP4, RFQ_MX_FP4>(d_raw, prep, L, s);
        if (rc != RFQ_OK) return rc;
        uint32_t status = 0;
        RFQ_HIP(hipMemcpyAsync(&status, prep + L.data_bytes + L.scale_bytes, 4, hipMemcpyDeviceToHost, s));
        RFQ_HIP(hipStreamSynchronize(s));
        if (status == 0) {
            if (kind_out) *kind_out = RFQ_MX_FP4;
            return RFQ_OK;
        }
        if (kind_req == RFQ_MX_FP4)
            return fail(RFQ_E_UNSUPPORTED, "rfq_mx_prepare: a block's magnitudes span more than the 4-bit codes hold");
        // AUTO: fall through to the 8-bit re-encoding
    }
    MxLayout L = mx_layout(RFQ_MX_FP8, rows, k);
    if (prep_bytes < L.total())
        return fail(RFQ_E_SIZE, "rfq_mx_prepare: prepared buffer has %zu bytes, needs %zu", prep_bytes, L.total());
    int rc = is4 ? run_prepare<RFQ_MXFP4, RFQ_MX_FP8>(d_raw, prep, L, s)
                 : run_prepare<RFQ_MXFP6_E2M3, RFQ_MX_FP8>(d_raw, prep, L, s);
    if (rc != RFQ_OK) return rc;
    if (kind_out) *kind_out = RFQ_MX_FP8;
    return RFQ_OK;
}

int launch_gemm_mx(const void *d_a, int a_kind, const void *d_w, int w_kind, void *d_out, int out_dtype, int m,
                   int n, int k, hipStream_t s)
{
    const uint8_t *a = static_cast<const uint8_t *>(d_a), *b = static_cast<const uint8_t *>(d_w);
    if (((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) != 0)
        return fail(RFQ_E_BADARG, "rfq_gemm_mx: prepared operands must be 16-byte aligned");
    const bool bf = out_dtype == RFQ_BF16;
    if (a_kind == RFQ_MX_FP4 && w_kind == RFQ_MX_FP4)
        return bf ? run_gemm<RFQ_MX_FP4, RFQ_MX_FP4, true>(a, b, d_out, m, n, k, s)
                  : run_gemm<RFQ_MX_FP4, RFQ_MX_FP4, false>(a, b, d_out, m, n, k, s);
    if (a_kind == RFQ_MX_FP4 && w_kind == RFQ_MX_FP8)
        return bf ? run_gemm<RFQ_MX_FP4, RFQ_MX_FP8, true>(a, b, d_out, m, n, k, s)
                  : run_gemm<RFQ_MX_FP4, RFQ_MX_FP8, false>(a, b, d_out, m, n, k, s);
    if (a_kind == RFQ_MX_FP8 && w_kind == RFQ_MX_FP4)
        return bf ? run_gemm<RFQ_MX_FP8, RFQ_MX_FP4, true>(a, b, d_out, m, n, k, s)
                  : run_gemm<RFQ_MX_FP8, RFQ_MX_FP4, false>(a, b, d_out, m, n, k, s);
    return bf ? run_gemm<RFQ_MX_FP8, RFQ_MX_FP8, true>(a, b, d_out, m, n, k, s)
              : run_gemm<RFQ_MX_FP8, RFQ_MX_FP8, false>(a, b, d_out, m, n, k, s);
}

} // namespace rfq
