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

// -DRFQ_MX_TRACE (tuning builds): every workgroup records wall-clock stamps
// (100 MHz) at kernel entry, loop entry, loop exit and exit.
#ifdef RFQ_MX_TRACE
__device__ unsigned long long *rfq_mx_trace;
#define RFQ_MX_STAMP(slot)                                                                                     \
    do {                                                                                                       \
        if (threadIdx.x == 0 && rfq_mx_trace) rfq_mx_trace[(size_t)blockIdx.x * 4 + (slot)] = wall_clock64(); \
    } while (0)
#else
#define RFQ_MX_STAMP(slot) do { } while (0)
#endif
// Ring depth (W slots in LDS = A fragment sets in registers) of the 4-bit kernel.
#ifndef RFQ_MX_RING
#define RFQ_MX_RING 6
#endif

namespace rfq {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
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
// k advances 128 per stage (two instruction k-steps).  One barrier per stage,
// in the middle of it: after it every wavefront is done with the current W
// slot and every wavefront's share of the next stage has landed.

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

// Workgroup = 4 wavefronts stacked along M, one per SIMD.  Wavefront w owns
// rows [64w, 64w+64) of the 256-row tile and ALL its TJ*32 columns: TI = 2 by TJ
// instruction tiles, 32*TJ fp32 accumulators per lane for the whole k loop.
//   W pages (shared by the four wavefronts) travel global -> LDS by direct
//     copies into a ring of RING stage slots, refilled RING stages ahead;
//   A pages (private to a wavefront) travel global -> registers, RING-1 stages
//     ahead, and never touch LDS.
// Splitting the operands this way matters: with both in LDS the LDS port
// (128 B/clk) saturates before the matrix cores do.
template <int BK_, int TJ, int RING_> struct GemmCfg {
    static constexpr int TI = 2, WM = 4, RING = RING_;
    static constexpr int BM = WM * TI * 32, BN = TJ * 32;
    static constexpr int PB = Pg<BK_>::BYTES;
    static constexpr int B_STAGE = TJ * 2 * PB;
    static constexpr int SB_RT = (TJ + 3) / 4 * 4;
    static constexpr int S_STAGE = SB_RT * 256;
    static constexpr int STAGE = B_STAGE + S_STAGE;
    static constexpr int WL = STAGE / 1024;                       // 1 KiB wave-copies per stage
    static constexpr int ND = (WL + 3) / 4;                       // per wavefront (padded with repeats)
};

template <int N> struct IC { static constexpr int value = N; };

template <int AK, int BK_, bool OUT_BF16, int TJ, int RING>
__global__ void __launch_bounds__(256)
gemm_mx_kernel(const uint8_t *__restrict__ ap, const uint8_t *__restrict__ bp, void *__restrict__ outp, int M, int N,
               MxLayout LA, MxLayout LB)
{
    RFQ_MX_STAMP(0);
    using C = GemmCfg<BK_, TJ, RING>;
    constexpr int TI = C::TI, PA = Pg<AK>::BYTES;
    constexpr int NMMA = TI * TJ;
    constexpr int A_PER_FRAG = AK == RFQ_MX_FP4 ? 1 : 2;
    constexpr int NA_OPS = TI * 2 * A_PER_FRAG + TI;          // vector loads per stage for A and its scales
    constexpr int A_PPS = (NA_OPS + NMMA - 3) / (NMMA - 2);   // A loads per slot: all issued before the hand-over at slot NMMA-2
    constexpr int D_PPS = (C::ND + NMMA - 1) / NMMA;          // W copies per slot
    // Vector-memory operations a wavefront issues after the last one of stage
    // s+1 and before the hand-over of stage s (see the schedule below).
    constexpr int HANDOVER_VMCNT = (RING - 2) * (NA_OPS + C::ND);
    constexpr int PROLOGUE_VMCNT = (RING - 1) * C::ND + (RING - 2) * NA_OPS;
    static_assert(HANDOVER_VMCNT < 64 && PROLOGUE_VMCNT < 64, "prefetch depth exceeds the 6-bit load counter");
    static_assert(TJ + 1 <= NMMA, "not enough matrix instructions to hide the fragment reads");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform, and the compiler may know it
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
    const int rtB0 = tn * TJ;
    const uint8_t *b_scale = bp + LB.data_bytes;
    const int nstages = LA.ks / 2;
    const int last = nstages - 1;

    // ---- A: this lane's page pointers (k-step 0) and scale pointers --------
    const uint8_t *a_ptr[TI], *as_ptr[TI];
#pragma unroll
    for (int i = 0; i < TI; i++) {
        int rt = tmi * (C::WM * TI) + wave * TI + i;
        if (rt >= LA.rt) rt = LA.rt - 1;
        a_ptr[i] = ap + (size_t)rt * LA.ks * PA + lane * 16;
        as_ptr[i] = ap + LA.data_bytes + (size_t)rt * LA.ks4 * 256 + lane * 4;
    }
    v8i areg[RING][TI][2];   // 8-bit A fragments
    v4i areg4[RING][TI][2];  // 4-bit A fragments
    int ascl[RING][TI];

    // ---- W: per-lane global source of each of this wavefront's wave-copies ---
    const uint8_t *src[C::ND];
    bool is_scale[C::ND];
    int dst_off[C::ND];
#pragma unroll
    for (int i = 0; i < C::ND; i++) {
        int j = wave + 4 * i;
        if (j >= C::WL) j = C::WL - 1;               // pad: repeat the last copy (same bytes, same place)
        dst_off[i] = j * 1024;
        if (j * 1024 < C::B_STAGE) {
            int off = j * 1024, rtl = off / (2 * C::PB), within = off % (2 * C::PB);
            int rt = rtB0 + rtl;
            if (rt >= LB.rt) rt = LB.rt - 1;
            src[i] = bp + (size_t)rt * LB.ks * C::PB + within + lane * 16;
            is_scale[i] = false;
        } else {
            int q = j - C::B_STAGE / 1024;           // 1 KiB = 4 row tiles x 256 bytes
            int rt = rtB0 + q * 4 + (lane >> 4);
            if (rt >= LB.rt) rt = LB.rt - 1;
            src[i] = b_scale + (size_t)rt * LB.ks4 * 256 + (lane & 15) * 16;
            is_scale[i] = true;
        }
    }
    // Prefetches past the last stage re-fetch the last stage (into slots and
    // registers nobody reads again): every stage then issues the same number
    // of operations and the wait counts below are constants.
    auto clamp_stage = [&](int st) { return st < last ? st : last; };
    // i-th copy of stage `st` by this wavefront into the ring slot at LDS address `slot`
    auto dma_piece = [&](int st, uint32_t slot, int i) {
        size_t adv = is_scale[i] ? (size_t)(st >> 1) * 256 : (size_t)st * 2 * C::PB;
        lds_dma16(src[i] + adv, __builtin_amdgcn_readfirstlane(slot + dst_off[i]));
    };
    auto slot_addr = [&](int ring_slot) {
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds + ring_slot * C::STAGE));
    };
    // One vector load of A's stage `st` into ring set SET: pieces 0..NA_OPS-1.
    // 4-bit A: the loads are written as assembly, like the W copies, so that
    // the compiler keeps no count of them either -- its own count would ignore
    // the W copies queued in between and drain them early.  Their results are
    // first read after the hand-over wait of the previous stage, and every
    // destination register stays live until then.  8-bit A (two loads per
    // fragment) stays with compiler-tracked loads.
    auto a_piece = [&](auto setc, int st, int piece) {
        constexpr int SET = decltype(setc)::value;
        if (piece < TI * 2 * A_PER_FRAG) {
            int f = piece / A_PER_FRAG, half = piece % A_PER_FRAG, i = f >> 1, ksl = f & 1;
            const uint8_t *pg = a_ptr[i] + (size_t)(st * 2 + ksl) * PA + half * 1024;
            if (AK == RFQ_MX_FP4) {
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(areg4[SET][i][ksl]) : "v"(pg) : "memory");
            } else {
                uint4 v = *reinterpret_cast<const uint4 *>(pg);
                areg[SET][i][ksl][4 * half + 0] = (int)v.x; areg[SET][i][ksl][4 * half + 1] = (int)v.y;
                areg[SET][i][ksl][4 * half + 2] = (int)v.z; areg[SET][i][ksl][4 * half + 3] = (int)v.w;
            }
        } else {
            int i = piece - TI * 2 * A_PER_FRAG;
            const uint8_t *sp = as_ptr[i] + (size_t)(st >> 1) * 256;
            if (AK == RFQ_MX_FP4) asm volatile("global_load_dword %0, %1, off" : "=v"(ascl[SET][i]) : "v"(sp) : "memory");
            else ascl[SET][i] = *reinterpret_cast<const int *>(sp);
        }
    };
    auto a_frag = [&](auto setc, int i, int ksl) -> v8i {
        constexpr int SET = decltype(setc)::value;
        if (AK == RFQ_MX_FP4)
            return __builtin_shufflevector(areg4[SET][i][ksl], areg4[SET][i][ksl], 0, 1, 2, 3, -1, -1, -1, -1);
        return areg[SET][i][ksl];
    };

    v16f acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
#pragma unroll
    for (int set = 0; set < RING; set++)
#pragma unroll
        for (int i = 0; i < TI; i++) {
            ascl[set][i] = 0;
#pragma unroll
            for (int k2 = 0; k2 < 2; k2++) {
#pragma unroll
                for (int e = 0; e < 8; e++) areg[set][i][k2][e] = 0;
#pragma unroll
                for (int e = 0; e < 4; e++) areg4[set][i][k2][e] = 0;
            }
        }

    // ---- prologue: W(0), A(0), W(1), A(1), ..., A(RING-2), W(RING-1); then stage 0 awaited
    auto prologue_stage = [&](auto setc) {
        constexpr int SET = decltype(setc)::value;
        const int st = clamp_stage(SET);
        const uint32_t slot = slot_addr(SET);
#pragma unroll
        for (int i = 0; i < C::ND; i++) dma_piece(st, slot, i);
        if (SET < RING - 1) {
#pragma unroll
            for (int pc = 0; pc < NA_OPS; pc++) a_piece(setc, st, pc);
        }
        asm volatile("" ::: "memory");
    };
    prologue_stage(IC<0>{});
    prologue_stage(IC<1>{});
    if (RING > 2) prologue_stage(IC<2 % RING>{});
    if (RING > 3) prologue_stage(IC<3 % RING>{});
    if (RING > 4) prologue_stage(IC<4 % RING>{});
    if (RING > 5) prologue_stage(IC<5 % RING>{});
    if (RING > 6) prologue_stage(IC<6 % RING>{});
    if (RING > 7) prologue_stage(IC<7 % RING>{});
    static_assert(RING >= 3 && RING <= 8, "ring depth");
    wait_vmcnt<PROLOGUE_VMCNT>();
    barrier_no_drain();

    // W fragments are double-buffered by hand (k-step 0 / k-step 1), W scales
    // by stage parity.
    v8i fb0[TJ], fb1[TJ];
    int sb[2][TJ];
    auto read_b = [&](const uint8_t *base, int ksl, int j, v8i (&fb)[TJ]) {
        fb[j] = read_frag<BK_>(base + (j * 2 + ksl) * C::PB, lane);
    };
    // A stage uses scale bytes 2*(st&1) and 2*(st&1)+1 of its dwords: shift
    // them down so the instruction's byte selectors are constants.
    auto read_bscale = [&](const uint8_t *base, int st, int j, int (&xb)[TJ]) {
        xb[j] = (int)(*reinterpret_cast<const uint32_t *>(base + C::B_STAGE + (j * 64 + lane) * 4) >> (16 * (st & 1)));
    };
#pragma unroll
    for (int j = 0; j < TJ; j++) {
        read_b(lds, 0, j, fb0);
        read_bscale(lds, 0, j, sb[0]);
    }

    // One stage with ring set SET = st % RING, PAR = st % 2.  It contains no
    // branch; everything that is not a matrix instruction is slotted between
    // two of them and sched_barrier pins that order.
    auto stage = [&](auto setc, auto parc, int st) {
        constexpr int SET = decltype(setc)::value, PAR = decltype(parc)::value;
        using AHEAD = IC<(SET + RING - 1) % RING>;
        const uint8_t *base = lds + SET * C::STAGE;
        const uint8_t *nbase = lds + ((SET + 1) % RING) * C::STAGE;
        const int st_a = clamp_stage(st + RING - 1), st_w = clamp_stage(st + RING);
        int sa[TI];
#pragma unroll
        for (int i = 0; i < TI; i++) sa[i] = (int)((uint32_t)ascl[SET][i] >> (16 * (st & 1)));

        // k-step 0; its shadow: W fragments of k-step 1, A loads RING-1 stages ahead, then the hand-over.
#pragma unroll
        for (int q = 0; q < NMMA; q++) {
            acc[q / TJ][q % TJ] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                a_frag(setc, q / TJ, 0), fb0[q % TJ], acc[q / TJ][q % TJ], Cbsz<AK>::V, Cbsz<BK_>::V, 0, sa[q / TJ], 0,
                sb[PAR][q % TJ]);
            __builtin_amdgcn_sched_barrier(0);
            if (q < TJ) read_b(base, 1, q, fb1);
#pragma unroll
            for (int pp = 0; pp < A_PPS; pp++)
                if (q * A_PPS + pp < NA_OPS) a_piece(AHEAD{}, st_a, q * A_PPS + pp);
            if (q == NMMA - 2) {
                // Hand-over: this wavefront's last reads of the slot are complete
                // (lgkmcnt), stage st+1 has landed in LDS and in registers
                // (vmcnt: only what was issued after it may still be in
                // flight), everyone agrees (barrier).
                __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0) only
                wait_vmcnt<HANDOVER_VMCNT>();
                barrier_no_drain();
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // k-step 1; its shadow: the slot's refill, W fragments and scales of the next stage.
        const uint32_t slot = slot_addr(SET);
#pragma unroll
        for (int q = 0; q < NMMA; q++) {
            acc[q / TJ][q % TJ] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                a_frag(setc, q / TJ, 1), fb1[q % TJ], acc[q / TJ][q % TJ], Cbsz<AK>::V, Cbsz<BK_>::V, 1, sa[q / TJ], 1,
                sb[PAR][q % TJ]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pp = 0; pp < D_PPS; pp++)
                if (q * D_PPS + pp < C::ND) dma_piece(st_w, slot, q * D_PPS + pp);
            if (q < TJ) {
                read_b(nbase, 0, q, fb0);
                read_bscale(nbase, st + 1, q, sb[PAR ^ 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    RFQ_MX_STAMP(1);
    // RING is even here or the parity is carried by a second copy of the body:
    // unroll by lcm(RING, 2) so that ring set and stage parity are constants.
    constexpr int UNROLL = (RING % 2 == 0) ? RING : 2 * RING;
    for (int st = 0; st < nstages; st += UNROLL) {
        stage(IC<0 % RING>{}, IC<0>{}, st);
        if (st + 1 < nstages) stage(IC<1 % RING>{}, IC<1>{}, st + 1);
        if (st + 2 < nstages) stage(IC<2 % RING>{}, IC<0>{}, st + 2);
        if (UNROLL > 3 && st + 3 < nstages) stage(IC<3 % RING>{}, IC<1>{}, st + 3);
        if (UNROLL > 4 && st + 4 < nstages) stage(IC<4 % RING>{}, IC<0>{}, st + 4);
        if (UNROLL > 5 && st + 5 < nstages) stage(IC<5 % RING>{}, IC<1>{}, st + 5);
        if (UNROLL > 6 && st + 6 < nstages) stage(IC<6 % RING>{}, IC<0>{}, st + 6);
        if (UNROLL > 7 && st + 7 < nstages) stage(IC<7 % RING>{}, IC<1>{}, st + 7);
        if (UNROLL > 8 && st + 8 < nstages) stage(IC<8 % RING>{}, IC<0>{}, st + 8);
        if (UNROLL > 9 && st + 9 < nstages) stage(IC<9 % RING>{}, IC<1>{}, st + 9);
    }
    static_assert(UNROLL <= 10, "unroll");
    // The trailing prefetches still write LDS slots and registers: drain them
    // before either is reused.
    wait_vmcnt<0>();
    RFQ_MX_STAMP(2);

    // Epilogue.  Accumulator register r of tile (i, j) is row
    // 8*(r/4) + 4*(lane/32) + r%4, column lane%32 of the tile: a lane owns
    // single elements scattered over rows.  Interior wavefront blocks go through
    // LDS (the ring is free now), one 32-row band at a time, and leave as whole
    // rows in 16-byte stores; ragged blocks fall back to element stores.
    constexpr int ES = OUT_BF16 ? 2 : 4;
    constexpr int ROW_BYTES = TJ * 32 * ES;                 // one band row of this wavefront
    constexpr int ROW_STRIDE = ROW_BYTES + 16;              // +4 dwords: the two half-waves (rows R, R+4) miss each other's banks
    constexpr int CPR = ROW_BYTES / 16;                     // 16-byte chunks per row
    const int m_base = tmi * C::BM + wave * TI * 32, n_base = tn * C::BN;
    const bool interior = m_base + TI * 32 <= M && n_base + TJ * 32 <= N && ((size_t)N * ES) % 16 == 0 &&
                          (reinterpret_cast<uintptr_t>(outp) & 15u) == 0;
    barrier_no_drain(); // every wavefront is past its last fragment read and its last copy
    uint8_t *stagebuf = lds + (size_t)wave * 32 * ROW_STRIDE;
    if (interior) {
#pragma unroll
        for (int i = 0; i < TI; i++) {
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int row = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    uint8_t *dst = stagebuf + row * ROW_STRIDE + (32 * j + (lane & 31)) * ES;
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
                    uint4 v = *reinterpret_cast<const uint4 *>(stagebuf + row * ROW_STRIDE + col16 * 16);
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
                    if (m < M && n < N) {
                        if (OUT_BF16)
                            reinterpret_cast<uint16_t *>(outp)[(size_t)m * N + n] = f32_to_bf16(acc[i][j][r]);
                        else
                            reinterpret_cast<float *>(outp)[(size_t)m * N + n] = acc[i][j][r];
                    }
                }
            }
    }
    RFQ_MX_STAMP(3);
}

template <int AK, int BK_, bool OUT_BF16, int TJ, int RING>
int launch_gemm_cfg(const uint8_t *a, const uint8_t *b, void *out, int m, int n, int k, hipStream_t s)
{
    using C = GemmCfg<BK_, TJ, RING>;
    MxLayout LA = mx_layout(AK, m, k), LB = mx_layout(BK_, n, k);
    constexpr size_t RINGB = (size_t)RING * C::STAGE;
    constexpr size_t STAGING = (size_t)4 * 32 * (TJ * 32 * (OUT_BF16 ? 2 : 4) + 16);
    constexpr size_t LDS = RINGB > STAGING ? RINGB : STAGING;
    static_assert(LDS <= 160 * 1024, "LDS budget");
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mx_kernel<AK, BK_, OUT_BF16, TJ, RING>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
    });
    if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemm_mx_kernel)");
    int tiles = ((m + C::BM - 1) / C::BM) * ((n + C::BN - 1) / C::BN);
    int per = (tiles + 7) / 8;
    hipLaunchKernelGGL((gemm_mx_kernel<AK, BK_, OUT_BF16, TJ, RING>), dim3(per * 8), dim3(256), LDS, s, a, b, out, m,
                       n, LA, LB);
    RFQ_LAUNCH_CHECK("gemm_mx_kernel");
    return RFQ_OK;
}

// Output tiles are 256 rows by 224 columns for 4-bit operands (28672 = 128 * 224
// fills 256 CUs exactly four times at M = 2048; 256-wide tiles would run 3.5
// rounds and do not fit the register file next to the prefetch ring).
// 8-bit operands need twice the registers per fragment: 128-column tiles.
template <int AK, int BK_, bool OUT_BF16>
int run_gemm(const uint8_t *a, const uint8_t *b, void *out, int m, int n, int k, hipStream_t s)
{
    if constexpr (AK == RFQ_MX_FP8 || BK_ == RFQ_MX_FP8)
        return launch_gemm_cfg<AK, BK_, OUT_BF16, 4, 4>(a, b, out, m, n, k, s);
    else
        return launch_gemm_cfg<AK, BK_, OUT_BF16, 7, RFQ_MX_RING>(a, b, out, m, n, k, s);
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
