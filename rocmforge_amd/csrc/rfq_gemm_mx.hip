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

// Ring depth (W slots in LDS = A fragment sets in registers) with 4-bit A
// fragments; 8-bit A fragments take twice the registers and half the depth.
constexpr int RFQ_MX_RING = 8;

namespace rfq {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// k-steps (64 elements) of a prepared matrix are padded with zero pages to a
// multiple of MX_KS_PAD, so that the GEMM's k loop is a whole number of trips
// through its unrolled prefetch ring and needs no remainder code.
constexpr int MX_KS_PAD = 16;

struct MxLayout {
    int rows, k, rt, ks, ks4, ks_real; // ks: padded k-steps per row tile; ks_real: k / 64
    size_t page_bytes, data_bytes, scale_bytes;
    __host__ __device__ size_t total() const { return data_bytes + scale_bytes + 16; } // +16: status words
};

__host__ __device__ inline MxLayout mx_layout(int kind, int rows, int k)
{
    MxLayout L;
    L.rows = rows; L.k = k;
    L.rt = (rows + 31) / 32;
    L.ks_real = k / 64;
    L.ks = (L.ks_real + MX_KS_PAD - 1) / MX_KS_PAD * MX_KS_PAD;
    L.ks4 = L.ks / 4;
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
    const v4i q = ld<v4i>(blk + 1);                   // one 16-byte load (any alignment) instead of 16 byte loads
#pragma unroll
    for (int j = 0; j < 16; j++) {
        uint32_t b = ((uint32_t)q[j >> 2] >> (8 * (j & 3))) & 255u;
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

// The scale bytes of k-steps 4j .. 4j+3 of a row tile are the four bytes of one dword per lane.  A workgroup's four
// wavefronts re-encode exactly those four pages (the padded k-step count is a multiple of 4 and so is a
// workgroup's first page), so the bytes meet in LDS and leave as one coalesced dword store per lane instead of
// four byte stores from four wavefronts into the same dword.
__device__ __forceinline__ void store_scales(uint8_t *prep, const MxLayout &L, int rt, int ks, int lane, int E)
{
    __shared__ uint8_t sc[4][64];
    sc[ks & 3][lane] = (uint8_t)E;
    __syncthreads();
    if ((ks & 3) == 0) {
        const uint32_t w = (uint32_t)sc[0][lane] | ((uint32_t)sc[1][lane] << 8) | ((uint32_t)sc[2][lane] << 16) | ((uint32_t)sc[3][lane] << 24);
        *reinterpret_cast<uint32_t *>(prep + L.data_bytes + ((size_t)rt * L.ks4 + (ks >> 2)) * 256 + (size_t)lane * 4) = w;
    }
}

template <int FMT, int KIND>
__global__ void __launch_bounds__(256)
mx_prepare_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ prep, MxLayout L)
{
    constexpr int BB = Fmt<FMT>::BB;
    size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
    int lane = (int)(g & 63);                                  // (the grid is exactly rt * ks pages: no thread is past the end)
    size_t page = g >> 6;
    int rt = (int)(page / L.ks), ks = (int)(page % L.ks);
    int row = rt * 32 + (lane & 31), kb = ks * 2 + (lane >> 5);
    uint32_t *status = reinterpret_cast<uint32_t *>(prep + L.data_bytes + L.scale_bytes);

    float v[32];
    if (row < L.rows && ks < L.ks_real) {
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
    store_scales(prep, L, rt, ks, lane, E);
}

// MXFP4 -> 4-bit operand with integer arithmetic only (the general kernel
// above goes through the 32 float values).  A raw code is sign | m with
// magnitude 2^p(m) times the block's 2^e, p = -1 (m = 0 with the sign set),
// 0, 0, 1, 1, 2, 2, 3 for m = 1..7, code 0 is 0.0
// (MxfpBlock::decode_e2m1, src/loader/mxfp.rs:234-244); the +-8 clamp caps
// the exponent e + p at 3.  The matrix core's E2M1 codes 1, 2, 4, 6 are 0.5,
// 1, 2, 4: with the largest exponent of the block on code 6 (scale byte =
// that exponent - 2) every other value is a code iff it is at most 3 octaves
// below.  Which exponents occur is found with nibble-parallel arithmetic on the
// four dwords, the code translation is two 8-entry byte tables (sign clear /
// set) looked up with v_perm_b32, four codes per instruction.
__global__ void __launch_bounds__(256)
mx_prepare_fp4_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ prep, MxLayout L)
{
    size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
    int lane = (int)(g & 63);                                  // (the grid is exactly rt * ks pages: no thread is past the end)
    size_t page = g >> 6;
    int rt = (int)(page / L.ks), ks = (int)(page % L.ks);
    int row = rt * 32 + (lane & 31), kb = ks * 2 + (lane >> 5);
    uint32_t *status = reinterpret_cast<uint32_t *>(prep + L.data_bytes + L.scale_bytes);

    int E = 127;
    uint32_t out[4] = {0u, 0u, 0u, 0u};
    if (row < L.rows && ks < L.ks_real) {
        const uint8_t *blk = raw + ((size_t)row * (L.k / 32) + kb) * 17;
        const int e = (int)(int8_t)blk[0];
        const v4i qi = ld<v4i>(blk + 1);
        const uint32_t q[4] = {(uint32_t)qi[0], (uint32_t)qi[1], (uint32_t)qi[2], (uint32_t)qi[3]};
        // bit 3 of a nibble of geN: that code has m >= N; cNN: m in that pair; neg0: m = 0 with the sign set
        uint32_t ge7 = 0, c56 = 0, c34 = 0, c12 = 0, neg0 = 0;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t y = q[d] & 0x77777777u;
            const uint32_t a1 = y + 0x77777777u, a3 = y + 0x55555555u, a5 = y + 0x33333333u, a7 = y + 0x11111111u;
            ge7 |= a7;
            c56 |= a5 & ~a7;
            c34 |= a3 & ~a5;
            c12 |= a1 & ~a3;
            neg0 |= ~a1 & q[d];
        }
        const uint32_t M8 = 0x88888888u;
        // bit p + 1 of `present`: an element with magnitude exponent p exists (2^-128 as the scale is 0.0: nothing does)
        uint32_t present = ((neg0 & M8) ? 1u : 0u) | ((c12 & M8) ? 2u : 0u) | ((c34 & M8) ? 4u : 0u) |
                           ((c56 & M8) ? 8u : 0u) | ((ge7 & M8) ? 16u : 0u);
        if (e == -128) present = 0;
        if (present != 0) {
            const int pmax = 30 - __builtin_clz(present), pmin = __builtin_ctz(present) - 1;
            const int cap = 3 - e;                                 // exponents above 3 are clamped to 3
            auto ex = [&](int p) { return e + (p < cap ? p : cap); };
            int Eu = ex(pmax) - 2;
            if (Eu < -127) Eu = -127;
            E = Eu + 127;
            if (ex(pmin) - Eu < -1) status[0] = 1u;               // more than the four codes span
            auto code = [&](int p) {                               // 0.5, 1, 2, 4 times the new scale
                int kx = ex(p) - Eu;
                kx = kx < -1 ? -1 : kx;
                return (uint32_t)(kx < 0 ? 1 : 2 * kx + 2);
            };
            const uint32_t gm1 = code(-1), g0 = code(0), g1 = code(1), g2 = code(2), g3 = code(3);
            const uint32_t t0_lo = (g0 << 8) | (g0 << 16) | (g1 << 24);          // m = 0 (with the sign clear: 0.0), 1, 2, 3
            const uint32_t t0_hi = g1 | (g2 << 8) | (g2 << 16) | (g3 << 24);     // m = 4..7
            const uint32_t t1_lo = t0_lo | 0x08080808u | gm1, t1_hi = t0_hi | 0x08080808u;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                // byte j of the raw dword: high nibble = element 2j, low nibble = element 2j+1;
                // byte j of the operand dword: low nibble = element 2j, high nibble = element 2j+1
                uint32_t r[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const uint32_t c = (h == 0 ? q[d] >> 4 : q[d]) & 0x0F0F0F0Fu;
                    const uint32_t sel = c & 0x07070707u, s8 = c & 0x08080808u;
                    const uint32_t plus = __builtin_amdgcn_perm(t0_hi, t0_lo, sel), minus = __builtin_amdgcn_perm(t1_hi, t1_lo, sel);
                    const uint32_t neg = (s8 << 1) - (s8 >> 3);   // 0x0F in the bytes whose sign bit is set
                    r[h] = (minus & neg) | (plus & ~neg);
                }
                out[d] = r[0] | (r[1] << 4);
            }
        }
    }
    uint4 *dst = reinterpret_cast<uint4 *>(prep + page * 1024 + (size_t)lane * 16);
    *dst = make_uint4(out[0], out[1], out[2], out[3]);
    store_scales(prep, L, rt, ks, lane, E);
}

// The status words (every page and every scale byte is written by the re-encoding kernels).
__global__ void mx_init_kernel(uint8_t *prep, MxLayout L)
{
    if (threadIdx.x < 4) reinterpret_cast<uint32_t *>(prep + L.data_bytes + L.scale_bytes)[threadIdx.x] = 0;
}

// ---- GEMM ---------------------------------------------------------------------
//
// k advances 128 per stage (two instruction k-steps).  One barrier per stage,
// in the middle of it: after it every wavefront is done with the current W
// slot and every wavefront's share of the next stage has landed.

template <int KIND> struct Pg { static constexpr int BYTES = KIND == RFQ_MX_FP4 ? 1024 : 2048; };
template <int KIND> struct Cbsz { static constexpr int V = KIND == RFQ_MX_FP4 ? 4 : 0; };

// An operand fragment as it is kept in registers: a 4-bit fragment is 4
// dwords.  The instruction names 8 registers whatever the format and ignores
// the upper 4 for 4-bit data; widen() leaves them undefined, so they cost no
// registers.
template <int KIND> struct Frag { using type = v8i; };
template <> struct Frag<RFQ_MX_FP4> { using type = v4i; };
__device__ __forceinline__ v8i widen(v8i f) { return f; }
__device__ __forceinline__ v8i widen(v4i f) { return __builtin_shufflevector(f, f, 0, 1, 2, 3, -1, -1, -1, -1); }

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding:
// vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]).
template <int N> __device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// The W copies are direct global -> LDS loads, 64 lanes x 16 bytes: lane l's
// 16 bytes land at M0 + 16*l.  They (and the 4-bit A loads) are written as
// assembly on purpose: the compiler then keeps no book on them, so it does not
// drain them (vmcnt(0)) in front of every LDS read or barrier; the kernel
// waits for exactly the stage it needs with wait_vmcnt.  Loads the compiler
// cannot see only make its own waits longer, never shorter: the counter
// retires in order.

// Tells the compiler that a pointer is the same in every lane (it then lives
// in scalar registers).
__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p)
{
    uint64_t v = reinterpret_cast<uint64_t>(p);
    uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return reinterpret_cast<const uint8_t *>(((uint64_t)hi << 32) | lo);
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
//
// Workgroups are persistent: one per CU, each walking its list of output
// tiles.  The operand stream does not stop at a tile boundary -- while a
// wavefront converts and stores the finished tile, the first RING stages of
// its next tile are already in flight or landed, and the stores drain behind
// the next tile's matrix work.
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
    static constexpr int RING_BYTES = RING * STAGE;
    // The epilogue stages RB full-width rows of a wavefront's 32-row band at a
    // time: as many as fit behind the ring in 160 KiB of LDS.
    template <bool OUT_BF16> static constexpr int staging_row_stride() { return TJ * 32 * (OUT_BF16 ? 2 : 4) + 16; }
    template <bool OUT_BF16> static constexpr int staging_rows()
    {
        int rb = 32;
        while (rb > 8 && RING_BYTES + 4 * rb * staging_row_stride<OUT_BF16>() > 160 * 1024) rb /= 2;
        return rb;
    }
    template <bool OUT_BF16> static constexpr int lds_bytes()
    {
        return RING_BYTES + 4 * staging_rows<OUT_BF16>() * staging_row_stride<OUT_BF16>();
    }
};

template <int N> struct IC { static constexpr int value = N; };

template <int AK, int BK_, bool OUT_BF16, int TJ, int RING>
__global__ void __launch_bounds__(256)
gemm_mx_kernel(const uint8_t *__restrict__ ap, const uint8_t *__restrict__ bp, void *__restrict__ outp, int M, int N,
               MxLayout LA, MxLayout LB)
{
    using C = GemmCfg<BK_, TJ, RING>;
    constexpr int TI = C::TI, PA = Pg<AK>::BYTES;
    constexpr int NMMA = TI * TJ;
    constexpr int A_PER_FRAG = AK == RFQ_MX_FP4 ? 1 : 2;
    constexpr int NA_OPS = TI * 2 * A_PER_FRAG + TI;          // vector loads per stage for A and its scales
    constexpr int A_PPS = (NA_OPS + NMMA - 3) / (NMMA - 2);   // A loads per slot: all issued before the hand-over at slot NMMA-2
    constexpr int D_PPS = (C::ND + NMMA - 1) / NMMA;          // W copies per slot
    // Loads a wavefront issues after the last one of stage s+1 and before the
    // hand-over of stage s (see the schedule below).  Loads complete in order
    // among themselves, so "at most this many operations outstanding" proves
    // that stage s+1 has arrived; stores in flight (from a tile's epilogue)
    // can only make the wait longer, never too short.
    constexpr int NA_CNT = NA_OPS, ND_CNT = C::ND;
    // (the counter has 6 bits; a smaller number only waits for more than necessary)
    constexpr int HANDOVER_EXACT = (RING - 2) * (NA_CNT + ND_CNT);
    constexpr int PROLOGUE_EXACT = (RING - 1) * ND_CNT + (RING - 2) * NA_CNT;
    constexpr int HANDOVER_VMCNT = HANDOVER_EXACT < 63 ? HANDOVER_EXACT : 63;
    constexpr int PROLOGUE_VMCNT = PROLOGUE_EXACT < 63 ? PROLOGUE_EXACT : 63;
    static_assert(TJ + 1 <= NMMA, "not enough matrix instructions to hide the fragment reads");
    static_assert(RING >= 4 && RING <= 8 && RING % 2 == 0, "ring depth: even, so that stage parity is a constant");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63, lane_id = lane;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform, and the compiler may know it
    // XCD-aware tile lists: consecutive workgroup ids land on different XCDs
    // (round robin over 8).  XCD x owns the contiguous run of tiles
    // [x*per, (x+1)*per), ordered M-tile fastest, and its workgroups take them
    // G8 apart: at any time an XCD works on a few W tiles times all M tiles, so
    // each W tile is fetched into one L2 only and A is shared by neighbours.
    const int tiles_m = (M + C::BM - 1) / C::BM, tiles_n = (N + C::BN - 1) / C::BN;
    const int total = tiles_m * tiles_n;
    const int per = (total + 7) / 8;
    const int xcd = blockIdx.x & 7, G8 = gridDim.x >> 3;
    auto tile_valid = [&](int idx) { return idx < per && xcd * per + idx < total; };
    if (!tile_valid(blockIdx.x >> 3)) return; // uniform over the workgroup
    const uint8_t *b_scale = bp + LB.data_bytes;
    const int nstages = LA.ks / 2;
    // (a whole number of trips through the unrolled ring: the prepared layout pads k)

    // ---- operand addresses.  A load names a wavefront-uniform base (scalar
    // registers, fixed for a tile), a per-lane byte offset (one register per
    // stream, advanced by one add per stage) and an immediate.  Prefetches run
    // ahead of the arithmetic and cross into the next tile RING stages before
    // a tile ends, so two sets of bases exist: `pf`, in use by the prefetch
    // streams, and `nx`, the tile after that one.  The switch happens at a fixed
    // place of the last trip through the ring, by scalar selects: there is no
    // branch between stages.
    const uint32_t lane16 = lane * 16;
    v8i areg[RING][TI][2];   // 8-bit A fragments
    v4i areg4[RING][TI][2];  // 4-bit A fragments
    int ascl[RING][TI];

    // This wavefront's wave-copies of a W stage: copy i moves KiB j = wave + 4i
    // of the stage image (pages first, then 256 scale bytes per row tile).
    // Only the last copy of a wavefront can be a scale copy.
    static_assert(C::S_STAGE <= 4096, "a wavefront may own at most one scale copy");
    static_assert((4 * (C::ND - 2) + 3) * 1024 < C::B_STAGE, "only the last copy may hold scales");
    int dst_off[C::ND];
#pragma unroll
    for (int i = 0; i < C::ND; i++) {
        int j = wave + 4 * i;
        j = j < C::WL ? j : C::WL - 1;                   // pad: repeat the last copy (same bytes, same place)
        dst_off[i] = j * 1024;
    }
    const bool last_is_scale = dst_off[C::ND - 1] >= C::B_STAGE;
    const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)lds); // LDS address of the ring
    // Bases of tile `idx`; wl receives the per-lane offset of this wavefront's
    // last W copy: lane*16 for a page copy, or the scale copy's offset (4 row
    // tiles x 16 lanes x 16 bytes).
    auto tile_bases = [&](int idx, const uint8_t *(&ba)[TI], const uint8_t *(&bas)[TI], const uint8_t *(&bw)[C::ND],
                          uint32_t &wl) __attribute__((always_inline)) {
        // (the lane number goes through an opaque statement so that nothing
        // derived from it is hoisted out of the tile loop and kept in registers)
        int lane = lane_id;
        asm volatile("" : "+v"(lane));
        const int t = xcd * per + idx, tmi = t % tiles_m, rtB0 = (t / tiles_m) * TJ;
#pragma unroll
        for (int i = 0; i < TI; i++) {
            int rt = tmi * (C::WM * TI) + wave * TI + i;
            rt = rt < LA.rt ? rt : LA.rt - 1;
            ba[i] = uniform_ptr(ap + (size_t)rt * LA.ks * PA);
            bas[i] = uniform_ptr(ap + LA.data_bytes + (size_t)rt * LA.ks4 * 256);
        }
        wl = lane * 16;
#pragma unroll
        for (int i = 0; i < C::ND; i++) {
            const int j = dst_off[i] / 1024;
            int off = j * 1024, rtl = off / (2 * C::PB), within = off % (2 * C::PB);
            int rt = rtB0 + rtl;
            rt = rt < LB.rt ? rt : LB.rt - 1;
            const uint8_t *pages = bp + (size_t)rt * LB.ks * C::PB + within;
            if (i == C::ND - 1) {
                int q = j - C::B_STAGE / 1024;           // 1 KiB = 4 row tiles x 256 bytes
                int rs = rtB0 + q * 4 + (lane >> 4);
                rs = rs < LB.rt ? rs : LB.rt - 1;        // >= rtB0: the tile exists
                const uint32_t wsc = (uint32_t)(rs - rtB0) * (uint32_t)LB.ks4 * 256u + (lane & 15) * 16;
                wl = last_is_scale ? wsc : wl;
                bw[i] = uniform_ptr(last_is_scale ? b_scale + (size_t)rtB0 * LB.ks4 * 256 : pages);
            } else {
                bw[i] = uniform_ptr(pages);
            }
        }
    };
    const uint8_t *pf_a[TI], *pf_as[TI], *pf_w[C::ND], *nx_a[TI], *nx_as[TI], *nx_w[C::ND];
    uint32_t wl_nx = 0;
    // per-lane offsets of the next A pages, A scales, W pages and this
    // wavefront's last W copy to prefetch
    uint32_t voffA, voffAS, voffW, voffWL;
    // what a stage adds to voffWL: pages move 2 pages on, scale dwords cover two stages
    const uint32_t incWL_even = last_is_scale ? 0u : 2u * C::PB, incWL_odd = last_is_scale ? 256u : 2u * C::PB;

    // i-th copy of a W stage by this wavefront into ring slot SLOT.  The LDS
    // address goes into M0 right before the copy (nothing else in this kernel
    // uses M0).
    auto dma_piece = [&](auto slotc, int i) {
        constexpr int SLOT = decltype(slotc)::value;
        const uint32_t voff = i == C::ND - 1 ? voffWL : voffW;
        const uint8_t *base = pf_w[i];
        const int doff = dst_off[i] + (int)lds0;
        asm volatile("s_add_u32 m0, %2, %3\n\t"
                     "global_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(voff), "s"(base), "s"(doff), "n"(SLOT * C::STAGE)
                     : "memory", "scc");
    };
    // One vector load of an A stage into ring set SET: pieces 0..NA_OPS-1.
    // 4-bit A: the loads are written as assembly, like the W copies, so that
    // the compiler keeps no count of them either -- its own count would ignore
    // the W copies queued in between and drain them early.  Their results are
    // first read after the hand-over wait of the previous stage, and every
    // destination register stays live until then.  8-bit A (two loads per
    // fragment) stays with compiler-tracked loads.
    auto a_piece = [&](auto setc, int piece) {
        constexpr int SET = decltype(setc)::value;
        if (piece < TI * 2 * A_PER_FRAG) {
            const int f = piece / A_PER_FRAG, half = piece % A_PER_FRAG, i = f >> 1, ksl = f & 1;
            if (AK == RFQ_MX_FP4) {
                const uint8_t *base = pf_a[i];
                const uint32_t voff = voffA;
                if (ksl == 0)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(areg4[SET][i][0]) : "v"(voff), "s"(base) : "memory");
                else
                    asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(areg4[SET][i][1]) : "v"(voff), "s"(base) : "memory");
            } else {
                // (the bases were rebuilt from scalar integers: naming the global address space keeps these global
                // loads; as flat loads they would also count against the LDS counter)
                typedef int v4i_g __attribute__((ext_vector_type(4)));
                typedef const __attribute__((address_space(1))) v4i_g *GlobalV4;
                const v4i_g v = *reinterpret_cast<GlobalV4>(reinterpret_cast<uintptr_t>(pf_a[i] + voffA + ksl * PA + half * 1024));
                areg[SET][i][ksl][4 * half + 0] = v[0]; areg[SET][i][ksl][4 * half + 1] = v[1];
                areg[SET][i][ksl][4 * half + 2] = v[2]; areg[SET][i][ksl][4 * half + 3] = v[3];
            }
        } else {
            const int i = piece - TI * 2 * A_PER_FRAG;
            const uint8_t *base = pf_as[i];
            const uint32_t voff = voffAS;
            if (AK == RFQ_MX_FP4) asm volatile("global_load_dword %0, %1, %2" : "=v"(ascl[SET][i]) : "v"(voff), "s"(base) : "memory");
            else {
                typedef const __attribute__((address_space(1))) int *GlobalI;
                ascl[SET][i] = *reinterpret_cast<GlobalI>(reinterpret_cast<uintptr_t>(base + voff));
            }
        }
    };
    auto a_frag = [&](auto setc, int i, int ksl) -> v8i {
        constexpr int SET = decltype(setc)::value;
        if (AK == RFQ_MX_FP4)
            return __builtin_shufflevector(areg4[SET][i][ksl], areg4[SET][i][ksl], 0, 1, 2, 3, -1, -1, -1, -1);
        return areg[SET][i][ksl];
    };

    v16f acc[TI][TJ];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    };
    zero_acc();
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
    const int idx0 = blockIdx.x >> 3;
    {
        uint32_t wl0;
        tile_bases(idx0, pf_a, pf_as, pf_w, wl0);
        voffA = lane16; voffAS = lane * 4; voffW = lane16; voffWL = wl0;
    }
    // offsets move on after every stage; scale dwords cover two stages
    auto step_a = [&](int s) { voffA += 2 * PA; if (s & 1) voffAS += 256; };
    auto step_w = [&](int s) { voffW += 2 * C::PB; voffWL += (s & 1) ? incWL_odd : incWL_even; };
    auto prologue_stage = [&](auto setc) {
        constexpr int SET = decltype(setc)::value;
#pragma unroll
        for (int i = 0; i < C::ND; i++) dma_piece(setc, i);
        step_w(SET);
        if (SET < RING - 1) {
#pragma unroll
            for (int pc = 0; pc < NA_OPS; pc++) a_piece(setc, pc);
            step_a(SET);
        }
        asm volatile("" ::: "memory");
    };
    prologue_stage(IC<0>{});
    prologue_stage(IC<1>{});
    prologue_stage(IC<2>{});
    prologue_stage(IC<3>{});
    if (RING > 4) prologue_stage(IC<4 % RING>{});
    if (RING > 5) prologue_stage(IC<5 % RING>{});
    if (RING > 6) prologue_stage(IC<6 % RING>{});
    if (RING > 7) prologue_stage(IC<7 % RING>{});
    wait_vmcnt<PROLOGUE_VMCNT>();
    barrier_no_drain();

    // W fragments are double-buffered by hand (k-step 0 / k-step 1), W scales
    // by stage parity.  LDS reads take a 16-bit immediate offset: one base
    // register per 64 KiB window of the ring.
    using WFrag = typename Frag<BK_>::type;
    WFrag fb0[TJ], fb1[TJ];
    int sb[2][TJ];
    typedef const __attribute__((address_space(3))) uint8_t *lds_u8_ptr;
    typedef const __attribute__((address_space(3))) v4i *lds_v4i_ptr;
    typedef const __attribute__((address_space(3))) int *lds_i32_ptr;
    lds_u8_ptr wf0 = (lds_u8_ptr)lds + lane16, wf1 = wf0 + 65536, wf2 = wf0 + 2 * 65536; // fragment reads: lane*16 + immediate
    lds_u8_ptr ws0 = (lds_u8_ptr)lds + lane * 4, ws1 = ws0 + 65536, ws2 = ws0 + 2 * 65536; // scale reads: lane*4 + immediate
    // keep the windows apart: no re-folding into one base plus a large constant
    asm volatile("" : "+v"(wf1), "+v"(wf2), "+v"(ws1), "+v"(ws2));
    static_assert(C::RING_BYTES <= 3 * 65536, "LDS windows");
    auto read_b = [&](int slot, int ksl, int j, WFrag (&fb)[TJ]) {
        const int off = slot * C::STAGE + (j * 2 + ksl) * C::PB;
        lds_u8_ptr w = (off >> 16) == 0 ? wf0 : (off >> 16) == 1 ? wf1 : wf2;
        v4i lo = *reinterpret_cast<lds_v4i_ptr>(w + (off & 65535));
        fb[j][0] = lo[0]; fb[j][1] = lo[1]; fb[j][2] = lo[2]; fb[j][3] = lo[3];
        if constexpr (BK_ != RFQ_MX_FP4) {
            const int off2 = off + 1024;
            lds_u8_ptr w2 = (off2 >> 16) == 0 ? wf0 : (off2 >> 16) == 1 ? wf1 : wf2;
            v4i hi = *reinterpret_cast<lds_v4i_ptr>(w2 + (off2 & 65535));
            fb[j][4] = hi[0]; fb[j][5] = hi[1]; fb[j][6] = hi[2]; fb[j][7] = hi[3];
        }
    };
    // Scale dword of lane l for row tile j sits at (j*64 + l)*4 of the scale part.
    auto read_bscale = [&](int slot, int j, int (&xb)[TJ]) {
        const int off = slot * C::STAGE + C::B_STAGE + j * 256;
        lds_u8_ptr w = (off >> 16) == 0 ? ws0 : (off >> 16) == 1 ? ws1 : ws2;
        xb[j] = *reinterpret_cast<lds_i32_ptr>(w + (off & 65535));
    };
#pragma unroll
    for (int j = 0; j < TJ; j++) {
        read_b(0, 0, j, fb0);
        read_bscale(0, j, sb[0]);
    }

    // One stage with ring set SET (a constant: the body is instantiated RING
    // times); `st` is the stage's number within its tile, st % RING == SET, and
    // because RING is even SET also gives the stage's parity: a scale dword
    // holds the bytes of two stages, the instruction's byte selectors are
    // 2*(st&1) + k-step.  The body contains no branch; everything that is not a
    // matrix instruction is slotted between two of them and sched_barrier pins
    // that order.
    auto stage = [&](auto setc, int st) {
        constexpr int SET = decltype(setc)::value, PAR = SET & 1;
        using AHEAD = IC<(SET + RING - 1) % RING>;
        // SET 0 of the last trip: the prefetch streams move on to the next tile
        const bool cross = SET == 0 && st == nstages - RING;

        // k-step 0; its shadow: W fragments of k-step 1, A loads RING-1 stages ahead, then the hand-over.
#pragma unroll
        for (int q = 0; q < NMMA; q++) {
            acc[q / TJ][q % TJ] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                a_frag(setc, q / TJ, 0), widen(fb0[q % TJ]), acc[q / TJ][q % TJ], Cbsz<AK>::V, Cbsz<BK_>::V,
                2 * PAR, ascl[SET][q / TJ], 2 * PAR, sb[PAR][q % TJ]);
            __builtin_amdgcn_sched_barrier(0);
            if (q < TJ) read_b(SET, 1, q, fb1);
#pragma unroll
            for (int pp = 0; pp < A_PPS; pp++)
                if (q * A_PPS + pp < NA_OPS) a_piece(AHEAD{}, q * A_PPS + pp);
            if (q == NMMA - 2) {
                // the A stream moves one stage on (slot st + RING - 1 has been issued)
                if (SET == 0) {
                    voffA = cross ? lane16 : voffA + 2 * PA;
                    voffAS = cross ? lane16 >> 2 : voffAS + (((SET + RING - 1) & 1) ? 256 : 0);
#pragma unroll
                    for (int i = 0; i < TI; i++) {
                        pf_a[i] = cross ? nx_a[i] : pf_a[i];
                        pf_as[i] = cross ? nx_as[i] : pf_as[i];
                    }
                } else {
                    step_a(SET + RING - 1);
                }
                // Hand-over: this wavefront's last reads of the slot are complete
                // (lgkmcnt), the next stage's data has landed in LDS and in
                // registers (vmcnt), everyone agrees (barrier).
                __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0) only
                wait_vmcnt<HANDOVER_VMCNT>();
                barrier_no_drain();
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // k-step 1; its shadow: the slot's refill, W fragments and scales of the next stage.
        if (SET == 0) {
            voffW = cross ? lane16 : voffW;
            voffWL = cross ? wl_nx : voffWL;
#pragma unroll
            for (int i = 0; i < C::ND; i++) pf_w[i] = cross ? nx_w[i] : pf_w[i];
        }
#pragma unroll
        for (int q = 0; q < NMMA; q++) {
            acc[q / TJ][q % TJ] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                a_frag(setc, q / TJ, 1), widen(fb1[q % TJ]), acc[q / TJ][q % TJ], Cbsz<AK>::V, Cbsz<BK_>::V,
                2 * PAR + 1, ascl[SET][q / TJ], 2 * PAR + 1, sb[PAR][q % TJ]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pp = 0; pp < D_PPS; pp++)
                if (q * D_PPS + pp < C::ND) dma_piece(setc, q * D_PPS + pp);
            if (q < TJ) {
                read_b((SET + 1) % RING, 0, q, fb0);
                read_bscale((SET + 1) % RING, q, sb[PAR ^ 1]);
            }
            if (q == NMMA - 1) step_w(SET);              // slot st + RING has been issued; RING is even
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Epilogue of one tile.  Accumulator register r of tile (i, j) is row
    // 8*(r/4) + 4*(lane/32) + r%4, column lane%32 of the tile: a lane owns
    // single elements scattered over rows.  A tile inside the matrix leaves straight
    // from the registers (32 lanes = one aligned 64- or 128-byte piece of a row per
    // store).  Staged through LDS into 16-byte row stores the launch measured the
    // same once the part's clock had settled (171.6 against 171.2 us at 2048 x 8192
    // x 28672) and 1-2 % longer over its first 240 launches: the stores are not what
    // the epilogue waits for, and this form needs no LDS.  A tile that crosses the
    // matrix edge goes, RB rows of a 32-row band at a time, through this wavefront's
    // LDS staging area (behind the ring) into a bounds-checked element loop.  LDS
    // operations of one wavefront execute in order, so no barrier is needed around
    // its private staging area.
    constexpr int ES = OUT_BF16 ? 2 : 4;
    constexpr int RB = C::template staging_rows<OUT_BF16>();
    constexpr int ROW_STRIDE = C::template staging_row_stride<OUT_BF16>(); // +4 dwords: the two half-waves (rows R, R+4) miss each other's banks
    auto epilogue = [&](int tile_idx) {
        // The lane number goes through an opaque statement: everything derived
        // from it is then computed here, where registers are free, instead of
        // being hoisted out of the tile loop and kept alive across the k loop.
        int lane = lane_id;
        asm volatile("" : "+v"(lane));
        const int t = xcd * per + tile_idx, tn = t / tiles_m, tmi = t % tiles_m;
        const int m_base = tmi * C::BM + wave * TI * 32, n_base = tn * C::BN;
        const bool interior = m_base + TI * 32 <= M && n_base + TJ * 32 <= N && ((size_t)N * ES) % 16 == 0 &&
                              (reinterpret_cast<uintptr_t>(outp) & 15u) == 0;
        typedef __attribute__((address_space(3))) uint8_t *lds_w8_ptr;
        lds_w8_ptr stage3 = (lds_w8_ptr)lds + C::RING_BYTES + wave * RB * ROW_STRIDE;
        // this lane's accumulator elements: rows 4*(lane/32) + {0..3, 8..11, 16..19, 24..27}, column lane%32 of a tile
        lds_w8_ptr wr = stage3 + 4 * (lane >> 5) * ROW_STRIDE + (lane & 31) * ES;
        if (interior) {
            // Straight from the accumulators: a register's lanes 0..31 are 32 consecutive columns of one row (64 bytes
            // of bf16, 128 of f32) and lanes 32..63 the row four below, so a store instruction writes two whole
            // aligned segments; the row is a scalar base, the lane a 32-bit offset, the tile column an immediate.
            uint8_t *tile_out = reinterpret_cast<uint8_t *>(outp) + ((size_t)m_base * N + n_base) * ES;
            const uint32_t voff = (uint32_t)(((lane >> 5) * 4 * (size_t)N + (lane & 31)) * ES);
            const size_t row_bytes = (size_t)N * ES;
            // (the bases are rebuilt from scalar integers: naming the global address space keeps these global stores)
            typedef __attribute__((address_space(1))) uint16_t *GlobalU16;
            typedef __attribute__((address_space(1))) float *GlobalF32;
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    uint8_t *row0 = const_cast<uint8_t *>(uniform_ptr(tile_out + (size_t)(32 * i + 8 * (r >> 2) + (r & 3)) * row_bytes));
                    uint8_t *row1 = const_cast<uint8_t *>(uniform_ptr(row0 + row_bytes));
#pragma unroll
                    for (int j = 0; j < TJ; j++) {
                        if (OUT_BF16) {
                            f32x2_t v = {acc[i][j][r], acc[i][j][r + 1]};
                            bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
                            uint32_t u;
                            __builtin_memcpy(&u, &b, 4);
                            __builtin_nontemporal_store((uint16_t)u, reinterpret_cast<GlobalU16>(reinterpret_cast<uintptr_t>(row0 + voff + 32 * j * ES)));
                            __builtin_nontemporal_store((uint16_t)(u >> 16), reinterpret_cast<GlobalU16>(reinterpret_cast<uintptr_t>(row1 + voff + 32 * j * ES)));
                        } else {
                            __builtin_nontemporal_store(acc[i][j][r], reinterpret_cast<GlobalF32>(reinterpret_cast<uintptr_t>(row0 + voff + 32 * j * ES)));
                            __builtin_nontemporal_store(acc[i][j][r + 1], reinterpret_cast<GlobalF32>(reinterpret_cast<uintptr_t>(row1 + voff + 32 * j * ES)));
                        }
                    }
                }
            return;
        }
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int h = 0; h < 32 / RB; h++) {
                // registers r in [h*RB/2, (h+1)*RB/2) are rows [h*RB, (h+1)*RB) of the band
#pragma unroll
                for (int j = 0; j < TJ; j++)
#pragma unroll
                    for (int r = h * RB / 2; r < (h + 1) * RB / 2; r += 2) {
                        const int off = (8 * (r >> 2) + (r & 3) - h * RB) * ROW_STRIDE + 32 * j * ES; // r even: r + 1 is the next row
                        if (OUT_BF16) {
                            // one conversion instruction per pair (round to nearest even), one 16-bit write per half
                            f32x2_t v = {acc[i][j][r], acc[i][j][r + 1]};
                            bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
                            uint32_t u;
                            __builtin_memcpy(&u, &b, 4);
                            *reinterpret_cast<__attribute__((address_space(3))) uint16_t *>(wr + off) = (uint16_t)u;
                            *reinterpret_cast<__attribute__((address_space(3))) uint16_t *>(wr + off + ROW_STRIDE) = (uint16_t)(u >> 16);
                        } else {
                            *reinterpret_cast<__attribute__((address_space(3))) float *>(wr + off) = acc[i][j][r];
                            *reinterpret_cast<__attribute__((address_space(3))) float *>(wr + off + ROW_STRIDE) = acc[i][j][r + 1];
                        }
                    }
                const int m0 = m_base + 32 * i + h * RB;
                {
                    const uint8_t *stagebuf = lds + C::RING_BYTES + (size_t)wave * RB * ROW_STRIDE;
                    const int ncols = TJ * 32;
#pragma nounroll
                    for (int e = lane; e < RB * ncols; e += 64) {
                        int row = e / ncols, col = e % ncols;
                        if (m0 + row < M && n_base + col < N) {
                            const uint8_t *sp = stagebuf + row * ROW_STRIDE + col * ES;
                            size_t o = (size_t)(m0 + row) * N + n_base + col;
                            if (OUT_BF16) reinterpret_cast<uint16_t *>(outp)[o] = *reinterpret_cast<const uint16_t *>(sp);
                            else reinterpret_cast<float *>(outp)[o] = *reinterpret_cast<const float *>(sp);
                        }
                    }
                }
            }
    };

    for (int idx = idx0; tile_valid(idx); idx += G8) {
        // past the last tile the streams fetch the start of the last tile again
        // (into registers / LDS nobody reads): every stage issues the same
        // number of loads and the wait counts are constants
        tile_bases(tile_valid(idx + G8) ? idx + G8 : idx, nx_a, nx_as, nx_w, wl_nx);
        for (int st = 0; st < nstages; st += RING) {
            stage(IC<0>{}, st);
            stage(IC<1>{}, st + 1);
            stage(IC<2>{}, st + 2);
            stage(IC<3>{}, st + 3);
            if (RING > 4) stage(IC<4 % RING>{}, st + 4);
            if (RING > 5) stage(IC<5 % RING>{}, st + 5);
            if (RING > 6) stage(IC<6 % RING>{}, st + 6);
            if (RING > 7) stage(IC<7 % RING>{}, st + 7);
        }
        epilogue(idx);
        zero_acc();
    }
    // The trailing prefetches still write LDS slots and registers: drain them
    // before the wavefront ends.
    wait_vmcnt<0>();
}

template <int AK, int BK_, bool OUT_BF16, int TJ, int RING>
int launch_gemm_cfg(const uint8_t *a, const uint8_t *b, void *out, int m, int n, int k, hipStream_t s)
{
    using C = GemmCfg<BK_, TJ, RING>;
    MxLayout LA = mx_layout(AK, m, k), LB = mx_layout(BK_, n, k);
    constexpr size_t LDS = C::template lds_bytes<OUT_BF16>();
    static_assert(LDS <= 160 * 1024, "LDS budget");
    static_assert((MX_KS_PAD / 2) % RING == 0, "the k padding of the prepared layout must cover the ring");
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mx_kernel<AK, BK_, OUT_BF16, TJ, RING>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
    });
    if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemm_mx_kernel)");
    const int tiles = ((m + C::BM - 1) / C::BM) * ((n + C::BN - 1) / C::BN);
    const int per = (tiles + 7) / 8;                       // tiles per XCD
    int g8 = device_cu_count() / 8;                        // workgroups per XCD: one per CU
    if (g8 < 1) g8 = 1;
    if (g8 > per) g8 = per;
    hipLaunchKernelGGL((gemm_mx_kernel<AK, BK_, OUT_BF16, TJ, RING>), dim3(g8 * 8), dim3(256), LDS, s, a, b, out, m,
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
        return launch_gemm_cfg<AK, BK_, OUT_BF16, 4, (AK == RFQ_MX_FP4 ? RFQ_MX_RING : RFQ_MX_RING / 2)>(a, b, out, m, n, k, s);
    else
        return launch_gemm_cfg<AK, BK_, OUT_BF16, 7, RFQ_MX_RING>(a, b, out, m, n, k, s);
}

template <int FMT, int KIND>
int run_prepare(const uint8_t *raw, uint8_t *prep, const MxLayout &L, bool clear_status, hipStream_t s)
{
    size_t threads = (size_t)L.rt * L.ks * 64;                  // a multiple of 1024: ks is padded to a multiple of 16
    if (clear_status) {                                         // (an unchecked request never reads the status words)
        hipLaunchKernelGGL(mx_init_kernel, dim3(1), dim3(64), 0, s, prep, L);
        RFQ_LAUNCH_CHECK("mx_init_kernel");
    }
    if (FMT == RFQ_MXFP4 && KIND == RFQ_MX_FP4)
        hipLaunchKernelGGL(mx_prepare_fp4_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, raw, prep, L);
    else
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
    const bool unchecked = kind_req == RFQ_MX_FP4_UNCHECKED;
    if (unchecked) kind_req = RFQ_MX_FP4;
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
        int rc = run_prepare<RFQ_MXFP4, RFQ_MX_FP4>(d_raw, prep, L, !unchecked, s);
        if (rc != RFQ_OK) return rc;
        if (unchecked) {                                         // the caller vouches for the data: no read-back, no sync
            if (kind_out) *kind_out = RFQ_MX_FP4;
            return RFQ_OK;
        }
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
    int rc = is4 ? run_prepare<RFQ_MXFP4, RFQ_MX_FP8>(d_raw, prep, L, true, s)
                 : run_prepare<RFQ_MXFP6_E2M3, RFQ_MX_FP8>(d_raw, prep, L, true, s);
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
