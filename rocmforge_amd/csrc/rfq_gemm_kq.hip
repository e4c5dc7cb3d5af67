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
// the second as one extra k-step per super-block over (min, S) pairs with S
// split into fp16 hi + lo (exact to 2^-22; min is exact in fp16).
//
// Two kernels per call.  arrange_a_kernel rewrites the activations into the
// order the matrix instruction reads them (and computes S for Q4_K), into a
// temporary the library keeps per stream.  gemm_kq_kernel: workgroup tile 256
// (m) x 128 (n), k advances 64 per stage, 256 threads = one wavefront per
// SIMD, each 64 m x 128 n = 2 x 4 instruction tiles (the weight fragment is
// the instruction's first operand, so a lane ends up with 4 consecutive n of
// one output row).
//   * Activations go global -> registers, straight into the operand registers:
//     1 KiB of consecutive bytes per wavefront load, four stages ahead.  They
//     never touch LDS, whose bandwidth the weight fragments need.
//   * Weights: thread t decodes the 32-element group t%2 of row t/2 of a
//     stage (a Q4_0/Q8_0 block, a Q4_K/Q6_K sub-block) from raw bytes loaded
//     four stages ahead, two stages before its use, into one of four LDS
//     buffers; every wavefront reads all four weight fragments of a k-step
//     from there.
//   * One wavefront per SIMD means nothing hides a stall: the body of a stage
//     is laid out by hand, one matrix instruction per slot with its share of
//     loads, decode steps and LDS traffic, and pinned in that order.
// Measured on this layout: the matrix pipe alone (same instruction mix, no
// other work) runs at about 35 clocks per instruction at a shader clock that
// power management holds near 1.5-1.7 GHz under this load; the loop runs at
// about 43.
#include <mutex>
#include <unordered_map>
#include <vector>
#include <type_traits>

#include "rfq_gemm_kq_decode.hpp"

// Temporary memory of rfq_gemm_f16_static, the entry point for callers that cannot allocate (stream capture,
// serving loops): the arranged activations and the Q4_K group sums of one call.  Every GPU the library runs on
// holds its own copy of this array until the process ends.  Host code never uses the array's name as an address:
// static_scratch() resolves the copy of the current device once and hands out that pointer.
constexpr size_t RFQ_STATIC_SCRATCH_BYTES = (size_t)16 << 20;
// This file is compiled in two parts (RFQ_KQ_PART): part 1 holds only the integer-operand kernel of GGUF_Q4_K, whose
// accumulators are multiplied by vector instructions between super-blocks and therefore want to live in ordinary
// vector registers (-amdgpu-mfma-vgpr-form: 83.6 -> 77.1 us at 512 x 4096 x 14336); the other kernels measured
// slower that way (Q4_K 65.6 -> 68.0 us) and are part 0, with the entry points and everything that owns memory.
#ifndef RFQ_KQ_PART
#define RFQ_KQ_PART 0
#endif
#if RFQ_KQ_PART == 0
static __device__ __align__(256) uint8_t scratch[RFQ_STATIC_SCRATCH_BYTES];
#endif

namespace rfq {
// (defined in part 1 of this file)
int launch_gguf_q4_k_int(const uint8_t *w, const void *a, void *out, bool out_f16, int m, int n, int k, uint8_t *static_tmp,
                         const uint8_t *arranged, hipStream_t s);
namespace {

using namespace kq;


constexpr int BM = 256, BN = 128, BK = 64;
constexpr int TI = 2, TJ = 4;                    // instruction tiles of a wavefront: 64 m x 128 n
constexpr int LDR = BK * 2 + 16;                 // bytes per LDS row: 64 fp16 + 16 pad (rows 36 dwords apart)
constexpr int W_BYTES = BN * LDR;                // one stage of decoded weights


// Activations in the order the matrix instruction reads them.  Unit (mt, st)
// = 32 rows x 64 k; inside it chunk c (0..3) of lane (fr, fh) holds
// A[32*mt + fr][64*st + 32*fh + 8*c .. +8] in the order of chunk_pos():
// at[((mt*nst + st)*4 + c)*64 + lane] in 16-byte units, so that a wavefront's
// load of one chunk is 1 KiB of consecutive bytes.  Rows past M and k past K
// are zero.
// With SUMS (K a multiple of 256) also S[m, g] = sum of the 32 activations of
// group g (fp32, in k order) as the fp16 pair (hi, lo) with hi + lo = S to
// 2^-22, again in operand order: the 16 bytes of lane (fr, fh) in unit
// (mt, super-block) are the pairs of sub-blocks 4*fh .. 4*fh+3 of row 32*mt+fr.
template <bool SUMS>
__global__ void __launch_bounds__(256)
arrange_a_kernel(const _Float16 *__restrict__ a, v4u *__restrict__ at, _Float16 *__restrict__ s2, int M, int K,
                 int tiles32, int nst)
{
    // A workgroup takes 32 rows x 256 k (four units): whole 512-byte row pieces
    // come in with consecutive lanes on consecutive bytes, and a wavefront per
    // unit reads its operand order back out of LDS.
    constexpr int ROWB = 512 + 16;                                // row stride = 4 banks mod 32
    __shared__ __attribute__((aligned(16))) uint8_t stage[32 * ROWB];
    const int groups4 = (nst + 3) / 4;
    const int mt = blockIdx.x / groups4, st0 = (blockIdx.x % groups4) * 4;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int row = p * 8 + (tid >> 5), col = tid & 31;       // 16-byte column of the 512-byte piece
        const int m = mt * 32 + row, k = st0 * 64 + col * 8;
        v4u v = {0, 0, 0, 0};
        if (m < M && k < K) v = *reinterpret_cast<const v4u *>(a + (size_t)m * K + k);
        *reinterpret_cast<v4u *>(stage + row * ROWB + col * 16) = v;
    }
    __syncthreads();
    const int st = st0 + wave;
    if (st >= nst) return;
    const int fr = lane & 31, fh = lane >> 5;
    const int k0 = st * 64 + fh * 32;
    const size_t unit = (size_t)mt * nst + st;
    v4u v[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        v[c] = *reinterpret_cast<const v4u *>(stage + fr * ROWB + wave * 128 + fh * 64 + c * 16);
        // dwords (k0 k1)(k2 k3)(k4 k5)(k6 k7) -> (k0 k4)(k1 k5)(k2 k6)(k3 k7)
        const v4u p = {__builtin_amdgcn_perm(v[c][2], v[c][0], 0x05040100u), __builtin_amdgcn_perm(v[c][2], v[c][0], 0x07060302u),
                       __builtin_amdgcn_perm(v[c][3], v[c][1], 0x05040100u), __builtin_amdgcn_perm(v[c][3], v[c][1], 0x07060302u)};
        at[(unit * 4 + c) * 64 + lane] = p;
    }
    if (SUMS && k0 < K) {                                         // (rows past M were staged as zeros: their sums are zero)
        float sum = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            v8h h;
            __builtin_memcpy(&h, &v[c], 16);
#pragma unroll
            for (int e = 0; e < 8; e++) sum += (float)h[e];
        }
        _Float16 hi, lo;
        fp16_pair(sum, hi, lo);
        const int g = k0 / 32, sb = g & 7;
        const size_t t = ((((size_t)mt * (K / 256) + (g >> 3)) * 2 + (sb >> 2)) * 32 + fr) * 4 + (sb & 3);
        typedef _Float16 h2 __attribute__((ext_vector_type(2), aligned(2)));
        *reinterpret_cast<h2 *>(s2 + 2 * t) = h2{hi, lo};              // (one store for the pair)
    }
}

// PLANES = 2: every stage of k is walked twice, first with the weights' fp16 values (hi) and then with what the
// rounding to fp16 left over (lo = fp16(v - hi)), as two consecutive stages of the same pipeline over the same
// activations and the same raw weight bytes (loaded once per pair): the contraction then carries the weights to 2^-22
// instead of 2^-12.
template <int FMT, bool OUT_F16, int PLANES>
__global__ void __launch_bounds__(256)
gemm_kq_kernel(const uint8_t *__restrict__ w, const v4u *__restrict__ at, const _Float16 *__restrict__ s2,
               void *__restrict__ outp, int M, int N, int Kfull, int kparts)
{
    // kparts > 1 (few output tiles, long k): the launch holds kparts workgroups per tile, each contracts a whole number
    // of super-blocks [k0, k0 + K) of the rows and writes its f32 partial tile to outp[part][M][N]; reduce_parts_kernel
    // adds the parts in order.
    const int K = Kfull / kparts;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // INT: integer operands sc * q; acc runs in units of the current super-block's d (f32), rescaled between super-blocks
    constexpr bool INT = FMT == KQ_GGUF_Q4_K_INT;
    constexpr bool SUMS = FMT == RFQ_Q4_K || INT;                 // the min term goes through the activations' group sums
    static_assert(!INT || PLANES == 1, "the integer operands are exact: one plane");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int fr = lane & 31, fh = lane >> 5;                     // fragment row, k half
    const int tiles_m = (M + BM - 1) / BM;
    // Workgroups are dealt round-robin to the 8 XCDs (blockIdx.x % 8), each with an L2 of its own: hand every XCD a
    // contiguous run of tiles, so that the m tiles of one W tile meet in one L2 and W comes from HBM once.
    const int nwg = gridDim.x;
    const int slot = nwg % 8 == 0 ? (int)(blockIdx.x % 8) * (nwg / 8) + (int)(blockIdx.x / 8) : (int)blockIdx.x;
    const int tiles_all = nwg / kparts, part = slot / tiles_all, tile = slot % tiles_all;
    const int k0 = part * K;
    const int tm = tile % tiles_m, tn = tile / tiles_m;             // the m tiles of one W tile are neighbours
    const int m0 = tm * BM, n0 = tn * BN;
    const int groups = K / 32;                                    // 32-element groups per row
    const size_t row_bytes = (size_t)(Kfull / Fmt<FMT>::BE) * Fmt<FMT>::BB;
    const size_t k0_bytes = (size_t)(k0 / Fmt<FMT>::BE) * Fmt<FMT>::BB;     // (kparts > 1: k0 is whole super-blocks)
    const int kstages_full = (Kfull + BK - 1) / BK;
    const int kstages = (K + BK - 1) / BK;                        // stages of k
    const int nstages = kstages * PLANES;                         // stages the pipeline walks

    // Weights: thread t decodes group t%2 of row t/2 of each stage into LDS.
    const int wr = tid >> 1, wh = tid & 1;
    // (a buffer descriptor from the tile's first row to the end of W, plus a 32-bit lane offset)
    const size_t w_left = (size_t)(N - n0) * row_bytes - k0_bytes;
    const Rsrc w_tile = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(w) + (size_t)n0 * row_bytes + k0_bytes, 0,
                                                          w_left < 0xFFFFFFFFu ? (int)(uint32_t)w_left : -1, 0x00020000);
    const uint32_t w_off = (uint32_t)((n0 + wr < N ? wr : N - 1 - n0) * (int)row_bytes);
    // Activations never pass through LDS: they arrive arranged in the order
    // the matrix instruction reads them (arrange_a_kernel), so each lane loads
    // its 4 x 16 bytes of a stage straight into the operand registers, and a
    // wavefront's load instruction covers 1 KiB of consecutive bytes.  k-step
    // c of a stage is k = 32*fh + 8*c .. +8 (any assignment of k to the
    // instruction's k slots works as long as both operands use it); the
    // weight fragment is read from LDS at the same k.
    const int tiles32 = (M + 31) / 32;
    // (buffer loads: a scalar descriptor per m tile, the stage as scalar
    // offset, the lane as 32-bit vector offset; no 64-bit vector arithmetic)
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lane16 = lane * 16;
    __amdgpu_buffer_rsrc_t a_tile[TI];
#pragma unroll
    for (int i = 0; i < TI; i++) {
        const int mt = m0 / 32 + wave_u * 2 + i;
        a_tile[i] = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<v4u *>(at + ((size_t)(mt < tiles32 ? mt : tiles32 - 1) * kstages_full + k0 / BK) * 256), 0, kstages * 4096, 0x00020000);
    }

    // Global loads run three stages ahead of the arithmetic through a ring of
    // four register sets (separate objects with compile-time indices: the
    // loop is unrolled by four, so nothing can index the ring at run time).
    // The loads are unconditional (clamped addresses): rows past M or N only
    // feed outputs that are never stored, and k past K meets zero weights.
    Raw32<FMT> raw0, raw1, raw2, raw3;
    v4u ra0[TI][4], ra1[TI][4], ra2[TI][4], ra3[TI][4];
    auto raw_of = [&](auto slotc) -> Raw32<FMT> & {
        constexpr int S = decltype(slotc)::value;
        if constexpr (S == 0) return raw0;
        else if constexpr (S == 1) return raw1;
        else if constexpr (S == 2) return raw2;
        else return raw3;
    };
    auto ra_of = [&](auto slotc) -> v4u (&)[TI][4] {
        constexpr int S = decltype(slotc)::value;
        if constexpr (S == 0) return ra0;
        else if constexpr (S == 1) return ra1;
        else if constexpr (S == 2) return ra2;
        else return ra3;
    };
    auto fetch_w = [&](auto slotc, int st) __attribute__((always_inline)) {
        // the last stage of a row with an odd number of groups has no second
        // group: both lanes of the row then read the first (zeroed when decoded)
        const int sc = (st < nstages ? st : nstages - 1) / PLANES;
        const int whc = Fmt<FMT>::BE == 32 && sc * 2 + 1 >= groups ? 0 : wh;
        if constexpr (INT) raw_of(slotc).template load_slot<decltype(slotc)::value>(w_tile, w_off, sc);   // (one plane: slot = stage % 4)
        else raw_of(slotc).load(w_tile, w_off, sc, whc);
    };
    auto fetch_a = [&](auto slotc, int st, int i, int c) __attribute__((always_inline)) {
        const int sc = (st < nstages ? st : nstages - 1) / PLANES;
        ra_of(slotc)[i][c] = __builtin_amdgcn_raw_buffer_load_b128(a_tile[i], lane16 + c * 1024, sc * 4096, 0);
    };
    auto fetch_a_all = [&](auto slotc, int st) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int c = 0; c < 4; c++) fetch_a(slotc, st, i, c);
    };
    uint32_t int_s2[2] = {0, 0}, int_o2[2] = {0, 0};              // INT: the scales of the super-block being settled, as fp16 operands
    // groups past the end of the row become zero weights (here, not at the
    // load: a select right behind the load would wait for it)
    auto settle = [&](auto slotc, int st, uint32_t pair) __attribute__((always_inline)) {
        Raw32<FMT> &raw = raw_of(slotc);
        Raw32<FMT> z;
        z.zero();
        // (group 2*stage + wh has the parity of wh; with one plane the ring slot is the stage's number within its super-block)
        // (INT: the super-block's scales come from its header hand-over, which precedes the settling of its four stages)
        if constexpr (INT) raw.settle_packed(wh, int_s2, int_o2, decltype(slotc)::value);
        else raw.settle(wh, pair, PLANES == 1 ? decltype(slotc)::value : (st / PLANES) & 3);
#pragma unroll
        // (the integer-operand decoder: sc = 0 makes every weight zero; its mask and offset dwords stay what every stage has)
        for (int i = 0; i < (INT ? 2 : Raw32<FMT>::ND); i++) raw.d[i] = (st / PLANES) * 2 + wh < groups ? raw.d[i] : z.d[i];
    };

    // Four LDS buffers of decoded weights (buffer = stage % 4, a compile-time
    // number inside the loop body, so every LDS offset is an immediate; two
    // base registers because an immediate reaches 64 KiB).
    const uint8_t *rd_base[2] = {lds + fr * LDR + fh * 64, lds + 2 * W_BYTES + fr * LDR + fh * 64};
    uint8_t *wr_base[2] = {lds + wr * LDR + wh * 64, lds + 2 * W_BYTES + wr * LDR + wh * 64};
    auto read_frag = [&](int buf, int j, int c) __attribute__((always_inline)) -> v8h {
        return *reinterpret_cast<const v8h *>(rd_base[buf >> 1] + (buf & 1) * W_BYTES + j * 32 * LDR + c * 16);
    };
    auto stash = [&](int buf, int c, const v8h (&hw)[4]) __attribute__((always_inline)) {
        *reinterpret_cast<v8h *>(wr_base[buf >> 1] + (buf & 1) * W_BYTES + c * 16) = hw[c];
    };

    v16f acc[TJ][TI];
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0.0f;

    // The Q4_K min term rides along as one extra k-step per super-block (four
    // stages = one trip through the ring): its 16 k slots are the (hi, lo)
    // halves of the group sums S of the super-block's 8 sub-blocks; the weight
    // is the sub-block's min in both slots.  The thread that decodes a row's
    // sub-blocks loads the super-block's header (8 scales, its 4 mins) with
    // the raw bytes of the super-block's first stage (ring slot 0), keeps it
    // in set B while decoding that super-block's first two stages and in set
    // A for the last two (one trip later), and writes the expanded mins to a
    // small LDS area that all wavefronts read as the weight fragment.  S
    // comes arranged in operand order, one 16-byte load per lane and m tile,
    // with the A registers of the trip's first stage.
    // (Every load is consumed in the loop iteration that issued it or at a
    // fixed compile-time distance, so the wait counts stay exact.)
    v4u hs_ring = {0, 0, 0, 0}, hsA = {0, 0, 0, 0}, hsB = {0, 0, 0, 0};
    uint32_t hm_ring = 0, hmA = 0, hmB = 0;
    v4u sa_cur[TI], sa_ring[TI];
    __amdgpu_buffer_rsrc_t s_tile[TI];
    v8h fm[TJ], fm_lo[TJ];
    typedef float v4f __attribute__((ext_vector_type(4)));
    v4f f4[2][4];                                                 // INT: the ratios of the tile rescaled next
    float d_unit = 1.0f;                                          // INT: the unit acc is in, for the row this thread decodes
    constexpr int MNR = 48;                                       // bytes per row of the min area (32 used)
    uint8_t *mn_wr = lds + 4 * W_BYTES + wr * MNR + wh * 16;
    const uint8_t *mn_rd = lds + 4 * W_BYTES + fr * MNR + fh * 16;
    if constexpr (SUMS) {
#pragma unroll
        for (int i = 0; i < TI; i++) {
            const int mt = m0 / 32 + wave_u * 2 + i;
            s_tile[i] = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint8_t *>(reinterpret_cast<const uint8_t *>(s2)) + ((size_t)(mt < tiles32 ? mt : tiles32 - 1) * (Kfull / 256) + k0 / 256) * 1024,
                0, (K / 256) * 1024, 0x00020000);
        }
    }
    auto fetch_hdr = [&](int trip) __attribute__((always_inline)) {
        if constexpr (FMT == RFQ_Q4_K) {
            const int blk = (trip < K / 256 ? trip : K / 256 - 1) * 256;
            hs_ring = __builtin_amdgcn_raw_buffer_load_b128(w_tile, w_off, blk, 0);
            hm_ring = __builtin_amdgcn_raw_buffer_load_b32(w_tile, w_off + 16 + 4 * wh, blk, 0);
        }
    };
    auto fetch_sums = [&](int trip) __attribute__((always_inline)) {
        if constexpr (SUMS) {
            const int t = trip < K / 256 ? trip : K / 256 - 1;
#pragma unroll
            for (int i = 0; i < TI; i++) sa_ring[i] = __builtin_amdgcn_raw_buffer_load_b128(s_tile[i], lane16, t * 1024, 0);
        }
    };
    // 4 i8 mins -> 8 fp16 (each twice): 0x6400 | (min ^ 0x80) reads 1024 + 128 + min
    auto stash_mins = [&]() __attribute__((always_inline)) {
        typedef _Float16 v2h __attribute__((ext_vector_type(2)));
        const v2h bias = {(_Float16)-1152.0f, (_Float16)-1152.0f};
        const uint32_t u = hmA ^ 0x80808080u;
        v8h h;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t bits = __builtin_amdgcn_perm(0x64646464u, u, 0x04000400u | (uint32_t)b | ((uint32_t)b << 16));
            v2h v;
            __builtin_memcpy(&v, &bits, 4);
            v = v + bias;
            h[2 * b] = v[0];
            h[2 * b + 1] = v[1];
        }
        *reinterpret_cast<v8h *>(mn_wr) = h;
    };
    constexpr int INT_AREA = 2 * BN * MNR + 2 * BN * 4;           // min fragments (hi, lo), ratio and unit of one super-block
    uint8_t *const int_base = lds + 4 * W_BYTES + BN * MNR;
    auto compute_min = [&](int parity) __attribute__((always_inline)) {
        if constexpr (SUMS && !INT) {
#pragma unroll
            for (int i = 0; i < TI; i++) {
                v8h fa;
                __builtin_memcpy(&fa, &sa_cur[i], 16);
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fm[j], fa, acc[j][i], 0, 0, 0);
                }
            }
        }
    };
    // INT: acc is kept in units of the running super-block's d: sum over the super-blocks so far of (d_b / d) * sum
    // (sc * q) * a - the matrix cores add the integer products, and between two super-blocks acc is multiplied by
    // d_prev / d_next per weight row (f32; sixteen such roundings at k = 4096).  The min term -(dmin * m) * S is
    // divided by d to join it.  A super-block's header goes to LDS when its first stage is settled (three stages
    // before it is multiplied), into one of two areas by the super-block's parity: the two min fragments, the
    // ratio that takes acc into its unit, and the unit itself (the epilogue multiplies by the last one).  A
    // super-block with d = 0 has zero weights (settle() clears its sc) and keeps the previous unit.
    struct NoHeader {};
    typename std::conditional<INT, typename Raw32<KQ_GGUF_Q4_K_INT>::Header, NoHeader>::type hdr;
    auto write_header = [&](int parity) __attribute__((always_inline)) {
        if constexpr (INT) {
            uint8_t *area = int_base + parity * INT_AREA;
            *reinterpret_cast<v8h *>(area + wr * MNR + wh * 16) = hdr.m_hi;
            *reinterpret_cast<v8h *>(area + BN * MNR + wr * MNR + wh * 16) = hdr.m_lo;
            *reinterpret_cast<float *>(area + 2 * BN * MNR + wh * BN * 4 + wr * 4) = wh ? d_unit : hdr.ratio;
        }
    };
    auto stash_header = [&](const Raw32<FMT> &raw, int parity) __attribute__((always_inline)) {
        if constexpr (INT) {
            raw.header(wh, d_unit, int_s2, int_o2, hdr);
            write_header(parity);
        }
    };
    // acc *= f[n] (register r of a tile: n = 8*(r/4) + 4*fh + r%4: four factors side by side); which = 0: the ratio
    // into the unit of the super-block of that parity, 1: that unit itself
    auto rescale = [&](int parity, int which) __attribute__((always_inline)) {
        if constexpr (INT) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            const uint8_t *src = int_base + parity * INT_AREA + 2 * BN * MNR + which * BN * 4 + fh * 16;
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const v4f f4 = *reinterpret_cast<const v4f *>(src + (j * 32 + 8 * g) * 4);
#pragma unroll
                    for (int i = 0; i < TI; i++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[j][i][4 * g + e] *= f4[e];
                }
        }
    };

    // One wavefront per SIMD: nothing hides a stall, so the body of a stage is
    // laid out by hand as 32 slots of one matrix instruction plus a share of
    // the stage's other work, and pinned in that order.  Iteration st (S =
    // st%4) multiplies stage st (LDS buffer S, A registers of ring slot S):
    //   * weight fragments are read one k-step ahead, the last ones from the
    //     next stage's buffer (written during the previous iteration);
    //   * decoding runs at an even pace, six of a group's twelve steps in
    //     slots 0..13 (second half of stage st+2) and six in slots 16..29
    //     (first half of stage st+3; two sets of fp16 registers, by stage
    //     parity); stage st+2 goes to LDS buffer S+2 in slots 17..23, and slot
    //     25 refills its raw registers (stage st+6);
    //   * (Q4_K) slot 24 of a trip's first stage writes the min fragment, slots
    //     28..31 of its last stage read it;
    //   * the four matrix instructions that read an A chunk are followed by
    //     the load that refills it (stage st+4).
    // One barrier per stage: behind it stage st+2 is visible, and nobody still
    // reads the buffer the next iteration overwrites (st+3 = st-1 mod 4).
    v8h fw[2][TJ];
    v8h hw_even[4], hw_odd[4];                                    // decoded weights of the even / odd stage in progress
    // Two planes: a pair's raw bytes are decoded once, during the hi stage's steps, into both operands; the lo values
    // wait here until the lo stage's turn to go to LDS (two sets: the next pair's steps start before that).
    v8h hw_lo0[4], hw_lo1[4];
    auto lo_of = [&](auto pc) -> v8h (&)[4] {
        if constexpr (decltype(pc)::value == 0) return hw_lo0;
        else return hw_lo1;
    };
    v2h dec_tmp[4];                                               // a chunk between its decode steps
    auto iter = [&](auto sc, int st) __attribute__((always_inline)) {
        constexpr int S = decltype(sc)::value, S1 = (S + 1) & 3, S2 = (S + 2) & 3, S3 = (S + 3) & 3;
        // With two planes the two stages of a pair (even ring slot = hi, odd = lo) are the same 64 k: the odd slot has
        // no registers of its own, it decodes and multiplies out of its even neighbour's (SH = the slot that holds
        // the data), which is refilled once both have used it.
        constexpr int SH0 = PLANES == 2 ? (S & ~1) : S, SH2 = PLANES == 2 ? (S2 & ~1) : S2, SH3 = PLANES == 2 ? (S3 & ~1) : S3;
        Raw32<FMT> &raw_late = raw_of(IC<SH2>{}), &raw_early = raw_of(IC<SH3>{});
        v8h (&hw_late)[4] = (S & 1) ? hw_odd : hw_even;
        v8h (&hw_early)[4] = (S & 1) ? hw_even : hw_odd;
        v4u (&ra)[TI][4] = ra_of(IC<SH0>{});
        if constexpr (SUMS) {
            if (S == 0) {                                          // this trip's sums arrived with stage st's A
#pragma unroll
                for (int i = 0; i < TI; i++) sa_cur[i] = sa_ring[i];
                fetch_sums(st / 4 + 1);
            }
        }
        if constexpr (FMT == RFQ_Q4_K) {
            if (S == 1) {                                          // stage st+3 opens the next super-block
                // (real moves: merged with hs_ring's registers, the copy would
                // turn into one at the end of the loop body that waits for the
                // refill issued below)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    uint32_t v;
                    asm volatile("v_mov_b32 %0, %1" : "=v"(v) : "v"(hs_ring[q]));
                    hsB[q] = v;
                }
                asm volatile("v_mov_b32 %0, %1" : "=v"(hmB) : "v"(hm_ring));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const int i = t >> 2, j = t & 3, p = c * 8 + t;
                v8h fa;
                __builtin_memcpy(&fa, &ra[i][c], 16);
                acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[c & 1][j], fa, acc[j][i], 0, 0, 0);
                if (t < 4) fw[(c + 1) & 1][t] = c < 3 ? read_frag(S, t, c + 1) : read_frag(S1, t, 0);
                {
                    constexpr int LATE[6] = {0, 3, 5, 8, 10, 13}, EARLY[6] = {16, 18, 20, 22, 26, 29};
#pragma unroll
                    for (int q = 0; q < 6; q++) {
                        if constexpr (PLANES == 1) {
                            if (p == LATE[q]) raw_late.template step<false>(6 + q, hw_late, hw_late, dec_tmp);
                            if (p == EARLY[q]) raw_early.template step<false>(q, hw_early, hw_early, dec_tmp);
                        } else {
                            if ((S2 & 1) == 0 && p == LATE[q]) raw_late.template step<true>(6 + q, hw_late, lo_of(IC<(S2 >> 1) & 1>{}), dec_tmp);
                            if ((S3 & 1) == 0 && p == EARLY[q]) raw_early.template step<true>(q, hw_early, lo_of(IC<(S3 >> 1) & 1>{}), dec_tmp);
                        }
                    }
                }
                if constexpr (INT) {
                    // The super-block's min term rides on its first stage: behind the first k-step's matrix
                    // instruction of a tile the hi fragment against the group sums, behind the second the lo fragment.
                    if (S == 0 && c < 2) {
                        v8h fs;
                        __builtin_memcpy(&fs, &sa_cur[i], 16);
                        acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(c == 0 ? fm[j] : fm_lo[j], fs, acc[j][i], 0, 0, 0);
                    }
                    // A tile goes into the next super-block's unit in the slot after its last matrix instruction
                    // of this one (the last tile at the start of the next stage); the ratios of a tile's 16
                    // weight rows are read one slot before.
                    const uint8_t *next_area = int_base + (((st >> 2) + 1) & 1) * INT_AREA;
                    if ((S == 3 && p >= 25) || (S == 0 && p == 0)) {
                        const int tile = S == 3 ? p - 25 : 7;
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[tile & 3][tile >> 2][r] *= f4[tile & 1][r >> 2][r & 3];
                    }
                    if (S == 3 && p >= 24) {
#pragma unroll
                        for (int g = 0; g < 4; g++)
                            f4[t & 1][g] = *reinterpret_cast<const v4f *>(next_area + 2 * BN * MNR + fh * 16 + (j * 32 + 8 * g) * 4);
                    }
                    // the fragments of the next super-block's min term
                    if (S == 3 && p >= 28) fm[p - 28] = *reinterpret_cast<const v8h *>(next_area + fr * MNR + fh * 16 + (p - 28) * 32 * MNR);
                    if (S == 0 && p < 4)
                        fm_lo[p] = *reinterpret_cast<const v8h *>(int_base + ((st >> 2) & 1) * INT_AREA + BN * MNR + fr * MNR + fh * 16 + p * 32 * MNR);
                    // stage st+3 opens the next super-block: its header goes to the other area before settle() reuses the dwords
                    // (in eight pieces between the stage's other work; no stage is being settled meanwhile)
                    if (S == 1) {
                        constexpr int AT[8] = {1, 2, 4, 6, 7, 9, 11, 14};
                        const Raw32<FMT> &next_hdr = raw_of(IC<S3>{});
                        if (p == AT[0]) next_hdr.template header_phase<0>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[1]) next_hdr.template header_phase<1>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[2]) next_hdr.template header_phase<2>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[3]) next_hdr.template header_phase<3>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[4]) next_hdr.template header_phase<4>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[5]) next_hdr.template header_phase<5>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[6]) next_hdr.template header_phase<6>(wh, d_unit, int_s2, int_o2, hdr);
                        if (p == AT[7]) write_header(((st + 3) >> 2) & 1);
                    }
                }
                if (p == 15 && SH3 == S3) settle(IC<S3>{}, st + 3, S == 0 ? hsA[3] : hsB[S3]);   // stage st+3 is number S3 of its super-block
                if (p >= 17 && p <= 23 && (p & 1)) {
                    if constexpr (PLANES == 2 && (S2 & 1) != 0) stash(S2, (p - 17) / 2, lo_of(IC<(S2 >> 1) & 1>{}));
                    else stash(S2, (p - 17) / 2, hw_late);
                }
                if (p == 25) {
                    if constexpr (PLANES == 1) fetch_w(IC<S2>{}, st + 6);
                    else if constexpr (S2 & 1) fetch_w(IC<SH2>{}, st + 5);   // both planes of the pair are decoded: its slot takes the next pair
                    if (S == 2) fetch_hdr((st + 6) / 4);
                }
                if constexpr (FMT == RFQ_Q4_K) {
                    // the min fragment of this trip: written in its first stage, read in its last
                    if (S == 0 && p == 24) stash_mins();
                    if (S == 3 && p >= 28) fm[p - 28] = *reinterpret_cast<const v8h *>(mn_rd + (p - 28) * 32 * MNR);
                }
                if constexpr (PLANES == 1) {
                    if (j == 3) fetch_a(sc, st + 4, i, c);
                } else if constexpr (S & 1) {
                    if (j == 3) fetch_a(IC<SH0>{}, st + 3, i, c);   // the lo stage was the chunk's last reader
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        lds_barrier();
    };
    {
        v8h hw[4];
        // (the loads the loop consumes first in each trip go out first here too:
        // the wait counts of the loop are the smaller of those seen on the two
        // ways into it)
        fetch_hdr(1);
        fetch_sums(0);
        if constexpr (FMT == RFQ_Q4_K) {
            hsA = __builtin_amdgcn_raw_buffer_load_b128(w_tile, w_off, 0, 0);
            hmA = __builtin_amdgcn_raw_buffer_load_b32(w_tile, w_off + 16 + 4 * wh, 0, 0);
        }
        fetch_w(IC<0>{}, 0);
        fetch_a_all(IC<0>{}, 0);
        if constexpr (PLANES == 1) {
            fetch_w(IC<1>{}, 1);
            fetch_a_all(IC<1>{}, 1);
        }
        fetch_w(IC<2>{}, 2);
        fetch_a_all(IC<2>{}, 2);
        if constexpr (PLANES == 1) {
            fetch_w(IC<3>{}, 3);
            fetch_a_all(IC<3>{}, 3);
        }
        // (a real move: the loop must not inherit a pending load on hmA, or its
        // first use in the loop body would wait for younger loads every trip)
        asm volatile("v_mov_b32 %0, %1" : "=v"(hmA) : "v"(hmA));
        stash_header(raw0, 0);
        settle(IC<0>{}, 0, hsA[0]);
#pragma unroll
        for (int T = 0; T < 12; T++) raw0.template step<PLANES == 2>(T, hw, hw_lo0, dec_tmp);
#pragma unroll
        for (int c = 0; c < 4; c++) stash(0, c, hw);
        if constexpr (PLANES == 1) {
            fetch_w(IC<0>{}, 4);
            settle(IC<1>{}, 1, hsA[1]);
#pragma unroll
            for (int T = 0; T < 12; T++) raw1.template step<false>(T, hw, hw, dec_tmp);
#pragma unroll
            for (int c = 0; c < 4; c++) stash(1, c, hw);
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) stash(1, c, hw_lo0);
        }
        if constexpr (PLANES == 1) fetch_w(IC<1>{}, 5);
        else fetch_w(IC<0>{}, 4);
        settle(IC<2>{}, 2, hsA[2]);
#pragma unroll
        for (int T = 0; T < 6; T++) raw2.template step<PLANES == 2>(T, hw_even, hw_lo1, dec_tmp);
        lds_barrier();
#pragma unroll
        for (int j = 0; j < TJ; j++) fw[0][j] = read_frag(0, j, 0);
        if constexpr (INT) {
#pragma unroll
            for (int j = 0; j < TJ; j++) fm[j] = *reinterpret_cast<const v8h *>(int_base + fr * MNR + fh * 16 + j * 32 * MNR);
#pragma unroll
            for (int r = 0; r < 16; r++) f4[1][r >> 2][r & 3] = 1.0f;   // (the first stage multiplies the empty last tile by these)
        }
    }
    // Whole trips through the ring only (no branch between the four bodies);
    // stages past the end multiply zero weights.
    for (int st = 0; st < nstages; st += 4) {
        iter(IC<0>{}, st);
        iter(IC<1>{}, st + 1);
        iter(IC<2>{}, st + 2);
        iter(IC<3>{}, st + 3);
        compute_min((st >> 2) & 1);
        if constexpr (FMT == RFQ_Q4_K) {
            hsA = hsB;
            hmA = hmB;
        }
    }

    // Register r of tile (j, i): n = 8*(r/4) + 4*(lane/32) + r%4 within the
    // tile (four consecutive n per r/4), m = lane%32.
    //
    // Whole tiles leave through LDS (free now: the loop ended on a barrier),
    // 32 rows of a wavefront at a time in an area of its own, so that each
    // output row goes out as full 16-byte pieces of consecutive n instead of 8-
    // or 16-byte pieces one row apart.
    rescale(((K / 256) - 1) & 1, 1);                               // INT: from the last super-block's unit to values
    typedef typename std::conditional<OUT_F16, _Float16, float>::type OutT;
    outp = reinterpret_cast<uint8_t *>(outp) + (size_t)part * M * N * sizeof(OutT);
    constexpr int ROWB = BN * (int)sizeof(OutT) + 16;             // bytes per staged row (row stride = 4 banks mod 32)
    static_assert(4 * 32 * ROWB <= 4 * W_BYTES, "staging area");
    if (m0 + BM <= M && n0 + BN <= N && (N * sizeof(OutT)) % 16 == 0 && (reinterpret_cast<uintptr_t>(outp) & 15u) == 0) {
        uint8_t *area = lds + wave * (32 * ROWB);
        constexpr int CPR = BN * (int)sizeof(OutT) / 16, RPI = 64 / CPR; // 16-byte chunks per row, rows per store instruction
        const int chunk = lane % CPR, row_l = lane / CPR;
#pragma unroll
        for (int i = 0; i < TI; i++) {
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    uint8_t *dst = area + fr * ROWB + (j * 32 + 8 * g + 4 * fh) * (int)sizeof(OutT);
                    if (OUT_F16) {
                        typedef _Float16 v4h __attribute__((ext_vector_type(4)));
                        *reinterpret_cast<v4h *>(dst) = v4h{(_Float16)acc[j][i][4 * g], (_Float16)acc[j][i][4 * g + 1],
                                                            (_Float16)acc[j][i][4 * g + 2], (_Float16)acc[j][i][4 * g + 3]};
                    } else {
                        typedef float v4f __attribute__((ext_vector_type(4)));
                        *reinterpret_cast<v4f *>(dst) = v4f{acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]};
                    }
                }
            // (the area belongs to this wavefront alone, and a wavefront's LDS
            // operations complete in order: no barrier between write and read)
#pragma unroll
            for (int it = 0; it < 32 / RPI; it++) {
                const int row = it * RPI + row_l;
                const v4u v = *reinterpret_cast<const v4u *>(area + row * ROWB + chunk * 16);
                uint8_t *o = reinterpret_cast<uint8_t *>(outp) +
                             ((size_t)(m0 + wave * 64 + i * 32 + row) * N + n0) * sizeof(OutT) + chunk * 16;
                __builtin_nontemporal_store(v, reinterpret_cast<v4u *>(o));
            }
        }
        return;
    }
    const bool vec_ok = (N % 4) == 0 && (reinterpret_cast<uintptr_t>(outp) & 15u) == 0;
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
        for (int i = 0; i < TI; i++) {
            const int m = m0 + wave * 64 + i * 32 + fr;
            if (m >= M) continue;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n = n0 + j * 32 + 8 * g + 4 * fh;
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

// out[i] = parts[0][i] + parts[1][i] + ... (in that order), i < count; four elements per thread where the count allows.
template <bool OUT_F16>
__global__ void __launch_bounds__(256)
reduce_parts_kernel(const float *__restrict__ parts, void *__restrict__ out, size_t count, int kparts)
{
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= count) return;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    const int live = count - i4 >= 4 ? 4 : (int)(count - i4);
    for (int p = 0; p < kparts; p++) {
        const float *src = parts + (size_t)p * count + i4;
        if (live == 4 && (count & 3) == 0) {
            const float4 f = *reinterpret_cast<const float4 *>(src);
            v[0] += f.x; v[1] += f.y; v[2] += f.z; v[3] += f.w;
        } else {
            for (int e = 0; e < live; e++) v[e] += src[e];
        }
    }
    if (live == 4 && (count & 3) == 0) {                               // one store per thread
        if (OUT_F16) {
            // (no alignment promise beyond the element's: global memory takes such stores at any address)
            typedef _Float16 h4 __attribute__((ext_vector_type(4), aligned(2)));
            *reinterpret_cast<h4 *>(reinterpret_cast<_Float16 *>(out) + i4) = h4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        } else {
            typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
            *reinterpret_cast<f4 *>(reinterpret_cast<float *>(out) + i4) = f4{v[0], v[1], v[2], v[3]};
        }
        return;
    }
    for (int e = 0; e < live; e++) {
        if (OUT_F16) reinterpret_cast<_Float16 *>(out)[i4 + e] = (_Float16)v[e];
        else reinterpret_cast<float *>(out)[i4 + e] = v[e];
    }
}

// Parts of k for a launch with few output tiles: as many as fill the part (256 CUs), whole super-blocks each.
int k_parts_for(int m, int n, int k)
{
    const int tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
    if (tiles > 128 || k % 256 != 0) return 1;
    for (int p = 256 / tiles < 8 ? 256 / tiles : 8; p >= 2; p--)
        if (k % (p * 256) == 0 && k / p >= 1024) return p;
    return 1;
}

// Bytes of the arranged activations of an [m, k] matrix, and of the group sums that follow them when k is whole
// super-blocks (the Q4_K kernel reads them; the others ignore them).
size_t arranged_at_bytes(int m, int k) { return (size_t)((m + 31) / 32) * ((k + BK - 1) / BK) * 4096; }
size_t arranged_s2_bytes(int m, int k) { return k % 256 == 0 ? (size_t)((m + 31) / 32) * (k / 256) * 1024 : 0; }

// `arranged` != nullptr: the caller's buffer from launch_arrange_a (activations and sums); a is not read.
template <int FMT, bool OUT_F16, int PLANES>
int launch_cfg(const uint8_t *w, const void *a, void *out, int m, int n, int k, uint8_t *static_tmp, const uint8_t *arranged,
               hipStream_t s)
{
    // four weight stages + the Q4_K min fragment (+ the integer-operand kernel's two header areas)
    constexpr int LDS = 4 * W_BYTES + BN * 48 + (FMT == KQ_GGUF_Q4_K_INT ? 2 * (2 * BN * 48 + 2 * BN * 4) : 0);
    static_assert(LDS <= 160 * 1024, "LDS budget");
    // (both output types: a launch split along k writes f32 parts whatever the caller's type)
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kq_kernel<FMT, OUT_F16, PLANES>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if (attr_err == hipSuccess && OUT_F16)
            attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kq_kernel<FMT, false, PLANES>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    });
    if (attr_err != hipSuccess) return hip_fail(attr_err, "hipFuncSetAttribute(gemm_kq_kernel)");
    const int tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
    if (arranged != nullptr) {
        // (the caller's buffer holds the arranged activations only: nowhere to put parts, no split along k)
        const v4u *at = reinterpret_cast<const v4u *>(arranged);
        const _Float16 *s2 = reinterpret_cast<const _Float16 *>(arranged + arranged_at_bytes(m, k));
        hipLaunchKernelGGL((gemm_kq_kernel<FMT, OUT_F16, PLANES>), dim3(tiles), dim3(256), LDS, s, w, at, s2, out, m, n, k, 1);
        RFQ_LAUNCH_CHECK("gemm_kq_kernel");
        return RFQ_OK;
    }
    // the temporary: the arranged activations, then the Q4_K group sums
    const int tiles32 = (m + 31) / 32, nst = (k + BK - 1) / BK;
    const size_t at_bytes = (size_t)tiles32 * nst * 4096;
    constexpr bool SUMS = FMT == RFQ_Q4_K || FMT == KQ_GGUF_Q4_K_INT;
    const size_t s2_bytes = SUMS ? (size_t)tiles32 * (k / 256) * 1024 : 0;
    // Few output tiles and a long k (an attention or down projection of 512 tokens: 64 tiles for 256 CUs): the launch is
    // split along k, the parts' f32 tiles follow the arranged activations in the temporary, reduce_parts_kernel adds them.
    int kparts = k_parts_for(m, n, k);
    const size_t head_bytes = (at_bytes + s2_bytes + 255) & ~(size_t)255;
    size_t parts_bytes = kparts > 1 ? (size_t)kparts * m * n * sizeof(float) : 0;
    uint8_t *tmp = static_tmp;
    bool transient = false;
    if (static_tmp != nullptr) {
        if (at_bytes + s2_bytes > RFQ_STATIC_SCRATCH_BYTES)
            return fail(RFQ_E_SIZE, "rfq_gemm_f16_static: m=%d k=%d needs %zu bytes of temporary memory, the static buffer holds %zu",
                        m, k, at_bytes + s2_bytes, RFQ_STATIC_SCRATCH_BYTES);
        if (head_bytes + parts_bytes > RFQ_STATIC_SCRATCH_BYTES) {                   // no room for parts: one pass over k
            kparts = 1;
            parts_bytes = 0;
        }
    } else if (int rc = workspace(s, head_bytes + parts_bytes, &tmp, &transient)) {
        return rc;
    }
    v4u *at = reinterpret_cast<v4u *>(tmp);
    _Float16 *s2 = reinterpret_cast<_Float16 *>(tmp + at_bytes);
    hipLaunchKernelGGL((arrange_a_kernel<SUMS>), dim3((unsigned)(tiles32 * ((nst + 3) / 4))), dim3(256), 0, s,
                       reinterpret_cast<const _Float16 *>(a), at, s2, m, k, tiles32, nst);
    if (kparts > 1) {
        float *parts = reinterpret_cast<float *>(tmp + head_bytes);
        const size_t count = (size_t)m * n;
        hipLaunchKernelGGL((gemm_kq_kernel<FMT, false, PLANES>), dim3(tiles * kparts), dim3(256), LDS, s, w, at, s2, parts, m, n, k, kparts);
        hipLaunchKernelGGL((reduce_parts_kernel<OUT_F16>), dim3((unsigned)((count + 1023) / 1024)), dim3(256), 0, s, parts, out, count, kparts);
    } else {
        hipLaunchKernelGGL((gemm_kq_kernel<FMT, OUT_F16, PLANES>), dim3(tiles), dim3(256), LDS, s, w, at, s2, out, m, n, k, 1);
    }
    hipError_t launch_err = hipGetLastError();
    if (transient) {
        hipError_t free_err = hipFreeAsync(tmp, s);
        if (launch_err == hipSuccess) launch_err = free_err;
    }
    if (launch_err != hipSuccess) return hip_fail(launch_err, "gemm_kq_kernel");
    return RFQ_OK;
}

#if RFQ_KQ_PART == 0
template <int FMT>
int launch_fmt(const uint8_t *w, const void *a, void *out, int out_dtype, int m, int n, int k, uint8_t *static_tmp,
               const uint8_t *arranged, hipStream_t s)
{
    // The 256-byte Q4_K layout is contracted in one plane (its large part, the integer mins, is exact and q * scale is
    // small beside it); every other format in two unless the caller asks for one.
    const bool f16 = (out_dtype & ~RFQ_GEMM_ONE_PLANE) == RFQ_F16;
    if constexpr (FMT == RFQ_GGUF_Q4_K) {
        // exact in one pass: integer operands, d and dmin applied in f32
        if ((out_dtype & RFQ_GEMM_ONE_PLANE) == 0) {
            if (k % 256 != 0) return fail(RFQ_E_SIZE, "rfq_gemm_f16: k=%d is not whole Q4_K super-blocks", k);
            return launch_gguf_q4_k_int(w, a, out, f16, m, n, k, static_tmp, arranged, s);
        }
    } else if constexpr (FMT != RFQ_Q4_K) {
        if ((out_dtype & RFQ_GEMM_ONE_PLANE) == 0)
            return f16 ? launch_cfg<FMT, true, 2>(w, a, out, m, n, k, static_tmp, arranged, s)
                       : launch_cfg<FMT, false, 2>(w, a, out, m, n, k, static_tmp, arranged, s);
    }
    return f16 ? launch_cfg<FMT, true, 1>(w, a, out, m, n, k, static_tmp, arranged, s)
               : launch_cfg<FMT, false, 1>(w, a, out, m, n, k, static_tmp, arranged, s);
}

// The address of this device's copy of `scratch`, resolved on the first call on each device.
int static_scratch(uint8_t **out)
{
    static std::mutex mu;
    static uint8_t *ptrs[64];
    int dev = 0;
    RFQ_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return fail(RFQ_E_BADARG, "rfq_gemm_f16_static: device %d outside 0..63", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (ptrs[dev] == nullptr) {
        void *p = nullptr;
        RFQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) return fail(RFQ_E_HIP, "rfq_gemm_f16_static: the static buffer has no device address");
        ptrs[dev] = static_cast<uint8_t *>(p);
    }
    *out = ptrs[dev];
    return RFQ_OK;
}

#endif // RFQ_KQ_PART == 0

} // namespace

#if RFQ_KQ_PART == 1
int launch_gguf_q4_k_int(const uint8_t *w, const void *a, void *out, bool out_f16, int m, int n, int k, uint8_t *static_tmp,
                         const uint8_t *arranged, hipStream_t s)
{
    return out_f16 ? launch_cfg<KQ_GGUF_Q4_K_INT, true, 1>(w, a, out, m, n, k, static_tmp, arranged, s)
                   : launch_cfg<KQ_GGUF_Q4_K_INT, false, 1>(w, a, out, m, n, k, static_tmp, arranged, s);
}
#else

// Temporary device memory for one call.  Up to WS_KEEP bytes it is a buffer
// the library keeps per stream (calls on one stream run in order, so the next
// call may overwrite it; different streams get different buffers) and replaces
// only when a larger one is needed: a stream-ordered allocation and release
// around every call costs about 6 us of idle GPU between calls.  Larger
// requests are allocated and released in stream order, per call.
// One host thread per stream: the pointer is handed out under the lock but used after it, so a second thread that
// grows the same stream's buffer meanwhile would free it under the first thread's launches.
// While the stream is being captured nothing is allocated or freed: the call
// gets the stream's buffer if it is large enough and an error otherwise.  A
// buffer handed out under capture is baked into the graph, so when a later
// call outgrows it the old buffer is retired (kept allocated) instead of
// freed; only release_workspaces() frees retired buffers.
namespace {
constexpr size_t WS_KEEP = (size_t)64 << 20;
struct Kept { uint8_t *ptr; size_t bytes; int device; bool captured; };
std::mutex ws_mutex;
std::unordered_map<hipStream_t, Kept> ws_kept;
std::vector<Kept> ws_retired;
} // namespace

int workspace(hipStream_t s, size_t bytes, uint8_t **out, bool *transient)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    RFQ_HIP(hipStreamIsCapturing(s, &cap));
    const bool capturing = cap != hipStreamCaptureStatusNone;
    if (bytes > WS_KEEP) {
        if (capturing)
            return fail(RFQ_E_UNSUPPORTED, "%zu bytes of temporary memory exceed what the library keeps per stream and cannot be allocated while the stream is being captured", bytes);
        *transient = true;
        RFQ_HIP(hipMallocAsync(reinterpret_cast<void **>(out), bytes, s));
        return RFQ_OK;
    }
    *transient = false;
    int device = 0;
    RFQ_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(ws_mutex);
    Kept &kept = ws_kept[s];
    if (kept.ptr == nullptr || kept.bytes < bytes || kept.device != device) {
        if (capturing)
            return fail(RFQ_E_UNSUPPORTED, "the call needs %zu bytes of temporary memory and the stream being captured holds %zu: run the call once on this stream before capturing it",
                        bytes, kept.device == device ? kept.bytes : (size_t)0);
        const Kept old = kept;
        kept = Kept{nullptr, 0, device, false};                                       // (whatever fails below, the entry no longer names the old buffer)
        if (old.ptr != nullptr) {
            if (old.captured || old.device != device) ws_retired.push_back(old);      // a graph (or another device's stream) may hold it
            else RFQ_HIP(hipFree(old.ptr));                                           // (waits for the work that uses it)
        }
        RFQ_HIP(hipMalloc(reinterpret_cast<void **>(&kept.ptr), bytes));
        kept.bytes = bytes;
    }
    if (capturing) kept.captured = true;
    *out = kept.ptr;
    return RFQ_OK;
}

// The buffer kept for one stream, before the caller destroys the stream: the handle's entry is erased (a later
// stream that gets the same handle value starts without a buffer).  A buffer a capture used stays allocated.
int release_stream_workspace(hipStream_t s)
{
    std::lock_guard<std::mutex> lock(ws_mutex);
    auto it = ws_kept.find(s);
    if (it == ws_kept.end()) return RFQ_OK;
    const Kept kept = it->second;
    ws_kept.erase(it);
    if (kept.ptr == nullptr) return RFQ_OK;
    if (kept.captured) {
        ws_retired.push_back(kept);
        return RFQ_OK;
    }
    int current = 0;
    RFQ_HIP(hipGetDevice(&current));
    hipError_t e = hipSetDevice(kept.device);
    if (e == hipSuccess) e = hipFree(kept.ptr);                                       // (waits for the work that uses it)
    const hipError_t back = hipSetDevice(current);
    if (e == hipSuccess) e = back;
    if (e != hipSuccess) return hip_fail(e, "rfq_release_stream_temporaries");
    return RFQ_OK;
}

int release_workspaces()
{
    std::lock_guard<std::mutex> lock(ws_mutex);
    if (ws_kept.empty() && ws_retired.empty()) return RFQ_OK;
    RFQ_HIP(hipDeviceSynchronize());
    int current = 0;
    RFQ_HIP(hipGetDevice(&current));
    hipError_t first = hipSuccess;
    for (auto &entry : ws_kept) ws_retired.push_back(entry.second);
    ws_kept.clear();
    for (const Kept &k : ws_retired) {
        if (k.ptr == nullptr) continue;
        hipError_t e = hipSetDevice(k.device);
        if (e == hipSuccess) e = hipFree(k.ptr);
        if (first == hipSuccess) first = e;
    }
    ws_retired.clear();
    hipError_t back = hipSetDevice(current);
    if (first == hipSuccess) first = back;
    if (first != hipSuccess) return hip_fail(first, "rfq_release_temporaries");
    return RFQ_OK;
}

int gemm_f16_k_parts(int m, int n, int k) { return k_parts_for(m, n, k); }

size_t gemm_f16_arranged_bytes(int m, int k)
{
    if (m <= 0 || k <= 0 || k % 8 != 0) return 0;
    return arranged_at_bytes(m, k) + arranged_s2_bytes(m, k);
}

int launch_arrange_a(const void *d_a, int m, int k, uint8_t *d_arranged, hipStream_t s)
{
    if ((reinterpret_cast<uintptr_t>(d_a) & 15u) != 0 || k % 8 != 0)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16_arrange: activations must be 16-byte aligned with k a multiple of 8");
    if ((reinterpret_cast<uintptr_t>(d_arranged) & 15u) != 0)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16_arrange: the arranged buffer must be 16-byte aligned");
    const int tiles32 = (m + 31) / 32, nst = (k + BK - 1) / BK;
    v4u *at = reinterpret_cast<v4u *>(d_arranged);
    _Float16 *s2 = reinterpret_cast<_Float16 *>(d_arranged + arranged_at_bytes(m, k));
    const dim3 grid((unsigned)(tiles32 * ((nst + 3) / 4)));
    if (k % 256 == 0)
        hipLaunchKernelGGL((arrange_a_kernel<true>), grid, dim3(256), 0, s, reinterpret_cast<const _Float16 *>(d_a), at, s2, m, k, tiles32, nst);
    else
        hipLaunchKernelGGL((arrange_a_kernel<false>), grid, dim3(256), 0, s, reinterpret_cast<const _Float16 *>(d_a), at, s2, m, k, tiles32, nst);
    RFQ_LAUNCH_CHECK("arrange_a_kernel");
    return RFQ_OK;
}

int launch_gemm_f16(int fmt, const uint8_t *d_w, const void *d_a, void *d_out, int out_dtype, int m, int n, int k,
                    bool use_static_scratch, const uint8_t *d_arranged, hipStream_t s)
{
    uint8_t *st = nullptr;
    if (use_static_scratch) {
        if (int rc = static_scratch(&st)) return rc;
    }
    if ((out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F16 && (out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F32)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16: out_dtype %d (want RFQ_F32 or RFQ_F16)", out_dtype);
    if (d_arranged != nullptr) {
        if ((reinterpret_cast<uintptr_t>(d_arranged) & 15u) != 0 || k % 8 != 0)
            return fail(RFQ_E_BADARG, "rfq_gemm_f16_arranged: the arranged buffer must be 16-byte aligned with k a multiple of 8");
    } else if ((reinterpret_cast<uintptr_t>(d_a) & 15u) != 0 || k % 8 != 0)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16: activations must be 16-byte aligned with k a multiple of 8");
    if ((reinterpret_cast<uintptr_t>(d_w) & 3u) != 0)               // buffer loads of whole dwords
        return fail(RFQ_E_BADARG, "rfq_gemm_f16: weights must be 4-byte aligned");
    switch (fmt) {
    case RFQ_Q4_0: return launch_fmt<RFQ_Q4_0>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_Q8_0: return launch_fmt<RFQ_Q8_0>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_Q4_K: return launch_fmt<RFQ_Q4_K>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_Q6_K: return launch_fmt<RFQ_Q6_K>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_GGUF_Q4_0: return launch_fmt<RFQ_GGUF_Q4_0>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_GGUF_Q8_0: return launch_fmt<RFQ_GGUF_Q8_0>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_GGUF_Q4_K: return launch_fmt<RFQ_GGUF_Q4_K>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    case RFQ_GGUF_Q6_K: return launch_fmt<RFQ_GGUF_Q6_K>(d_w, d_a, d_out, out_dtype, m, n, k, st, d_arranged, s);
    default: return fail(RFQ_E_UNSUPPORTED, "rfq_gemm_f16: no fp16 matrix-core kernel for format %d", fmt);
    }
}

#endif // RFQ_KQ_PART

} // namespace rfq
