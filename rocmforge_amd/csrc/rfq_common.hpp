// Shared declarations for librfq (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "rfq.h"

namespace rfq {

// ---- format traits ---------------------------------------------------------
template <int FMT> struct Fmt;
template <> struct Fmt<RFQ_Q4_0> { static constexpr int BE = 32, BB = 20; };
template <> struct Fmt<RFQ_Q8_0> { static constexpr int BE = 32, BB = 36; };
template <> struct Fmt<RFQ_Q4_K> { static constexpr int BE = 256, BB = 256; };
template <> struct Fmt<RFQ_Q6_K> { static constexpr int BE = 256, BB = 256; };
template <> struct Fmt<RFQ_Q2_K> { static constexpr int BE = 256, BB = 256; };
template <> struct Fmt<RFQ_Q3_K> { static constexpr int BE = 256, BB = 256; };
template <> struct Fmt<RFQ_Q5_K> { static constexpr int BE = 256, BB = 256; };
template <> struct Fmt<RFQ_MXFP4> { static constexpr int BE = 32, BB = 17; };
template <> struct Fmt<RFQ_MXFP6_E2M3> { static constexpr int BE = 32, BB = 25; };
template <> struct Fmt<RFQ_GGUF_Q4_0> { static constexpr int BE = 32, BB = 18; };
template <> struct Fmt<RFQ_GGUF_Q8_0> { static constexpr int BE = 32, BB = 34; };
template <> struct Fmt<RFQ_GGUF_Q4_K> { static constexpr int BE = 256, BB = 144; };
template <> struct Fmt<RFQ_GGUF_Q6_K> { static constexpr int BE = 256, BB = 210; };
template <> struct Fmt<RFQ_MM_Q8_0> { static constexpr int BE = 32, BB = 36; };
template <> struct Fmt<RFQ_MM_Q4_K> { static constexpr int BE = 256, BB = 256; };
template <> struct Fmt<RFQ_MM_Q6_K> { static constexpr int BE = 256, BB = 256; };

// MXFP6_E3M2 is decoded exactly like E2M3 by the reference
// (src/loader/dequant.rs:693), so it shares every kernel.
inline int canonical_format(int fmt) { return fmt == RFQ_MXFP6_E3M2 ? RFQ_MXFP6_E2M3 : fmt; }

inline int fmt_block_elems(int fmt)
{
    switch (fmt) {
    case RFQ_Q4_0: case RFQ_Q8_0: case RFQ_MXFP4: case RFQ_MXFP6_E2M3: case RFQ_MXFP6_E3M2: return 32;
    case RFQ_GGUF_Q4_0: case RFQ_GGUF_Q8_0: case RFQ_MM_Q8_0: return 32;
    case RFQ_Q4_K: case RFQ_Q6_K: case RFQ_GGUF_Q4_K: case RFQ_GGUF_Q6_K: case RFQ_MM_Q4_K: case RFQ_MM_Q6_K: return 256;
    case RFQ_Q2_K: case RFQ_Q3_K: case RFQ_Q5_K: return 256;
    default: return 0;
    }
}
// The loader's other K types (src/loader/dequant.rs:150-420): decoded by rfq_dequant*, on no matmul path.
inline bool fmt_dequant_only(int fmt) { return fmt == RFQ_Q2_K || fmt == RFQ_Q3_K || fmt == RFQ_Q5_K; }
// The matmul module's own decoders (src/kernels/matmul/quantized/): dequantisation and the two GEMV orientations.
inline bool fmt_mm_variant(int fmt) { return fmt == RFQ_MM_Q8_0 || fmt == RFQ_MM_Q4_K || fmt == RFQ_MM_Q6_K; }
inline int fmt_block_bytes(int fmt)
{
    switch (fmt) {
    case RFQ_Q4_0: return 20;
    case RFQ_Q8_0: case RFQ_MM_Q8_0: return 36;
    case RFQ_Q4_K: case RFQ_Q6_K: case RFQ_Q2_K: case RFQ_Q3_K: case RFQ_Q5_K: case RFQ_MM_Q4_K: case RFQ_MM_Q6_K: return 256;
    case RFQ_MXFP4: return 17;
    case RFQ_MXFP6_E2M3: case RFQ_MXFP6_E3M2: return 25;
    case RFQ_GGUF_Q4_0: return 18;
    case RFQ_GGUF_Q8_0: return 34;
    case RFQ_GGUF_Q4_K: return 144;
    case RFQ_GGUF_Q6_K: return 210;
    default: return 0;
    }
}

// ---- error plumbing (rfq_api.hip) ------------------------------------------
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);
#define RFQ_HIP(call)                                              \
    do {                                                           \
        hipError_t e_ = (call);                                    \
        if (e_ != hipSuccess) return ::rfq::hip_fail(e_, #call);   \
    } while (0)
// Kernel launches report through hipGetLastError.
#define RFQ_LAUNCH_CHECK(what)                                     \
    do {                                                           \
        hipError_t e_ = hipGetLastError();                         \
        if (e_ != hipSuccess) return ::rfq::hip_fail(e_, what);    \
    } while (0)

int device_cu_count();
// Temporary device memory for one call on stream s: a buffer the library keeps
// per stream for modest sizes (*transient = false: leave it alone), a
// stream-ordered allocation the caller releases with hipFreeAsync otherwise.
int workspace(hipStream_t s, size_t bytes, uint8_t **out, bool *transient);
int release_workspaces();
int release_stream_workspace(hipStream_t s);
// Host bytes -> device memory through the per-device ring of pinned slots (rfq_upload.hip).
int upload_bytes(const void *h_src, size_t bytes, void *d_dst, hipStream_t s);
int release_upload_rings();

// ---- launchers implemented per .hip file -----------------------------------
int launch_dequant(int fmt, const uint8_t *d_in, size_t in_bytes, float *d_out, size_t n, hipStream_t s);
int launch_get_rows(int fmt, const void *d_table, int n_vocab, int n_embd, const uint32_t *d_tokens, int n_tokens,
                    float *d_out, int *d_status, hipStream_t s);
// src_fmt: RFQ_TABLE_F32 for f32 rows, else a packed format whose rows are decoded on the fly.
int launch_rms_norm(int src_fmt, const void *d_x, const float *d_weight, float *d_out, int rows, int hidden, float eps,
                    hipStream_t s);
int launch_swiglu(const float *d_gate, const float *d_up, float *d_out, size_t total, hipStream_t s);
int launch_gemv(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int m, int n, int k, hipStream_t s);
// rfq_gemv.hip is compiled in four parts (the kernels of some formats each; part 0 also holds launch_gemv and
// launch_gemv_fused, which hand a call to its format's part).  `fuse` points at the part-internal GemvFuse.
struct GemvLastKernel { const char *name; int fmt, a, b, c; };
extern thread_local GemvLastKernel g_gemv_last_kernel;   // which kernel this thread's last GEMV launch took
struct GemvTraceRequest { unsigned long long *d_buf; size_t capacity_waves; int waves_written; };
extern thread_local GemvTraceRequest g_gemv_trace_request;   // set around a launch that is to stamp its timeline
#define RFQ_GEMV_PART_DECL(N)                                                                                                 \
    int launch_gemv_part##N(int canonical, const uint8_t *d_w, const float *d_x, float *d_y, int m, int n, int k, hipStream_t s); \
    int launch_gemv_fused_part##N(int canonical, const uint8_t *d_w, const float *d_x, float *d_y, int rows, int k,          \
                                  const void *fuse, hipStream_t s);
RFQ_GEMV_PART_DECL(0)
RFQ_GEMV_PART_DECL(1)
RFQ_GEMV_PART_DECL(2)
RFQ_GEMV_PART_DECL(3)
#undef RFQ_GEMV_PART_DECL
constexpr int GEMV_TRACE_STAMPS = 20;                    // readings per wavefront, see WaveTrace in rfq_gemv.hip
int launch_gemv_traced(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int n, int k, unsigned long long *d_trace,
                       size_t capacity_waves, int *waves, hipStream_t s);
// y[n] = sum_l x[l] * Wd[l * n + j] over the flat stream of n * k elements (one row of x).
int launch_gemv_kn(int fmt, const uint8_t *d_w, const float *d_x, float *d_y, int n, int k, hipStream_t s);
int launch_gemv_fused(int fmt, const uint8_t *d_w, const uint8_t *d_w2, const float *d_x, const float *d_norm_w,
                      float eps, float *d_y, int n, int k, hipStream_t s);
// use_static_scratch: the temporaries live in the library's static device array instead of workspace().
size_t gemm_f16_arranged_bytes(int m, int k);
int gemm_f16_k_parts(int m, int n, int k);
int launch_arrange_a(const void *d_a, int m, int k, uint8_t *d_arranged, hipStream_t s);
// d_arranged != nullptr: activations already in operand order (launch_arrange_a); d_a is not read.
int launch_gemm_f16(int fmt, const uint8_t *d_w, const void *d_a, void *d_out, int out_dtype, int m, int n,
                    int k, bool use_static_scratch, const uint8_t *d_arranged, hipStream_t s);
size_t mx_prepared_bytes(int fmt, int kind, int rows, int k);
int launch_mx_prepare(int fmt, int kind_req, const uint8_t *d_raw, int rows, int k, void *d_prep,
                      size_t prep_bytes, int *kind_out, hipStream_t s);
int launch_gemm_mx(const void *d_a, int a_kind, const void *d_w, int w_kind, void *d_out, int out_dtype, int m,
                   int n, int k, hipStream_t s);

#if defined(__HIPCC__)
// ---- device-side decode helpers ---------------------------------------------

// Loads that make no alignment promise (gfx950 global memory accepts any
// byte address for dword..dwordx4 accesses).
template <typename T> __device__ __forceinline__ T ld(const uint8_t *p)
{
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

// The same with the non-temporal hint, for the nibble bytes of the 256-byte Q4_K layouts: a lane takes 16 of every 28
// (or 20) bytes there in ONE load, the rest of the line is never wanted, and keeping such lines out of the caches
// leaves them to what is reused -- x, the block headers neighbouring lanes share (Q4_K 14336 x 4096 GEMV: 11.33 ->
// 10.84 us, 128256 x 4096: 93.4 -> 82.6 us; with the hint on the 2-byte scale and 1-byte min loads as well the gain
// is gone).  Not for layouts whose cache lines are consumed by two load instructions of a lane or by neighbouring
// lanes in turn -- there the second access finds the line gone: measured with the hint, Q6_K 13.9 -> 16.4 us,
// GGUF_Q4_K 8.0 -> 9.1 us, GGUF_Q8_0 6.1 -> 6.5 us; Q4_0 and Q8_0 no change.
template <typename T> __device__ __forceinline__ T ld_once(const uint8_t *p)
{
    static_assert(sizeof(T) % 4 == 0, "whole dwords");
    constexpr int N = sizeof(T) / 4;
    typedef uint32_t v4_t __attribute__((ext_vector_type(4), aligned(1)));
    typedef uint32_t v2_t __attribute__((ext_vector_type(2), aligned(1)));
    typedef uint32_t v1_t __attribute__((aligned(1)));
    uint32_t w[N];
    int i = 0;
#pragma unroll
    for (; i + 4 <= N; i += 4) {
        const v4_t v = __builtin_nontemporal_load(reinterpret_cast<const v4_t *>(p + 4 * i));
        w[i] = v[0]; w[i + 1] = v[1]; w[i + 2] = v[2]; w[i + 3] = v[3];
    }
    if (i + 2 <= N) {
        const v2_t v = __builtin_nontemporal_load(reinterpret_cast<const v2_t *>(p + 4 * i));
        w[i] = v[0]; w[i + 1] = v[1];
        i += 2;
    }
    if (i < N) w[i] = __builtin_nontemporal_load(reinterpret_cast<const v1_t *>(p + 4 * i));
    T out;
    __builtin_memcpy(&out, w, sizeof(T));
    return out;
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h)
{
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v; // exact widening, subnormals kept
}

// 2^e for the MXFP exponent byte read as i8, reproducing f32::powi(2.0, e):
// exact for -127..127 (2^-127 is subnormal), 0.0 for -128 (the repeated
// squaring overflows and the reciprocal of +inf is taken).
__device__ __forceinline__ float mx_scale(int e)
{
    uint32_t bits = e >= -126 ? (uint32_t)(e + 127) << 23 : (e == -127 ? 0x00400000u : 0u);
    return __uint_as_float(bits);
}

// MxfpBlock::decode_e2m1 (src/loader/mxfp.rs:234-244): 0 for code 0, otherwise
// sign * (1 + mant) * 2^(exp-1)  ==  +-2^(((code&7)+1)/2 - 1).
__device__ __forceinline__ float decode_e2m1(uint32_t q)
{
    uint32_t c = q & 7u;
    uint32_t bits = ((q & 8u) << 28) | ((126u + ((c + 1u) >> 1)) << 23);
    return q == 0u ? 0.0f : __uint_as_float(bits);
}

// MxfpBlock::decode_e2m3 (src/loader/mxfp.rs:283-293): 0 for code 0, otherwise
// sign * (1 + mant/8) * 2^(exp-1); the fields map straight onto an f32.
__device__ __forceinline__ float decode_e2m3(uint32_t q)
{
    uint32_t bits = ((q & 32u) << 26) | ((126u + ((q >> 3) & 3u)) << 23) | ((q & 7u) << 20);
    return q == 0u ? 0.0f : __uint_as_float(bits);
}

// f32::clamp for finite bounds.
__device__ __forceinline__ float clampf(float v, float lo, float hi) { return fminf(fmaxf(v, lo), hi); }

// get_scale_min_k4 of ggml-quants.c: 6-bit scale (low 8 bits of the result) and
// min (bits 8..15) number j of the 8 packed into 12 bytes, given as 3 dwords.
// Worked out for the pair (2c, 2c+1), c = j >> 1, as two bytes at a time, so that
// the two sub-blocks of a 64-element chunk share everything but the last shift.
__device__ __forceinline__ uint32_t gguf_scale_min_k4(int j, uint32_t s0, uint32_t s1, uint32_t s2)
{
    const int c = j >> 1, sh = 16 * (c & 1);
    const uint32_t a = (s0 >> sh) & 0xFFFFu, b = (s1 >> sh) & 0xFFFFu, cc = (s2 >> sh) & 0xFFFFu;
    // j < 4: sc = a & 63, m = b & 63;  j >= 4: sc = (cc & 15) | ((a >> 6) << 4), m = (cc >> 4) | ((b >> 6) << 4)
    const uint32_t sc2 = c < 2 ? (a & 0x3F3Fu) : ((cc & 0x0F0Fu) | ((a >> 2) & 0x3030u));
    const uint32_t mn2 = c < 2 ? (b & 0x3F3Fu) : (((cc >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u));
    const int hs = 8 * (j & 1);
    return ((sc2 >> hs) & 255u) | (((mn2 >> hs) & 255u) << 8);
}

// f16_to_f32_cpu of the matmul module (src/kernels/matmul/quantized/common.rs:44-60).  Its mantissa term is
// `((bits & 0x03FF) << 13) as u32` on a u16: the shift is done in 16 bits, so only mantissa bits 0..2 survive
// (as bits 13..15); its test for zero and subnormals compares the already re-biased exponent with 0 and never
// holds.  Every pattern widens as sign | (field + 112) << 23 | (bits & 7) << 13.
__device__ __forceinline__ float f16_bits_to_f32_mm(uint16_t h)
{
    const uint32_t b = h;
    return __uint_as_float(((b & 0x8000u) << 16) | ((((b >> 10) & 31u) + 112u) << 23) | ((b & 7u) << 13));
}

// Signed 6-bit field (two's complement) starting at bit `off` of w.
__device__ __forceinline__ int sbfe6(uint32_t w, uint32_t off) { return ((int)(w << (26u - off))) >> 26; }
#endif

} // namespace rfq
