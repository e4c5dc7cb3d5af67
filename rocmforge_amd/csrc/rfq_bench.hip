// Native timing loops for the benchmark driver (see include/rfq_bench.h).
#include "rfq_bench.h"

#include "rfq_common.hpp"

namespace {

template <typename Step>
int timed_loop(int warmup, int steps, void *stream, float *elapsed_ms, Step step)
{
    using namespace rfq;
    if (steps <= 0 || warmup < 0 || !elapsed_ms) return fail(RFQ_E_BADARG, "rfq_bench: bad warmup/steps/elapsed_ms");
    hipStream_t s = (hipStream_t)stream;
    for (int i = 0; i < warmup; i++) {
        int rc = step(i);
        if (rc != RFQ_OK) return rc;
    }
    hipEvent_t e0, e1;
    RFQ_HIP(hipEventCreate(&e0));
    RFQ_HIP(hipEventCreate(&e1));
    RFQ_HIP(hipStreamSynchronize(s));
    RFQ_HIP(hipEventRecord(e0, s));
    int rc = RFQ_OK;
    for (int i = 0; i < steps && rc == RFQ_OK; i++) rc = step(warmup + i);
    hipError_t er = hipEventRecord(e1, s);
    hipError_t es = hipEventSynchronize(e1);
    float ms = 0.f;
    hipError_t et = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != RFQ_OK) return rc;
    if (er != hipSuccess) return hip_fail(er, "hipEventRecord");
    if (es != hipSuccess) return hip_fail(es, "hipEventSynchronize");
    if (et != hipSuccess) return hip_fail(et, "hipEventElapsedTime");
    *elapsed_ms = ms;
    return RFQ_OK;
}

// Reads n16 16-byte words and keeps nothing: thread t takes words t, t + T, t + 2T, ... (T = all threads), D at a
// time in flight.  The store can never happen (a 32-bit fold of arbitrary data equal to a value the host picks at
// random per launch would be needed), but the compiler cannot know that, so the loads stay.
template <bool NT, int D>
__global__ void __launch_bounds__(1024)
read_floor_kernel(const uint8_t *__restrict__ p, size_t n16, uint32_t never, uint32_t *sink)
{
    typedef uint32_t v4_t __attribute__((ext_vector_type(4)));
    const size_t T = (size_t)gridDim.x * blockDim.x, t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const v4_t *w = reinterpret_cast<const v4_t *>(p);
    uint32_t acc = 0;
    for (size_t i = t; i < n16; i += D * T) {
        v4_t v[D];
#pragma unroll
        for (int d = 0; d < D; d++) {
            const size_t j = i + d * T < n16 ? i + d * T : t;       // (past the end: re-read the first word, a cache hit)
            v[d] = NT ? __builtin_nontemporal_load(w + j) : w[j];
        }
#pragma unroll
        for (int d = 0; d < D; d++) acc += (v[d][0] ^ v[d][1]) + (v[d][2] ^ v[d][3]);
    }
    if (acc == never && never != 0) sink[t & 63] = acc;
}

} // namespace

extern "C" {

int rfq_bench_read_floor(const void *const *d_copies, int copies, size_t bytes, int blocks, int threads, int nt, int depth,
                         int warmup, int steps, void *stream, float *elapsed_ms)
{
    if (!d_copies || copies <= 0 || bytes < 16 || blocks <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0 ||
        (depth != 4 && depth != 8 && depth != 16))
        return rfq::fail(RFQ_E_BADARG, "rfq_bench_read_floor: bad arguments");
    static uint32_t *sink = nullptr;                        // 64 words, never written
    if (!sink) RFQ_HIP(hipMalloc(reinterpret_cast<void **>(&sink), 256));
    hipStream_t s = (hipStream_t)stream;
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int i) {
        const uint8_t *p = static_cast<const uint8_t *>(d_copies[i % copies]);
        const uint32_t never = 0x9E3779B9u * (uint32_t)(i + 1) | 1u;
        const dim3 g(blocks), b(threads);
        const size_t n16 = bytes / 16;
        if (nt && depth == 4) hipLaunchKernelGGL((read_floor_kernel<true, 4>), g, b, 0, s, p, n16, never, sink);
        else if (nt && depth == 8) hipLaunchKernelGGL((read_floor_kernel<true, 8>), g, b, 0, s, p, n16, never, sink);
        else if (nt) hipLaunchKernelGGL((read_floor_kernel<true, 16>), g, b, 0, s, p, n16, never, sink);
        else if (depth == 4) hipLaunchKernelGGL((read_floor_kernel<false, 4>), g, b, 0, s, p, n16, never, sink);
        else if (depth == 8) hipLaunchKernelGGL((read_floor_kernel<false, 8>), g, b, 0, s, p, n16, never, sink);
        else hipLaunchKernelGGL((read_floor_kernel<false, 16>), g, b, 0, s, p, n16, never, sink);
        RFQ_LAUNCH_CHECK("read_floor_kernel");
        return (int)RFQ_OK;
    });
}

int rfq_bench_gemv(int fmt, const void *const *d_w_copies, int copies, size_t w_bytes, const float *d_x, float *d_y,
                   int m, int n, int k, int warmup, int steps, void *stream, float *elapsed_ms)
{
    if (!d_w_copies || copies <= 0) return rfq::fail(RFQ_E_BADARG, "rfq_bench_gemv: no weight copies");
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int i) {
        return rfq_gemv(fmt, d_w_copies[i % copies], w_bytes, d_x, d_y, m, n, k, stream);
    });
}

int rfq_bench_dequant(int fmt, const void *const *d_in_copies, int copies, size_t packed_bytes, float *d_out,
                      size_t n_elems, int out_copies, int warmup, int steps, void *stream, float *elapsed_ms)
{
    if (!d_in_copies || copies <= 0 || out_copies <= 0) return rfq::fail(RFQ_E_BADARG, "rfq_bench_dequant: no copies");
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int i) {
        return rfq_dequant(fmt, d_in_copies[i % copies], packed_bytes, d_out + (size_t)(i % out_copies) * n_elems, n_elems, stream);
    });
}

int rfq_bench_get_rows(int fmt, const void *d_table, size_t table_bytes, int n_vocab, int n_embd, const uint32_t *d_tokens,
                       int n_tokens, float *d_out, int out_copies, int warmup, int steps, void *stream, float *elapsed_ms)
{
    if (out_copies <= 0) return rfq::fail(RFQ_E_BADARG, "rfq_bench_get_rows: no output copies");
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int i) {
        return rfq_get_rows(fmt, d_table, table_bytes, n_vocab, n_embd, d_tokens, n_tokens,
                            d_out + (size_t)(i % out_copies) * n_tokens * n_embd, nullptr, stream);
    });
}

int rfq_bench_gemm_f16(int fmt, const void *d_w, size_t w_bytes, const void *d_a_f16, void *d_out, int out_dtype,
                       int m, int n, int k, int warmup, int steps, void *stream, float *elapsed_ms)
{
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int) {
        return rfq_gemm_f16(fmt, d_w, w_bytes, d_a_f16, d_out, out_dtype, m, n, k, stream);
    });
}

int rfq_bench_gemm_f16_arranged(int fmt, const void *d_w, size_t w_bytes, const void *d_arranged, size_t arranged_bytes,
                                void *d_out, int out_dtype, int m, int n, int k, int warmup, int steps, void *stream,
                                float *elapsed_ms)
{
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int) {
        return rfq_gemm_f16_arranged(fmt, d_w, w_bytes, d_arranged, arranged_bytes, d_out, out_dtype, m, n, k, stream);
    });
}

int rfq_bench_gemm_mx(const void *d_a_prep, size_t a_prep_bytes, int a_kind, const void *d_w_prep, size_t w_prep_bytes,
                      int w_kind, void *d_out, int out_dtype, int m, int n, int k, int warmup, int steps, void *stream,
                      float *elapsed_ms)
{
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int) {
        return rfq_gemm_mx(d_a_prep, a_prep_bytes, a_kind, d_w_prep, w_prep_bytes, w_kind, d_out, out_dtype, m, n, k, stream);
    });
}

int rfq_bench_gemm_mx_prefill(const void *d_a_raw, size_t a_raw_bytes, void *d_a_prep, size_t a_prep_bytes,
                              const void *d_w_prep, size_t w_prep_bytes, int w_kind, void *d_out, int out_dtype, int m,
                              int n, int k, int warmup, int steps, void *stream, float *elapsed_ms)
{
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int) {
        int kind = 0;
        int rc = rfq_mx_prepare(RFQ_MXFP4, RFQ_MX_FP4_UNCHECKED, d_a_raw, a_raw_bytes, m, k, d_a_prep, a_prep_bytes, &kind, stream);
        if (rc != RFQ_OK) return rc;
        return rfq_gemm_mx(d_a_prep, a_prep_bytes, kind, d_w_prep, w_prep_bytes, w_kind, d_out, out_dtype, m, n, k, stream);
    });
}

int rfq_bench_mlp_swiglu(int fmt_gate_up, const void *const *d_gate_copies, const void *const *d_up_copies,
                         size_t gate_up_bytes, int fmt_down, const void *const *d_down_copies, size_t down_bytes,
                         int copies, const float *d_x, const float *d_norm_weight, float eps, float *d_out, int m,
                         int hidden_size, int intermediate_size, void *d_scratch, size_t scratch_bytes, int one_call,
                         int warmup, int steps, void *stream, float *elapsed_ms)
{
    if (!d_gate_copies || !d_up_copies || !d_down_copies || copies <= 0)
        return rfq::fail(RFQ_E_BADARG, "rfq_bench_mlp_swiglu: no weight copies");
    if (one_call)
        return timed_loop(warmup, steps, stream, elapsed_ms, [&](int i) {
            const int c = i % copies;
            return rfq_mlp_swiglu(fmt_gate_up, d_gate_copies[c], d_up_copies[c], gate_up_bytes, fmt_down, d_down_copies[c],
                                  down_bytes, d_x, d_norm_weight, eps, d_out, m, hidden_size, intermediate_size, d_scratch,
                                  scratch_bytes, stream);
        });
    // the same arithmetic as five calls of the separate entry points
    const size_t need = rfq_mlp_scratch_bytes(m, hidden_size, intermediate_size);
    if (!d_scratch || scratch_bytes < need) return rfq::fail(RFQ_E_SIZE, "rfq_bench_mlp_swiglu: scratch too small");
    const size_t mi = (((size_t)m * intermediate_size * 4) + 15) & ~(size_t)15;
    const size_t mh = (((size_t)m * hidden_size * 4) + 15) & ~(size_t)15;
    uint8_t *base = static_cast<uint8_t *>(d_scratch);
    float *h = reinterpret_cast<float *>(base), *xn = reinterpret_cast<float *>(base + mi);
    float *gate = reinterpret_cast<float *>(base + mi + mh), *up = reinterpret_cast<float *>(base + 2 * mi + mh);
    return timed_loop(warmup, steps, stream, elapsed_ms, [&](int i) {
        const int c = i % copies;
        const float *xin = d_x;
        int rc = RFQ_OK;
        if (d_norm_weight) {
            rc = rfq_rms_norm(d_x, d_norm_weight, xn, m, hidden_size, eps, stream);
            xin = xn;
        }
        if (rc == RFQ_OK) rc = rfq_gemv(fmt_gate_up, d_gate_copies[c], gate_up_bytes, xin, gate, m, intermediate_size, hidden_size, stream);
        if (rc == RFQ_OK) rc = rfq_gemv(fmt_gate_up, d_up_copies[c], gate_up_bytes, xin, up, m, intermediate_size, hidden_size, stream);
        if (rc == RFQ_OK) rc = rfq_swiglu(gate, up, h, m, intermediate_size, stream);
        if (rc == RFQ_OK) rc = rfq_gemv(fmt_down, d_down_copies[c], down_bytes, h, d_out, m, hidden_size, intermediate_size, stream);
        return rc;
    });
}

} // extern "C"
