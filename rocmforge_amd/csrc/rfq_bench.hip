// Native timing loops for the benchmark driver (see include/rfq_bench.h).
#include "rfq_bench.h"

#include <type_traits>
#include <vector>

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

// What the fp16 matrix pipe delivers, alone and beside the operand traffic of a fused kernel.  Every wavefront runs
// `iters` rounds of NACC independent matrix instructions (VARIANT 0: v_mfma_f32_32x32x16_f16, 8 per round; 1:
// v_mfma_f32_16x16x32_f16, 28 per round); per round it also issues VALU * NACC packed fp16 multiplies (standing for a
// fused kernel's decode work), LDSR 16-byte-per-lane fragment reads from LDS and GLD 16-byte-per-lane loads from a 2 MiB
// window of global memory that all workgroups share (cache hits).  What a round loads feeds the next round's matrix
// instructions, as in a software-pipelined GEMM.  Lane 0 of every wavefront records the shader clock (s_memtime) and
// the constant 100 MHz clock (s_memrealtime) around its loop.  The kernel's LDS request keeps it to one workgroup per CU.
typedef _Float16 probe_v8h __attribute__((ext_vector_type(8)));
typedef _Float16 probe_v2h __attribute__((ext_vector_type(2)));
typedef float probe_v16f __attribute__((ext_vector_type(16)));
typedef float probe_v4f __attribute__((ext_vector_type(4)));
constexpr int PROBE_LDS_BYTES = 96 * 1024, PROBE_WINDOW_BYTES = 2 << 20;

template <int VARIANT, int VALU, int LDSR, int GLD>
__global__ void __launch_bounds__(512)
mfma_f16_probe_kernel(const probe_v8h *__restrict__ in, const probe_v8h *__restrict__ window, float *__restrict__ out,
                      unsigned long long *__restrict__ clocks, int iters)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t probe_lds[];
    constexpr int NACC = VARIANT == 0 ? 8 : 28, NA = GLD > 0 ? GLD : 1, NB = LDSR > 0 ? LDSR : 1;
    typedef typename std::conditional<VARIANT == 0, probe_v16f, probe_v4f>::type Acc;
    constexpr int NR = VARIANT == 0 ? 16 : 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    probe_v8h *lds = reinterpret_cast<probe_v8h *>(probe_lds);
    for (int i = threadIdx.x; i < 64 * 1024 / 16; i += blockDim.x) lds[i] = in[i & 1023];
    __syncthreads();
    probe_v8h a[2][NA], b[2][NB];
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int g = 0; g < NA; g++) a[h][g] = in[(threadIdx.x + 64 * g) & 1023];
#pragma unroll
        for (int r = 0; r < NB; r++) b[h][r] = in[(512 + threadIdx.x + 64 * r) & 1023];
    }
    probe_v2h t[4];
#pragma unroll
    for (int q = 0; q < 4; q++) t[q] = probe_v2h{a[0][0][2 * q], b[0][0][2 * q + 1]};
    const probe_v2h one = {in[1023][0], in[1023][1]};                 // 1.0 from memory: a constant would be folded away
    Acc acc[NACC];
#pragma unroll
    for (int q = 0; q < NACC; q++)
#pragma unroll
        for (int r = 0; r < NR; r++) acc[q][r] = 0.0f;
    auto round = [&](int it, int cur) __attribute__((always_inline)) {
        const int nxt = cur ^ 1;
#pragma unroll
        for (int g = 0; g < GLD; g++)
            a[nxt][g] = window[((((it * GLD + g) * 8 + wave) * 64) & (PROBE_WINDOW_BYTES / 16 - 1)) + lane];
#pragma unroll
        for (int r = 0; r < LDSR; r++) b[nxt][r] = lds[((((it * LDSR + r) * 8 + wave) * 64) & (64 * 1024 / 16 - 1)) + lane];
#pragma unroll
        for (int q = 0; q < NACC; q++) {
            if constexpr (VARIANT == 0) acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[cur][q % NA], b[cur][q % NB], acc[q], 0, 0, 0);
            else acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[cur][q % NA], b[cur][q % NB], acc[q], 0, 0, 0);
#pragma unroll
            for (int v = 0; v < VALU; v++) t[(q + v) & 3] = t[(q + v) & 3] * one;
        }
    };
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; it += 2) {
        round(it, 0);
        round(it + 1, 1);
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    float s = 0.0f;
#pragma unroll
    for (int q = 0; q < NACC; q++)
#pragma unroll
        for (int r = 0; r < NR; r++) s += acc[q][r];
#pragma unroll
    for (int q = 0; q < 4; q++) s += (float)t[q][0] + (float)t[q][1];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (lane == 0) {
        const size_t w = (size_t)blockIdx.x * (blockDim.x / 64) + wave;
        clocks[2 * w] = c1 - c0;
        clocks[2 * w + 1] = r1 - r0;
    }
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

int rfq_bench_gemv_timeline(int fmt, const void *const *d_w_copies, int copies, size_t w_bytes, const float *d_x,
                            float *d_y, int n, int k, int warmup, void *stream, unsigned long long *d_trace,
                            size_t capacity_waves, int *waves, int *stamps_per_wave)
{
    if (!d_w_copies || copies <= 0 || !d_trace || !waves || !stamps_per_wave)
        return rfq::fail(RFQ_E_BADARG, "rfq_bench_gemv_timeline: null argument");
    *stamps_per_wave = rfq::GEMV_TRACE_STAMPS;
    if (warmup < 1) warmup = 1;                          // (an ordinary call first: it checks the arguments)
    for (int i = 0; i < warmup; i++) {
        const int rc = rfq_gemv(fmt, d_w_copies[i % copies], w_bytes, d_x, d_y, 1, n, k, stream);
        if (rc != RFQ_OK) return rc;
    }
    const int rc = rfq::launch_gemv_traced(fmt, (const uint8_t *)d_w_copies[warmup % copies], d_x, d_y, n, k, d_trace, capacity_waves,
                                           waves, (hipStream_t)stream);
    if (rc != RFQ_OK) return rc;
    const hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    return e == hipSuccess ? RFQ_OK : rfq::hip_fail(e, "rfq_bench_gemv_timeline: hipStreamSynchronize");
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

int rfq_bench_mfma_f16_probe(int variant, int valu_per_mfma, int lds_reads_per_round, int global_loads_per_round,
                             int workgroups, int waves_per_workgroup, int random_operands, int iters, int launches,
                             void *stream, float *last_launch_us, float *clocks_per_mfma, float *shader_ghz, float *tflops)
{
    using namespace rfq;
    if ((variant != 0 && variant != 1) || workgroups <= 0 || workgroups > 4096 ||
        (waves_per_workgroup != 4 && waves_per_workgroup != 8) || iters <= 0 || iters % 2 != 0 || launches <= 0 ||
        !last_launch_us || !clocks_per_mfma || !shader_ghz || !tflops)
        return fail(RFQ_E_BADARG, "rfq_bench_mfma_f16_probe: bad arguments");
    hipStream_t s = (hipStream_t)stream;
    const int threads = 64 * waves_per_workgroup, waves = workgroups * waves_per_workgroup;
    const int nacc = variant == 0 ? 8 : 28;
    std::vector<uint16_t> host(PROBE_WINDOW_BYTES / 2);
    uint32_t lcg = 12345u;
    for (auto &h : host) {
        lcg = lcg * 1664525u + 1013904223u;
        // random fp16 values of magnitude 2^-4 .. 2 with random mantissas and signs, or all zero
        h = random_operands ? (uint16_t)(((lcg >> 16) & 0x83FFu) | ((11u + ((lcg >> 8) % 5u)) << 10)) : (uint16_t)0;
    }
    std::vector<uint16_t> first(host.begin(), host.begin() + 1024 * 8);
    first[1023 * 8] = first[1023 * 8 + 1] = 0x3C00;
    void *d_in = nullptr, *d_win = nullptr, *d_out = nullptr, *d_clk = nullptr;
    RFQ_HIP(hipMalloc(&d_in, first.size() * 2));
    RFQ_HIP(hipMalloc(&d_win, host.size() * 2));
    RFQ_HIP(hipMalloc(&d_out, (size_t)workgroups * threads * 4));
    RFQ_HIP(hipMalloc(&d_clk, (size_t)waves * 16));
    RFQ_HIP(hipMemcpy(d_in, first.data(), first.size() * 2, hipMemcpyHostToDevice));
    RFQ_HIP(hipMemcpy(d_win, host.data(), host.size() * 2, hipMemcpyHostToDevice));
    const void *fn = nullptr;
#define RFQ_PROBE_CASE(V, VA, L, G) \
    if (variant == V && valu_per_mfma == VA && lds_reads_per_round == L && global_loads_per_round == G) \
        fn = reinterpret_cast<const void *>(&mfma_f16_probe_kernel<V, VA, L, G>);
    RFQ_PROBE_CASE(0, 0, 0, 0) RFQ_PROBE_CASE(0, 2, 0, 0) RFQ_PROBE_CASE(0, 4, 0, 0) RFQ_PROBE_CASE(0, 0, 4, 0)
    RFQ_PROBE_CASE(0, 0, 8, 0) RFQ_PROBE_CASE(0, 0, 0, 2) RFQ_PROBE_CASE(0, 0, 0, 4) RFQ_PROBE_CASE(0, 0, 4, 2)
    RFQ_PROBE_CASE(0, 3, 4, 2) RFQ_PROBE_CASE(0, 2, 4, 2) RFQ_PROBE_CASE(0, 3, 6, 0)
    RFQ_PROBE_CASE(1, 0, 0, 0) RFQ_PROBE_CASE(1, 2, 0, 0) RFQ_PROBE_CASE(1, 1, 0, 0) RFQ_PROBE_CASE(1, 0, 7, 4) RFQ_PROBE_CASE(1, 1, 7, 4)
    RFQ_PROBE_CASE(1, 2, 7, 4) RFQ_PROBE_CASE(1, 0, 7, 0) RFQ_PROBE_CASE(1, 0, 0, 4)
#undef RFQ_PROBE_CASE
    if (!fn) return fail(RFQ_E_UNSUPPORTED, "rfq_bench_mfma_f16_probe: combination not compiled");
    RFQ_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, PROBE_LDS_BYTES));
    hipEvent_t e0, e1;
    RFQ_HIP(hipEventCreate(&e0));
    RFQ_HIP(hipEventCreate(&e1));
    const void *in = d_in, *win = d_win;
    float *out = static_cast<float *>(d_out);
    unsigned long long *clk = static_cast<unsigned long long *>(d_clk);
    void *args[] = {(void *)&in, (void *)&win, (void *)&out, (void *)&clk, (void *)&iters};
    for (int i = 0; i < launches; i++) {
        if (i == launches - 1) RFQ_HIP(hipEventRecord(e0, s));
        RFQ_HIP(hipLaunchKernel(fn, dim3(workgroups), dim3(threads), args, PROBE_LDS_BYTES, s));
    }
    RFQ_HIP(hipEventRecord(e1, s));
    RFQ_HIP(hipEventSynchronize(e1));
    float ms = 0.0f;
    RFQ_HIP(hipEventElapsedTime(&ms, e0, e1));
    std::vector<unsigned long long> ticks((size_t)waves * 2);
    RFQ_HIP(hipMemcpy(ticks.data(), d_clk, ticks.size() * 8, hipMemcpyDeviceToHost));
    double core = 0.0, real = 0.0;
    for (int w = 0; w < waves; w++) {
        core += (double)ticks[2 * w];
        real += (double)ticks[2 * w + 1];
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(d_in);
    (void)hipFree(d_win);
    (void)hipFree(d_out);
    (void)hipFree(d_clk);
    const double per_wave = (double)iters * nacc;
    *last_launch_us = ms * 1000.0f;
    // clocks per matrix instruction and SIMD: a SIMD's wavefronts share its matrix pipe
    *clocks_per_mfma = (float)(core / waves / per_wave / (waves_per_workgroup / 4));
    *shader_ghz = real > 0.0 ? (float)(core / real * 0.1) : 0.0f;               // the constant clock ticks at 100 MHz
    *tflops = (float)(per_wave * waves * (variant == 0 ? 32768.0 : 16384.0) / (ms * 1e-3) / 1e12);
    return RFQ_OK;
}

} // extern "C"
