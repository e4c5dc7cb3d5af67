// C ABI entry points of librfq: argument validation on the host, then one
// launcher per operation.  No kernel is launched before its operand sizes have
// been checked against what the kernel and its grid assume.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "rfq_common.hpp"

namespace rfq {

static thread_local char g_err[512] = "";

int fail(int status, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t e, const char *what)
{
    snprintf(g_err, sizeof g_err, "%s: %s", what, hipGetErrorString(e));
    return e == hipErrorOutOfMemory ? RFQ_E_NOMEM : RFQ_E_HIP;
}

int device_cu_count()
{
    // One value per device id; devices are few, so a small fixed table.
    static int cus[64];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cus[dev] = v;
    }
    return cus[dev];
}

static bool known_format(int fmt) { return fmt_block_elems(fmt) != 0; }

// Weight bytes of an [n, k] matrix, or 0 if k does not divide into blocks.
static size_t matrix_bytes(int fmt, int n, int k)
{
    int be = fmt_block_elems(fmt);
    if (be == 0 || k % be != 0) return 0;
    return (size_t)n * (size_t)(k / be) * (size_t)fmt_block_bytes(fmt);
}

static int check_gemv(const char *who, int fmt, const void *w, size_t w_bytes, bool have_bytes, const void *x,
                      const void *y, int m, int n, int k, bool mm_ok = false)
{
    if (!known_format(fmt)) return fail(RFQ_E_BADARG, "%s: unknown format %d", who, fmt);
    if (fmt_dequant_only(fmt)) return fail(RFQ_E_UNSUPPORTED, "%s: format %d is decoded by rfq_dequant only", who, fmt);
    if (fmt_mm_variant(fmt) && !mm_ok)
        return fail(RFQ_E_UNSUPPORTED, "%s: format %d (a decoder of the matmul module) is taken by rfq_dequant*, rfq_gemv, rfq_gemv_kn and rfq_matmul_host_weights* only", who, fmt);
    if (!w || !x || !y) return fail(RFQ_E_BADARG, "%s: null pointer", who);
    if (m <= 0 || n <= 0 || k <= 0)
        return fail(RFQ_E_BADARG, "%s: dimensions must be positive (m=%d n=%d k=%d)", who, m, n, k);
    size_t need = matrix_bytes(fmt, n, k);
    if (need == 0)
        return fail(RFQ_E_SIZE, "%s: k=%d is not a multiple of the %d-element block", who, k, fmt_block_elems(fmt));
    if (have_bytes && w_bytes != need)
        return fail(RFQ_E_SIZE, "%s: weight buffer has %zu bytes, [%d x %d] needs %zu", who, w_bytes, n, k, need);
    return RFQ_OK;
}

} // namespace rfq

using namespace rfq;

extern "C" {

int rfq_version(void) { return RFQ_VERSION; }

const char *rfq_last_error(void) { return g_err; }

int rfq_release_temporaries(void)
{
    int rc = rfq::release_workspaces();
    int rc2 = rfq::release_upload_rings();
    return rc != RFQ_OK ? rc : rc2;
}

int rfq_release_stream_temporaries(void *stream) { return rfq::release_stream_workspace((hipStream_t)stream); }

int rfq_upload(const void *h_src, size_t bytes, void *d_dst, void *stream)
{
    if (bytes == 0) return RFQ_OK;
    if (!h_src || !d_dst) return fail(RFQ_E_BADARG, "rfq_upload: null pointer");
    return upload_bytes(h_src, bytes, d_dst, (hipStream_t)stream);
}

size_t rfq_block_elems(int fmt) { return (size_t)fmt_block_elems(fmt); }
size_t rfq_block_bytes(int fmt) { return (size_t)fmt_block_bytes(fmt); }

size_t rfq_packed_bytes(int fmt, size_t n_elems)
{
    size_t be = (size_t)fmt_block_elems(fmt);
    if (be == 0) return 0;
    return ((n_elems + be - 1) / be) * (size_t)fmt_block_bytes(fmt);
}

int rfq_dequant(int fmt, const void *d_packed, size_t packed_bytes, float *d_out, size_t n_elems, void *stream)
{
    if (!known_format(fmt)) return fail(RFQ_E_BADARG, "rfq_dequant: unknown format %d", fmt);
    if (n_elems == 0) return RFQ_OK;
    if (!d_out) return fail(RFQ_E_BADARG, "rfq_dequant: null output");
    if (!d_packed && packed_bytes) return fail(RFQ_E_BADARG, "rfq_dequant: null input with %zu bytes", packed_bytes);
    return launch_dequant(fmt, (const uint8_t *)d_packed, packed_bytes, d_out, n_elems, (hipStream_t)stream);
}

int rfq_get_rows(int fmt, const void *d_table, size_t table_bytes, int n_vocab, int n_embd, const uint32_t *d_tokens,
                 int n_tokens, float *d_out, int *d_status, void *stream)
{
    const bool f32 = fmt == RFQ_TABLE_F32;
    if (!f32 && !known_format(fmt)) return fail(RFQ_E_BADARG, "rfq_get_rows: unknown format %d", fmt);
    if (fmt_dequant_only(fmt) || fmt_mm_variant(fmt))
        return fail(RFQ_E_UNSUPPORTED, "rfq_get_rows: format %d is decoded by rfq_dequant only", fmt);
    if (n_vocab <= 0 || n_embd <= 0 || n_tokens < 0)
        return fail(RFQ_E_BADARG, "rfq_get_rows: n_vocab=%d n_embd=%d n_tokens=%d", n_vocab, n_embd, n_tokens);
    const int be = f32 ? 4 : fmt_block_elems(fmt);
    if (n_embd % be != 0) return fail(RFQ_E_SIZE, "rfq_get_rows: n_embd=%d is not a multiple of %d", n_embd, be);
    const size_t need = f32 ? (size_t)n_vocab * n_embd * 4 : (size_t)n_vocab * (n_embd / be) * fmt_block_bytes(fmt);
    if (table_bytes != need)
        return fail(RFQ_E_SIZE, "rfq_get_rows: table has %zu bytes, a %d x %d table needs %zu", table_bytes, n_vocab,
                    n_embd, need);
    if (n_tokens == 0) return RFQ_OK;
    if (!d_table || !d_tokens || !d_out) return fail(RFQ_E_BADARG, "rfq_get_rows: null pointer");
    if ((reinterpret_cast<uintptr_t>(d_out) & 15u) != 0 || (f32 && (reinterpret_cast<uintptr_t>(d_table) & 15u) != 0))
        return fail(RFQ_E_BADARG, "rfq_get_rows: output (and an f32 table) must be 16-byte aligned");
    return launch_get_rows(fmt, d_table, n_vocab, n_embd, d_tokens, n_tokens, d_out, d_status, (hipStream_t)stream);
}

int rfq_dequant_upload(int fmt, const uint8_t *h_packed, size_t packed_bytes, float *d_out, size_t n_elems,
                       void *stream)
{
    if (!known_format(fmt)) return fail(RFQ_E_BADARG, "rfq_dequant_upload: unknown format %d", fmt);
    if (n_elems == 0) return RFQ_OK;
    if (!d_out) return fail(RFQ_E_BADARG, "rfq_dequant_upload: null output");
    if (!h_packed && packed_bytes) return fail(RFQ_E_BADARG, "rfq_dequant_upload: null input");
    hipStream_t s = (hipStream_t)stream;
    // Only the bytes the decoder can reach are uploaded.
    size_t need = rfq_packed_bytes(fmt, n_elems);
    size_t bytes = packed_bytes < need ? packed_bytes : need;
    void *d_in = nullptr;
    if (bytes) {
        RFQ_HIP(hipMalloc(&d_in, bytes));
        if (int up = upload_bytes(h_packed, bytes, d_in, s)) { (void)hipStreamSynchronize(s); (void)hipFree(d_in); return up; }
    }
    int rc = launch_dequant(fmt, (const uint8_t *)d_in, bytes, d_out, n_elems, s);
    hipError_t e = hipStreamSynchronize(s);
    if (d_in) (void)hipFree(d_in);
    if (rc != RFQ_OK) return rc;
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return RFQ_OK;
}

int rfq_dequant_host(int fmt, const uint8_t *h_packed, size_t packed_bytes, float *h_out, size_t n_elems)
{
    if (!known_format(fmt)) return fail(RFQ_E_BADARG, "rfq_dequant_host: unknown format %d", fmt);
    if (n_elems == 0) return RFQ_OK;
    if (!h_out) return fail(RFQ_E_BADARG, "rfq_dequant_host: null output");
    float *d_out = nullptr;
    RFQ_HIP(hipMalloc((void **)&d_out, n_elems * sizeof(float)));
    int rc = rfq_dequant_upload(fmt, h_packed, packed_bytes, d_out, n_elems, nullptr);
    if (rc == RFQ_OK) {
        hipError_t e = hipMemcpy(h_out, d_out, n_elems * sizeof(float), hipMemcpyDeviceToHost);
        if (e != hipSuccess) rc = hip_fail(e, "hipMemcpy(D2H)");
    }
    (void)hipFree(d_out);
    return rc;
}

int rfq_gemv(int fmt, const void *d_w, size_t w_bytes, const float *d_x, float *d_y, int m, int n, int k,
             void *stream)
{
    int rc = check_gemv("rfq_gemv", fmt, d_w, w_bytes, true, d_x, d_y, m, n, k, true);
    if (rc != RFQ_OK) return rc;
    for (int r0 = 0; r0 < m; r0 += 8) {                 // the decode kernels take up to eight rows of x per launch
        const int rows = m - r0 < 8 ? m - r0 : 8;
        rc = launch_gemv(fmt, (const uint8_t *)d_w, d_x + (size_t)r0 * k, d_y + (size_t)r0 * n, rows, n, k, (hipStream_t)stream);
        if (rc != RFQ_OK) return rc;
    }
    return RFQ_OK;
}

static int matmul_raw(const char *who, int fmt, const float *d_act, const uint8_t *d_w, float *d_out, int m, int n,
                      int k, void *stream)
{
    int rc = check_gemv(who, fmt, d_w, 0, false, d_act, d_out, m, n, k);
    if (rc != RFQ_OK) return rc;
    if (m > 8) return fail(RFQ_E_UNSUPPORTED, "%s: m=%d > 8; use rfq_gemm_f16 for prefill", who, m);
    return launch_gemv(fmt, d_w, d_act, d_out, m, n, k, (hipStream_t)stream);
}

int rfq_matmul_q4_0(const float *a, const uint8_t *w, float *o, int m, int n, int k, void *s)
{
    return matmul_raw("rfq_matmul_q4_0", RFQ_Q4_0, a, w, o, m, n, k, s);
}
int rfq_matmul_q8_0(const float *a, const uint8_t *w, float *o, int m, int n, int k, void *s)
{
    return matmul_raw("rfq_matmul_q8_0", RFQ_Q8_0, a, w, o, m, n, k, s);
}
int rfq_matmul_q4_k(const float *a, const uint8_t *w, float *o, int m, int n, int k, void *s)
{
    return matmul_raw("rfq_matmul_q4_k", RFQ_Q4_K, a, w, o, m, n, k, s);
}
int rfq_matmul_q6_k(const float *a, const uint8_t *w, float *o, int m, int n, int k, void *s)
{
    return matmul_raw("rfq_matmul_q6_k", RFQ_Q6_K, a, w, o, m, n, k, s);
}

int rfq_matmul_host_weights(int fmt, const uint8_t *h_w, size_t w_bytes, const float *d_input, size_t n_rows,
                            size_t n_cols, float *d_out, void *stream)
{
    if (n_rows == 0 || n_cols == 0 || n_rows > 0x7fffffffu || n_cols > 0x7fffffffu)
        return fail(RFQ_E_BADARG, "rfq_matmul_host_weights: bad shape %zu x %zu", n_rows, n_cols);
    int rc = check_gemv("rfq_matmul_host_weights", fmt, h_w, w_bytes, true, d_input, d_out, 1, (int)n_rows, (int)n_cols, true);
    if (rc != RFQ_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    void *d_w = nullptr;
    RFQ_HIP(hipMalloc(&d_w, w_bytes));
    if (int up = upload_bytes(h_w, w_bytes, d_w, s)) { (void)hipStreamSynchronize(s); (void)hipFree(d_w); return up; }
    rc = launch_gemv(fmt, (const uint8_t *)d_w, d_input, d_out, 1, (int)n_rows, (int)n_cols, s);
    hipError_t e = hipStreamSynchronize(s);
    (void)hipFree(d_w);
    if (rc != RFQ_OK) return rc;
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return RFQ_OK;
}

// Shape and size checks of the flat-stream orientation: n * k elements in whole blocks.
static int check_gemv_kn(const char *who, int fmt, const void *w, size_t w_bytes, const void *x, const void *y, int m,
                         int n, int k)
{
    if (!known_format(fmt)) return fail(RFQ_E_BADARG, "%s: unknown format %d", who, fmt);
    if (fmt_dequant_only(fmt)) return fail(RFQ_E_UNSUPPORTED, "%s: format %d is decoded by rfq_dequant only", who, fmt);
    if (!w || !x || !y) return fail(RFQ_E_BADARG, "%s: null pointer", who);
    if (m <= 0 || n <= 0 || k <= 0)
        return fail(RFQ_E_BADARG, "%s: dimensions must be positive (m=%d n=%d k=%d)", who, m, n, k);
    const size_t elems = (size_t)n * (size_t)k, be = (size_t)fmt_block_elems(fmt);
    if (elems % be != 0)
        return fail(RFQ_E_SIZE, "%s: n * k = %zu is not a multiple of the %zu-element block", who, elems, be);
    const size_t need = elems / be * (size_t)fmt_block_bytes(fmt);
    if (w_bytes != need)
        return fail(RFQ_E_SIZE, "%s: weight buffer has %zu bytes, %d x %d elements need %zu", who, w_bytes, k, n, need);
    return RFQ_OK;
}

int rfq_gemv_kn(int fmt, const void *d_w, size_t w_bytes, const float *d_x, float *d_y, int m, int n, int k, void *stream)
{
    int rc = check_gemv_kn("rfq_gemv_kn", fmt, d_w, w_bytes, d_x, d_y, m, n, k);
    if (rc != RFQ_OK) return rc;
    for (int i = 0; i < m; i++) {
        rc = launch_gemv_kn(fmt, (const uint8_t *)d_w, d_x + (size_t)i * k, d_y + (size_t)i * n, n, k, (hipStream_t)stream);
        if (rc != RFQ_OK) return rc;
    }
    return RFQ_OK;
}

int rfq_matmul_host_weights_kn(int fmt, const uint8_t *h_w, size_t w_bytes, const float *d_input, size_t n_rows,
                               size_t n_cols, float *d_out, void *stream)
{
    if (n_rows == 0 || n_cols == 0 || n_rows > 0x7fffffffu || n_cols > 0x7fffffffu)
        return fail(RFQ_E_BADARG, "rfq_matmul_host_weights_kn: bad shape %zu x %zu", n_rows, n_cols);
    int rc = check_gemv_kn("rfq_matmul_host_weights_kn", fmt, h_w, w_bytes, d_input, d_out, 1, (int)n_rows, (int)n_cols);
    if (rc != RFQ_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    void *d_w = nullptr;
    RFQ_HIP(hipMalloc(&d_w, w_bytes));
    if (int up = upload_bytes(h_w, w_bytes, d_w, s)) { (void)hipStreamSynchronize(s); (void)hipFree(d_w); return up; }
    rc = launch_gemv_kn(fmt, (const uint8_t *)d_w, d_input, d_out, (int)n_rows, (int)n_cols, s);
    hipError_t e = hipStreamSynchronize(s);
    (void)hipFree(d_w);
    if (rc != RFQ_OK) return rc;
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return RFQ_OK;
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int rfq_rms_norm(const float *d_input, const float *d_weight, float *d_output, int seq_len, int hidden_size, float eps,
                 void *stream)
{
    if (seq_len < 0 || hidden_size <= 0)
        return fail(RFQ_E_BADARG, "rfq_rms_norm: seq_len=%d hidden_size=%d", seq_len, hidden_size);
    if (hidden_size % 4 != 0) return fail(RFQ_E_SIZE, "rfq_rms_norm: hidden_size=%d is not a multiple of 4", hidden_size);
    if (seq_len == 0) return RFQ_OK;
    if (!d_input || !d_weight || !d_output) return fail(RFQ_E_BADARG, "rfq_rms_norm: null pointer");
    if (!aligned16(d_input) || !aligned16(d_weight) || !aligned16(d_output))
        return fail(RFQ_E_BADARG, "rfq_rms_norm: input, weight and output must be 16-byte aligned");
    return launch_rms_norm(RFQ_TABLE_F32, d_input, d_weight, d_output, seq_len, hidden_size, eps, (hipStream_t)stream);
}

int rfq_swiglu(const float *d_gate, const float *d_up, float *d_output, int seq_len, int intermediate_size, void *stream)
{
    if (seq_len < 0 || intermediate_size < 0)
        return fail(RFQ_E_BADARG, "rfq_swiglu: seq_len=%d intermediate_size=%d", seq_len, intermediate_size);
    const size_t total = (size_t)seq_len * (size_t)intermediate_size;
    if (total == 0) return RFQ_OK;
    if (!d_gate || !d_up || !d_output) return fail(RFQ_E_BADARG, "rfq_swiglu: null pointer");
    return launch_swiglu(d_gate, d_up, d_output, total, (hipStream_t)stream);
}

int rfq_dequant_rms_norm(int fmt, const void *d_packed, size_t packed_bytes, const float *d_weight, float *d_output,
                         int seq_len, int hidden_size, float eps, void *stream)
{
    if (!known_format(fmt)) return fail(RFQ_E_BADARG, "rfq_dequant_rms_norm: unknown format %d", fmt);
    if (fmt_dequant_only(fmt) || fmt_mm_variant(fmt))
        return fail(RFQ_E_UNSUPPORTED, "rfq_dequant_rms_norm: format %d is decoded by rfq_dequant only", fmt);
    if (seq_len < 0 || hidden_size <= 0)
        return fail(RFQ_E_BADARG, "rfq_dequant_rms_norm: seq_len=%d hidden_size=%d", seq_len, hidden_size);
    const size_t need = matrix_bytes(fmt, seq_len > 0 ? seq_len : 1, hidden_size);
    if (need == 0)
        return fail(RFQ_E_SIZE, "rfq_dequant_rms_norm: hidden_size=%d is not a multiple of the %d-element block", hidden_size,
                    fmt_block_elems(fmt));
    if (seq_len == 0) return RFQ_OK;
    if (packed_bytes != need)
        return fail(RFQ_E_SIZE, "rfq_dequant_rms_norm: input has %zu bytes, [%d x %d] needs %zu", packed_bytes, seq_len,
                    hidden_size, need);
    if (!d_packed || !d_weight || !d_output) return fail(RFQ_E_BADARG, "rfq_dequant_rms_norm: null pointer");
    if (!aligned16(d_weight) || !aligned16(d_output))
        return fail(RFQ_E_BADARG, "rfq_dequant_rms_norm: weight and output must be 16-byte aligned");
    return launch_rms_norm(fmt, d_packed, d_weight, d_output, seq_len, hidden_size, eps, (hipStream_t)stream);
}

int rfq_rms_norm_gemv(int fmt, const void *d_w, size_t w_bytes, const float *d_x, const float *d_norm_weight, float eps,
                      float *d_y, int m, int n, int k, float *d_scratch, void *stream)
{
    int rc = check_gemv("rfq_rms_norm_gemv", fmt, d_w, w_bytes, true, d_x, d_y, m, n, k);
    if (rc != RFQ_OK) return rc;
    if (!d_norm_weight) return fail(RFQ_E_BADARG, "rfq_rms_norm_gemv: null norm weight");
    if (m > 8) return fail(RFQ_E_UNSUPPORTED, "rfq_rms_norm_gemv: m=%d > 8", m);
    hipStream_t s = (hipStream_t)stream;
    if (m == 1) {
        rc = launch_gemv_fused(fmt, (const uint8_t *)d_w, nullptr, d_x, d_norm_weight, eps, d_y, n, k, s);
        if (rc != RFQ_E_UNSUPPORTED) return rc;
    }
    if (!d_scratch) return fail(RFQ_E_BADARG, "rfq_rms_norm_gemv: m=%d k=%d needs d_scratch (m * k floats)", m, k);
    if (k % 4 != 0 || !aligned16(d_x) || !aligned16(d_norm_weight) || !aligned16(d_scratch))
        return fail(RFQ_E_BADARG, "rfq_rms_norm_gemv: x, norm weight and scratch must be 16-byte aligned, k a multiple of 4");
    rc = launch_rms_norm(RFQ_TABLE_F32, d_x, d_norm_weight, d_scratch, m, k, eps, s);
    if (rc != RFQ_OK) return rc;
    return launch_gemv(fmt, (const uint8_t *)d_w, d_scratch, d_y, m, n, k, s);
}

// scratch layout: h[m, inter] | xn[m, hidden] | gate[m, inter] | up[m, inter], each rounded to 16 bytes
static size_t pad16(size_t b) { return (b + 15) & ~(size_t)15; }

size_t rfq_mlp_scratch_bytes(int m, int hidden_size, int intermediate_size)
{
    if (m <= 0 || hidden_size <= 0 || intermediate_size <= 0) return 0;
    return 3 * pad16((size_t)m * intermediate_size * 4) + pad16((size_t)m * hidden_size * 4);
}

int rfq_mlp_swiglu(int fmt_gate_up, const void *d_gate_w, const void *d_up_w, size_t gate_up_bytes, int fmt_down,
                   const void *d_down_w, size_t down_bytes, const float *d_x, const float *d_norm_weight, float eps,
                   float *d_out, int m, int hidden_size, int intermediate_size, void *d_scratch, size_t scratch_bytes,
                   void *stream)
{
    int rc = check_gemv("rfq_mlp_swiglu (gate)", fmt_gate_up, d_gate_w, gate_up_bytes, true, d_x, d_out, m,
                        intermediate_size, hidden_size);
    if (rc != RFQ_OK) return rc;
    rc = check_gemv("rfq_mlp_swiglu (up)", fmt_gate_up, d_up_w, gate_up_bytes, true, d_x, d_out, m, intermediate_size,
                    hidden_size);
    if (rc != RFQ_OK) return rc;
    rc = check_gemv("rfq_mlp_swiglu (down)", fmt_down, d_down_w, down_bytes, true, d_x, d_out, m, hidden_size,
                    intermediate_size);
    if (rc != RFQ_OK) return rc;
    if (m > 8) return fail(RFQ_E_UNSUPPORTED, "rfq_mlp_swiglu: m=%d > 8", m);
    const size_t need = rfq_mlp_scratch_bytes(m, hidden_size, intermediate_size);
    if (!d_scratch || scratch_bytes < need || !aligned16(d_scratch))
        return fail(RFQ_E_SIZE, "rfq_mlp_swiglu: scratch of %zu bytes (16-byte aligned) needed, %zu given", need,
                    scratch_bytes);
    hipStream_t s = (hipStream_t)stream;
    const size_t mi = pad16((size_t)m * intermediate_size * 4);
    uint8_t *base = static_cast<uint8_t *>(d_scratch);
    float *h = reinterpret_cast<float *>(base);
    float *xn = reinterpret_cast<float *>(base + mi);
    float *gate = reinterpret_cast<float *>(base + mi + pad16((size_t)m * hidden_size * 4));
    float *up = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(gate) + mi);
    rc = RFQ_E_UNSUPPORTED;
    if (m == 1)
        rc = launch_gemv_fused(fmt_gate_up, (const uint8_t *)d_gate_w, (const uint8_t *)d_up_w, d_x, d_norm_weight, eps, h,
                               intermediate_size, hidden_size, s);
    if (rc == RFQ_E_UNSUPPORTED) {
        const float *xin = d_x;
        if (d_norm_weight) {
            if (hidden_size % 4 != 0 || !aligned16(d_x) || !aligned16(d_norm_weight))
                return fail(RFQ_E_BADARG, "rfq_mlp_swiglu: x and norm weight must be 16-byte aligned, hidden_size a multiple of 4");
            rc = launch_rms_norm(RFQ_TABLE_F32, d_x, d_norm_weight, xn, m, hidden_size, eps, s);
            if (rc != RFQ_OK) return rc;
            xin = xn;
        }
        rc = launch_gemv(fmt_gate_up, (const uint8_t *)d_gate_w, xin, gate, m, intermediate_size, hidden_size, s);
        if (rc != RFQ_OK) return rc;
        rc = launch_gemv(fmt_gate_up, (const uint8_t *)d_up_w, xin, up, m, intermediate_size, hidden_size, s);
        if (rc != RFQ_OK) return rc;
        rc = launch_swiglu(gate, up, h, (size_t)m * intermediate_size, s);
    }
    if (rc != RFQ_OK) return rc;
    return launch_gemv(fmt_down, (const uint8_t *)d_down_w, h, d_out, m, hidden_size, intermediate_size, s);
}

int rfq_gemm_f16(int fmt, const void *d_w, size_t w_bytes, const void *d_a_f16, void *d_out, int out_dtype, int m,
                 int n, int k, void *stream)
{
    int rc = check_gemv("rfq_gemm_f16", fmt, d_w, w_bytes, true, d_a_f16, d_out, m, n, k);
    if (rc != RFQ_OK) return rc;
    if ((out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F32 && (out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F16)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16: out_dtype %d is neither F32 nor F16", out_dtype);
    return launch_gemm_f16(fmt, (const uint8_t *)d_w, d_a_f16, d_out, out_dtype, m, n, k, false, nullptr, (hipStream_t)stream);
}

int rfq_gemm_f16_static(int fmt, const void *d_w, size_t w_bytes, const void *d_a_f16, void *d_out, int out_dtype, int m,
                        int n, int k, void *stream)
{
    int rc = check_gemv("rfq_gemm_f16_static", fmt, d_w, w_bytes, true, d_a_f16, d_out, m, n, k);
    if (rc != RFQ_OK) return rc;
    if ((out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F32 && (out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F16)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16_static: out_dtype %d is neither F32 nor F16", out_dtype);
    return launch_gemm_f16(fmt, (const uint8_t *)d_w, d_a_f16, d_out, out_dtype, m, n, k, true, nullptr, (hipStream_t)stream);
}

size_t rfq_gemm_f16_arranged_bytes(int m, int k) { return gemm_f16_arranged_bytes(m, k); }
int rfq_gemm_f16_k_parts(int m, int n, int k) { return m > 0 && n > 0 && k > 0 ? gemm_f16_k_parts(m, n, k) : 1; }

int rfq_gemm_f16_arrange(const void *d_a_f16, int m, int k, void *d_arranged, size_t arranged_bytes, void *stream)
{
    if (!d_a_f16 || !d_arranged) return fail(RFQ_E_BADARG, "rfq_gemm_f16_arrange: null pointer");
    if (m <= 0 || k <= 0) return fail(RFQ_E_BADARG, "rfq_gemm_f16_arrange: bad shape m=%d k=%d", m, k);
    const size_t need = gemm_f16_arranged_bytes(m, k);
    if (need == 0) return fail(RFQ_E_SIZE, "rfq_gemm_f16_arrange: k=%d is not a multiple of 8", k);
    if (arranged_bytes < need)
        return fail(RFQ_E_SIZE, "rfq_gemm_f16_arrange: the buffer has %zu bytes, [%d x %d] needs %zu", arranged_bytes, m, k, need);
    return launch_arrange_a(d_a_f16, m, k, (uint8_t *)d_arranged, (hipStream_t)stream);
}

int rfq_gemm_f16_arranged(int fmt, const void *d_w, size_t w_bytes, const void *d_arranged, size_t arranged_bytes,
                          void *d_out, int out_dtype, int m, int n, int k, void *stream)
{
    int rc = check_gemv("rfq_gemm_f16_arranged", fmt, d_w, w_bytes, true, d_arranged, d_out, m, n, k);
    if (rc != RFQ_OK) return rc;
    if ((out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F32 && (out_dtype & ~RFQ_GEMM_ONE_PLANE) != RFQ_F16)
        return fail(RFQ_E_BADARG, "rfq_gemm_f16_arranged: out_dtype %d is neither F32 nor F16", out_dtype);
    const size_t need = gemm_f16_arranged_bytes(m, k);
    if (need == 0 || arranged_bytes < need)
        return fail(RFQ_E_SIZE, "rfq_gemm_f16_arranged: the arranged activations have %zu bytes, [%d x %d] needs %zu",
                    arranged_bytes, m, k, need);
    return launch_gemm_f16(fmt, (const uint8_t *)d_w, nullptr, d_out, out_dtype, m, n, k, false, (const uint8_t *)d_arranged,
                           (hipStream_t)stream);
}

size_t rfq_mx_prepared_bytes(int fmt, int kind, int rows, int k)
{
    return mx_prepared_bytes(fmt, kind, rows, k);
}

int rfq_mx_prepare(int fmt, int kind_req, const void *d_raw, size_t raw_bytes, int rows, int k, void *d_prepared,
                   size_t prepared_bytes, int *kind_out, void *stream)
{
    if (fmt != RFQ_MXFP4 && fmt != RFQ_MXFP6_E2M3 && fmt != RFQ_MXFP6_E3M2)
        return fail(RFQ_E_BADARG, "rfq_mx_prepare: format %d is not an MXFP format", fmt);
    if (!d_raw || !d_prepared) return fail(RFQ_E_BADARG, "rfq_mx_prepare: null pointer");
    if (rows <= 0 || k <= 0) return fail(RFQ_E_BADARG, "rfq_mx_prepare: bad shape %d x %d", rows, k);
    if (k % 128 != 0) return fail(RFQ_E_SIZE, "rfq_mx_prepare: k=%d is not a multiple of 128", k);
    if (kind_req != RFQ_MX_AUTO && kind_req != RFQ_MX_FP4 && kind_req != RFQ_MX_FP8 && kind_req != RFQ_MX_FP4_UNCHECKED)
        return fail(RFQ_E_BADARG, "rfq_mx_prepare: unknown kind %d", kind_req);
    size_t need = matrix_bytes(fmt, rows, k);
    if (raw_bytes != need)
        return fail(RFQ_E_SIZE, "rfq_mx_prepare: raw buffer has %zu bytes, [%d x %d] needs %zu", raw_bytes, rows, k, need);
    return launch_mx_prepare(fmt, kind_req, (const uint8_t *)d_raw, rows, k, d_prepared, prepared_bytes, kind_out,
                             (hipStream_t)stream);
}

int rfq_gemm_mx(const void *d_a_prep, size_t a_prep_bytes, int a_kind, const void *d_w_prep, size_t w_prep_bytes,
                int w_kind, void *d_out, int out_dtype, int m, int n, int k, void *stream)
{
    if (!d_a_prep || !d_w_prep || !d_out) return fail(RFQ_E_BADARG, "rfq_gemm_mx: null pointer");
    if (m <= 0 || n <= 0 || k <= 0) return fail(RFQ_E_BADARG, "rfq_gemm_mx: bad shape m=%d n=%d k=%d", m, n, k);
    if (k % 128 != 0) return fail(RFQ_E_SIZE, "rfq_gemm_mx: k=%d is not a multiple of 128", k);
    if ((a_kind != RFQ_MX_FP4 && a_kind != RFQ_MX_FP8) || (w_kind != RFQ_MX_FP4 && w_kind != RFQ_MX_FP8))
        return fail(RFQ_E_BADARG, "rfq_gemm_mx: operand kinds must be FP4 or FP8 (a=%d w=%d)", a_kind, w_kind);
    if (out_dtype != RFQ_F32 && out_dtype != RFQ_BF16)
        return fail(RFQ_E_BADARG, "rfq_gemm_mx: out_dtype %d is neither F32 nor BF16", out_dtype);
    // (the layout of a prepared operand depends on its kind and shape only; an FP4 operand is always MXFP4)
    const size_t a_need = mx_prepared_bytes(a_kind == RFQ_MX_FP4 ? RFQ_MXFP4 : RFQ_MXFP6_E2M3, a_kind, m, k);
    const size_t w_need = mx_prepared_bytes(w_kind == RFQ_MX_FP4 ? RFQ_MXFP4 : RFQ_MXFP6_E2M3, w_kind, n, k);
    if (a_need == 0 || a_prep_bytes < a_need)
        return fail(RFQ_E_SIZE, "rfq_gemm_mx: prepared A has %zu bytes, [%d x %d] of kind %d needs %zu", a_prep_bytes, m, k,
                    a_kind, a_need);
    if (w_need == 0 || w_prep_bytes < w_need)
        return fail(RFQ_E_SIZE, "rfq_gemm_mx: prepared W has %zu bytes, [%d x %d] of kind %d needs %zu", w_prep_bytes, n, k,
                    w_kind, w_need);
    return launch_gemm_mx(d_a_prep, a_kind, d_w_prep, w_kind, d_out, out_dtype, m, n, k, (hipStream_t)stream);
}

} // extern "C"
