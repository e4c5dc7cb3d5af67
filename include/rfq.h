/*
 * rfq.h -- C ABI of librfq: MI355X (gfx950) kernels for ROCmForge's
 * quantized-weight path: block dequantisation fused into the decode GEMV and
 * the prefill GEMM.
 *
 * The library is a drop-in for the device side of ROCmForge's operator
 * surface.  Each entry point names the reference interface it replaces
 * (paths relative to the ROCmForge tree).  Conventions:
 *   - plain C types only; "d_" pointers are device pointers (what
 *     HipBuffer::as_ptr() returns, src/backend/hip_backend/memory.rs:540-547),
 *     "h_" pointers are host pointers;
 *   - packed weights are the bytes exactly as ROCmForge stores them,
 *     little-endian, blocks running along K, matrix rows contiguous
 *     ([n_rows, n_cols] row-major, the layout documented at
 *     src/kernels/matmul/quantized/q4_0.rs:139-148);
 *   - every function returns an rfq_status (0 = success, like HIP_SUCCESS,
 *     src/backend/hip_backend/ffi.rs:78); rfq_last_error() gives the text;
 *   - device entry points only enqueue work on the caller's stream
 *     (hipStream_t passed as void*, NULL = the default stream) and never
 *     synchronise, unless the comment says otherwise;
 *   - the caller owns every buffer; the library keeps no reference to them.
 */
#ifndef RFQ_H
#define RFQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Raised whenever an exported signature or the meaning of a format changes: a caller compares
 * rfq_version() with the RFQ_VERSION it was built against before its first call. */
#define RFQ_VERSION 104 /* 0.1.4 */

#if defined(_WIN32)
#define RFQ_API
#else
#define RFQ_API __attribute__((visibility("default")))
#endif

/* Block formats; the values are GgufTensorType's ids
 * (src/loader/tensor_type.rs:16-32). */
typedef enum rfq_format {
    RFQ_Q4_0 = 2,        /* 20 B / 32: f32 scale + 16 nibble bytes           */
    RFQ_Q8_0 = 8,        /* 36 B / 32: f32 scale + 32 offset-binary bytes    */
    RFQ_Q2_K = 10,       /* 256 B / 256: 16 f16 scales, 16 f16 mins, 2-bit codes (+ one high bit); rfq_dequant* only */
    RFQ_Q3_K = 11,       /* 256 B / 256: 16 f16 scales, 3-bit codes (+ high bits), q - 4;          rfq_dequant* only */
    RFQ_Q4_K = 12,       /* 256 B / 256: 8 f16 scales, 8 i8 mins, nibbles    */
    RFQ_Q5_K = 13,       /* 256 B / 256: 16 f16 scales, 16 i8 mins, 5-bit codes;                    rfq_dequant* only */
    RFQ_Q6_K = 14,       /* 256 B / 256: 16 f16 scales, 6-bit stream         */
    RFQ_MXFP4 = 20,      /* 17 B / 32: i8 exponent + 16 nibble bytes         */
    RFQ_MXFP6_E2M3 = 21, /* 25 B / 32: i8 exponent + 24 packed bytes         */
    RFQ_MXFP6_E3M2 = 22, /* decoded exactly like E2M3 (src/loader/dequant.rs:693) */
    /* The block layouts of GGUF model files (public ggml definitions; 100 + the
     * ggml type id).  ROCmForge has no decoder for them -- its loader sizes such
     * tensors with its own layouts above (src/loader/gguf/tensor_info.rs:108-130,
     * src/loader/gguf_tensor.rs:41-60) -- so there is no reference arithmetic to
     * match: results follow ggml's dequantize_row_* (ggml-quants.c).  Accepted by
     * rfq_dequant*, rfq_get_rows, rfq_dequant_rms_norm, rfq_gemv, rfq_matmul_host_weights,
     * rfq_rms_norm_gemv, rfq_mlp_swiglu and rfq_gemm_f16. */
    RFQ_GGUF_Q4_0 = 102, /* 18 B / 32: f16 d, 16 bytes (low nibbles = elements 0-15, high = 16-31); d*(q-8) */
    RFQ_GGUF_Q8_0 = 108, /* 34 B / 32: f16 d, 32 int8; d*q                                                 */
    RFQ_GGUF_Q4_K = 112, /* 144 B / 256: f16 d, dmin, 12 B of 6-bit scales/mins, 128 nibble bytes          */
    RFQ_GGUF_Q6_K = 114, /* 210 B / 256: 128 B low nibbles, 64 B high bit pairs, 16 i8 scales, f16 d       */
    /* The decoders the matmul module carries beside the loader's
     * (src/kernels/matmul/quantized/; 200 + the id of the format they are a
     * variant of).  They are what matmul_q8_0 and the *_cpu_fallback paths feed
     * to the f32 matmul, and they read the same bytes differently from the
     * formats above.  Accepted by rfq_dequant*, rfq_gemv, rfq_gemv_kn and
     * rfq_matmul_host_weights*.  (That module's dequantize_q4_0, q4_0.rs:89-134,
     * is RFQ_Q4_0 itself: same bytes, same arithmetic.) */
    RFQ_MM_Q8_0 = 208,   /* 36 B / 32: f32 scale + 32 two's-complement int8 bytes; scale * q
                            (quantized/q8_0.rs:18-56)                                                      */
    RFQ_MM_Q4_K = 212,   /* 256 B / 256: as RFQ_Q4_K but the nibbles of sub-block sb start at 32 + 20 * sb,
                            and the f16 scale is widened by f16_to_f32_cpu (quantized/common.rs:44-60:
                            its mantissa shift runs in 16 bits and its zero/subnormal branch is dead, so
                            a pattern b reads +-2^(field - 15) * (1 + (b & 7) / 1024) -- 0x3E00 is 1.0,
                            0x0000 is 2^-15); min + q * scale (quantized/q4_k.rs:90-148)                   */
    RFQ_MM_Q6_K = 214    /* 256 B / 256: the RFQ_Q6_K stream with the scales widened by f16_to_f32_cpu
                            (quantized/q6_k.rs:90-148)                                                     */
} rfq_format;
/* rfq_get_rows also gathers from a plain f32 table (GgufTensorType F32 = 0). */
#define RFQ_TABLE_F32 0

typedef enum rfq_status {
    RFQ_OK = 0,
    RFQ_E_BADARG = -1,      /* null pointer, non-positive dimension, unknown enum   */
    RFQ_E_SIZE = -2,        /* byte count does not match the shape                  */
    RFQ_E_UNSUPPORTED = -3, /* valid request this build has no kernel for; the Rust
                               wrapper maps it to HipError::KernelLoadFailed so the
                               *_with_fallback paths still fall back
                               (src/kernels/quant/q4_0.rs:236-251)                  */
    RFQ_E_HIP = -4,         /* a HIP runtime call failed                            */
    RFQ_E_NOMEM = -5        /* device or host allocation failed                     */
} rfq_status;

typedef enum rfq_dtype { RFQ_F32 = 0, RFQ_F16 = 1, RFQ_BF16 = 2 } rfq_dtype;
/* Or-ed into the out_dtype of rfq_gemm_f16 / _static / _arranged: contract every decoded weight as ONE fp16
 * operand (relative 2^-12 per weight) instead of two (see rfq_gemm_f16); about half the time, outside the
 * 1e-3 tolerance on outputs that are small against the typical size. */
#define RFQ_GEMM_ONE_PLANE 0x100

/* Operand encodings of a prepared MXFP matrix (see rfq_mx_prepare). */
typedef enum rfq_mx_kind { RFQ_MX_AUTO = 0, RFQ_MX_FP4 = 4, RFQ_MX_FP8 = 8, RFQ_MX_FP4_UNCHECKED = 0x104 } rfq_mx_kind;

/* ---- library ------------------------------------------------------------ */

RFQ_API int rfq_version(void);
/* Thread-local description of the last failure on this thread ("" if none). */
RFQ_API const char *rfq_last_error(void);
/* rfq_gemm_f16, rfq_gemv_kn and rfq_gemv (Q8_0, m > 1) keep up to 64 MiB of
 * temporary device memory per stream between calls (a stream's first call, or
 * a larger shape than before, allocates; a larger request replaces the
 * buffer).  Under stream capture such a call uses the buffer the stream
 * already has and fails with RFQ_E_UNSUPPORTED if it would have to allocate or
 * grow: run the call once on the stream before capturing.  A captured graph
 * holds the buffer's address, so the library never frees a buffer it handed
 * out during a capture when it grows -- only this function does: it frees
 * every kept buffer (it waits for the device first) and rfq_upload's pinned
 * staging slots, and thereby invalidates graphs captured earlier; the next
 * call allocates again.  Buffers are kept per stream handle:
 * rfq_release_stream_temporaries(stream) gives up the one of a stream that is
 * about to be destroyed (it frees the buffer once the stream's work is done;
 * a buffer that a capture used stays allocated until rfq_release_temporaries),
 * so that a later stream with the same handle value does not inherit it.
 * Calls that use a stream's kept buffer must come from one host thread at a
 * time per stream (a second thread that makes the buffer grow would free it
 * under the first thread's launches); different streams are independent.
 * No counterpart in the reference, whose kernels take no temporaries. */
RFQ_API int rfq_release_temporaries(void);
RFQ_API int rfq_release_stream_temporaries(void *stream);
/* Host bytes (pageable: a slice of the memory-mapped model file) -> device
 * memory, in stream order.  The bytes go through a ring of four pinned 8 MiB
 * slots the library keeps per device: a few host threads fill a slot while the
 * earlier slots' transfers are in flight.  On return the source may be
 * released; the device copy completes in stream order (the call itself blocks
 * only while it waits for a free slot).  Not for use under graph capture.
 * Replaces the pageable hipMemcpy / hipMemcpyAsync of HipBuffer::copy_from_host
 * (src/backend/hip_backend/memory.rs:135-170, 203-250) and
 * AsyncLoader::upload_to_buffer / upload_to_buffer_offset
 * (src/backend/hip_backend/async_ops.rs:66-180) as the loader uses them
 * (src/loader/gguf/gpu_upload.rs:57-125); rfq_dequant_upload and
 * rfq_matmul_host_weights upload through it too. */
RFQ_API int rfq_upload(const void *h_src, size_t bytes, void *d_dst, void *stream);
/* Elements per block / bytes per block the decoders stride by
 * (GgufTensorType::block_size, src/loader/tensor_type.rs:77-88; strides at
 * src/kernels/quant/q4_0.rs:269, q8_0.rs:33, q4_k.rs:206, q6_k.rs:206,
 * src/loader/dequant.rs:47,91).  0 for an unknown format. */
RFQ_API size_t rfq_block_elems(int fmt);
RFQ_API size_t rfq_block_bytes(int fmt);
/* ceil(n_elems / block_elems) * block_bytes. */
RFQ_API size_t rfq_packed_bytes(int fmt, size_t n_elems);

/* ---- dequantisation ------------------------------------------------------ */

/* Packed bytes on the device -> f32 on the device, bit-exact with the CPU
 * decoders, including their short-input behaviour: out is n_elems floats,
 * every element the CPU loop would not reach is written as 0.0.
 * Replaces the kernel launches inside dequantize_q4_0_kernel_cached
 * (src/kernels/quant/q4_0.rs:107-153), dequantize_q4_k_gpu_kernel
 * (q4_k.rs:99-148), dequantize_q6_k_gpu_kernel (q6_k.rs:102-149) and the
 * unused mxfp/q8_0 dequant kernels (kernels/mxfp_dequant.hip, q8_0_dequant.hip);
 * for Q2_K / Q3_K / Q5_K, the CPU loops dequant_q2_k / q3_k / q5_k
 * (src/loader/dequant.rs:150-420) that loader::dequantize dispatches to. */
RFQ_API int rfq_dequant(int fmt, const void *d_packed, size_t packed_bytes, float *d_out, size_t n_elems,
                void *stream);

/* Host bytes -> device f32: uploads through a temporary device buffer, runs
 * rfq_dequant, synchronises the stream and frees the temporary -- the whole
 * body of dequantize_q4_0_kernel_cached / dequantize_q4_k_gpu_kernel /
 * dequantize_q6_k_gpu_kernel (same files as above). */
RFQ_API int rfq_dequant_upload(int fmt, const uint8_t *h_packed, size_t packed_bytes, float *d_out,
                       size_t n_elems, void *stream);

/* Host bytes -> host f32 through the GPU (upload, kernel, download;
 * synchronous).  Backs rocmforge::loader::dequant_q4_0 / dequant_q8_0 /
 * dequant_q4_k / dequant_q6_k (src/loader/mod.rs:116-127), dequant_mxfp4 /
 * dequant_mxfp6 (src/loader/dequant.rs:41,85) and the quantised arms of
 * loader::dequantize (dequant.rs:673-700). */
RFQ_API int rfq_dequant_host(int fmt, const uint8_t *h_packed, size_t packed_bytes, float *h_out,
                     size_t n_elems);

/* ---- decode GEMV (and small batches) -------------------------------------- */

/* d_y[m, n] = d_x[m, k] . dequant(W)[n, k]^T, fp32 accumulation, k a multiple
 * of the block size, w_bytes == n * (k / block_elems) * block_bytes.  Built for
 * decode, 1 <= m <= 8 (one launch); larger m runs eight rows per launch and
 * re-reads W each time -- a prefill belongs to rfq_gemm_f16 / rfq_gemm_mx.
 * Replaces matmul_q4_0_gpu (src/kernels/matmul/quantized/q4_0.rs:209-260) and
 * its q4_k / q6_k twins (q4_k.rs:221-268, q6_k.rs:211-258), for every format. */
RFQ_API int rfq_gemv(int fmt, const void *d_w, size_t w_bytes, const float *d_x, float *d_y, int m, int n,
             int k, void *stream);

/* The other orientation: d_y[m, n] = d_x[m, k] . Wd[k, n], where Wd is the
 * packed stream decoded as ONE flat array of n * k elements and element
 * (l, j) is Wd[l * n + j] -- the blocks run along n.  This is what the
 * reference computes on the bytes it is handed, whatever the doc comments of
 * its wrappers say about [n_rows, n_cols]: the fused kernel indexes
 * weight_linear_idx = k_idx * n + col (kernels/q4_0_matmul.hip:207, q4_k_matmul.hip:270, reached
 * through matmul_q4_0_gpu, src/kernels/matmul/quantized/q4_0.rs:209-260), and
 * the fallback hands the flat dequantised buffer to the f32 matmul as b[k, n]
 * (matmul_q4_0_cpu_fallback, q4_0.rs:274-311; cpu_matmul_f32,
 * src/tensor/matmul.rs:219-233: b[l * n + j]).  The same weight bytes give
 * different numbers through rfq_gemv (rows of k) and through this call.
 * n * k a multiple of the block size, w_bytes == n * k / block_elems *
 * block_bytes, any m >= 1 (one pass over W per row of x).  The sum over l is
 * split over workgroups in a fixed order (the result does not vary from run
 * to run); the partial sums live in the temporary memory described at
 * rfq_release_temporaries (at most 8 MiB). */
RFQ_API int rfq_gemv_kn(int fmt, const void *d_w, size_t w_bytes, const float *d_x, float *d_y, int m, int n,
                        int k, void *stream);

/* The reference's raw-pointer launch signatures, argument order
 * (activations, weights, output, m, n, k) as in matmul_q4_0_gpu
 * (src/kernels/matmul/quantized/q4_0.rs:209-217) and the kernels' own
 * parameter lists (kernels/q4_0_matmul.hip:153-160).  The byte size of the
 * weights is implied by n and k.  These read W as [n, k], rows of k -- the
 * layout the reference documents (q4_0.rs:139-148) -- and are rfq_gemv under
 * another argument order; what the reference's kernel computes on the same
 * buffer is rfq_gemv_kn. */
RFQ_API int rfq_matmul_q4_0(const float *d_act, const uint8_t *d_w, float *d_out, int m, int n, int k, void *stream);
RFQ_API int rfq_matmul_q8_0(const float *d_act, const uint8_t *d_w, float *d_out, int m, int n, int k, void *stream);
RFQ_API int rfq_matmul_q4_k(const float *d_act, const uint8_t *d_w, float *d_out, int m, int n, int k, void *stream);
RFQ_API int rfq_matmul_q6_k(const float *d_act, const uint8_t *d_w, float *d_out, int m, int n, int k, void *stream);

/* Host-resident weights, device input and output, m = 1: allocate, upload,
 * multiply, synchronise, free -- the observable behaviour of matmul_q4_0 /
 * matmul_q4_k / matmul_q6_k / matmul_q8_0
 * (src/kernels/matmul/quantized/q4_0.rs:153-203, q4_k.rs:173-215,
 * q6_k.rs:163-205, q8_0.rs:69-106).  d_out receives n_rows floats. */
RFQ_API int rfq_matmul_host_weights(int fmt, const uint8_t *h_w, size_t w_bytes, const float *d_input,
                            size_t n_rows, size_t n_cols, float *d_out, void *stream);
/* The same call in the orientation of rfq_gemv_kn: d_out[j] = sum_l
 * d_input[l] * Wd[l * n_rows + j], the numbers matmul_q4_0_cpu_fallback
 * (src/kernels/matmul/quantized/q4_0.rs:274-311, fmt = RFQ_Q4_0) and matmul_q8_0
 * (quantized/q8_0.rs:69-106, fmt = RFQ_MM_Q8_0) produce: they dequantise on the
 * CPU (fmt = RFQ_MM_Q4_K / RFQ_MM_Q6_K for that module's K decoders), upload
 * the f32 array and multiply with m = 1, k = n_cols, n = n_rows. */
RFQ_API int rfq_matmul_host_weights_kn(int fmt, const uint8_t *h_w, size_t w_bytes, const float *d_input,
                                       size_t n_rows, size_t n_cols, float *d_out, void *stream);

/* ---- embedding rows ---------------------------------------------------------- */

/* d_out[i, :] = row d_tokens[i] of the [n_vocab, n_embd] table, dequantised
 * (fmt = a block format, n_embd a multiple of its block) or copied (fmt =
 * RFQ_TABLE_F32, n_embd a multiple of 4), for i < n_tokens.  Replaces
 * get_rows (src/ggml/hip_backend/ops/get_rows.rs:6-53, RowMajor) and the
 * token copy to the host in front of it (op_dispatch.rs:70-100): the ids are
 * read on the device.  Where the reference fails with "Token ID exceeds vocab
 * size" this leaves the row zero and, if d_status (a device int) is given,
 * stores 1 + the smallest offending index there (0 when every id was valid);
 * the call itself only enqueues.  d_out 16-byte aligned. */
RFQ_API int rfq_get_rows(int fmt, const void *d_table, size_t table_bytes, int n_vocab, int n_embd,
                         const uint32_t *d_tokens, int n_tokens, float *d_out, int *d_status, void *stream);

/* ---- neighbours of the matmul in a decoder layer ---------------------------- */

/* d_out[r, j] = (d_x[r, j] / sqrt(mean_j d_x[r, j]^2 + eps)) * d_weight[j] for
 * seq_len rows of hidden_size floats (hidden_size a multiple of 4, all three
 * pointers 16-byte aligned).  Replaces rms_norm_gpu_kernel
 * (src/mlp/kernels.rs:261-330, kernels/rms_norm.hip:40-84). */
RFQ_API int rfq_rms_norm(const float *d_input, const float *d_weight, float *d_output, int seq_len, int hidden_size,
                         float eps, void *stream);

/* d_output[i] = d_gate[i] * (d_up[i] * sigmoid(d_up[i])) over seq_len *
 * intermediate_size elements: the activation is applied to the UP projection,
 * as the reference defines it.  Replaces swiglu_gpu_kernel
 * (src/mlp/kernels.rs:177-240, kernels/swiglu.hip:40-62). */
RFQ_API int rfq_swiglu(const float *d_gate, const float *d_up, float *d_output, int seq_len, int intermediate_size,
                       void *stream);

/* RMSNorm of rows that are still packed: d_packed holds seq_len rows of
 * hidden_size elements in format fmt (hidden_size a multiple of the block), the
 * rows are decoded on the fly and normalised as in rfq_rms_norm; no f32 copy
 * of the input exists.  Replaces fused_q4_0_rmsnorm
 * (src/ggml/hip_backend/ops/fused_ops.rs:149-160,
 * kernels/fused_dequant_rmsnorm.hip:87-163), for every format. */
RFQ_API int rfq_dequant_rms_norm(int fmt, const void *d_packed, size_t packed_bytes, const float *d_weight,
                                 float *d_output, int seq_len, int hidden_size, float eps, void *stream);

/* d_y[m, n] = RMSNorm(d_x[m, k]; d_norm_weight, eps) . dequant(W)[n, k]^T: the
 * normalisation that precedes a projection in a decoder layer and the
 * projection (rfq_gemv) in one call.  For m = 1 and 512 < k <= 16384 it is one
 * launch and the normalised vector never exists in memory; other shapes run
 * rfq_rms_norm into d_scratch (m * k floats, 16-byte aligned; may be NULL when
 * the one-launch case applies) and then rfq_gemv.  The reference has the two
 * steps only as separate f32 operations (kernels/rms_norm.hip, hipBLAS SGEMM:
 * src/ggml/hip_backend/op_dispatch.rs:1001-1014). */
RFQ_API int rfq_rms_norm_gemv(int fmt, const void *d_w, size_t w_bytes, const float *d_x, const float *d_norm_weight,
                              float eps, float *d_y, int m, int n, int k, float *d_scratch, void *stream);

/* The SwiGLU MLP of a decoder layer over quantised weights, 1 <= m <= 8 rows:
 *   xn  = d_norm_weight ? RMSNorm(d_x; d_norm_weight, eps) : d_x      [m, hidden]
 *   h   = swiglu(xn . dequant(gate)^T, xn . dequant(up)^T)            [m, inter]
 *   out = h . dequant(down)^T                                         [m, hidden]
 * gate and up are [inter, hidden] in fmt_gate_up (gate_up_bytes each), down is
 * [hidden, inter] in fmt_down; rows are outputs, blocks run along k, as
 * rfq_gemv takes them.  For m = 1 this is two launches: gate and up rows are
 * walked together, normalisation and activation happen inside that kernel, and
 * only h goes through d_scratch.  Replaces HipBackend::mlp_swiglu
 * (src/backend/hip_backend/backend.rs:1153-1278: three f32 SGEMMs, a SwiGLU
 * kernel and two synchronisations) for quantised weights.  d_scratch:
 * rfq_mlp_scratch_bytes(m, hidden, inter) bytes, 16-byte aligned, owned by
 * the caller; nothing is allocated and nothing synchronises. */
RFQ_API size_t rfq_mlp_scratch_bytes(int m, int hidden_size, int intermediate_size);
RFQ_API int rfq_mlp_swiglu(int fmt_gate_up, const void *d_gate_w, const void *d_up_w, size_t gate_up_bytes,
                           int fmt_down, const void *d_down_w, size_t down_bytes, const float *d_x,
                           const float *d_norm_weight, float eps, float *d_out, int m, int hidden_size,
                           int intermediate_size, void *d_scratch, size_t scratch_bytes, void *stream);

/* ---- prefill GEMM ----------------------------------------------------------- */

/* d_out[m, n] = d_a[m, k] (fp16) . dequant(W)[n, k]^T on the fp16 matrix
 * cores with fp32 accumulation; out_dtype is RFQ_F32 or RFQ_F16, optionally
 * or-ed with RFQ_GEMM_ONE_PLANE.  Formats: Q4_0, Q8_0, Q4_K, Q6_K and the four
 * GGUF file layouts.  Weights are decoded to f32 as the format defines and
 * contracted as two fp16 operands, hi = fp16(v) and lo = fp16(v - hi) (v to
 * 2^-22: the result is that of an fp32 contraction, 5e-6 of rms(out) from the
 * reference's at 512 x 4096 x 14336); the 256-byte Q4_K layout, whose integer
 * mins are contracted exactly and apart, takes q * scale as one operand, and
 * RFQ_GGUF_Q4_K is contracted exactly in one pass (integer operands sc * q,
 * the super-block's d and dmin applied in f32).  With
 * RFQ_GEMM_ONE_PLANE every format takes one rounded operand (8e-4 of rms(out)).  k a multiple of 256
 * for the K-formats, of 32 otherwise; d_a_f16 16-byte aligned, d_w 4-byte aligned.  Up to 64 MiB of
 * temporary device memory (the activations in matrix-operand order) is kept
 * per stream between calls; larger temporaries are allocated and released in
 * stream order.  (A stream's first call, or a larger shape than before,
 * allocates: run the call once on the stream before capturing it into a graph.)
 * A shape with few output tiles and a long k (an attention or down projection
 * of 512 tokens: 64 tiles of 256 x 128 for 256 CUs) is split along k into
 * rfq_gemm_f16_k_parts(m, n, k) parts of whole super-blocks, whose f32 tiles
 * (parts * m * n * 4 more bytes of temporary) a second kernel adds in a fixed
 * order: the results are deterministic and differ from a single pass only in
 * the order of the fp32 sums.  The reference has no fused prefill GEMM (its matmul_q* hard-wire
 * m = 1, src/kernels/matmul/quantized/q4_0.rs:169; larger m goes through
 * dequantise + hipBLAS SGEMM, src/tensor/matmul.rs:134-214); this is the same
 * contraction. */
RFQ_API int rfq_gemm_f16(int fmt, const void *d_w, size_t w_bytes, const void *d_a_f16, void *d_out,
                 int out_dtype, int m, int n, int k, void *stream);

/* rfq_gemm_f16 for callers that cannot allocate device memory: code under
 * stream capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference.  Same arguments, same kernels and bit-identical
 * results (a shape that rfq_gemm_f16 splits along k is split here too when the
 * parts' f32 tiles fit the array beside the rest, and taken in one pass over k
 * otherwise: then the order of the fp32 sums differs), but the temporaries (the
 * activations in matrix-operand order, the Q4_K group sums, the parts) live in a
 * 16 MiB array that is part of the library's device
 * image, one copy per GPU, held until the process ends; the call allocates
 * and frees nothing.  Shapes whose temporaries exceed the array fail with
 * RFQ_E_SIZE: ceil(m / 32) * ceil(k / 64) * 4096 bytes, plus ceil(m / 32) * k * 4
 * for RFQ_Q4_K (m * k up to about 7.8 million elements; 512 x 4096 takes 4.25 MiB).
 * Every call on a GPU shares that GPU's array: calls that may overlap on one
 * GPU (different streams, different threads) race; calls on one stream do not.
 * The first call on each device looks the array's address up (make that call
 * outside stream capture). */
RFQ_API int rfq_gemm_f16_static(int fmt, const void *d_w, size_t w_bytes, const void *d_a_f16, void *d_out,
                                int out_dtype, int m, int n, int k, void *stream);

/* The same GEMM with the re-ordering of the activations taken out of the call,
 * for several projections of one input (the Q, K and V weights of a layer,
 * gate and up): rfq_gemm_f16_arrange writes A[m, k] (fp16, 16-byte aligned, k a
 * multiple of 8) once, in matrix-operand order plus the per-group sums the
 * RFQ_Q4_K kernel wants, into a caller's buffer of
 * rfq_gemm_f16_arranged_bytes(m, k) bytes (16-byte aligned; 0 = bad shape);
 * rfq_gemm_f16_arranged multiplies any of the formats of rfq_gemm_f16 with it.
 * Results are bit-identical to rfq_gemm_f16 on the same A where that call takes
 * one pass over k (rfq_gemm_f16_k_parts(m, n, k) == 1; this entry point never
 * splits: it has no temporary for the parts).  Neither call
 * allocates or keeps anything, so both may be recorded under stream capture.
 * The reference has no fused prefill GEMM (see rfq_gemm_f16); its
 * counterpart is the shared input of the three SGEMMs of
 * HipBackend::mlp_swiglu (src/backend/hip_backend/backend.rs:1153-1278). */
RFQ_API size_t rfq_gemm_f16_arranged_bytes(int m, int k);
/* How many parts along k rfq_gemm_f16 takes for this shape (1 = a single pass). */
RFQ_API int rfq_gemm_f16_k_parts(int m, int n, int k);
RFQ_API int rfq_gemm_f16_arrange(const void *d_a_f16, int m, int k, void *d_arranged, size_t arranged_bytes,
                                 void *stream);
RFQ_API int rfq_gemm_f16_arranged(int fmt, const void *d_w, size_t w_bytes, const void *d_arranged,
                                  size_t arranged_bytes, void *d_out, int out_dtype, int m, int n, int k,
                                  void *stream);

/* MXFP matrices feed the gfx950 block-scaled matrix instruction, whose element
 * and scale encodings differ from the bytes ROCmForge stores (signed exponent
 * byte, its own E2M1/E2M3 value tables, a +-8 / +-7.5 clamp).  A matrix
 * [rows, k] (k a multiple of 128) is therefore re-encoded once, value for
 * value, into a caller-owned device buffer:
 *   RFQ_MX_FP4: every block of the matrix is expressible as OCP E2M1 codes
 *               with a (possibly shifted) E8M0 scale -- 4-bit operand, full rate;
 *   RFQ_MX_FP8: E4M3 codes, which hold every value the reference decoders can
 *               produce; always possible; half rate.  MXFP6 always takes this.
 * rfq_mx_prepared_bytes: buffer size for the given kind (AUTO -> the FP8 size).
 * rfq_mx_prepare: kind_req = AUTO picks FP4 when the whole matrix allows it
 *   (this reads one flag back and therefore synchronises the stream); FP8
 *   never synchronises; FP4 fails with RFQ_E_UNSUPPORTED (after a sync) when a
 *   block is not expressible.  *kind_out receives the encoding written.
 *   FP4_UNCHECKED (a request only; the buffer's kind is FP4) is FP4 without
 *   the read-back and the synchronisation, for activations re-encoded per
 *   prefill: the caller vouches that every block fits, which holds for
 *   whatever MxfpBlock::pack_mxfp4 (src/loader/mxfp.rs:118-161) produced (it
 *   never emits the sign-only code, the one value below the four codes'
 *   span); a block that does not fit is re-encoded wrongly without notice.
 *   rfq_mx_prepared_bytes takes FP4 for it.
 * This is the one-time weight upload step (src/loader/gguf/gpu_upload.rs:57-125
 * does the analogous dequantise-at-load for the K formats). */
RFQ_API size_t rfq_mx_prepared_bytes(int fmt, int kind, int rows, int k);
RFQ_API int rfq_mx_prepare(int fmt, int kind_req, const void *d_raw, size_t raw_bytes, int rows, int k,
                   void *d_prepared, size_t prepared_bytes, int *kind_out, void *stream);

/* d_out[m, n] = A[m, k] . W[n, k]^T from two prepared operands, fp32
 * accumulation in the matrix core, out_dtype RFQ_F32 or RFQ_BF16.
 * m, n multiples of 32 are not required; k a multiple of 128 is.
 * a_prep_bytes / w_prep_bytes are the sizes of the two prepared buffers: each
 * must be at least what rfq_mx_prepared_bytes gives for (a_kind, m, k) and
 * (w_kind, n, k) -- a buffer sized for RFQ_MX_AUTO that came out as FP4 is larger --
 * so a shape beyond what was prepared is refused (RFQ_E_SIZE) instead of read
 * out of bounds. */
RFQ_API int rfq_gemm_mx(const void *d_a_prep, size_t a_prep_bytes, int a_kind, const void *d_w_prep,
                size_t w_prep_bytes, int w_kind, void *d_out, int out_dtype, int m, int n, int k, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* RFQ_H */
