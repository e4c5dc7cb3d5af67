/*
 * rfq_bench.h -- timing loops exported by librfq for the benchmark driver.
 *
 * Not part of the operator surface: these are the native counterpart of the
 * hand-rolled "warm up, then time N iterations" loops in ROCmForge's
 * benches/matmul_bench.rs:343-378 and benches/dequant_bench.rs:391-404.  Each
 * enqueues `warmup` untimed and `steps` timed calls of the corresponding
 * rfq_* entry point back to back on `stream`, brackets the timed ones with HIP
 * events recorded on that same stream, synchronises, and returns the elapsed
 * device time of the timed region in milliseconds.  Keeping the loop native
 * keeps the host's launch rate above the ~10 us kernels being measured.
 */
#ifndef RFQ_BENCH_H
#define RFQ_BENCH_H

#include "rfq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Step i multiplies by weight copy d_w_copies[i % copies] (all of w_bytes):
 * with enough copies no step finds its weights in the last-level cache. */
RFQ_API int rfq_bench_gemv(int fmt, const void *const *d_w_copies, int copies, size_t w_bytes, const float *d_x,
                           float *d_y, int m, int n, int k, int warmup, int steps, void *stream,
                           float *elapsed_ms);

/* Where the time of one decode GEMV launch (m = 1) goes, seen from inside the kernel: after `warmup` ordinary calls
 * over the rotating weight copies, one launch of a build of the same kernel in which every wavefront reads the
 * constant 100 MHz clock (s_memrealtime, 10 ns a tick) at fixed points and stores the readings; the call returns
 * after the launch has finished.  d_trace (device memory, capacity_waves * 20 readings of 8 bytes) receives
 * [wavefront][reading]: 0 wavefront started, 1 its part of x in registers (the reading stands behind the requests for
 * x and for the first rows of weights, which issue in order and block while the CU's memory pipeline is full: with
 * the loads of x removed it comes no earlier), 2 x converted (before the barrier),
 * 3 past the barrier, 4 the prepared x of its units in registers, 5 + 2 i row i of its first group of rows in
 * registers, 6 + 2 i row i reduced (i < 7), 19 the group's results stored.  *waves = wavefronts written, 0 when the
 * kernel this format and shape take has no such build (Q4_K and MXFP4 with 65..128 units per row and seven rows
 * per group, GGUF_Q4_K with seven rows per group: the 14336 x 4096 projections). */
RFQ_API int rfq_bench_gemv_timeline(int fmt, const void *const *d_w_copies, int copies, size_t w_bytes, const float *d_x,
                                    float *d_y, int n, int k, int warmup, void *stream, unsigned long long *d_trace,
                                    size_t capacity_waves, int *waves, int *stamps_per_wave);

/* Step i reads input copy i % copies and writes the n_elems floats at
 * d_out + (i % out_copies) * n_elems: with enough of both, neither the packed
 * input nor the previous output of the same lines sits in the last-level cache. */
RFQ_API int rfq_bench_dequant(int fmt, const void *const *d_in_copies, int copies, size_t packed_bytes, float *d_out,
                              size_t n_elems, int out_copies, int warmup, int steps, void *stream, float *elapsed_ms);

/* rfq_get_rows in a native loop (step i gathers into d_out + (i % out_copies) * n_tokens * n_embd). */
RFQ_API int rfq_bench_get_rows(int fmt, const void *d_table, size_t table_bytes, int n_vocab, int n_embd,
                               const uint32_t *d_tokens, int n_tokens, float *d_out, int out_copies, int warmup,
                               int steps, void *stream, float *elapsed_ms);

/* Name and template arguments of the kernel that the calling thread's last rfq_gemv / rfq_rms_norm_gemv /
 * rfq_mlp_swiglu launch took ("" before the first), e.g. "gemv_idot_kernel<Q4_K,1,2,7>": lets the driver name the
 * kernel it timed from the dispatch actually taken instead of a constant. */
RFQ_API const char *rfq_bench_last_gemv_kernel(void);

/* The floor of a one-launch step that has to fetch `bytes` from HBM: a kernel that only reads copy i % copies
 * (16-byte loads, consecutive lanes on consecutive addresses, `depth` = 4, 8 or 16 loads of a thread in flight at
 * once, non-temporal when nt != 0), folds the words into one value and stores nothing, launched back to back like the
 * GEMV it is compared with: `blocks` workgroups of `threads` (a multiple of 64, at most 1024). */
RFQ_API int rfq_bench_read_floor(const void *const *d_copies, int copies, size_t bytes, int blocks, int threads, int nt,
                                 int depth, int warmup, int steps, void *stream, float *elapsed_ms);

RFQ_API int rfq_bench_gemm_f16(int fmt, const void *d_w, size_t w_bytes, const void *d_a_f16, void *d_out,
                               int out_dtype, int m, int n, int k, int warmup, int steps, void *stream,
                               float *elapsed_ms);

/* rfq_gemm_f16_arranged on activations arranged once before the loop. */
RFQ_API int rfq_bench_gemm_f16_arranged(int fmt, const void *d_w, size_t w_bytes, const void *d_arranged,
                                        size_t arranged_bytes, void *d_out, int out_dtype, int m, int n, int k,
                                        int warmup, int steps, void *stream, float *elapsed_ms);

RFQ_API int rfq_bench_gemm_mx(const void *d_a_prep, size_t a_prep_bytes, int a_kind, const void *d_w_prep,
                              size_t w_prep_bytes, int w_kind, void *d_out, int out_dtype, int m, int n, int k,
                              int warmup, int steps, void *stream, float *elapsed_ms);

/* A prefill step as a caller that holds raw MXFP4 activations runs it: re-encode A for the matrix core
 * (rfq_mx_prepare, RFQ_MX_FP4_UNCHECKED: no read-back, no synchronisation) into d_a_prep, then rfq_gemm_mx
 * against the weights prepared once at upload. */
RFQ_API int rfq_bench_gemm_mx_prefill(const void *d_a_raw, size_t a_raw_bytes, void *d_a_prep, size_t a_prep_bytes,
                                      const void *d_w_prep, size_t w_prep_bytes, int w_kind, void *d_out, int out_dtype,
                                      int m, int n, int k, int warmup, int steps, void *stream, float *elapsed_ms);

/* Step i runs the MLP over weight set i % copies.  one_call != 0: rfq_mlp_swiglu;
 * one_call == 0: the same arithmetic as five calls (rfq_rms_norm, rfq_gemv for
 * gate and up, rfq_swiglu, rfq_gemv for down), for comparison. */
RFQ_API int rfq_bench_mlp_swiglu(int fmt_gate_up, const void *const *d_gate_copies, const void *const *d_up_copies,
                                 size_t gate_up_bytes, int fmt_down, const void *const *d_down_copies,
                                 size_t down_bytes, int copies, const float *d_x, const float *d_norm_weight,
                                 float eps, float *d_out, int m, int hidden_size, int intermediate_size,
                                 void *d_scratch, size_t scratch_bytes, int one_call, int warmup, int steps,
                                 void *stream, float *elapsed_ms);

/* What the fp16 matrix pipe delivers, alone and beside the operand traffic of a fused kernel (the ceiling
 * rfq_gemm_f16 is held against): `workgroups` x `waves_per_workgroup` (4 or 8; one workgroup per CU) wavefronts each
 * run iters (even) rounds of independent matrix instructions -- variant 0: 8 x v_mfma_f32_32x32x16_f16 per round, 1:
 * 28 x v_mfma_f32_16x16x32_f16 -- plus, per round, valu_per_mfma packed fp16 multiplies per matrix instruction,
 * lds_reads_per_round 16-byte-per-lane fragment reads from LDS and global_loads_per_round 16-byte-per-lane loads from
 * a 2 MiB window in global memory (cache hits); loaded fragments are the next round's operands.  Only some
 * combinations are compiled (RFQ_E_UNSUPPORTED otherwise).  The kernel is launched `launches` times back to back; the
 * last launch is timed, and the shader clocks each wavefront counted around its loop (s_memtime, against the constant
 * 100 MHz clock) give clocks per instruction and SIMD and the clock the part held. */
RFQ_API int rfq_bench_mfma_f16_probe(int variant, int valu_per_mfma, int lds_reads_per_round, int global_loads_per_round,
                                     int workgroups, int waves_per_workgroup, int random_operands, int iters,
                                     int launches, void *stream, float *last_launch_us, float *clocks_per_mfma,
                                     float *shader_ghz, float *tflops);

#ifdef __cplusplus
}
#endif
#endif /* RFQ_BENCH_H */
