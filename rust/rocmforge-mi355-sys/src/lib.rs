//! Raw declarations of `librfq` (`include/rfq.h`), one for every exported function, in the header's order.
//!
//! Device pointers are what `HipBuffer::as_ptr()` returns (src/backend/hip_backend/memory.rs:540-547); a stream is
//! the backend's `hipStream_t` passed as `*mut c_void` (null = the default stream).  Every function returns an
//! `rfq_status` (`RFQ_OK` = 0 like `HIP_SUCCESS`, src/backend/hip_backend/ffi.rs:78); `rfq_last_error` gives the text.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_float, c_int, c_void};

// rfq_format: GgufTensorType ids (src/loader/tensor_type.rs:16-32) ...
pub const RFQ_Q4_0: c_int = 2;
pub const RFQ_Q8_0: c_int = 8;
pub const RFQ_Q2_K: c_int = 10;
pub const RFQ_Q3_K: c_int = 11;
pub const RFQ_Q4_K: c_int = 12;
pub const RFQ_Q5_K: c_int = 13;
pub const RFQ_Q6_K: c_int = 14;
pub const RFQ_MXFP4: c_int = 20;
pub const RFQ_MXFP6_E2M3: c_int = 21;
pub const RFQ_MXFP6_E3M2: c_int = 22;
// ... the block layouts of GGUF model files (100 + the ggml type id) ...
pub const RFQ_GGUF_Q4_0: c_int = 102;
pub const RFQ_GGUF_Q8_0: c_int = 108;
pub const RFQ_GGUF_Q4_K: c_int = 112;
pub const RFQ_GGUF_Q6_K: c_int = 114;
// ... and the decoders of src/kernels/matmul/quantized/ (200 + the id of the format they are a variant of)
pub const RFQ_MM_Q8_0: c_int = 208;
pub const RFQ_MM_Q4_K: c_int = 212;
pub const RFQ_MM_Q6_K: c_int = 214;
pub const RFQ_TABLE_F32: c_int = 0;
/// Or-ed into the `out_dtype` of `rfq_gemm_f16*`: one fp16 operand per weight instead of two.
pub const RFQ_GEMM_ONE_PLANE: c_int = 0x100;

// rfq_status
pub const RFQ_OK: c_int = 0;
pub const RFQ_E_BADARG: c_int = -1;
pub const RFQ_E_SIZE: c_int = -2;
pub const RFQ_E_UNSUPPORTED: c_int = -3;
pub const RFQ_E_HIP: c_int = -4;
pub const RFQ_E_NOMEM: c_int = -5;

// rfq_dtype
pub const RFQ_F32: c_int = 0;
pub const RFQ_F16: c_int = 1;
pub const RFQ_BF16: c_int = 2;

// rfq_mx_kind
pub const RFQ_MX_AUTO: c_int = 0;
pub const RFQ_MX_FP4: c_int = 4;
pub const RFQ_MX_FP8: c_int = 8;
pub const RFQ_MX_FP4_UNCHECKED: c_int = 0x104;

pub const RFQ_VERSION: c_int = 104;

#[link(name = "rfq")]
extern "C" {
    // ---- library
    pub fn rfq_version() -> c_int;
    pub fn rfq_last_error() -> *const c_char;
    pub fn rfq_release_temporaries() -> c_int;
    pub fn rfq_release_stream_temporaries(stream: *mut c_void) -> c_int;
    pub fn rfq_upload(h_src: *const c_void, bytes: usize, d_dst: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn rfq_block_elems(fmt: c_int) -> usize;
    pub fn rfq_block_bytes(fmt: c_int) -> usize;
    pub fn rfq_packed_bytes(fmt: c_int, n_elems: usize) -> usize;

    // ---- dequantisation
    pub fn rfq_dequant(fmt: c_int, d_packed: *const c_void, packed_bytes: usize, d_out: *mut f32, n_elems: usize,
                       stream: *mut c_void) -> c_int;
    pub fn rfq_dequant_upload(fmt: c_int, h_packed: *const u8, packed_bytes: usize, d_out: *mut f32, n_elems: usize,
                              stream: *mut c_void) -> c_int;
    pub fn rfq_dequant_host(fmt: c_int, h_packed: *const u8, packed_bytes: usize, h_out: *mut f32,
                            n_elems: usize) -> c_int;

    // ---- decode GEMV (and small batches)
    pub fn rfq_gemv(fmt: c_int, d_w: *const c_void, w_bytes: usize, d_x: *const f32, d_y: *mut f32, m: c_int, n: c_int,
                    k: c_int, stream: *mut c_void) -> c_int;
    pub fn rfq_gemv_kn(fmt: c_int, d_w: *const c_void, w_bytes: usize, d_x: *const f32, d_y: *mut f32, m: c_int,
                       n: c_int, k: c_int, stream: *mut c_void) -> c_int;
    pub fn rfq_matmul_q4_0(d_act: *const f32, d_w: *const u8, d_out: *mut f32, m: c_int, n: c_int, k: c_int,
                           stream: *mut c_void) -> c_int;
    pub fn rfq_matmul_q8_0(d_act: *const f32, d_w: *const u8, d_out: *mut f32, m: c_int, n: c_int, k: c_int,
                           stream: *mut c_void) -> c_int;
    pub fn rfq_matmul_q4_k(d_act: *const f32, d_w: *const u8, d_out: *mut f32, m: c_int, n: c_int, k: c_int,
                           stream: *mut c_void) -> c_int;
    pub fn rfq_matmul_q6_k(d_act: *const f32, d_w: *const u8, d_out: *mut f32, m: c_int, n: c_int, k: c_int,
                           stream: *mut c_void) -> c_int;
    pub fn rfq_matmul_host_weights(fmt: c_int, h_w: *const u8, w_bytes: usize, d_input: *const f32, n_rows: usize,
                                   n_cols: usize, d_out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn rfq_matmul_host_weights_kn(fmt: c_int, h_w: *const u8, w_bytes: usize, d_input: *const f32, n_rows: usize,
                                      n_cols: usize, d_out: *mut f32, stream: *mut c_void) -> c_int;

    // ---- embedding rows
    pub fn rfq_get_rows(fmt: c_int, d_table: *const c_void, table_bytes: usize, n_vocab: c_int, n_embd: c_int,
                        d_tokens: *const u32, n_tokens: c_int, d_out: *mut f32, d_status: *mut c_int,
                        stream: *mut c_void) -> c_int;

    // ---- neighbours of the matmul in a decoder layer
    pub fn rfq_rms_norm(d_input: *const f32, d_weight: *const f32, d_output: *mut f32, seq_len: c_int,
                        hidden_size: c_int, eps: c_float, stream: *mut c_void) -> c_int;
    pub fn rfq_swiglu(d_gate: *const f32, d_up: *const f32, d_output: *mut f32, seq_len: c_int,
                      intermediate_size: c_int, stream: *mut c_void) -> c_int;
    pub fn rfq_dequant_rms_norm(fmt: c_int, d_packed: *const c_void, packed_bytes: usize, d_weight: *const f32,
                                d_output: *mut f32, seq_len: c_int, hidden_size: c_int, eps: c_float,
                                stream: *mut c_void) -> c_int;
    pub fn rfq_rms_norm_gemv(fmt: c_int, d_w: *const c_void, w_bytes: usize, d_x: *const f32,
                             d_norm_weight: *const f32, eps: c_float, d_y: *mut f32, m: c_int, n: c_int, k: c_int,
                             d_scratch: *mut f32, stream: *mut c_void) -> c_int;
    pub fn rfq_mlp_scratch_bytes(m: c_int, hidden_size: c_int, intermediate_size: c_int) -> usize;
    pub fn rfq_mlp_swiglu(fmt_gate_up: c_int, d_gate_w: *const c_void, d_up_w: *const c_void, gate_up_bytes: usize,
                          fmt_down: c_int, d_down_w: *const c_void, down_bytes: usize, d_x: *const f32,
                          d_norm_weight: *const f32, eps: c_float, d_out: *mut f32, m: c_int, hidden_size: c_int,
                          intermediate_size: c_int, d_scratch: *mut c_void, scratch_bytes: usize,
                          stream: *mut c_void) -> c_int;

    // ---- prefill GEMM
    pub fn rfq_gemm_f16(fmt: c_int, d_w: *const c_void, w_bytes: usize, d_a_f16: *const c_void, d_out: *mut c_void,
                        out_dtype: c_int, m: c_int, n: c_int, k: c_int, stream: *mut c_void) -> c_int;
    pub fn rfq_gemm_f16_static(fmt: c_int, d_w: *const c_void, w_bytes: usize, d_a_f16: *const c_void,
                               d_out: *mut c_void, out_dtype: c_int, m: c_int, n: c_int, k: c_int,
                               stream: *mut c_void) -> c_int;
    pub fn rfq_gemm_f16_arranged_bytes(m: c_int, k: c_int) -> usize;
    pub fn rfq_gemm_f16_k_parts(m: c_int, n: c_int, k: c_int) -> c_int;
    pub fn rfq_gemm_f16_arrange(d_a_f16: *const c_void, m: c_int, k: c_int, d_arranged: *mut c_void,
                                arranged_bytes: usize, stream: *mut c_void) -> c_int;
    pub fn rfq_gemm_f16_arranged(fmt: c_int, d_w: *const c_void, w_bytes: usize, d_arranged: *const c_void,
                                 arranged_bytes: usize, d_out: *mut c_void, out_dtype: c_int, m: c_int, n: c_int,
                                 k: c_int, stream: *mut c_void) -> c_int;
    pub fn rfq_mx_prepared_bytes(fmt: c_int, kind: c_int, rows: c_int, k: c_int) -> usize;
    pub fn rfq_mx_prepare(fmt: c_int, kind_req: c_int, d_raw: *const c_void, raw_bytes: usize, rows: c_int, k: c_int,
                          d_prepared: *mut c_void, prepared_bytes: usize, kind_out: *mut c_int,
                          stream: *mut c_void) -> c_int;
    pub fn rfq_gemm_mx(d_a_prep: *const c_void, a_prep_bytes: usize, a_kind: c_int, d_w_prep: *const c_void,
                       w_prep_bytes: usize, w_kind: c_int, d_out: *mut c_void, out_dtype: c_int, m: c_int, n: c_int,
                       k: c_int, stream: *mut c_void) -> c_int;
}

/// Text of the last failure on this thread (`""` if none).
pub fn last_error() -> String {
    unsafe { std::ffi::CStr::from_ptr(rfq_last_error()) }.to_string_lossy().into_owned()
}
