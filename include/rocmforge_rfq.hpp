/*
 * rocmforge_rfq.hpp -- C++17 host-side mirror of the ROCmForge operator surface
 * for the quantized-weight path, on top of the C ABI in rfq.h.
 *
 * ROCmForge's host code is Rust; this header restates, name for name, the
 * types and functions its benches and tests use on this path, so that C++
 * callers (and the host tests in tests/host/) read like the reference's own:
 *
 *   GgufTensorType        src/loader/tensor_type.rs:16-112
 *   TensorShape           src/loader/mmap_loader.rs:117-174
 *   GgufTensor            src/loader/gguf_tensor.rs:8-75
 *   loader::dequant_*     src/loader/mod.rs:116-127, src/loader/dequant.rs:41-132
 *   loader::dequantize    src/loader/dequant.rs:673-700
 *   HipBuffer             src/backend/hip_backend/memory.rs:19-31, 540-580
 *   HipBackend            src/backend/hip_backend/backend.rs:104-200
 *   matmul_q4_0 / q8_0 / q4_k / q6_k
 *                         src/kernels/matmul/quantized/q4_0.rs:153, q8_0.rs:69, q4_k.rs:173, q6_k.rs:163
 *   matmul_q4_0_gpu       src/kernels/matmul/quantized/q4_0.rs:209-260
 *   dequantize_q4_0_kernel_cached, dequantize_q4_k_gpu_kernel, dequantize_q6_k_gpu_kernel
 *                         src/kernels/quant/q4_0.rs:107, q4_k.rs:99, q6_k.rs:102
 *   QuantFormat, QuantizedMatmulOp, BatchMatmulResult, BatchQuantizedMatmul
 *                         src/ggml/hip_backend/ops/batch_quantized.rs:20-255
 *   validate_matmul_q4_0 / q8_0 (the checks of execute_matmul_q4_0 / q8_0)
 *                         src/ggml/hip_backend/op_dispatch.rs:951-1083
 *   get_rows, validate_token_ids
 *                         src/ggml/hip_backend/ops/get_rows.rs:6-65
 *   rms_norm_gpu_kernel, swiglu_gpu_kernel
 *                         src/mlp/kernels.rs:261-330, 177-240
 *   fused_q4_0_rmsnorm    src/ggml/hip_backend/ops/fused_ops.rs:149-160
 *   DeviceTensor, mlp_swiglu (HipBackend::mlp_swiglu over quantised weights)
 *                         src/backend/hip_backend/backend.rs:1385-1388, 1153-1278
 *   Op (the quantised matmuls), execute_matmul_quantized
 *                         src/ggml/op.rs:4-30, src/ggml/hip_backend/op_dispatch.rs:951-1083
 *
 * Rust's Result<T, E> becomes Result<T> below (ok / value / error text); no
 * exceptions cross the C ABI.  Everything computes on the GPU through librfq:
 * there is no CPU fallback here.
 */
#ifndef ROCMFORGE_RFQ_HPP
#define ROCMFORGE_RFQ_HPP

#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdint>
#include <cstring>
#include <limits>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "rfq.h"

namespace rocmforge {

// ---- Result -----------------------------------------------------------------
template <typename T> struct Result {
    bool ok = false;
    T value{};
    std::string error;
    static Result Ok(T v) { Result r; r.ok = true; r.value = std::move(v); return r; }
    static Result Err(std::string e) { Result r; r.error = std::move(e); return r; }
    explicit operator bool() const { return ok; }
};
struct Unit {};
using Status = Result<Unit>;
inline Status ok_status() { return Status::Ok(Unit{}); }

namespace detail {
inline Status from_rfq(int rc, const char *what)
{
    if (rc == RFQ_OK) return ok_status();
    return Status::Err(std::string(what) + ": " + rfq_last_error());
}
inline size_t checked_mul(size_t a, size_t b)
{
    if (a != 0 && b > std::numeric_limits<size_t>::max() / a) return std::numeric_limits<size_t>::max();
    return a * b;
}
inline size_t div_ceil(size_t a, size_t b) { return (a + b - 1) / b; }
} // namespace detail

// ---- GgufTensorType (src/loader/tensor_type.rs:16-112) -------------------------
enum class GgufTensorType : uint32_t {
    F32 = 0, F16 = 1, Q4_0 = 2, Q8_0 = 8, Q2_K = 10, Q3_K = 11, Q4_K = 12, Q5_K = 13, Q6_K = 14,
    Mxfp4 = 20, Mxfp6E2m3 = 21, Mxfp6E3m2 = 22
};

inline Result<GgufTensorType> tensor_type_from_u32(uint32_t v)
{
    switch (v) {
    case 0: case 1: case 2: case 8: case 10: case 11: case 12: case 13: case 14: case 20: case 21: case 22:
        return Result<GgufTensorType>::Ok(static_cast<GgufTensorType>(v));
    default: // ids 3, 6, 7 (Q4_1, Q5_0, Q5_1) and everything unknown are rejected
        return Result<GgufTensorType>::Err("Unknown tensor type: " + std::to_string(v));
    }
}
inline const char *to_string(GgufTensorType t)
{
    switch (t) {
    case GgufTensorType::F32: return "FP32";
    case GgufTensorType::F16: return "FP16";
    case GgufTensorType::Q4_0: return "Q4_0";
    case GgufTensorType::Q8_0: return "Q8_0";
    case GgufTensorType::Q2_K: return "Q2_K";
    case GgufTensorType::Q3_K: return "Q3_K";
    case GgufTensorType::Q4_K: return "Q4_K";
    case GgufTensorType::Q5_K: return "Q5_K";
    case GgufTensorType::Q6_K: return "Q6_K";
    case GgufTensorType::Mxfp4: return "MXFP4";
    case GgufTensorType::Mxfp6E2m3: return "MXFP6_E2M3";
    case GgufTensorType::Mxfp6E3m2: return "MXFP6_E3M2";
    }
    return "?";
}
// elements per block (1 for the plain float types)
inline size_t block_size(GgufTensorType t)
{
    switch (t) {
    case GgufTensorType::F32: case GgufTensorType::F16: return 1;
    case GgufTensorType::Q4_0: case GgufTensorType::Q8_0: case GgufTensorType::Mxfp4:
    case GgufTensorType::Mxfp6E2m3: case GgufTensorType::Mxfp6E3m2: return 32;
    default: return 256;
    }
}
inline bool is_quantized(GgufTensorType t) { return t != GgufTensorType::F32 && t != GgufTensorType::F16; }
// bytes for the float types, the block size (in elements) for block formats -- as the reference defines it
inline size_t element_size(GgufTensorType t)
{
    if (t == GgufTensorType::F32) return 4;
    if (t == GgufTensorType::F16) return 2;
    return block_size(t);
}

// ---- TensorShape (src/loader/mmap_loader.rs:117-174) ---------------------------
class TensorShape {
public:
    static TensorShape from_dims(const std::vector<size_t> &dims)
    {
        TensorShape s;
        s.dims_ = dims;
        s.strides_.assign(dims.size(), 1);
        for (size_t i = dims.size(); i-- > 0;)
            if (i + 1 < dims.size()) s.strides_[i] = detail::checked_mul(s.strides_[i + 1], dims[i + 1]);
        return s;
    }
    const std::vector<size_t> &dims() const { return dims_; }
    const std::vector<size_t> &strides() const { return strides_; }
    size_t total_elements() const
    {
        size_t n = 1;
        for (size_t d : dims_) n = detail::checked_mul(n, d);
        return n;
    }

private:
    std::vector<size_t> dims_, strides_;
};

// ---- GgufTensor (src/loader/gguf_tensor.rs:8-75) ---------------------------------
struct GgufTensor {
    std::string name;
    TensorShape shape;
    GgufTensorType tensor_type = GgufTensorType::F32;
    std::string quant_type;
    uint64_t offset = 0;
    std::vector<uint8_t> data;

    GgufTensor() = default;
    GgufTensor(std::string n, TensorShape s, GgufTensorType t, uint64_t off)
        : name(std::move(n)), shape(std::move(s)), tensor_type(t), quant_type(to_string(t)), offset(off)
    {
    }
    size_t total_elements() const { return shape.total_elements(); }
    // Bytes the loader expects.  Q4_0 is counted as 4 + 32 per block here although the
    // decoder strides by 20 (src/loader/gguf_tensor.rs:45-49): kept as the reference has it.
    size_t data_size() const
    {
        const size_t n = total_elements();
        switch (tensor_type) {
        case GgufTensorType::F32: return detail::checked_mul(n, 4);
        case GgufTensorType::F16: return detail::checked_mul(n, 2);
        case GgufTensorType::Q4_0: case GgufTensorType::Q8_0: return detail::checked_mul(detail::div_ceil(n, 32), 36);
        case GgufTensorType::Mxfp4: return detail::checked_mul(detail::div_ceil(n, 32), 17);
        case GgufTensorType::Mxfp6E2m3: case GgufTensorType::Mxfp6E3m2:
            return detail::checked_mul(detail::div_ceil(n, 32), 25);
        default: return detail::checked_mul(detail::div_ceil(n, 256), 256);
        }
    }
};

// ---- loader ---------------------------------------------------------------------
namespace loader {

namespace detail_ {
inline std::vector<float> through_gpu(int fmt, const uint8_t *data, size_t len, size_t n_elements)
{
    // the reference returns n_elements values, zero where the input was too short
    std::vector<float> out(n_elements, 0.0f);
    if (n_elements == 0) return out;
    static const uint8_t none = 0;
    int rc = rfq_dequant_host(fmt, len ? data : &none, len, out.data(), n_elements);
    if (rc != RFQ_OK) out.assign(n_elements, std::numeric_limits<float>::quiet_NaN()); // loud, not silent
    return out;
}
} // namespace detail_

inline std::vector<float> dequant_q4_0(const std::vector<uint8_t> &data, size_t n_elements)
{
    return detail_::through_gpu(RFQ_Q4_0, data.data(), data.size(), n_elements);
}
inline std::vector<float> dequant_q8_0(const std::vector<uint8_t> &data, size_t n_elements)
{
    return detail_::through_gpu(RFQ_Q8_0, data.data(), data.size(), n_elements);
}
inline std::vector<float> dequant_q4_k(const std::vector<uint8_t> &data, size_t n_elements)
{
    return detail_::through_gpu(RFQ_Q4_K, data.data(), data.size(), n_elements);
}
inline std::vector<float> dequant_q6_k(const std::vector<uint8_t> &data, size_t n_elements)
{
    return detail_::through_gpu(RFQ_Q6_K, data.data(), data.size(), n_elements);
}
// dequant_q5_k / dequant_q3_k / dequant_q2_k (src/loader/dequant.rs:150-225, 243-320, 326-420)
inline Result<std::vector<float>> dequant_q5_k(const GgufTensor &t)
{
    return Result<std::vector<float>>::Ok(detail_::through_gpu(RFQ_Q5_K, t.data.data(), t.data.size(), t.total_elements()));
}
inline Result<std::vector<float>> dequant_q3_k(const GgufTensor &t)
{
    return Result<std::vector<float>>::Ok(detail_::through_gpu(RFQ_Q3_K, t.data.data(), t.data.size(), t.total_elements()));
}
inline Result<std::vector<float>> dequant_q2_k(const GgufTensor &t)
{
    return Result<std::vector<float>>::Ok(detail_::through_gpu(RFQ_Q2_K, t.data.data(), t.data.size(), t.total_elements()));
}
inline Result<std::vector<float>> dequant_mxfp4(const GgufTensor &t)
{
    return Result<std::vector<float>>::Ok(detail_::through_gpu(RFQ_MXFP4, t.data.data(), t.data.size(), t.total_elements()));
}
inline Result<std::vector<float>> dequant_mxfp6(const GgufTensor &t)
{
    return Result<std::vector<float>>::Ok(
        detail_::through_gpu(RFQ_MXFP6_E2M3, t.data.data(), t.data.size(), t.total_elements()));
}

// src/loader/dequant.rs:673-700.  F32 / F16 are plain host conversions
// (chunks_exact: a trailing partial element is dropped).
inline Result<std::vector<float>> dequantize(const GgufTensor &t)
{
    using R = Result<std::vector<float>>;
    switch (t.tensor_type) {
    case GgufTensorType::F32: {
        std::vector<float> out(t.data.size() / 4);
        std::memcpy(out.data(), t.data.data(), out.size() * 4);
        return R::Ok(std::move(out));
    }
    case GgufTensorType::F16: {
        std::vector<float> out(t.data.size() / 2);
        for (size_t i = 0; i < out.size(); i++) {
            uint16_t h;
            std::memcpy(&h, t.data.data() + 2 * i, 2);
            uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u, bits;
            if (e == 0) {
                if (m == 0) bits = sign;
                else { // subnormal: normalise
                    int sh = 0;
                    while (!(m & 1024u)) { m <<= 1; sh++; }
                    bits = sign | ((uint32_t)(113 - sh) << 23) | ((m & 1023u) << 13);
                }
            } else if (e == 31) bits = sign | 0x7F800000u | (m << 13);
            else bits = sign | ((e + 112u) << 23) | (m << 13);
            std::memcpy(&out[i], &bits, 4);
        }
        return R::Ok(std::move(out));
    }
    case GgufTensorType::Q4_0: return R::Ok(dequant_q4_0(t.data, t.total_elements()));
    case GgufTensorType::Q8_0: return R::Ok(dequant_q8_0(t.data, t.total_elements()));
    case GgufTensorType::Q4_K: return R::Ok(dequant_q4_k(t.data, t.total_elements()));
    case GgufTensorType::Q6_K: return R::Ok(dequant_q6_k(t.data, t.total_elements()));
    case GgufTensorType::Q2_K: return dequant_q2_k(t);
    case GgufTensorType::Q3_K: return dequant_q3_k(t);
    case GgufTensorType::Q5_K: return dequant_q5_k(t);
    case GgufTensorType::Mxfp4: return dequant_mxfp4(t);
    case GgufTensorType::Mxfp6E2m3: case GgufTensorType::Mxfp6E3m2: return dequant_mxfp6(t);
    default: return R::Err(std::string("dequantize: ") + to_string(t.tensor_type) + " is outside this library's path");
    }
}

} // namespace loader

// ---- HipBuffer / HipBackend -------------------------------------------------------
class HipBuffer {
public:
    static Result<HipBuffer> create(size_t size)
    {
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, size ? size : 1);
        if (e != hipSuccess) return Result<HipBuffer>::Err(std::string("hipMalloc failed: ") + hipGetErrorString(e));
        HipBuffer b;
        b.inner_ = std::shared_ptr<void>(p, [](void *q) { (void)hipFree(q); }); // freed on the last drop
        b.size_ = size;
        return Result<HipBuffer>::Ok(std::move(b));
    }
    size_t size() const { return size_; }
    void *as_ptr() const { return inner_.get(); }
    template <typename T> Status copy_from_host(const std::vector<T> &src)
    {
        const size_t bytes = src.size() * sizeof(T);
        if (bytes > size_) return Status::Err("copy_from_host: source larger than the buffer");
        hipError_t e = hipSuccess;
        if (bytes >= ((size_t)1 << 20)) {
            // large sources (tensor data) go through the library's pinned staging ring; the copy stays
            // synchronous, as the reference's hipMemcpy is (src/backend/hip_backend/memory.rs:135-170)
            Status up = detail::from_rfq(rfq_upload(src.data(), bytes, as_ptr(), nullptr), "copy_from_host");
            if (!up.ok) return up;
            e = hipStreamSynchronize(nullptr);
        } else {
            e = hipMemcpy(as_ptr(), src.data(), bytes, hipMemcpyHostToDevice);
        }
        return e == hipSuccess ? ok_status() : Status::Err(std::string("hipMemcpy H2D failed: ") + hipGetErrorString(e));
    }
    template <typename T> Status copy_to_host(std::vector<T> &dst) const
    {
        if (dst.size() * sizeof(T) > size_) return Status::Err("copy_to_host: destination larger than the buffer");
        hipError_t e = hipMemcpy(dst.data(), as_ptr(), dst.size() * sizeof(T), hipMemcpyDeviceToHost);
        return e == hipSuccess ? ok_status() : Status::Err(std::string("hipMemcpy D2H failed: ") + hipGetErrorString(e));
    }

private:
    std::shared_ptr<void> inner_;
    size_t size_ = 0;
};

// One stream, as the reference's process-wide backend has (the default stream here).
class HipBackend {
public:
    static Result<HipBackend> create()
    {
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess || n == 0) return Result<HipBackend>::Err("no HIP device");
        return Result<HipBackend>::Ok(HipBackend{});
    }
    void *stream() const { return nullptr; }
    Status synchronize() const
    {
        hipError_t e = hipStreamSynchronize(nullptr);
        return e == hipSuccess ? ok_status() : Status::Err(std::string("synchronize failed: ") + hipGetErrorString(e));
    }
};

// ---- dequantisation to device buffers (src/kernels/quant/q4_0.rs:107 and twins) ------
inline Status dequantize_q4_0_kernel_cached(const HipBackend &b, const std::vector<uint8_t> &q, const HipBuffer &out,
                                            size_t num_elements)
{
    if (out.size() < num_elements * sizeof(float)) return Status::Err("output buffer too small");
    return detail::from_rfq(rfq_dequant_upload(RFQ_Q4_0, q.data(), q.size(), (float *)out.as_ptr(), num_elements, b.stream()),
                            "dequantize_q4_0_kernel_cached");
}
inline Status dequantize_q4_k_gpu_kernel(const HipBackend &b, const std::vector<uint8_t> &q, const HipBuffer &out,
                                         size_t num_elements)
{
    if (out.size() < num_elements * sizeof(float)) return Status::Err("output buffer too small");
    return detail::from_rfq(rfq_dequant_upload(RFQ_Q4_K, q.data(), q.size(), (float *)out.as_ptr(), num_elements, b.stream()),
                            "dequantize_q4_k_gpu_kernel");
}
inline Status dequantize_q6_k_gpu_kernel(const HipBackend &b, const std::vector<uint8_t> &q, const HipBuffer &out,
                                         size_t num_elements)
{
    if (out.size() < num_elements * sizeof(float)) return Status::Err("output buffer too small");
    return detail::from_rfq(rfq_dequant_upload(RFQ_Q6_K, q.data(), q.size(), (float *)out.as_ptr(), num_elements, b.stream()),
                            "dequantize_q6_k_gpu_kernel");
}

// ---- quantized matmul (src/kernels/matmul/quantized/*.rs) ---------------------------
// Host weights, device input [1 x n_cols] and output [1 x n_rows]; synchronous like the reference.
inline Status matmul_host(int fmt, const char *who, const HipBackend &b, const std::vector<uint8_t> &w,
                          const HipBuffer &input, size_t n_rows, size_t n_cols, const HipBuffer &output)
{
    if (input.size() < n_cols * sizeof(float)) return Status::Err(std::string(who) + ": input buffer too small");
    if (output.size() < n_rows * sizeof(float)) return Status::Err(std::string(who) + ": output buffer too small");
    return detail::from_rfq(rfq_matmul_host_weights(fmt, w.data(), w.size(), (const float *)input.as_ptr(), n_rows, n_cols,
                                                    (float *)output.as_ptr(), b.stream()),
                            who);
}
inline Status matmul_q4_0(const HipBackend &b, const std::vector<uint8_t> &w, const HipBuffer &in, size_t n_rows,
                          size_t n_cols, const HipBuffer &out)
{
    return matmul_host(RFQ_Q4_0, "matmul_q4_0", b, w, in, n_rows, n_cols, out);
}
inline Status matmul_q8_0(const HipBackend &b, const std::vector<uint8_t> &w, const HipBuffer &in, size_t n_rows,
                          size_t n_cols, const HipBuffer &out)
{
    return matmul_host(RFQ_Q8_0, "matmul_q8_0", b, w, in, n_rows, n_cols, out);
}
inline Status matmul_q4_k(const HipBackend &b, const std::vector<uint8_t> &w, const HipBuffer &in, size_t n_rows,
                          size_t n_cols, const HipBuffer &out)
{
    return matmul_host(RFQ_Q4_K, "matmul_q4_k", b, w, in, n_rows, n_cols, out);
}
inline Status matmul_q6_k(const HipBackend &b, const std::vector<uint8_t> &w, const HipBuffer &in, size_t n_rows,
                          size_t n_cols, const HipBuffer &out)
{
    return matmul_host(RFQ_Q6_K, "matmul_q6_k", b, w, in, n_rows, n_cols, out);
}
// raw device pointers, argument order (activations, weights, output, m, n, k)
inline Status matmul_q4_0_gpu(const HipBackend &b, const float *act, const uint8_t *w, float *out, size_t m, size_t n,
                              size_t k)
{
    return detail::from_rfq(rfq_matmul_q4_0(act, w, out, (int)m, (int)n, (int)k, b.stream()), "matmul_q4_0_gpu");
}

// ---- what the reference computes on the bytes (the other orientation, the module's own decoders) ----
// The wrappers above read W as [n_rows, n_cols], the layout the reference documents
// (src/kernels/matmul/quantized/q4_0.rs:139-148).  Its code does something else with the same buffer: the fused
// kernel indexes k_idx * n + col (kernels/q4_0_matmul.hip:207) and the CPU paths hand the flat dequantised array
// to the f32 matmul as b[k, n] (cpu_matmul_f32, src/tensor/matmul.rs:219-233), so out[j] = sum_l in[l] * Wd[l * n_rows + j].
// These reproduce those numbers; `layout` selects between the two readings.
enum class WeightLayout { RowsOfK /* documented */, FlatKN /* computed */ };

// matmul_q4_0_cpu_fallback (src/kernels/matmul/quantized/q4_0.rs:274-311): dequantize_q4_0 (same file, :89-134: the
// loader's arithmetic), then the f32 matmul with m = 1, k = n_cols, n = n_rows over the flat array.
inline Status matmul_q4_0_cpu_fallback(const HipBackend &b, const std::vector<uint8_t> &w, const HipBuffer &in,
                                       size_t n_rows, size_t n_cols, const HipBuffer &out)
{
    if (in.size() < n_cols * sizeof(float)) return Status::Err("matmul_q4_0_cpu_fallback: input buffer too small");
    if (out.size() < n_rows * sizeof(float)) return Status::Err("matmul_q4_0_cpu_fallback: output buffer too small");
    return detail::from_rfq(rfq_matmul_host_weights_kn(RFQ_Q4_0, w.data(), w.size(), (const float *)in.as_ptr(), n_rows, n_cols,
                                                       (float *)out.as_ptr(), b.stream()),
                            "matmul_q4_0_cpu_fallback");
}
// The body of matmul_q8_0 as the reference has it (quantized/q8_0.rs:69-106): its own dequantize_q8_0 (:18-56, the
// bytes as two's-complement int8), then the same f32 matmul over the flat array.
inline Status matmul_q8_0_as_computed(const HipBackend &b, const std::vector<uint8_t> &w, const HipBuffer &in, size_t n_rows,
                                      size_t n_cols, const HipBuffer &out)
{
    if (in.size() < n_cols * sizeof(float)) return Status::Err("matmul_q8_0: input buffer too small");
    if (out.size() < n_rows * sizeof(float)) return Status::Err("matmul_q8_0: output buffer too small");
    return detail::from_rfq(rfq_matmul_host_weights_kn(RFQ_MM_Q8_0, w.data(), w.size(), (const float *)in.as_ptr(), n_rows,
                                                       n_cols, (float *)out.as_ptr(), b.stream()),
                            "matmul_q8_0");
}
// matmul_q4_0_gpu with the indexing of the kernel it launches (quantized/q4_0.rs:209-260, kernels/q4_0_matmul.hip:207).
inline Status matmul_q4_0_gpu(const HipBackend &b, const float *act, const uint8_t *w, float *out, size_t m, size_t n,
                              size_t k, WeightLayout layout)
{
    if (layout == WeightLayout::RowsOfK) return matmul_q4_0_gpu(b, act, w, out, m, n, k);
    return detail::from_rfq(rfq_gemv_kn(RFQ_Q4_0, w, detail::checked_mul(n, k) / 32 * 20, act, out, (int)m, (int)n, (int)k, b.stream()),
                            "matmul_q4_0_gpu");
}
// The module's CPU decoders, evaluated on the GPU (bit-exact): dequantize_q8_0 / dequantize_q4_k / dequantize_q6_k of
// src/kernels/matmul/quantized/ (q8_0.rs:18-56, q4_k.rs:90-148, q6_k.rs:90-148); dequantize_q4_0 (q4_0.rs:89-134) is
// loader::dequant_q4_0.
namespace matmul_quantized {
inline std::vector<float> dequantize_q4_0(const std::vector<uint8_t> &d, size_t n) { return loader::dequant_q4_0(d, n); }
inline std::vector<float> dequantize_q8_0(const std::vector<uint8_t> &d, size_t n) { return loader::detail_::through_gpu(RFQ_MM_Q8_0, d.data(), d.size(), n); }
inline std::vector<float> dequantize_q4_k(const std::vector<uint8_t> &d, size_t n) { return loader::detail_::through_gpu(RFQ_MM_Q4_K, d.data(), d.size(), n); }
inline std::vector<float> dequantize_q6_k(const std::vector<uint8_t> &d, size_t n) { return loader::detail_::through_gpu(RFQ_MM_Q6_K, d.data(), d.size(), n); }
} // namespace matmul_quantized

// ---- batch description types (src/ggml/hip_backend/ops/batch_quantized.rs:20-255) --------
enum class QuantFormat { Q4_0, Q4_K, Q6_K, Q8_0 };
inline float bytes_per_element(QuantFormat f)
{
    switch (f) {
    case QuantFormat::Q4_0: return 20.0f / 32.0f;
    case QuantFormat::Q8_0: return 36.0f / 32.0f;
    default: return 1.0f;
    }
}
inline const char *name(QuantFormat f)
{
    switch (f) {
    case QuantFormat::Q4_0: return "Q4_0";
    case QuantFormat::Q4_K: return "Q4_K";
    case QuantFormat::Q6_K: return "Q6_K";
    default: return "Q8_0";
    }
}
inline int rfq_format_of(QuantFormat f)
{
    switch (f) {
    case QuantFormat::Q4_0: return RFQ_Q4_0;
    case QuantFormat::Q4_K: return RFQ_Q4_K;
    case QuantFormat::Q6_K: return RFQ_Q6_K;
    default: return RFQ_Q8_0;
    }
}
struct QuantizedMatmulOp {
    std::vector<uint8_t> weights; // [n_rows x n_cols], row-major blocks
    size_t m = 1, n = 0, k = 0;
    QuantFormat format = QuantFormat::Q4_0;
    QuantizedMatmulOp(std::vector<uint8_t> w, size_t n_rows, size_t n_cols, QuantFormat f)
        : weights(std::move(w)), m(1), n(n_rows), k(n_cols), format(f)
    {
    }
    Status execute(const HipBackend &b, const HipBuffer &input, const HipBuffer &output) const
    {
        return matmul_host(rfq_format_of(format), name(format), b, weights, input, n, k, output);
    }
};

// BatchMatmulResult, BatchQuantizedMatmul (src/ggml/hip_backend/ops/batch_quantized.rs:92-255): a list of
// quantised matmuls that share one input vector, run one after the other, each into an output it allocates.
struct BatchMatmulResult {
    std::vector<HipBuffer> outputs;
    std::vector<float> timings_ms;
    float total_time_ms = 0.0f;
};
class BatchQuantizedMatmul {
public:
    explicit BatchQuantizedMatmul(HipBackend backend) : backend_(backend) {}
    BatchQuantizedMatmul with_profiling() const { BatchQuantizedMatmul b = *this; b.enable_profiling_ = true; return b; }
    BatchQuantizedMatmul with_async() const { BatchQuantizedMatmul b = *this; b.enable_async_ = true; return b; }
    // process_batch (:139-160)
    Result<std::vector<HipBuffer>> process_batch(const HipBuffer &input, const std::vector<QuantizedMatmulOp> &ops) const
    {
        std::vector<HipBuffer> results;
        results.reserve(ops.size());
        for (const QuantizedMatmulOp &op : ops) {
            auto out = HipBuffer::create(op.m * op.n * sizeof(float));
            if (!out.ok) return Result<std::vector<HipBuffer>>::Err(out.error);
            Status st = op.execute(backend_, input, out.value);
            if (!st.ok) return Result<std::vector<HipBuffer>>::Err(std::string(name(op.format)) + " matmul failed: " + st.error);
            results.push_back(out.value);
        }
        return Result<std::vector<HipBuffer>>::Ok(std::move(results));
    }
    // process_batch_profiled (:166-190): host wall-clock per operation (each operation synchronises)
    Result<BatchMatmulResult> process_batch_profiled(const HipBuffer &input, const std::vector<QuantizedMatmulOp> &ops) const
    {
        BatchMatmulResult res;
        const auto start = std::chrono::steady_clock::now();
        for (const QuantizedMatmulOp &op : ops) {
            auto out = HipBuffer::create(op.m * op.n * sizeof(float));
            if (!out.ok) return Result<BatchMatmulResult>::Err(out.error);
            const auto t0 = std::chrono::steady_clock::now();
            Status st = op.execute(backend_, input, out.value);
            if (!st.ok) return Result<BatchMatmulResult>::Err(std::string(name(op.format)) + " matmul failed: " + st.error);
            res.timings_ms.push_back(std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count());
            res.outputs.push_back(out.value);
        }
        res.total_time_ms = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - start).count();
        return Result<BatchMatmulResult>::Ok(std::move(res));
    }

private:
    HipBackend backend_;
    bool enable_profiling_ = false, enable_async_ = false;
};

// The shape checks of execute_matmul_q4_0 / q8_0 (src/ggml/hip_backend/op_dispatch.rs:951-1083):
// 2-D operands, weight bytes = ceil(rows*cols/32) * block bytes, input k = weight columns.
inline Status validate_matmul(const char *op, size_t block_bytes, const std::vector<size_t> &weights_shape,
                              size_t weights_bytes, const std::vector<size_t> &input_shape)
{
    if (weights_shape.size() != 2 || input_shape.size() != 2) return Status::Err(std::string(op) + " expects 2D tensors");
    const size_t n_rows = weights_shape[0], n_cols = weights_shape[1];
    const size_t expected = ((n_rows * n_cols + 31) / 32) * block_bytes;
    if (weights_bytes != expected)
        return Status::Err(std::string(op) + " weights size mismatch: expected " + std::to_string(expected) +
                           " bytes, got " + std::to_string(weights_bytes));
    if (input_shape[1] != n_cols)
        return Status::Err(std::string(op) + " dimension mismatch: k=" + std::to_string(input_shape[1]) +
                           " weights_k=" + std::to_string(n_cols));
    return ok_status();
}
inline Status validate_matmul_q4_0(const std::vector<size_t> &ws, size_t wbytes, const std::vector<size_t> &is)
{
    return validate_matmul("MatMulQ4_0", 20, ws, wbytes, is);
}
inline Status validate_matmul_q8_0(const std::vector<size_t> &ws, size_t wbytes, const std::vector<size_t> &is)
{
    return validate_matmul("MatMulQ8_0", 36, ws, wbytes, is);
}

// ---- GetRows (src/ggml/hip_backend/ops/get_rows.rs) ----------------------------------
// validate_token_ids (:55-65): the first id outside the vocabulary is an error.
inline Status validate_token_ids(const std::vector<uint32_t> &tokens, size_t vocab_size)
{
    for (uint32_t t : tokens)
        if ((size_t)t >= vocab_size)
            return Status::Err("Token ID " + std::to_string(t) + " exceeds vocab size " + std::to_string(vocab_size));
    return ok_status();
}
// get_rows (:6-53), RowMajor: output row i = table row tokens[i].  `format` is a
// block format for a packed table or RFQ_TABLE_F32 for the f32 table the
// reference holds; the ids go to the device once and are read there.
inline Status get_rows(const HipBackend &b, const HipBuffer &weights, const std::vector<uint32_t> &tokens, size_t n_embd,
                       size_t n_vocab, int format, const HipBuffer &output)
{
    Status ids = validate_token_ids(tokens, n_vocab);          // same error, same moment as the reference (:18-23)
    if (!ids.ok) return ids;
    if (output.size() < tokens.size() * n_embd * sizeof(float)) return Status::Err("get_rows: output buffer too small");
    if (tokens.empty()) return ok_status();
    auto dev_tokens = HipBuffer::create(tokens.size() * sizeof(uint32_t));
    if (!dev_tokens.ok) return Status::Err(dev_tokens.error);
    Status up = dev_tokens.value.copy_from_host(tokens);
    if (!up.ok) return up;
    int rc = rfq_get_rows(format, weights.as_ptr(), weights.size(), (int)n_vocab, (int)n_embd,
                          (const uint32_t *)dev_tokens.value.as_ptr(), (int)tokens.size(), (float *)output.as_ptr(), nullptr,
                          b.stream());
    if (rc != RFQ_OK) return detail::from_rfq(rc, "get_rows");
    return b.synchronize();                                    // the token buffer is dropped on return
}

// ---- neighbours of the matmul in a decoder layer -------------------------------------
// rms_norm_gpu_kernel (src/mlp/kernels.rs:261-330): raw device pointers, enqueue only; the
// caller synchronises on the same backend, as the reference's doc comment demands.
inline Status rms_norm_gpu_kernel(const HipBackend &b, const float *input, const float *weight, float *output,
                                  uint32_t seq_len, uint32_t hidden_size, float eps)
{
    return detail::from_rfq(rfq_rms_norm(input, weight, output, (int)seq_len, (int)hidden_size, eps, b.stream()),
                            "Failed to launch rms_norm kernel");
}
// swiglu_gpu_kernel (src/mlp/kernels.rs:177-240): output = gate * swish(up).
inline Status swiglu_gpu_kernel(const HipBackend &b, const float *gate, const float *up, float *output, uint32_t seq_len,
                                uint32_t intermediate_size)
{
    return detail::from_rfq(rfq_swiglu(gate, up, output, (int)seq_len, (int)intermediate_size, b.stream()),
                            "Failed to launch swiglu kernel");
}
// fused_q4_0_rmsnorm (src/ggml/hip_backend/ops/fused_ops.rs:149-160): packed Q4_0 rows in, normalised f32 rows out.
inline Status fused_q4_0_rmsnorm(const HipBackend &b, const uint8_t *q4_0_input, const float *weight, float *output,
                                 uint32_t seq_len, uint32_t hidden_size, float eps)
{
    const size_t bytes = (size_t)seq_len * (hidden_size / 32) * 20;
    return detail::from_rfq(rfq_dequant_rms_norm(RFQ_Q4_0, q4_0_input, bytes, weight, output, (int)seq_len, (int)hidden_size,
                                                 eps, b.stream()),
                            "Fused dequant+RMSNorm kernel failed");
}

// DeviceTensor (src/backend/hip_backend/backend.rs:1385-1388): a device buffer and its shape; `format` is
// RFQ_TABLE_F32 for f32 data or the block format of packed data (the reference's tensors are f32 only).
struct DeviceTensor {
    HipBuffer buffer;
    TensorShape shape;
    int format = RFQ_TABLE_F32;
};

// HipBackend::mlp_swiglu (src/backend/hip_backend/backend.rs:1153-1278) with the three matrices quantised:
// gate and up [intermediate_size, hidden_size], down [hidden_size, intermediate_size] (rows are outputs, as
// the quantised matmuls store them), hidden_states and output f32 [seq_len, hidden_size], seq_len <= 8.
// The reference's shape checks, in its order and wording; no temporaries are left behind and the call
// synchronises before returning, as the reference does.
inline Status mlp_swiglu(const HipBackend &b, const DeviceTensor &hidden_states, const DeviceTensor &gate_weight,
                         const DeviceTensor &up_weight, const DeviceTensor &down_weight, DeviceTensor &output)
{
    const auto &hs = hidden_states.shape.dims(), &gs = gate_weight.shape.dims(), &us = up_weight.shape.dims(),
               &ds = down_weight.shape.dims(), &os = output.shape.dims();
    if (hs.size() != 2) return Status::Err("hidden_states must be 2D [seq_len, hidden_size]");
    if (gs.size() != 2 || gs[1] != hs[1]) return Status::Err("gate_weight must be 2D [intermediate_size, hidden_size]");
    if (us.size() != 2 || us[1] != hs[1]) return Status::Err("up_weight must be 2D [intermediate_size, hidden_size]");
    if (ds.size() != 2 || ds[0] != hs[1]) return Status::Err("down_weight must be 2D [hidden_size, intermediate_size]");
    if (os != hs) return Status::Err("output must match hidden_states shape [seq_len, hidden_size]");
    const size_t seq_len = hs[0], hidden_size = hs[1], intermediate_size = gs[0];
    if (us[0] != intermediate_size || ds[1] != intermediate_size) return Status::Err("All intermediate dimensions must match");
    if (gate_weight.format != up_weight.format) return Status::Err("gate_weight and up_weight must share a format");
    const size_t scratch_bytes = rfq_mlp_scratch_bytes((int)seq_len, (int)hidden_size, (int)intermediate_size);
    auto scratch = HipBuffer::create(scratch_bytes);
    if (!scratch.ok) return Status::Err("Failed to allocate SwiGLU buffer: " + scratch.error);
    int rc = rfq_mlp_swiglu(gate_weight.format, gate_weight.buffer.as_ptr(), up_weight.buffer.as_ptr(),
                            gate_weight.buffer.size(), down_weight.format, down_weight.buffer.as_ptr(),
                            down_weight.buffer.size(), (const float *)hidden_states.buffer.as_ptr(), nullptr, 0.0f,
                            (float *)output.buffer.as_ptr(), (int)seq_len, (int)hidden_size, (int)intermediate_size,
                            scratch.value.as_ptr(), scratch_bytes, b.stream());
    if (rc != RFQ_OK) return detail::from_rfq(rc, "mlp_swiglu");
    return b.synchronize();
}

// ---- quantised matmul ops over device-resident weights ------------------------------------
// Op (src/ggml/op.rs:4-30) has MatMulQ4_0 and MatMulQ8_0; the other four formats of this path get
// ops of the same shape.  execute_matmul_q4_0 / q8_0 (src/ggml/hip_backend/op_dispatch.rs:951-1083)
// copy the weights device -> host and hand them to matmul_q4_0, which uploads them again; here
// the packed weights stay where they are.  Checks, order and wording follow the reference.
enum class Op { MatMulQ4_0, MatMulQ8_0, MatMulQ4_K, MatMulQ6_K, MatMulMxfp4, MatMulMxfp6 };
inline const char *name(Op op)
{
    switch (op) {
    case Op::MatMulQ4_0: return "MatMulQ4_0";
    case Op::MatMulQ8_0: return "MatMulQ8_0";
    case Op::MatMulQ4_K: return "MatMulQ4_K";
    case Op::MatMulQ6_K: return "MatMulQ6_K";
    case Op::MatMulMxfp4: return "MatMulMxfp4";
    default: return "MatMulMxfp6";
    }
}
inline int rfq_format_of(Op op)
{
    switch (op) {
    case Op::MatMulQ4_0: return RFQ_Q4_0;
    case Op::MatMulQ8_0: return RFQ_Q8_0;
    case Op::MatMulQ4_K: return RFQ_Q4_K;
    case Op::MatMulQ6_K: return RFQ_Q6_K;
    case Op::MatMulMxfp4: return RFQ_MXFP4;
    default: return RFQ_MXFP6_E2M3;
    }
}
// output[m, n_rows] = input[m, n_cols] . dequant(weights[n_rows, n_cols])^T; any m (rows go through the
// decode kernels eight at a time).  Enqueue only.
inline Status execute_matmul_quantized(const HipBackend &b, Op op, const DeviceTensor &weights, const DeviceTensor &input,
                                       DeviceTensor &output)
{
    const std::string who = name(op);
    const auto &ws = weights.shape.dims(), &is = input.shape.dims();
    if (ws.size() != 2 || is.size() != 2) return Status::Err(who + " expects 2D tensors");
    const int fmt = rfq_format_of(op);
    const size_t n_rows = ws[0], n_cols = ws[1], be = rfq_block_elems(fmt), bb = rfq_block_bytes(fmt);
    const size_t expected = ((n_rows * n_cols + be - 1) / be) * bb;
    if (weights.buffer.size() != expected)
        return Status::Err(who + " weights size mismatch: expected " + std::to_string(expected) + " bytes, got " +
                           std::to_string(weights.buffer.size()));
    if (is[1] != n_cols)
        return Status::Err(who + " dimension mismatch: k=" + std::to_string(is[1]) + " weights_k=" + std::to_string(n_cols));
    const size_t m = is[0];
    if (output.buffer.size() < m * n_rows * sizeof(float)) return Status::Err(who + " output buffer too small");
    for (size_t r0 = 0; r0 < m; r0 += 8) {
        const size_t rows = m - r0 < 8 ? m - r0 : 8;
        int rc = rfq_gemv(fmt, weights.buffer.as_ptr(), weights.buffer.size(), (const float *)input.buffer.as_ptr() + r0 * n_cols,
                          (float *)output.buffer.as_ptr() + r0 * n_rows, (int)rows, (int)n_rows, (int)n_cols, b.stream());
        if (rc != RFQ_OK) return detail::from_rfq(rc, name(op));
    }
    return ok_status();
}

} // namespace rocmforge
#endif /* ROCMFORGE_RFQ_HPP */
