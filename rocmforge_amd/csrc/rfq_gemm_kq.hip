#include "rfq_common.hpp"
namespace rfq {
int launch_gemm_f16(int fmt, const uint8_t *, const void *, void *, int, int, int, int, hipStream_t)
{
    return fail(RFQ_E_UNSUPPORTED, "rfq_gemm_f16: no kernel for format %d yet", fmt);
}
} // namespace rfq
