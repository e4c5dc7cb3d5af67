#include "rfq_common.hpp"
namespace rfq {
size_t mx_prepared_bytes(int, int, int, int) { return 0; }
int launch_mx_prepare(int, int, const uint8_t *, int, int, void *, size_t, int *, hipStream_t)
{
    return fail(RFQ_E_UNSUPPORTED, "rfq_mx_prepare: not built yet");
}
int launch_gemm_mx(const void *, int, const void *, int, void *, int, int, int, int, hipStream_t)
{
    return fail(RFQ_E_UNSUPPORTED, "rfq_gemm_mx: not built yet");
}
} // namespace rfq
