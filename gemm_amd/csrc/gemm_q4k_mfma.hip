/* placeholder translation unit: replaced by the matrix-core kernels */
#include "qlin_device.h"
#include "qlin_internal.h"
namespace qlin {
hipError_t launch_gemm_q4k_bf16(const void *, const uint16_t *, float *, int, int, int, int, int, hipStream_t) {
    return hipErrorNotSupported;
}
size_t moe_workspace_bytes(int, int, int, int, int) { return 256; }
hipError_t launch_moe_ffn_q4k(const void *, const void *, const void *, const uint16_t *, const int32_t *,
                              const float *, float *, int, int, int, int, int, void *, hipStream_t) {
    return hipErrorNotSupported;
}
}  // namespace qlin
