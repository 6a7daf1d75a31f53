// Dequant-fused GEMM  Y[m,n] = sum_k X[m,k] * W[n,k]  (placeholder until the MFMA kernel lands).
#include "internal.hpp"

namespace pmh {

size_t qgemm_workspace_bytes(int64_t, int64_t) { return 0; }

hipError_t launch_qgemm(uint32_t, const uint8_t *, int64_t, int64_t, const void *, uint32_t, int64_t, void *, uint32_t,
                        uint32_t, void *, hipStream_t) {
    return hipErrorNotSupported;
}

}  // namespace pmh
