// Matrix-core variants of the implicit GEMM (placeholder until the MFMA kernels land).
#include "common.h"

namespace tcbnn {
int launch_bgemm_mfma(const BgemmParams& p, int variant, hipStream_t stream) {
    (void)p;
    (void)stream;
    return fail(TCBNN_EUNSUPPORTED, "MFMA variant %d is not built", variant);
}
void bgemm_mfma_kernel_name(const BgemmParams& p, int variant, char* buf, size_t len) {
    (void)p;
    snprintf(buf, len, "bgemm_mfma_kernel<%d>", variant);
}
}  // namespace tcbnn
