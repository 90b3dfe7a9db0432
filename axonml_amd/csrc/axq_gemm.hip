// Prefill-path quantized matmul (placeholder until the MFMA kernel lands).
#include "axq_internal.h"

int axq_dev_gemm_bf16(axq_ctx *ctx, const axq_weight *, const uint16_t *, int, float *) {
    return axq_fail(ctx, AXQ_ERR_KERNEL_LAUNCH_FAILED, "axq_gemm_bf16: not built yet");
}
