// Decode model (placeholder; filled in after the GEMV path is verified).
#include "axq_internal.h"

extern "C" {
int axq_model_create(axq_ctx *ctx, const axq_model_config *, axq_model **) {
    return axq_fail(ctx, AXQ_ERR_KERNEL_LAUNCH_FAILED, "axq_model_create: not built yet");
}
void axq_model_free(axq_model *) {}
int axq_model_set_embedding_f16(axq_model *, const uint16_t *, int) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_set_norm(axq_model *, int, int, const float *, int) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_set_linear(axq_model *, int, int, const axq_weight *) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_random_init(axq_model *, int, float, uint64_t) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_reset(axq_model *) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_forward(axq_model *, int32_t, float *, int32_t *) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_generate(axq_model *, const int32_t *, int, int, int32_t *, float *, float *) { return AXQ_ERR_INVALID_ARGUMENT; }
int axq_model_seq_len(const axq_model *) { return -1; }
}
