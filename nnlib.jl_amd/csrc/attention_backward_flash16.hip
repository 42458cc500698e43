// MFMA backward for bf16/f16 inputs (placeholder selection logic until the kernels land).
#include "common.h"
#include "attention_params.h"

bool attention_bwd_flash16_supports(const AttnBwdParams &) { return false; }
size_t attention_bwd_flash16_workspace(const AttnParams &) { return 0; }
int32_t launch_attention_bwd_flash16(const AttnBwdParams &, hipStream_t) {
    return mi_set_error(MI_EINVAL, "MFMA attention backward is not available for this call");
}
