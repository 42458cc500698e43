// fp32 MFMA flash forward (placeholder until the kernel lands: reports "not supported" so that
// the dispatcher falls back to the generic kernel).
#include "common.h"
#include "attention_params.h"
bool attention_flash32_supports(const AttnParams &) { return false; }
int32_t launch_attention_flash32(const AttnParams &, hipStream_t) {
    return mi_set_error(MI_EINVAL, "fp32 flash kernel not built");
}
