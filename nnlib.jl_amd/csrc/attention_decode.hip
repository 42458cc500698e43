// split-kv decode path (placeholder until the kernel lands).
#include "common.h"
#include "attention_params.h"
bool attention_decode_supports(const AttnParams &) { return false; }
size_t attention_decode_workspace(const AttnParams &) { return 0; }
int32_t launch_attention_decode(const AttnParams &, hipStream_t) {
    return mi_set_error(MI_EINVAL, "decode kernel not built");
}
