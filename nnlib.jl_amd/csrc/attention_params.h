// Kernel-side view of one attention call (validated copy of mi_attn_desc).
#pragma once
#include "common.h"

struct AttnParams {
    const void *q, *k, *v;
    void *out, *weights;
    const void *bias;
    const uint8_t *mask;
    void *workspace;
    float *stats;      // optional: row statistics for the backward call, three planes [B*H][Lq rounded up to 128]
    int64_t bias_strides[4], mask_strides[4];
    int64_t E, Ev, Lq, Lkv, H, B, D, Dv;
    int32_t dtype, weights_dtype, causal;
    // fused dropout of the weights: element (kv, q, h, b) is kept when mi_dropout_keep(drop_key,
    // kv + Lkv*(q + Lq*(h + H*b)), drop_thresh); kept weights are multiplied by drop_scale.  thresh 0 = off
    uint64_t drop_key;
    uint32_t drop_thresh;
    float drop_scale;
};

#ifdef __HIPCC__
// factor fused dropout multiplies weight (kv, q, h, b) by: 0 (dropped), drop_scale (kept), 1 without dropout
__device__ inline float attention_drop_factor(const AttnParams &p, int64_t kv, int64_t q, int64_t h, int64_t b) {
    if (p.drop_thresh == 0) return 1.0f;
    return mi_dropout_keep(p.drop_key, (uint64_t)(kv + p.Lkv * (q + p.Lq * (h + p.H * b))), p.drop_thresh) ? p.drop_scale : 0.0f;
}
#endif

// One backward call: the forward call it differentiates plus cotangents and gradient buffers.
struct AttnBwdParams {
    AttnParams p;
    const void *dout, *dweights;
    void *dq, *dk, *dv;
    float *dbias;      // addressed with p.bias_strides
    float *stats;      // per (query, head, batch) softmax statistics: the workspace, or the buffer a forward call saved
    int32_t have_stats; // the forward call already filled the first two planes of `stats`
    void *workspace;
};

// size of the statistics planes shared by the forward kernels that save them and the backward kernels
__host__ __device__ static inline int64_t attention_stats_lq_pad(int64_t Lq) { return (Lq + 127) / 128 * 128; }
static inline size_t attention_stats_bytes(const AttnParams &p) {
    return sizeof(float) * 3 * (size_t)(p.B * p.H) * (size_t)attention_stats_lq_pad(p.Lq);
}

int32_t launch_attention_bwd_generic(const AttnBwdParams &bp, hipStream_t st);
int32_t launch_attention_bwd_flash16(const AttnBwdParams &bp, hipStream_t st);
bool attention_bwd_flash16_supports(const AttnBwdParams &bp);
int32_t launch_attention_bwd_flash32(const AttnBwdParams &bp, hipStream_t st);
bool attention_bwd_flash32_supports(const AttnBwdParams &bp);
size_t attention_bwd_flash16_workspace(const AttnParams &p);
size_t attention_bwd_generic_workspace(const AttnParams &p);
int32_t attention_validate(const mi_attn_desc *d, AttnParams *out, bool for_backward = false);

int32_t launch_attention_generic(const AttnParams &p, hipStream_t st);
int32_t launch_attention_flash16(const AttnParams &p, hipStream_t st);
int32_t launch_attention_flash32(const AttnParams &p, hipStream_t st);
int32_t launch_attention_decode(const AttnParams &p, hipStream_t st);
size_t attention_decode_workspace(const AttnParams &p);
bool attention_flash16_supports(const AttnParams &p);
bool attention_flash32_supports(const AttnParams &p);
bool attention_decode_supports(const AttnParams &p);
