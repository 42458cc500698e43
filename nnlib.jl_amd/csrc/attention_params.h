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
    // plan constraint of the entry point without caller workspace: stay on the software-pipelined kernel (which needs
    // none) where the key-split plan would ask for more than the built-in workspace holds
    bool keep_pipelined = false;
    // and the same for the packed dense mask of the pipelined kernel: a caller whose workspace cannot hold it gets the
    // general kernel, which reads the mask as it is
    bool lean_workspace = false;
    // gradient kernels: the head dim the logits are scaled by (1 / sqrt) when it is not D, i.e. when q and k arrive
    // zero-padded to the head dim of v (attention_backward.hip pads the narrower of the two); 0: D
    int64_t scale_D = 0;
};

// A dense mask packed for the software-pipelined forward kernel (attention.hip: pack_mask_words_kernel): one 16-byte
// piece per query and group of 128 keys, word j bit k = mask[128 g + 32 j + k, query] != 0 (0 for keys past Lkv and for
// queries past Lq); pieces laid out [slice][group][Lq rounded up to 256], slice = h * stride_h + b * stride_b pieces
// (0 where the mask is shared between heads / batch elements).
struct AttnMaskWords {
    const void *words;
    int64_t stride_h, stride_b;
    int32_t lq_pad, groups;
};

#ifdef __HIPCC__
// factor fused dropout multiplies weight (kv, q, h, b) by: 0 (dropped), drop_scale (kept), 1 without dropout
__device__ inline float attention_drop_factor(const AttnParams &p, int64_t kv, int64_t q, int64_t h, int64_t b) {
    if (p.drop_thresh == 0) return 1.0f;
    return mi_dropout_keep(p.drop_key, (uint64_t)(kv + p.Lkv * (q + p.Lq * (h + p.H * b))), p.drop_thresh) ? p.drop_scale : 0.0f;
}

// The same for the 16 accumulator registers of a lane that holds, for one query, the keys of a 32-key block
// in runs of four: run g holds the weights at linear indices i0 + 8g + e (i0: the lane's first key of the block).
// ALIGNED: Lkv is a multiple of 4, so a run is one hash group; otherwise each weight is looked up alone.
template <bool ALIGNED>
__device__ inline void attention_drop_factors_run4(const AttnParams &p, uint64_t i0, int g, float (&f)[4]) {
    if (ALIGNED) {
        const uint64_t bits = mi_dropout_group_bits(p.drop_key, (i0 + 8 * g) >> 2);
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = mi_dropout_keep_in(bits, e, p.drop_thresh) ? p.drop_scale : 0.0f;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = mi_dropout_keep(p.drop_key, i0 + 8 * g + e, p.drop_thresh) ? p.drop_scale : 0.0f;
    }
}

// The transposed case: a lane holds ONE key (kv; the four lanes of a quad hold kv = 4t .. 4t+3) and, in register
// e of a run, query q0 + e.  Each lane hashes the group of query q0 + (lane & 3) and the quad exchanges the words,
// so a quad still computes one hash per four weights.  f[e]: the factor of weight (kv, q0 + e).  Needs Lkv % 4 == 0.
__device__ inline void attention_drop_factors_quad(const AttnParams &p, int64_t kv, int64_t q0, int64_t h, int64_t b, float (&f)[4]) {
    const uint64_t col0 = (uint64_t)(kv + p.Lkv * (q0 + p.Lq * (h + p.H * b)));
    {
        const int sub = (int)(kv & 3);                         // == lane & 3 for the 32-aligned key blocks of the kernels
        const uint64_t mine = mi_dropout_group_bits(p.drop_key, (col0 + (uint64_t)p.Lkv * (uint64_t)sub) >> 2);
        const int lo = (int)(uint32_t)mine, hi = (int)(uint32_t)(mine >> 32);
        // the word of quad lane E (quad_perm broadcast), of which a lane keeps its own 16-bit field
#define MI_QUAD_FIELD(E)                                                                             \
        {                                                                                            \
            const int blo = __builtin_amdgcn_mov_dpp(lo, (E) * 0x55, 0xF, 0xF, true);                \
            const int bhi = __builtin_amdgcn_mov_dpp(hi, (E) * 0x55, 0xF, 0xF, true);                \
            const uint32_t word = (uint32_t)(sub < 2 ? blo : bhi);                                   \
            f[E] = ((word >> (16 * (sub & 1))) & 0xFFFFu) >= p.drop_thresh ? p.drop_scale : 0.0f;    \
        }
        MI_QUAD_FIELD(0) MI_QUAD_FIELD(1) MI_QUAD_FIELD(2) MI_QUAD_FIELD(3)
#undef MI_QUAD_FIELD
    }
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
    // dense mask packed for the key-stationary gradient kernels: word [slice][query tile of 64][key] holds the mask
    // bits of the tile's queries for that key; slice = h * mb_h + b * mb_b (0 where the mask is shared)
    const uint64_t *mask_bits;
    int64_t mb_h, mb_b, mb_lkv_pad, mb_nqt;
    // key-padding mask measured on the device: per (head, batch) pair [b * H + h] the context length, or 0 when the
    // mask of the pair is not a kept prefix; null when the call does not take that path
    const int32_t *kv_len;
    // dQ kernel split over the keys (few query tiles, many keys; calls with saved statistics): Float32 partial sums
    // [piece][B][Lq][E], summed by a small kernel; dq_nsplit = 1 and null otherwise
    float *dq_partial;
    int32_t dq_nsplit;
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
size_t attention_bwd_flash32_lengths_bytes(const AttnBwdParams &bp);
size_t attention_bwd_flash16_workspace(const AttnParams &p);
size_t attention_bwd_flash16_mask_bits_bytes(const AttnParams &p);   // 0 when the call does not take the packed-mask path
size_t attention_bwd_flash16_lengths_bytes(const AttnBwdParams &bp);  // 0 when the call does not take the context-length path
int attention_bwd_flash16_dq_nsplit(const AttnBwdParams &bp);         // pieces the dQ kernel's key range is cut into (1: no split)
size_t attention_bwd_flash16_dq_partial_bytes(const AttnBwdParams &bp);   // the same rule serves the Float32 kernels
// dq[i] = sum over the pieces of partial[piece][i], i < n (a multiple of 4), converted to `dtype`
int32_t launch_dq_merge(int32_t dtype, const float *partial, void *dq, int nsplit, int64_t n, hipStream_t st);
// lens[b * H + h] = number of keys kept when the key-padding mask of the pair keeps exactly a prefix, else 0
int32_t launch_key_mask_lengths(const AttnParams &p, int32_t *lens, hipStream_t st);
size_t attention_bwd_generic_workspace(const AttnParams &p);
int32_t attention_validate(const mi_attn_desc *d, AttnParams *out, bool for_backward = false);

int32_t launch_attention_generic(const AttnParams &p, hipStream_t st);
int32_t launch_attention_f64(const AttnParams &p, hipStream_t st);   // Float64 arrays (attention_f64.hip)
int32_t launch_attention_flash16(const AttnParams &p, hipStream_t st);
int32_t launch_attention_flash32(const AttnParams &p, hipStream_t st);
int32_t launch_attention_decode(const AttnParams &p, hipStream_t st);
size_t attention_decode_workspace(const AttnParams &p);
bool attention_flash16_supports(const AttnParams &p);
bool attention_flash32_supports(const AttnParams &p);
size_t attention_flash32_lengths_bytes(const AttnParams &p);
int attention_flash32_nsplit(const AttnParams &p);   // pieces the key range is cut into (1: no split)
bool attention_decode_supports(const AttnParams &p);
