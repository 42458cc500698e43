// mi_attention_fwd: validation (mirrors the reference's argument checks) and kernel selection.
#include "common.h"
#include "attention_params.h"
#include <mutex>

// kv_len: null, or per (head, batch) context lengths (FlashArgs::kv_len)
int32_t launch_flash16_bf16_d64(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, bool lengths_variant = false);
int32_t launch_flash16_bf16_d128(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, bool lengths_variant = false);
int32_t launch_flash16_f16_d64(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, bool lengths_variant = false);
int32_t launch_flash16_f16_d128(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, bool lengths_variant = false);
int32_t launch_flash16_bf16_d256(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, bool lengths_variant = false);
int32_t launch_flash16_f16_d256(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, bool lengths_variant = false);
int32_t launch_flash16_fast_bf16(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, const AttnMaskWords *mw = nullptr);
int32_t launch_flash16_fast_f16(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, const AttnMaskWords *mw = nullptr);
bool flash16_fast_supports_bf16(const AttnParams &);
bool flash16_fast_supports_f16(const AttnParams &);
int32_t launch_flash16_fast_bf16_d64(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, const AttnMaskWords *mw = nullptr);
int32_t launch_flash16_fast_f16_d64(const AttnParams &, hipStream_t, const int32_t *kv_len = nullptr, const AttnMaskWords *mw = nullptr);
bool flash16_fast_supports_bf16_d64(const AttnParams &);
bool flash16_fast_supports_f16_d64(const AttnParams &);

#include "flash_common.h"

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

// ---- merge of split-kv partials -------------------------------------------------------------------
// out[e, q, b] = sum_s o_s * 2^(m_s - m) / sum_s l_s * 2^(m_s - m), m = max_s m_s.  A row whose every
// piece was fully masked has m = -Inf and comes out NaN, as the unsplit kernel (and the reference) gives.
template <typename T>
__global__ __launch_bounds__(256) void flash_merge_kernel(const float *ws, typename T::type *out, int nsplit, int64_t B,
                                                           int64_t Lq, int64_t Ev, int64_t H) {
    // one thread per 4 consecutive output features (same head: head dims are multiples of 4)
    const int64_t e = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const int64_t qi = blockIdx.y, b = blockIdx.z;
    if (e >= Ev) return;
    const int64_t h = e / (Ev / H);
    const float *wml = ws + (int64_t)nsplit * B * Lq * Ev + ((b * H + h) * Lq + qi) * 2;
    const int64_t ml_step = B * H * Lq * 2, o_step = B * Lq * Ev;
    const float *wo = ws + (b * Lq + qi) * Ev + e;
    float m = MI_NEG_INF;
    for (int s = 0; s < nsplit; s++) m = fmaxf(m, wml[s * ml_step]);
    floatx4_t o = {0.0f, 0.0f, 0.0f, 0.0f};
    float l = 0.0f;
#pragma unroll 4
    for (int s = 0; s < nsplit; s++) {
        const floatx2_t ml = *(const floatx2_t *)(wml + s * ml_step);
        const floatx4_t o4 = *(const floatx4_t *)(wo + s * o_step);
        const float w = mi_exp2(ml[0] - m);
        l = fmaf(ml[1], w, l);
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = fmaf(o4[i], w, o[i]);
    }
    const float inv = 1.0f / l;
    typename T::vec4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = T::from_f32(o[i] * inv);
    *(typename T::vec4 *)(out + Ev * (Lq * b + qi) + e) = r;
}

int32_t launch_flash_merge(const AttnParams &p, int nsplit, hipStream_t st) {
    if (p.Lq > 65535 || p.B > 65535) return mi_set_error(MI_ESHAPE, "split-kv merge supports at most 65535 queries and batches");
    dim3 grid((unsigned)((p.Ev / 4 + 255) / 256), (unsigned)p.Lq, (unsigned)p.B);
    const float *ws = (const float *)p.workspace;
    if (p.dtype == MI_BF16)
        hipLaunchKernelGGL(flash_merge_kernel<BF16>, grid, dim3(256), 0, st, ws, (__bf16 *)p.out, nsplit, p.B, p.Lq, p.Ev, p.H);
    else if (p.dtype == MI_F32)
        hipLaunchKernelGGL(flash_merge_kernel<F32>, grid, dim3(256), 0, st, ws, (float *)p.out, nsplit, p.B, p.Lq, p.Ev, p.H);
    else
        hipLaunchKernelGGL(flash_merge_kernel<F16>, grid, dim3(256), 0, st, ws, (_Float16 *)p.out, nsplit, p.B, p.Lq, p.Ev, p.H);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

// true when the call takes the software-pipelined kernel (which never splits)
static bool takes_fast_path(const AttnParams &p);

bool attention_flash16_supports(const AttnParams &p) {
    if (p.dtype != MI_F16 && p.dtype != MI_BF16) return false;
    // head dims: multiples of 8 (16-byte chunks) up to the 256-wide tiles; the tile width (64, 128 or 256) is the
    // smallest that holds both, and what it has beyond them is zero-padded in flight
    if (p.D < 8 || p.Dv < 8 || p.D > 256 || p.Dv > 256 || (p.D & 7) || (p.Dv & 7)) return false;
    if (!aligned16(p.q) || !aligned16(p.k) || (p.out && (!aligned16(p.v) || !aligned16(p.out)))) return false;
    // one workgroup per (query tile, head, batch) in a 1-D grid
    const int64_t tiles = (p.Lq + 127) / 128;
    if (tiles * p.H * p.B > 2147483647LL) return false;
    return true;
}

static bool fast_kernel_fits(const AttnParams &p) {   // everything but the mask
    if (p.dtype == MI_BF16) return flash16_fast_supports_bf16(p) || flash16_fast_supports_bf16_d64(p);
    if (p.dtype == MI_F16) return flash16_fast_supports_f16(p) || flash16_fast_supports_f16_d64(p);
    return false;
}
static bool takes_fast_path(const AttnParams &p) {
    if (p.mask || !fast_kernel_fits(p)) return false;
    // The pipelined kernel never splits the keys and has one workgroup per 256 queries of a (head, batch) pair: with
    // few queries and many keys (cross-attention, a short chunk of queries against a long context) it would leave most
    // of the chip idle, where the general kernel cuts the key range into pieces.  Measured, pipelined / general:
    // f16, head dim 64, 256 queries x 8192 keys, 64 pairs (64 workgroups against 512 pieces): 0.113 / 0.061 ms;
    // bf16, head dim 128: the same shape 0.168 / 0.102, 128 x 4096 0.086 / 0.043, 256 x 2048 0.048 / 0.038,
    // 512 x 8192 with 48 pairs (96 workgroups) 0.168 / 0.163.  At 128 workgroups the two are level without a causal
    // mask (2048 x 2048, 16 pairs: 0.049 / 0.054; 1024 x 4096, 32 pairs: 0.089 / 0.087); with one, the pipelined
    // kernel's unequal jobs lose (4096 x 4096, 8 pairs: 0.091 / 0.079).  Above that the pipelined kernel wins.
    const int64_t fast_wgs = ((p.Lq + 255) / 256) * p.H * p.B;
    if (!p.keep_pipelined && (fast_wgs < 128 || (fast_wgs == 128 && p.causal)) && flash_pick_nsplit(p, 128) > 1) return false;
    return true;
}

// ---- key-padding masks that are context lengths ------------------------------------------------------------------
// Batches of sequences padded to one length carry a mask that keeps a prefix of the keys of each (head, batch) pair.
// For such a pair the mask is just a shorter L_kv, which the software-pipelined kernel handles at full speed (and it
// skips the padding instead of computing and discarding it).  Whether a mask is of that kind is only known on the
// device, so: a small kernel measures every pair (length of the kept prefix, or 0 when the mask is anything else, an
// empty one included), then BOTH forward kernels are launched and every (head, batch) pair is computed by exactly
// one of them: the pipelined kernel takes the pairs with a length, the general kernel the others.
static bool takes_length_path(const AttnParams &p) {
    // a call this small is bound by its launches: one kernel with mask code instead of the classification and the two
    // kernels behind it (16-bit, 32 pairs of 128 x 128 with a mask column per batch element: 13.5 -> 9.5 us with the
    // weights, 11.2 -> 6.5 without; 512 x 512: 30.3 -> 26.0 and 19.3 -> 14.7)
    if ((p.Lq + 127) / 128 * p.H * p.B <= 128 && p.Lkv <= 512) return false;
    return flash_is_query_independent_mask(p) && flash_pick_nsplit(p, 128) == 1 && p.H * p.B <= 2147483647LL / 4;
}
static size_t length_path_workspace(const AttnParams &p) { return ((size_t)(p.H * p.B) * sizeof(int32_t) + 15) & ~(size_t)15; }

__global__ __launch_bounds__(256) void key_mask_lengths_kernel(const uint8_t *mask, int64_t s0, int64_t s2, int64_t s3, int64_t Lkv,
                                                              int64_t H, int32_t *lens) {
    const int64_t h = blockIdx.x % H, b = blockIdx.x / H;
    const uint8_t *m = mask + h * s2 + b * s3;   // one byte per key, any key stride and alignment
    int last = -1, count = 0;
    for (int64_t j = threadIdx.x; j < Lkv; j += 256)
        if (m[j * s0]) {
            last = (int)j;
            count++;
        }
    __shared__ int s_last[4], s_count[4];
    for (int off = 32; off > 0; off >>= 1) {
        const int o_last = __shfl_xor(last, off, 64);
        last = o_last > last ? o_last : last;
        count += __shfl_xor(count, off, 64);
    }
    if ((threadIdx.x & 63) == 0) {
        s_last[threadIdx.x >> 6] = last;
        s_count[threadIdx.x >> 6] = count;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int l = s_last[0], c = s_count[0];
        for (int w = 1; w < 4; w++) {
            l = s_last[w] > l ? s_last[w] : l;
            c += s_count[w];
        }
        lens[blockIdx.x] = (c > 0 && c == l + 1) ? c : 0;
    }
}

int32_t launch_key_mask_lengths(const AttnParams &p, int32_t *lens, hipStream_t st) {
    if (p.H * p.B > 2147483647LL) return mi_set_error(MI_ESHAPE, "attention: too many (head, batch) pairs");
    hipLaunchKernelGGL(key_mask_lengths_kernel, dim3((unsigned)(p.H * p.B)), dim3(256), 0, st, p.mask, p.mask_strides[0],
                       p.mask_strides[2], p.mask_strides[3], p.Lkv, p.H, lens);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

static int32_t launch_general16(const AttnParams &p, hipStream_t st, const int32_t *kv_len, bool lv = false) {
    const int64_t dmax = p.D > p.Dv ? p.D : p.Dv;
    if (p.dtype == MI_BF16)
        return dmax <= 64    ? launch_flash16_bf16_d64(p, st, kv_len, lv)
               : dmax <= 128 ? launch_flash16_bf16_d128(p, st, kv_len, lv)
                             : launch_flash16_bf16_d256(p, st, kv_len, lv);
    return dmax <= 64 ? launch_flash16_f16_d64(p, st, kv_len, lv) : dmax <= 128 ? launch_flash16_f16_d128(p, st, kv_len, lv) : launch_flash16_f16_d256(p, st, kv_len, lv);
}

static int32_t launch_fast16(const AttnParams &p, hipStream_t st, const int32_t *kv_len, const AttnMaskWords *mw = nullptr) {
    if (p.dtype == MI_BF16 && flash16_fast_supports_bf16(p)) return launch_flash16_fast_bf16(p, st, kv_len, mw);
    if (p.dtype == MI_F16 && flash16_fast_supports_f16(p)) return launch_flash16_fast_f16(p, st, kv_len, mw);
    if (p.dtype == MI_BF16) return launch_flash16_fast_bf16_d64(p, st, kv_len, mw);
    return launch_flash16_fast_f16_d64(p, st, kv_len, mw);
}

// ---- dense masks for the software-pipelined kernel ------------------------------------------------------------------
// A mask that depends on the query (src/attention.jl:122-124 takes any array that broadcasts against the logits) costs
// the general kernel a byte per score, staged through LDS.  The pipelined kernel takes it as bits instead: a pre-pass
// packs the mask once per call into one word per query and 32-key block (AttnMaskWords; 1/8 of the mask's bytes, read
// by every head and batch element that shares the mask), and the kernel turns a word into its 16 scores' worth of
// -Inf with two instructions per score.  Any strides: the pre-pass reads bytes.
static AttnMaskWords mask_words_layout(const AttnParams &p) {
    AttnMaskWords mw;
    mw.words = p.workspace;
    mw.lq_pad = (int32_t)((p.Lq + 255) / 256 * 256);
    mw.groups = (int32_t)((p.Lkv + 127) / 128);
    const int64_t slice = (int64_t)mw.groups * mw.lq_pad;
    const bool per_h = p.mask_strides[2] != 0 && p.H > 1, per_b = p.mask_strides[3] != 0 && p.B > 1;
    mw.stride_h = per_h ? slice : 0;
    mw.stride_b = per_b ? slice * (per_h ? p.H : 1) : 0;
    return mw;
}
static size_t mask_words_bytes(const AttnParams &p) {
    const AttnMaskWords mw = mask_words_layout(p);
    const int64_t slices = (mw.stride_h ? p.H : 1) * (mw.stride_b ? p.B : 1);
    return (size_t)slices * (size_t)mw.groups * (size_t)mw.lq_pad * 16;
}
static bool takes_mask_words_path(const AttnParams &p) {
    static const bool off = getenv("MI355ATTN_NO_MASK_WORDS") != nullptr;   // A/B switch: masks go to the general kernel
    if (off) return false;
    if (!p.mask || p.bias || p.drop_thresh || p.lean_workspace || !fast_kernel_fits(p) || p.Lq > 2147483647LL - 256 || p.Lkv > 2147483647LL - 128) return false;
    // as for calls without a mask: few workgroups against a key range the general kernel would split
    const int64_t fast_wgs = ((p.Lq + 255) / 256) * p.H * p.B;
    if ((fast_wgs < 128 || (fast_wgs == 128 && p.causal)) && flash_pick_nsplit(p, 128) > 1) return false;
    return true;
}

// One wavefront per (query, slice, run of 8 groups = 1024 keys); all loads of a run are requested before the first is
// looked at.  WORDS (unit key stride, rows 4-byte aligned): a lane loads four keys at a time, makes their four bits, and
// the eight lanes of a 32-key block OR their shifted nibbles together (three exchanges).  Otherwise a byte per lane and
// half group, through the mask's strides, and two ballots per group.
constexpr int PACK_RUN = 8;
template <bool WORDS>
__global__ __launch_bounds__(256) void pack_mask_words_kernel(const uint8_t *mask, int64_t s0, int64_t s1, int64_t s2, int64_t s3, int64_t Lq,
                                                             int64_t Lkv, int64_t nh, int64_t items, int32_t runs, AttnMaskWords mw) {
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);   // (run, query, head slice, batch slice), run fastest
    if (item >= items) return;
    const int run = (int)(item % runs);
    const int64_t row = item / runs, q = row % mw.lq_pad, sl = row / mw.lq_pad, h = sl % nh, b = sl / nh;
    u32x4_t *dst = (u32x4_t *)mw.words + h * mw.stride_h + b * mw.stride_b + q;
    const uint8_t *src = mask + q * s1 + h * s2 + b * s3;
    const int g0 = run * PACK_RUN;
    if constexpr (WORDS) {
        uint32_t four[PACK_RUN / 2];   // one load covers 256 keys: two groups
#pragma unroll
        for (int u = 0; u < PACK_RUN / 2; u++) {
            const int64_t key = (int64_t)(g0 + 2 * u) * 128 + 4 * lane;
            four[u] = 0;
            if (q < Lq && key + 3 < Lkv) four[u] = *(const uint32_t *)(src + key);
            else if (q < Lq)
                for (int e = 0; e < 4; e++)
                    if (key + e < Lkv) four[u] |= (uint32_t)src[key + e] << (8 * e);
        }
#pragma unroll
        for (int u = 0; u < PACK_RUN / 2; u++) {
            const uint32_t x = four[u];
            uint32_t v = ((x & 0xFFu) ? 1u : 0u) | ((x & 0xFF00u) ? 2u : 0u) | ((x & 0xFF0000u) ? 4u : 0u) | ((x & 0xFF000000u) ? 8u : 0u);
            v <<= 4 * (lane & 7);
            v |= (uint32_t)__shfl_xor((int)v, 1, 64);
            v |= (uint32_t)__shfl_xor((int)v, 2, 64);
            v |= (uint32_t)__shfl_xor((int)v, 4, 64);
            // lane 8j holds the word of block j of the 256 keys: word j % 4 of group g0 + 2u + j / 4
            const int g = g0 + 2 * u + (lane >> 5);
            if ((lane & 7) == 0 && g < mw.groups) ((uint32_t *)(dst + (int64_t)g * mw.lq_pad))[(lane >> 3) & 3] = v;
        }
    } else {
        uint8_t byte[PACK_RUN][2];
#pragma unroll
        for (int u = 0; u < PACK_RUN; u++)
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int64_t key = (int64_t)(g0 + u) * 128 + 64 * half + lane;
                byte[u][half] = q < Lq && key < Lkv ? src[key * s0] : (uint8_t)0;
            }
#pragma unroll
        for (int u = 0; u < PACK_RUN; u++) {
            const uint64_t lo = __builtin_amdgcn_ballot_w64(byte[u][0] != 0), hi = __builtin_amdgcn_ballot_w64(byte[u][1] != 0);
            if (lane == 0 && g0 + u < mw.groups)
                dst[(int64_t)(g0 + u) * mw.lq_pad] = (u32x4_t){(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
        }
    }
}

static int32_t launch_pack_mask_words(const AttnParams &p, const AttnMaskWords &mw, hipStream_t st) {
    const int64_t nh = mw.stride_h ? p.H : 1, nb = mw.stride_b ? p.B : 1;
    const int32_t runs = (mw.groups + PACK_RUN - 1) / PACK_RUN;
    const int64_t items = (int64_t)mw.lq_pad * nh * nb * runs;
    if ((items + 3) / 4 > 2147483647LL) return mi_set_error(MI_ESHAPE, "attention: mask too large to pack");
    const bool words = p.mask_strides[0] == 1 && ((((uintptr_t)p.mask) | (uintptr_t)p.mask_strides[1] | (uintptr_t)p.mask_strides[2] | (uintptr_t)p.mask_strides[3]) & 3) == 0;
    if (words)
        hipLaunchKernelGGL(pack_mask_words_kernel<true>, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, p.mask, p.mask_strides[0],
                           p.mask_strides[1], p.mask_strides[2], p.mask_strides[3], p.Lq, p.Lkv, nh, items, runs, mw);
    else
        hipLaunchKernelGGL(pack_mask_words_kernel<false>, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, p.mask, p.mask_strides[0],
                           p.mask_strides[1], p.mask_strides[2], p.mask_strides[3], p.Lq, p.Lkv, nh, items, runs, mw);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

int32_t launch_attention_flash16(const AttnParams &p, hipStream_t st) {
    if (takes_length_path(p)) {
        int32_t *lens = (int32_t *)p.workspace;
        int32_t rc = launch_key_mask_lengths(p, lens, st);
        if (rc != MI_OK) return rc;
        // pairs with a context length: the software-pipelined kernel where it fits the call, else the general kernel's
        // variant without mask code (weights, dropout, other head dims); the other pairs: the key-mask variant
        rc = fast_kernel_fits(p) ? launch_fast16(p, st, lens) : launch_general16(p, st, lens, true);
        if (rc != MI_OK) return rc;
        return launch_general16(p, st, lens);
    }
    if (takes_mask_words_path(p)) {
        const AttnMaskWords mw = mask_words_layout(p);
        const int32_t rc = launch_pack_mask_words(p, mw, st);
        if (rc != MI_OK) return rc;
        return launch_fast16(p, st, nullptr, &mw);
    }
    if (takes_fast_path(p)) return launch_fast16(p, st, nullptr);
    return launch_general16(p, st, nullptr);
}

// Validation.  The first four conditions are the reference's ArgumentErrors
// (src/attention.jl:55-78); with (E, L, B) sizes passed as scalars, "batch dimensions equal",
// "qk feature dims equal" and "kv lengths equal" hold by construction, which leaves divisibility.
int32_t attention_validate(const mi_attn_desc *d, AttnParams *out, bool for_backward) {
    if (!d) return mi_set_error(MI_EINVAL, "mi_attention: desc is NULL");
    if (d->struct_size != (int32_t)sizeof(mi_attn_desc))
        return mi_set_error(MI_EINVAL, "mi_attention: desc.struct_size is %d, library expects %zu", d->struct_size,
                            sizeof(mi_attn_desc));
    // Float64 arrays: the forward call only (a double-precision vector kernel, attention_f64.hip)
    if (!(for_backward ? mi_dtype_ok(d->dtype) : mi_dtype_ok_f64(d->dtype)))
        return mi_set_error(MI_EDTYPE, "mi_attention: unknown dtype %d", d->dtype);
    if (d->E < 0 || d->Ev < 0 || d->Lq < 0 || d->Lkv < 0 || d->B < 0)
        return mi_set_error(MI_ESHAPE, "mi_attention: negative size");
    if (d->H < 1) return mi_set_error(MI_ESHAPE, "mi_attention: nheads must be at least 1 (got %lld)", (long long)d->H);
    if (d->E % d->H != 0 || d->Ev % d->H != 0)
        return mi_set_error(MI_ESHAPE,
                            "First dimension in query, key and value must be divisible by `nheads`. Instead: "
                            "size(q,1) = size(k,1) = %lld, size(v,1) = %lld, nheads = %lld",
                            (long long)d->E, (long long)d->Ev, (long long)d->H);
    if (d->causal && d->Lq != d->Lkv)
        return mi_set_error(MI_ESHAPE, "mi_attention: a causal (len, len) mask needs Lq == Lkv (got %lld, %lld)",
                            (long long)d->Lq, (long long)d->Lkv);
    if (!for_backward && !d->out && !d->weights) return mi_set_error(MI_EINVAL, "mi_attention: both out and weights are NULL");
    if (d->weights && d->weights_dtype != d->dtype && (d->weights_dtype != MI_F32 || d->dtype == MI_F64))
        return mi_set_error(MI_EDTYPE, "mi_attention: weights_dtype must equal dtype or (16-bit inputs) be MI_F32");
    if (d->dtype == MI_F64 && d->stats) return mi_set_error(MI_EDTYPE, "mi_attention: row statistics are not kept for Float64 calls");
    const bool empty = d->Lq == 0 || d->B == 0 || (d->E == 0 && d->Ev == 0);
    if (!empty) {
        if (d->Lkv > 0 && d->E > 0 && (!d->q || !d->k)) return mi_set_error(MI_EINVAL, "mi_attention: q or k is NULL");
        if ((d->out || for_backward) && d->Lkv > 0 && d->Ev > 0 && !d->v)
            return mi_set_error(MI_EINVAL, "mi_attention: v is NULL but out is not");
    }
    for (int i = 0; i < 4; i++) {
        if (d->bias && d->bias_strides[i] < 0) return mi_set_error(MI_ESHAPE, "mi_attention: negative bias stride");
        if (d->mask && d->mask_strides[i] < 0) return mi_set_error(MI_ESHAPE, "mi_attention: negative mask stride");
    }
    AttnParams p;
    p.q = d->q; p.k = d->k; p.v = d->v; p.out = d->out; p.weights = d->weights;
    p.bias = d->bias; p.mask = d->mask; p.workspace = d->workspace;
    p.stats = d->stats;
    if (d->stats && (((uintptr_t)d->stats) & 15) != 0) return mi_set_error(MI_EINVAL, "mi_attention: stats must be 16-byte aligned");
    for (int i = 0; i < 4; i++) {
        p.bias_strides[i] = d->bias ? d->bias_strides[i] : 0;
        p.mask_strides[i] = d->mask ? d->mask_strides[i] : 0;
    }
    p.E = d->E; p.Ev = d->Ev; p.Lq = d->Lq; p.Lkv = d->Lkv; p.H = d->H; p.B = d->B;
    p.D = d->E / d->H; p.Dv = d->Ev / d->H;
    p.dtype = d->dtype;
    p.weights_dtype = d->weights ? d->weights_dtype : d->dtype;
    p.causal = d->causal != 0;
    if (!(d->dropout_p >= 0.0f && d->dropout_p <= 1.0f))
        return mi_set_error(MI_EINVAL, "dropout expects a probability 0 <= p <= 1");   // src/dropout.jl:43
    p.drop_key = mi_stream_key(d->dropout_seed, MI_DROPOUT_STREAM);
    p.drop_thresh = mi_dropout_threshold(d->dropout_p);
    p.drop_scale = d->dropout_p < 1.0f ? 1.0f / (1.0f - d->dropout_p) : 0.0f;
    *out = p;
    return MI_OK;
}

static int32_t choose(const mi_attn_desc *d, const AttnParams &p, size_t *ws) {
    *ws = 0;
    if ((d->flags & MI_ATTN_FORCE_GENERIC) || p.dtype == MI_F64) return MI_ATTN_KERNEL_GENERIC;
    if (attention_decode_supports(p)) {
        *ws = attention_decode_workspace(p);
        return MI_ATTN_KERNEL_DECODE;
    }
    if (attention_flash16_supports(p)) {
        if (takes_length_path(p)) *ws = length_path_workspace(p);   // one context length per (head, batch) pair
        else if (takes_mask_words_path(p)) *ws = mask_words_bytes(p);
        else if (!takes_fast_path(p)) *ws = flash_split_workspace(p, flash_pick_nsplit(p, 128));
        return MI_ATTN_KERNEL_FLASH16;
    }
    if (attention_flash32_supports(p)) {
        const int nsplit = attention_flash32_nsplit(p);
        *ws = nsplit > 1 ? flash_split_workspace(p, nsplit) : attention_flash32_lengths_bytes(p);
        return MI_ATTN_KERNEL_FLASH32;
    }
    return MI_ATTN_KERNEL_GENERIC;
}

MI_API int32_t mi_attention_plan(const mi_attn_desc *d, int32_t *kernel, size_t *workspace_bytes) {
    AttnParams p;
    int32_t rc = attention_validate(d, &p);
    if (rc != MI_OK) return rc;
    size_t ws = 0;
    int32_t k = choose(d, p, &ws);
    if (kernel) *kernel = k;
    if (workspace_bytes) *workspace_bytes = ws;
    return MI_OK;
}

MI_API int32_t mi_attention_stats_size(const mi_attn_desc *d, size_t *bytes) {
    if (!bytes) return mi_set_error(MI_EINVAL, "mi_attention_stats_size: bytes is NULL");
    AttnParams p;
    int32_t rc = attention_validate(d, &p, true);
    if (rc != MI_OK) return rc;
    *bytes = attention_stats_bytes(p);
    return MI_OK;
}

MI_API int32_t mi_attention_workspace_size(const mi_attn_desc *d, size_t *bytes) {
    if (!bytes) return mi_set_error(MI_EINVAL, "mi_attention_workspace_size: bytes is NULL");
    return mi_attention_plan(d, nullptr, bytes);
}

// ---- the forward call on a workspace that lives in the library's own device image ------------------------------
// For callers that cannot allocate device memory (under stream capture, in loops that must not touch the allocator):
// the split-kv partials, raw single-query scores and context lengths go into a file-scope device array instead of a
// caller-provided workspace.  Every GPU the library runs on holds its own copy of the array at its own address, which
// hipGetSymbolAddress reports for the device that is current; in host code the array's name is not that address.
static __device__ __align__(256) unsigned char scratch[MI_ATTN_STATIC_WORKSPACE_BYTES];

#define MI_MAX_DEVICES 64
static void *g_scratch_ptr[MI_MAX_DEVICES];   // per device: address of `scratch` there, null = not asked yet
static std::mutex g_scratch_lock;

// Address of `scratch` on the current device (asked once per device).
int32_t attention_static_scratch(void **out) {
    int dev = -1;
    MI_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MI_MAX_DEVICES) return mi_set_error(MI_EINVAL, "mi_attention_fwd_static: device %d is beyond the %d this library tracks", dev, MI_MAX_DEVICES);
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        MI_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return mi_set_error(MI_EHIP, "mi_attention_fwd_static: the device image holds no workspace array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return MI_OK;
}

static int32_t attention_forward(const mi_attn_desc *d, mi_stream s, bool static_workspace);

MI_API int32_t mi_attention_fwd(const mi_attn_desc *d, mi_stream s) { return attention_forward(d, s, false); }
MI_API int32_t mi_attention_fwd_static(const mi_attn_desc *d, mi_stream s) { return attention_forward(d, s, true); }

static int32_t attention_forward(const mi_attn_desc *d, mi_stream s, bool static_workspace) {
    AttnParams p;
    int32_t rc = attention_validate(d, &p);
    if (rc != MI_OK) return rc;
    hipStream_t st = (hipStream_t)s;
    if (p.Lq == 0 || p.B == 0) return MI_OK;  // empty outputs
    if (p.Lkv == 0) {
        // softmax over an empty column has no entries; the product with the (Dv x 0) values is all zeros
        if (p.out) return mi_fill_zero(p.out, (size_t)(p.Ev * p.Lq * p.B) * mi_dtype_size(p.dtype), s);
        return MI_OK;
    }
    size_t ws = 0;
    int32_t kernel = choose(d, p, &ws);
    const size_t have = static_workspace ? (size_t)MI_ATTN_STATIC_WORKSPACE_BYTES : (d->workspace ? d->workspace_bytes : (size_t)0);
    if (ws > have && kernel == MI_ATTN_KERNEL_FLASH16 && p.mask) {
        // a dense mask too large to pack into the workspace at hand: the general kernel reads it as it is
        p.lean_workspace = true;
        kernel = choose(d, p, &ws);
    }
    if (ws > have && kernel == MI_ATTN_KERNEL_FLASH16) {
        // few queries against many keys: the key-split plan is the faster one, but the pipelined kernel needs no
        // workspace at all, so a caller without (enough of) one is served rather than refused
        p.keep_pipelined = true;
        kernel = choose(d, p, &ws);
    }
    if (static_workspace) {
        // every kernel writes what it later reads of the workspace, so what an earlier call left there needs no clearing
        if (ws > MI_ATTN_STATIC_WORKSPACE_BYTES)
            return mi_set_error(MI_EWORKSPACE, "mi_attention_fwd_static: this call needs a workspace of %zu bytes, the built-in one has %zu; "
                                "use mi_attention_fwd with a caller-provided workspace", ws, (size_t)MI_ATTN_STATIC_WORKSPACE_BYTES);
        p.workspace = nullptr;
        if (ws > 0) {
            rc = attention_static_scratch(&p.workspace);
            if (rc != MI_OK) return rc;
        }
    } else if (ws > 0 && (!d->workspace || d->workspace_bytes < ws))
        return mi_set_error(MI_EWORKSPACE, "mi_attention_fwd: workspace of %zu bytes required, %zu given", ws,
                            d->workspace ? d->workspace_bytes : (size_t)0);
    switch (kernel) {
    case MI_ATTN_KERNEL_DECODE: return launch_attention_decode(p, st);
    case MI_ATTN_KERNEL_FLASH16: return launch_attention_flash16(p, st);
    case MI_ATTN_KERNEL_FLASH32: return launch_attention_flash32(p, st);
    default: return p.dtype == MI_F64 ? launch_attention_f64(p, st) : launch_attention_generic(p, st);
    }
}
