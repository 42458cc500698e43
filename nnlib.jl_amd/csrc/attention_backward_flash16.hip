// MFMA attention backward for bf16/f16 inputs: eligibility, workspace size and dispatch to the
// per-(dtype, head dim) instantiations of attention_backward_flash16.inc.
#include "common.h"
#include "attention_params.h"
#include "flash_common.h"

int32_t launch_bwd_flash16_bf16_d64(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_bf16_d128(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_f16_d64(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_f16_d128(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_bf16_d256(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_f16_d256(const AttnBwdParams &, hipStream_t);

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

bool attention_bwd_flash16_supports(const AttnBwdParams &bp) {
    const AttnParams &p = bp.p;
    if (p.dtype != MI_F16 && p.dtype != MI_BF16) return false;
    // one head dim for q, k and v: a multiple of 8 (16-byte chunks) up to the 256-wide tiles
    if (p.D != p.Dv || p.D < 8 || p.D > 256 || (p.D & 7)) return false;
    // the kernels need the forward result (for delta), take no weight cotangent and give no bias gradient
    if (!p.out || bp.dweights) return false;   // a bias gradient is summed with atomics by the dQ kernel
    if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v) || !aligned16(p.out) || !aligned16(bp.dout)) return false;
    if ((bp.dq && !aligned16(bp.dq)) || (bp.dk && !aligned16(bp.dk)) || (bp.dv && !aligned16(bp.dv))) return false;
    // tiles are fetched with 32-bit byte offsets from the (batch, head) slice
    if (p.Lq * p.E * 2 >= 2147483647LL || p.Lkv * p.E * 2 >= 2147483647LL) return false;
    const int64_t tiles = (p.Lq + 127) / 128 > (p.Lkv + 127) / 128 ? (p.Lq + 127) / 128 : (p.Lkv + 127) / 128;
    return tiles * p.H * p.B <= 2147483647LL;
}

// three float planes [B*H][Lq rounded up to 128]: row maximum (log2 units), 1 / row sum, delta
size_t attention_bwd_flash16_workspace(const AttnParams &p) { return attention_stats_bytes(p); }

// ---- dense masks packed into bits for the key-stationary kernels ----------------------------------------------
// A dense mask without bias keeps the lean gradient kernels (raw scores, two wavefronts per SIMD).  The dQ kernel
// stages the mask tiles through LDS as the forward kernel does; in the dK / dV kernels a lane owns one key and walks
// the queries, so it wants the mask of (its key, the 64 queries of a tile) as one 64-bit word: a small kernel packs
// those words once per call, [slice][query tile][key], slices being the distinct (head, batch) planes of the mask.
static bool takes_mask_bits(const AttnParams &p) {
    if (!p.mask || p.bias || p.D > 128 || flash_is_query_independent_mask(p) || (p.Lkv & 3) != 0) return false;
    FlashArgs a;
    a.p = p;
    a.p.weights = nullptr;
    flash_fill_vec_flags(a);
    return a.mask_lds != 0;   // the dQ kernel's staged mask tiles: unit key stride, 16-byte aligned rows
}
static int64_t mask_bits_slices(const AttnParams &p) { return (p.mask_strides[2] ? p.H : 1) * (p.mask_strides[3] ? p.B : 1); }
static int64_t mask_bits_lkv_pad(const AttnParams &p) { return (p.Lkv + 255) / 256 * 256; }

size_t attention_bwd_flash16_mask_bits_bytes(const AttnParams &p) {
    if (!takes_mask_bits(p)) return 0;
    return sizeof(uint64_t) * (size_t)(mask_bits_slices(p) * ((p.Lq + 63) / 64) * mask_bits_lkv_pad(p));
}

__global__ __launch_bounds__(256) void mask_bits_kernel(const uint8_t *mask, int64_t s0, int64_t s1, int64_t s2, int64_t s3, int64_t Lq,
                                                        int64_t Lkv, int64_t lkv_pad, int64_t heads, uint64_t *out) {
    const int64_t kv = (int64_t)blockIdx.x * 256 + threadIdx.x, qt = blockIdx.y, slice = blockIdx.z;
    const int64_t h = slice % heads, b = slice / heads;   // heads == 1: the mask is shared by the heads (stride 0)
    uint64_t word = 0;
    if (kv < Lkv) {
        const uint8_t *col = mask + kv * s0 + h * s2 + b * s3;
#pragma unroll 8
        for (int i = 0; i < 64; i++) {
            const int64_t q = qt * 64 + i;
            if (q < Lq && col[q * s1]) word |= (uint64_t)1 << i;
        }
    }
    out[(slice * gridDim.y + qt) * lkv_pad + kv] = word;
}

// Key-padding masks: the (head, batch) pairs are classified on the device and the pairs whose mask is a context
// length run the unmasked kernels on that many keys (workgroups past it only write zeros).
size_t attention_bwd_flash16_lengths_bytes(const AttnBwdParams &bp) {
    // with dropout the kernels without mask code need whole hash groups per run of four keys (Lkv a multiple of 4)
    if (!flash_is_query_independent_mask(bp.p) || (bp.p.drop_thresh && (bp.p.Lkv & 3) != 0) || bp.p.H * bp.p.B > 2147483647LL / 4) return 0;
    return ((size_t)(bp.p.H * bp.p.B) * sizeof(int32_t) + 15) & ~(size_t)15;
}

// ---- dQ kernel split over the keys ---------------------------------------------------------------------------
// The dQ kernel has one workgroup per (query tile, head, batch): cross-attention with few queries and many keys
// leaves most of the chip idle (32 workgroups for 128 queries, 16 heads, 2 batch elements).  With saved statistics
// every key piece is independent, so the key range is cut like the forward kernel's and the Float32 partial sums are
// added up by dq_merge_kernel.
int attention_bwd_flash16_dq_nsplit(const AttnBwdParams &bp) {
    const AttnParams &p = bp.p;
    if (!bp.have_stats || !bp.dq || p.causal) return 1;
    const int64_t wgs = ((p.Lq + 127) / 128) * p.H * p.B;
    if (wgs >= 256 || p.Lkv < 2048) return 1;
    int64_t n = (512 + wgs - 1) / wgs;
    if (n > p.Lkv / 512) n = p.Lkv / 512;
    if (n > 32) n = 32;
    return n < 2 ? 1 : (int)n;
}
size_t attention_bwd_flash16_dq_partial_bytes(const AttnBwdParams &bp) {
    const int n = attention_bwd_flash16_dq_nsplit(bp);
    return n > 1 ? sizeof(float) * (size_t)n * (size_t)(bp.p.B * bp.p.Lq * bp.p.E) : 0;
}

template <typename T>
__global__ __launch_bounds__(256) void dq_merge_kernel(const float *ws, typename T::type *dq, int nsplit, int64_t n) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;   // E is a multiple of 8: whole groups of 4
    if (i >= n) return;
    floatx4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = 0; s < nsplit; s++) {
        const floatx4_t v = *(const floatx4_t *)(ws + (int64_t)s * n + i);
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] += v[e];
    }
    typename T::vec4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = T::from_f32(acc[e]);
    *(typename T::vec4 *)(dq + i) = r;
}

int32_t launch_attention_bwd_flash16(const AttnBwdParams &bp_in, hipStream_t st) {
    AttnBwdParams bp = bp_in;
    const AttnParams &p = bp.p;
    bp.dq_nsplit = attention_bwd_flash16_dq_nsplit(bp);
    if (bp.dq_nsplit > 1)   // implies saved statistics: the workspace holds [packed mask bits][lengths][these partial sums]
        bp.dq_partial = (float *)((char *)bp.workspace + attention_bwd_flash16_mask_bits_bytes(p) + attention_bwd_flash16_lengths_bytes(bp));
    if (attention_bwd_flash16_lengths_bytes(bp) != 0) {   // after the statistics planes when those live in the workspace (no packed mask bits here)
        int32_t *lens = (int32_t *)((char *)bp.workspace + (bp.have_stats ? 0 : attention_bwd_flash16_workspace(p)));
        const int32_t rc = launch_key_mask_lengths(p, lens, st);
        if (rc != MI_OK) return rc;
        bp.kv_len = lens;
    }
    if (takes_mask_bits(p)) {
        const int64_t nqt = (p.Lq + 63) / 64, pad = mask_bits_lkv_pad(p), slices = mask_bits_slices(p);
        if (nqt > 65535 || slices > 65535) return mi_set_error(MI_ESHAPE, "attention gradient: mask packing supports at most 65535 query tiles and mask planes");
        uint64_t *bits = (uint64_t *)((char *)bp.workspace + (bp.have_stats ? 0 : attention_bwd_flash16_workspace(p)));
        const int64_t heads = p.mask_strides[2] ? p.H : 1;
        hipLaunchKernelGGL(mask_bits_kernel, dim3((unsigned)(pad / 256), (unsigned)nqt, (unsigned)slices), dim3(256), 0, st, p.mask,
                           p.mask_strides[0], p.mask_strides[1], p.mask_strides[2], p.mask_strides[3], p.Lq, p.Lkv, pad, heads, bits);
        MI_LAUNCH_CHECK();
        bp.mask_bits = bits;
        bp.mb_h = p.mask_strides[2] ? 1 : 0;
        bp.mb_b = p.mask_strides[3] ? heads : 0;
        bp.mb_lkv_pad = pad;
        bp.mb_nqt = nqt;
    }
    int32_t rc;
    if (p.dtype == MI_BF16)
        rc = p.D <= 64 ? launch_bwd_flash16_bf16_d64(bp, st) : p.D <= 128 ? launch_bwd_flash16_bf16_d128(bp, st) : launch_bwd_flash16_bf16_d256(bp, st);
    else
        rc = p.D <= 64 ? launch_bwd_flash16_f16_d64(bp, st) : p.D <= 128 ? launch_bwd_flash16_f16_d128(bp, st) : launch_bwd_flash16_f16_d256(bp, st);
    if (rc != MI_OK || bp.dq_nsplit <= 1) return rc;
    return launch_dq_merge(p.dtype, bp.dq_partial, bp.dq, bp.dq_nsplit, p.B * p.Lq * p.E, st);
}

int32_t launch_dq_merge(int32_t dtype, const float *partial, void *dq, int nsplit, int64_t n, hipStream_t st) {
    const dim3 grid((unsigned)((n / 4 + 255) / 256));
    if (dtype == MI_BF16) hipLaunchKernelGGL(dq_merge_kernel<BF16>, grid, dim3(256), 0, st, partial, (__bf16 *)dq, nsplit, n);
    else if (dtype == MI_F16) hipLaunchKernelGGL(dq_merge_kernel<F16>, grid, dim3(256), 0, st, partial, (_Float16 *)dq, nsplit, n);
    else hipLaunchKernelGGL(dq_merge_kernel<F32>, grid, dim3(256), 0, st, partial, (float *)dq, nsplit, n);
    MI_LAUNCH_CHECK();
    return MI_OK;
}
