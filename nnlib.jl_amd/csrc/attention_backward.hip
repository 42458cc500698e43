// mi_attention_bwd: validation and kernel selection for the gradient of dot_product_attention.
#include "common.h"
#include "attention_params.h"

static int32_t validate_bwd(const mi_attn_bwd_desc *d, AttnBwdParams *out) {
    if (!d) return mi_set_error(MI_EINVAL, "mi_attention_bwd: desc is NULL");
    if (d->struct_size != (int32_t)sizeof(mi_attn_bwd_desc))
        return mi_set_error(MI_EINVAL, "mi_attention_bwd: desc.struct_size is %d, library expects %zu", d->struct_size,
                            sizeof(mi_attn_bwd_desc));
    AttnBwdParams bp;
    int32_t rc = attention_validate(&d->fwd, &bp.p, true);
    if (rc != MI_OK) return rc;
    const AttnParams &p = bp.p;
    const bool empty = p.Lq == 0 || p.B == 0 || p.Lkv == 0 || (p.E == 0 && p.Ev == 0);
    if (!empty && !d->dout) return mi_set_error(MI_EINVAL, "mi_attention_bwd: dout is NULL");
    if (!d->dq && !d->dk && !d->dv && !d->dbias) return mi_set_error(MI_EINVAL, "mi_attention_bwd: no gradient requested");
    if (d->dbias && !d->fwd.bias) return mi_set_error(MI_EINVAL, "mi_attention_bwd: dbias given but the forward call has no bias");
    bp.dout = d->dout;
    bp.dweights = d->dweights;
    bp.dq = d->dq;
    bp.dk = d->dk;
    bp.dv = d->dv;
    bp.dbias = d->dbias;
    bp.workspace = d->workspace;
    bp.mask_bits = nullptr;
    bp.kv_len = nullptr;
    bp.dq_partial = nullptr;
    bp.dq_nsplit = 1;
    bp.mb_h = bp.mb_b = bp.mb_lkv_pad = bp.mb_nqt = 0;
    bp.have_stats = d->fwd.stats != nullptr;
    bp.stats = bp.have_stats ? d->fwd.stats : (float *)d->workspace;
    *out = bp;
    return MI_OK;
}

static int32_t choose_bwd(const mi_attn_bwd_desc *d, const AttnBwdParams &bp, size_t *ws) {
    if (!(d->fwd.flags & MI_ATTN_FORCE_GENERIC) && attention_bwd_flash16_supports(bp)) {
        *ws = (bp.have_stats ? 0 : attention_bwd_flash16_workspace(bp.p)) + attention_bwd_flash16_mask_bits_bytes(bp.p) +
              attention_bwd_flash16_lengths_bytes(bp) + attention_bwd_flash16_dq_partial_bytes(bp);
        return MI_ATTN_KERNEL_FLASH16;
    }
    if (!(d->fwd.flags & MI_ATTN_FORCE_GENERIC) && attention_bwd_flash32_supports(bp)) {
        *ws = (bp.have_stats ? 0 : attention_stats_bytes(bp.p)) + attention_bwd_flash32_lengths_bytes(bp) +
              attention_bwd_flash16_dq_partial_bytes(bp);
        return MI_ATTN_KERNEL_FLASH32;
    }
    if (bp.have_stats) {   // the generic kernels keep their own statistics, in their own layout
        *ws = attention_bwd_generic_workspace(bp.p);
        return MI_ATTN_KERNEL_GENERIC;
    }
    *ws = attention_bwd_generic_workspace(bp.p);
    return MI_ATTN_KERNEL_GENERIC;
}

MI_API int32_t mi_attention_bwd_plan(const mi_attn_bwd_desc *d, int32_t *kernel, size_t *workspace_bytes) {
    AttnBwdParams bp;
    int32_t rc = validate_bwd(d, &bp);
    if (rc != MI_OK) return rc;
    size_t ws = 0;
    const int32_t k = choose_bwd(d, bp, &ws);
    if (kernel) *kernel = k;
    if (workspace_bytes) *workspace_bytes = ws;
    return MI_OK;
}

MI_API int32_t mi_attention_bwd(const mi_attn_bwd_desc *d, mi_stream s) {
    AttnBwdParams bp;
    int32_t rc = validate_bwd(d, &bp);
    if (rc != MI_OK) return rc;
    const AttnParams &p = bp.p;
    hipStream_t st = (hipStream_t)s;
    const size_t es = mi_dtype_size(p.dtype);
    if (p.Lq == 0 || p.B == 0 || p.Lkv == 0 || (p.E == 0 && p.Ev == 0)) {
        // no (query, key) pair exists: every gradient is zero (dbias is left as the caller zeroed it)
        if (bp.dq && (rc = mi_fill_zero(bp.dq, (size_t)(p.E * p.Lq * p.B) * es, s)) != MI_OK) return rc;
        if (bp.dk && (rc = mi_fill_zero(bp.dk, (size_t)(p.E * p.Lkv * p.B) * es, s)) != MI_OK) return rc;
        if (bp.dv && (rc = mi_fill_zero(bp.dv, (size_t)(p.Ev * p.Lkv * p.B) * es, s)) != MI_OK) return rc;
        return MI_OK;
    }
    size_t ws = 0;
    const int32_t kernel = choose_bwd(d, bp, &ws);
    if (ws > 0 && (!d->workspace || d->workspace_bytes < ws))
        return mi_set_error(MI_EWORKSPACE, "mi_attention_bwd: workspace of %zu bytes required, %zu given", ws,
                            d->workspace ? d->workspace_bytes : (size_t)0);
    if ((((uintptr_t)d->workspace) & 15) != 0) return mi_set_error(MI_EWORKSPACE, "mi_attention_bwd: workspace must be 16-byte aligned");
    if (kernel == MI_ATTN_KERNEL_FLASH16) return launch_attention_bwd_flash16(bp, st);
    if (kernel == MI_ATTN_KERNEL_FLASH32) return launch_attention_bwd_flash32(bp, st);
    bp.stats = (float *)d->workspace;
    bp.have_stats = 0;
    return launch_attention_bwd_generic(bp, st);
}
