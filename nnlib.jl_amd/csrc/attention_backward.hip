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

// ---- calls without the forward result ----------------------------------------------------------------------------
// The MFMA gradient kernels need the forward result x (for delta = sum_d x * dx).  A caller that did not keep it
// passes fwd.out = NULL; where those kernels could otherwise take the call, the library recomputes x (and the softmax
// row statistics, where the forward kernel saves them) with one forward call into the head of the workspace, instead
// of dropping to the generic kernels, which are hundreds of times slower on such shapes.  The decision is made here,
// not in the host layers: mi_attention_bwd_plan reports the kernel family and a workspace that has room for it.
struct Recompute {
    bool on = false, with_stats = false;
    size_t y_bytes = 0, stats_bytes = 0, fwd_ws = 0;
};
static inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

// Fills `eff` with the descriptor the kernels are chosen for: *d itself, or, when the forward result is to be
// recomputed, *d with stand-in pointers for it (planning reads no memory; mi_attention_bwd puts the real ones in).
static int32_t resolve_bwd(const mi_attn_bwd_desc *d, mi_attn_bwd_desc *eff, Recompute *rc) {
    *eff = *d;
    *rc = Recompute();
    if (d->fwd.out || d->dweights || (d->fwd.flags & MI_ATTN_FORCE_GENERIC) || !d->dout) return MI_OK;
    AttnBwdParams bp;
    int32_t st = validate_bwd(d, &bp);
    if (st != MI_OK) return st;
    const AttnParams &p = bp.p;
    if (p.Lq == 0 || p.B == 0 || p.Lkv == 0 || (p.E == 0 && p.Ev == 0)) return MI_OK;
    mi_attn_bwd_desc probe = *d;
    probe.fwd.out = (void *)d->dout;   // the right size and alignment class
    st = validate_bwd(&probe, &bp);
    if (st != MI_OK) return st;
    size_t ws = 0;
    if (choose_bwd(&probe, bp, &ws) == MI_ATTN_KERNEL_GENERIC) return MI_OK;
    // what the forward call would be, and whether its kernel saves the row statistics
    mi_attn_desc f = d->fwd;
    f.out = (void *)d->dout;
    f.weights = nullptr;
    f.stats = (float *)d->dout;        // stand-in: 16-byte alignment is all the planner looks at
    f.workspace = nullptr;
    f.workspace_bytes = 0;
    int32_t kf = 0;
    size_t fws = 0;
    st = mi_attention_plan(&f, &kf, &fws);
    if (st != MI_OK) return st;
    rc->with_stats = kf == MI_ATTN_KERNEL_FLASH16 || kf == MI_ATTN_KERNEL_FLASH32;
    if (!rc->with_stats) {
        f.stats = nullptr;
        st = mi_attention_plan(&f, &kf, &fws);
        if (st != MI_OK) return st;
    }
    rc->on = true;
    rc->y_bytes = align256((size_t)(p.Ev * p.Lq * p.B) * mi_dtype_size(p.dtype));
    rc->stats_bytes = rc->with_stats ? align256(attention_stats_bytes(p)) : 0;
    rc->fwd_ws = fws;
    eff->fwd.out = (void *)d->dout;
    if (rc->with_stats && !eff->fwd.stats) eff->fwd.stats = (float *)d->dout;
    return MI_OK;
}

MI_API int32_t mi_attention_bwd_plan(const mi_attn_bwd_desc *d, int32_t *kernel, size_t *workspace_bytes) {
    AttnBwdParams bp;
    int32_t rc = validate_bwd(d, &bp);
    if (rc != MI_OK) return rc;
    mi_attn_bwd_desc eff;
    Recompute re;
    rc = resolve_bwd(d, &eff, &re);
    if (rc != MI_OK) return rc;
    rc = validate_bwd(&eff, &bp);
    if (rc != MI_OK) return rc;
    size_t ws = 0;
    const int32_t k = choose_bwd(&eff, bp, &ws);
    if (re.on) ws = re.y_bytes + re.stats_bytes + (ws > re.fwd_ws ? ws : re.fwd_ws);   // the two calls share the tail
    if (kernel) *kernel = k;
    if (workspace_bytes) *workspace_bytes = ws;
    return MI_OK;
}

MI_API int32_t mi_attention_bwd(const mi_attn_bwd_desc *d, mi_stream s) {
    AttnBwdParams bp;
    int32_t rc = validate_bwd(d, &bp);
    if (rc != MI_OK) return rc;
    mi_attn_bwd_desc eff;
    Recompute re;
    rc = resolve_bwd(d, &eff, &re);
    if (rc != MI_OK) return rc;
    if (re.on) {
        size_t need = 0;
        rc = mi_attention_bwd_plan(d, nullptr, &need);
        if (rc != MI_OK) return rc;
        if (!d->workspace || d->workspace_bytes < need)
            return mi_set_error(MI_EWORKSPACE, "mi_attention_bwd: workspace of %zu bytes required, %zu given", need,
                                d->workspace ? d->workspace_bytes : (size_t)0);
        if ((((uintptr_t)d->workspace) & 255) != 0)
            return mi_set_error(MI_EWORKSPACE, "mi_attention_bwd: without the forward result the workspace must be 256-byte aligned");
        char *base = (char *)d->workspace;
        char *tail = base + re.y_bytes + re.stats_bytes;
        const size_t tail_bytes = d->workspace_bytes - re.y_bytes - re.stats_bytes;
        mi_attn_desc f = d->fwd;
        f.out = base;
        f.weights = nullptr;
        f.stats = re.with_stats ? (float *)(base + re.y_bytes) : nullptr;
        f.workspace = re.fwd_ws ? tail : nullptr;
        f.workspace_bytes = re.fwd_ws ? tail_bytes : 0;
        rc = mi_attention_fwd(&f, s);
        if (rc != MI_OK) return rc;
        eff = *d;
        eff.fwd.out = base;
        if (re.with_stats) eff.fwd.stats = (float *)(base + re.y_bytes);
        eff.workspace = tail;
        eff.workspace_bytes = tail_bytes;
    }
    d = &eff;
    rc = validate_bwd(d, &bp);
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
