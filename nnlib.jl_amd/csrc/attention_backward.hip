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

static int32_t bwd_plan_impl(const mi_attn_bwd_desc *d, int32_t *kernel, size_t *workspace_bytes) {
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

static int32_t bwd_impl(const mi_attn_bwd_desc *d, mi_stream s, int64_t scale_D) {
    AttnBwdParams bp;
    int32_t rc = validate_bwd(d, &bp);
    if (rc != MI_OK) return rc;
    mi_attn_bwd_desc eff;
    Recompute re;
    rc = resolve_bwd(d, &eff, &re);
    if (rc != MI_OK) return rc;
    if (re.on) {
        size_t need = 0;
        rc = bwd_plan_impl(d, nullptr, &need);
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
    bp.p.scale_D = scale_D;
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

// ---- different head dims for q / k and for v -------------------------------------------------------------------------
// The MFMA gradient kernels take one head dim.  A call whose q / k head dim D differs from v's Dv (src/attention.jl:55-78
// allows it, and the forward kernels take it) used to drop to the generic kernels, hundreds of times slower.  Instead the
// narrower side is copied into the workspace with its heads zero-padded to the wider dim: v, dy and the forward result
// when Dv < D (their padding contributes nothing to dP and delta, and the padded dV columns are dropped on the way back),
// q and k when D < Dv (zero features add nothing to the scores; the logits keep their scale 1 / sqrt(D) through
// AttnParams::scale_D; the padded dQ / dK columns are dropped).  Cost: copies of O(L E) next to work of O(L^2 E).
template <typename T>
__global__ __launch_bounds__(256) void pad_heads_kernel(const T *src, T *dst, int64_t rows, int64_t H, int64_t d_src, int64_t d_dst) {
    // 16-byte pieces; dst[row][h][x] = x < d_src ? src[row][h][x] : 0 for x < d_dst (narrowing when d_dst < d_src)
    constexpr int V = 16 / (int)sizeof(T);
    const int64_t per_row = H * (d_dst / V), n = rows * per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / per_row, c = i % per_row, h = c / (d_dst / V), x = (c % (d_dst / V)) * V;
        u32x4_t v = {0, 0, 0, 0};
        if (x < d_src) v = *(const u32x4_t *)(src + (row * H + h) * d_src + x);
        *(u32x4_t *)(dst + (row * H + h) * d_dst + x) = v;
    }
}

static int32_t launch_pad_heads(int32_t dtype, const void *src, void *dst, int64_t rows, int64_t H, int64_t d_src, int64_t d_dst, hipStream_t st) {
    const int64_t v = 16 / (int64_t)mi_dtype_size(dtype), n = rows * H * (d_dst / v);
    if (n == 0) return MI_OK;
    const unsigned grid = (unsigned)((n + 255) / 256 > 65536 ? 65536 : (n + 255) / 256);
    if (mi_dtype_size(dtype) == 2) hipLaunchKernelGGL(pad_heads_kernel<uint16_t>, dim3(grid), dim3(256), 0, st, (const uint16_t *)src, (uint16_t *)dst, rows, H, d_src, d_dst);
    else hipLaunchKernelGGL(pad_heads_kernel<uint32_t>, dim3(grid), dim3(256), 0, st, (const uint32_t *)src, (uint32_t *)dst, rows, H, d_src, d_dst);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

struct PadPlan {
    bool on = false, pad_v = false;   // pad_v: v / dy / x are the narrow side (Dv < D), else q / k
    int64_t Dmax = 0;
    size_t in_bytes[3] = {0, 0, 0}, out_bytes[2] = {0, 0};   // padded inputs (v, dy, x | q, k) and outputs (dv | dq, dk)
    size_t total = 0;
};

static PadPlan plan_padding(const mi_attn_bwd_desc *d) {
    PadPlan pp;
    AttnBwdParams bp;
    if (!d || !d->fwd.out || d->dweights || (d->fwd.flags & MI_ATTN_FORCE_GENERIC) || validate_bwd(d, &bp) != MI_OK) return pp;
    const AttnParams &p = bp.p;
    if (p.D == p.Dv || p.Lq == 0 || p.Lkv == 0 || p.B == 0 || p.E == 0 || p.Ev == 0) return pp;
    const bool half = p.dtype == MI_F16 || p.dtype == MI_BF16;
    if (!half && p.dtype != MI_F32) return pp;
    const int64_t v = half ? 8 : 4, cap = half ? 256 : 128, dmax = p.D > p.Dv ? p.D : p.Dv;
    if ((p.D % v) || (p.Dv % v) || dmax > cap) return pp;
    const auto al = [](const void *x) { return (((uintptr_t)x) & 15) == 0; };   // the copies move 16-byte pieces
    if (!al(p.q) || !al(p.k) || !al(p.v) || !al(p.out) || !al(d->dout) || !al(d->dq) || !al(d->dk) || !al(d->dv)) return pp;
    const size_t es = mi_dtype_size(p.dtype), eq = (size_t)(dmax * p.H) * es;
    pp.on = true;
    pp.pad_v = p.Dv < p.D;
    pp.Dmax = dmax;
    if (pp.pad_v) {
        pp.in_bytes[0] = align256(eq * (size_t)(p.Lkv * p.B));                 // v
        pp.in_bytes[1] = pp.in_bytes[2] = align256(eq * (size_t)(p.Lq * p.B)); // dy, x
        pp.out_bytes[0] = bp.dv ? align256(eq * (size_t)(p.Lkv * p.B)) : 0;    // dv
    } else {
        pp.in_bytes[0] = align256(eq * (size_t)(p.Lq * p.B));                  // q
        pp.in_bytes[1] = align256(eq * (size_t)(p.Lkv * p.B));                 // k
        pp.out_bytes[0] = bp.dq ? align256(eq * (size_t)(p.Lq * p.B)) : 0;     // dq
        pp.out_bytes[1] = bp.dk ? align256(eq * (size_t)(p.Lkv * p.B)) : 0;    // dk
    }
    pp.total = pp.in_bytes[0] + pp.in_bytes[1] + pp.in_bytes[2] + pp.out_bytes[0] + pp.out_bytes[1];
    return pp;
}

// the descriptor of the padded call; `base` = start of the padded buffers (null while planning: stand-in pointers)
static mi_attn_bwd_desc padded_desc(const mi_attn_bwd_desc *d, const PadPlan &pp, char *base) {
    mi_attn_bwd_desc e = *d;
    char *at = base ? base : (char *)(uintptr_t)4096;   // planning looks at alignment only
    char *in0 = at, *in1 = in0 + pp.in_bytes[0], *in2 = in1 + pp.in_bytes[1], *out0 = in2 + pp.in_bytes[2], *out1 = out0 + pp.out_bytes[0];
    if (pp.pad_v) {
        e.fwd.Ev = pp.Dmax * d->fwd.H;
        e.fwd.v = in0;
        e.dout = in1;
        e.fwd.out = in2;
        if (d->dv) e.dv = out0;
    } else {
        e.fwd.E = pp.Dmax * d->fwd.H;
        e.fwd.q = in0;
        e.fwd.k = in1;
        if (d->dq) e.dq = out0;
        if (d->dk) e.dk = out1;
    }
    e.workspace = base ? base + pp.total : nullptr;
    e.workspace_bytes = base && d->workspace_bytes > pp.total ? d->workspace_bytes - pp.total : 0;
    return e;
}

MI_API int32_t mi_attention_bwd_plan(const mi_attn_bwd_desc *d, int32_t *kernel, size_t *workspace_bytes) {
    const PadPlan pp = plan_padding(d);
    if (!pp.on) return bwd_plan_impl(d, kernel, workspace_bytes);
    const mi_attn_bwd_desc e = padded_desc(d, pp, nullptr);
    size_t ws = 0;
    int32_t k = 0;
    const int32_t rc = bwd_plan_impl(&e, &k, &ws);
    if (rc != MI_OK) return rc;
    if (k == MI_ATTN_KERNEL_GENERIC) return bwd_plan_impl(d, kernel, workspace_bytes);   // padding buys nothing there
    if (kernel) *kernel = k;
    if (workspace_bytes) *workspace_bytes = pp.total + ws;
    return MI_OK;
}

MI_API int32_t mi_attention_bwd(const mi_attn_bwd_desc *d, mi_stream s) {
    const PadPlan pp = plan_padding(d);
    if (pp.on) {
        size_t need = 0;
        int32_t k = 0;
        int32_t rc = mi_attention_bwd_plan(d, &k, &need);
        if (rc != MI_OK) return rc;
        if (k != MI_ATTN_KERNEL_GENERIC) {
            if (!d->workspace || d->workspace_bytes < need)
                return mi_set_error(MI_EWORKSPACE, "mi_attention_bwd: workspace of %zu bytes required, %zu given", need,
                                    d->workspace ? d->workspace_bytes : (size_t)0);
            if ((((uintptr_t)d->workspace) & 255) != 0)
                return mi_set_error(MI_EWORKSPACE, "mi_attention_bwd: with different head dims for q / k and v the workspace must be 256-byte aligned");
            const mi_attn_bwd_desc e = padded_desc(d, pp, (char *)d->workspace);
            hipStream_t st = (hipStream_t)s;
            const mi_attn_desc &f = d->fwd;
            const int64_t D = f.E / f.H, Dv = f.Ev / f.H, rq = f.Lq * f.B, rk = f.Lkv * f.B;
            if (pp.pad_v) {
                if ((rc = launch_pad_heads(f.dtype, f.v, (void *)e.fwd.v, rk, f.H, Dv, pp.Dmax, st)) != MI_OK) return rc;
                if ((rc = launch_pad_heads(f.dtype, d->dout, (void *)e.dout, rq, f.H, Dv, pp.Dmax, st)) != MI_OK) return rc;
                if ((rc = launch_pad_heads(f.dtype, f.out, e.fwd.out, rq, f.H, Dv, pp.Dmax, st)) != MI_OK) return rc;
            } else {
                if ((rc = launch_pad_heads(f.dtype, f.q, (void *)e.fwd.q, rq, f.H, D, pp.Dmax, st)) != MI_OK) return rc;
                if ((rc = launch_pad_heads(f.dtype, f.k, (void *)e.fwd.k, rk, f.H, D, pp.Dmax, st)) != MI_OK) return rc;
            }
            if ((rc = bwd_impl(&e, s, D)) != MI_OK) return rc;
            if (pp.pad_v) {
                if (d->dv && (rc = launch_pad_heads(f.dtype, e.dv, d->dv, rk, f.H, pp.Dmax, Dv, st)) != MI_OK) return rc;
            } else {
                if (d->dq && (rc = launch_pad_heads(f.dtype, e.dq, d->dq, rq, f.H, pp.Dmax, D, st)) != MI_OK) return rc;
                if (d->dk && (rc = launch_pad_heads(f.dtype, e.dk, d->dk, rk, f.H, pp.Dmax, D, st)) != MI_OK) return rc;
            }
            return MI_OK;
        }
    }
    return bwd_impl(d, s, 0);
}
