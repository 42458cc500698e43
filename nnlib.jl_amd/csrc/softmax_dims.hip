// The softmax family over ANY set of dimensions (src/softmax.jl:56, 133, 200 take any `dims`, as Base's reductions
// do).  The kernels reduce over a run of adjacent dimensions, viewed as (inner, len, outer).  A set that is such a run
// goes straight to them; any other set is brought to the front with a permuting copy (what `permutedims` does in the
// reference's Base calls), reduced over the leading run, and permuted back.  The permuted copies live in a workspace
// of the caller; mi_softmax_dims_workspace sizes it (0 for a run of adjacent dimensions).
#include "common.h"

namespace {

constexpr int MAXD = 8;

struct Plan {
    bool run;                      // dims form a run of adjacent dimensions (or nothing is reduced)
    int64_t inner, len, outer;     // geometry of the run, or (1, len, outer) of the permuted array
    int64_t n;                     // elements of the array
    int nd;
    int64_t psize[MAXD], pstride[MAXD];   // permuted view of the source: sizes, and strides into the dense source
    int64_t isize[MAXD], istride[MAXD];   // view of the dense permuted array that reads back in the original order
};

int32_t make_plan(const char *who, int32_t ndim, const int64_t *sizes, uint32_t dims_mask, Plan *pl) {
    if (ndim < 0 || ndim > MAXD || (ndim > 0 && !sizes)) return mi_set_error(MI_EINVAL, "%s: 0 to 8 dimensions", who);
    int64_t stride[MAXD], n = 1;
    for (int d = 0; d < ndim; d++) {
        if (sizes[d] < 0) return mi_set_error(MI_EINVAL, "%s: negative size", who);
        stride[d] = n;
        n *= sizes[d];
    }
    pl->n = n;
    pl->nd = ndim;
    const uint32_t mask = ndim >= 32 ? dims_mask : (dims_mask & ((1u << ndim) - 1u));   // dimensions past ndim have extent 1
    if (mask == 0) {   // nothing to reduce over within the array: every element is its own slice
        pl->run = true;
        pl->inner = n;
        pl->len = 1;
        pl->outer = 1;
        return MI_OK;
    }
    int lo = 0, hi = ndim - 1;
    while (!((mask >> lo) & 1u)) lo++;
    while (!((mask >> hi) & 1u)) hi--;
    bool run = true;
    for (int d = lo; d <= hi; d++) run = run && ((mask >> d) & 1u);
    pl->run = run;
    if (run) {
        pl->inner = pl->len = pl->outer = 1;
        for (int d = 0; d < lo; d++) pl->inner *= sizes[d];
        for (int d = lo; d <= hi; d++) pl->len *= sizes[d];
        for (int d = hi + 1; d < ndim; d++) pl->outer *= sizes[d];
        return MI_OK;
    }
    // perm: the reduced dimensions first, then the others, each group in its own order
    int perm[MAXD], k = 0;
    pl->inner = pl->len = pl->outer = 1;
    for (int d = 0; d < ndim; d++)
        if ((mask >> d) & 1u) {
            perm[k++] = d;
            pl->len *= sizes[d];
        }
    for (int d = 0; d < ndim; d++)
        if (!((mask >> d) & 1u)) {
            perm[k++] = d;
            pl->outer *= sizes[d];
        }
    int64_t pdense[MAXD], acc = 1;
    for (int i = 0; i < ndim; i++) {
        pl->psize[i] = sizes[perm[i]];
        pl->pstride[i] = stride[perm[i]];
        pdense[i] = acc;                 // dense stride of permuted dimension i
        acc *= pl->psize[i];
    }
    for (int i = 0; i < ndim; i++) {     // original dimension perm[i] lives at permuted position i
        pl->isize[perm[i]] = sizes[perm[i]];
        pl->istride[perm[i]] = pdense[i];
    }
    return MI_OK;
}

size_t elem_size(int32_t dtype) { return mi_dtype_size(dtype); }

int32_t check_ws(const char *who, const void *ws, size_t have, size_t need) {
    if (need == 0) return MI_OK;
    if (!ws || have < need) return mi_set_error(MI_EWORKSPACE, "%s: workspace of %zu bytes required, %zu given", who, need, ws ? have : (size_t)0);
    if ((((uintptr_t)ws) & 15) != 0) return mi_set_error(MI_EWORKSPACE, "%s: workspace must be 16-byte aligned", who);
    return MI_OK;
}
size_t slot_bytes(const Plan &pl, int32_t dtype) { return ((size_t)pl.n * elem_size(dtype) + 255) & ~(size_t)255; }

int32_t to_front(const Plan &pl, int32_t dtype, const void *src, void *dst, mi_stream s) {
    return mi_strided_copy_nd(dst, src, (int32_t)elem_size(dtype), pl.nd, pl.psize, pl.pstride, s);
}
int32_t back(const Plan &pl, int32_t dtype, const void *src, void *dst, mi_stream s) {
    return mi_strided_copy_nd(dst, src, (int32_t)elem_size(dtype), pl.nd, pl.isize, pl.istride, s);
}

}  // namespace

MI_API int32_t mi_softmax_dims_workspace(int32_t dtype, int32_t ndim, const int64_t *sizes, uint32_t dims_mask, size_t *bytes) {
    if (!bytes) return mi_set_error(MI_EINVAL, "mi_softmax_dims_workspace: bytes is NULL");
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_softmax_dims_workspace: unknown dtype %d", dtype);
    Plan pl;
    int32_t rc = make_plan("mi_softmax_dims_workspace", ndim, sizes, dims_mask, &pl);
    if (rc != MI_OK) return rc;
    *bytes = pl.run ? 0 : 2 * slot_bytes(pl, dtype);   // enough for every entry point of this file
    return MI_OK;
}

MI_API int32_t mi_softmax_dims(int32_t op, int32_t dtype, const void *x, void *y, int32_t ndim, const int64_t *sizes, uint32_t dims_mask,
                               void *workspace, size_t workspace_bytes, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_softmax_dims: unknown dtype %d", dtype);
    Plan pl;
    int32_t rc = make_plan("mi_softmax_dims", ndim, sizes, dims_mask, &pl);
    if (rc != MI_OK) return rc;
    if (pl.n == 0) return MI_OK;
    if (pl.run) return mi_softmax(op, dtype, x, y, pl.inner, pl.len, pl.outer, s);
    const size_t slot = slot_bytes(pl, dtype);
    if ((rc = check_ws("mi_softmax_dims", workspace, workspace_bytes, 2 * slot)) != MI_OK) return rc;
    if (!x || !y) return mi_set_error(MI_EINVAL, "mi_softmax_dims: null pointer");
    char *xp = (char *)workspace, *yp = xp + slot;
    if ((rc = to_front(pl, dtype, x, xp, s)) != MI_OK) return rc;
    if ((rc = mi_softmax(op, dtype, xp, yp, 1, pl.len, pl.outer, s)) != MI_OK) return rc;
    return back(pl, dtype, yp, y, s);
}

MI_API int32_t mi_logsumexp_dims(int32_t dtype, const void *x, void *y, int32_t ndim, const int64_t *sizes, uint32_t dims_mask,
                                 void *workspace, size_t workspace_bytes, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_logsumexp_dims: unknown dtype %d", dtype);
    Plan pl;
    int32_t rc = make_plan("mi_logsumexp_dims", ndim, sizes, dims_mask, &pl);
    if (rc != MI_OK) return rc;
    if (pl.n == 0) return MI_OK;
    if (pl.run) return mi_logsumexp(dtype, x, y, pl.inner, pl.len, pl.outer, s);
    const size_t slot = slot_bytes(pl, dtype);
    if ((rc = check_ws("mi_logsumexp_dims", workspace, workspace_bytes, slot)) != MI_OK) return rc;
    if (!x || !y) return mi_set_error(MI_EINVAL, "mi_logsumexp_dims: null pointer");
    if ((rc = to_front(pl, dtype, x, workspace, s)) != MI_OK) return rc;
    // the result keeps the other dimensions in their order and has extent 1 along the reduced ones: in memory that is
    // the (outer) vector the kernel writes, whichever way round the unit dimensions sit
    return mi_logsumexp(dtype, workspace, y, 1, pl.len, pl.outer, s);
}

MI_API int32_t mi_softmax_bwd_dims(int32_t op, int32_t dtype, const void *dy, const void *y, void *dx, int32_t ndim, const int64_t *sizes,
                                   uint32_t dims_mask, void *workspace, size_t workspace_bytes, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_softmax_bwd_dims: unknown dtype %d", dtype);
    Plan pl;
    int32_t rc = make_plan("mi_softmax_bwd_dims", ndim, sizes, dims_mask, &pl);
    if (rc != MI_OK) return rc;
    if (pl.n == 0) return MI_OK;
    if (pl.run) return mi_softmax_bwd(op, dtype, dy, y, dx, pl.inner, pl.len, pl.outer, s);
    const size_t slot = slot_bytes(pl, dtype);
    if ((rc = check_ws("mi_softmax_bwd_dims", workspace, workspace_bytes, 2 * slot)) != MI_OK) return rc;
    if (!dy || !y || !dx) return mi_set_error(MI_EINVAL, "mi_softmax_bwd_dims: null pointer");
    char *dyp = (char *)workspace, *yp = dyp + slot;
    if ((rc = to_front(pl, dtype, dy, dyp, s)) != MI_OK) return rc;
    if ((rc = to_front(pl, dtype, y, yp, s)) != MI_OK) return rc;
    if ((rc = mi_softmax_bwd(op, dtype, dyp, yp, dyp, 1, pl.len, pl.outer, s)) != MI_OK) return rc;   // dx may alias dy
    return back(pl, dtype, dyp, dx, s);
}

MI_API int32_t mi_logsumexp_bwd_dims(int32_t dtype, const void *dy, const void *x, const void *lse, void *dx, int32_t ndim,
                                     const int64_t *sizes, uint32_t dims_mask, void *workspace, size_t workspace_bytes, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_logsumexp_bwd_dims: unknown dtype %d", dtype);
    Plan pl;
    int32_t rc = make_plan("mi_logsumexp_bwd_dims", ndim, sizes, dims_mask, &pl);
    if (rc != MI_OK) return rc;
    if (pl.n == 0) return MI_OK;
    if (pl.run) return mi_logsumexp_bwd(dtype, dy, x, lse, dx, pl.inner, pl.len, pl.outer, s);
    const size_t slot = slot_bytes(pl, dtype);
    if ((rc = check_ws("mi_logsumexp_bwd_dims", workspace, workspace_bytes, 2 * slot)) != MI_OK) return rc;
    if (!dy || !x || !lse || !dx) return mi_set_error(MI_EINVAL, "mi_logsumexp_bwd_dims: null pointer");
    char *xp = (char *)workspace, *dxp = xp + slot;
    if ((rc = to_front(pl, dtype, x, xp, s)) != MI_OK) return rc;
    // dy and lse have extent 1 along the reduced dimensions: the same memory in either order (see mi_logsumexp_dims)
    if ((rc = mi_logsumexp_bwd(dtype, dy, xp, lse, dxp, 1, pl.len, pl.outer, s)) != MI_OK) return rc;
    return back(pl, dtype, dxp, dx, s);
}
