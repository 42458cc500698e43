// softmax / logsoftmax / logsumexp and the softmax gradients over any run of adjacent dimensions.
// The array is viewed as (inner, len, outer), element (i, j, o) at i + inner*(j + len*o), and the
// reduction runs over j.  Replaces, for device arrays, NNlib's
//   _softmax!      src/softmax.jl:69-79        (dims other than 1; dims = 1 keeps its own kernels in softmax.hip)
//   _logsoftmax!   src/softmax.jl:137-147
//   logsumexp      src/softmax.jl:200-203
//   _∇softmax!     src/softmax.jl:107-110      dx = dy*y - y*sum(dy*y)
//   _∇logsoftmax!  src/softmax.jl:175-177      dx = dy - sum(dy)*exp(y)
// Arithmetic in fp32.
//
// A workgroup of 256 threads owns TI consecutive `inner` positions of one `outer` slice (TI = a power
// of two <= 64, chosen by the host from `inner`) and splits j over TJ = 256/TI slices; consecutive
// lanes touch consecutive addresses whenever inner >= TI or inner == 1.  Columns of up to CACHE*TJ
// elements stay in registers between the passes (one HBM read, one write); longer ones are re-read.
#include "common.h"

namespace {

enum { OP_SOFTMAX = 0, OP_LOGSOFTMAX = 1, OP_LOGSUMEXP = 2, OP_GRAD_SOFTMAX = 3, OP_GRAD_LOGSOFTMAX = 4 };
constexpr int CACHE = 16;

struct Geometry {
    int64_t inner, len, outer, n_itiles;
    int ti_log2;
};

// reduce over the j-slices of a workgroup: lanes with equal (lane & (TI-1)) within a wavefront by
// butterfly, then the four wavefronts through LDS
template <bool IS_MAX>
__device__ inline float reduce_slices(float v, int ti_log2, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, ti = 1 << ti_log2;
    for (int o = 32; o >= ti; o >>= 1) {
        const float u = __shfl_xor(v, o, 64);
        v = IS_MAX ? fmaxf(v, u) : v + u;
    }
    __syncthreads();  // previous use of `red`
    if (lane < ti) red[wave * 64 + lane] = v;
    __syncthreads();
    const int il = lane & (ti - 1);
    float r = red[il];
#pragma unroll
    for (int w = 1; w < 4; w++) r = IS_MAX ? fmaxf(r, red[w * 64 + il]) : r + red[w * 64 + il];
    return r;
}

// the reference's elementwise rules given the column maximum m
__device__ inline float softmax_term(float x, float m) {   // src/softmax.jl:72-75
    if (m == MI_POS_INF) return x == MI_POS_INF ? 1.0f : 0.0f;
    return expf(x - m);
}
__device__ inline float logsoftmax_shift(float x, float m) {   // src/softmax.jl:140-144
    if (m == MI_POS_INF) return x == MI_POS_INF ? 0.0f : MI_NEG_INF;
    return x - m;
}

template <typename T, int OP>
__global__ __launch_bounds__(256) void softmax_nd_kernel(const typename T::type *x, const typename T::type *x2,
                                                          typename T::type *y, Geometry g) {
    typedef typename T::type t;
    __shared__ float red[256];
    const int ti = 1 << g.ti_log2, tj = 256 >> g.ti_log2;
    const int il = threadIdx.x & (ti - 1), js = threadIdx.x >> g.ti_log2;
    const int64_t n_tiles = g.n_itiles * g.outer;
    const bool cached = g.len <= (int64_t)CACHE * tj;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t o = tile / g.n_itiles, i = (tile % g.n_itiles) * ti + il;
        const bool ok = i < g.inner;
        const int64_t base = i + g.inner * g.len * o;
        const t *xc = x + base;
        const t *x2c = x2 ? x2 + base : nullptr;
        t *yc = y + base;
        float v[CACHE], v2[(OP >= OP_GRAD_SOFTMAX) ? CACHE : 1];

        if constexpr (OP == OP_GRAD_SOFTMAX || OP == OP_GRAD_LOGSOFTMAX) {
            // x = dy, x2 = y (the forward result)
            float s = 0.0f;
            if (cached) {
#pragma unroll
                for (int c = 0; c < CACHE; c++) {
                    const int64_t j = js + (int64_t)tj * c;
                    const bool in = ok && j < g.len;
                    v[c] = in ? T::to_f32(xc[g.inner * j]) : 0.0f;
                    v2[c] = in ? T::to_f32(x2c[g.inner * j]) : 0.0f;
                    s += OP == OP_GRAD_SOFTMAX ? v[c] * v2[c] : v[c];
                }
            } else if (ok) {
                for (int64_t j = js; j < g.len; j += tj) {
                    const float dy = T::to_f32(xc[g.inner * j]);
                    s += OP == OP_GRAD_SOFTMAX ? dy * T::to_f32(x2c[g.inner * j]) : dy;
                }
            }
            s = reduce_slices<false>(s, g.ti_log2, red);
            if (cached) {
#pragma unroll
                for (int c = 0; c < CACHE; c++) {
                    const int64_t j = js + (int64_t)tj * c;
                    if (ok && j < g.len)
                        yc[g.inner * j] = T::from_f32(OP == OP_GRAD_SOFTMAX ? v2[c] * (v[c] - s) : v[c] - s * expf(v2[c]));
                }
            } else if (ok) {
                for (int64_t j = js; j < g.len; j += tj) {
                    const float dy = T::to_f32(xc[g.inner * j]), yy = T::to_f32(x2c[g.inner * j]);
                    yc[g.inner * j] = T::from_f32(OP == OP_GRAD_SOFTMAX ? yy * (dy - s) : dy - s * expf(yy));
                }
            }
            continue;
        }

        // forward ops: maximum, then sum of exponentials, then the result.  fmaxf skips a NaN, but the
        // NaN still reaches every element of its column through the sum, as in the reference.
        float m = MI_NEG_INF;
        if (cached) {
#pragma unroll
            for (int c = 0; c < CACHE; c++) {
                const int64_t j = js + (int64_t)tj * c;
                v[c] = (ok && j < g.len) ? T::to_f32(xc[g.inner * j]) : MI_NEG_INF;
                m = fmaxf(m, v[c]);
            }
        } else if (ok) {
            for (int64_t j = js; j < g.len; j += tj) {
                m = fmaxf(m, T::to_f32(xc[g.inner * j]));
            }
        }
        m = reduce_slices<true>(m, g.ti_log2, red);
        float s = 0.0f;
        auto term = [&](float xv) {
            if (OP == OP_SOFTMAX) return softmax_term(xv, m);
            if (OP == OP_LOGSOFTMAX) return expf(logsoftmax_shift(xv, m));
            return expf(xv - m);   // logsumexp: no special cases (src/softmax.jl:202)
        };
        if (cached) {
#pragma unroll
            for (int c = 0; c < CACHE; c++) {
                const int64_t j = js + (int64_t)tj * c;
                if (ok && j < g.len) s += term(v[c]);
            }
        } else if (ok) {
            for (int64_t j = js; j < g.len; j += tj) s += term(T::to_f32(xc[g.inner * j]));
        }
        s = reduce_slices<false>(s, g.ti_log2, red);
        if (OP == OP_LOGSUMEXP) {
            if (ok && js == 0) y[i + g.inner * o] = T::from_f32(m + logf(s));
            continue;
        }
        const float logs = logf(s);
        auto result = [&](float xv) {
            if (OP == OP_SOFTMAX) return softmax_term(xv, m) / s;
            return logsoftmax_shift(xv, m) - logs;
        };
        if (cached) {
#pragma unroll
            for (int c = 0; c < CACHE; c++) {
                const int64_t j = js + (int64_t)tj * c;
                if (ok && j < g.len) yc[g.inner * j] = T::from_f32(result(v[c]));
            }
        } else if (ok) {
            for (int64_t j = js; j < g.len; j += tj) yc[g.inner * j] = T::from_f32(result(T::to_f32(xc[g.inner * j])));
        }
    }
}

template <typename T, int OP>
void launch_nd(const void *x, const void *x2, void *y, int64_t inner, int64_t len, int64_t outer, hipStream_t st) {
    typedef typename T::type t;
    Geometry g;
    g.inner = inner;
    g.len = len;
    g.outer = outer;
    g.ti_log2 = 0;
    while ((1 << g.ti_log2) < 64 && ((int64_t)1 << g.ti_log2) < inner) g.ti_log2++;
    g.n_itiles = (inner + (1 << g.ti_log2) - 1) >> g.ti_log2;
    int64_t blocks = g.n_itiles * outer;
    if (blocks > 262144) blocks = 262144;
    hipLaunchKernelGGL((softmax_nd_kernel<T, OP>), dim3((unsigned)blocks), dim3(256), 0, st, (const t *)x, (const t *)x2,
                       (t *)y, g);
}

template <int OP>
int32_t dispatch(const char *name, int32_t dtype, const void *x, const void *x2, void *y, int64_t inner, int64_t len,
                 int64_t outer, mi_stream s) {
    if (!mi_dtype_ok(dtype)) return mi_set_error(MI_EDTYPE, "%s: unknown dtype %d", name, dtype);
    if (inner < 0 || len < 0 || outer < 0) return mi_set_error(MI_EINVAL, "%s: negative size", name);
    if (inner == 0 || outer == 0 || (len == 0 && OP != OP_LOGSUMEXP)) return MI_OK;
    if (!x || !y || (OP >= OP_GRAD_SOFTMAX && !x2)) return mi_set_error(MI_EINVAL, "%s: null pointer", name);
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F32) launch_nd<F32, OP>(x, x2, y, inner, len, outer, st);
    else if (dtype == MI_F16) launch_nd<F16, OP>(x, x2, y, inner, len, outer, st);
    else launch_nd<BF16, OP>(x, x2, y, inner, len, outer, st);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

}  // namespace

MI_API int32_t mi_softmax(int32_t op, int32_t dtype, const void *x, void *y, int64_t inner, int64_t len, int64_t outer,
                          mi_stream s) {
    if (op == MI_SOFTMAX) {
        if (inner == 1) return mi_softmax_dim1(dtype, x, y, len, outer, s);
        return dispatch<OP_SOFTMAX>("mi_softmax", dtype, x, nullptr, y, inner, len, outer, s);
    }
    if (op == MI_LOGSOFTMAX) return dispatch<OP_LOGSOFTMAX>("mi_softmax", dtype, x, nullptr, y, inner, len, outer, s);
    return mi_set_error(MI_EINVAL, "mi_softmax: op must be MI_SOFTMAX or MI_LOGSOFTMAX, got %d", op);
}

MI_API int32_t mi_logsumexp(int32_t dtype, const void *x, void *y, int64_t inner, int64_t len, int64_t outer, mi_stream s) {
    return dispatch<OP_LOGSUMEXP>("mi_logsumexp", dtype, x, nullptr, y, inner, len, outer, s);
}

MI_API int32_t mi_softmax_bwd(int32_t op, int32_t dtype, const void *dy, const void *y, void *dx, int64_t inner, int64_t len,
                              int64_t outer, mi_stream s) {
    if (op == MI_SOFTMAX) return dispatch<OP_GRAD_SOFTMAX>("mi_softmax_bwd", dtype, dy, y, dx, inner, len, outer, s);
    if (op == MI_LOGSOFTMAX) return dispatch<OP_GRAD_LOGSOFTMAX>("mi_softmax_bwd", dtype, dy, y, dx, inner, len, outer, s);
    return mi_set_error(MI_EINVAL, "mi_softmax_bwd: op must be MI_SOFTMAX or MI_LOGSOFTMAX, got %d", op);
}
