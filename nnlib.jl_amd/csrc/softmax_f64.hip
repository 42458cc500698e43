// Softmax family for Float64 arrays (the reference's `float(T)` result type for Float64 and integer inputs:
// src/softmax.jl:56, test/softmax.jl:4-29): softmax, logsoftmax, logsumexp and the two gradients over a run of
// adjacent dimensions, the array viewed as (inner, len, outer) and reduced over len.  Plain double-precision vector
// code: every one of these is bound by memory traffic, and the matrix cores have nothing to do here.
//
// Order of operations as src/softmax.jl:69-79, 137-147, 200-203, 107-110, 175-177: maximum by comparison (a NaN never
// becomes the maximum and poisons the column through its own exponential), the +Inf branch of :73-75, one exponential
// per element, division by the sum.
//
//   inner == 1  one wavefront per column; columns of up to 1024 elements stay in registers (one read, one write),
//               longer ones are streamed three times (maximum, sum, result; the re-reads come from L2 for columns
//               that fit it);
//   inner  > 1  one thread per (inner, outer) position walking its column with stride `inner`: adjacent threads
//               read adjacent addresses.
#include "common.h"

namespace {

enum { OP64_SOFTMAX = 0, OP64_LOGSOFTMAX = 1, OP64_LOGSUMEXP = 2, OP64_GRAD_SOFTMAX = 3, OP64_GRAD_LOGSOFTMAX = 4 };

constexpr double NEG_INF64 = -__builtin_huge_val();
constexpr double POS_INF64 = __builtin_huge_val();

__device__ inline double wave_max64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const double o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}
__device__ inline double wave_sum64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// first pass value of element v against the column maximum m: what the sum adds up
template <int OP>
__device__ inline double term64(double v, double m) {
    if (OP == OP64_SOFTMAX) {
        if (m == POS_INF64) return v == POS_INF64 ? 1.0 : 0.0;
        return exp(v - m);
    }
    if (OP == OP64_LOGSOFTMAX) {
        const double d = m == POS_INF64 ? (v == POS_INF64 ? 0.0 : NEG_INF64) : v - m;
        return exp(d);
    }
    return exp(v - m);   // logsumexp
}
// result for element v given the column's maximum and sum
template <int OP>
__device__ inline double result64(double v, double m, double s) {
    if (OP == OP64_SOFTMAX) return term64<OP>(v, m) / s;
    const double d = m == POS_INF64 ? (v == POS_INF64 ? 0.0 : NEG_INF64) : v - m;
    return d - log(s);
}

// ---- inner == 1: a wavefront per column ---------------------------------------------------------------------------
constexpr int CACHE = 16;   // elements per lane held in registers: columns up to 64 * 16

template <int OP, bool CACHED>
__global__ __launch_bounds__(256) void softmax64_col_kernel(const double *__restrict__ x, const double *__restrict__ x2,
                                                            double *__restrict__ y, int64_t len, int64_t outer) {
    const int lane = threadIdx.x & 63;
    const int64_t waves = (int64_t)gridDim.x * 4;
    for (int64_t col = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); col < outer; col += waves) {
        const double *xc = x + col * len;
        const double *gc = OP >= OP64_GRAD_SOFTMAX ? x2 + col * len : nullptr;   // x = dy, x2 = y for the gradients
        double *yc = y + (OP == OP64_LOGSUMEXP ? col : col * len);
        double r[CACHE], g[CACHE];
        if (CACHED) {
#pragma unroll
            for (int u = 0; u < CACHE; u++) {
                const int64_t j = lane + 64 * u;
                r[u] = j < len ? xc[j] : (OP >= OP64_GRAD_SOFTMAX ? 0.0 : NEG_INF64);
                if (OP >= OP64_GRAD_SOFTMAX) g[u] = j < len ? gc[j] : 0.0;
            }
        }
        if (OP >= OP64_GRAD_SOFTMAX) {
            // softmax: dx = dy*y - y*sum(dy*y); logsoftmax: dx = dy - sum(dy)*exp(y)
            double s = 0.0;
            if (CACHED) {
#pragma unroll
                for (int u = 0; u < CACHE; u++) s += OP == OP64_GRAD_SOFTMAX ? r[u] * g[u] : r[u];
            } else {
                for (int64_t j = lane; j < len; j += 64) s += OP == OP64_GRAD_SOFTMAX ? xc[j] * gc[j] : xc[j];
            }
            s = wave_sum64(s);
            if (CACHED) {
#pragma unroll
                for (int u = 0; u < CACHE; u++) {
                    const int64_t j = lane + 64 * u;
                    if (j < len) yc[j] = OP == OP64_GRAD_SOFTMAX ? r[u] * g[u] - g[u] * s : r[u] - s * exp(g[u]);
                }
            } else {
                for (int64_t j = lane; j < len; j += 64) {
                    const double dy = xc[j], yy = gc[j];
                    yc[j] = OP == OP64_GRAD_SOFTMAX ? dy * yy - yy * s : dy - s * exp(yy);
                }
            }
            continue;
        }
        double m = NEG_INF64;
        if (CACHED) {
#pragma unroll
            for (int u = 0; u < CACHE; u++) m = r[u] > m ? r[u] : m;
        } else {
            for (int64_t j = lane; j < len; j += 64) {
                const double v = xc[j];
                m = v > m ? v : m;
            }
        }
        m = wave_max64(m);
        double s = 0.0;
        if (CACHED) {
#pragma unroll
            for (int u = 0; u < CACHE; u++)
                if (lane + 64 * u < len) s += term64<OP>(r[u], m);
        } else {
            for (int64_t j = lane; j < len; j += 64) s += term64<OP>(xc[j], m);
        }
        s = wave_sum64(s);
        if (OP == OP64_LOGSUMEXP) {
            if (lane == 0) yc[0] = m + log(s);
            continue;
        }
        if (CACHED) {
#pragma unroll
            for (int u = 0; u < CACHE; u++) {
                const int64_t j = lane + 64 * u;
                if (j < len) yc[j] = result64<OP>(r[u], m, s);
            }
        } else {
            for (int64_t j = lane; j < len; j += 64) yc[j] = result64<OP>(xc[j], m, s);
        }
    }
}

// ---- inner > 1: a thread per (inner, outer) position ----------------------------------------------------------------
template <int OP>
__global__ __launch_bounds__(256) void softmax64_strided_kernel(const double *__restrict__ x, const double *__restrict__ x2,
                                                                double *__restrict__ y, int64_t inner, int64_t len, int64_t outer) {
    const int64_t n = inner * outer, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) {
        const int64_t i = idx % inner, o = idx / inner;
        const double *xc = x + i + inner * len * o;
        const double *gc = OP >= OP64_GRAD_SOFTMAX ? x2 + i + inner * len * o : nullptr;
        double *yc = OP == OP64_LOGSUMEXP ? y + idx : y + i + inner * len * o;
        if (OP >= OP64_GRAD_SOFTMAX) {
            double s = 0.0;
            for (int64_t j = 0; j < len; j++) s += OP == OP64_GRAD_SOFTMAX ? xc[j * inner] * gc[j * inner] : xc[j * inner];
            for (int64_t j = 0; j < len; j++) {
                const double dy = xc[j * inner], yy = gc[j * inner];
                yc[j * inner] = OP == OP64_GRAD_SOFTMAX ? dy * yy - yy * s : dy - s * exp(yy);
            }
            continue;
        }
        double m = NEG_INF64;
        for (int64_t j = 0; j < len; j++) {
            const double v = xc[j * inner];
            m = v > m ? v : m;
        }
        double s = 0.0;
        for (int64_t j = 0; j < len; j++) s += term64<OP>(xc[j * inner], m);
        if (OP == OP64_LOGSUMEXP) {
            yc[0] = m + log(s);
            continue;
        }
        for (int64_t j = 0; j < len; j++) yc[j * inner] = result64<OP>(xc[j * inner], m, s);
    }
}

// dx[i,j,o] = dy[i,o] * exp(x[i,j,o] - lse[i,o]); NaN where the result of logsumexp is not finite (src/softmax.jl:205-212
// computes exp(x - max) there, which is NaN)
__global__ __launch_bounds__(256) void logsumexp_bwd64_kernel(const double *dy, const double *x, const double *lse, double *dx,
                                                              int64_t inner, int64_t len, int64_t outer) {
    const int64_t n = inner * len * outer, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) {
        const int64_t i = idx % inner, o = idx / (inner * len);
        const double z = lse[i + inner * o], g = dy[i + inner * o];
        const bool finite = z > NEG_INF64 && z < POS_INF64;
        dx[idx] = finite ? g * exp(x[idx] - z) : __builtin_nan("");
    }
}

template <int OP>
void launch64(const double *x, const double *x2, double *y, int64_t inner, int64_t len, int64_t outer, hipStream_t st) {
    if (inner == 1) {
        int64_t blocks = (outer + 3) / 4;
        if (blocks > 131072) blocks = 131072;
        if (len <= 64 * CACHE) hipLaunchKernelGGL((softmax64_col_kernel<OP, true>), dim3((unsigned)blocks), dim3(256), 0, st, x, x2, y, len, outer);
        else hipLaunchKernelGGL((softmax64_col_kernel<OP, false>), dim3((unsigned)blocks), dim3(256), 0, st, x, x2, y, len, outer);
        return;
    }
    int64_t blocks = (inner * outer + 255) / 256;
    if (blocks > 131072) blocks = 131072;
    hipLaunchKernelGGL((softmax64_strided_kernel<OP>), dim3((unsigned)blocks), dim3(256), 0, st, x, x2, y, inner, len, outer);
}

}  // namespace

// op: 0 softmax, 1 logsoftmax, 2 logsumexp (y: (inner, outer)), 3 / 4 their gradients (x = dy, x2 = y).  Sizes are
// positive and pointers checked by the caller (the entry points of softmax.hip / softmax_nd.hip).
int32_t launch_softmax_family_f64(int op, const void *x, const void *x2, void *y, int64_t inner, int64_t len, int64_t outer, hipStream_t st) {
    const double *a = (const double *)x, *b = (const double *)x2;
    double *c = (double *)y;
    switch (op) {
    case OP64_SOFTMAX: launch64<OP64_SOFTMAX>(a, b, c, inner, len, outer, st); break;
    case OP64_LOGSOFTMAX: launch64<OP64_LOGSOFTMAX>(a, b, c, inner, len, outer, st); break;
    case OP64_LOGSUMEXP: launch64<OP64_LOGSUMEXP>(a, b, c, inner, len, outer, st); break;
    case OP64_GRAD_SOFTMAX: launch64<OP64_GRAD_SOFTMAX>(a, b, c, inner, len, outer, st); break;
    default: launch64<OP64_GRAD_LOGSOFTMAX>(a, b, c, inner, len, outer, st); break;
    }
    MI_LAUNCH_CHECK();
    return MI_OK;
}

int32_t launch_logsumexp_bwd_f64(const void *dy, const void *x, const void *lse, void *dx, int64_t inner, int64_t len, int64_t outer,
                                 hipStream_t st) {
    int64_t blocks = (inner * len * outer + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(logsumexp_bwd64_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const double *)dy, (const double *)x,
                       (const double *)lse, (double *)dx, inner, len, outer);
    MI_LAUNCH_CHECK();
    return MI_OK;
}
