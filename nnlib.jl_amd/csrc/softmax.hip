// softmax over the first (contiguous) dimension of a column-major (rows, cols) matrix.
// Replaces NNlib's _softmax! for dims = 1 (src/softmax.jl:69-79); arithmetic in fp32.
#include "common.h"

// The reference's elementwise rule: with column maximum m,
//   m == +Inf : e = (x == +Inf) ? 1 : 0          (src/softmax.jl:74-75)
//   otherwise : e = exp(x - m)                   (src/softmax.jl:72; -Inf - -Inf = NaN stays NaN)
__device__ static inline float softmax_term(float x, float m) {
    if (m == MI_POS_INF) return x == MI_POS_INF ? 1.0f : 0.0f;
    return expf(x - m);
}

__device__ static inline float block_reduce(float v, float *red, bool is_max) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    v = is_max ? mi_wave_max(v) : mi_wave_sum(v);
    __syncthreads(); // protect `red` from the previous use
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < nw; w++) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// One workgroup per column.  Columns of up to CACHE*blockDim elements are held in
// registers between the passes (one HBM read, one write); longer columns are re-read.
template <typename T, int CACHE>
__global__ __launch_bounds__(256) void softmax_dim1_kernel(const typename T::type *x,
                                                            typename T::type *y, int64_t rows,
                                                            int64_t cols) {
    __shared__ float red[8];
    for (int64_t c = blockIdx.x; c < cols; c += gridDim.x) {
        const typename T::type *xc = x + c * rows;
        typename T::type *yc = y + c * rows;
        const bool cached = rows <= (int64_t)CACHE * blockDim.x;
        float v[CACHE];
        float m = MI_NEG_INF;
        if (cached) {
#pragma unroll
            for (int i = 0; i < CACHE; i++) {
                int64_t r = (int64_t)i * blockDim.x + threadIdx.x;
                v[i] = r < rows ? T::to_f32(xc[r]) : MI_NEG_INF;
                m = fmaxf(m, v[i]);
            }
        } else {
            for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) m = fmaxf(m, T::to_f32(xc[r]));
        }
        m = block_reduce(m, red, true);
        float s = 0.0f;
        if (cached) {
#pragma unroll
            for (int i = 0; i < CACHE; i++) {
                int64_t r = (int64_t)i * blockDim.x + threadIdx.x;
                if (r < rows) {
                    v[i] = softmax_term(v[i], m);
                    s += v[i];
                }
            }
        } else {
            for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) s += softmax_term(T::to_f32(xc[r]), m);
        }
        s = block_reduce(s, red, false);
        if (cached) {
#pragma unroll
            for (int i = 0; i < CACHE; i++) {
                int64_t r = (int64_t)i * blockDim.x + threadIdx.x;
                if (r < rows) yc[r] = T::from_f32(v[i] / s);
            }
        } else {
            for (int64_t r = threadIdx.x; r < rows; r += blockDim.x)
                yc[r] = T::from_f32(softmax_term(T::to_f32(xc[r]), m) / s);
        }
    }
}

// Short columns: one wavefront per column, four columns per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void softmax_dim1_wave_kernel(const typename T::type *x,
                                                                 typename T::type *y, int64_t rows,
                                                                 int64_t cols) {
    const int lane = threadIdx.x & 63;
    int64_t c = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t cstride = (int64_t)gridDim.x * 4;
    for (; c < cols; c += cstride) {
        const typename T::type *xc = x + c * rows;
        typename T::type *yc = y + c * rows;
        float v[4];
        float m = MI_NEG_INF;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int64_t r = i * 64 + lane;
            v[i] = r < rows ? T::to_f32(xc[r]) : MI_NEG_INF;
            m = fmaxf(m, v[i]);
        }
        m = mi_wave_max(m);
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int64_t r = i * 64 + lane;
            if (r < rows) {
                v[i] = softmax_term(v[i], m);
                s += v[i];
            }
        }
        s = mi_wave_sum(s);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int64_t r = i * 64 + lane;
            if (r < rows) yc[r] = T::from_f32(v[i] / s);
        }
    }
}

// Columns of up to 64 * NCH * VEC elements whose rows can be moved in 16-byte pieces: one wavefront per
// column, NCH pieces per lane held in registers, reductions by wavefront shuffles only (no LDS, no
// barrier): one read and one write per element with four columns in flight per workgroup.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void softmax_dim1_wave_vec_kernel(const typename T::type *x, typename T::type *y,
                                                                     int64_t rows, int64_t cols) {
    typedef typename T::type t;
    constexpr int VEC = 16 / (int)sizeof(t);
    const int lane = threadIdx.x & 63;
    const int64_t nchunks = rows / VEC;
    int64_t c = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t cstride = (int64_t)gridDim.x * 4;
    for (; c < cols; c += cstride) {
        const t *xc = x + c * rows;
        t *yc = y + c * rows;
        float v[NCH][VEC];
        float m = MI_NEG_INF;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int64_t ch = lane + 64 * i;
            if (ch < nchunks) {
                const u32x4_t raw = *(const u32x4_t *)(xc + ch * VEC);
                if constexpr (VEC == 4) {
                    const floatx4_t f = __builtin_bit_cast(floatx4_t, raw);
#pragma unroll
                    for (int e = 0; e < VEC; e++) v[i][e] = f[e];
                } else {
                    const typename T::vec8 h = __builtin_bit_cast(typename T::vec8, raw);
#pragma unroll
                    for (int e = 0; e < VEC; e++) v[i][e] = T::to_f32(h[e]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) v[i][e] = MI_NEG_INF;
            }
#pragma unroll
            for (int e = 0; e < VEC; e++) m = fmaxf(m, v[i][e]);
        }
        m = mi_wave_max(m);
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NCH; i++)
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                // padding lanes hold -Inf: their term is 0 unless the whole column is -Inf (then NaN, as for real entries)
                v[i][e] = (lane + 64 * i < nchunks) ? softmax_term(v[i][e], m) : 0.0f;
                s += v[i][e];
            }
        s = mi_wave_sum(s);
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int64_t ch = lane + 64 * i;
            if (ch < nchunks) {
                if constexpr (VEC == 4) {
                    floatx4_t f;
#pragma unroll
                    for (int e = 0; e < VEC; e++) f[e] = v[i][e] / s;
                    *(floatx4_t *)(yc + ch * VEC) = f;
                } else {
                    typename T::vec8 h;
#pragma unroll
                    for (int e = 0; e < VEC; e++) h[e] = T::from_f32(v[i][e] / s);
                    *(u32x4_t *)(yc + ch * VEC) = __builtin_bit_cast(u32x4_t, h);
                }
            }
        }
    }
}

template <typename T>
static void launch_softmax(const void *x, void *y, int64_t rows, int64_t cols, hipStream_t st) {
    typedef typename T::type t;
    constexpr int VEC = 16 / (int)sizeof(t);
    const bool vec_ok = rows % VEC == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0;
    if (vec_ok && rows > 256 && rows <= 64 * 8 * VEC) {
        int64_t blocks = (cols + 3) / 4;
        if (blocks > 262144) blocks = 262144;
        const dim3 g((unsigned)blocks), b(256);
        const int64_t nch = (rows / VEC + 63) / 64;
        if (nch <= 2) hipLaunchKernelGGL((softmax_dim1_wave_vec_kernel<T, 2>), g, b, 0, st, (const t *)x, (t *)y, rows, cols);
        else if (nch <= 4) hipLaunchKernelGGL((softmax_dim1_wave_vec_kernel<T, 4>), g, b, 0, st, (const t *)x, (t *)y, rows, cols);
        else hipLaunchKernelGGL((softmax_dim1_wave_vec_kernel<T, 8>), g, b, 0, st, (const t *)x, (t *)y, rows, cols);
        return;
    }
    if (rows <= 256) {
        int64_t blocks = (cols + 3) / 4;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(softmax_dim1_wave_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, st, (const t *)x, (t *)y,
                           rows, cols);
    } else {
        int64_t blocks = cols > 65536 ? 65536 : cols;
        hipLaunchKernelGGL((softmax_dim1_kernel<T, 16>), dim3((unsigned)blocks), dim3(256), 0, st, (const t *)x, (t *)y,
                           rows, cols);
    }
}

MI_API int32_t mi_softmax_dim1(int32_t dtype, const void *x, void *y, int64_t rows, int64_t cols, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_softmax_dim1: unknown dtype %d", dtype);
    if (rows < 0 || cols < 0) return mi_set_error(MI_EINVAL, "mi_softmax_dim1: negative size");
    if (rows == 0 || cols == 0) return MI_OK;
    if (!x || !y) return mi_set_error(MI_EINVAL, "mi_softmax_dim1: null pointer");
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F64) return launch_softmax_family_f64(0, x, nullptr, y, 1, rows, cols, st);
    if (dtype == MI_F32) launch_softmax<F32>(x, y, rows, cols, st);
    else if (dtype == MI_F16) launch_softmax<F16>(x, y, rows, cols, st);
    else launch_softmax<BF16>(x, y, rows, cols, st);
    MI_LAUNCH_CHECK();
    return MI_OK;
}
