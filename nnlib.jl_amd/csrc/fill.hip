// Reproducible input generators, dtype conversion and make_causal_mask.
#include "common.h"
#include <type_traits>

__device__ static inline uint64_t counter_bits(uint64_t seed, uint64_t stream_id, uint64_t i) {
    return mi_counter_bits(mi_stream_key(seed, stream_id), i);
}

template <typename T>
__global__ void randn_kernel(typename T::type *p, int64_t n, uint64_t seed, uint64_t stream_id, float scale) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint64_t r = counter_bits(seed, stream_id, (uint64_t)i);
        // two uniforms in (0,1]: 24 bits each
        float u1 = ((float)((r >> 40) & 0xFFFFFF) + 1.0f) * (1.0f / 16777216.0f);
        float u2 = ((float)((r >> 8) & 0xFFFFFF) + 1.0f) * (1.0f / 16777216.0f);
        float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
        p[i] = T::from_f32(scale * z);
    }
}

__global__ void bernoulli_kernel(uint8_t *p, int64_t n, uint64_t seed, uint64_t stream_id, float keep) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint64_t r = counter_bits(seed, stream_id, (uint64_t)i);
        float u = (float)((r >> 40) & 0xFFFFFF) * (1.0f / 16777216.0f);
        p[i] = (uint8_t)(u < keep);
    }
}

// dropout(x, p; dims = :)  (src/dropout.jl:38-53)
template <typename T>
__global__ void dropout_kernel(const typename T::type *x, typename T::type *y, int64_t n, uint64_t key, uint32_t thresh,
                               float scale) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) y[i] = T::from_f32(mi_dropout_keep(key, (uint64_t)i, thresh) ? T::to_f32(x[i]) * scale : 0.0f);
}

// dropout(x, p; dims): one keep decision per index along `dims`, shared along every other dimension
// (the random array has extent 1 there, _dropout_shape in src/dropout.jl).  mstride[d] is the stride of
// dimension d in that array, 0 for the shared ones; its column-major linear index is the counter.
struct DropDims {
    int64_t size[8], mstride[8];
    int32_t nd;
};
template <typename T>
__global__ void dropout_dims_kernel(const typename T::type *x, typename T::type *y, int64_t n, DropDims g, uint64_t key,
                                    uint32_t thresh, float scale) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        int64_t rest = i, at = 0;
        for (int d = 0; d < g.nd; d++) {
            at += (rest % g.size[d]) * g.mstride[d];
            rest /= g.size[d];
        }
        y[i] = T::from_f32(mi_dropout_keep(key, (uint64_t)at, thresh) ? T::to_f32(x[i]) * scale : 0.0f);
    }
}

template <typename TD, typename TS>
__global__ void convert_kernel(typename TD::type *d, const typename TS::type *s, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) d[i] = TD::from_f32(TS::to_f32(s[i]));
}

// dst (contiguous, column-major d0 x d1 x d2) = src addressed with element strides (s0, s1, s2):
// materialises a lazy PermutedDimsArray / transpose view (what the reference's copy(X) does in
// _copy_if_faster, src/batched/batchedmul.jl:76-83)
template <int BYTES>
__global__ void strided_copy_kernel(void *dst, const void *src, int64_t d0, int64_t d1, int64_t d2, int64_t s0, int64_t s1,
                                    int64_t s2) {
    typedef typename std::conditional<BYTES == 16, u32x4_t, typename std::conditional<BYTES == 8, uint64_t, typename std::conditional<BYTES == 4, uint32_t,
            typename std::conditional<BYTES == 2, uint16_t, uint8_t>::type>::type>::type>::type word;
    const int64_t n = d0 * d1 * d2;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += stride) {
        const int64_t i0 = idx % d0, i1 = (idx / d0) % d1, i2 = idx / (d0 * d1);
        ((word *)dst)[idx] = ((const word *)src)[i0 * s0 + i1 * s1 + i2 * s2];
    }
}

// the same for up to 8 dimensions (permutedims of an N-d array)
struct CopyDims {
    int64_t size[8], stride[8];
    int32_t nd;
};
template <int BYTES>
__global__ void strided_copy_nd_kernel(void *dst, const void *src, int64_t n, CopyDims g) {
    typedef typename std::conditional<BYTES == 16, u32x4_t, typename std::conditional<BYTES == 8, uint64_t, typename std::conditional<BYTES == 4, uint32_t,
            typename std::conditional<BYTES == 2, uint16_t, uint8_t>::type>::type>::type>::type word;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += stride) {
        int64_t rest = idx, at = 0;
        for (int d = 0; d < g.nd; d++) {
            at += (rest % g.size[d]) * g.stride[d];
            rest /= g.size[d];
        }
        ((word *)dst)[idx] = ((const word *)src)[at];
    }
}

// m[i + j*len] = (i <= j): reference src/attention.jl:145,149-153
__global__ void causal_mask_kernel(uint8_t *m, int64_t len) {
    int64_t n = len * len;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += stride) {
        int64_t i = idx % len, j = idx / len;
        m[idx] = (uint8_t)(i <= j);
    }
}

static inline int grid_for(int64_t n) {
    int64_t b = (n + 255) / 256;
    return (int)(b < 1 ? 1 : (b > 16384 ? 16384 : b));
}

MI_API int32_t mi_randn_fill(void *ptr, int32_t dtype, int64_t n, uint64_t seed, uint64_t stream_id,
                             float scale, mi_stream s) {
    if (!mi_dtype_ok(dtype)) return mi_set_error(MI_EDTYPE, "mi_randn_fill: unknown dtype %d", dtype);
    if (n < 0) return mi_set_error(MI_EINVAL, "mi_randn_fill: negative length");
    if (n == 0) return MI_OK;
    if (!ptr) return mi_set_error(MI_EINVAL, "mi_randn_fill: null pointer");
    dim3 g(grid_for(n)), b(256);
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F32) hipLaunchKernelGGL(randn_kernel<F32>, g, b, 0, st, (float *)ptr, n, seed, stream_id, scale);
    else if (dtype == MI_F16) hipLaunchKernelGGL(randn_kernel<F16>, g, b, 0, st, (_Float16 *)ptr, n, seed, stream_id, scale);
    else hipLaunchKernelGGL(randn_kernel<BF16>, g, b, 0, st, (__bf16 *)ptr, n, seed, stream_id, scale);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_bernoulli_fill(uint8_t *mask, int64_t n, uint64_t seed, uint64_t stream_id, float keep_prob,
                                 mi_stream s) {
    if (n < 0) return mi_set_error(MI_EINVAL, "mi_bernoulli_fill: negative length");
    if (n == 0) return MI_OK;
    if (!mask) return mi_set_error(MI_EINVAL, "mi_bernoulli_fill: null pointer");
    hipLaunchKernelGGL(bernoulli_kernel, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)s, mask, n, seed, stream_id,
                       keep_prob);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_dropout(int32_t dtype, const void *x, void *y, int64_t n, float p, uint64_t seed, mi_stream s) {
    if (!mi_dtype_ok(dtype)) return mi_set_error(MI_EDTYPE, "mi_dropout: unknown dtype %d", dtype);
    if (n < 0) return mi_set_error(MI_EINVAL, "mi_dropout: negative length");
    if (!(p >= 0.0f && p <= 1.0f)) return mi_set_error(MI_EINVAL, "dropout expects a probability 0 <= p <= 1");   // src/dropout.jl:43
    if (n == 0) return MI_OK;
    if (!x || !y) return mi_set_error(MI_EINVAL, "mi_dropout: null pointer");
    const uint64_t key = mi_stream_key(seed, MI_DROPOUT_STREAM);
    const uint32_t thresh = mi_dropout_threshold(p);
    const float scale = p < 1.0f ? 1.0f / (1.0f - p) : 0.0f;
    dim3 g(grid_for(n)), b(256);
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F32) hipLaunchKernelGGL(dropout_kernel<F32>, g, b, 0, st, (const float *)x, (float *)y, n, key, thresh, scale);
    else if (dtype == MI_F16) hipLaunchKernelGGL(dropout_kernel<F16>, g, b, 0, st, (const _Float16 *)x, (_Float16 *)y, n, key, thresh, scale);
    else hipLaunchKernelGGL(dropout_kernel<BF16>, g, b, 0, st, (const __bf16 *)x, (__bf16 *)y, n, key, thresh, scale);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_dropout_dims(int32_t dtype, const void *x, void *y, int32_t ndim, const int64_t *sizes, uint32_t dims_mask,
                               float p, uint64_t seed, mi_stream s) {
    if (!mi_dtype_ok(dtype)) return mi_set_error(MI_EDTYPE, "mi_dropout_dims: unknown dtype %d", dtype);
    if (ndim < 0 || ndim > 8 || (ndim > 0 && !sizes)) return mi_set_error(MI_EINVAL, "mi_dropout_dims: 0 to 8 dimensions");
    if (!(p >= 0.0f && p <= 1.0f)) return mi_set_error(MI_EINVAL, "dropout expects a probability 0 <= p <= 1");
    DropDims g;
    g.nd = ndim;
    int64_t n = 1, ms = 1;
    for (int d = 0; d < ndim; d++) {
        if (sizes[d] < 0) return mi_set_error(MI_EINVAL, "mi_dropout_dims: negative size");
        g.size[d] = sizes[d];
        const bool own = (dims_mask >> d) & 1;
        g.mstride[d] = own ? ms : 0;
        if (own) ms *= sizes[d];
        n *= sizes[d];
    }
    if (n == 0) return MI_OK;
    if (!x || !y) return mi_set_error(MI_EINVAL, "mi_dropout_dims: null pointer");
    const uint64_t key = mi_stream_key(seed, MI_DROPOUT_STREAM);
    const uint32_t thresh = mi_dropout_threshold(p);
    const float scale = p < 1.0f ? 1.0f / (1.0f - p) : 0.0f;
    dim3 gr(grid_for(n)), b(256);
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F32) hipLaunchKernelGGL(dropout_dims_kernel<F32>, gr, b, 0, st, (const float *)x, (float *)y, n, g, key, thresh, scale);
    else if (dtype == MI_F16) hipLaunchKernelGGL(dropout_dims_kernel<F16>, gr, b, 0, st, (const _Float16 *)x, (_Float16 *)y, n, g, key, thresh, scale);
    else hipLaunchKernelGGL(dropout_dims_kernel<BF16>, gr, b, 0, st, (const __bf16 *)x, (__bf16 *)y, n, g, key, thresh, scale);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <typename TD>
static void launch_convert_from(void *d, const void *src, int32_t ds, int64_t n, hipStream_t st) {
    dim3 g(grid_for(n)), b(256);
    typedef typename TD::type td;
    if (ds == MI_F32) hipLaunchKernelGGL((convert_kernel<TD, F32>), g, b, 0, st, (td *)d, (const float *)src, n);
    else if (ds == MI_F16) hipLaunchKernelGGL((convert_kernel<TD, F16>), g, b, 0, st, (td *)d, (const _Float16 *)src, n);
    else hipLaunchKernelGGL((convert_kernel<TD, BF16>), g, b, 0, st, (td *)d, (const __bf16 *)src, n);
}

// conversions that involve Float64: to it from every real element type (what `float(T)` of an integer array is,
// src/softmax.jl:56), and from it to the narrower floating-point types
template <typename TD, typename TS>
__global__ __launch_bounds__(256) void convert_plain_kernel(TD *dst, const TS *src, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = (TD)src[i];
}
template <typename TD>
static bool launch_convert_plain_from(void *d, const void *src, int32_t ds, int64_t n, hipStream_t st) {
    dim3 g(grid_for(n)), b(256);
    switch (ds) {
    case MI_F64: hipLaunchKernelGGL((convert_plain_kernel<TD, double>), g, b, 0, st, (TD *)d, (const double *)src, n); return true;
    case MI_F32: hipLaunchKernelGGL((convert_plain_kernel<TD, float>), g, b, 0, st, (TD *)d, (const float *)src, n); return true;
    case MI_F16: hipLaunchKernelGGL((convert_plain_kernel<TD, _Float16>), g, b, 0, st, (TD *)d, (const _Float16 *)src, n); return true;
    case MI_BF16: hipLaunchKernelGGL((convert_plain_kernel<TD, __bf16>), g, b, 0, st, (TD *)d, (const __bf16 *)src, n); return true;
    case MI_I32: hipLaunchKernelGGL((convert_plain_kernel<TD, int32_t>), g, b, 0, st, (TD *)d, (const int32_t *)src, n); return true;
    case MI_I64: hipLaunchKernelGGL((convert_plain_kernel<TD, int64_t>), g, b, 0, st, (TD *)d, (const int64_t *)src, n); return true;
    default: return false;
    }
}

MI_API int32_t mi_convert(void *dst, int32_t dd, const void *src, int32_t ds, int64_t n, mi_stream s) {
    if (dd == MI_F64 || ds == MI_F64) {
        if (n < 0) return mi_set_error(MI_EINVAL, "mi_convert: negative length");
        if (n == 0) return MI_OK;
        if (!dst || !src) return mi_set_error(MI_EINVAL, "mi_convert: null pointer");
        hipStream_t st64 = (hipStream_t)s;
        bool ok = false;
        dim3 g64(grid_for(n)), b64(256);
        const double *s64 = (const double *)src;
        ok = true;
        if (dd == MI_F64) ok = launch_convert_plain_from<double>(dst, src, ds, n, st64);
        else if (dd == MI_F32) hipLaunchKernelGGL((convert_plain_kernel<float, double>), g64, b64, 0, st64, (float *)dst, s64, n);
        else if (dd == MI_F16) hipLaunchKernelGGL((convert_plain_kernel<_Float16, double>), g64, b64, 0, st64, (_Float16 *)dst, s64, n);
        else if (dd == MI_BF16) hipLaunchKernelGGL((convert_plain_kernel<__bf16, double>), g64, b64, 0, st64, (__bf16 *)dst, s64, n);
        else ok = false;
        if (!ok) return mi_set_error(MI_EDTYPE, "mi_convert: no conversion from dtype %d to dtype %d", ds, dd);
        MI_LAUNCH_CHECK();
        return MI_OK;
    }
    if (!mi_dtype_ok(dd) || !mi_dtype_ok(ds)) return mi_set_error(MI_EDTYPE, "mi_convert: unknown dtype");
    if (n < 0) return mi_set_error(MI_EINVAL, "mi_convert: negative length");
    if (n == 0) return MI_OK;
    if (!dst || !src) return mi_set_error(MI_EINVAL, "mi_convert: null pointer");
    hipStream_t st = (hipStream_t)s;
    if (dd == MI_F32) launch_convert_from<F32>(dst, src, ds, n, st);
    else if (dd == MI_F16) launch_convert_from<F16>(dst, src, ds, n, st);
    else launch_convert_from<BF16>(dst, src, ds, n, st);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_strided_copy(void *dst, const void *src, int32_t elem_bytes, int64_t d0, int64_t d1, int64_t d2, int64_t s0,
                               int64_t s1, int64_t s2, mi_stream s) {
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8 && elem_bytes != 16)
        return mi_set_error(MI_EINVAL, "mi_strided_copy: element size must be 1, 2, 4, 8 or 16 bytes");
    if (d0 < 0 || d1 < 0 || d2 < 0 || s0 < 0 || s1 < 0 || s2 < 0) return mi_set_error(MI_EINVAL, "mi_strided_copy: negative size or stride");
    const int64_t n = d0 * d1 * d2;
    if (n == 0) return MI_OK;
    if (!dst || !src) return mi_set_error(MI_EINVAL, "mi_strided_copy: null pointer");
    dim3 g(grid_for(n)), b(256);
    hipStream_t st = (hipStream_t)s;
    if (elem_bytes == 16) hipLaunchKernelGGL(strided_copy_kernel<16>, g, b, 0, st, dst, src, d0, d1, d2, s0, s1, s2);
    else if (elem_bytes == 8) hipLaunchKernelGGL(strided_copy_kernel<8>, g, b, 0, st, dst, src, d0, d1, d2, s0, s1, s2);
    else if (elem_bytes == 4) hipLaunchKernelGGL(strided_copy_kernel<4>, g, b, 0, st, dst, src, d0, d1, d2, s0, s1, s2);
    else if (elem_bytes == 2) hipLaunchKernelGGL(strided_copy_kernel<2>, g, b, 0, st, dst, src, d0, d1, d2, s0, s1, s2);
    else hipLaunchKernelGGL(strided_copy_kernel<1>, g, b, 0, st, dst, src, d0, d1, d2, s0, s1, s2);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_strided_copy_nd(void *dst, const void *src, int32_t elem_bytes, int32_t ndim, const int64_t *sizes,
                                  const int64_t *strides, mi_stream s) {
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8 && elem_bytes != 16)
        return mi_set_error(MI_EINVAL, "mi_strided_copy_nd: element size must be 1, 2, 4, 8 or 16 bytes");
    if (ndim < 0 || ndim > 8 || (ndim > 0 && (!sizes || !strides))) return mi_set_error(MI_EINVAL, "mi_strided_copy_nd: 0 to 8 dimensions");
    CopyDims g;
    g.nd = ndim;
    int64_t n = 1;
    for (int d = 0; d < ndim; d++) {
        if (sizes[d] < 0 || strides[d] < 0) return mi_set_error(MI_EINVAL, "mi_strided_copy_nd: negative size or stride");
        g.size[d] = sizes[d];
        g.stride[d] = strides[d];
        n *= sizes[d];
    }
    if (n == 0) return MI_OK;
    if (!dst || !src) return mi_set_error(MI_EINVAL, "mi_strided_copy_nd: null pointer");
    dim3 gr(grid_for(n)), b(256);
    hipStream_t st = (hipStream_t)s;
    if (elem_bytes == 16) hipLaunchKernelGGL(strided_copy_nd_kernel<16>, gr, b, 0, st, dst, src, n, g);
    else if (elem_bytes == 8) hipLaunchKernelGGL(strided_copy_nd_kernel<8>, gr, b, 0, st, dst, src, n, g);
    else if (elem_bytes == 4) hipLaunchKernelGGL(strided_copy_nd_kernel<4>, gr, b, 0, st, dst, src, n, g);
    else if (elem_bytes == 2) hipLaunchKernelGGL(strided_copy_nd_kernel<2>, gr, b, 0, st, dst, src, n, g);
    else hipLaunchKernelGGL(strided_copy_nd_kernel<1>, gr, b, 0, st, dst, src, n, g);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_make_causal_mask(uint8_t *m, int64_t len, mi_stream s) {
    if (len < 0) return mi_set_error(MI_EINVAL, "mi_make_causal_mask: negative length");
    if (len == 0) return MI_OK;
    if (!m) return mi_set_error(MI_EINVAL, "mi_make_causal_mask: null pointer");
    hipLaunchKernelGGL(causal_mask_kernel, dim3(grid_for(len * len)), dim3(256), 0, (hipStream_t)s, m, len);
    MI_LAUNCH_CHECK();
    return MI_OK;
}
