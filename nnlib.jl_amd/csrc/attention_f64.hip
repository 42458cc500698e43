// Attention forward for Float64 arrays (the element type of the reference's own golden vectors,
// test/attention.jl:17-34): every product, the softmax and all sums in double precision.
//
// One workgroup per (query row, head, batch), the reference's order of operations (src/attention.jl:112-127):
//   s_j = sum_d k[d,h,j,b] * (q[d,h,i,b] / sqrt(D))  -> + bias -> mask -> softmax_j (src/softmax.jl:69-79) -> fdrop
//   -> sum_j a_j v[:,h,j,b]
// The scores of a row are computed once and kept in LDS while the row has at most SCORE_CACHE keys (three passes over
// them: maximum, sum, weights); longer rows recompute them per pass.  A plain vector kernel: the path exists for
// parity with Float64 callers (and as the double-precision cross-check of the matrix-core kernels), not for speed.
#include "common.h"
#include "attention_params.h"

namespace {

constexpr int SCORE_CACHE = 4096;   // doubles: 32 KiB of LDS
constexpr double NEG_INF64 = -__builtin_huge_val();
constexpr double POS_INF64 = __builtin_huge_val();

__device__ inline double block_reduce64(double v, double *red, bool is_max) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const double o = __shfl_xor(v, off, 64);
        v = is_max ? (o > v ? o : v) : v + o;
    }
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    double r = red[0];
    for (int w = 1; w < 4; w++) r = is_max ? (red[w] > r ? red[w] : r) : r + red[w];
    return r;
}

__device__ inline double term64(double s, double m) {
    if (m == POS_INF64) return s == POS_INF64 ? 1.0 : 0.0;   // src/softmax.jl:73-75
    return exp(s - m);
}

__global__ __launch_bounds__(256) void attention_f64_kernel(AttnParams p, int cached) {
    extern __shared__ double smem64[];
    double *qs = smem64;                   // D: q / sqrt(D)
    double *pj = smem64 + p.D;             // 256: weights of the current chunk of keys
    double *sc = pj + 256;                 // cached scores of the row (when they fit)
    __shared__ double red[4];

    const int64_t i = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const double *q = (const double *)p.q + p.D * h + p.E * (i + p.Lq * b);
    const double *k = (const double *)p.k + p.D * h + p.E * (p.Lkv * b);
    const double *bias = (const double *)p.bias;
    const int64_t boff = i * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3];
    const int64_t moff = i * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3];

    const double sq = sqrt((double)p.D);
    for (int d = tid; d < p.D; d += 256) qs[d] = q[d] / sq;
    __syncthreads();

    auto score = [&](int64_t j) -> double {
        const double *kj = k + p.E * j;
        double s = 0.0;
        for (int d = 0; d < p.D; d++) s = fma(kj[d], qs[d], s);
        if (bias) s += bias[boff + j * p.bias_strides[0]];
        if (p.mask && !p.mask[moff + j * p.mask_strides[0]]) s = NEG_INF64;
        if (p.causal && j > i) s = NEG_INF64;
        return s;
    };
    if (cached) {
        for (int64_t j = tid; j < p.Lkv; j += 256) sc[j] = score(j);
        __syncthreads();
    }
    auto get = [&](int64_t j) -> double { return cached ? sc[j] : score(j); };

    double m = NEG_INF64;
    for (int64_t j = tid; j < p.Lkv; j += 256) {
        const double s = get(j);
        m = s > m ? s : m;
    }
    m = block_reduce64(m, red, true);
    double l = 0.0;
    for (int64_t j = tid; j < p.Lkv; j += 256) l += term64(get(j), m);
    l = block_reduce64(l, red, false);

    double *w = p.weights ? (double *)p.weights + p.Lkv * (i + p.Lq * (h + p.H * b)) : nullptr;
    const double *v = p.out ? (const double *)p.v + p.Dv * h + p.Ev * (p.Lkv * b) : nullptr;
    // each thread owns output features tid, tid + 256, ... (at most 4: Dv <= 1024 checked on the host)
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    for (int64_t j0 = 0; j0 < p.Lkv; j0 += 256) {
        const int64_t j = j0 + tid;
        double a = 0.0;
        if (j < p.Lkv) {
            a = term64(get(j), m) / l;
            if (p.drop_thresh)   // fdrop = dropout: src/attention.jl:126, src/dropout.jl:38-53
                a = mi_dropout_keep(p.drop_key, (uint64_t)(j + p.Lkv * (i + p.Lq * (h + p.H * b))), p.drop_thresh)
                        ? a * (double)p.drop_scale : 0.0;
            if (w) w[j] = a;
        }
        if (v) {
            __syncthreads();
            pj[tid] = a;
            __syncthreads();
            const int64_t nj = p.Lkv - j0 < 256 ? p.Lkv - j0 : 256;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int d = tid + u * 256;
                if (d < p.Dv)
                    for (int64_t jj = 0; jj < nj; jj++) acc[u] = fma(pj[jj], v[d + p.Ev * (j0 + jj)], acc[u]);
            }
        }
    }
    if (p.out) {
        double *o = (double *)p.out + p.Dv * h + p.Ev * (i + p.Lq * b);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int d = tid + u * 256;
            if (d < p.Dv) o[d] = acc[u];
        }
    }
}

}  // namespace

int32_t launch_attention_f64(const AttnParams &p, hipStream_t st) {
    if (p.Dv > 1024 || p.D > 2048)
        return mi_set_error(MI_ESHAPE, "Float64 attention kernel supports head dims up to 2048 (qk) / 1024 (v); got %lld / %lld",
                            (long long)p.D, (long long)p.Dv);
    if (p.H > 65535 || p.B > 65535)
        return mi_set_error(MI_ESHAPE, "Float64 attention kernel supports at most 65535 heads and 65535 batches");
    const int cached = p.Lkv <= SCORE_CACHE;
    const size_t smem = sizeof(double) * (size_t)(p.D + 256 + (cached ? p.Lkv : 0));
    static bool attr_set = false;   // idempotent: a race between threads is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)attention_f64_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)(sizeof(double) * (2048 + 256 + SCORE_CACHE))));
        attr_set = true;
    }
    dim3 grid((unsigned)p.Lq, (unsigned)p.H, (unsigned)p.B);
    hipLaunchKernelGGL(attention_f64_kernel, grid, dim3(256), smem, st, p, cached);
    MI_LAUNCH_CHECK();
    return MI_OK;
}
