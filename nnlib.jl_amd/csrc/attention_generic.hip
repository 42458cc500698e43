// Generic attention forward: any head dim, any dtype, strided bias/mask, scalar FMA.
// One workgroup per (query row, head, batch).  It is the fallback for shapes the MFMA
// kernels do not take and the on-device cross-check for them.
//
// Follows the reference's order of operations (src/attention.jl:112-127):
//   s_j = sum_d k[d,h,j,b] * (q[d,h,i,b] / sqrt(D))  -> + bias -> mask -> softmax_j -> sum_j a_j v[:,h,j,b]
#include "common.h"
#include "attention_params.h"

__device__ static inline float generic_term(float s, float m) {
    if (m == MI_POS_INF) return s == MI_POS_INF ? 1.0f : 0.0f;
    return expf(s - m);
}

__device__ static inline float generic_block_reduce(float v, float *red, bool is_max) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    v = is_max ? mi_wave_max(v) : mi_wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < nw; w++) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

template <typename T, typename TW>
__global__ __launch_bounds__(256) void attention_generic_kernel(AttnParams p) {
    extern __shared__ float smem[];
    float *qs = smem;         // D floats: q / sqrt(D)
    float *pj = smem + p.D;   // 256 floats: weights of the current kv chunk
    __shared__ float red[8];

    const int64_t i = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    typedef typename T::type t;
    const t *q = (const t *)p.q + p.D * h + p.E * (i + p.Lq * b);
    const t *k = (const t *)p.k + p.D * h + p.E * (p.Lkv * b);
    const t *bias = (const t *)p.bias;
    const int64_t boff = i * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3];
    const int64_t moff = i * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3];

    const float sq = sqrtf((float)p.D);
    for (int d = tid; d < p.D; d += blockDim.x) qs[d] = T::to_f32(q[d]) / sq;
    __syncthreads();

    auto score = [&](int64_t j) -> float {
        const t *kj = k + p.E * j;
        float s = 0.0f;
        for (int d = 0; d < p.D; d++) s = fmaf(T::to_f32(kj[d]), qs[d], s);
        if (bias) s += T::to_f32(bias[boff + j * p.bias_strides[0]]);
        if (p.mask && !p.mask[moff + j * p.mask_strides[0]]) s = MI_NEG_INF;
        if (p.causal && j > i) s = MI_NEG_INF;
        return s;
    };

    float m = MI_NEG_INF;
    for (int64_t j = tid; j < p.Lkv; j += blockDim.x) m = fmaxf(m, score(j));
    m = generic_block_reduce(m, red, true);
    float l = 0.0f;
    for (int64_t j = tid; j < p.Lkv; j += blockDim.x) l += generic_term(score(j), m);
    l = generic_block_reduce(l, red, false);

    TW *w = p.weights ? (TW *)p.weights + p.Lkv * (i + p.Lq * (h + p.H * b)) : nullptr;
    const t *v = p.out ? (const t *)p.v + p.Dv * h + p.Ev * (p.Lkv * b) : nullptr;
    // each thread owns output features tid, tid+256, ... (at most 4: Dv <= 1024 checked on the host)
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t j0 = 0; j0 < p.Lkv; j0 += blockDim.x) {
        int64_t j = j0 + tid;
        float a = 0.0f;
        if (j < p.Lkv) {
            a = generic_term(score(j), m) / l;
            if (p.drop_thresh)   // fdrop = dropout: src/attention.jl:126, src/dropout.jl:38-53
                a = mi_dropout_keep(p.drop_key, (uint64_t)(j + p.Lkv * (i + p.Lq * (h + p.H * b))), p.drop_thresh) ? a * p.drop_scale : 0.0f;
            if (w) w[j] = (TW)a;
        }
        if (v) {
            __syncthreads();
            pj[tid] = a;
            __syncthreads();
            int64_t nj = p.Lkv - j0 < blockDim.x ? p.Lkv - j0 : blockDim.x;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                int d = tid + u * 256;
                if (d < p.Dv)
                    for (int64_t jj = 0; jj < nj; jj++) acc[u] = fmaf(pj[jj], T::to_f32(v[d + p.Ev * (j0 + jj)]), acc[u]);
            }
        }
    }
    if (p.out) {
        t *o = (t *)p.out + p.Dv * h + p.Ev * (i + p.Lq * b);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int d = tid + u * 256;
            if (d < p.Dv) o[d] = T::from_f32(acc[u]);
        }
    }
}

template <typename T, typename TW>
static int32_t launch_generic_t(const AttnParams &p, hipStream_t st) {
    dim3 grid((unsigned)p.Lq, (unsigned)p.H, (unsigned)p.B);
    size_t smem = sizeof(float) * (size_t)(p.D + 256);
    hipLaunchKernelGGL((attention_generic_kernel<T, TW>), grid, dim3(256), smem, st, p);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

int32_t launch_attention_generic(const AttnParams &p, hipStream_t st) {
    if (p.Dv > 1024 || p.D > 8192)
        return mi_set_error(MI_ESHAPE, "generic attention kernel supports head dims up to 8192 (qk) / 1024 (v); got %lld / %lld",
                            (long long)p.D, (long long)p.Dv);
    if (p.H > 65535 || p.B > 65535)
        return mi_set_error(MI_ESHAPE, "generic attention kernel supports at most 65535 heads and 65535 batches");
    const bool w32 = p.weights_dtype == MI_F32;
    switch (p.dtype) {
    case MI_F32: return launch_generic_t<F32, float>(p, st);
    case MI_F16: return w32 ? launch_generic_t<F16, float>(p, st) : launch_generic_t<F16, _Float16>(p, st);
    default: return w32 ? launch_generic_t<BF16, float>(p, st) : launch_generic_t<BF16, __bf16>(p, st);
    }
}
