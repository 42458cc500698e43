// Generic attention backward: any head dim up to 1024, any dtype, strided bias/mask, scalar FMA.
// It is the fallback for shapes the MFMA backward kernels do not take, the only path that accepts a
// cotangent of the returned weights or produces a bias gradient, and the on-device cross-check.
//
// The reference has no hand-written rule for attention; AD reverses src/attention.jl:86-127 through
// the rrule of batched_mul (src/batched/batchedmul.jl:96-110) and _∇softmax! (src/softmax.jl:107-110).
// With a = softmax weights, g = the factor fused dropout multiplied them by (1 without dropout: the
// forward used and returned a g), da[j,i] = g (v_j . dx_i + dweights[j,i]), delta_i = sum_j a da,
// ds = a (da - delta):
//   dv_j = sum_i a g [j,i] dx_i    dk_j = sum_i ds[j,i] q_i / sqrt(D)      dq_i = sum_j ds[j,i] k_j / sqrt(D)
//   dbias += ds (summed over the dims the bias broadcasts along)
//
// Two kernels: one workgroup per query row (statistics m, l, delta into the workspace, and dq), then
// one workgroup per key row (dk, dv, dbias) that recomputes the weights from the statistics.
#include "common.h"
#include "attention_params.h"

namespace {

__device__ inline float term(float s, float m) {   // src/softmax.jl:72-75
    if (m == MI_POS_INF) return s == MI_POS_INF ? 1.0f : 0.0f;
    return expf(s - m);
}

__device__ inline float block_reduce(float v, float *red, bool is_max) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v = is_max ? mi_wave_max(v) : mi_wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < 4; w++) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// stats: [B][H][Lq][3] floats (m, l, delta)
template <typename T>
__global__ __launch_bounds__(256) void bwd_generic_query_kernel(AttnBwdParams bp) {
    const AttnParams &p = bp.p;
    extern __shared__ float smem[];
    float *qs = smem;              // D: q / sqrt(D)
    float *dxs = qs + p.D;         // Dv: dx_i
    float *dsj = dxs + p.Dv;       // 256: ds of the current key chunk
    __shared__ float red[4];
    typedef typename T::type t;
    const int64_t i = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const t *q = (const t *)p.q + p.D * h + p.E * (i + p.Lq * b);
    const t *k = (const t *)p.k + p.D * h + p.E * (p.Lkv * b);
    const t *v = (const t *)p.v + p.Dv * h + p.Ev * (p.Lkv * b);
    const t *dx = (const t *)bp.dout + p.Dv * h + p.Ev * (i + p.Lq * b);
    const t *bias = (const t *)p.bias;
    const t *dw = bp.dweights ? (const t *)bp.dweights + p.Lkv * (i + p.Lq * (h + p.H * b)) : nullptr;
    const int64_t boff = i * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3];
    const int64_t moff = i * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3];
    const float sq = sqrtf((float)p.D);
    for (int d = tid; d < p.D; d += 256) qs[d] = T::to_f32(q[d]) / sq;
    for (int d = tid; d < p.Dv; d += 256) dxs[d] = T::to_f32(dx[d]);
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
    auto dalpha = [&](int64_t j) -> float {
        const float g = attention_drop_factor(p, j, i, h, b);
        if (g == 0.0f) return 0.0f;
        const t *vj = v + p.Ev * j;
        float s = 0.0f;
        for (int d = 0; d < p.Dv; d++) s = fmaf(T::to_f32(vj[d]), dxs[d], s);
        if (dw) s += T::to_f32(dw[j]);
        return g * s;
    };

    float m = MI_NEG_INF;
    for (int64_t j = tid; j < p.Lkv; j += 256) m = fmaxf(m, score(j));
    m = block_reduce(m, red, true);
    float l = 0.0f;
    for (int64_t j = tid; j < p.Lkv; j += 256) l += term(score(j), m);
    l = block_reduce(l, red, false);
    float delta = 0.0f;
    for (int64_t j = tid; j < p.Lkv; j += 256) {
        const float a = term(score(j), m) / l;
        if (a != 0.0f) delta += a * dalpha(j);   // dropped keys contribute nothing (their da may be anything)
    }
    delta = block_reduce(delta, red, false);
    if (tid == 0) {
        float *st = bp.stats + 3 * (i + p.Lq * (h + p.H * b));
        st[0] = m;
        st[1] = l;
        st[2] = delta;
    }
    if (!bp.dq) return;
    // dq_i[d] = sum_j ds_j k_j[d] / sqrt(D); each thread owns features tid, tid+256, ...
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t j0 = 0; j0 < p.Lkv; j0 += 256) {
        const int64_t j = j0 + tid;
        float ds = 0.0f;
        if (j < p.Lkv) {
            const float a = term(score(j), m) / l;
            ds = a != 0.0f ? a * (dalpha(j) - delta) : (a != a ? a : 0.0f);
        }
        __syncthreads();
        dsj[tid] = ds;
        __syncthreads();
        const int64_t nj = p.Lkv - j0 < 256 ? p.Lkv - j0 : 256;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int d = tid + u * 256;
            if (d < p.D)
                for (int64_t jj = 0; jj < nj; jj++) acc[u] = fmaf(dsj[jj], T::to_f32(k[d + p.E * (j0 + jj)]), acc[u]);
        }
    }
    t *dq = (t *)bp.dq + p.D * h + p.E * (i + p.Lq * b);
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int d = tid + u * 256;
        if (d < p.D) dq[d] = T::from_f32(acc[u] / sq);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void bwd_generic_key_kernel(AttnBwdParams bp) {
    const AttnParams &p = bp.p;
    extern __shared__ float smem[];
    float *ks = smem;              // D: k_j
    float *vs = ks + p.D;          // Dv: v_j
    float *ai = vs + p.Dv;         // 256: weights of the current query chunk
    float *dsi = ai + 256;         // 256: ds of the current query chunk
    typedef typename T::type t;
    const int64_t j = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const t *q = (const t *)p.q + p.D * h + p.E * (p.Lq * b);
    const t *k = (const t *)p.k + p.D * h + p.E * (j + p.Lkv * b);
    const t *v = (const t *)p.v + p.Dv * h + p.Ev * (j + p.Lkv * b);
    const t *dx = (const t *)bp.dout + p.Dv * h + p.Ev * (p.Lq * b);
    const t *bias = (const t *)p.bias;
    const float *stats = bp.stats + 3 * p.Lq * (h + p.H * b);
    const float sq = sqrtf((float)p.D);
    for (int d = tid; d < p.D; d += 256) ks[d] = T::to_f32(k[d]);
    for (int d = tid; d < p.Dv; d += 256) vs[d] = T::to_f32(v[d]);
    __syncthreads();

    float acck[4] = {0.0f, 0.0f, 0.0f, 0.0f}, accv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t i0 = 0; i0 < p.Lq; i0 += 256) {
        const int64_t i = i0 + tid;
        float a = 0.0f, ds = 0.0f;
        if (i < p.Lq) {
            const t *qi = q + p.E * i;
            float s = 0.0f;
            for (int d = 0; d < p.D; d++) s = fmaf(ks[d], T::to_f32(qi[d]) / sq, s);
            if (bias) s += T::to_f32(bias[j * p.bias_strides[0] + i * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3]]);
            if (p.mask && !p.mask[j * p.mask_strides[0] + i * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3]])
                s = MI_NEG_INF;
            if (p.causal && j > i) s = MI_NEG_INF;
            a = term(s, stats[3 * i]) / stats[3 * i + 1];
            const float g = attention_drop_factor(p, j, i, h, b);
            if (a != 0.0f) {
                float da = 0.0f;
                if (g != 0.0f) {
                    const t *dxi = dx + p.Ev * i;
                    for (int d = 0; d < p.Dv; d++) da = fmaf(vs[d], T::to_f32(dxi[d]), da);
                    if (bp.dweights) da += T::to_f32(((const t *)bp.dweights)[j + p.Lkv * (i + p.Lq * (h + p.H * b))]);
                }
                ds = a * (g * da - stats[3 * i + 2]);
            } else if (a != a) {
                ds = a;
            }
            a *= g;   // the value product used the weights after dropout
            if (bp.dbias && ds != 0.0f)
                atomicAdd(bp.dbias + j * p.bias_strides[0] + i * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3], ds);
        }
        __syncthreads();
        ai[tid] = a;
        dsi[tid] = ds;
        __syncthreads();
        const int64_t ni = p.Lq - i0 < 256 ? p.Lq - i0 : 256;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int d = tid + u * 256;
            if (d < p.D)
                for (int64_t ii = 0; ii < ni; ii++) acck[u] = fmaf(dsi[ii], T::to_f32(q[d + p.E * (i0 + ii)]), acck[u]);
            if (d < p.Dv)
                for (int64_t ii = 0; ii < ni; ii++) accv[u] = fmaf(ai[ii], T::to_f32(dx[d + p.Ev * (i0 + ii)]), accv[u]);
        }
    }
    t *dk = bp.dk ? (t *)bp.dk + p.D * h + p.E * (j + p.Lkv * b) : nullptr;
    t *dv = bp.dv ? (t *)bp.dv + p.Dv * h + p.Ev * (j + p.Lkv * b) : nullptr;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int d = tid + u * 256;
        if (dk && d < p.D) dk[d] = T::from_f32(acck[u] / sq);
        if (dv && d < p.Dv) dv[d] = T::from_f32(accv[u]);
    }
}

template <typename T>
int32_t launch_t(const AttnBwdParams &bp, hipStream_t st) {
    const AttnParams &p = bp.p;
    hipLaunchKernelGGL(bwd_generic_query_kernel<T>, dim3((unsigned)p.Lq, (unsigned)p.H, (unsigned)p.B), dim3(256),
                       sizeof(float) * (size_t)(p.D + p.Dv + 256), st, bp);
    MI_LAUNCH_CHECK();
    if (bp.dk || bp.dv || bp.dbias) {
        hipLaunchKernelGGL(bwd_generic_key_kernel<T>, dim3((unsigned)p.Lkv, (unsigned)p.H, (unsigned)p.B), dim3(256),
                           sizeof(float) * (size_t)(p.D + p.Dv + 512), st, bp);
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}

}  // namespace

size_t attention_bwd_generic_workspace(const AttnParams &p) { return sizeof(float) * 3 * (size_t)(p.Lq * p.H * p.B); }

int32_t launch_attention_bwd_generic(const AttnBwdParams &bp, hipStream_t st) {
    const AttnParams &p = bp.p;
    if (p.D > 1024 || p.Dv > 1024)
        return mi_set_error(MI_ESHAPE, "generic attention backward supports head dims up to 1024; got %lld / %lld", (long long)p.D,
                            (long long)p.Dv);
    if (p.H > 65535 || p.B > 65535)
        return mi_set_error(MI_ESHAPE, "generic attention backward supports at most 65535 heads and 65535 batches");
    switch (p.dtype) {
    case MI_F32: return launch_t<F32>(bp, st);
    case MI_F16: return launch_t<F16>(bp, st);
    default: return launch_t<BF16>(bp, st);
    }
}
