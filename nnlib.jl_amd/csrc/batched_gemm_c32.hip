// batched_mul for ComplexF32 arrays: C[:,:,b] = alpha * op(A[:,:,b]) * op(B[:,:,b]) + beta * C[:,:,b]
// with every operand addressed by element strides (row, column, batch) and an optional conjugation.
// That covers what the reference sends to cgemm ('N', 'T' and, for BatchedAdjoint{<:Complex}, 'C':
// src/batched/batchedmul.jl:261-296, src/gemm.jl:31) and the strided layouts it hands to
// batched_mul_generic! (src/batched/batchedmul.jl:306-325: PermutedDimsArray inputs and outputs, an
// adjoint of a non-unit-stride parent) in one kernel, without copies.
//
// 64 x 64 output tile per 256-thread workgroup, 4 x 4 complex results per thread, k in steps of 16
// through LDS; scalar complex multiply-adds in Float32 (4 real FMAs each).
#include "common.h"

namespace {

struct CGemmArgs {
    const float2 *A, *B;
    float2 *C;
    int64_t m, n, k;
    int64_t a_rs, a_cs, a_bs, b_rs, b_cs, b_bs, c_rs, c_cs, c_bs;   // element strides of op(A) (m x k), op(B) (k x n), C
    int32_t conj_a, conj_b;
    float alpha_re, alpha_im, beta_re, beta_im;
};

__device__ inline float2 cmul(float2 a, float2 b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }
__device__ inline void cfma(float2 a, float2 b, float2 &c) {
    c.x = fmaf(a.x, b.x, c.x);
    c.x = fmaf(-a.y, b.y, c.x);
    c.y = fmaf(a.x, b.y, c.y);
    c.y = fmaf(a.y, b.x, c.y);
}

__global__ __launch_bounds__(256) void gemm_c32_kernel(CGemmArgs g) {
    constexpr int TM = 64, TK = 16;
    __shared__ float2 As[TK][TM + 1], Bs[TK][TM + 1];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int64_t m0 = (int64_t)blockIdx.x * TM, n0 = (int64_t)blockIdx.y * TM, bz = blockIdx.z;
    const float2 *A = g.A + bz * g.a_bs, *B = g.B + bz * g.b_bs;
    float2 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = make_float2(0.0f, 0.0f);
    // consecutive threads walk the unit-stride direction of each operand where there is one
    const bool a_rows_fast = g.a_rs <= g.a_cs, b_rows_fast = g.b_cs <= g.b_rs;   // for B the "row" of the tile is n
    for (int64_t k0 = 0; k0 < g.k; k0 += TK) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int e = tid + 256 * u;
            const int i = a_rows_fast ? e % TM : e / TK, kk = a_rows_fast ? e / TM : e % TK;
            float2 v = make_float2(0.0f, 0.0f);
            if (m0 + i < g.m && k0 + kk < g.k) v = A[(m0 + i) * g.a_rs + (k0 + kk) * g.a_cs];
            if (g.conj_a) v.y = -v.y;
            As[kk][i] = v;
            const int j = b_rows_fast ? e % TM : e / TK, kb = b_rows_fast ? e / TM : e % TK;
            float2 w = make_float2(0.0f, 0.0f);
            if (n0 + j < g.n && k0 + kb < g.k) w = B[(k0 + kb) * g.b_rs + (n0 + j) * g.b_cs];
            if (g.conj_b) w.y = -w.y;
            Bs[kb][j] = w;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; kk++) {
            float2 a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = As[kk][tx + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = Bs[kk][ty + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) cfma(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    float2 *C = g.C + bz * g.c_bs;
    const float2 alpha = make_float2(g.alpha_re, g.alpha_im), beta = make_float2(g.beta_re, g.beta_im);
    const bool have_beta = beta.x != 0.0f || beta.y != 0.0f;   // beta = 0 overwrites (a NaN in C does not spread), as BLAS does
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t mi = m0 + tx + 16 * i, nj = n0 + ty + 16 * j;
            if (mi < g.m && nj < g.n) {
                float2 *c = C + mi * g.c_rs + nj * g.c_cs;
                float2 r = cmul(alpha, acc[i][j]);
                if (have_beta) {
                    const float2 old = cmul(beta, *c);
                    r.x += old.x;
                    r.y += old.y;
                }
                *c = r;
            }
        }
}

}  // namespace

MI_API int32_t mi_batched_mul_c32(int64_t m, int64_t n, int64_t k, float alpha_re, float alpha_im, const void *A, int64_t a_rs,
                                  int64_t a_cs, int64_t a_bs, int32_t conj_a, const void *B, int64_t b_rs, int64_t b_cs,
                                  int64_t b_bs, int32_t conj_b, float beta_re, float beta_im, void *C, int64_t c_rs,
                                  int64_t c_cs, int64_t c_bs, int64_t batch, mi_stream s) {
    if (m < 0 || n < 0 || k < 0 || batch < 0) return mi_set_error(MI_ESHAPE, "mi_batched_mul_c32: negative size");
    if (m == 0 || n == 0 || batch == 0) return MI_OK;
    if (!C || (k > 0 && (!A || !B))) return mi_set_error(MI_EINVAL, "mi_batched_mul_c32: null pointer");
    if ((((uintptr_t)A) | ((uintptr_t)B) | ((uintptr_t)C)) & 7) return mi_set_error(MI_EINVAL, "mi_batched_mul_c32: arrays must be 8-byte aligned");
    if ((n + 63) / 64 > 65535) return mi_set_error(MI_ESHAPE, "mi_batched_mul_c32: n is too large for one launch");
    hipStream_t st = (hipStream_t)s;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {   // gridDim.z is limited to 65535: issue the batch in slabs
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        CGemmArgs g = {(const float2 *)A + b0 * a_bs, (const float2 *)B + b0 * b_bs, (float2 *)C + b0 * c_bs, m, n, k,
                       a_rs, a_cs, a_bs, b_rs, b_cs, b_bs, c_rs, c_cs, c_bs, conj_a, conj_b, alpha_re, alpha_im, beta_re, beta_im};
        hipLaunchKernelGGL(gemm_c32_kernel, dim3((unsigned)((m + 63) / 64), (unsigned)((n + 63) / 64), (unsigned)nb), dim3(256), 0, st, g);
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}
