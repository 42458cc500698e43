// batched_mul for ComplexF32 arrays: C[:,:,b] = alpha * op(A[:,:,b]) * op(B[:,:,b]) + beta * C[:,:,b]
// with every operand addressed by element strides (row, column, batch) and an optional conjugation.
// That covers what the reference sends to cgemm ('N', 'T' and, for BatchedAdjoint{<:Complex}, 'C':
// src/batched/batchedmul.jl:261-296, src/gemm.jl:31) and the strided layouts it hands to
// batched_mul_generic! (src/batched/batchedmul.jl:306-325: PermutedDimsArray inputs and outputs, an
// adjoint of a non-unit-stride parent) in one kernel, without copies.
//
// 64 x 64 output tile per 256-thread workgroup, k in steps of 16 through LDS, products on the Float32
// matrix cores (v_mfma_f32_32x32x2_f32).  A complex product is a real one of twice the size: with C, A
// and B viewed as real arrays whose rows (for B: whose k) alternate real and imaginary parts,
//   C'[2i+p, j] = sum_k  A^[2i+p, 2k] * Br[k, j] + A^[2i+p, 2k+1] * Bi[k, j],
//   A^[2i, 2k] = Ar   A^[2i, 2k+1] = -Ai   A^[2i+1, 2k] = Ai   A^[2i+1, 2k+1] = Ar,
// i.e. 8 real FLOP per complex multiply-add, the same count as the scalar form.  A^ is never stored: a
// lane picks the part it needs from the complex tile in LDS and flips its sign.
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

__global__ __launch_bounds__(256) void gemm_c32_kernel(CGemmArgs g) {
    constexpr int TM = 64, TK = 16, LD = 2 * (TM + 1);   // LD: floats per k row of a tile
    __shared__ float2 As[2][TK][TM + 1], Bs[2][TK][TM + 1];
    const int tid = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.x * TM, n0 = (int64_t)blockIdx.y * TM, bz = blockIdx.z;
    const float2 *A = g.A + bz * g.a_bs, *B = g.B + bz * g.b_bs;
    // Each wavefront owns 16 complex rows (32 real rows) x 64 columns: two 32 x 32 blocks, computed
    // transposed (first MFMA operand from B) so that the lanes of an accumulator register run along m.
    const int lane = tid & 63, wr = tid >> 6, l = lane & 31, h = lane >> 5, part = l & 1;
    const int a_word = 2 * (16 * wr + (l >> 1)) + (part != h);          // which float of the complex A element
    const uint32_t a_sign = (part == 0 && h == 1) ? 0x80000000u : 0u;   // A^[2i, 2k+1] = -Ai
    const int b_word = 2 * l + h;                                        // real part for k' even, imaginary for odd
    floatx16_t acc[2];
    acc[0] = (floatx16_t){0};
    acc[1] = (floatx16_t){0};
    // consecutive threads walk the unit-stride direction of each operand where there is one
    const bool a_rows_fast = g.a_rs <= g.a_cs, b_rows_fast = g.b_cs <= g.b_rs;   // for B the "row" of the tile is n
    // a tile inside C on a k step inside k loads without bounds tests (nearly every step of a large product)
    const bool inside = m0 + TM <= g.m && n0 + TM <= g.n;
    // The next k step waits in registers while the matrix instructions of this one run (a timing build without the
    // global loads ran 1.45x faster than the single-buffered loop: their latency was what the loop waited for), and goes
    // to the other LDS buffer half way through them.
    float2 va[4], vb[4];
    auto fetch = [&](int64_t k0) {
        const bool interior = inside && k0 + TK <= g.k;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int e = tid + 256 * u;
            const int i = a_rows_fast ? e % TM : e / TK, kk = a_rows_fast ? e / TM : e % TK;
            float2 v = make_float2(0.0f, 0.0f);
            if (interior || (m0 + i < g.m && k0 + kk < g.k)) v = A[(m0 + i) * g.a_rs + (k0 + kk) * g.a_cs];
            if (g.conj_a) v.y = -v.y;
            va[u] = v;
            const int j = b_rows_fast ? e % TM : e / TK, kb = b_rows_fast ? e / TM : e % TK;
            float2 w = make_float2(0.0f, 0.0f);
            if (interior || (n0 + j < g.n && k0 + kb < g.k)) w = B[(k0 + kb) * g.b_rs + (n0 + j) * g.b_cs];
            if (g.conj_b) w.y = -w.y;
            vb[u] = w;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int e = tid + 256 * u;
            const int i = a_rows_fast ? e % TM : e / TK, kk = a_rows_fast ? e / TM : e % TK;
            As[buf][kk][i] = va[u];
            const int j = b_rows_fast ? e % TM : e / TK, kb = b_rows_fast ? e / TM : e % TK;
            Bs[buf][kb][j] = vb[u];
        }
    };
    if (g.k > 0) {
        fetch(0);
        stash(0);
    }
    __syncthreads();
    for (int64_t k0 = 0, kt = 0; k0 < g.k; k0 += TK, kt++) {
        const int buf = (int)(kt & 1);
        const bool more = k0 + TK < g.k;
        if (more) fetch(k0 + TK);
        const float *Af = (const float *)&As[buf][0][0], *Bf = (const float *)&Bs[buf][0][0];
#pragma unroll
        for (int kk = 0; kk < TK; kk++) {
            if (kk == TK / 2 && more) stash(buf ^ 1);
            const float a = __uint_as_float(__float_as_uint(Af[kk * LD + a_word]) ^ a_sign);
            const float b0 = Bf[kk * LD + b_word], b1 = Bf[kk * LD + 64 + b_word];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(b0, a, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(b1, a, acc[1], 0, 0, 0);
        }
        __syncthreads();
    }
    // acc[jb][r]: column n0 + 32*jb + 8*(r/4) + 4*h + r%4, complex row m0 + 16*wr + l/2, real (part 0) or
    // imaginary (part 1) component; the other component sits in the neighbouring lane
    float *C = (float *)(g.C + bz * g.c_bs);
    const float other_alpha = part ? g.alpha_im : -g.alpha_im, other_beta = part ? g.beta_im : -g.beta_im;
    const bool have_beta = g.beta_re != 0.0f || g.beta_im != 0.0f;   // beta = 0 overwrites (a NaN in C does not spread), as BLAS does
    const int64_t mi = m0 + 16 * wr + (l >> 1);
#pragma unroll
    for (int jb = 0; jb < 2; jb++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float mine = acc[jb][r], other = __shfl_xor(mine, 1, 64);
            float out = fmaf(g.alpha_re, mine, other_alpha * other);
            const int64_t nj = n0 + 32 * jb + 8 * (r >> 2) + 4 * h + (r & 3);
            if (mi < g.m && nj < g.n) {
                float *c = C + 2 * (mi * g.c_rs + nj * g.c_cs);
                if (have_beta) out += fmaf(g.beta_re, c[part], other_beta * c[part ^ 1]);
                c[part] = out;
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
