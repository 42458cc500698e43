// Tiled strided batched GEMM for Float32 on the fp32 matrix cores (v_mfma_f32_32x32x2_f32): the fast
// path of mi_batched_gemm for operands whose rows can be moved in 16-byte pieces.  Stands where the
// reference calls sgemm per slice (src/gemm.jl:141-149, reached through _batched_gemm!,
// src/batched/batchedmul.jl:298).  Products and sums are true fp32.
//
// Workgroup = 4 wavefronts (2 x 2), output tile 128 (m) x 128 (n), 64 x 64 per wavefront as 2 x 2 MFMA
// blocks; k advances 16 per stage through double-buffered LDS tiles kept as [k][row] (row contiguous),
// so an MFMA operand (one float per lane: row = lane % 32, k = 2*step + lane / 32) is a conflict-free
// 4-byte read whatever the memory layout of the matrix.  As in the other GEMM kernels the MFMA runs on
// the transposed problem so that a half-wave stores 32 consecutive elements of a C column.
#include "common.h"

namespace {

constexpr int TM = 128, TN = 128, KC = 16;
constexpr int LDT = 128 + 4;   // floats per k-row of a tile (+4: the strided stores of k-contiguous operands spread over banks)

struct Gemm32Args {
    const float *A, *B;
    float *C;
    int64_t m, n, k, lda, ldb, ldc, sA, sB, sC;
    float alpha, beta;
};

// RM: element (row, kk) at X[row + kk*ld] (contiguous along row); else at X[kk + row*ld]
template <bool RM>
struct Operand32 {
    const float *X;
    int64_t ld, rows, k, row0;
    floatx4_t reg[2];   // 512 pieces of 16 bytes per tile, 2 per thread

    __device__ void load(int64_t k0) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = tid + 256 * u;
            const floatx4_t z = {0.f, 0.f, 0.f, 0.f};
            if (RM) {
                const int kk = c >> 5, r4 = (c & 31) * 4;     // 32 pieces per k-row
                reg[u] = (k0 + kk < k && row0 + r4 < rows) ? *(const floatx4_t *)(X + (row0 + r4) + (k0 + kk) * ld) : z;
            } else {
                const int r = c >> 2, k4 = (c & 3) * 4;       // 4 pieces per row
                reg[u] = (row0 + r < rows && k0 + k4 < k) ? *(const floatx4_t *)(X + (k0 + k4) + (row0 + r) * ld) : z;
            }
        }
    }
    __device__ void store(float *tile) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = tid + 256 * u;
            if (RM) {
                const int kk = c >> 5, r4 = (c & 31) * 4;
                *(floatx4_t *)(tile + kk * LDT + r4) = reg[u];
            } else {
                const int r = c >> 2, k4 = (c & 3) * 4;
#pragma unroll
                for (int e = 0; e < 4; e++) tile[(k4 + e) * LDT + r] = reg[u][e];
            }
        }
    }
};

template <bool A_RM, bool B_RM>
__global__ __launch_bounds__(256, 2) void gemm32_kernel(Gemm32Args g) {
    __shared__ __attribute__((aligned(16))) float As[2][KC * LDT];
    __shared__ __attribute__((aligned(16))) float Bs[2][KC * LDT];
    const int64_t bz = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
    const int r = lane & 31, hh = lane >> 5;

    Operand32<A_RM> a;
    Operand32<B_RM> b;
    a.X = g.A + bz * g.sA;
    a.ld = g.lda;
    a.rows = g.m;
    a.k = g.k;
    a.row0 = (int64_t)blockIdx.x * TM;
    b.X = g.B + bz * g.sB;
    b.ld = g.ldb;
    b.rows = g.n;
    b.k = g.k;
    b.row0 = (int64_t)blockIdx.y * TN;

    floatx16_t acc[2][2];   // [n block][m block]
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = (floatx16_t){0};

    const int nk = (int)((g.k + KC - 1) / KC);
    a.load(0);
    b.load(0);
    a.store(As[0]);
    b.store(Bs[0]);
    __syncthreads();
    for (int it = 0; it < nk; it++) {
        const int buf = it & 1;
        if (it + 1 < nk) {
            a.load((int64_t)(it + 1) * KC);
            b.load((int64_t)(it + 1) * KC);
        }
        const float *at = As[buf] + 64 * wm + r, *bt = Bs[buf] + 64 * wn + r;
#pragma unroll
        for (int ks = 0; ks < KC / 2; ks++) {
            float av[2], bv[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                av[j] = at[(2 * ks + hh) * LDT + 32 * j];
                bv[j] = bt[(2 * ks + hh) * LDT + 32 * j];
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[i], av[j], acc[i][j], 0, 0, 0);
        }
        if (it + 1 < nk) {
            a.store(As[buf ^ 1]);
            b.store(Bs[buf ^ 1]);
        }
        __syncthreads();
    }

    // accumulator register v of lane (r, hh) of block (i, j): n = 32i + 8*(v/4) + 4*hh + v%4, m = 32j + r
    float *C = g.C + bz * g.sC;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int64_t mi = a.row0 + 64 * wm + 32 * j + r;
        if (mi >= g.m) continue;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t nj = b.row0 + 64 * wn + 32 * i + 8 * (v / 4) + 4 * hh + (v % 4);
                if (nj < g.n) {
                    float *c = C + mi + nj * g.ldc;
                    float val = g.alpha * acc[i][j][v];
                    if (g.beta != 0.0f) val += g.beta * *c;
                    *c = val;
                }
            }
    }
}

}  // namespace

// true when every 16-byte piece the kernel moves is aligned and wholly inside or outside its matrix
bool batched_gemm32_supports(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, const void *A, int64_t lda,
                             int64_t sA, const void *B, int64_t ldb, int64_t sB) {
    if (dtype != MI_F32) return false;
    if (k < 1 || m * n < 64 * 64) return false;   // tiny products: the small-tile kernel wastes less
    auto al = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if (!al(A) || !al(B) || (lda & 3) || (ldb & 3) || (sA & 3) || (sB & 3)) return false;
    if ((transA ? k : m) & 3) return false;
    if ((transB ? n : k) & 3) return false;
    return (n + TN - 1) / TN <= 65535;
}

int32_t launch_batched_gemm32(int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha, const void *A, int64_t lda,
                              int64_t sA, const void *B, int64_t ldb, int64_t sB, float beta, void *C, int64_t ldc, int64_t sC,
                              int64_t batch, hipStream_t st) {
    const bool a_rm = !transA, b_rm = transB != 0;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {   // gridDim.z is limited to 65535: issue the batch in slabs
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        Gemm32Args g = {(const float *)A + b0 * sA, (const float *)B + b0 * sB, (float *)C + b0 * sC,
                        m, n, k, lda, ldb, ldc, sA, sB, sC, alpha, beta};
        dim3 grid((unsigned)((m + TM - 1) / TM), (unsigned)((n + TN - 1) / TN), (unsigned)nb);
        if (a_rm && b_rm) hipLaunchKernelGGL((gemm32_kernel<true, true>), grid, dim3(256), 0, st, g);
        else if (a_rm) hipLaunchKernelGGL((gemm32_kernel<true, false>), grid, dim3(256), 0, st, g);
        else if (b_rm) hipLaunchKernelGGL((gemm32_kernel<false, true>), grid, dim3(256), 0, st, g);
        else hipLaunchKernelGGL((gemm32_kernel<false, false>), grid, dim3(256), 0, st, g);
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}
