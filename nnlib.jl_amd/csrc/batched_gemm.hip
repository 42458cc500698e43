// Strided batched GEMM on MFMA: C[:,:,b] = alpha*op(A[:,:,b])*op(B[:,:,b]) + beta*C[:,:,b].
// Device replacement for the reference's batched_gemm! (src/gemm.jl:89-188), reached
// through the _batched_gemm! hook (src/batched/batchedmul.jl:298).  Column-major.
//
// Workgroup = 4 wavefronts, output tile 64 (m) x 64 (n), each wavefront one 32x32 block.
// The MFMA is issued on the transposed problem (rows = n, columns = m) so that a lane's
// accumulator column is an m index: the 32 lanes of a half-wave then store 32 consecutive
// elements of a C column.
#include "common.h"

// tiled 16-bit fast path (batched_gemm16.hip)
bool batched_gemm16_supports(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, const void *A, int64_t lda,
                             int64_t sA, const void *B, int64_t ldb, int64_t sB);
int32_t launch_batched_gemm16(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                              int64_t lda, int64_t sA, const void *B, int64_t ldb, int64_t sB, float beta, void *C, int64_t ldc,
                              int64_t sC, int64_t batch, hipStream_t st);

// tiled Float32 fast path (batched_gemm32.hip)
bool batched_gemm32_supports(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, const void *A, int64_t lda,
                             int64_t sA, const void *B, int64_t ldb, int64_t sB);
int32_t launch_batched_gemm32(int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha, const void *A, int64_t lda,
                              int64_t sA, const void *B, int64_t ldb, int64_t sB, float beta, void *C, int64_t ldc, int64_t sC,
                              int64_t batch, hipStream_t st);

namespace {

constexpr int TM = 64, TN = 64;

template <typename T> struct GemmTraits;
template <> struct GemmTraits<F32> {
    static constexpr int KC = 16;  // k elements per LDS stage
    static constexpr int LD = 17;  // LDS row stride (elements), odd => conflict-free b32 reads
};
template <> struct GemmTraits<F16> {
    static constexpr int KC = 32;
    static constexpr int LD = 40;  // 80-byte rows: 16-byte aligned, conflict-free b128 reads
};
template <> struct GemmTraits<BF16> {
    static constexpr int KC = 32;
    static constexpr int LD = 40;
};

struct GemmArgs {
    const void *A, *B;
    void *C;
    int64_t m, n, k, lda, ldb, ldc, sA, sB, sC;
    float alpha, beta;
    int transA, transB;
};

// stage a (rows x KC) slab of op(X) into LDS as dst[row][kk]; zero beyond the matrix edge
template <typename T, int ROWS>
__device__ inline void stage(typename T::type *dst, const typename T::type *X, int64_t ld, int trans, int64_t row0,
                             int64_t nrows, int64_t k0, int64_t k) {
    constexpr int KC = GemmTraits<T>::KC, LD = GemmTraits<T>::LD;
    const int tid = threadIdx.x;
    typedef typename T::type t;
    if (!trans) {
        // op(X)[r, kk] = X[r + kk*ld]: consecutive threads walk r (contiguous)
        const int r = tid % ROWS;
#pragma unroll
        for (int u = 0; u < KC * ROWS / 256; u++) {
            const int kk = tid / ROWS + u * (256 / ROWS);
            t val = (t)0;
            if (row0 + r < nrows && k0 + kk < k) val = X[(row0 + r) + (k0 + kk) * ld];
            dst[r * LD + kk] = val;
        }
    } else {
        // op(X)[r, kk] = X[kk + r*ld]: consecutive threads walk kk (contiguous)
        const int kk = tid % KC;
#pragma unroll
        for (int u = 0; u < KC * ROWS / 256; u++) {
            const int r = tid / KC + u * (256 / KC);
            t val = (t)0;
            if (row0 + r < nrows && k0 + kk < k) val = X[(k0 + kk) + (row0 + r) * ld];
            dst[r * LD + kk] = val;
        }
    }
}

template <typename T>
__device__ inline floatx16_t mma_stage(const typename T::type *As, const typename T::type *Bs, floatx16_t acc,
                                       int wm, int wn);

template <>
__device__ inline floatx16_t mma_stage<F32>(const float *As, const float *Bs, floatx16_t acc, int wm, int wn) {
    constexpr int KC = GemmTraits<F32>::KC, LD = GemmTraits<F32>::LD;
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int t = 0; t < KC / 2; t++) {
        float bn = Bs[(wn * 32 + r) * LD + 2 * t + hh];  // MFMA row operand: n index
        float am = As[(wm * 32 + r) * LD + 2 * t + hh];  // MFMA column operand: m index
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bn, am, acc, 0, 0, 0);
    }
    return acc;
}

template <typename T>
__device__ inline floatx16_t mma_stage16(const typename T::type *As, const typename T::type *Bs, floatx16_t acc,
                                         int wm, int wn) {
    constexpr int KC = GemmTraits<T>::KC, LD = GemmTraits<T>::LD;
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int t = 0; t < KC / 16; t++) {
        typename T::vec8 bn = *(const typename T::vec8 *)(Bs + (wn * 32 + r) * LD + 16 * t + 8 * hh);
        typename T::vec8 am = *(const typename T::vec8 *)(As + (wm * 32 + r) * LD + 16 * t + 8 * hh);
        acc = T::mfma32(bn, am, acc);
    }
    return acc;
}
template <>
__device__ inline floatx16_t mma_stage<F16>(const _Float16 *As, const _Float16 *Bs, floatx16_t acc, int wm, int wn) {
    return mma_stage16<F16>(As, Bs, acc, wm, wn);
}
template <>
__device__ inline floatx16_t mma_stage<BF16>(const __bf16 *As, const __bf16 *Bs, floatx16_t acc, int wm, int wn) {
    return mma_stage16<BF16>(As, Bs, acc, wm, wn);
}

template <typename T>
__global__ __launch_bounds__(256) void batched_gemm_kernel(GemmArgs g) {
    constexpr int KC = GemmTraits<T>::KC, LD = GemmTraits<T>::LD;
    typedef typename T::type t;
    __shared__ __attribute__((aligned(16))) t As[TM * LD];
    __shared__ __attribute__((aligned(16))) t Bs[TN * LD];

    const int64_t bz = blockIdx.z;
    const t *A = (const t *)g.A + bz * g.sA;
    const t *B = (const t *)g.B + bz * g.sB;
    t *C = (t *)g.C + bz * g.sC;
    const int64_t m0 = (int64_t)blockIdx.x * TM, n0 = (int64_t)blockIdx.y * TN;
    const int wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;

    floatx16_t acc = {0};
    for (int64_t k0 = 0; k0 < g.k; k0 += KC) {
        __syncthreads();
        // op(A) is m x k: rows = m.  op(B) is k x n: staged by its columns, i.e. rows of op(B)^T = n.
        stage<T, TM>(As, A, g.lda, g.transA, m0, g.m, k0, g.k);
        stage<T, TN>(Bs, B, g.ldb, !g.transB, n0, g.n, k0, g.k);
        __syncthreads();
        acc = mma_stage<T>(As, Bs, acc, wm, wn);
    }
    // accumulator v of lane (r, hh): n = 8*(v/4) + 4*hh + v%4, m = r
    const int64_t mi = m0 + wm * 32 + r;
    if (mi < g.m) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int64_t nj = n0 + wn * 32 + 8 * (v / 4) + 4 * hh + (v % 4);
            if (nj < g.n) {
                t *c = C + mi + nj * g.ldc;
                float val = g.alpha * acc[v];
                if (g.beta != 0.0f) val += g.beta * T::to_f32(*c);
                *c = T::from_f32(val);
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void scale_c_kernel(typename T::type *C, int64_t m, int64_t n, int64_t ldc,
                                                       int64_t sC, float beta) {
    // k == 0: C = beta*C (or 0)
    typename T::type *c = C + (int64_t)blockIdx.z * sC;
    int64_t total = m * n;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t i = idx % m, j = idx / m;
        typename T::type *e = c + i + j * ldc;
        *e = beta == 0.0f ? T::from_f32(0.0f) : T::from_f32(beta * T::to_f32(*e));
    }
}

template <typename T>
int32_t launch(const GemmArgs &g, int64_t batch, hipStream_t st) {
    // gridDim.z is limited to 65535: issue the batch in slabs
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
        int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        GemmArgs a = g;
        typedef typename T::type t;
        a.A = (const t *)g.A + b0 * g.sA;
        a.B = (const t *)g.B + b0 * g.sB;
        a.C = (t *)g.C + b0 * g.sC;
        if (g.k == 0) {
            int64_t blocks = (g.m * g.n + 255) / 256;
            if (blocks > 4096) blocks = 4096;
            hipLaunchKernelGGL(scale_c_kernel<T>, dim3((unsigned)blocks, 1, (unsigned)nb), dim3(256), 0, st, (t *)a.C,
                               g.m, g.n, g.ldc, g.sC, g.beta);
        } else {
            dim3 grid((unsigned)((g.m + TM - 1) / TM), (unsigned)((g.n + TN - 1) / TN), (unsigned)nb);
            hipLaunchKernelGGL(batched_gemm_kernel<T>, grid, dim3(256), 0, st, a);
        }
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}

inline int trans_flag(char c) {
    switch (c) {
    case 'N': case 'n': return 0;
    case 'T': case 't': case 'C': case 'c': return 1;
    default: return -1;
    }
}

}  // namespace

MI_API int32_t mi_batched_gemm(int32_t dtype, char transA, char transB, int64_t m, int64_t n, int64_t k, float alpha,
                               const void *A, int64_t lda, int64_t strideA, const void *B, int64_t ldb,
                               int64_t strideB, float beta, void *C, int64_t ldc, int64_t strideC, int64_t batch,
                               mi_stream s) {
    if (!mi_dtype_ok(dtype)) return mi_set_error(MI_EDTYPE, "mi_batched_gemm: unknown dtype %d", dtype);
    const int ta = trans_flag(transA), tb = trans_flag(transB);
    if (ta < 0 || tb < 0) return mi_set_error(MI_EINVAL, "mi_batched_gemm: trans flags must be 'N', 'T' or 'C'");
    if (m < 0 || n < 0 || k < 0 || batch < 0) return mi_set_error(MI_ESHAPE, "mi_batched_gemm: negative dimension");
    if (strideA < 0 || strideB < 0 || strideC < 0) return mi_set_error(MI_ESHAPE, "mi_batched_gemm: negative batch stride");
    // BLAS leading-dimension rules (the reference passes max(1, stride(X,2)), src/gemm.jl:148-150)
    const int64_t rowsA = ta ? k : m, rowsB = tb ? n : k;
    if (lda < (rowsA > 1 ? rowsA : 1) || ldb < (rowsB > 1 ? rowsB : 1) || ldc < (m > 1 ? m : 1))
        return mi_set_error(MI_ESHAPE, "mi_batched_gemm: leading dimension too small (lda=%lld ldb=%lld ldc=%lld)",
                            (long long)lda, (long long)ldb, (long long)ldc);
    if (m == 0 || n == 0 || batch == 0) return MI_OK;
    if (!C || (k > 0 && (!A || !B))) return mi_set_error(MI_EINVAL, "mi_batched_gemm: null pointer");
    if (batch > 1 && strideC == 0) return mi_set_error(MI_ESHAPE, "mi_batched_gemm: C cannot be broadcast over the batch");
    if ((m + TM - 1) / TM > 2147483647LL || (n + TN - 1) / TN > 65535)
        return mi_set_error(MI_ESHAPE, "mi_batched_gemm: matrix too large for one launch (n tiles > 65535)");
    GemmArgs g = {A, B, C, m, n, k, lda, ldb, ldc, strideA, strideB, strideC, alpha, beta, ta, tb};
    hipStream_t st = (hipStream_t)s;
    if (batched_gemm16_supports(dtype, ta, tb, m, n, k, A, lda, strideA, B, ldb, strideB))
        return launch_batched_gemm16(dtype, ta, tb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, st);
    if (batched_gemm32_supports(dtype, ta, tb, m, n, k, A, lda, strideA, B, ldb, strideB))
        return launch_batched_gemm32(ta, tb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, st);
    if (dtype == MI_F32) return launch<F32>(g, batch, st);
    if (dtype == MI_F16) return launch<F16>(g, batch, st);
    return launch<BF16>(g, batch, st);
}
