// batched_mul! for the element types the 16-/32-bit kernels do not take.
//
//   mi_batched_gemm_f64      Float64, BLAS-style 'N' / 'T' operands (what the reference hands to dgemm_,
//                            src/gemm.jl:27-32, 141-149) on the fp64 matrix cores (v_mfma_f64_16x16x4_f64).
//   mi_batched_mul_generic   any mix of Float64 / Float32 / Float16 / BFloat16 / Int32 / Int64 / ComplexF32 /
//                            ComplexF64 operands with fully strided addressing and conjugation flags: what the
//                            reference gives to batched_mul_generic! (src/batched/batchedmul.jl:306-325), i.e.
//                            eltypes that differ, integers, ComplexF64, and layouts no BLAS call addresses.
//                            Arithmetic is in the element type of C, as Julia's mul! does after promotion;
//                            integer products wrap like Julia's (two's complement).
#include "common.h"
#include <type_traits>

namespace {

// ---- fp64 MFMA kernel -------------------------------------------------------------------------------------
// Workgroup = 4 wavefronts, TS x TS tile of C (64 or 128); a wavefront owns a quarter of it as (TS/32)^2 MFMA blocks
// of 16 x 16.  v_mfma_f64_16x16x4_f64: lane l supplies A[row = l % 16][k = l / 16] and B[k = l / 16][col = l % 16]; it
// receives D[row = l / 16 + 4 * v][col = l % 16] in register pair v = 0..3 (checked on the hardware with structured
// inputs).  Operand tiles sit in LDS k-major: As[k][row], Bs[k][col], rows padded so that the four k groups of a
// wavefront's read start in different banks (64-wide tiles: 8 banks apart; 128-wide: 32 apart, i.e. the two k groups of
// each half-wave cover all 64 banks exactly).  A 64-wide tile moves 16 KiB per 16 k for 64 matrix instructions, which
// at full matrix rate is more than L2 delivers (9 TB/s over the chip); the 128-wide tile halves that.
typedef __attribute__((__vector_size__(4 * sizeof(double)))) double doublex4_t;
constexpr int TK = 16;

template <int TS>
struct Tile64 {
    static constexpr int PAD = TS == 64 ? 4 : 16;
    static constexpr int LD = TS + PAD;
    static constexpr int NWV = 4;                       // wavefronts: 2 along m, 2 along n
    static constexpr int NT = 64 * NWV;
    static constexpr int PER = TS * TK / NT;            // elements per thread, operand and k step
    static constexpr int NBI = TS / 32, NBJ = TS / (8 * NWV);   // 16 x 16 blocks per wavefront along m and n
    static constexpr size_t SMEM = sizeof(double) * 2 * 2 * TK * LD;
    // Position of row / column x in the tile's k row (128-wide tiles).  An operand that is contiguous along k in memory
    // is stored by lanes that run along k first (16 k x 4 columns per instruction): with rows 16 slots apart mod 32
    // those 64 stores would land on 8 slots; flipping bits 2-3 of the column with k/2 spreads them over all 32 (two
    // stores per slot, the minimum for 512 bytes).  Reads of 16 consecutive columns of one k row stay a permutation.
    __device__ static inline int swz(int k, int x) { return TS == 64 ? x : x ^ (((k >> 1) & 3) << 2); }
};

template <bool TRANSA, bool TRANSB, int TS>
// The 128-wide tile is held to 256 registers: two workgroups per CU run 1.4x faster than one with 379 registers, and
// faster than one workgroup of eight wavefronts with 64 x 32 each.
__global__ __launch_bounds__(Tile64<TS>::NT, TS == 128 ? 2 : 1) void gemm64_kernel(int64_t m, int64_t n, int64_t k, double alpha, const double *A, int64_t lda,
                                                     int64_t strideA, const double *B, int64_t ldb, int64_t strideB, double beta,
                                                     double *C, int64_t ldc, int64_t strideC, int64_t tiles_m) {
    typedef Tile64<TS> TC;
    constexpr int LD = TC::LD, PER = TC::PER, NBI = TC::NBI, NBJ = TC::NBJ, NT = TC::NT;
    extern __shared__ __attribute__((aligned(16))) unsigned char gemm64_smem[];
    double (*As)[TK][LD] = (double (*)[TK][LD])gemm64_smem;          // [2][TK][LD]
    double (*Bs)[TK][LD] = As + 2;                                    // [2][TK][LD]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile = blockIdx.x;
    const int64_t row0 = (tile % tiles_m) * TS, col0 = (tile / tiles_m) * TS;
    const int64_t batch = blockIdx.y;
    A += batch * strideA;
    B += batch * strideB;
    C += batch * strideC;

    // Each thread moves PER elements of each operand tile per k step; the fast thread index runs along the direction
    // that is contiguous in memory.  Element u of a thread is its element 0 moved by a wavefront-uniform step (along k
    // for an operand stored with its tile rows contiguous, along the rows otherwise), so one per-lane offset serves all
    // of them and the rest of the address is scalar.
    constexpr int RSTEP = NT / TK, KSTEP = NT / TS;   // rows / k between consecutive elements of a thread
    const int ai = TRANSA ? tid / TK : tid % TS, ak = TRANSA ? tid % TK : tid / TS;   // tile row and k of element 0 (A)
    const int bj = TRANSB ? tid % TS : tid / TK, bk = TRANSB ? tid / TS : tid % TK;   // tile column and k of element 0 (B)
    const int64_t voffA = TRANSA ? ak + (row0 + ai) * lda : (row0 + ai) + ak * lda;
    const int64_t voffB = TRANSB ? (col0 + bj) + bk * ldb : bk + (col0 + bj) * ldb;
    const int64_t kstepA = TRANSA ? 1 : lda, ustepA = TRANSA ? RSTEP * lda : KSTEP * lda;
    const int64_t kstepB = TRANSB ? ldb : 1, ustepB = TRANSB ? KSTEP * ldb : RSTEP * ldb;
    double ra[PER], rb[PER];
    // interior: the tile lies inside C and the k step inside k, so no element needs a bounds test (nor the branch
    // around its load): the case nearly every step of a large product is
    const bool inside = row0 + TS <= m && col0 + TS <= n;
    auto fetch_at = [&](int64_t k0, auto interior) {
        const double *pa = A + k0 * kstepA, *pb = B + k0 * kstepB;
#pragma unroll
        for (int u = 0; u < PER; u++) {
            const bool oka = interior.value || (row0 + ai + (TRANSA ? RSTEP * u : 0) < m && k0 + ak + (TRANSA ? 0 : KSTEP * u) < k);
            ra[u] = oka ? (pa + u * ustepA)[voffA] : 0.0;
            const bool okb = interior.value || (col0 + bj + (TRANSB ? 0 : RSTEP * u) < n && k0 + bk + (TRANSB ? KSTEP * u : 0) < k);
            rb[u] = okb ? (pb + u * ustepB)[voffB] : 0.0;
        }
    };
    auto fetch = [&](int64_t k0) {
        if (inside && k0 + TK <= k) fetch_at(k0, std::true_type());
        else fetch_at(k0, std::false_type());
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int u = 0; u < PER; u++) {
            const int i = ai + (TRANSA ? RSTEP * u : 0), ka = ak + (TRANSA ? 0 : KSTEP * u);
            As[buf][ka][TC::swz(ka, i)] = ra[u];
            const int j = bj + (TRANSB ? 0 : RSTEP * u), kb = bk + (TRANSB ? KSTEP * u : 0);
            Bs[buf][kb][TC::swz(kb, j)] = rb[u];
        }
    };

    doublex4_t acc[NBI][NBJ];
#pragma unroll
    for (int i = 0; i < NBI; i++)
#pragma unroll
        for (int j = 0; j < NBJ; j++) acc[i][j] = (doublex4_t){0.0, 0.0, 0.0, 0.0};
    const int wr = (wave & 1) * (16 * NBI), wc = (wave >> 1) * (16 * NBJ);   // this wavefront's corner of the tile
    const int li = lane & 15, lk = lane >> 4;
    // swz(ks + lk, x) for the lane's reads: the flipped bits lie inside li, and k steps 0, 8 / 4, 12 share a value
    const int li_even = TC::swz(lk, li), li_odd = TC::swz(4 + lk, li);

    const int64_t nk = (k + TK - 1) / TK;
    if (nk > 0) {
        fetch(0);
        stash(0);
    }
    __syncthreads();
    for (int64_t kt = 0; kt < nk; kt++) {
        const int buf = (int)(kt & 1);
        if (kt + 1 < nk) fetch((kt + 1) * TK);
#pragma unroll
        for (int ks = 0; ks < TK; ks += 4) {
            // The next tile goes to the other LDS buffer half way through the matrix instructions, not after
            // them: the wait for the global loads and the LDS writes then sit behind queued matrix work.  Both
            // workgroups of a compute unit run in step, so at the end of the loop body they would idle the matrix pipes together.
            if (ks == TK / 2 && kt + 1 < nk) stash(buf ^ 1);
            double a[NBI], b[NBJ];
#pragma unroll
            for (int i = 0; i < NBI; i++) a[i] = As[buf][ks + lk][wr + 16 * i + ((ks & 4) ? li_odd : li_even)];
#pragma unroll
            for (int j = 0; j < NBJ; j++) b[j] = Bs[buf][ks + lk][wc + 16 * j + ((ks & 4) ? li_odd : li_even)];
#pragma unroll
            for (int i = 0; i < NBI; i++)
#pragma unroll
                for (int j = 0; j < NBJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // beta == 0 overwrites C without reading it (BLAS semantics: NaNs in C do not propagate)
#pragma unroll
    for (int i = 0; i < NBI; i++)
#pragma unroll
        for (int j = 0; j < NBJ; j++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int64_t gr = row0 + wr + 16 * i + lk + 4 * v, gc = col0 + wc + 16 * j + li;
                if (gr < m && gc < n) {
                    double *c = C + gr + gc * ldc;
                    const double x = alpha * acc[i][j][v];
                    *c = beta == 0.0 ? x : x + beta * *c;
                }
            }
}

template <bool TA, bool TB, int TS>
int32_t launch_gemm64(int64_t m, int64_t n, int64_t k, double alpha, const double *a, int64_t lda, int64_t strideA, const double *b,
                      int64_t ldb, int64_t strideB, double beta, double *c, int64_t ldc, int64_t strideC, int64_t batch, hipStream_t st) {
    const int64_t tm = (m + TS - 1) / TS, tn = (n + TS - 1) / TS;
    if (tm * tn > 2147483647LL) return mi_set_error(MI_ESHAPE, "mi_batched_gemm_f64: too many tiles");
    auto kern = gemm64_kernel<TA, TB, TS>;
    constexpr size_t SMEM = Tile64<TS>::SMEM;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, so a race is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(tm * tn), (unsigned)batch), dim3(Tile64<TS>::NT), SMEM, st, m, n, k, alpha, a, lda, strideA, b, ldb, strideB,
                       beta, c, ldc, strideC, tm);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

// ---- generic strided kernel --------------------------------------------------------------------------------
struct cdouble {
    double re, im;
};
struct cfloat {
    float re, im;
};

template <typename T>
struct Num;   // arithmetic of the element type of C
template <>
struct Num<double> {
    __device__ static double zero() { return 0.0; }
    __device__ static double fma(double a, double b, double c) { return __builtin_fma(a, b, c); }
    __device__ static double mul(double a, double b) { return a * b; }
    __device__ static double add(double a, double b) { return a + b; }
    __device__ static double scalar(double re, double) { return re; }
    __device__ static bool is_zero(double a) { return a == 0.0; }
    __device__ static double conj(double a) { return a; }
};
template <>
struct Num<float> {
    __device__ static float zero() { return 0.0f; }
    __device__ static float fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
    __device__ static float mul(float a, float b) { return a * b; }
    __device__ static float add(float a, float b) { return a + b; }
    __device__ static float scalar(double re, double) { return (float)re; }
    __device__ static bool is_zero(float a) { return a == 0.0f; }
    __device__ static float conj(float a) { return a; }
};
template <typename I, typename U>
struct NumInt {   // wraps on overflow, like Julia's integer arithmetic
    __device__ static I zero() { return 0; }
    __device__ static I fma(I a, I b, I c) { return (I)((U)a * (U)b + (U)c); }
    __device__ static I mul(I a, I b) { return (I)((U)a * (U)b); }
    __device__ static I add(I a, I b) { return (I)((U)a + (U)b); }
    __device__ static I scalar(double re, double) { return (I)(long long)re; }
    __device__ static bool is_zero(I a) { return a == 0; }
    __device__ static I conj(I a) { return a; }
};
template <>
struct Num<int64_t> : NumInt<int64_t, uint64_t> {};
template <>
struct Num<int32_t> : NumInt<int32_t, uint32_t> {};
template <>
struct Num<cdouble> {
    __device__ static cdouble zero() { return {0.0, 0.0}; }
    __device__ static cdouble fma(cdouble a, cdouble b, cdouble c) {
        return {__builtin_fma(a.re, b.re, __builtin_fma(-a.im, b.im, c.re)), __builtin_fma(a.re, b.im, __builtin_fma(a.im, b.re, c.im))};
    }
    __device__ static cdouble mul(cdouble a, cdouble b) { return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re}; }
    __device__ static cdouble add(cdouble a, cdouble b) { return {a.re + b.re, a.im + b.im}; }
    __device__ static cdouble scalar(double re, double im) { return {re, im}; }
    __device__ static bool is_zero(cdouble a) { return a.re == 0.0 && a.im == 0.0; }
    __device__ static cdouble conj(cdouble a) { return {a.re, -a.im}; }
};
template <>
struct Num<cfloat> {
    __device__ static cfloat zero() { return {0.0f, 0.0f}; }
    __device__ static cfloat fma(cfloat a, cfloat b, cfloat c) {
        return {__builtin_fmaf(a.re, b.re, __builtin_fmaf(-a.im, b.im, c.re)), __builtin_fmaf(a.re, b.im, __builtin_fmaf(a.im, b.re, c.im))};
    }
    __device__ static cfloat mul(cfloat a, cfloat b) { return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re}; }
    __device__ static cfloat add(cfloat a, cfloat b) { return {a.re + b.re, a.im + b.im}; }
    __device__ static cfloat scalar(double re, double im) { return {(float)re, (float)im}; }
    __device__ static bool is_zero(cfloat a) { return a.re == 0.0f && a.im == 0.0f; }
    __device__ static cfloat conj(cfloat a) { return {a.re, -a.im}; }
};

// value of element i of an array of element type `dt`, converted to T the way Julia's convert(T, x) does for the
// promotions that occur (real -> wider real, integer -> float, real -> complex, ComplexF32 -> ComplexF64)
template <typename T>
struct Load;
template <typename R>
__device__ inline R load_real(const void *p, int dt, int64_t i) {
    switch (dt) {
    case MI_F64: return (R)((const double *)p)[i];
    case MI_F32: return (R)((const float *)p)[i];
    case MI_F16: return (R)(float)((const _Float16 *)p)[i];
    case MI_BF16: return (R)(float)((const __bf16 *)p)[i];
    case MI_I32: return (R)((const int32_t *)p)[i];
    case MI_I64: return (R)((const int64_t *)p)[i];
    default: return (R)0;
    }
}
template <>
struct Load<double> {
    __device__ static double at(const void *p, int dt, int64_t i) { return load_real<double>(p, dt, i); }
};
template <>
struct Load<float> {
    __device__ static float at(const void *p, int dt, int64_t i) { return load_real<float>(p, dt, i); }
};
template <>
struct Load<int64_t> {
    __device__ static int64_t at(const void *p, int dt, int64_t i) { return dt == MI_I32 ? (int64_t)((const int32_t *)p)[i] : ((const int64_t *)p)[i]; }
};
template <>
struct Load<int32_t> {
    __device__ static int32_t at(const void *p, int dt, int64_t i) { return ((const int32_t *)p)[i]; }
};
template <>
struct Load<cdouble> {
    __device__ static cdouble at(const void *p, int dt, int64_t i) {
        if (dt == MI_C128) return ((const cdouble *)p)[i];
        if (dt == MI_C64) {
            const cfloat c = ((const cfloat *)p)[i];
            return {(double)c.re, (double)c.im};
        }
        return {load_real<double>(p, dt, i), 0.0};
    }
};
template <>
struct Load<cfloat> {
    __device__ static cfloat at(const void *p, int dt, int64_t i) {
        if (dt == MI_C64) return ((const cfloat *)p)[i];
        return {load_real<float>(p, dt, i), 0.0f};
    }
};

struct GenericArgs {
    int64_t m, n, k, batch;
    const void *A, *B;
    void *C;
    int64_t as[3], bs[3], cs[3];   // element strides of (row, column, batch) after op
    int dta, dtb, conj_a, conj_b;
    double alpha_re, alpha_im, beta_re, beta_im;
};

// 32 x 32 tile of C per workgroup, 2 x 2 outputs per thread, k in steps of 32 through LDS
template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GenericArgs g, int64_t tiles_m) {
    constexpr int TS = 32;
    __shared__ T As[TS][TS + 1];   // [k][row]
    __shared__ T Bs[TS][TS + 1];   // [k][col]
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int64_t row0 = (blockIdx.x % tiles_m) * TS, col0 = (blockIdx.x / tiles_m) * TS, b = blockIdx.y;
    T acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = Num<T>::zero();
    for (int64_t k0 = 0; k0 < g.k; k0 += TS) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int e = tid + 256 * u;
            const int i = e % TS, kk = e / TS;
            const int64_t gi = row0 + i, gk = k0 + kk;
            T v = Num<T>::zero();
            if (gi < g.m && gk < g.k) {
                v = Load<T>::at(g.A, g.dta, gi * g.as[0] + gk * g.as[1] + b * g.as[2]);
                if (g.conj_a) v = Num<T>::conj(v);
            }
            As[kk][i] = v;
            const int64_t gj = col0 + i;   // the same (fast, slow) split for B: fast index = column
            T w = Num<T>::zero();
            if (gj < g.n && gk < g.k) {
                w = Load<T>::at(g.B, g.dtb, gk * g.bs[0] + gj * g.bs[1] + b * g.bs[2]);
                if (g.conj_b) w = Num<T>::conj(w);
            }
            Bs[kk][i] = w;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < TS; kk++) {
            const T a0 = As[kk][tx], a1 = As[kk][tx + 16], b0 = Bs[kk][ty], b1 = Bs[kk][ty + 16];
            acc[0][0] = Num<T>::fma(a0, b0, acc[0][0]);
            acc[1][0] = Num<T>::fma(a1, b0, acc[1][0]);
            acc[0][1] = Num<T>::fma(a0, b1, acc[0][1]);
            acc[1][1] = Num<T>::fma(a1, b1, acc[1][1]);
        }
        __syncthreads();
    }
    const T alpha = Num<T>::scalar(g.alpha_re, g.alpha_im), beta = Num<T>::scalar(g.beta_re, g.beta_im);
    const bool overwrite = Num<T>::is_zero(beta);   // beta == 0: C is not read (a NaN there does not propagate)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int64_t gr = row0 + tx + 16 * i, gc = col0 + ty + 16 * j;
            if (gr < g.m && gc < g.n) {
                T *c = (T *)g.C + gr * g.cs[0] + gc * g.cs[1] + b * g.cs[2];
                const T x = Num<T>::mul(alpha, acc[i][j]);
                *c = overwrite ? x : Num<T>::add(x, Num<T>::mul(beta, *c));
            }
        }
}

template <typename T>
void launch_generic(const GenericArgs &g, hipStream_t st) {
    const int64_t tm = (g.m + 31) / 32, tn = (g.n + 31) / 32;
    hipLaunchKernelGGL(gemm_generic_kernel<T>, dim3((unsigned)(tm * tn), (unsigned)g.batch), dim3(256), 0, st, g, tm);
}

bool is_complex(int dt) { return dt == MI_C64 || dt == MI_C128; }
bool is_integer(int dt) { return dt == MI_I32 || dt == MI_I64; }
bool known(int dt) { return dt >= MI_F32 && dt <= MI_I64; }

// can a value of type `from` be converted exactly the way Julia's promotion to `to` does
bool converts(int from, int to) {
    if (from == to) return true;
    switch (to) {
    case MI_F64: return !is_complex(from);
    case MI_F32: return from == MI_F16 || from == MI_BF16 || is_integer(from);
    case MI_I64: return from == MI_I32;
    case MI_C128: return true;
    case MI_C64: return from == MI_F32 || from == MI_F16 || from == MI_BF16 || is_integer(from);
    default: return false;
    }
}

}  // namespace

MI_API int32_t mi_batched_gemm_f64(char transA, char transB, int64_t m, int64_t n, int64_t k, double alpha, const void *A, int64_t lda,
                                   int64_t strideA, const void *B, int64_t ldb, int64_t strideB, double beta, void *C, int64_t ldc,
                                   int64_t strideC, int64_t batch, mi_stream s) {
    auto flag = [](char c, bool *t) {
        if (c == 'N' || c == 'n') *t = false;
        else if (c == 'T' || c == 't' || c == 'C' || c == 'c') *t = true;
        else return false;
        return true;
    };
    bool ta, tb;
    if (!flag(transA, &ta) || !flag(transB, &tb)) return mi_set_error(MI_EINVAL, "mi_batched_gemm_f64: trans flags must be 'N', 'T' or 'C'");
    if (m < 0 || n < 0 || k < 0 || batch < 0) return mi_set_error(MI_ESHAPE, "mi_batched_gemm_f64: negative size");
    if (m == 0 || n == 0 || batch == 0) return MI_OK;
    if (!C || (k > 0 && (!A || !B))) return mi_set_error(MI_EINVAL, "mi_batched_gemm_f64: null pointer");
    if (lda < (ta ? k : m) || ldb < (tb ? n : k) || ldc < m || lda < 1 || ldb < 1)
        return mi_set_error(MI_ESHAPE, "mi_batched_gemm_f64: leading dimension smaller than the matrix it strides");
    if (strideA < 0 || strideB < 0 || strideC < 0) return mi_set_error(MI_ESHAPE, "mi_batched_gemm_f64: negative batch stride");
    if (batch > 65535) return mi_set_error(MI_ESHAPE, "mi_batched_gemm_f64: at most 65535 batch slices per call");
    hipStream_t st = (hipStream_t)s;
    const double *a = (const double *)A, *b = (const double *)B;
    double *c = (double *)C;
    // 128 x 128 tiles where those still give every compute unit a workgroup
    const bool large = m >= 128 && n >= 128 && ((m + 127) / 128) * ((n + 127) / 128) * batch >= 256;
#define MI_GEMM64(TA_, TB_)                                                                                                              \
    (large ? launch_gemm64<TA_, TB_, 128>(m, n, k, alpha, a, lda, strideA, b, ldb, strideB, beta, c, ldc, strideC, batch, st)             \
           : launch_gemm64<TA_, TB_, 64>(m, n, k, alpha, a, lda, strideA, b, ldb, strideB, beta, c, ldc, strideC, batch, st))
    if (!ta && !tb) return MI_GEMM64(false, false);
    if (ta && !tb) return MI_GEMM64(true, false);
    if (!ta && tb) return MI_GEMM64(false, true);
    return MI_GEMM64(true, true);
#undef MI_GEMM64
}

MI_API int32_t mi_batched_mul_generic(int32_t dtype_c, int32_t dtype_a, int32_t dtype_b, int64_t m, int64_t n, int64_t k, double alpha_re,
                                      double alpha_im, const void *A, int64_t a_row_stride, int64_t a_col_stride, int64_t a_batch_stride,
                                      int32_t conj_a, const void *B, int64_t b_row_stride, int64_t b_col_stride, int64_t b_batch_stride,
                                      int32_t conj_b, double beta_re, double beta_im, void *C, int64_t c_row_stride, int64_t c_col_stride,
                                      int64_t c_batch_stride, int64_t batch, mi_stream s) {
    if (!known(dtype_c) || !known(dtype_a) || !known(dtype_b) || dtype_c == MI_F16 || dtype_c == MI_BF16)
        return mi_set_error(MI_EDTYPE, "mi_batched_mul_generic: C must be Float32, Float64, Int32, Int64, ComplexF32 or ComplexF64 (got %d), "
                            "A and B any supported element type (got %d, %d)", dtype_c, dtype_a, dtype_b);
    if (!converts(dtype_a, dtype_c) || !converts(dtype_b, dtype_c))
        return mi_set_error(MI_EDTYPE, "mi_batched_mul_generic: element types %d and %d do not promote to that of C (%d)", dtype_a, dtype_b, dtype_c);
    if (m < 0 || n < 0 || k < 0 || batch < 0) return mi_set_error(MI_ESHAPE, "mi_batched_mul_generic: negative size");
    if (m == 0 || n == 0 || batch == 0) return MI_OK;
    if (!C || (k > 0 && (!A || !B))) return mi_set_error(MI_EINVAL, "mi_batched_mul_generic: null pointer");
    if (a_row_stride < 0 || a_col_stride < 0 || a_batch_stride < 0 || b_row_stride < 0 || b_col_stride < 0 || b_batch_stride < 0 ||
        c_row_stride < 0 || c_col_stride < 0 || c_batch_stride < 0)
        return mi_set_error(MI_ESHAPE, "mi_batched_mul_generic: negative stride");
    if (!is_complex(dtype_c) && (alpha_im != 0.0 || beta_im != 0.0))
        return mi_set_error(MI_EINVAL, "mi_batched_mul_generic: complex alpha / beta with a real C");
    if (is_integer(dtype_c) && (alpha_re != floor(alpha_re) || beta_re != floor(beta_re)))
        return mi_set_error(MI_EINVAL, "mi_batched_mul_generic: alpha and beta must be integers for an integer C");   // Julia: InexactError
    if (batch > 65535) return mi_set_error(MI_ESHAPE, "mi_batched_mul_generic: at most 65535 batch slices per call");
    if (((m + 31) / 32) * ((n + 31) / 32) > 2147483647LL) return mi_set_error(MI_ESHAPE, "mi_batched_mul_generic: too many tiles");
    GenericArgs g;
    g.m = m; g.n = n; g.k = k; g.batch = batch;
    g.A = A; g.B = B; g.C = C;
    g.as[0] = a_row_stride; g.as[1] = a_col_stride; g.as[2] = a_batch_stride;
    g.bs[0] = b_row_stride; g.bs[1] = b_col_stride; g.bs[2] = b_batch_stride;
    g.cs[0] = c_row_stride; g.cs[1] = c_col_stride; g.cs[2] = c_batch_stride;
    g.dta = dtype_a; g.dtb = dtype_b;
    g.conj_a = conj_a != 0 && is_complex(dtype_a);
    g.conj_b = conj_b != 0 && is_complex(dtype_b);
    g.alpha_re = alpha_re; g.alpha_im = alpha_im; g.beta_re = beta_re; g.beta_im = beta_im;
    hipStream_t st = (hipStream_t)s;
    switch (dtype_c) {
    case MI_F64: launch_generic<double>(g, st); break;
    case MI_F32: launch_generic<float>(g, st); break;
    case MI_I64: launch_generic<int64_t>(g, st); break;
    case MI_I32: launch_generic<int32_t>(g, st); break;
    case MI_C128: launch_generic<cdouble>(g, st); break;
    default: launch_generic<cfloat>(g, st); break;
    }
    MI_LAUNCH_CHECK();
    return MI_OK;
}
