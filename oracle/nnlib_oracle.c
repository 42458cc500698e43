/*
 * CPU oracle for the attention path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C on host memory, what NNlib.jl computes for
 * dot_product_attention / dot_product_attention_scores / softmax(dims=1) /
 * batched_mul.  It exists so that the HIP kernels can be checked against the
 * reference's algorithm; nothing in the shipped library links, loads or calls
 * it.  Only the tests, the smoke check and the benchmark's CPU-baseline leg
 * may use it.
 *
 * All arrays are column-major (Julia layout).  Index (d, i, b) of a
 * (E, L, B) array lives at d + i*E + b*E*L.
 *
 * Two families:
 *   orc_attention_f64      direct evaluation of the defining formula in
 *                          double precision (no temporaries shaped like the
 *                          reference's; an independent statement).
 *   orc_nnlib_attention_f32 the reference's op sequence in Float32, one
 *                          temporary per reference temporary, threaded the
 *                          way the reference threads it.
 *
 * Pinned by (see tests/test_oracle.py): the golden output/weights vectors of
 * reference test/attention.jl:25-34, scores==attention-weights equivalence
 * (:17-23), mask zero patterns (:36-52), the softmax doctest values
 * (src/softmax.jl:20-36), the +-Inf/NaN table (test/softmax.jl:63-70), the
 * masked-input cases (test/ext_cuda/softmax.jl:34-78), per-slice brute-force
 * GEMM with alpha/beta and batch-1 broadcast (test/batchedmul.jl:6-28,
 * 99-106), plus closed forms.  Not pinned by any reference test: the NaN
 * result for a fully masked column (follows from src/softmax.jl:73-75 by
 * reading only) -- "parity unpinned" for that single behaviour.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* single-slice SGEMM, column-major, C = alpha*op(A)*op(B) + beta*C    */
/* Stands in for the BLAS ?gemm_ that src/gemm.jl:141-149 ccalls.      */
/* ------------------------------------------------------------------ */

#define MR 8
#define NR 16
#define KC 256
#define MC 128
#define NC 1024

typedef float v8f __attribute__((vector_size(32), aligned(4)));

/* micro kernel: acc[NR][MR] = Ap (kc x MR packed) * Bp (kc x NR packed) */
__attribute__((target_clones("avx512f", "avx2,fma", "default")))
static void micro_8x16(int kc, const float *restrict Ap, const float *restrict Bp,
                       float *restrict acc)
{
    v8f c[NR];
    for (int j = 0; j < NR; j++) c[j] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
    for (int p = 0; p < kc; p++) {
        v8f a = *(const v8f *)(Ap + (size_t)p * MR);
        const float *b = Bp + (size_t)p * NR;
        for (int j = 0; j < NR; j++) c[j] += a * b[j];
    }
    for (int j = 0; j < NR; j++) *(v8f *)(acc + j * MR) = c[j];
}

static inline float op_at(const float *X, int64_t ld, int trans, int64_t r, int64_t c)
{
    return trans ? X[c + r * ld] : X[r + c * ld];
}

/*
 * Optional: a BLAS sgemm_ (Fortran interface) to run the slices with, as the reference does
 * (ccall of sgemm_ through libblastrampoline, src/gemm.jl:141-149).  Unset (NULL) = the kernel
 * above.  The benchmark's CPU baseline sets it when the host has a BLAS; the parity tests leave
 * it unset, so parity never depends on a library's rounding.
 */
typedef void (*sgemm_fn)(const char *, const char *, const int *, const int *, const int *,
                         const float *, const float *, const int *, const float *, const int *,
                         const float *, float *, const int *);
static sgemm_fn g_sgemm = NULL;
ORC_API void orc_set_sgemm(void *fn) { g_sgemm = (sgemm_fn)fn; }
ORC_API int orc_has_sgemm(void) { return g_sgemm != NULL; }

/* trans flags: 0 = 'N', 1 = 'T'. */
static void sgemm_slice(int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha,
                        const float *A, int64_t lda, const float *B, int64_t ldb, float beta,
                        float *C, int64_t ldc)
{
    if (g_sgemm && m > 0 && n > 0 && m < 2147483647 && n < 2147483647 && k < 2147483647 &&
        lda < 2147483647 && ldb < 2147483647 && ldc < 2147483647) {
        const char ta = transA ? 'T' : 'N', tb = transB ? 'T' : 'N';
        const int mi = (int)m, ni = (int)n, ki = (int)k, la = (int)lda, lb = (int)ldb, lc = (int)ldc;
        g_sgemm(&ta, &tb, &mi, &ni, &ki, &alpha, A, &la, B, &lb, &beta, C, &lc);
        return;
    }
    /* reference BLAS semantics: beta == 0 overwrites C without reading it */
    for (int64_t j = 0; j < n; j++)
        for (int64_t i = 0; i < m; i++) {
            float *c = &C[i + j * ldc];
            *c = (beta == 0.0f) ? 0.0f : beta * (*c);
        }
    if (k == 0 || alpha == 0.0f) return;

    float *Ap = (float *)aligned_alloc(64, sizeof(float) * (size_t)MC * KC);
    float *Bp = (float *)aligned_alloc(64, sizeof(float) * (size_t)NC * KC);
    float acc[MR * NR] __attribute__((aligned(64)));

    for (int64_t jc = 0; jc < n; jc += NC) {
        int64_t nc = n - jc < NC ? n - jc : NC;
        for (int64_t pc = 0; pc < k; pc += KC) {
            int kc = (int)(k - pc < KC ? k - pc : KC);
            /* pack B panel: for each NR column strip, kc x NR, zero padded */
            for (int64_t jr = 0; jr < nc; jr += NR)
                for (int p = 0; p < kc; p++)
                    for (int j = 0; j < NR; j++) {
                        int64_t col = jc + jr + j;
                        Bp[(size_t)jr * kc + (size_t)p * NR + j] =
                            col < n ? op_at(B, ldb, transB, pc + p, col) : 0.0f;
                    }
            for (int64_t ic = 0; ic < m; ic += MC) {
                int64_t mc = m - ic < MC ? m - ic : MC;
                for (int64_t ir = 0; ir < mc; ir += MR)
                    for (int p = 0; p < kc; p++)
                        for (int i = 0; i < MR; i++) {
                            int64_t row = ic + ir + i;
                            Ap[(size_t)ir * kc + (size_t)p * MR + i] =
                                row < m ? op_at(A, lda, transA, row, pc + p) : 0.0f;
                        }
                for (int64_t jr = 0; jr < nc; jr += NR)
                    for (int64_t ir = 0; ir < mc; ir += MR) {
                        micro_8x16(kc, Ap + (size_t)ir * kc, Bp + (size_t)jr * kc, acc);
                        int64_t mi = mc - ir < MR ? mc - ir : MR;
                        int64_t nj = nc - jr < NR ? nc - jr : NR;
                        for (int64_t j = 0; j < nj; j++)
                            for (int64_t i = 0; i < mi; i++)
                                C[(ic + ir + i) + (jc + jr + j) * ldc] += alpha * acc[j * MR + i];
                    }
            }
        }
    }
    free(Ap);
    free(Bp);
}

/* ------------------------------------------------------------------ */
/* batched GEMM with the reference's thread policy                      */
/* reference: src/gemm.jl:89-188                                        */
/* ------------------------------------------------------------------ */

typedef struct {
    int transA, transB;
    int64_t m, n, k;
    float alpha, beta;
    const float *A;
    int64_t lda, strideA;
    const float *B;
    int64_t ldb, strideB;
    float *C;
    int64_t ldc, strideC;
    int64_t k0, k1; /* batch range of this task */
} gemm_task;

static void *gemm_part(void *arg)
{
    gemm_task *t = (gemm_task *)arg;
    for (int64_t b = t->k0; b < t->k1; b++)
        sgemm_slice(t->transA, t->transB, t->m, t->n, t->k, t->alpha, t->A + b * t->strideA,
                    t->lda, t->B + b * t->strideB, t->ldb, t->beta, t->C + b * t->strideC, t->ldc);
    return NULL;
}

/*
 * C[:,:,b] = alpha*op(A[:,:,b])*op(B[:,:,b]) + beta*C[:,:,b], b in [0,batch).
 * strideA/strideB == 0 means that operand has a single slice shared by every
 * batch (src/gemm.jl:117-118).  lenA/lenB are the element counts of A and B,
 * which decide the task count exactly as src/gemm.jl:121-123 does:
 *     n_threads = min(nthreads, 1 + max(length(A), length(B)) / 8000)
 * and the batch range is cut into ceil(batch/n_threads)-sized parts (:132).
 */
ORC_API void orc_batched_gemm_f32(int transA, int transB, int64_t m, int64_t n, int64_t k,
                                  float alpha, const float *A, int64_t lda, int64_t strideA,
                                  int64_t lenA, const float *B, int64_t ldb, int64_t strideB,
                                  int64_t lenB, float beta, float *C, int64_t ldc, int64_t strideC,
                                  int64_t batch, int nthreads)
{
    if (batch <= 0) return;
    int64_t big = lenA > lenB ? lenA : lenB;
    int64_t want = 1 + big / 8000;
    int64_t nt = nthreads < want ? nthreads : want;
    if (nt < 1) nt = 1;
    int64_t chunk = (batch + nt - 1) / nt;
    int64_t nparts = (batch + chunk - 1) / chunk;

    gemm_task *tasks = (gemm_task *)malloc(sizeof(gemm_task) * (size_t)nparts);
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nparts);
    for (int64_t p = 0; p < nparts; p++) {
        gemm_task t = {transA, transB, m,   n,       k, alpha, beta,          A,
                       lda,    strideA, B,  ldb,     strideB,  C,    ldc,    strideC,
                       p * chunk, (p + 1) * chunk < batch ? (p + 1) * chunk : batch};
        tasks[p] = t;
    }
    if (nparts == 1) {
        gemm_part(&tasks[0]);
    } else {
        for (int64_t p = 0; p < nparts; p++) pthread_create(&tid[p], NULL, gemm_part, &tasks[p]);
        for (int64_t p = 0; p < nparts; p++) pthread_join(tid[p], NULL);
    }
    free(tasks);
    free(tid);
}

/* ------------------------------------------------------------------ */
/* softmax over the first (contiguous) dimension                        */
/* reference: src/softmax.jl:69-79 and fast_maximum :118                */
/* ------------------------------------------------------------------ */

/*
 * x, y: (rows, cols) column-major, y may alias x.  Same four passes as the
 * reference: column max -> exp(x - max) (or the +-Inf rule) -> column sum ->
 * divide.  The reference chooses between its two elementwise formulas with
 * one global test (all column maxima finite); per column both formulas agree
 * whenever that column's max is finite, so the choice is made per column.
 * Like the reference's passes this is single threaded.
 */
ORC_API void orc_softmax_dim1_f32(const float *x, float *y, int64_t rows, int64_t cols)
{
    float *mx = (float *)malloc(sizeof(float) * (size_t)(cols > 0 ? cols : 1));
    for (int64_t c = 0; c < cols; c++) {
        const float *xc = x + c * rows;
        float m = -INFINITY;
        for (int64_t r = 0; r < rows; r++) m = xc[r] > m ? xc[r] : m; /* fastmath max */
        mx[c] = m;
    }
    for (int64_t c = 0; c < cols; c++) {
        const float *xc = x + c * rows;
        float *yc = y + c * rows;
        float m = mx[c];
        if (isfinite(m)) {
            for (int64_t r = 0; r < rows; r++) yc[r] = expf(xc[r] - m);
        } else {
            for (int64_t r = 0; r < rows; r++) {
                float v = xc[r];
                yc[r] = (m == INFINITY) ? ((v == INFINITY) ? 1.0f : 0.0f) : expf(v - m);
            }
        }
    }
    for (int64_t c = 0; c < cols; c++) {
        const float *yc = y + c * rows;
        float s = 0.0f;
        for (int64_t r = 0; r < rows; r++) s += yc[r];
        mx[c] = s;
    }
    for (int64_t c = 0; c < cols; c++) {
        float *yc = y + c * rows;
        float s = mx[c];
        for (int64_t r = 0; r < rows; r++) yc[r] /= s;
    }
    free(mx);
}

ORC_API void orc_softmax_dim1_f64(const double *x, double *y, int64_t rows, int64_t cols)
{
    for (int64_t c = 0; c < cols; c++) {
        const double *xc = x + c * rows;
        double *yc = y + c * rows;
        double m = -INFINITY;
        for (int64_t r = 0; r < rows; r++) m = xc[r] > m ? xc[r] : m;
        double s = 0.0;
        for (int64_t r = 0; r < rows; r++) {
            double v = xc[r], e;
            if (m == INFINITY) e = (v == INFINITY) ? 1.0 : 0.0;
            else e = exp(v - m);
            yc[r] = e;
            s += e;
        }
        for (int64_t r = 0; r < rows; r++) yc[r] /= s;
    }
}

/* ------------------------------------------------------------------ */
/* make_causal_mask: m[i,j] = (i <= j), (len,len) column-major          */
/* reference: src/attention.jl:149-153                                  */
/* ------------------------------------------------------------------ */
ORC_API void orc_make_causal_mask(uint8_t *m, int64_t len)
{
    for (int64_t j = 0; j < len; j++)
        for (int64_t i = 0; i < len; i++) m[i + j * len] = (uint8_t)(i <= j);
}

/* ------------------------------------------------------------------ */
/* the reference's attention, op by op, Float32                         */
/* reference: src/attention.jl:52-127                                   */
/* ------------------------------------------------------------------ */

/*
 * Strides are in elements of the broadcast operand for the four logical dims
 * (kv, q, head, batch) of the score tensor; 0 = that dim is broadcast.
 * bias == NULL / mask == NULL skip the step exactly as the `nothing` methods
 * do (src/attention.jl:129,133).  mask: nonzero = keep.
 *
 * q (E, Lq, B), k (E, Lkv, B), v (Ev, Lkv, B); H divides E and Ev.
 * out (Ev, Lq, B); alpha (Lkv, Lq, H, B).
 */
ORC_API void orc_nnlib_attention_f32(const float *q, const float *k, const float *v,
                                     const float *bias, const int64_t *bias_strides,
                                     const uint8_t *mask, const int64_t *mask_strides, int64_t E,
                                     int64_t Ev, int64_t Lq, int64_t Lkv, int64_t H, int64_t B,
                                     float *out, float *alpha, int nthreads)
{
    const int64_t D = E / H, Dv = Ev / H;
    const int64_t HB = H * B;
    /* kt = permutedims(k4, (3,1,2,4))  -> (Lkv, D, H, B)          attention.jl:117 */
    float *kt = (float *)malloc(sizeof(float) * (size_t)(Lkv * D * HB));
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t d = 0; d < D; d++)
                for (int64_t j = 0; j < Lkv; j++)
                    kt[j + Lkv * (d + D * (h + H * b))] = k[d + D * h + E * (j + Lkv * b)];
    /* qt = permutedims(q4, (1,3,2,4)) ./ sqrt(T(D)) -> (D, Lq, H, B)   attention.jl:118 */
    float *qt = (float *)malloc(sizeof(float) * (size_t)(D * Lq * HB));
    const float sq = sqrtf((float)D);
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t i = 0; i < Lq; i++)
                for (int64_t d = 0; d < D; d++)
                    qt[d + D * (i + Lq * (h + H * b))] = q[d + D * h + E * (i + Lq * b)] / sq;
    /* logits = batched_mul(kt, qt) -> (Lkv, Lq, H*B)                 attention.jl:119 */
    const int64_t S1 = Lkv * Lq;
    float *logits = alpha; /* reuse caller's alpha storage as the score tensor */
    orc_batched_gemm_f32(0, 0, Lkv, Lq, D, 1.0f, kt, Lkv, Lkv * D, Lkv * D * HB, qt, D, D * Lq,
                         D * Lq * HB, 0.0f, logits, Lkv, S1, HB, nthreads);
    free(kt);
    free(qt);
    /* logits .+ bias                                                  attention.jl:131 */
    if (bias) {
        for (int64_t b = 0; b < B; b++)
            for (int64_t h = 0; h < H; h++)
                for (int64_t i = 0; i < Lq; i++) {
                    float *col = logits + Lkv * (i + Lq * (h + H * b));
                    const float *bc = bias + i * bias_strides[1] + h * bias_strides[2] +
                                      b * bias_strides[3];
                    for (int64_t j = 0; j < Lkv; j++) col[j] += bc[j * bias_strides[0]];
                }
    }
    /* ifelse.(mask, logits, typemin(T))                               attention.jl:135-138 */
    if (mask) {
        for (int64_t b = 0; b < B; b++)
            for (int64_t h = 0; h < H; h++)
                for (int64_t i = 0; i < Lq; i++) {
                    float *col = logits + Lkv * (i + Lq * (h + H * b));
                    const uint8_t *mc = mask + i * mask_strides[1] + h * mask_strides[2] +
                                        b * mask_strides[3];
                    for (int64_t j = 0; j < Lkv; j++)
                        if (!mc[j * mask_strides[0]]) col[j] = -INFINITY;
                }
    }
    /* alpha = softmax(logits; dims=1)                                 attention.jl:125 */
    orc_softmax_dim1_f32(logits, alpha, Lkv, Lq * HB);
    if (!out) return; /* dot_product_attention_scores stops here */
    /* vt = permutedims(v4, (1,3,2,4)) -> (Dv, Lkv, H, B)              attention.jl:96 */
    float *vt = (float *)malloc(sizeof(float) * (size_t)(Dv * Lkv * HB));
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t j = 0; j < Lkv; j++)
                memcpy(vt + Dv * (j + Lkv * (h + H * b)), v + Dv * h + Ev * (j + Lkv * b),
                       sizeof(float) * (size_t)Dv);
    /* x = batched_mul(vt, alpha) -> (Dv, Lq, H*B)                     attention.jl:97 */
    float *x = (float *)malloc(sizeof(float) * (size_t)(Dv * Lq * HB));
    orc_batched_gemm_f32(0, 0, Dv, Lq, Lkv, 1.0f, vt, Dv, Dv * Lkv, Dv * Lkv * HB, alpha, Lkv, S1,
                         S1 * HB, 0.0f, x, Dv, Dv * Lq, HB, nthreads);
    free(vt);
    /* permutedims(x, (1,3,2,4)) then join_heads -> (Ev, Lq, B)        attention.jl:98,159 */
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t i = 0; i < Lq; i++)
                memcpy(out + Dv * h + Ev * (i + Lq * b), x + Dv * (i + Lq * (h + H * b)),
                       sizeof(float) * (size_t)Dv);
    free(x);
}

/* ------------------------------------------------------------------ */
/* defining formula in double precision                                 */
/*   logits[j,i,h,b] = sum_d k[d,h,j,b] * (q[d,h,i,b] / sqrt(D))         */
/*   alpha = softmax_j(mask ? logits + bias : -Inf)                      */
/*   x[d,h,i,b] = sum_j alpha[j,i,h,b] * v[d,h,j,b]                      */
/* (the @tullio comments at src/attention.jl:94-95,115-116)              */
/* ------------------------------------------------------------------ */
ORC_API void orc_attention_f64(const double *q, const double *k, const double *v,
                               const double *bias, const int64_t *bias_strides,
                               const uint8_t *mask, const int64_t *mask_strides, int64_t E,
                               int64_t Ev, int64_t Lq, int64_t Lkv, int64_t H, int64_t B,
                               double *out, double *alpha)
{
    const int64_t D = E / H, Dv = Ev / H;
    const double sq = sqrt((double)D);
    double *col = (double *)malloc(sizeof(double) * (size_t)(Lkv > 0 ? Lkv : 1));
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t i = 0; i < Lq; i++) {
                const double *qi = q + D * h + E * (i + Lq * b);
                for (int64_t j = 0; j < Lkv; j++) {
                    const double *kj = k + D * h + E * (j + Lkv * b);
                    double s = 0.0;
                    for (int64_t d = 0; d < D; d++) s += kj[d] * (qi[d] / sq);
                    if (bias)
                        s += bias[j * bias_strides[0] + i * bias_strides[1] +
                                  h * bias_strides[2] + b * bias_strides[3]];
                    if (mask && !mask[j * mask_strides[0] + i * mask_strides[1] +
                                      h * mask_strides[2] + b * mask_strides[3]])
                        s = -INFINITY;
                    col[j] = s;
                }
                orc_softmax_dim1_f64(col, col, Lkv, 1);
                if (alpha) memcpy(alpha + Lkv * (i + Lq * (h + H * b)), col, sizeof(double) * (size_t)Lkv);
                if (out) {
                    double *o = out + Dv * h + Ev * (i + Lq * b);
                    for (int64_t d = 0; d < Dv; d++) o[d] = 0.0;
                    for (int64_t j = 0; j < Lkv; j++) {
                        const double *vj = v + Dv * h + Ev * (j + Lkv * b);
                        double a = col[j];
                        for (int64_t d = 0; d < Dv; d++) o[d] += a * vj[d];
                    }
                }
            }
    free(col);
}

/* brute-force per-slice GEMM in double: test/batchedmul.jl:6-16 */
ORC_API void orc_batched_gemm_f64(int transA, int transB, int64_t m, int64_t n, int64_t k,
                                  double alpha, const double *A, int64_t lda, int64_t strideA,
                                  const double *B, int64_t ldb, int64_t strideB, double beta,
                                  double *C, int64_t ldc, int64_t strideC, int64_t batch)
{
    for (int64_t b = 0; b < batch; b++) {
        const double *Ab = A + b * strideA, *Bb = B + b * strideB;
        double *Cb = C + b * strideC;
        for (int64_t j = 0; j < n; j++)
            for (int64_t i = 0; i < m; i++) {
                double s = 0.0;
                for (int64_t p = 0; p < k; p++) {
                    double a = transA ? Ab[p + i * lda] : Ab[i + p * lda];
                    double bb = transB ? Bb[j + p * ldb] : Bb[p + j * ldb];
                    s += a * bb;
                }
                double *c = &Cb[i + j * ldc];
                *c = alpha * s + (beta == 0.0 ? 0.0 : beta * (*c));
            }
    }
}
