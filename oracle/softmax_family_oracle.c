/*
 * CPU oracle for the softmax family over arbitrary dims.  TEST INFRASTRUCTURE ONLY (same rules as
 * nnlib_oracle.c: nothing in the shipped library links, loads or calls it).
 *
 * Restates, in plain C, NNlib.jl's
 *   _softmax!       src/softmax.jl:69-79
 *   _logsoftmax!    src/softmax.jl:137-147
 *   logsumexp       src/softmax.jl:200-203
 *   _∇softmax!      src/softmax.jl:107-110
 *   _∇logsoftmax!   src/softmax.jl:175-177
 * for a reduction over a run of adjacent dimensions: the array is viewed as (inner, len, outer),
 * element (i, j, o) at i + inner*(j + len*o), reduced over j.
 *
 * Pinned by (tests/test_oracle.py): the doctest tables for dims = 1 and dims = 2
 * (src/softmax.jl:20-36), logsoftmax known answers [-2999, -2998, 0] and [-999 -1998 -2997; 0 0 0]
 * (test/softmax.jl:30-34), the gradient known answers [1 1 1; -1 -1 -1], zeros, and the
 * 3x6 table computed with PyTorch's LogSoftmax (test/softmax.jl:36-58), the +-Inf/NaN table incl.
 * dims = 2, dims = : and dims = (1,2) (test/softmax.jl:63-74), logsumexp against
 * mean(x - logsoftmax(x)) (test/softmax.jl:100-106), and closed forms.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define ORC_API __attribute__((visibility("default")))

#define AT(i, j, o) ((i) + inner * ((j) + len * (o)))

#define DEFINE_FAMILY(SUF, real, EXP, LOG)                                                          \
    /* op 0 = softmax, 1 = logsoftmax; y may alias x */                                              \
    ORC_API void orc_softmax_nd_##SUF(int op, const real *x, real *y, int64_t inner, int64_t len,   \
                                      int64_t outer)                                                \
    {                                                                                                \
        for (int64_t o = 0; o < outer; o++)                                                          \
            for (int64_t i = 0; i < inner; i++) {                                                    \
                real m = (real)-INFINITY; /* fast_maximum: reduce(max; init = -Inf) */               \
                for (int64_t j = 0; j < len; j++) m = x[AT(i, j, o)] > m ? x[AT(i, j, o)] : m;       \
                real s = 0;                                                                          \
                if (op == 0) {                                                                       \
                    for (int64_t j = 0; j < len; j++) {                                              \
                        real v = x[AT(i, j, o)], e;                                                  \
                        if (m == (real)INFINITY) e = (v == (real)INFINITY) ? 1 : 0;                  \
                        else e = EXP(v - m);                                                         \
                        y[AT(i, j, o)] = e;                                                          \
                        s += e;                                                                      \
                    }                                                                                \
                    for (int64_t j = 0; j < len; j++) y[AT(i, j, o)] /= s;                           \
                } else {                                                                             \
                    for (int64_t j = 0; j < len; j++) {                                              \
                        real v = x[AT(i, j, o)], d;                                                  \
                        if (m == (real)INFINITY) d = (v == (real)INFINITY) ? 0 : (real)-INFINITY;    \
                        else d = v - m;                                                              \
                        y[AT(i, j, o)] = d;                                                          \
                        s += EXP(d);                                                                 \
                    }                                                                                \
                    real l = LOG(s);                                                                 \
                    for (int64_t j = 0; j < len; j++) y[AT(i, j, o)] -= l;                           \
                }                                                                                    \
            }                                                                                        \
    }                                                                                                \
    /* y: (inner, outer) */                                                                          \
    ORC_API void orc_logsumexp_##SUF(const real *x, real *y, int64_t inner, int64_t len,            \
                                     int64_t outer)                                                 \
    {                                                                                                \
        for (int64_t o = 0; o < outer; o++)                                                          \
            for (int64_t i = 0; i < inner; i++) {                                                    \
                real m = (real)-INFINITY;                                                            \
                for (int64_t j = 0; j < len; j++) m = x[AT(i, j, o)] > m ? x[AT(i, j, o)] : m;       \
                real s = 0;                                                                          \
                for (int64_t j = 0; j < len; j++) s += EXP(x[AT(i, j, o)] - m);                      \
                y[i + inner * o] = m + LOG(s);                                                       \
            }                                                                                        \
    }                                                                                                \
    /* pullback of logsumexp (rrule, src/softmax.jl:205-212): tmp = exp(x - max),                  \
     * dx = dy .* tmp ./ sum(tmp).  dy: (inner, outer) */                                            \
    ORC_API void orc_logsumexp_bwd_##SUF(const real *dy, const real *x, real *dx, int64_t inner,     \
                                         int64_t len, int64_t outer)                                \
    {                                                                                                \
        for (int64_t o = 0; o < outer; o++)                                                          \
            for (int64_t i = 0; i < inner; i++) {                                                    \
                real m = (real)-INFINITY;                                                            \
                for (int64_t j = 0; j < len; j++) m = x[AT(i, j, o)] > m ? x[AT(i, j, o)] : m;       \
                real s = 0;                                                                          \
                for (int64_t j = 0; j < len; j++) s += EXP(x[AT(i, j, o)] - m);                      \
                for (int64_t j = 0; j < len; j++)                                                    \
                    dx[AT(i, j, o)] = dy[i + inner * o] * EXP(x[AT(i, j, o)] - m) / s;               \
            }                                                                                        \
    }                                                                                                \
    /* op 0: dx = dy*y - y*sum(dy*y); op 1: dx = dy - sum(dy)*exp(y).  dx may alias dy */            \
    ORC_API void orc_softmax_bwd_##SUF(int op, const real *dy, const real *y, real *dx,             \
                                       int64_t inner, int64_t len, int64_t outer)                   \
    {                                                                                                \
        for (int64_t o = 0; o < outer; o++)                                                          \
            for (int64_t i = 0; i < inner; i++) {                                                    \
                real s = 0;                                                                          \
                for (int64_t j = 0; j < len; j++)                                                    \
                    s += op == 0 ? dy[AT(i, j, o)] * y[AT(i, j, o)] : dy[AT(i, j, o)];               \
                for (int64_t j = 0; j < len; j++) {                                                  \
                    real g = dy[AT(i, j, o)], yy = y[AT(i, j, o)];                                   \
                    dx[AT(i, j, o)] = op == 0 ? g * yy - yy * s : g - s * EXP(yy);                   \
                }                                                                                    \
            }                                                                                        \
    }

DEFINE_FAMILY(f32, float, expf, logf)
DEFINE_FAMILY(f64, double, exp, log)
