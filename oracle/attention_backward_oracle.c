/*
 * CPU oracle for the gradient of dot_product_attention.  TEST INFRASTRUCTURE ONLY (same rules as
 * nnlib_oracle.c).
 *
 * NNlib has no hand-written rrule for attention: reverse-mode AD walks the forward op sequence of
 * src/attention.jl:86-127 backwards through the rules the package does define.  This file restates
 * that chain in double precision, one step per forward op:
 *
 *   x  = batched_mul(vt, alpha)            -> d_alpha = vt' * dx,  dvt = dx * alpha'
 *                                             (rrule of batched_mul, src/batched/batchedmul.jl:96-110)
 *   alpha = softmax(logits; dims = 1)      -> d_logits = d_alpha .* alpha - alpha .* sum(d_alpha .* alpha)
 *                                             (_∇softmax!, src/softmax.jl:107-110)
 *   logits = ifelse.(mask, logits, -Inf)   -> zero where dropped (alpha is 0 there)
 *   logits = logits .+ bias                -> d_bias = d_logits summed over the broadcast dims
 *   logits = batched_mul(kt, q ./ sqrt(D)) -> dk = d_logits * (q/sqrt(D))',  dq = kt' * d_logits / sqrt(D)
 *
 * An optional cotangent of the returned weights is added to d_alpha (the forward returns (x, alpha)).
 *
 * fdrop = dropout (src/attention.jl:126, src/dropout.jl:38-53) multiplies alpha elementwise by a fixed
 * array g (0 where dropped, 1/(1-p) where kept) before the value product and before alpha is returned;
 * its pullback multiplies the cotangent by the same g:
 *   alpha_d = alpha .* g,  x = batched_mul(vt, alpha_d)  -> d_alpha = g .* (vt' * dx + d_returned)
 * `keep_scale` is that g (NULL = identity).
 *
 * Pinned by (tests/test_attention_backward_oracle.py): central finite differences of the forward
 * oracle (itself pinned by the golden vectors of test/attention.jl:25-34) for q, k, v and bias, on the
 * reference's own gradient-test shapes (test/attention.jl:70-76), with masks, causal masks and
 * several heads; and an independent numpy einsum statement.  The reference's test is the same kind
 * of check (gradtest compares the AD result with finite differences).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* alpha: (Lkv, Lq, H, B) forward weights before dropout (from orc_attention_f64).
 * dout: (Ev, Lq, B); dweights, keep_scale: NULL or (Lkv, Lq, H, B).
 * dq (E, Lq, B), dk (E, Lkv, B), dv (Ev, Lkv, B): overwritten.
 * dbias: NULL, or an array addressed with bias_strides (0 = broadcast dim, summed); ADDED into. */
ORC_API void orc_attention_bwd_f64(const double *q, const double *k, const double *v,
                                   const double *alpha, const double *dout, const double *dweights,
                                   const double *keep_scale, const int64_t *bias_strides, int64_t E, int64_t Ev, int64_t Lq,
                                   int64_t Lkv, int64_t H, int64_t B, double *dq, double *dk,
                                   double *dv, double *dbias)
{
    const int64_t D = E / H, Dv = Ev / H;
    const double sq = sqrt((double)D);
    memset(dq, 0, sizeof(double) * (size_t)(E * Lq * B));
    memset(dk, 0, sizeof(double) * (size_t)(E * Lkv * B));
    memset(dv, 0, sizeof(double) * (size_t)(Ev * Lkv * B));
    double *da = (double *)malloc(sizeof(double) * (size_t)(Lkv > 0 ? Lkv : 1));
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t i = 0; i < Lq; i++) {
                const double *a = alpha + Lkv * (i + Lq * (h + H * b));
                const double *dx = dout + Dv * h + Ev * (i + Lq * b);
                const double *qi = q + D * h + E * (i + Lq * b);
                double *dqi = dq + D * h + E * (i + Lq * b);
                double dot = 0.0;
                for (int64_t j = 0; j < Lkv; j++) {
                    const double *vj = v + Dv * h + Ev * (j + Lkv * b);
                    double *dvj = dv + Dv * h + Ev * (j + Lkv * b);
                    const double g = keep_scale ? keep_scale[j + Lkv * (i + Lq * (h + H * b))] : 1.0;
                    double s = 0.0;
                    for (int64_t d = 0; d < Dv; d++) {
                        s += vj[d] * dx[d];          /* d_alpha_d = vt' * dx  */
                        dvj[d] += a[j] * g * dx[d];  /* dvt = dx * alpha_d'   */
                    }
                    if (dweights) s += dweights[j + Lkv * (i + Lq * (h + H * b))];
                    s *= g;                          /* pullback of alpha .* g */
                    da[j] = s;
                    dot += s * a[j];
                }
                for (int64_t j = 0; j < Lkv; j++) {
                    const double dl = da[j] * a[j] - a[j] * dot; /* _∇softmax! */
                    const double *kj = k + D * h + E * (j + Lkv * b);
                    double *dkj = dk + D * h + E * (j + Lkv * b);
                    if (dbias)
                        dbias[j * bias_strides[0] + i * bias_strides[1] + h * bias_strides[2] +
                              b * bias_strides[3]] += dl;
                    for (int64_t d = 0; d < D; d++) {
                        dkj[d] += dl * (qi[d] / sq);
                        dqi[d] += kj[d] * dl / sq;
                    }
                }
            }
    free(da);
}
