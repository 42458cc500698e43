// Pieces shared by the MFMA flash-attention kernels (16-bit and fp32 inputs): launch arguments and
// the per-tile "scale, bias, mask, online softmax, optional weight write-out" step, which works on
// S^T accumulators in the 32x32 MFMA layout and is therefore independent of the input precision.
//
// Accumulator layout (verified on hardware): register v of lane l of a 32x32 block holds
//   key row 8*(v/4) + 4*(l/32) + v%4, query column l%32.
#pragma once
#include "common.h"
#include "attention_params.h"

constexpr int FLASH_BN = 64;  // keys per tile

struct FlashArgs {
    AttnParams p;
    float c;           // log2(e) / sqrt(D)
    int32_t n_qtiles;
    int32_t bias_vec;  // bias rows may be read 4 keys at a time
    int32_t mask_vec;
    int32_t w_vec;     // weight rows may be written 4 keys at a time
    int32_t nsplit;    // key range is cut into this many pieces, one workgroup each (1 = no split)
    int32_t tiles_per_split;
};

// Split-kv bookkeeping shared by the planner (workspace size) and the launchers.
// Partials live in the caller's workspace: o as [split][B][Lq][Ev] floats, then (m, l) as
// [split][B][H][Lq][2] floats, m in log2 units.
inline int flash_pick_nsplit(const AttnParams &p, int bm) {
    if (p.weights || !p.out) return 1;                      // weights need the global maximum up front
    const int64_t wgs = ((p.Lq + bm - 1) / bm) * p.H * p.B;
    if (wgs >= 512 || p.Lkv < 2048) return 1;
    int64_t n = (1024 + wgs - 1) / wgs;
    const int64_t max_by_len = p.Lkv / 512;                 // at least 512 keys per piece
    if (n > max_by_len) n = max_by_len;
    if (n > 64) n = 64;
    return n < 1 ? 1 : (int)n;
}
inline size_t flash_split_workspace(const AttnParams &p, int nsplit) {
    if (nsplit <= 1) return 0;
    return sizeof(float) * (size_t)nsplit * (size_t)p.B * (size_t)p.Lq * (size_t)(p.Ev + 2 * p.H);
}
int32_t launch_flash_merge(const AttnParams &p, int nsplit, hipStream_t st);

enum { PHASE_ONLINE = 0, PHASE_STATS = 1, PHASE_FINAL = 2 };

inline void flash_fill_vec_flags(FlashArgs &a) {
    const AttnParams &p = a.p;
    auto mult4 = [](int64_t x) { return (x & 3) == 0; };
    const size_t es = mi_dtype_size(p.dtype);
    a.bias_vec = p.bias && p.bias_strides[0] == 1 && mult4(p.bias_strides[1]) && mult4(p.bias_strides[2]) &&
                 mult4(p.bias_strides[3]) && mult4(p.Lkv) && (((uintptr_t)p.bias) & (4 * es - 1)) == 0;
    a.mask_vec = p.mask && p.mask_strides[0] == 1 && mult4(p.mask_strides[1]) && mult4(p.mask_strides[2]) &&
                 mult4(p.mask_strides[3]) && mult4(p.Lkv) && (((uintptr_t)p.mask) & 3) == 0;
    a.w_vec = p.weights && mult4(p.Lkv) && (((uintptr_t)p.weights) & 15) == 0;
}

// On entry s[qb][kb] holds raw dot products k.q of tile rows [j0, j0+64) for the wavefront's query
// blocks; on exit it holds exp2(x - m) (ONLINE / STATS) or the final normalised weights (FINAL),
// with m, l (and, ONLINE only, the output accumulators o) updated.
//   T      element traits of the bias array
//   NDV    number of 32-row blocks of the output accumulator
template <typename T, int QB, int NDV, bool CAUSAL, bool EXTRAS, int PHASE, typename TW>
__device__ inline void flash_softmax_tile(const FlashArgs &a, floatx16_t (&s)[QB][2], floatx16_t (&o)[QB][NDV],
                                          float (&fm)[QB], float (&fl)[QB], int64_t b, int64_t h, int64_t iw,
                                          int64_t j0) {
    const AttnParams &p = a.p;
    typedef typename T::type elem_t;
    constexpr int BN = FLASH_BN;
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;
    const bool edge = (j0 + BN > p.Lkv) || (CAUSAL && j0 + BN - 1 > iw);
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
        const int64_t qi = iw + 32 * qb + r;
        const bool qok = qi < p.Lq;
        // ---- scale, bias, mask: x = log2(e) * (reference logit) --------------------------------
        if (EXTRAS) {
            const elem_t *bias = (const elem_t *)p.bias;
            const int64_t boff = qi * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3];
            const int64_t moff = qi * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3];
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int64_t kv = j0 + 32 * kb + 8 * g + 4 * hh;
                    float bv[4] = {0.f, 0.f, 0.f, 0.f};
                    bool keep[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) keep[e] = kv + e < p.Lkv && (!CAUSAL || kv + e <= qi);
                    if (bias && qok) {
                        if (a.bias_vec) {
                            if (kv < p.Lkv) {
                                typename T::vec4 t4 = *(const typename T::vec4 *)(bias + boff + kv);
#pragma unroll
                                for (int e = 0; e < 4; e++) bv[e] = T::to_f32(t4[e]);
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (kv + e < p.Lkv) bv[e] = T::to_f32(bias[boff + (kv + e) * p.bias_strides[0]]);
                        }
                    }
                    if (p.mask && qok) {
                        if (a.mask_vec) {
                            if (kv < p.Lkv) {
                                uint32_t m4 = *(const uint32_t *)(p.mask + moff + kv);
#pragma unroll
                                for (int e = 0; e < 4; e++) keep[e] = keep[e] && ((m4 >> (8 * e)) & 0xFF);
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (kv + e < p.Lkv) keep[e] = keep[e] && p.mask[moff + (kv + e) * p.mask_strides[0]];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float x = fmaf(s[qb][kb][4 * g + e], a.c, bv[e] * MI_LOG2E);
                        s[qb][kb][4 * g + e] = keep[e] ? x : MI_NEG_INF;
                    }
                }
        } else if (edge) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int64_t kv = j0 + 32 * kb + 8 * (v / 4) + 4 * hh + (v % 4);
                    const bool keep = kv < p.Lkv && (!CAUSAL || kv <= qi);
                    s[qb][kb][v] = keep ? s[qb][kb][v] : MI_NEG_INF;
                }
        }
        // Without EXTRAS the accumulators still hold raw dot products; the positive factor c is
        // folded into the exponent below (max commutes with a positive scale).
        const float cs = EXTRAS ? 1.0f : a.c;

        float pmul = 1.0f, msafe;
        if (PHASE != PHASE_FINAL) {
            float mx = MI_NEG_INF;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int v = 0; v < 16; v++) mx = fmaxf(mx, s[qb][kb][v]);
            mx = fmaxf(mx, mi_swap32(mx));
            const float mold = fm[qb];
            const float mnew = fmaxf(mold, mx);
            msafe = mnew == MI_NEG_INF ? 0.0f : mnew;
            float resc = mi_exp2((mold - msafe) * cs);
            if (EXTRAS && mold == mnew) resc = 1.0f;  // also covers +Inf == +Inf
            fm[qb] = mnew;
            fl[qb] *= resc;
            if (PHASE == PHASE_ONLINE) {
#pragma unroll
                for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
                    for (int v = 0; v < 16; v++) o[qb][dvb][v] *= resc;
            }
        } else {
            msafe = fm[qb] == MI_NEG_INF ? 0.0f : fm[qb];
            pmul = fl[qb];  // holds 1 / (row sum) in the final phase
        }
        const float moff2 = -msafe * cs;
        float lsum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float x = s[qb][kb][v];
                float e = mi_exp2(fmaf(x, cs, moff2));
                if (EXTRAS) e = (x == MI_POS_INF) ? 1.0f : e;  // src/softmax.jl:74-75
                if (PHASE == PHASE_FINAL) e *= pmul;
                lsum += e;
                s[qb][kb][v] = e;
            }
        if (PHASE != PHASE_FINAL) fl[qb] += lsum;

        if (PHASE == PHASE_FINAL && p.weights && qok) {
            TW *w = (TW *)p.weights + p.Lkv * (qi + p.Lq * (h + p.H * b));
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int64_t kv = j0 + 32 * kb + 8 * g + 4 * hh;
                    if (a.w_vec) {
                        if (kv < p.Lkv) {
                            typedef TW tw4 __attribute__((ext_vector_type(4)));
                            tw4 t4;
#pragma unroll
                            for (int e = 0; e < 4; e++) t4[e] = (TW)s[qb][kb][4 * g + e];
                            *(tw4 *)(w + kv) = t4;
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (kv + e < p.Lkv) w[kv + e] = (TW)s[qb][kb][4 * g + e];
                    }
                }
        }
    }
}

// Causal calls that return weights: keys after the last tile a wavefront visited are all dropped for
// its queries; their weights are exact zeros, which still have to be written.
template <int QB, typename TW>
__device__ inline void flash_zero_skipped_weights(const FlashArgs &a, int64_t b, int64_t h, int64_t iw, int n_tiles) {
    const AttnParams &p = a.p;
    constexpr int BN = FLASH_BN;
    const int lane = threadIdx.x & 63;
    int64_t kcov = ((iw + 32 * QB - 1) / BN + 1) * BN;
    if (kcov > (int64_t)n_tiles * BN) kcov = (int64_t)n_tiles * BN;
    for (int row = 0; row < 32 * QB; row++) {
        const int64_t qi = iw + row;
        if (qi >= p.Lq) break;
        TW *w = (TW *)p.weights + p.Lkv * (qi + p.Lq * (h + p.H * b));
        for (int64_t kv = kcov + lane; kv < p.Lkv; kv += 64) w[kv] = (TW)0.0f;
    }
}
