// Split-kv attention for a single query per (head, batch) ("decode" shape, Lq = 1), bf16 / f16 / Float32; calls with
// two to four queries (no weights, a mask only if it does not depend on the query) run through the same kernels
// with that many softmax states per wavefront (template parameter NQ).
//
// The work is a stream over K and V: every byte is read once and used once, so the kernel is
// organised around HBM, not around the matrix cores.  A kv row (all heads) is E contiguous elements;
// a wavefront owns a 1 KiB segment of the row (512 16-bit features: 4 heads at D = 128, 8 heads at D = 64; half as
// many in Float32), each lane one 16-byte load (8 or 4 consecutive features), and walks a contiguous range of kv
// rows.  The dot product over a head is finished with a butterfly over the lanes that share the head.
// Each (segment, kv-split, batch) wavefront keeps an online-softmax state (m, l, o[8]) and writes it
// to a workspace; a second small kernel merges the splits.
//
// Same arithmetic as the reference chain (src/attention.jl:112-127, fdrop = identity, no bias):
//   s_j = sum_d k[d,j] * q[d] / sqrt(D),  a = softmax_j(s),  x[d] = sum_j a_j v[d,j].
// An optional mask (src/attention.jl:133-138; with a single query every mask is a key mask, e.g. the context
// lengths of a padded batch) costs one byte per key row and head: dropped keys get the score -Inf, a (head,
// batch) pair with no key kept gives NaN like the reference.
// When the caller wants the attention weights too (the reference always returns them), the first kernel also writes
// the raw scores (Float32, 4 bytes per key and head: a few per mille of the K / V stream), the merge kernel leaves the
// final maximum and 1 / sum per (head, batch), and a third, elementwise kernel turns the scores into weights.
#include "common.h"
#include "attention_params.h"

namespace {

constexpr int ROWS = 8;        // kv rows in flight per lane and tensor
// features per lane (one 16-byte load) and per wavefront
template <typename T> constexpr int epl() { return 16 / (int)sizeof(typename T::type); }
template <typename T> constexpr int seg_width() { return 64 * epl<T>(); }

struct DecodeArgs {
    AttnParams p;
    float c;           // log2(e) / sqrt(D)
    int32_t nsplit;
    int32_t rows_per_split;
    int32_t nseg;      // ceil(E / 512)
    float *scores;     // weights requested: [B][H][Lkv] raw dot products (-Inf where masked), else null
    float *final_ml;   // weights requested: [B][H][2] final maximum (raw units) and 1 / sum
};

__device__ inline void unpack8(const u32x4_t &v, float *out, BF16) {
    const bf16x8_t h = __builtin_bit_cast(bf16x8_t, v);
#pragma unroll
    for (int e = 0; e < 8; e++) out[e] = (float)h[e];
}
__device__ inline void unpack8(const u32x4_t &v, float *out, F16) {
    const f16x8_t h = __builtin_bit_cast(f16x8_t, v);
#pragma unroll
    for (int e = 0; e < 8; e++) out[e] = (float)h[e];
}
__device__ inline void unpack8(const u32x4_t &v, float *out, F32) {   // four features
    const floatx4_t h = __builtin_bit_cast(floatx4_t, v);
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = h[e];
}

// workspace layout: [B][nsplit][E] floats of o, then [B][nsplit][H] of m, then [B][nsplit][H] of l
// NQ: queries of one batch element that a wavefront carries through the stream (1, 2 or 4).  A handful of queries
// against a long context (a few speculated tokens, a short chunk) is the same stream over K and V with NQ states: every
// K / V row is read once for all of them, where the tiled kernel reads head-dim-wide pieces of it per head.
template <typename T, int D, bool MASKED, bool SCORES, int NQ = 1>
__global__ __launch_bounds__(256) void decode_split_kernel(DecodeArgs a) {
    const AttnParams &p = a.p;
    typedef typename T::type t;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int EPL = epl<T>(), SEG = seg_width<T>(), LPH = D / EPL;   // features per lane and wavefront, lanes per head
    constexpr int NH = SEG / D;                        // heads per wavefront
    __shared__ float sc_lds[SCORES ? 4 * NH * 64 : 1]; // scores on their way out: [wavefront][head][64 keys]
    const int seg = blockIdx.x * 4 + wave;
    const int split = blockIdx.y;
    const int64_t ngroups = (p.Lq + NQ - 1) / NQ;      // groups of NQ queries per batch element
    const int64_t b = blockIdx.z / ngroups, q0 = (blockIdx.z % ngroups) * NQ;
    const int64_t f = (int64_t)seg * SEG + lane * EPL; // first feature of this lane
    const bool lane_ok = f < p.E;                      // E is a multiple of EPL (D is 64 or 128)
    if (seg >= a.nseg) return;

    const t *kb = (const t *)p.k + p.E * p.Lkv * b + (lane_ok ? f : 0);
    const t *vb = (const t *)p.v + p.E * p.Lkv * b + (lane_ok ? f : 0);
    float qf[NQ][EPL] = {};
#pragma unroll
    for (int n = 0; n < NQ; n++) {   // queries past Lq: copies of the last one, computed and not stored
        const int64_t qi = q0 + n < p.Lq ? q0 + n : p.Lq - 1;
        if (lane_ok) unpack8(*(const u32x4_t *)((const t *)p.q + p.E * (qi + p.Lq * b) + f), qf[n], T());
    }

    // Without the score output the splits take the 8-row blocks of the key range in turn (block t belongs to split
    // t mod nsplit) instead of one contiguous range each: the splits of a batch element run side by side, so at any
    // moment the chip reads one moving window of consecutive rows rather than nsplit separate streams (a plain read
    // of 8 GiB on this GPU: 6.97 TB/s with interleaved workgroups against 6.2-6.35 with a contiguous chunk per workgroup).
    // The online softmax does not depend on the order.  With scores the ranges stay contiguous: they leave in runs of
    // 64 consecutive keys.
    const bool interleave = !SCORES;
    const int64_t j_begin = interleave ? (int64_t)split * ROWS : (int64_t)split * a.rows_per_split;
    int64_t j_end = interleave ? p.Lkv : j_begin + a.rows_per_split;
    if (j_end > p.Lkv) j_end = p.Lkv;
    const int64_t j_step = interleave ? (int64_t)a.nsplit * ROWS : ROWS;

    float m[NQ], l[NQ], o[NQ][EPL] = {};
#pragma unroll
    for (int n = 0; n < NQ; n++) {
        m[n] = MI_NEG_INF;
        l[n] = 0.0f;
    }
    const u32x4_t zero = {0, 0, 0, 0};
    // mask bytes of this lane's head: element (kv, 0, h, b)
    const uint8_t *mrow = MASKED ? p.mask + (lane_ok ? f / D : 0) * p.mask_strides[2] + b * p.mask_strides[3] : nullptr;

    for (int64_t j = j_begin; j < j_end; j += j_step) {
        u32x4_t kr[ROWS], vr[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const bool ok = lane_ok && j + r < j_end;
            kr[r] = ok ? *(const u32x4_t *)(kb + p.E * (j + r)) : zero;
        }
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const bool ok = lane_ok && j + r < j_end;
            vr[r] = ok ? *(const u32x4_t *)(vb + p.E * (j + r)) : zero;
        }
        bool keep[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) keep[r] = j + r < j_end && (!MASKED || mrow[(j + r) * p.mask_strides[0]] != 0);
        float s[NQ][ROWS];
        float mx[NQ];
#pragma unroll
        for (int n = 0; n < NQ; n++) mx[n] = MI_NEG_INF;
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            float kf[EPL];
            unpack8(kr[r], kf, T());
#pragma unroll
            for (int n = 0; n < NQ; n++) {
                float d = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; e++) d = fmaf(kf[e], qf[n][e], d);
#pragma unroll
                for (int off = 1; off < LPH; off <<= 1) d += __shfl_xor(d, off, 64);
                s[n][r] = keep[r] ? d : MI_NEG_INF;
                mx[n] = fmaxf(mx[n], s[n][r]);
            }
        }
        float mref[NQ];
#pragma unroll
        for (int n = 0; n < NQ; n++) {
            const float mnew = fmaxf(m[n], mx[n]);            // finite without a mask: at least one row of the chunk is valid
            mref[n] = (MASKED && mnew == MI_NEG_INF) ? 0.0f : mnew;   // nothing kept so far: every term below is 0
            const float resc = mi_exp2((m[n] - mref[n]) * a.c);
            m[n] = mnew;
            l[n] *= resc;
#pragma unroll
            for (int e = 0; e < EPL; e++) o[n][e] *= resc;
        }
        // fused dropout (src/attention.jl:126 with fdrop = dropout; calls without returned weights, Lkv a multiple of 4):
        // the row sum takes the weight as the softmax gives it, the value product takes it times the keep factor of
        // weight (key, query, head, batch) in the shared counter stream.  A chunk starts at a multiple of 8 keys, so it
        // is two hash groups of four; the hashes hide under the K / V stream.
        float fac[NQ][ROWS];
#pragma unroll
        for (int n = 0; n < NQ; n++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) fac[n][r] = 1.0f;
        if (p.drop_thresh != 0) {
            const int64_t hd = lane_ok ? f / D : 0;
#pragma unroll
            for (int n = 0; n < NQ; n++) {
                const int64_t qi = q0 + n < p.Lq ? q0 + n : p.Lq - 1;
                const uint64_t i0 = (uint64_t)(j + p.Lkv * (qi + p.Lq * (hd + p.H * b)));
#pragma unroll
                for (int g = 0; g < ROWS / 4; g++) {
                    const uint64_t bits = mi_dropout_group_bits(p.drop_key, (i0 + 4 * g) >> 2);
#pragma unroll
                    for (int e = 0; e < 4; e++) fac[n][4 * g + e] = mi_dropout_keep_in(bits, e, p.drop_thresh) ? p.drop_scale : 0.0f;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            float vf[EPL];
            unpack8(vr[r], vf, T());
#pragma unroll
            for (int n = 0; n < NQ; n++) {
                const float pr = mi_exp2((s[n][r] - mref[n]) * a.c);
                l[n] += pr;
                const float pd = pr * fac[n][r];
#pragma unroll
                for (int e = 0; e < EPL; e++) o[n][e] = fmaf(pd, vf[e], o[n][e]);
            }
        }
        if (SCORES) {
            // Scores leave in runs of 64 keys per head (256 contiguous bytes): written 32 bytes at a time, one piece per
            // head and iteration, the scattered small writes cost the K / V stream a fifth of its rate.  The first lane
            // of each head parks the 8 scores of this iteration in the wavefront's LDS rows; every 8th iteration the
            // 64 lanes write one row per head.
            const int slot8 = (int)(((j - j_begin) / ROWS) & 7);
            if ((lane & (LPH - 1)) == 0) {
                float *row = sc_lds + (wave * NH + lane / LPH) * 64 + 8 * slot8;
                *(floatx4_t *)row = (floatx4_t){s[0][0], s[0][1], s[0][2], s[0][3]};
                *(floatx4_t *)(row + 4) = (floatx4_t){s[0][4], s[0][5], s[0][6], s[0][7]};
            }
            if (slot8 == 7 || j + ROWS >= j_end) {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const int64_t jrun = j - 8 * slot8;     // first key of the run
#pragma unroll
                for (int hl = 0; hl < NH; hl++) {
                    const int64_t h = (int64_t)seg * NH + hl;
                    const float val = sc_lds[(wave * NH + hl) * 64 + lane];
                    if (h < p.H && jrun + lane < j_end) a.scores[((int64_t)b * p.H + h) * p.Lkv + jrun + lane] = val;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
        }
    }
    if (!lane_ok) return;
    // partial results: one slot per (batch element, query, split); the merge kernel sees B * Lq batch elements
    float *ws = (float *)p.workspace;
    const int64_t nbq = p.B * p.Lq;
#pragma unroll
    for (int n = 0; n < NQ; n++) {
        if (q0 + n >= p.Lq) break;
        const int64_t slot = (b * p.Lq + q0 + n) * a.nsplit + split;
        float *wo = ws + slot * p.E + f;
        *(floatx4_t *)wo = (floatx4_t){o[n][0], o[n][1], o[n][2], o[n][3]};
        if constexpr (EPL == 8) *(floatx4_t *)(wo + 4) = (floatx4_t){o[n][4], o[n][5], o[n][6], o[n][7]};
        if ((lane & (LPH - 1)) == 0) {
            const int64_t h = f / D;
            float *wm = ws + nbq * a.nsplit * p.E;
            float *wl = wm + nbq * a.nsplit * p.H;
            wm[slot * p.H + h] = m[n];
            wl[slot * p.H + h] = l[n];
        }
    }
}

// Merge of the splits with the usual log-sum-exp rule.  One workgroup per (256 features, batch): the
// weights 2^(m_s - m) of every (head, split) pair are computed once into LDS, then each thread sums its
// feature over the splits, eight independent loads at a time.
template <typename T>
__global__ __launch_bounds__(256) void decode_merge_kernel(DecodeArgs a) {
    const AttnParams &p = a.p;
    __shared__ float wgt[4 * 1024];   // [heads of this workgroup <= 4][nsplit <= 1024]
    __shared__ float inv_l[4];
    const int64_t b = blockIdx.y;
    const int64_t f0 = (int64_t)blockIdx.x * 256, f = f0 + threadIdx.x;
    const float *ws = (const float *)p.workspace;
    const float *wm = ws + (int64_t)p.B * a.nsplit * p.E;
    const float *wl = wm + (int64_t)p.B * a.nsplit * p.H;
    const int64_t h0 = f0 / p.D;
    const int nh = (int)(256 / p.D);                 // 2 or 4 heads per workgroup
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave < nh && h0 + wave < p.H) {
        // one wavefront per head: maximum over the splits, then the weights and the total sum
        const int64_t h = h0 + wave;
        float m = MI_NEG_INF;
        for (int s = lane; s < a.nsplit; s += 64) m = fmaxf(m, wm[(b * a.nsplit + s) * p.H + h]);
        m = mi_wave_max(m);
        float l = 0.0f;
        for (int s = lane; s < a.nsplit; s += 64) {
            const int64_t slot = b * a.nsplit + s;
            const float w = mi_exp2((wm[slot * p.H + h] - m) * a.c);
            wgt[wave * 1024 + s] = w;
            l = fmaf(wl[slot * p.H + h], w, l);
        }
        l = mi_wave_sum(l);
        if (lane == 0) {
            inv_l[wave] = 1.0f / l;
            if (a.final_ml) {   // a head belongs to exactly one workgroup of this kernel (256 is a multiple of the head dim)
                a.final_ml[(b * p.H + h) * 2] = m;
                a.final_ml[(b * p.H + h) * 2 + 1] = 1.0f / l;
            }
        }
    }
    __syncthreads();
    if (f >= p.E) return;
    const int hl = (int)(f / p.D - h0);
    const float *src = ws + b * a.nsplit * p.E + f;
    const float *w = wgt + hl * 1024;
    float o = 0.0f;
    int s = 0;
    for (; s + 8 <= a.nsplit; s += 8) {
        float x[8];
#pragma unroll
        for (int u = 0; u < 8; u++) x[u] = src[(int64_t)(s + u) * p.E];
#pragma unroll
        for (int u = 0; u < 8; u++) o = fmaf(x[u], w[s + u], o);
    }
    for (; s < a.nsplit; s++) o = fmaf(src[(int64_t)s * p.E], w[s], o);
    ((typename T::type *)p.out)[p.E * b + f] = T::from_f32(o * inv_l[hl]);
}

// weights[kv, 0, h, b] = 2^((s - m) c) / l from the saved scores; a (head, batch) pair with every key masked has
// s = m = -Inf and gets NaN, as the reference's softmax gives
template <typename TW>
__global__ __launch_bounds__(256) void decode_weights_kernel(DecodeArgs a, TW *weights) {
    const AttnParams &p = a.p;
    const int64_t hb = blockIdx.y, j = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const float m = a.final_ml[hb * 2], inv = a.final_ml[hb * 2 + 1];
    const float *src = a.scores + hb * p.Lkv;
    TW *dst = weights + hb * p.Lkv;
#pragma unroll
    for (int e = 0; e < 4; e++)
        if (j + e < p.Lkv) dst[j + e] = (TW)(mi_exp2((src[j + e] - m) * a.c) * inv);
}

// queries per wavefront: 1, 2, or 4 (three queries run as four)
int decode_nq(const AttnParams &p) { return p.Lq <= 1 ? 1 : p.Lq == 2 ? 2 : 4; }

int pick_nsplit(const AttnParams &p) {
    // enough wavefronts to cover the chip several times over, at least 256 rows per split
    const int64_t SEG = p.dtype == MI_F32 ? seg_width<F32>() : seg_width<BF16>();
    const int64_t nseg = (p.E + SEG - 1) / SEG;
    const int64_t groups = p.B * ((p.Lq + decode_nq(p) - 1) / decode_nq(p));   // (batch element, query group) pairs
    int64_t want = 8192 / (nseg * groups > 0 ? nseg * groups : 1);   // (C5: 2048, 4096, 16384 ... 65536 wavefronts all measured slower)
    int64_t maxs = (p.Lkv + 255) / 256;
    if (want > maxs) want = maxs;
    if (want < 1) want = 1;
    if (want > 1024) want = 1024;
    return (int)want;
}

}  // namespace

bool attention_decode_supports(const AttnParams &p) {
    if (p.Lq < 1 || p.Lq > 4 || p.bias || p.causal || !p.out || p.stats) return false;   // saved statistics: the tiled kernels write them
    if (p.drop_thresh && (p.weights || (p.Lkv & 3) != 0)) return false;   // fused dropout: in the streaming kernel only, whole hash groups
    // two to four queries: without the weights, and with a mask only when it does not depend on the query
    if (p.Lq > 1 && (p.weights || (p.mask && p.mask_strides[1] != 0) || p.B * p.Lq > 65535)) return false;
    if (p.weights && p.H * p.B > 65535) return false;
    if (p.D != p.Dv || (p.D != 64 && p.D != 128)) return false;
    if (p.Lkv < 512) return false;   // short contexts: the tiled kernel is fine
    if (p.B > 65535) return false;
    auto al = [](const void *x) { return (((uintptr_t)x) & 15) == 0; };
    return al(p.q) && al(p.k) && al(p.v);
}

size_t attention_decode_workspace(const AttnParams &p) {
    const size_t ns = (size_t)pick_nsplit(p);
    // partial results of the splits, then (weights requested) the raw scores and the final statistics
    return sizeof(float) * (ns * (size_t)(p.B * p.Lq) * (size_t)(p.E + 2 * p.H) + (p.weights ? (size_t)(p.Lkv * p.H * p.B + 2 * p.H * p.B) : 0));
}

int32_t launch_attention_decode(const AttnParams &p, hipStream_t st) {
    DecodeArgs a;
    a.p = p;
    a.c = MI_LOG2E / sqrtf((float)p.D);
    a.nsplit = pick_nsplit(p);
    a.rows_per_split = (int32_t)((p.Lkv + a.nsplit - 1) / a.nsplit);
    a.nsplit = (int32_t)((p.Lkv + a.rows_per_split - 1) / a.rows_per_split);  // no empty split
    const int64_t SEG = p.dtype == MI_F32 ? seg_width<F32>() : seg_width<BF16>();
    a.nseg = (int32_t)((p.E + SEG - 1) / SEG);
    if ((((uintptr_t)p.workspace) & 15) != 0)
        return mi_set_error(MI_EWORKSPACE, "decode workspace must be 16-byte aligned");
    a.scores = a.final_ml = nullptr;
    if (p.weights) {
        // placed after the partial results, which are sized for pick_nsplit() splits (never fewer than a.nsplit)
        a.scores = (float *)p.workspace + (size_t)pick_nsplit(p) * (size_t)p.B * (size_t)(p.E + 2 * p.H);
        a.final_ml = a.scores + p.Lkv * p.H * p.B;
    }
    const int nq = decode_nq(p);
    dim3 grid((unsigned)((a.nseg + 3) / 4), (unsigned)a.nsplit, (unsigned)(p.B * ((p.Lq + nq - 1) / nq)));
    dim3 mgrid((unsigned)((p.E + 255) / 256), (unsigned)(p.B * p.Lq));
    DecodeArgs am = a;      // the merge kernel takes every (batch element, query) pair for a batch element of its own:
    am.p.B = p.B * p.Lq;    // q and the output are (E, Lq, B) arrays, the partial results [B * Lq][split][...]
    am.p.Lq = 1;
#define DECODE_LAUNCH(TT, DD)                                                                                        \
    {                                                                                                                \
        if (p.weights) {                                                                                             \
            if (p.mask) hipLaunchKernelGGL((decode_split_kernel<TT, DD, true, true>), grid, dim3(256), 0, st, a);     \
            else hipLaunchKernelGGL((decode_split_kernel<TT, DD, false, true>), grid, dim3(256), 0, st, a);           \
        } else if (nq == 1) {                                                                                        \
            if (p.mask) hipLaunchKernelGGL((decode_split_kernel<TT, DD, true, false>), grid, dim3(256), 0, st, a);    \
            else hipLaunchKernelGGL((decode_split_kernel<TT, DD, false, false>), grid, dim3(256), 0, st, a);          \
        } else if (nq == 2) {                                                                                        \
            if (p.mask) hipLaunchKernelGGL((decode_split_kernel<TT, DD, true, false, 2>), grid, dim3(256), 0, st, a); \
            else hipLaunchKernelGGL((decode_split_kernel<TT, DD, false, false, 2>), grid, dim3(256), 0, st, a);       \
        } else {                                                                                                     \
            if (p.mask) hipLaunchKernelGGL((decode_split_kernel<TT, DD, true, false, 4>), grid, dim3(256), 0, st, a); \
            else hipLaunchKernelGGL((decode_split_kernel<TT, DD, false, false, 4>), grid, dim3(256), 0, st, a);       \
        }                                                                                                            \
    }
    if (p.dtype == MI_BF16) {
        if (p.D == 128) DECODE_LAUNCH(BF16, 128) else DECODE_LAUNCH(BF16, 64)
        MI_LAUNCH_CHECK();
        hipLaunchKernelGGL(decode_merge_kernel<BF16>, mgrid, dim3(256), 0, st, am);
    } else if (p.dtype == MI_F32) {
        if (p.D == 128) DECODE_LAUNCH(F32, 128) else DECODE_LAUNCH(F32, 64)
        MI_LAUNCH_CHECK();
        hipLaunchKernelGGL(decode_merge_kernel<F32>, mgrid, dim3(256), 0, st, am);
    } else {
        if (p.D == 128) DECODE_LAUNCH(F16, 128) else DECODE_LAUNCH(F16, 64)
        MI_LAUNCH_CHECK();
        hipLaunchKernelGGL(decode_merge_kernel<F16>, mgrid, dim3(256), 0, st, am);
    }
#undef DECODE_LAUNCH
    MI_LAUNCH_CHECK();
    if (p.weights) {
        dim3 wgrid((unsigned)((p.Lkv + 1023) / 1024), (unsigned)(p.H * p.B));
        if (p.weights_dtype == MI_F32) hipLaunchKernelGGL(decode_weights_kernel<float>, wgrid, dim3(256), 0, st, a, (float *)p.weights);
        else if (p.dtype == MI_BF16) hipLaunchKernelGGL(decode_weights_kernel<__bf16>, wgrid, dim3(256), 0, st, a, (__bf16 *)p.weights);
        else hipLaunchKernelGGL(decode_weights_kernel<_Float16>, wgrid, dim3(256), 0, st, a, (_Float16 *)p.weights);
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}
