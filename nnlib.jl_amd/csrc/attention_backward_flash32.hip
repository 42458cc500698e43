// Attention backward for Float32 inputs on the fp32 matrix cores (v_mfma_f32_32x32x2_f32), head dim 64
// or 128.  Same decomposition as the 16-bit kernels in attention_backward_flash16.inc (the chain AD
// builds from src/attention.jl:86-127 through the rrule of batched_mul, src/batched/batchedmul.jl:96-110,
// and _∇softmax!, src/softmax.jl:107-110):
//
//   kernel 1 (query tile stationary): row statistics (saved by the forward call, or a first pass over
//            the keys), then dQ^T += K^T dS^T; statistics and delta go to the workspace
//   kernel 2 (key tile stationary): S = Q K^T, dP = dO V^T against streamed query tiles,
//            dV^T += dO^T P, dK^T += Q^T dS; for head dim 64 without bias / mask arrays it runs as a
//            dV kernel and a dK kernel at two wavefronts per SIMD
//
// With one fp32 per register nothing is converted or transposed: the streamed tile is the A operand of
// the first products through 16-byte LDS reads (contraction index permuted as in attention_flash32.hip:
// k-step 4c+j of half-wave hh multiplies feature 8c + 4hh + j), the accumulator registers of P / dS are
// the B operand of the second products as they stand, and the A operand of those is a plain 4-byte read
// of tile[row][feature = lane].  Products and sums are true fp32.
//
// Calls without bias / mask arrays and without dropout run their products on the 16-bit matrix cores instead, through
// three bf16 planes per operand (bwd32s_* below: Float32 accuracy at 2.7x less matrix-pipe time), unless
// MI355ATTN_F32_MFMA=1 in the environment asks for the Float32 instruction, as in the forward kernel.
#include "flash_common.h"
#include <cstdlib>

namespace {

typedef F32 T;
constexpr int BN = FLASH_BN;   // rows per streamed tile

template <int D>
struct Cfg {
    static constexpr int KS = D + 4;                    // tile row stride (floats): conflict-free 16-byte row reads
    static constexpr int TILEF = BN * KS;               // floats per tile
    static constexpr int CHUNKS = BN * D / 4 / 256;     // 16-byte chunks per thread, tile and tensor
    static constexpr int NDV = D / 32;
    static constexpr size_t SMEM = sizeof(float) * (4 * TILEF + 2 * 3 * BN);   // two tensors + statistics, double buffered
};

__device__ inline floatx4_t ldg16f(const float *p, bool ok) {
    return mi_load16_or_zero<floatx4_t>(p, ok);
}

// Streams [BN][D] tiles of up to two row-major arrays through registers into double-buffered LDS tiles;
// rows from `nrows` on and feature chunks from the head dim `dh` on (D is the tile width) read as zeros.
template <int D>
struct TileStream32 {
    static constexpr int KS = Cfg<D>::KS, CHUNKS = Cfg<D>::CHUNKS;
    const float *base1, *base2;   // base2 may be null
    int64_t stride, nrows;
    int dh;
    float *s1, *s2;
    floatx4_t r1[CHUNKS], r2[CHUNKS];
    __device__ void load(int64_t row0) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = threadIdx.x + 256 * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            const bool ok = row0 + row < nrows && col < dh;
            r1[u] = ldg16f(base1 + stride * (row0 + row) + col, ok);
            if (base2) r2[u] = ldg16f(base2 + stride * (row0 + row) + col, ok);
        }
    }
    __device__ void store(int buf) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = threadIdx.x + 256 * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            *(floatx4_t *)(s1 + (buf * BN + row) * KS + col) = r1[u];
            if (base2) *(floatx4_t *)(s2 + (buf * BN + row) * KS + col) = r2[u];
        }
    }
};

// acc += tile rows [32kb, 32kb+32) (A operand) x stationary rows x (B operand), contraction over D
template <int D>
__device__ inline floatx16_t first_product(const float *tile, int kb, const float (&x)[D / 2], floatx16_t acc, int r, int hh) {
    const float *t = tile + (32 * kb + r) * Cfg<D>::KS + 4 * hh;
#pragma unroll
    for (int c = 0; c < D / 8; c++) {
        const floatx4_t k4 = *(const floatx4_t *)(t + 8 * c);
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(k4[j], x[4 * c + j], acc, 0, 0, 0);
    }
    return acc;
}

// out[dvb] += tile^T (features x rows of block kb) x w (rows x stationary): register v of w belongs to tile row
// 32kb + 8(v/4) + 4hh + v%4, which is also the contraction index the MFMA assigns to this half-wave
template <int D>
__device__ inline void second_product(const float *tile, int kb, const floatx16_t &w, floatx16_t (&out)[D / 32], int r, int hh) {
    const float *t = tile + (32 * kb + 4 * hh) * Cfg<D>::KS + r;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const float *src = t + (8 * (v / 4) + (v % 4)) * Cfg<D>::KS;
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++) out[dvb] = __builtin_amdgcn_mfma_f32_32x32x2f32(src[32 * dvb], w[v], out[dvb], 0, 0, 0);
    }
}

// stationary row in the permuted feature order of first_product
template <int D>
__device__ inline void load_stationary(float (&x)[D / 2], const float *row, bool ok, int hh, int dh) {
    floatx4_t q4[D / 8];   // every load of the row is issued before the first is used
#pragma unroll
    for (int c = 0; c < D / 8; c++) q4[c] = ldg16f(row + 8 * c + 4 * hh, ok && 8 * c + 4 * hh < dh);
#pragma unroll
    for (int c = 0; c < D / 8; c++)
#pragma unroll
        for (int j = 0; j < 4; j++) x[4 * c + j] = q4[c][j];
}

__device__ inline int64_t lq_pad(int64_t Lq) { return attention_stats_lq_pad(Lq); }

// ---- kernel 1: statistics and dQ --------------------------------------------------------------------
// DROP (per-element paths only): the forward call dropped weights; the kernels redraw the factor g.
template <int D, bool CAUSAL, int EXTRAS, bool HAVE_STATS, bool DROP = false>
__global__ __launch_bounds__(256, (D == 64 && EXTRAS == EXTRAS_NONE) ? 2 : 1) void bwd32_dq_kernel(FlashArgs a, AttnBwdParams bp) {
    constexpr int TILEF = Cfg<D>::TILEF, NDV = Cfg<D>::NDV;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    float *Ks = (float *)bwd_smem, *Vs = Ks + 2 * TILEF;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * a.nb;   // this launch's batch elements: [a.b0, a.b0 + a.nb)
    const int split = (int)(blockIdx.x % a.nsplit);   // piece of the key range (a.nsplit > 1: calls with saved statistics only)
    const int64_t bid = blockIdx.x / a.nsplit;
    const int64_t hb = bid % HB, qt = a.n_qtiles - 1 - bid / HB;
    const int64_t h = hb % p.H, b = a.b0 + hb / p.H;
    const int64_t i0 = qt * 128, iw = i0 + 32 * wave, qi = iw + r;
    const bool qok = qi < p.Lq;

    float qx[D / 2], dox[D / 2];
    float delta = 0.0f;
    {
        const int64_t off = p.E * (qi + p.Lq * b) + p.D * h;   // E == Ev for these kernels
        load_stationary<D>(qx, (const float *)p.q + off, qok, hh, (int)p.D);
        load_stationary<D>(dox, (const float *)bp.dout + off, qok, hh, (int)p.D);
        float ox[D / 2];
        load_stationary<D>(ox, (const float *)p.out + off, qok, hh, (int)p.D);
#pragma unroll
        for (int e = 0; e < D / 2; e++) delta = fmaf(ox[e], dox[e], delta);
        delta += mi_swap32(delta);
    }

    // Key-padding masks measured on the device (FlashArgs::kv_len): a (head, batch) pair whose mask keeps a prefix of
    // the keys is an unmasked problem with that many keys (the kernels without mask code take it and leave the other
    // pairs to the kernels with it, which are launched as well)
    int64_t kv_len = p.Lkv;
    if (a.kv_len) {
        const int64_t len = a.kv_len[b * p.H + h];
        if ((EXTRAS == EXTRAS_NONE) == (len == 0)) return;
        if (EXTRAS == EXTRAS_NONE) kv_len = len;
    }
    int64_t kv_end = kv_len;
    if (CAUSAL && i0 + 128 < kv_end) kv_end = i0 + 128;
    const int n_tiles = (int)((kv_end + BN - 1) / BN);

    TileStream32<D> ts;
    ts.base1 = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    ts.dh = (int)p.D;
    ts.stride = p.E;
    ts.nrows = kv_len;
    ts.s1 = Ks;
    ts.s2 = Vs;
    floatx16_t unused_o[1][NDV];
    float fm[1] = {MI_NEG_INF}, fl[1] = {0.0f};
    const float cs = EXTRAS ? MI_LOG2E : a.c;
    const int64_t plane = p.B * p.H * lq_pad(p.Lq), at = (b * p.H + h) * lq_pad(p.Lq) + qi;
    if (HAVE_STATS) {
        fm[0] = bp.stats[at] / cs;
        fl[0] = bp.stats[plane + at];
        if (hh == 0) bp.stats[2 * plane + at] = qok ? delta : 0.0f;
    }

    // pass 1: row maximum and row sum (K tiles only)
    ts.base2 = nullptr;
    if (!HAVE_STATS) {
        ts.load(0);
        ts.store(0);
    }
    __syncthreads();
    for (int jt = 0; !HAVE_STATS && jt < n_tiles; jt++) {
        const int buf = jt & 1;
        const int64_t j0 = (int64_t)jt * BN;
        if (jt + 1 < n_tiles) ts.load(j0 + BN);
        if (!CAUSAL || j0 <= iw + 31) {
            floatx16_t s[1][2] = {{(floatx16_t){0}, (floatx16_t){0}}};
#pragma unroll
            for (int kb = 0; kb < 2; kb++) s[0][kb] = first_product<D>(Ks + buf * TILEF, kb, qx, s[0][kb], r, hh);
            flash_softmax_tile<T, 1, NDV, CAUSAL, EXTRAS, PHASE_STATS, float>(a, s, unused_o, fm, fl, b, h, iw, j0, FlashStaged<1>(), 0, 0, nullptr,
                                                                              kv_len);
        }
        if (jt + 1 < n_tiles) ts.store(buf ^ 1);
        __syncthreads();
    }
    if (!HAVE_STATS) {
        fl[0] = 1.0f / (fl[0] + mi_swap32(fl[0]));   // all keys dropped: 1/0 = Inf, the weights become 0*Inf = NaN
        if (hh == 0) {
            // rows past Lq belong to the padding of the last tile: statistics that make their weights zero
            bp.stats[at] = qok ? fm[0] * cs : 0.0f;
            bp.stats[plane + at] = qok ? fl[0] : 0.0f;
            bp.stats[2 * plane + at] = qok ? delta : 0.0f;
        }
    }
    if (!bp.dq && !bp.dbias) return;

    // pass 2: P, dP = V dO^T, dS = P (dP - delta), dQ^T += K^T dS^T
    const unsigned dbias_lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)bwd_smem + (unsigned)Cfg<D>::SMEM + wave * FLASH_WSTAGE_BYTES;
    floatx16_t dq[NDV];
#pragma unroll
    for (int dvb = 0; dvb < NDV; dvb++) dq[dvb] = (floatx16_t){0};
    ts.base2 = (const float *)p.v + p.Ev * (p.Lkv * b) + p.D * h;
    int jt0 = 0, jt1 = n_tiles;
    if (a.nsplit > 1) {
        jt0 = split * a.tiles_per_split;
        if (jt0 + a.tiles_per_split < jt1) jt1 = jt0 + a.tiles_per_split;
    }
    ts.load((int64_t)jt0 * BN);
    __syncthreads();   // pass 1 may still be reading the tiles
    ts.store(0);
    __syncthreads();
    const float m2 = fm[0] * cs, linv = fl[0];
    for (int jt = jt0; jt < jt1; jt++) {
        const int buf = (jt - jt0) & 1;
        const int64_t j0 = (int64_t)jt * BN;
        if (jt + 1 < jt1) ts.load(j0 + BN);
        if (!CAUSAL || j0 <= iw + 31) {
            const float *kt = Ks + buf * TILEF, *vt = Vs + buf * TILEF;
            if constexpr (EXTRAS == EXTRAS_NONE) {
                const bool edge = (j0 + BN > kv_len) || (CAUSAL && j0 + BN - 1 > iw);
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
                    if (CAUSAL && j0 + 32 * kb > iw + 31) break;   // every key of this block is after every query of the wavefront
                    floatx16_t sb = first_product<D>(kt, kb, qx, (floatx16_t){0}, r, hh);
                    const floatx16_t dpb = first_product<D>(vt, kb, dox, (floatx16_t){0}, r, hh);
                    int lim = BN;   // keys of the tile this lane's query keeps, counted from the lane's first key of a group of four
                    if (edge) {
                        int64_t lim64 = kv_len - j0;
                        if (CAUSAL && qi - j0 + 1 < lim64) lim64 = qi - j0 + 1;
                        lim = (lim64 > BN ? BN : (lim64 < 0 ? 0 : (int)lim64)) - 4 * hh;
                    }
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int kvl = 32 * kb + 8 * (v / 4) + (v % 4);
                        const float pw = (!edge || kvl < lim) ? mi_exp2(fmaf(sb[v], cs, -m2)) * linv : 0.0f;
                        sb[v] = pw * (dpb[v] - delta);
                    }
                    second_product<D>(kt, kb, sb, dq, r, hh);
                }
            } else {
                floatx16_t s[1][2] = {{(floatx16_t){0}, (floatx16_t){0}}};
                floatx16_t dp[2];
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
                    s[0][kb] = first_product<D>(kt, kb, qx, s[0][kb], r, hh);
                    dp[kb] = first_product<D>(vt, kb, dox, (floatx16_t){0}, r, hh);
                }
                flash_softmax_tile<T, 1, NDV, CAUSAL, EXTRAS, PHASE_FINAL, float>(a, s, unused_o, fm, fl, b, h, iw, j0);
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
                    if (DROP) {
                        // fused dropout: the forward multiplied the weight by g (0 or 1/(1-p)), its pullback multiplies dP
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            float gf[4];
                            attention_drop_factors_run4<false>(bp.p, (uint64_t)(p.Lkv * (qi + p.Lq * (h + p.H * b)) + 4 * hh + j0 + 32 * kb), g, gf);
#pragma unroll
                            for (int e = 0; e < 4; e++) dp[kb][4 * g + e] *= gf[e];
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; v++) s[0][kb][v] *= dp[kb][v] - delta;
                if (bp.dbias) {
                        // the bias adds to the logits, so its gradient is dS, summed over the dimensions it broadcasts
                        // along (stride 0): Float32 atomics, one per weight that is not an exact zero
                        float *db = bp.dbias + h * p.bias_strides[2] + b * p.bias_strides[3];
                        const int64_t kv0 = j0 + 32 * kb;
                        if (p.bias_strides[0] == 1) {
                            const int64_t nq = p.Lq - iw, nk = p.Lkv - kv0;
                            flash_atomic_add_block(dbias_lds, s[0][kb], db + kv0 + iw * p.bias_strides[1], p.bias_strides[1],
                                                   (int)(nq > 32 ? 32 : nq), (int)(nk > 32 ? 32 : (nk < 0 ? 0 : nk)), a.dbias_plain != 0);
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; v++) {
                                const int64_t kvv = kv0 + 8 * (v / 4) + 4 * hh + (v % 4);
                                if (qok && kvv < p.Lkv && s[0][kb][v] != 0.0f)
                                    atomicAdd(db + qi * p.bias_strides[1] + kvv * p.bias_strides[0], s[0][kb][v]);
                            }
                        }
                    }
                    second_product<D>(kt, kb, s[0][kb], dq, r, hh);
                }
            }
        }
        if (jt + 1 < n_tiles) ts.store(buf ^ 1);
        __syncthreads();
    }
    if (qok && bp.dq) {
        // one piece of the key range (a.nsplit > 1): its share of dQ goes to the workspace for the merge kernel
        float *dqrow = a.nsplit > 1 ? bp.dq_partial + ((int64_t)split * p.B * p.Lq + qi + p.Lq * b) * p.E + p.D * h
                                    : (float *)bp.dq + p.E * (qi + p.Lq * b) + p.D * h;
#pragma unroll
        for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                floatx4_t o4;
#pragma unroll
                for (int e = 0; e < 4; e++) o4[e] = dq[dvb][4 * g + e] * a.cn;
                if (32 * dvb + 8 * g + 4 * hh < p.D) *(floatx4_t *)(dqrow + 32 * dvb + 8 * g + 4 * hh) = o4;
            }
    }
}

// ---- kernel 2: dK and dV ----------------------------------------------------------------------------
enum { BWD_DV = 1, BWD_DK = 2 };
template <int D, bool CAUSAL, int EXTRAS, int WHICH, bool DROP = false>
__global__ __launch_bounds__(256, (WHICH != 3 && D == 64 && EXTRAS == EXTRAS_NONE) ? 2 : 1) void bwd32_dkdv_kernel(FlashArgs a, AttnBwdParams bp) {
    constexpr int TILEF = Cfg<D>::TILEF, NDV = Cfg<D>::NDV;
    constexpr bool DO_DV = (WHICH & BWD_DV) != 0, DO_DK = (WHICH & BWD_DK) != 0;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    float *Qs = (float *)bwd_smem, *dOs = Qs + 2 * TILEF;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t hb = blockIdx.x % HB, kt_idx = blockIdx.x / HB;   // with causal masks the early key tiles are the long ones
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t j0 = kt_idx * 128, jw = j0 + 32 * wave, kv = jw + r;
    const bool kok = kv < p.Lkv;
    // context lengths (see the dQ kernel): keys from the pair's length on get zero gradients, and a workgroup whose
    // keys all lie there has nothing else to do
    int64_t kv_len = p.Lkv;
    if (a.kv_len) {
        const int64_t len = a.kv_len[b * p.H + h];
        if ((EXTRAS == EXTRAS_NONE) == (len == 0)) return;
        if (EXTRAS == EXTRAS_NONE) kv_len = len;
    }
    const bool kvalid = EXTRAS == EXTRAS_NONE ? kv < kv_len : kok;
    if (EXTRAS == EXTRAS_NONE && j0 >= kv_len) {
        if (kok) {
            const int64_t off = p.E * (kv + p.Lkv * b) + p.D * h;
            const floatx4_t z4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    if (32 * dvb + 8 * g + 4 * hh >= p.D) continue;
                    if (DO_DK && bp.dk) *(floatx4_t *)((float *)bp.dk + off + 32 * dvb + 8 * g + 4 * hh) = z4;
                    if (DO_DV && bp.dv) *(floatx4_t *)((float *)bp.dv + off + 32 * dvb + 8 * g + 4 * hh) = z4;
                }
        }
        return;
    }

    float kx[D / 2], vx[DO_DK ? D / 2 : 1];
    {
        const int64_t off = p.E * (kv + p.Lkv * b) + p.D * h;
        load_stationary<D>(kx, (const float *)p.k + off, kvalid, hh, (int)p.D);
        if constexpr (DO_DK) load_stationary<D>(vx, (const float *)p.v + off, kvalid, hh, (int)p.D);
    }
    floatx16_t dk[NDV], dv[NDV];
#pragma unroll
    for (int dvb = 0; dvb < NDV; dvb++) dk[dvb] = dv[dvb] = (floatx16_t){0};

    const int64_t plane = p.B * p.H * lq_pad(p.Lq);
    // the row statistics of a query tile travel with it through LDS (48 threads x 4 floats)
    const float *st_src = bp.stats + (b * p.H + h) * lq_pad(p.Lq) + (int64_t)(tid >> 4) * plane + 4 * (tid & 15);
    float *st_lds = (float *)bwd_smem + 4 * TILEF;
    floatx4_t st_reg = {0, 0, 0, 0};
    const float *bias = (const float *)p.bias;
    const int64_t boff = kv * p.bias_strides[0] + h * p.bias_strides[2] + b * p.bias_strides[3];
    const int64_t moff = kv * p.mask_strides[0] + h * p.mask_strides[2] + b * p.mask_strides[3];
    const float cs = EXTRAS ? MI_LOG2E : a.c;

    TileStream32<D> ts;
    ts.base1 = (const float *)p.q + p.E * (p.Lq * b) + p.D * h;
    ts.base2 = (const float *)bp.dout + p.E * (p.Lq * b) + p.D * h;
    ts.dh = (int)p.D;
    ts.stride = p.E;
    ts.nrows = p.Lq;
    ts.s1 = Qs;
    ts.s2 = dOs;
    const int n_qt = (int)((p.Lq + BN - 1) / BN);
    const int it0 = CAUSAL ? (int)(j0 / BN) : 0;   // query tiles before the first key of the workgroup see none of its keys
    if (it0 < n_qt) {
        ts.load((int64_t)it0 * BN);
        ts.store(0);
        if (tid < 48) *(floatx4_t *)(st_lds + 4 * tid) = *(const floatx4_t *)(st_src + (int64_t)it0 * BN);
    }
    __syncthreads();
    for (int it = it0; it < n_qt; it++) {
        const int buf = (it - it0) & 1;
        const int64_t i0 = (int64_t)it * BN;
        if (it + 1 < n_qt) {
            ts.load(i0 + BN);
            if (tid < 48) st_reg = *(const floatx4_t *)(st_src + i0 + BN);
        }
        if (!CAUSAL || i0 + BN - 1 >= jw) {
            const float *qt = Qs + buf * TILEF, *dot = dOs + buf * TILEF;
            const float *st = st_lds + buf * (3 * BN);
            const bool diag = CAUSAL && i0 < jw + 32;   // some (query, key) pair of this tile has key > query
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                floatx16_t s = first_product<D>(qt, kb, kx, (floatx16_t){0}, r, hh);
                floatx16_t dp = (floatx16_t){0};
                if constexpr (DO_DK) dp = first_product<D>(dot, kb, vx, dp, r, hh);
                // accumulator register 4g+e of this lane: query i0 + 32kb + 8g + 4hh + e, key kv
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int64_t qg = i0 + 32 * kb + 8 * g + 4 * hh;
                    const int sq = 32 * kb + 8 * g + 4 * hh;
                    const floatx4_t m4 = *(const floatx4_t *)(st + sq);
                    const floatx4_t linv4 = *(const floatx4_t *)(st + BN + sq);
                    floatx4_t delta4 = {0.0f, 0.0f, 0.0f, 0.0f};
                    if (DO_DK) delta4 = *(const floatx4_t *)(st + 2 * BN + sq);
                    if constexpr (EXTRAS == EXTRAS_NONE) {
                        // rows past Lq carry statistics (0, 0, 0): their weights vanish; keys past Lkv only feed
                        // accumulator columns that are never stored
                        const int dq_ = (int)(jw - qg) + r;   // key index minus query index of element e = 0
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            float pw = mi_exp2(fmaf(s[4 * g + e], cs, -m4[e])) * linv4[e];
                            if (diag) pw = dq_ - e > 0 ? 0.0f : pw;
                            s[4 * g + e] = pw;
                            if (DO_DK) dp[4 * g + e] = pw * (dp[4 * g + e] - delta4[e]);
                        }
                        continue;
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int64_t qi = qg + e;
                        const bool in = kok && qi < p.Lq;
                        float x = s[4 * g + e] * a.cn;
                        if (bias && in) x += bias[boff + qi * p.bias_strides[1]];
                        if (p.mask && in && !p.mask[moff + qi * p.mask_strides[1]]) x = MI_NEG_INF;
                        if (diag && kv > qi) x = MI_NEG_INF;
                        const float m = m4[e];
                        float pw;
                        if (m == MI_POS_INF) pw = x == MI_POS_INF ? linv4[e] : 0.0f;   // src/softmax.jl:74-75
                        else pw = mi_exp2(fmaf(x, cs, m == MI_NEG_INF ? 0.0f : -m)) * linv4[e];
                        pw = in ? pw : 0.0f;
                        // fused dropout: the value product saw pw * gd, and the pullback multiplies dP by gd
                        const float gd = DROP ? attention_drop_factor(bp.p, kv, qi, h, b) : 1.0f;
                        s[4 * g + e] = pw * gd;
                        if (DO_DK) dp[4 * g + e] = pw * (gd * dp[4 * g + e] - delta4[e]);
                    }
                }
                if constexpr (DO_DV) second_product<D>(dot, kb, s, dv, r, hh);
                if constexpr (DO_DK) second_product<D>(qt, kb, dp, dk, r, hh);
            }
        }
        if (it + 1 < n_qt) {
            ts.store(buf ^ 1);
            if (tid < 48) *(floatx4_t *)(st_lds + (buf ^ 1) * (3 * BN) + 4 * tid) = st_reg;
        }
        __syncthreads();
    }
    if (kok) {
        const int64_t off = p.E * (kv + p.Lkv * b) + p.D * h;
#pragma unroll
        for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if (32 * dvb + 8 * g + 4 * hh >= p.D) continue;
                floatx4_t k4, v4;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    k4[e] = (EXTRAS != EXTRAS_NONE || kvalid) ? dk[dvb][4 * g + e] * a.cn : 0.0f;
                    v4[e] = (EXTRAS != EXTRAS_NONE || kvalid) ? dv[dvb][4 * g + e] : 0.0f;
                }
                if (DO_DK && bp.dk) *(floatx4_t *)((float *)bp.dk + off + 32 * dvb + 8 * g + 4 * hh) = k4;
                if (DO_DV && bp.dv) *(floatx4_t *)((float *)bp.dv + off + 32 * dvb + 8 * g + 4 * hh) = v4;
            }
    }
}

// ---- the same kernels without bias / mask arrays or dropout, products on the 16-bit matrix cores ----
// Each Float32 product runs as six v_mfma_f32_32x32x16_bf16 over three bf16 planes per operand (the planes
// and their arithmetic: common.h; layout and reads of the plane tiles: run_tiles32s in attention_flash32.hip).
// Streamed tiles are split once when they are staged (one LDS tile per tensor, the next one waits in
// registers), the stationary rows once per workgroup, P and dS once per block in registers; the A operand of
// the second products comes from the same row-major planes through the transposing read.
// Keeps the compiler from hoisting one product's LDS operand reads across the previous phase of the step (head dim 64:
// left alone it holds dozens of operand registers in flight and spills the stationary planes; with the fences the
// 64-wide kernels run 3-13 % faster, the 128-wide ones, which have registers to spare, 5-20 % slower)
#define SCHED_FENCE() do { if (D == 64) __builtin_amdgcn_sched_barrier(0); } while (0)
typedef bf16x8_t plane8;
typedef bf16x4_t plane4;
typedef short s16x4_t __attribute__((ext_vector_type(4)));

template <int D>
struct CfgS {
    static constexpr int ROWB = D * 2;               // bytes per tile row of one plane
    static constexpr int PLANEB = BN * ROWB;         // one plane of one tile
    static constexpr int TILEB = 3 * PLANEB;         // hi, mid, lo
    static constexpr size_t SMEM = 2 * TILEB + sizeof(float) * 2 * 3 * BN;   // two tensors + statistics (double buffered)
    // chunk swizzle of the 16-bit kernels (conflict-free 16-byte operand reads and transposing reads)
    __device__ static inline int swz(int row) {
        if (D >= 128) return ((row & 3) << 2) | ((row >> 2) & 3);
        const int x = (row >> 1) & 7;
        return ((x & 1) << 2) | (x >> 1);
    }
};

__device__ inline floatx16_t mfma_bf16(plane8 a, plane8 b, floatx16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

// c += a b with a, b given as planes (small terms first)
__device__ inline floatx16_t mfma_split(const plane8 (&a)[3], const plane8 (&b)[3], floatx16_t c) {
    c = mfma_bf16(a[2], b[0], c);
    c = mfma_bf16(a[0], b[2], c);
    c = mfma_bf16(a[1], b[1], c);
    c = mfma_bf16(a[1], b[0], c);
    c = mfma_bf16(a[0], b[1], c);
    return mfma_bf16(a[0], b[0], c);
}

// TileStream32 with the split at the LDS store: one tile per tensor, as LDS byte addresses
template <int D, int NT = 256>
struct PlaneStream {
    typedef CfgS<D> C;
    static constexpr int CHUNKS = BN * D / 4 / NT;   // float4 pieces per thread, tile and tensor
    const float *base1, *base2;   // base2 may be null
    int64_t stride, nrows;
    int dh;
    unsigned s1, s2;
    floatx4_t r1[CHUNKS], r2[CHUNKS];
    __device__ void load(int64_t row0) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = threadIdx.x + NT * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            const bool ok = row0 + row < nrows && col < dh;
            r1[u] = ldg16f(base1 + stride * (row0 + row) + col, ok);
            if (base2) r2[u] = ldg16f(base2 + stride * (row0 + row) + col, ok);
        }
    }
    // four consecutive features of one row: 8 bytes in each of the three planes
    __device__ static void put(unsigned tile, int row, int col, const floatx4_t &x) {
        typedef __attribute__((address_space(3))) u32x2_t *lds8_t;
        uint32_t pl[3][2];
        const bool odd = split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        if (odd) {   // an Inf or NaN in the chunk (rare)
            split3_pair_guarded(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair_guarded(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        }
        const unsigned at = tile + (unsigned)row * C::ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
        for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * C::PLANEB) = (u32x2_t){pl[q][0], pl[q][1]};
    }
    __device__ void store() {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = threadIdx.x + NT * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            put(s1, row, col, r1[u]);
            if (base2) put(s2, row, col, r2[u]);
        }
    }
};

// first_product on plane tiles: the lane's A operand of k-step t is chunk 2t + hh of tile row 32kb + r in each plane
template <int D>
__device__ inline floatx16_t first_product_s(unsigned tile, int kb, const plane8 (&x)[3][D / 16], floatx16_t acc, int r, int hh) {
    typedef CfgS<D> C;
    typedef __attribute__((address_space(3))) const plane8 *lds_plane8_t;
    const unsigned t0 = tile + (unsigned)(32 * kb + r) * C::ROWB;
    const int sw = C::swz(r);
#pragma unroll
    for (int t = 0; t < D / 16; t++) {
        plane8 ta[3];
#pragma unroll
        for (int q = 0; q < 3; q++) ta[q] = *(lds_plane8_t)(uintptr_t)(t0 + q * C::PLANEB + (((2 * t + hh) ^ sw) << 4));
        const plane8 xb[3] = {x[0][t], x[1][t], x[2][t]};
        acc = mfma_split(ta, xb, acc);
    }
    return acc;
}

// first_product_s with the stationary planes in LDS as well ([3][rows][ROWB], chunks swizzled like a tile's): `xrow` is
// the byte address of the lane's row in the hi plane, XPLANEB the distance between planes
template <int D, int XPLANEB>
__device__ inline floatx16_t first_product_sl(unsigned tile, int kb, unsigned xrow, int xsw, floatx16_t acc, int r, int hh) {
    typedef CfgS<D> C;
    typedef __attribute__((address_space(3))) const plane8 *lds_plane8_t;
    const unsigned t0 = tile + (unsigned)(32 * kb + r) * C::ROWB;
    const int sw = C::swz(r);
#pragma unroll
    for (int t = 0; t < D / 16; t++) {
        plane8 ta[3], xb[3];
#pragma unroll
        for (int q = 0; q < 3; q++) {
            ta[q] = *(lds_plane8_t)(uintptr_t)(t0 + q * C::PLANEB + (((2 * t + hh) ^ sw) << 4));
            xb[q] = *(lds_plane8_t)(uintptr_t)(xrow + q * XPLANEB + (((2 * t + hh) ^ xsw) << 4));
        }
        acc = mfma_split(ta, xb, acc);
    }
    return acc;
}

// second_product on plane tiles: the B operand of k-step u is accumulator registers 8u .. 8u+7 of w (tile rows 0-3,
// 8-11 | 4-7, 12-15 of the 16), split in registers; tile^T comes through the transposing read in that row order
template <int D>
__device__ inline void second_product_s(unsigned tile, int kb, const floatx16_t &w, floatx16_t (&out)[D / 32], int lane) {
    typedef CfgS<D> C;
    const int hh = lane >> 5;
    const int vrow = 4 * hh + ((lane & 15) >> 2);
    const int vchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), vsub = 8 * (lane & 1);
    const unsigned vt = tile + (unsigned)vrow * C::ROWB + vsub;
    const int sw_lo = C::swz(vrow), sw_hi = C::swz(vrow + 8);
    auto tr = [](unsigned addr) {
        const s16x4_t x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t *)(uintptr_t)addr);
        return __builtin_bit_cast(plane4, x);
    };
#pragma unroll
    for (int u = 0; u < 2; u++) {
        uint32_t ww[3][4];
#pragma unroll
        for (int e = 0; e < 4; e++) split3_pair(w[8 * u + 2 * e], w[8 * u + 2 * e + 1], ww[0][e], ww[1][e], ww[2][e]);   // a NaN stays NaN in the hi plane
        plane8 wb[3];
#pragma unroll
        for (int q = 0; q < 3; q++) wb[q] = __builtin_bit_cast(plane8, (u32x4_t){ww[q][0], ww[q][1], ww[q][2], ww[q][3]});
        const unsigned src = vt + (unsigned)(32 * kb + 16 * u) * C::ROWB;
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++) {
            plane8 ta[3];
#pragma unroll
            for (int q = 0; q < 3; q++) {
                const plane4 lo = tr(src + q * C::PLANEB + (((4 * dvb + vchunk) ^ sw_lo) << 4));
                const plane4 hi = tr(src + q * C::PLANEB + 8 * C::ROWB + (((4 * dvb + vchunk) ^ sw_hi) << 4));
                ta[q] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
            out[dvb] = mfma_split(ta, wb, out[dvb]);
        }
    }
}

// stationary row as planes: the lane's features of k-step t are 16t + 8hh .. + 7 (the B-operand layout of the 16-bit instruction)
template <int D>
__device__ inline void load_stationary_s(plane8 (&x)[3][D / 16], const float *row, bool ok, int hh, int dh) {
    floatx4_t raw[D / 16][2];   // every load of the row is issued before the first is used: one memory round trip
#pragma unroll
    for (int t = 0; t < D / 16; t++)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int d0 = 16 * t + 8 * hh + 4 * half;
            raw[t][half] = ldg16f(row + d0, ok && d0 < dh);
        }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < D / 16; t++) {
        uint32_t xw[3][4];
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const floatx4_t q4 = raw[t][half];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint32_t w[3];
                if (split3_pair(q4[2 * j], q4[2 * j + 1], w[0], w[1], w[2])) split3_pair_guarded(q4[2 * j], q4[2 * j + 1], w[0], w[1], w[2]);
#pragma unroll
                for (int q = 0; q < 3; q++) xw[q][2 * half + j] = w[q];
            }
        }
#pragma unroll
        for (int q = 0; q < 3; q++) x[q][t] = __builtin_bit_cast(plane8, (u32x4_t){xw[q][0], xw[q][1], xw[q][2], xw[q][3]});
    }
}

template <int D, bool CAUSAL, bool HAVE_STATS, int NW>
// One workgroup per compute unit: the lane's Q and dO planes, dQ and the two score blocks need some 380 registers.
// NW = 4: everything in registers, one wavefront per SIMD; the next tile is fetched during the products where
// registers are left for it (head dim 64), before the barrier otherwise.  NW = 8 (head dim 64, 256 queries a
// workgroup): the dO planes live in LDS behind the tiles (each wavefront reads its own rows back as the B operand of
// dP), which brings a lane under 256 registers, i.e. two wavefronts per SIMD sharing one pair of tiles.
__global__ __launch_bounds__(64 * NW, 1) void bwd32s_dq_kernel(FlashArgs a, AttnBwdParams bp) {
    typedef CfgS<D> C;
    constexpr int NDV = D / 32, NT = 64 * NW;
    constexpr bool X_LDS = NW == 8;
    constexpr bool AHEAD = D == 64 && !X_LDS;
    constexpr int XPLANEB = 32 * NW * C::ROWB;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    const unsigned Ks = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)bwd_smem, Vs = Ks + C::TILEB;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * a.nb;
    const int split = (int)(blockIdx.x % a.nsplit);   // piece of the key range (a.nsplit > 1: calls with saved statistics only)
    const int64_t bid = blockIdx.x / a.nsplit;
    const int64_t hb = bid % HB, qt = a.n_qtiles - 1 - bid / HB;
    const int64_t h = hb % p.H, b = a.b0 + hb / p.H;
    const int64_t i0 = qt * (32 * NW), iw = i0 + 32 * wave, qi = iw + r;
    const bool qok = qi < p.Lq;

    int64_t kv_len = p.Lkv;
    if (a.kv_len) {   // context lengths: pairs without one belong to the kernels with mask code
        kv_len = a.kv_len[b * p.H + h];
        if (kv_len == 0) return;
    }

    plane8 qx[3][D / 16], dox[X_LDS ? 1 : 3][D / 16];
    const unsigned xrow = Ks + 2 * C::TILEB + sizeof(float) * 2 * 3 * BN + (unsigned)(32 * wave + r) * C::ROWB;
    const int xsw = C::swz(r);
    float delta = 0.0f;
    {
        const int64_t off = p.E * (qi + p.Lq * b) + p.D * h;   // E == Ev for these kernels
        if constexpr (X_LDS) {
            typedef __attribute__((address_space(3))) plane8 *lds_plane8_t;
            plane8 tmp[3][D / 16];
            load_stationary_s<D>(tmp, (const float *)bp.dout + off, qok, hh, (int)p.D);
#pragma unroll
            for (int q = 0; q < 3; q++)
#pragma unroll
                for (int t = 0; t < D / 16; t++) *(lds_plane8_t)(uintptr_t)(xrow + q * XPLANEB + (((2 * t + hh) ^ xsw) << 4)) = tmp[q][t];
        } else {
            load_stationary_s<D>(dox, (const float *)bp.dout + off, qok, hh, (int)p.D);
        }
        load_stationary_s<D>(qx, (const float *)p.q + off, qok, hh, (int)p.D);
        floatx4_t o4[D / 8], d4[D / 8];   // all loads first
#pragma unroll
        for (int c = 0; c < D / 8; c++) {
            const bool ok = qok && 8 * c + 4 * hh < p.D;
            o4[c] = ldg16f((const float *)p.out + off + 8 * c + 4 * hh, ok);
            d4[c] = ldg16f((const float *)bp.dout + off + 8 * c + 4 * hh, ok);
        }
#pragma unroll
        for (int c = 0; c < D / 8; c++)
#pragma unroll
            for (int j = 0; j < 4; j++) delta = fmaf(o4[c][j], d4[c][j], delta);
        delta += mi_swap32(delta);
    }

    int64_t kv_end = kv_len;
    if (CAUSAL && i0 + 32 * NW < kv_end) kv_end = i0 + 32 * NW;
    const int n_tiles = (int)((kv_end + BN - 1) / BN);

    PlaneStream<D, NT> ts;
    ts.base1 = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    ts.dh = (int)p.D;
    ts.stride = p.E;
    ts.nrows = kv_len;
    ts.s1 = Ks;
    ts.s2 = Vs;
    floatx16_t unused_o[1][NDV];
    float fm[1] = {MI_NEG_INF}, fl[1] = {0.0f};
    const float cs = a.c;
    const int64_t plane = p.B * p.H * lq_pad(p.Lq), at = (b * p.H + h) * lq_pad(p.Lq) + qi;
    const bool padded = qi < lq_pad(p.Lq);   // the statistics planes end there; a 256-query workgroup may reach past it
    if (HAVE_STATS && padded) {
        fm[0] = bp.stats[at] / cs;
        fl[0] = bp.stats[plane + at];
        if (hh == 0) bp.stats[2 * plane + at] = qok ? delta : 0.0f;
    }

    // pass 1: row maximum and row sum (K tiles only)
    ts.base2 = nullptr;
    if (!HAVE_STATS) {
        ts.load(0);
        ts.store();
    }
    __syncthreads();
    for (int jt = 0; !HAVE_STATS && jt < n_tiles; jt++) {
        const int64_t j0 = (int64_t)jt * BN;
        const bool more = jt + 1 < n_tiles;
        if (more) ts.load(j0 + BN);
        if (!CAUSAL || j0 <= iw + 31) {
            floatx16_t s[1][2] = {{(floatx16_t){0}, (floatx16_t){0}}};
#pragma unroll
            for (int kb = 0; kb < 2; kb++) s[0][kb] = first_product_s<D>(Ks, kb, qx, s[0][kb], r, hh);
            flash_softmax_tile<T, 1, NDV, CAUSAL, EXTRAS_NONE, PHASE_STATS, float>(a, s, unused_o, fm, fl, b, h, iw, j0, FlashStaged<1>(), 0, 0, nullptr,
                                                                                   kv_len);
        }
        if (more) {
            __syncthreads();   // every wavefront is done with the tile in LDS
            ts.store();
        }
        __syncthreads();
    }
    if (!HAVE_STATS) {
        fl[0] = 1.0f / (fl[0] + mi_swap32(fl[0]));
        if (hh == 0 && padded) {
            bp.stats[at] = qok ? fm[0] * cs : 0.0f;
            bp.stats[plane + at] = qok ? fl[0] : 0.0f;
            bp.stats[2 * plane + at] = qok ? delta : 0.0f;
        }
    }
    if (!bp.dq) return;

    // pass 2: P, dP = V dO^T, dS = P (dP - delta), dQ^T += K^T dS^T
    floatx16_t dq[NDV];
#pragma unroll
    for (int dvb = 0; dvb < NDV; dvb++) dq[dvb] = (floatx16_t){0};
    ts.base2 = (const float *)p.v + p.Ev * (p.Lkv * b) + p.D * h;
    int jt0 = 0, jt1 = n_tiles;
    if (a.nsplit > 1) {
        jt0 = split * a.tiles_per_split;
        if (jt0 + a.tiles_per_split < jt1) jt1 = jt0 + a.tiles_per_split;
    }
    ts.load((int64_t)jt0 * BN);
    __syncthreads();   // pass 1 may still be reading the tile
    ts.store();
    __syncthreads();
    const float m2 = fm[0] * cs, linv = fl[0];
    for (int jt = jt0; jt < jt1; jt++) {
        const int64_t j0 = (int64_t)jt * BN;
        const bool more = jt + 1 < jt1;
        if (more && AHEAD) ts.load(j0 + BN);
        if (!CAUSAL || j0 <= iw + 31) {
            const bool edge = (j0 + BN > kv_len) || (CAUSAL && j0 + BN - 1 > iw);
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                if (CAUSAL && j0 + 32 * kb > iw + 31) break;   // every key of this block is after every query of the wavefront
                floatx16_t sb = first_product_s<D>(Ks, kb, qx, (floatx16_t){0}, r, hh);
                SCHED_FENCE();
                floatx16_t dpb;
                if constexpr (X_LDS) dpb = first_product_sl<D, XPLANEB>(Vs, kb, xrow, xsw, (floatx16_t){0}, r, hh);
                else dpb = first_product_s<D>(Vs, kb, dox, (floatx16_t){0}, r, hh);
                SCHED_FENCE();
                int lim = BN;   // keys of the tile this lane's query keeps, counted from the lane's first key of a group of four
                if (edge) {
                    int64_t lim64 = kv_len - j0;
                    if (CAUSAL && qi - j0 + 1 < lim64) lim64 = qi - j0 + 1;
                    lim = (lim64 > BN ? BN : (lim64 < 0 ? 0 : (int)lim64)) - 4 * hh;
                }
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int kvl = 32 * kb + 8 * (v / 4) + (v % 4);
                    const float pw = (!edge || kvl < lim) ? mi_exp2(fmaf(sb[v], cs, -m2)) * linv : 0.0f;
                    sb[v] = pw * (dpb[v] - delta);
                }
                SCHED_FENCE();
                second_product_s<D>(Ks, kb, sb, dq, lane);
                SCHED_FENCE();
            }
        }
        if (more) {
            if (!AHEAD) ts.load(j0 + BN);
            __syncthreads();
            ts.store();
        }
        __syncthreads();
    }
    if (qok) {
        float *dqrow = a.nsplit > 1 ? bp.dq_partial + ((int64_t)split * p.B * p.Lq + qi + p.Lq * b) * p.E + p.D * h
                                    : (float *)bp.dq + p.E * (qi + p.Lq * b) + p.D * h;
#pragma unroll
        for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                floatx4_t o4;
#pragma unroll
                for (int e = 0; e < 4; e++) o4[e] = dq[dvb][4 * g + e] * a.cn;
                if (32 * dvb + 8 * g + 4 * hh < p.D) *(floatx4_t *)(dqrow + 32 * dvb + 8 * g + 4 * hh) = o4;
            }
    }
}

template <int D, bool CAUSAL, int WHICH>
// Head dim 64 fits two workgroups per compute unit, each fetching its next tiles only once the products are done (no
// staging registers live across them): the other workgroup covers the latency.  WHICH = BWD_DV | BWD_DK: both
// gradients from one S and dP, one workgroup per compute unit (see launch_set_planes).
__global__ __launch_bounds__(256, D == 64 && WHICH != 3 ? 2 : 1) void bwd32s_dkdv_kernel(FlashArgs a, AttnBwdParams bp) {
    typedef CfgS<D> C;
    constexpr int NDV = D / 32;
    constexpr bool DO_DV = (WHICH & BWD_DV) != 0, DO_DK = (WHICH & BWD_DK) != 0;   // 3: both from one S and dP
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    const unsigned Qs = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)bwd_smem, dOs = Qs + C::TILEB;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t hb = blockIdx.x % HB, kt_idx = blockIdx.x / HB;   // with causal masks the early key tiles are the long ones
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t j0 = kt_idx * 128, jw = j0 + 32 * wave, kv = jw + r;
    const bool kok = kv < p.Lkv;
    int64_t kv_len = p.Lkv;
    if (a.kv_len) {
        kv_len = a.kv_len[b * p.H + h];
        if (kv_len == 0) return;
    }
    const bool kvalid = kv < kv_len;
    const int64_t off = p.E * (kv + p.Lkv * b) + p.D * h;
    if (j0 >= kv_len) {   // keys from the pair's length on get zero gradients
        if (kok) {
            const floatx4_t z4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    if (32 * dvb + 8 * g + 4 * hh < p.D) {
                        if (DO_DV && bp.dv) *(floatx4_t *)((float *)bp.dv + off + 32 * dvb + 8 * g + 4 * hh) = z4;
                        if (DO_DK && bp.dk) *(floatx4_t *)((float *)bp.dk + off + 32 * dvb + 8 * g + 4 * hh) = z4;
                    }
        }
        return;
    }

    plane8 kx[3][D / 16], vx[DO_DK ? 3 : 1][D / 16];
    load_stationary_s<D>(kx, (const float *)p.k + off, kvalid, hh, (int)p.D);
    if constexpr (DO_DK) load_stationary_s<D>(vx, (const float *)p.v + off, kvalid, hh, (int)p.D);
    floatx16_t accv[DO_DV ? NDV : 1], acck[DO_DK ? NDV : 1];
#pragma unroll
    for (int dvb = 0; dvb < (DO_DV ? NDV : 1); dvb++) accv[dvb] = (floatx16_t){0};
#pragma unroll
    for (int dvb = 0; dvb < (DO_DK ? NDV : 1); dvb++) acck[dvb] = (floatx16_t){0};

    const int64_t plane = p.B * p.H * lq_pad(p.Lq);
    // the row statistics of a query tile travel with it through LDS (48 threads x 4 floats)
    const float *st_src = bp.stats + (b * p.H + h) * lq_pad(p.Lq) + (int64_t)(tid >> 4) * plane + 4 * (tid & 15);
    float *st_lds = (float *)(bwd_smem + 2 * C::TILEB);
    floatx4_t st_reg = {0, 0, 0, 0};
    const float cs = a.c;

    PlaneStream<D> ts;
    ts.base1 = (const float *)p.q + p.E * (p.Lq * b) + p.D * h;
    ts.base2 = (const float *)bp.dout + p.E * (p.Lq * b) + p.D * h;
    ts.dh = (int)p.D;
    ts.stride = p.E;
    ts.nrows = p.Lq;
    ts.s1 = Qs;
    ts.s2 = dOs;
    const int n_qt = (int)((p.Lq + BN - 1) / BN);
    const int it0 = CAUSAL ? (int)(j0 / BN) : 0;   // query tiles before the first key of the workgroup see none of its keys
    if (it0 < n_qt) {
        ts.load((int64_t)it0 * BN);
        ts.store();
        if (tid < 48) *(floatx4_t *)(st_lds + 4 * tid) = *(const floatx4_t *)(st_src + (int64_t)it0 * BN);
    }
    __syncthreads();
    for (int it = it0; it < n_qt; it++) {
        const int buf = (it - it0) & 1;
        const int64_t i0 = (int64_t)it * BN;
        const bool more = it + 1 < n_qt;
        if (more && tid < 48) st_reg = *(const floatx4_t *)(st_src + i0 + BN);
        if (!CAUSAL || i0 + BN - 1 >= jw) {
            const float *st = st_lds + buf * (3 * BN);
            const bool diag = CAUSAL && i0 < jw + 32;   // some (query, key) pair of this tile has key > query
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                floatx16_t s = first_product_s<D>(Qs, kb, kx, (floatx16_t){0}, r, hh);
                SCHED_FENCE();
                floatx16_t dp = (floatx16_t){0};
                if constexpr (DO_DK) dp = first_product_s<D>(dOs, kb, vx, dp, r, hh);
                SCHED_FENCE();
                // accumulator register 4g+e of this lane: query i0 + 32kb + 8g + 4hh + e, key kv.  Rows past Lq carry
                // statistics (0, 0, 0): their weights vanish; keys past the length only feed columns that store zeros
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int sq = 32 * kb + 8 * g + 4 * hh;
                    const floatx4_t m4 = *(const floatx4_t *)(st + sq);
                    const floatx4_t linv4 = *(const floatx4_t *)(st + BN + sq);
                    floatx4_t delta4 = {0.0f, 0.0f, 0.0f, 0.0f};
                    if (DO_DK) delta4 = *(const floatx4_t *)(st + 2 * BN + sq);
                    const int dq_ = (int)(jw - (i0 + sq)) + r;   // key index minus query index of element e = 0
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float pw = mi_exp2(fmaf(s[4 * g + e], cs, -m4[e])) * linv4[e];
                        if (diag) pw = dq_ - e > 0 ? 0.0f : pw;
                        if (DO_DK) dp[4 * g + e] = pw * (dp[4 * g + e] - delta4[e]);
                        s[4 * g + e] = pw;
                    }
                }
                SCHED_FENCE();
                if constexpr (DO_DV) {
                    second_product_s<D>(dOs, kb, s, accv, lane);
                    SCHED_FENCE();
                }
                if constexpr (DO_DK) {
                    second_product_s<D>(Qs, kb, dp, acck, lane);
                    SCHED_FENCE();
                }
            }
        }
        if (more) {
            ts.load(i0 + BN);
            __syncthreads();   // every wavefront is done with the tiles in LDS
            ts.store();
            if (tid < 48) *(floatx4_t *)(st_lds + (buf ^ 1) * (3 * BN) + 4 * tid) = st_reg;
        }
        __syncthreads();
    }
    if (kok) {
#pragma unroll
        for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if (32 * dvb + 8 * g + 4 * hh >= p.D) continue;
                if constexpr (DO_DV) {
                    floatx4_t g4;
#pragma unroll
                    for (int e = 0; e < 4; e++) g4[e] = kvalid ? accv[dvb][4 * g + e] : 0.0f;
                    if (bp.dv) *(floatx4_t *)((float *)bp.dv + off + 32 * dvb + 8 * g + 4 * hh) = g4;
                }
                if constexpr (DO_DK) {
                    floatx4_t g4;
#pragma unroll
                    for (int e = 0; e < 4; e++) g4[e] = kvalid ? acck[dvb][4 * g + e] * a.cn : 0.0f;
                    if (bp.dk) *(floatx4_t *)((float *)bp.dk + off + 32 * dvb + 8 * g + 4 * hh) = g4;
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------------
// Gradient calls that leave most of the chip idle (few (head, batch) pairs, short sequences).  The kernels above give a
// workgroup 128 queries or 128 keys; these give it 32, with four wavefronts that each take one 32-row block of every
// 128-row chunk of the other sequence and add up their partial gradients through LDS at the end: four times the
// workgroups, a quarter of the products, the softmax arithmetic and the operand splits per wavefront.  The stationary
// rows (Q and dO, or K and V) are split once per workgroup, a quarter per wavefront, and read back from LDS as the B
// operand.  They need the forward call's statistics; dK and dV come from one kernel that computes S and dP once
// (seven products for the gradient instead of eight).
template <int D>
struct SmallBwd {
    typedef CfgS<D> C;
    static constexpr int XPLANEB = 32 * C::ROWB;            // one plane of a stationary 32-row block
    static constexpr int XB = 3 * XPLANEB;                  // a stationary block
    static constexpr unsigned OFF_X = 4 * C::TILEB;         // behind the two chunks (two tiles each)
    static constexpr unsigned OFF_ST = OFF_X + 2 * XB;      // statistics of a query chunk: [3][128] floats
    static constexpr size_t SMEM = OFF_ST + 3 * 128 * sizeof(float);
    static constexpr int XCHUNKS = 32 * D / 4 / 256, CHUNKS = BN * D / 4 / 256;
    static_assert(2 * 4 * 64 * (D / 2) * sizeof(float) <= 4 * C::TILEB, "the partial gradients of four wavefronts fit the chunk buffers");

    // a quarter of a stationary 32-row block per wavefront: loaded, split, stored as planes at `x`
    __device__ static void split_block(unsigned x, const float *base, int64_t stride, int64_t row0, int64_t nrows, int dh, float scale) {
        typedef __attribute__((address_space(3))) u32x2_t *lds8_t;
        floatx4_t reg[XCHUNKS];
#pragma unroll
        for (int u = 0; u < XCHUNKS; u++) {
            const int i = threadIdx.x + 256 * u;
            const int64_t row = row0 + i / (D / 4);
            const int col = (i % (D / 4)) * 4;
            reg[u] = ldg16f(base + stride * row + col, row < nrows && col < dh);
        }
#pragma unroll
        for (int u = 0; u < XCHUNKS; u++) {
            const int i = threadIdx.x + 256 * u;
            const int row = i / (D / 4), col = (i % (D / 4)) * 4;
            const floatx4_t v = reg[u] * scale;
            uint32_t pl[3][2];
            const bool odd = split3_pair(v[0], v[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(v[2], v[3], pl[0][1], pl[1][1], pl[2][1]);
            if (odd) {   // an Inf or NaN in the chunk (rare)
                split3_pair_guarded(v[0], v[1], pl[0][0], pl[1][0], pl[2][0]);
                split3_pair_guarded(v[2], v[3], pl[0][1], pl[1][1], pl[2][1]);
            }
            const unsigned at = x + (unsigned)row * C::ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
            for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * XPLANEB) = (u32x2_t){pl[q][0], pl[q][1]};
        }
    }

    // a 128-row chunk of two tensors: loaded into registers, later split into the two-tile buffers at s1 and s2
    struct Chunk {
        floatx4_t r1[2][CHUNKS], r2[2][CHUNKS];
        __device__ void load(const float *b1, const float *b2, int64_t stride, int64_t row0, int64_t nrows, int dh) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int u = 0; u < CHUNKS; u++) {
                    const int i = threadIdx.x + 256 * u;
                    const int64_t row = row0 + 64 * t + i / (D / 4);
                    const int col = (i % (D / 4)) * 4;
                    const bool ok = row < nrows && col < dh;
                    r1[t][u] = ldg16f(b1 + stride * row + col, ok);
                    r2[t][u] = ldg16f(b2 + stride * row + col, ok);
                }
        }
        __device__ void store(unsigned s1, unsigned s2) const {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int u = 0; u < CHUNKS; u++) {
                    const int i = threadIdx.x + 256 * u;
                    const int row = i / (D / 4), col = (i % (D / 4)) * 4;
                    PlaneStream<D>::put(s1 + t * C::TILEB, row, col, r1[t][u]);
                    PlaneStream<D>::put(s2 + t * C::TILEB, row, col, r2[t][u]);
                }
        }
    };

    // the partial gradients of the four wavefronts added up: each wavefront sums and stores a quarter of the lane's row
    __device__ static void reduce_store(float *xout, const floatx16_t (&acc)[D / 32], float *grad_row, bool ok, int dh, float scale, bool zero) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, hh = lane >> 5;
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
            for (int v = 0; v < 16; v++) xout[(wave * (D / 2) + 16 * dvb + v) * 64 + lane] = acc[dvb][v];
        __syncthreads();
        if (ok) {
            constexpr int PER = D / 32;
#pragma unroll
            for (int i = 0; i < PER; i++) {
                const int piece = wave * PER + i, dvb = piece >> 2, g = piece & 3;
                floatx4_t o4 = (floatx4_t){0};
#pragma unroll
                for (int w = 0; w < 4; w++)
#pragma unroll
                    for (int e = 0; e < 4; e++) o4[e] += xout[(w * (D / 2) + 16 * dvb + 4 * g + e) * 64 + lane];
                if (zero) o4 = (floatx4_t){0};
                if (32 * dvb + 8 * g + 4 * hh < dh) *(floatx4_t *)(grad_row + 32 * dvb + 8 * g + 4 * hh) = o4 * scale;
            }
        }
    }
};

// MASKED: a Bool mask array of any strides (no bias): one byte per (key, query) pair of the lane, requested before the
// products
template <int D, bool CAUSAL, bool MASKED>
__global__ __launch_bounds__(256, 1) void bwd32s_dq_small_kernel(FlashArgs a, AttnBwdParams bp) {
    typedef CfgS<D> C;
    typedef SmallBwd<D> SB;
    constexpr int NDV = D / 32;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)bwd_smem;
    const unsigned Ks = lds0, Vs = lds0 + 2 * C::TILEB, Xq = lds0 + SB::OFF_X, Xdo = Xq + SB::XB;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t n_qblocks = (p.Lq + 31) / 32;
    const int64_t hb = blockIdx.x % HB, qblk = n_qblocks - 1 - blockIdx.x / HB;
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t iw = qblk * 32, qi = iw + r;
    const bool qok = qi < p.Lq;

    const int64_t head = p.E * (p.Lq * b) + p.D * h;   // E == Ev for these kernels
    SB::split_block(Xq, (const float *)p.q + head, p.E, iw, p.Lq, (int)p.D, 1.0f);
    SB::split_block(Xdo, (const float *)bp.dout + head, p.E, iw, p.Lq, (int)p.D, 1.0f);
    typename SB::Chunk ch;
    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h, *vbase = (const float *)p.v + p.E * (p.Lkv * b) + p.D * h;
    int64_t kv_end = p.Lkv;
    if (CAUSAL && iw + 32 < kv_end) kv_end = iw + 32;
    const int n_chunks = (int)((kv_end + 127) / 128);
    if (bp.dq && n_chunks > 0) ch.load(kbase, vbase, p.E, 0, p.Lkv, (int)p.D);

    // delta = rowsum(O * dO) of the lane's query, saved for the dK / dV kernel
    float delta = 0.0f;
    {
        const int64_t off = head + p.E * qi;
        floatx4_t o4[D / 8], d4[D / 8];
#pragma unroll
        for (int c = 0; c < D / 8; c++) {
            const bool ok = qok && 8 * c + 4 * hh < p.D;
            o4[c] = ldg16f((const float *)p.out + off + 8 * c + 4 * hh, ok);
            d4[c] = ldg16f((const float *)bp.dout + off + 8 * c + 4 * hh, ok);
        }
#pragma unroll
        for (int c = 0; c < D / 8; c++)
#pragma unroll
            for (int j = 0; j < 4; j++) delta = fmaf(o4[c][j], d4[c][j], delta);
        delta += mi_swap32(delta);
    }
    const int64_t pad = lq_pad(p.Lq), plane = p.B * p.H * pad, at = (b * p.H + h) * pad + qi;
    const float m2 = bp.stats[at], linv = bp.stats[plane + at];
    if (wave == 0 && hh == 0) bp.stats[2 * plane + at] = qok ? delta : 0.0f;
    if (wave == 1 && qblk == n_qblocks - 1)   // rows no query block covers: a finite delta, their weights are zeros
        for (int64_t q2 = iw + 32 + lane; q2 < pad; q2 += 64) bp.stats[2 * plane + (b * p.H + h) * pad + q2] = 0.0f;
    if (!bp.dq) return;

    floatx16_t dq[NDV];
#pragma unroll
    for (int dvb = 0; dvb < NDV; dvb++) dq[dvb] = (floatx16_t){0};
    const float cs = a.c;
    const unsigned xq_row = Xq + (unsigned)r * C::ROWB, xdo_row = Xdo + (unsigned)r * C::ROWB;
    const int xsw = C::swz(r);
    const unsigned blk_tile = (unsigned)(wave >> 1) * C::TILEB;
    const int kb = wave & 1;
    for (int c = 0; c < n_chunks; c++) {
        if (c > 0) __syncthreads();   // every wavefront is done with chunk c - 1
        ch.store(Ks, Vs);
        __syncthreads();              // chunk c (and the stationary planes) in LDS
        if (c + 1 < n_chunks) ch.load(kbase, vbase, p.E, 128 * (int64_t)(c + 1), p.Lkv, (int)p.D);
        const int64_t j0 = 128 * (int64_t)c + 32 * wave;   // the wavefront's key block
        if (j0 < p.Lkv && (!CAUSAL || j0 <= iw + 31)) {
            uint8_t mk[16];
            if constexpr (MASKED) {
                const uint8_t *mrow = p.mask + (qok ? qi : 0) * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3];
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int64_t key = j0 + 8 * (v / 4) + 4 * hh + (v % 4);
                    mk[v] = mrow[(key < p.Lkv ? key : 0) * p.mask_strides[0]];
                }
            }
            floatx16_t sb = first_product_sl<D, SB::XPLANEB>(Ks + blk_tile, kb, xq_row, xsw, (floatx16_t){0}, r, hh);
            SCHED_FENCE();
            floatx16_t dpb = first_product_sl<D, SB::XPLANEB>(Vs + blk_tile, kb, xdo_row, xsw, (floatx16_t){0}, r, hh);
            SCHED_FENCE();
            if (bp.p.drop_thresh != 0) {   // fused dropout: the forward multiplied the weight by g (0 or 1 / (1 - p)), its pullback multiplies dP
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float gf[4];
                    attention_drop_factors_run4<false>(bp.p, (uint64_t)(p.Lkv * (qi + p.Lq * (h + p.H * b)) + 4 * hh + j0), g, gf);
#pragma unroll
                    for (int e = 0; e < 4; e++) dpb[4 * g + e] *= gf[e];
                }
            }
            // keys of the block this lane's query keeps, counted from the lane's first key of a group of four
            int64_t lim64 = p.Lkv - j0;
            if (CAUSAL && qi - j0 + 1 < lim64) lim64 = qi - j0 + 1;
            const int lim = (lim64 > 32 ? 32 : (lim64 < 0 ? 0 : (int)lim64)) - 4 * hh;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int kvl = 8 * (v / 4) + (v % 4);
                bool keep = kvl < lim;
                if constexpr (MASKED) keep = keep && mk[v] != 0;
                const float pw = keep ? mi_exp2(fmaf(sb[v], cs, -m2)) * linv : 0.0f;
                sb[v] = pw * (dpb[v] - delta);
            }
            SCHED_FENCE();
            second_product_s<D>(Ks + blk_tile, kb, sb, dq, lane);
            SCHED_FENCE();
        }
    }
    __syncthreads();   // the partial gradients share the chunk buffers
    SB::reduce_store((float *)bwd_smem, dq, (float *)bp.dq + head + p.E * qi, qok, (int)p.D, a.cn, false);
}

template <int D, bool CAUSAL, bool MASKED>
__global__ __launch_bounds__(256, 1) void bwd32s_dkdv_small_kernel(FlashArgs a, AttnBwdParams bp) {
    typedef CfgS<D> C;
    typedef SmallBwd<D> SB;
    constexpr int NDV = D / 32;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)bwd_smem;
    const unsigned Qs = lds0, dOs = lds0 + 2 * C::TILEB, Xk = lds0 + SB::OFF_X, Xv = Xk + SB::XB;
    float *st_lds = (float *)(bwd_smem + SB::OFF_ST);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t hb = blockIdx.x % HB, kblk = blockIdx.x / HB;   // with causal masks the early key blocks are the long ones
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t jw = kblk * 32, kv = jw + r;
    const bool kok = kv < p.Lkv;

    const int64_t khead = p.E * (p.Lkv * b) + p.D * h, qhead = p.E * (p.Lq * b) + p.D * h;
    SB::split_block(Xk, (const float *)p.k + khead, p.E, jw, p.Lkv, (int)p.D, 1.0f);
    SB::split_block(Xv, (const float *)p.v + khead, p.E, jw, p.Lkv, (int)p.D, 1.0f);
    const float *qbase = (const float *)p.q + qhead, *dobase = (const float *)bp.dout + qhead;
    const int64_t pad = lq_pad(p.Lq), plane = p.B * p.H * pad;
    // the statistics of a query chunk travel with it through LDS: 96 threads x 4 floats (maximum, 1 / row sum, delta)
    const float *st_src = bp.stats + (b * p.H + h) * pad + (int64_t)(tid >> 5) * plane + 4 * (tid & 31);
    const int n_qchunks = (int)((p.Lq + 127) / 128);
    const int c0 = CAUSAL ? (int)(jw / 128) : 0;   // query chunks before the first key of the workgroup see none of its keys
    typename SB::Chunk ch;
    floatx4_t st_reg = {0, 0, 0, 0};
    if (c0 < n_qchunks) {
        ch.load(qbase, dobase, p.E, 128 * (int64_t)c0, p.Lq, (int)p.D);
        if (tid < 96) st_reg = *(const floatx4_t *)(st_src + 128 * (int64_t)c0);
    }
    floatx16_t acck[NDV], accv[NDV];
#pragma unroll
    for (int dvb = 0; dvb < NDV; dvb++) acck[dvb] = accv[dvb] = (floatx16_t){0};
    const float cs = a.c;
    const unsigned xk_row = Xk + (unsigned)r * C::ROWB, xv_row = Xv + (unsigned)r * C::ROWB;
    const int xsw = C::swz(r);
    const unsigned blk_tile = (unsigned)(wave >> 1) * C::TILEB;
    const int kb = wave & 1;
    for (int c = c0; c < n_qchunks; c++) {
        if (c > c0) __syncthreads();   // every wavefront is done with chunk c - 1
        ch.store(Qs, dOs);
        if (tid < 96) *(floatx4_t *)(st_lds + 4 * tid) = st_reg;
        __syncthreads();               // chunk c (and the stationary planes) in LDS
        if (c + 1 < n_qchunks) {
            ch.load(qbase, dobase, p.E, 128 * (int64_t)(c + 1), p.Lq, (int)p.D);
            if (tid < 96) st_reg = *(const floatx4_t *)(st_src + 128 * (int64_t)(c + 1));
        }
        const int64_t i0 = 128 * (int64_t)c + 32 * wave;   // the wavefront's query block
        if (i0 < p.Lq && (!CAUSAL || i0 + 31 >= jw)) {
            uint8_t mk[16];
            if constexpr (MASKED) {
                const uint8_t *mcol = p.mask + (kok ? kv : 0) * p.mask_strides[0] + h * p.mask_strides[2] + b * p.mask_strides[3];
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int64_t qq = i0 + 8 * (v / 4) + 4 * hh + (v % 4);
                    mk[v] = mcol[(qq < p.Lq ? qq : 0) * p.mask_strides[1]];
                }
            }
            floatx16_t s = first_product_sl<D, SB::XPLANEB>(Qs + blk_tile, kb, xk_row, xsw, (floatx16_t){0}, r, hh);
            SCHED_FENCE();
            floatx16_t dp = first_product_sl<D, SB::XPLANEB>(dOs + blk_tile, kb, xv_row, xsw, (floatx16_t){0}, r, hh);
            SCHED_FENCE();
            // accumulator register 4g+e of this lane: query i0 + 8g + 4hh + e, key kv.  Rows past Lq carry statistics
            // (0, 0, 0): their weights vanish; keys past the length only feed columns that store zeros
            const bool diag = CAUSAL && i0 < jw + 32;   // some (query, key) pair of this block has key > query
            const bool drop = bp.p.drop_thresh != 0;
            const float *st = st_lds + 32 * wave;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int sq = 8 * g + 4 * hh;
                const floatx4_t m4 = *(const floatx4_t *)(st + sq);
                const floatx4_t linv4 = *(const floatx4_t *)(st + 128 + sq);
                const floatx4_t delta4 = *(const floatx4_t *)(st + 256 + sq);
                const int dq_ = (int)(jw - (i0 + sq)) + r;   // key index minus query index of element e = 0
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float pw = mi_exp2(fmaf(s[4 * g + e], cs, -m4[e])) * linv4[e];
                    if (diag) pw = dq_ - e > 0 ? 0.0f : pw;
                    if constexpr (MASKED) pw = mk[4 * g + e] != 0 ? pw : 0.0f;
                    // fused dropout: the value product saw pw * gd, and the pullback multiplies dP by gd
                    const float gd = drop ? attention_drop_factor(bp.p, kv, i0 + sq + e, h, b) : 1.0f;
                    s[4 * g + e] = pw * gd;
                    dp[4 * g + e] = pw * (gd * dp[4 * g + e] - delta4[e]);
                }
            }
            SCHED_FENCE();
            if (bp.dv) second_product_s<D>(dOs + blk_tile, kb, s, accv, lane);
            SCHED_FENCE();
            if (bp.dk) second_product_s<D>(Qs + blk_tile, kb, dp, acck, lane);
            SCHED_FENCE();
        }
    }
    __syncthreads();   // the partial gradients share the chunk buffers
    float *xout = (float *)bwd_smem;
    const int64_t off = khead + p.E * kv;
    if (bp.dv) SB::reduce_store(xout, accv, (float *)bp.dv + off, kok, (int)p.D, 1.0f, false);
    if (bp.dk) SB::reduce_store(xout + 4 * 64 * (D / 2), acck, (float *)bp.dk + off, kok, (int)p.D, a.cn, false);
}

// Products on the 16-bit matrix cores through three bf16 planes unless the caller's environment asks for the
// Float32 matrix instruction (MI355ATTN_F32_MFMA=1), as in the forward kernel.
bool exact_instruction_wanted() {
    static const bool wanted = [] {
        const char *e = getenv("MI355ATTN_F32_MFMA");
        return e && e[0] == '1';
    }();
    return wanted;
}

template <int D, bool CAUSAL>
int32_t launch_set_planes(const FlashArgs &a, const AttnBwdParams &bp, hipStream_t st) {
    const AttnParams &p = a.p;
    constexpr size_t SMEM = CfgS<D>::SMEM;
    // the dQ kernel on eight wavefronts (256 queries a workgroup) where those workgroups still fill the chip
    constexpr int NW_WIDE = D == 64 ? 8 : 4;
    constexpr size_t SMEM_WIDE = SMEM + 3 * 32 * NW_WIDE * CfgS<D>::ROWB;
    const int64_t wide_tiles = (p.Lq + 32 * NW_WIDE - 1) / (32 * NW_WIDE);
    // (not for sequences of at most 128 queries, where half of its wavefronts would have none: 4-6 % slower there)
    const bool wide = NW_WIDE > 4 && bp.dq_nsplit <= 1 && wide_tiles * p.H * p.B >= 256 && p.Lq > 128;
    auto k1 = bp.have_stats ? bwd32s_dq_kernel<D, CAUSAL, true, 4> : bwd32s_dq_kernel<D, CAUSAL, false, 4>;
    auto k1w = bp.have_stats ? bwd32s_dq_kernel<D, CAUSAL, true, NW_WIDE> : bwd32s_dq_kernel<D, CAUSAL, false, NW_WIDE>;
    auto k2 = bwd32s_dkdv_kernel<D, CAUSAL, BWD_DV>;
    auto k3 = bwd32s_dkdv_kernel<D, CAUSAL, BWD_DK>;
    // Both from one S and dP (seven products for the gradient instead of eight) at one workgroup per compute unit: the
    // two stationary rows and two accumulators of a lane do not fit 256 registers (428-512 bytes of scratch at two
    // workgroups per unit).  Measured against the pair: C2-shaped gradient 0.437 -> 0.425 ms, the same without the causal
    // mask 0.823 -> 0.712, 2048 x 2048 with 32 pairs 0.538 -> 0.440 (causal) and 0.777 -> 0.661, 4096 x 4096 with 8 pairs
    // 0.94 -> 0.75.  128-wide tiles keep the pair (512 registers either way, 688-1108 bytes of scratch fused).
    auto k23 = bwd32s_dkdv_kernel<D, CAUSAL, BWD_DV | BWD_DK>;
    static const bool fused_dkdv = D == 64 && getenv("MI355ATTN_F32_DKDV_PAIR") == nullptr;   // the switch: for comparisons
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, so a race is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dq_kernel<D, CAUSAL, true, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dq_kernel<D, CAUSAL, false, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        if (NW_WIDE > 4) {
            MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dq_kernel<D, CAUSAL, true, NW_WIDE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_WIDE));
            MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dq_kernel<D, CAUSAL, false, NW_WIDE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_WIDE));
        }
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)k2, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)k3, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)k23, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        attr_set = true;
    }
    // few 32-row blocks (at most two workgroups per compute unit) and the forward call's statistics: the workgroups per
    // 32 queries / 32 keys
    static const bool no_small = getenv("MI355ATTN_NO_QUAD") != nullptr;
    const int64_t q_blocks = (p.Lq + 31) / 32 * p.H * p.B, k_blocks = (p.Lkv + 31) / 32 * p.H * p.B;
    bool small_q = false, small_k = false;
    if constexpr (D == 64) {
        // measured at 32 pairs: 512 blocks 91 against 144 us (causal 65 against 134), 1024 blocks 73 against 66.  The dQ
        // kernel reads the statistics it is given; the dK / dV kernel reads what the dQ kernel before it left in
        // bp.stats, whichever that was
        const bool can = !a.kv_len && !no_small;
        // (sequences of one block take them at any number of pairs: 2048 pairs of 32 x 32 176 -> 150 us; two blocks per
        // sequence lose beyond the limit: 1024 pairs of 64 x 64 98 against 153)
        small_q = can && bp.have_stats && bp.dq_nsplit <= 1 && (q_blocks <= 512 || p.Lq <= 32);
        small_k = can && (k_blocks <= 512 || p.Lkv <= 32);
        // no statistics from the caller: where the forward kernels of this shape of call apply (a workgroup per 32
        // queries, at most 512 keys), their statistics-only run (no values, no output) fills bp.stats first
        if (can && !bp.have_stats && bp.dq_nsplit <= 1 && q_blocks <= 256 && p.Lkv <= 512 && p.scale_D == 0 && !exact_instruction_wanted()) {
            AttnParams pf = p;
            pf.out = nullptr;
            pf.weights = nullptr;
            pf.workspace = nullptr;
            pf.stats = bp.stats;
            const int32_t rc = launch_attention_flash32(pf, st);
            if (rc != MI_OK) return rc;
            small_q = true;
        }
        if (small_q || small_k) {
            static bool small_attr_set = false;
            if (!small_attr_set) {
                MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dq_small_kernel<D, CAUSAL, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SmallBwd<D>::SMEM));
                MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dkdv_small_kernel<D, CAUSAL, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SmallBwd<D>::SMEM));
                small_attr_set = true;
            }
        }
    }
    FlashArgs a1 = a;
    if (bp.dq_nsplit > 1) {   // the dQ kernel's key range in pieces (the dK / dV kernels keep a.nsplit = 1)
        a1.nsplit = bp.dq_nsplit;
        a1.tiles_per_split = (int32_t)(((p.Lkv + BN - 1) / BN + bp.dq_nsplit - 1) / bp.dq_nsplit);
    }
    if (small_q) {
        if constexpr (D == 64) hipLaunchKernelGGL((bwd32s_dq_small_kernel<D, CAUSAL, false>), dim3((unsigned)q_blocks), dim3(256), SmallBwd<D>::SMEM, st, a, bp);
    } else if (wide) {
        a1.n_qtiles = (int32_t)wide_tiles;
        hipLaunchKernelGGL(k1w, dim3((unsigned)(wide_tiles * p.H * p.B)), dim3(64 * NW_WIDE), SMEM_WIDE, st, a1, bp);
    } else {
        hipLaunchKernelGGL(k1, dim3((unsigned)((int64_t)a.n_qtiles * p.H * p.B * a1.nsplit)), dim3(256), SMEM, st, a1, bp);
    }
    MI_LAUNCH_CHECK();
    const dim3 g2((unsigned)(((p.Lkv + 127) / 128) * p.H * p.B));
    if (small_k) {
        if constexpr (D == 64)
            if (bp.dv || bp.dk) hipLaunchKernelGGL((bwd32s_dkdv_small_kernel<D, CAUSAL, false>), dim3((unsigned)k_blocks), dim3(256), SmallBwd<D>::SMEM, st, a, bp);
    } else if (bp.dv && bp.dk && fused_dkdv) {
        hipLaunchKernelGGL(k23, g2, dim3(256), SMEM, st, a, bp);
    } else {
        if (bp.dv) hipLaunchKernelGGL(k2, g2, dim3(256), SMEM, st, a, bp);
        if (bp.dk) hipLaunchKernelGGL(k3, g2, dim3(256), SMEM, st, a, bp);
    }
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <int D, bool CAUSAL, int EXTRAS, bool DROP = false>
int32_t launch_set(const FlashArgs &a, const AttnBwdParams &bp, hipStream_t st) {
    if constexpr (EXTRAS == EXTRAS_NONE && !DROP)
        if (!bp.dbias && !exact_instruction_wanted()) return launch_set_planes<D, CAUSAL>(a, bp, st);
    const AttnParams &p = a.p;
    constexpr size_t SMEM = Cfg<D>::SMEM;
    constexpr size_t SMEM_Q = SMEM + (EXTRAS == EXTRAS_NONE ? 0 : 4 * FLASH_WSTAGE_BYTES);   // the dQ kernel's staging for the bias gradient
    // Two kernels (dV, then dK) where that buys two wavefronts per SIMD (head dim 64 without bias / mask
    // arrays) or is needed to fit the register file at all (head dim 128: K, V, dK and dV of a lane are
    // 256 registers before anything else); one pass otherwise.
    constexpr bool SPLIT = (EXTRAS == EXTRAS_NONE && D == 64) || D == 128;
    auto k1 = bp.have_stats ? bwd32_dq_kernel<D, CAUSAL, EXTRAS, true, DROP> : bwd32_dq_kernel<D, CAUSAL, EXTRAS, false, DROP>;
    auto k2 = bwd32_dkdv_kernel<D, CAUSAL, EXTRAS, SPLIT ? BWD_DV : 3, DROP>;
    auto k3 = bwd32_dkdv_kernel<D, CAUSAL, EXTRAS, SPLIT ? BWD_DK : 3, DROP>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, so a race is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32_dq_kernel<D, CAUSAL, EXTRAS, true, DROP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_Q));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32_dq_kernel<D, CAUSAL, EXTRAS, false, DROP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_Q));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)k2, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)k3, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM));
        attr_set = true;
    }
    // Bias gradient without atomics where a workgroup owns the entries it adds to; entries shared by the batch
    // elements are kept apart by one launch per batch element (the same rule as the 16-bit kernels)
    FlashArgs a1 = a;
    if (bp.dq_nsplit > 1) {   // the dQ kernel's key range in pieces (the dK / dV kernels below keep a.nsplit = 1)
        a1.nsplit = bp.dq_nsplit;
        a1.tiles_per_split = (int32_t)(((p.Lkv + BN - 1) / BN + bp.dq_nsplit - 1) / bp.dq_nsplit);
    }
    const bool own_rows = bp.dbias && p.bias_strides[0] == 1 && (p.bias_strides[1] != 0 || p.Lq == 1) && (p.bias_strides[2] != 0 || p.H == 1);
    const bool per_batch = own_rows && p.bias_strides[3] == 0 && p.B > 1;
    if (own_rows && (!per_batch || (int64_t)a.n_qtiles * p.H >= 256)) a1.dbias_plain = 1;
    if (a1.dbias_plain && per_batch) {
        a1.nb = 1;
        for (int64_t b = 0; b < p.B; b++) {
            a1.b0 = (int32_t)b;
            hipLaunchKernelGGL(k1, dim3((unsigned)((int64_t)a.n_qtiles * p.H * a1.nsplit)), dim3(256), SMEM_Q, st, a1, bp);
        }
    } else {
        hipLaunchKernelGGL(k1, dim3((unsigned)((int64_t)a.n_qtiles * p.H * p.B * a1.nsplit)), dim3(256), SMEM_Q, st, a1, bp);
    }
    MI_LAUNCH_CHECK();
    const dim3 g2((unsigned)(((p.Lkv + 127) / 128) * p.H * p.B));
    if (SPLIT) {
        if (bp.dv) hipLaunchKernelGGL(k2, g2, dim3(256), SMEM, st, a, bp);
        if (bp.dk) hipLaunchKernelGGL(k3, g2, dim3(256), SMEM, st, a, bp);
        MI_LAUNCH_CHECK();
    } else if (bp.dk || bp.dv) {
        hipLaunchKernelGGL(k2, g2, dim3(256), SMEM, st, a, bp);
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}

template <int D>
int32_t launch_d(const FlashArgs &a, const AttnBwdParams &bp, hipStream_t st) {
    if (a.kv_len) {   // key-padding mask measured on the device: both kernel sets, every (head, batch) pair in exactly one
        const int32_t rc = bp.p.causal ? launch_set<D, true, EXTRAS_NONE>(a, bp, st) : launch_set<D, false, EXTRAS_NONE>(a, bp, st);
        if (rc != MI_OK) return rc;
        return bp.p.causal ? launch_set<D, true, EXTRAS_DIRECT>(a, bp, st) : launch_set<D, false, EXTRAS_DIRECT>(a, bp, st);
    }
    const bool extras = bp.p.bias || bp.p.mask || bp.p.drop_thresh;
    if (bp.p.drop_thresh)   // dropout runs on the per-element paths
        return bp.p.causal ? launch_set<D, true, EXTRAS_DIRECT, true>(a, bp, st) : launch_set<D, false, EXTRAS_DIRECT, true>(a, bp, st);
    if (bp.p.causal) return extras ? launch_set<D, true, EXTRAS_DIRECT>(a, bp, st) : launch_set<D, true, EXTRAS_NONE>(a, bp, st);
    return extras ? launch_set<D, false, EXTRAS_DIRECT>(a, bp, st) : launch_set<D, false, EXTRAS_NONE>(a, bp, st);
}

}  // namespace

// context lengths of a key-padding mask (no dropout: that runs on the per-element paths), one per (head, batch) pair
size_t attention_bwd_flash32_lengths_bytes(const AttnBwdParams &bp) {
    if (bp.p.drop_thresh || !flash_is_query_independent_mask(bp.p) || bp.p.H * bp.p.B > 2147483647LL / 4) return 0;
    return ((size_t)(bp.p.H * bp.p.B) * sizeof(int32_t) + 15) & ~(size_t)15;
}

bool attention_bwd_flash32_supports(const AttnBwdParams &bp) {
    const AttnParams &p = bp.p;
    if (p.dtype != MI_F32) return false;
    // one head dim for q, k and v: a multiple of 4 (16-byte chunks) up to the 128-wide tiles
    if (p.D != p.Dv || p.D < 4 || p.D > 128 || (p.D & 3)) return false;
    // the kernels need the forward result (for delta), take no weight cotangent and give no bias gradient
    if (!p.out || bp.dweights) return false;   // a bias gradient is summed with atomics by the dQ kernel
    auto al = [](const void *x) { return (((uintptr_t)x) & 15) == 0; };
    if (!al(p.q) || !al(p.k) || !al(p.v) || !al(p.out) || !al(bp.dout)) return false;
    if ((bp.dq && !al(bp.dq)) || (bp.dk && !al(bp.dk)) || (bp.dv && !al(bp.dv))) return false;
    const int64_t tiles = (p.Lq + 127) / 128 > (p.Lkv + 127) / 128 ? (p.Lq + 127) / 128 : (p.Lkv + 127) / 128;
    return tiles * p.H * p.B <= 2147483647LL;
}

namespace {
// Small calls with a Bool mask array and / or fused dropout, no bias: the workgroups per 32 queries / 32 keys read the
// mask bytes of their pairs themselves (any strides; a key-padding mask needs no classification of context lengths)
// and redraw the keep decisions
bool small_extras_call(const AttnBwdParams &bp) {
    static const bool no_small = getenv("MI355ATTN_NO_QUAD") != nullptr;
    const AttnParams &p = bp.p;
    if (no_small || (!p.mask && !p.drop_thresh) || p.bias || bp.dbias || p.D > 64 || exact_instruction_wanted() || bp.dq_nsplit > 1) return false;
    const int64_t q_blocks = (p.Lq + 31) / 32 * p.H * p.B, k_blocks = (p.Lkv + 31) / 32 * p.H * p.B;
    if (q_blocks > 512 || k_blocks > 512) return false;
    // without the caller's statistics the forward kernels' statistics-only run has to apply (see launch_set_planes)
    return bp.have_stats || (q_blocks <= 256 && p.Lkv <= 512 && p.scale_D == 0);
}

template <bool CAUSAL, bool MASKED>
int32_t launch_small_extras(const FlashArgs &a, const AttnBwdParams &bp, hipStream_t st) {
    constexpr int D = 64;
    const AttnParams &p = a.p;
    static bool attr_set = false;
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dq_small_kernel<D, CAUSAL, MASKED>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SmallBwd<D>::SMEM));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)bwd32s_dkdv_small_kernel<D, CAUSAL, MASKED>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SmallBwd<D>::SMEM));
        attr_set = true;
    }
    if (!bp.have_stats) {   // the statistics are those of the weights before dropout
        AttnParams pf = p;
        pf.out = nullptr;
        pf.weights = nullptr;
        pf.workspace = nullptr;
        pf.stats = bp.stats;
        pf.drop_thresh = 0;
        const int32_t rc = launch_attention_flash32(pf, st);
        if (rc != MI_OK) return rc;
    }
    const int64_t q_blocks = (p.Lq + 31) / 32 * p.H * p.B, k_blocks = (p.Lkv + 31) / 32 * p.H * p.B;
    hipLaunchKernelGGL((bwd32s_dq_small_kernel<D, CAUSAL, MASKED>), dim3((unsigned)q_blocks), dim3(256), SmallBwd<D>::SMEM, st, a, bp);
    if (bp.dv || bp.dk) hipLaunchKernelGGL((bwd32s_dkdv_small_kernel<D, CAUSAL, MASKED>), dim3((unsigned)k_blocks), dim3(256), SmallBwd<D>::SMEM, st, a, bp);
    MI_LAUNCH_CHECK();
    return MI_OK;
}
}  // namespace

int32_t launch_attention_bwd_flash32(const AttnBwdParams &bp_in, hipStream_t st) {
    AttnBwdParams bp = bp_in;
    // few queries, many keys, saved statistics: the dQ kernel's key range in pieces (the 16-bit kernels' rule); the
    // workspace then holds [context lengths][partial sums]
    bp.dq_nsplit = attention_bwd_flash16_dq_nsplit(bp);
    if (bp.dq_nsplit > 1) bp.dq_partial = (float *)((char *)bp.workspace + attention_bwd_flash32_lengths_bytes(bp));
    FlashArgs a;
    a.p = bp.p;
    a.p.weights = nullptr;
    a.p.workspace = nullptr;
    a.p.stats = nullptr;
    a.cn = 1.0f / sqrtf((float)(bp.p.scale_D ? bp.p.scale_D : bp.p.D));
    a.c = MI_LOG2E * a.cn;
    a.n_qtiles = (int32_t)((bp.p.Lq + 127) / 128);
    a.nsplit = 1;
    a.tiles_per_split = 0;
    a.b0 = 0;
    a.nb = (int32_t)bp.p.B;
    a.dbias_plain = 0;
    flash_fill_vec_flags(a);
    a.bias_lds = a.mask_lds = 0;
    a.p.drop_thresh = 0;   // the shared softmax step yields the weights before dropout; the kernels apply bp.p's dropout themselves
    if (small_extras_call(bp)) {
        if (bp.p.mask) return bp.p.causal ? launch_small_extras<true, true>(a, bp, st) : launch_small_extras<false, true>(a, bp, st);
        return bp.p.causal ? launch_small_extras<true, false>(a, bp, st) : launch_small_extras<false, false>(a, bp, st);
    }
    if (attention_bwd_flash32_lengths_bytes(bp) != 0) {
        // the lengths follow the statistics planes when those live in the workspace too
        int32_t *lens = (int32_t *)((char *)bp.workspace + (bp.have_stats ? 0 : attention_stats_bytes(bp.p)));
        const int32_t rc = launch_key_mask_lengths(bp.p, lens, st);
        if (rc != MI_OK) return rc;
        a.kv_len = lens;
    }
    const int32_t rc = bp.p.D <= 64 ? launch_d<64>(a, bp, st) : launch_d<128>(a, bp, st);
    if (rc != MI_OK || bp.dq_nsplit <= 1) return rc;
    return launch_dq_merge(MI_F32, bp.dq_partial, bp.dq, bp.dq_nsplit, bp.p.B * bp.p.Lq * bp.p.E, st);
}
