// Flash-style attention forward for Float32 inputs.
//
// Same decomposition as the 16-bit kernel: S^T = K Q^T with keys as MFMA rows and queries as
// columns, online softmax per lane-owned query column, O^T += V^T P^T.  Inputs, outputs, softmax and
// every sum are Float32; the two products run either
//   * on the 16-bit matrix cores through three bf16 planes per operand (run_tiles32s: six
//     v_mfma_f32_32x32x16_bf16 per Float32 product, Float32 accuracy; the default), or
//   * on the Float32 instruction v_mfma_f32_32x32x2_f32 (run_tiles32; MI355ATTN_F32_MFMA=1 in the
//     environment).  With one fp32 per register no transposition is needed there: the A operand of the
//     second product is a plain 4-byte LDS read of V[key][feature = lane], the B operand is the softmax
//     accumulator register itself, and the contraction index of QK^T is permuted so that a lane fetches K
//     with 16-byte LDS reads (k-step 4c+j of half-wave hh multiplies feature d = 8c + 4hh + j; Q is loaded
//     with the same map).
// Both keep the 1e-4 parity bound with a wide margin (errors of 1e-6 against float64).
#include "flash_common.h"
#include <cstdlib>
#include <type_traits>

namespace {

typedef F32 T;
constexpr int BN = FLASH_BN;

template <int D, int QB>
struct Frag32 {
    float q[QB][D / 2];
    floatx16_t o[QB][D / 32];
    float m[QB], l[QB];
};

template <int D>
struct Cfg {
    static constexpr int KS = D + 4;   // K row stride (floats): rows 4 banks apart, conflict-free b128 reads
    static constexpr int VS = D + 8;   // V row stride (floats): rows 4 apart land 32 banks apart
    static constexpr int CHUNKS = BN * D / 4 / 256;  // 16-byte chunks per thread, tile and tensor
    static constexpr size_t SMEM = sizeof(float) * 2 * BN * (KS + VS);
};

__device__ inline floatx4_t ldg16f(const float *p, bool ok) {
    return mi_load16_or_zero<floatx4_t>(p, ok);
}

template <int D, int QB, bool CAUSAL, bool EXTRAS, int PHASE>
// kv_len: keys of this (head, batch) pair (L_kv, or a shorter context length)
__device__ inline void run_tiles32(const FlashArgs &a, Frag32<D, QB> &f, float *Ks, float *Vs, int64_t kv_len, int64_t b, int64_t h,
                                   int64_t iw, int n_tiles, unsigned wlds = 0, int jt0 = 0) {
    constexpr int KS = Cfg<D>::KS, VS = Cfg<D>::VS, CHUNKS = Cfg<D>::CHUNKS;
    const AttnParams &p = a.p;
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hh = lane >> 5;
    constexpr bool NEED_V = PHASE != PHASE_STATS;
    const bool do_pv = NEED_V && p.out != nullptr;

    // D is the tile width; the head dims p.D / p.Dv may be smaller (multiples of 4): the rest is loaded as zeros
    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    const float *vbase = NEED_V && p.v ? (const float *)p.v + p.Ev * (p.Lkv * b) + p.Dv * h : nullptr;
    const int dqk = (int)p.D, dv = (int)p.Dv;

    floatx4_t kreg[CHUNKS], vreg[CHUNKS];
    auto load_tile = [&](int jt) {
        const int64_t j0 = (int64_t)jt * BN;
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            const bool ok = j0 + row < kv_len;
            kreg[u] = ldg16f(kbase + p.E * (j0 + row) + col, ok && col < dqk);
            if (NEED_V) vreg[u] = ldg16f(vbase + p.Ev * (j0 + row) + col, ok && do_pv && col < dv);
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            *(floatx4_t *)(Ks + (buf * BN + row) * KS + col) = kreg[u];
            if (NEED_V) *(floatx4_t *)(Vs + (buf * BN + row) * VS + col) = vreg[u];
        }
    };

    if (n_tiles <= jt0) return;
    load_tile(jt0);
    __syncthreads();
    store_tile(0);
    __syncthreads();

    for (int jt = jt0; jt < n_tiles; jt++) {
        const int buf = (jt - jt0) & 1;
        const int64_t j0 = (int64_t)jt * BN;
        if (jt + 1 < n_tiles) load_tile(jt + 1);

        const bool active = !CAUSAL || j0 <= iw + 32 * QB - 1;
        if (active) {
            floatx16_t s[QB][2];
#pragma unroll
            for (int qb = 0; qb < QB; qb++)
#pragma unroll
                for (int kb = 0; kb < 2; kb++) s[qb][kb] = (floatx16_t){0};
            // the two key blocks alternate, so that consecutive MFMAs never wait for each other's accumulator
            const float *kt = Ks + (buf * BN + r) * KS + 4 * hh;
#pragma unroll
            for (int c = 0; c < D / 8; c++) {
                const floatx4_t k4a = *(const floatx4_t *)(kt + 8 * c);
                const floatx4_t k4b = *(const floatx4_t *)(kt + 32 * KS + 8 * c);
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int qb = 0; qb < QB; qb++) {
                        s[qb][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(k4a[j], f.q[qb][4 * c + j], s[qb][0], 0, 0, 0);
                        s[qb][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(k4b[j], f.q[qb][4 * c + j], s[qb][1], 0, 0, 0);
                    }
            }

            flash_softmax_tile<T, QB, D / 32, CAUSAL, EXTRAS ? EXTRAS_DIRECT : EXTRAS_NONE, PHASE, float>(a, s, f.o, f.m, f.l, b, h, iw, j0,
                                                                                                          FlashStaged<QB>(), 0, wlds, nullptr, kv_len);

            if (do_pv) {
                // k-step v of key block kb multiplies key 32*kb + 8*(v/4) + 4*hh + v%4: exactly the key
                // whose weight sits in accumulator register v of this lane
                const float *vt = Vs + (buf * BN + 4 * hh) * VS + r;
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const float *src = vt + (32 * kb + 8 * (v / 4) + (v % 4)) * VS;
#pragma unroll
                        for (int dvb = 0; dvb < D / 32; dvb++) {
                            const float va = src[32 * dvb];
#pragma unroll
                            for (int qb = 0; qb < QB; qb++)
                                f.o[qb][dvb] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, s[qb][kb][v], f.o[qb][dvb], 0, 0, 0);
                        }
                    }
            }
        }
        if (jt + 1 < n_tiles) store_tile(buf ^ 1);
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------------------------------
// Float32 products on the 16-bit matrix cores (the planes and their arithmetic: common.h).  K and V tiles are
// split once when they are staged (three bf16 planes per tile in LDS, laid out and read like the tiles of the
// 16-bit kernel), Q once per workgroup, the softmax weights once per tile in registers.
typedef bf16x8_t plane8;
typedef bf16x4_t plane4;
typedef short s16x4_t __attribute__((ext_vector_type(4)));

template <int D>
struct CfgS {
    static constexpr int ROWB = D * 2;              // bytes per tile row of one plane
    static constexpr int PLANEB = BN * ROWB;        // one plane of one tile
    static constexpr int TILEB = 3 * PLANEB;        // K or V tile: hi, mid, lo planes
    static constexpr int CHUNKS = BN * D / 4 / 256; // float4 pieces per thread, tile and tensor
    static constexpr size_t SMEM = 2 * TILEB;       // one K and one V tile (the next one waits in registers)
    // chunk swizzle of the 16-bit kernel (conflict-free 16-byte operand reads and transposing reads)
    __device__ static inline int swz(int row) {
        if (D >= 128) return ((row & 3) << 2) | ((row >> 2) & 3);
        const int x = (row >> 1) & 7;
        return ((x & 1) << 2) | (x >> 1);
    }
};

template <int D, int QB>
struct Frag32S {
    plane8 q[QB][3][D / 16];
    floatx16_t o[QB][D / 32];
    float m[QB], l[QB];
};

__device__ inline plane4 lds_tr4s(unsigned addr) {
    s16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t *)(uintptr_t)addr);
    return __builtin_bit_cast(plane4, r);
}

__device__ inline floatx16_t mfma_bf16(plane8 a, plane8 b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// c += a b with a, b given as planes (small terms first).  Alternating two accumulators between consecutive
// instructions instead measured 4-8 % slower.
__device__ inline floatx16_t mfma_split(const plane8 (&a)[3], const plane8 (&b)[3], floatx16_t c) {
    c = mfma_bf16(a[2], b[0], c);
    c = mfma_bf16(a[0], b[2], c);
    c = mfma_bf16(a[1], b[1], c);
    c = mfma_bf16(a[1], b[0], c);
    c = mfma_bf16(a[0], b[1], c);
    return mfma_bf16(a[0], b[0], c);
}

// S^T = K Q^T of one 64-key tile whose planes sit at LDS address Ks: s[query block][key block]
// (KBLK = 1: of the 32-key block whose first row sits at Ks)
template <int D, int QB, int KBLK = 2>
__device__ inline void scores32s(const Frag32S<D, QB> &f, unsigned Ks, floatx16_t (&s)[QB][KBLK]) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB;
    typedef __attribute__((address_space(3))) const plane8 *lds_plane8_t;
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int qb = 0; qb < QB; qb++)
#pragma unroll
        for (int kb = 0; kb < KBLK; kb++) s[qb][kb] = (floatx16_t){0};
    // lane's K operand: row r (+32 per key block), chunk 2t + hh, in each plane
    const unsigned kt = Ks + (unsigned)r * ROWB;
    const int ksw = C::swz(r);
#pragma unroll
    for (int t = 0; t < D / 16; t++)
#pragma unroll
        for (int kb = 0; kb < KBLK; kb++) {
            plane8 ka[3];
#pragma unroll
            for (int q = 0; q < 3; q++)
                ka[q] = *(lds_plane8_t)(uintptr_t)(kt + q * PLANEB + kb * 32 * ROWB + (((2 * t + hh) ^ ksw) << 4));
#pragma unroll
            for (int qb = 0; qb < QB; qb++) {
                const plane8 qq[3] = {f.q[qb][0][t], f.q[qb][1][t], f.q[qb][2][t]};
                s[qb][kb] = mfma_split(ka, qq, s[qb][kb]);
            }
        }
}

// O^T += V^T P^T for one 64-key tile (KBLK = 1: one 32-key block): the weights in s (accumulator layout), V's planes
// (the block's first row) at LDS address Vs
template <int D, int QB, int KBLK = 2>
__device__ inline void weights_times_values32s(Frag32S<D, QB> &f, unsigned Vs, const floatx16_t (&s)[QB][KBLK]) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB;
    const int lane = threadIdx.x & 63, hh = lane >> 5;
    // P^T operand of k-step u of key block kb: accumulator registers 8u .. 8u+7 (keys 0-3, 8-11 | 4-7, 12-15
    // of the 16); V^T comes from the row-major planes with the transposing read in that same key order
    const int vrow = 4 * hh + ((lane & 15) >> 2);
    const int vchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), vsub = 8 * (lane & 1);
    const unsigned vt = Vs + (unsigned)vrow * ROWB + vsub;
    const int vsw_lo = C::swz(vrow), vsw_hi = C::swz(vrow + 8);
#pragma unroll
    for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
        for (int u = 0; u < 2; u++) {
            plane8 pk[QB][3];
#pragma unroll
            for (int qb = 0; qb < QB; qb++) {
                uint32_t w[3][4];
#pragma unroll
                for (int e = 0; e < 4; e++)   // a NaN weight (fully masked column) stays NaN in the hi plane
                    split3_pair(s[qb][kb][8 * u + 2 * e], s[qb][kb][8 * u + 2 * e + 1], w[0][e], w[1][e], w[2][e]);
#pragma unroll
                for (int q = 0; q < 3; q++) pk[qb][q] = __builtin_bit_cast(plane8, (u32x4_t){w[q][0], w[q][1], w[q][2], w[q][3]});
            }
#pragma unroll
            for (int dvb = 0; dvb < D / 32; dvb++) {
                const unsigned src = vt + (32 * kb + 16 * u) * ROWB;
                plane8 va[3];
#pragma unroll
                for (int q = 0; q < 3; q++) {
                    const plane4 lo = lds_tr4s(src + q * PLANEB + (((4 * dvb + vchunk) ^ vsw_lo) << 4));
                    const plane4 hi = lds_tr4s(src + q * PLANEB + 8 * ROWB + (((4 * dvb + vchunk) ^ vsw_hi) << 4));
                    va[q] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
#pragma unroll
                for (int qb = 0; qb < QB; qb++) f.o[qb][dvb] = mfma_split(va, pk[qb], f.o[qb][dvb]);
            }
        }
}

template <int D, int QB, bool CAUSAL, bool EXTRAS, int PHASE>
__device__ inline void run_tiles32s(const FlashArgs &a, Frag32S<D, QB> &f, unsigned Ks, unsigned Vs, int64_t kv_len, int64_t b, int64_t h,
                                    int64_t iw, int n_tiles, unsigned wlds = 0, int jt0 = 0) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB, CHUNKS = C::CHUNKS;
    const AttnParams &p = a.p;
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hh = lane >> 5;
    constexpr bool NEED_V = PHASE != PHASE_STATS;
    const bool do_pv = NEED_V && p.out != nullptr;
    typedef __attribute__((address_space(3))) u32x2_t *lds8_t;
    typedef __attribute__((address_space(3))) const plane8 *lds_plane8_t;

    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    const float *vbase = NEED_V && p.v ? (const float *)p.v + p.Ev * (p.Lkv * b) + p.Dv * h : nullptr;
    const int dqk = (int)p.D, dv = (int)p.Dv;

    floatx4_t kreg[CHUNKS], vreg[CHUNKS];
    auto load_tile = [&](int jt) {
        const int64_t j0 = (int64_t)jt * BN;
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            const bool ok = j0 + row < kv_len;
            kreg[u] = ldg16f(kbase + p.E * (j0 + row) + col, ok && col < dqk);
            if (NEED_V) vreg[u] = ldg16f(vbase + p.Ev * (j0 + row) + col, ok && do_pv && col < dv);
        }
    };
    // four consecutive features of one key: 8 bytes in each of the three planes
    auto store_split = [&](unsigned tile, int row, int col, const floatx4_t &x) {
        uint32_t pl[3][2];
        const bool odd = split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        if (odd) {   // an Inf or NaN in the chunk (rare)
            split3_pair_guarded(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair_guarded(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        }
        const unsigned at = tile + (unsigned)row * ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
        for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * PLANEB) = (u32x2_t){pl[q][0], pl[q][1]};
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            store_split(Ks, row, col, kreg[u]);
            if (NEED_V) store_split(Vs, row, col, vreg[u]);
        }
    };

    if (n_tiles <= jt0) return;
    load_tile(jt0);
    __syncthreads();   // a previous phase may still be reading the tile
    store_tile();
    __syncthreads();

    for (int jt = jt0; jt < n_tiles; jt++) {
        const int64_t j0 = (int64_t)jt * BN;
        const bool more = jt + 1 < n_tiles;
        if (more) load_tile(jt + 1);

        const bool active = !CAUSAL || j0 <= iw + 32 * QB - 1;
        if (active) {
            floatx16_t s[QB][2];
            scores32s<D, QB>(f, Ks, s);

            flash_softmax_tile<T, QB, D / 32, CAUSAL, EXTRAS ? EXTRAS_DIRECT : EXTRAS_NONE, PHASE, float>(a, s, f.o, f.m, f.l, b, h, iw, j0,
                                                                                                          FlashStaged<QB>(), 0, wlds, nullptr, kv_len);

            if (do_pv) weights_times_values32s<D, QB>(f, Vs, s);
        }
        if (more) {
            __syncthreads();   // every wavefront is done with the tile in LDS
            store_tile();
        }
        __syncthreads();
    }
}

template <int D, int QB, bool SPLIT>
struct FragSel { typedef Frag32<D, QB> type; };
template <int D, int QB>
struct FragSel<D, QB, true> { typedef Frag32S<D, QB> type; };

template <int D, int QB, bool CAUSAL, bool EXTRAS, bool WEIGHTS, bool SPLIT>
// Head dim 64 without bias / mask fits two workgroups per CU (256 registers, 70 KiB of LDS each; 56 KiB with the
// bf16 planes, bias / mask or not).
__global__ __launch_bounds__(256, (D == 64 && !EXTRAS) ? 2 : 1) void flash32_kernel(FlashArgs a) {
    constexpr int KS = Cfg<D>::KS, VS = Cfg<D>::VS;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char flash_smem[];
    float *Ks = (float *)flash_smem;     // [2][BN][KS]
    float *Vs = Ks + 2 * BN * KS;        // [2][BN][VS]
    (void)VS;
    // bf16 planes: one K tile, one V tile, as LDS byte addresses
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)flash_smem;
    const unsigned Kp = lds0, Vp = lds0 + CfgS<D>::TILEB;
    constexpr size_t TILES_SMEM = SPLIT ? CfgS<D>::SMEM : Cfg<D>::SMEM;
    constexpr int BM = 128 * QB;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int split = (int)(blockIdx.x % a.nsplit);   // split-kv: this workgroup's piece of the key range
    const int64_t id = blockIdx.x / a.nsplit;
    const int64_t hb = id % HB;
    const int64_t qt = a.n_qtiles - 1 - id / HB;   // heaviest (latest) query tiles first
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t i0 = qt * BM, iw = i0 + (int64_t)wave * 32 * QB;
    // Key-padding masks measured on the device (FlashArgs::kv_len): a (head, batch) pair whose mask keeps a prefix of
    // the keys is an unmasked problem with that many keys, which the variant without bias / mask code takes; the
    // variant with it computes the other pairs.  Both are launched; every pair belongs to exactly one.
    int64_t kv_len = p.Lkv;
    if (a.kv_len) {
        const int64_t len = a.kv_len[b * p.H + h];
        if (EXTRAS == (len != 0)) return;
        if (!EXTRAS) kv_len = len;
    }

    typename FragSel<D, QB, SPLIT>::type f;
    const float *qbase = (const float *)p.q + p.E * (p.Lq * b) + p.D * h;
    const float sq = sqrtf((float)p.D);
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
        const int64_t qi = iw + 32 * qb + r;
        if constexpr (SPLIT) {
            // lane's features of k-step t: 16t + 8hh .. + 7 (the B-operand layout of the 16-bit instruction)
            uint32_t qw[3][D / 16][4];
            floatx4_t raw[D / 16][2];   // every load of the row is issued before the first is used: one memory round trip
#pragma unroll
            for (int t = 0; t < D / 16; t++)
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    const int d0 = 16 * t + 8 * hh + 4 * half;
                    raw[t][half] = ldg16f(qbase + p.E * qi + d0, qi < p.Lq && d0 < p.D);
                }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < D / 16; t++)
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    const floatx4_t q4 = raw[t][half];
                    // the reference divides q by sqrt(D) first (src/attention.jl:118)
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        uint32_t w[3];
                        const float x0 = q4[2 * j] / sq, x1 = q4[2 * j + 1] / sq;
                        if (split3_pair(x0, x1, w[0], w[1], w[2])) split3_pair_guarded(x0, x1, w[0], w[1], w[2]);
#pragma unroll
                        for (int q = 0; q < 3; q++) qw[q][t][2 * half + j] = w[q];
                    }
                }
#pragma unroll
            for (int q = 0; q < 3; q++)
#pragma unroll
                for (int t = 0; t < D / 16; t++) f.q[qb][q][t] = __builtin_bit_cast(plane8, (u32x4_t){qw[q][t][0], qw[q][t][1], qw[q][t][2], qw[q][t][3]});
        } else {
#pragma unroll
            for (int c = 0; c < D / 8; c++) {
                const floatx4_t q4 = ldg16f(qbase + p.E * qi + 8 * c + 4 * hh, qi < p.Lq && 8 * c + 4 * hh < p.D);
                // the reference divides q by sqrt(D) before the product (src/attention.jl:118)
#pragma unroll
                for (int j = 0; j < 4; j++) f.q[qb][4 * c + j] = q4[j] / sq;
            }
        }
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++) f.o[qb][dvb] = (floatx16_t){0};
        f.m[qb] = MI_NEG_INF;
        f.l[qb] = 0.0f;
    }
    // one entry point for both tile loops
    auto run = [&](auto phase, int n, unsigned wlds, int jt0) {
        constexpr int PHASE = decltype(phase)::value;
        if constexpr (SPLIT) run_tiles32s<D, QB, CAUSAL, EXTRAS, PHASE>(a, f, Kp, Vp, kv_len, b, h, iw, n, wlds, jt0);
        else run_tiles32<D, QB, CAUSAL, EXTRAS, PHASE>(a, f, Ks, Vs, kv_len, b, h, iw, n, wlds, jt0);
    };

    int64_t kv_end = kv_len;
    if (CAUSAL && i0 + BM < kv_end) kv_end = i0 + BM;
    const int n_tiles = (int)((kv_end + BN - 1) / BN);

    if (!WEIGHTS) {
        int jt0 = 0, jt1 = n_tiles;
        if (a.nsplit > 1) {
            jt0 = split * a.tiles_per_split;
            if (jt0 + a.tiles_per_split < jt1) jt1 = jt0 + a.tiles_per_split;
        }
        run(std::integral_constant<int, PHASE_ONLINE>(), jt1, 0u, jt0);
        if (a.nsplit > 1) {
            // partial result of this key piece for flash_merge_kernel: unnormalised o, row maximum (log2 units), row sum
            float *wo = (float *)p.workspace + ((int64_t)split * p.B + b) * p.Lq * p.Ev + p.Dv * h;
            float *wml = (float *)p.workspace + (int64_t)a.nsplit * p.B * p.Lq * p.Ev + (((int64_t)split * p.B + b) * p.H + h) * p.Lq * 2;
#pragma unroll
            for (int qb = 0; qb < QB; qb++) {
                const int64_t qi = iw + 32 * qb + r;
                const float l = f.l[qb] + mi_swap32(f.l[qb]);
                if (qi < p.Lq) {
#pragma unroll
                    for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            floatx4_t o4;
#pragma unroll
                            for (int e = 0; e < 4; e++) o4[e] = f.o[qb][dvb][4 * g + e];
                            if (32 * dvb + 8 * g + 4 * hh < p.Dv) *(floatx4_t *)(wo + p.Ev * qi + 32 * dvb + 8 * g + 4 * hh) = o4;
                        }
                    if (hh == 0) {
                        wml[2 * qi] = f.m[qb] * MI_LOG2E;
                        wml[2 * qi + 1] = l;
                    }
                }
            }
            return;
        }
    } else {
        run(std::integral_constant<int, PHASE_STATS>(), n_tiles, 0u, 0);
#pragma unroll
        for (int qb = 0; qb < QB; qb++) {
            const float l = f.l[qb] + mi_swap32(f.l[qb]);
            f.l[qb] = 1.0f / l;
        }
        // weight tiles leave through a wavefront-private LDS region behind the K / V buffers
        const unsigned wlds = lds0 + (unsigned)TILES_SMEM + wave * FLASH_WSTAGE_BYTES;
        run(std::integral_constant<int, PHASE_FINAL>(), n_tiles, wlds, 0);
        if (CAUSAL && p.weights) flash_zero_skipped_weights<QB, float>(a, b, h, iw, n_tiles);
        else if (p.weights && kv_len < p.Lkv) flash_zero_skipped_weights<QB, float>(a, b, h, iw, n_tiles, false);   // keys past the context length
    }

    if (p.out) {
        float *obase = (float *)p.out + p.Ev * (p.Lq * b) + p.Dv * h;
#pragma unroll
        for (int qb = 0; qb < QB; qb++) {
            const int64_t qi = iw + 32 * qb + r;
            float inv = 1.0f;
            if (!WEIGHTS) {
                const float l = f.l[qb] + mi_swap32(f.l[qb]);
                inv = 1.0f / l;
            }
            if (p.stats && hh == 0) flash_save_stats(p, b, h, qi, f.m[qb] * MI_LOG2E, WEIGHTS ? f.l[qb] : inv);
            if (qi < p.Lq) {
#pragma unroll
                for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        floatx4_t o4;
#pragma unroll
                        for (int e = 0; e < 4; e++) o4[e] = f.o[qb][dvb][4 * g + e] * inv;
                        if (32 * dvb + 8 * g + 4 * hh < p.Dv) *(floatx4_t *)(obase + p.Ev * qi + 32 * dvb + 8 * g + 4 * hh) = o4;
                    }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Small problems with the weights returned (the reference's default call, src/attention.jl:83): at most RES_TILES
// tiles of keys.  flash32_kernel walks such a call as a chain of dependent steps (queries, K tile, statistics, K and
// V tile again, weights), each waiting for memory or for a barrier.  Here every load of the call is issued at the
// start, K and V are split into planes once, the scores of all tiles stay in registers between the statistics and the
// weights, and the workgroup meets at two barriers (K in LDS; V in LDS, split under the score products).
constexpr int RES_TILES = 2;
constexpr int64_t RESIDENT_QUAD_MAX_BLOCKS = 256;   // 32-query blocks up to which a call runs one workgroup per block

// The reference divides q by sqrt(D) first (src/attention.jl:118).  When sqrt(D) is a power of two (D = 16, 64, 256)
// the product with its reciprocal is that quotient bit for bit, at a tenth of the instructions of a division.
__device__ inline bool sqrt_is_power_of_two(float sq) { return (__builtin_bit_cast(uint32_t, sq) & 0x7fffffu) == 0; }
template <int D>
__device__ inline void scale_queries(floatx4_t (&q4)[D / 16][2], float head_dim) {
    const float sq = sqrtf(head_dim), inv_sq = 1.0f / sq;
    if (sqrt_is_power_of_two(sq)) {
#pragma unroll
        for (int t = 0; t < D / 16; t++)
#pragma unroll
            for (int half = 0; half < 2; half++) q4[t][half] *= inv_sq;
    } else {
#pragma unroll
        for (int t = 0; t < D / 16; t++)
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int e = 0; e < 4; e++) q4[t][half][e] /= sq;
    }
}

template <int D, bool CAUSAL, bool EXTRAS>
__global__ __launch_bounds__(256, 1) void flash32_resident_kernel(FlashArgs a) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB, CHUNKS = C::CHUNKS, TILEB = C::TILEB;
    constexpr int XT = EXTRAS ? EXTRAS_DIRECT : EXTRAS_NONE;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char flash_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)flash_smem;
    const unsigned Kp = lds0, Vp = lds0 + RES_TILES * TILEB;   // K tiles, V tiles, then the weight staging regions
    typedef __attribute__((address_space(3))) u32x2_t *lds8_t;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t hb = blockIdx.x % HB, qt = a.n_qtiles - 1 - blockIdx.x / HB;
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t i0 = qt * 128, iw = i0 + (int64_t)wave * 32, qi = iw + r;
    int64_t kv_end = p.Lkv;
    if (CAUSAL && i0 + 128 < kv_end) kv_end = i0 + 128;
    const int n_tiles = (int)((kv_end + BN - 1) / BN);   // <= RES_TILES: checked by the host
    const bool do_pv = p.out != nullptr;

    // ---- every load of the call: K, the wavefront's queries, V
    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    const float *vbase = do_pv ? (const float *)p.v + p.Ev * (p.Lkv * b) + p.Dv * h : nullptr;
    const float *qrow = (const float *)p.q + p.E * (qi + p.Lq * b) + p.D * h;
    const int dqk = (int)p.D, dv = (int)p.Dv;
    floatx4_t kreg[RES_TILES][CHUNKS], vreg[RES_TILES][CHUNKS], q4[D / 16][2];
#pragma unroll
    for (int t = 0; t < RES_TILES; t++)
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int64_t row = (int64_t)t * BN + c / (D / 4);
            const int col = (c % (D / 4)) * 4;
            kreg[t][u] = ldg16f(kbase + p.E * row + col, t < n_tiles && row < p.Lkv && col < dqk);
        }
#pragma unroll
    for (int t = 0; t < D / 16; t++)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int d0 = 16 * t + 8 * hh + 4 * half;   // the B-operand layout of the 16-bit instruction
            q4[t][half] = ldg16f(qrow + d0, qi < p.Lq && d0 < dqk);
        }
#pragma unroll
    for (int t = 0; t < RES_TILES; t++)
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int64_t row = (int64_t)t * BN + c / (D / 4);
            const int col = (c % (D / 4)) * 4;
            vreg[t][u] = ldg16f(vbase + p.Ev * row + col, do_pv && t < n_tiles && row < p.Lkv && col < dv);
        }

    // four consecutive features of one key: 8 bytes in each of the three planes
    auto store_split = [&](unsigned tile, int row, int col, const floatx4_t &x) {
        uint32_t pl[3][2];
        const bool odd = split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        if (odd) {   // an Inf or NaN in the chunk (rare)
            split3_pair_guarded(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair_guarded(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        }
        const unsigned at = tile + (unsigned)row * ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
        for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * PLANEB) = (u32x2_t){pl[q][0], pl[q][1]};
    };
    auto store_tile = [&](unsigned tile, const floatx4_t (&reg)[CHUNKS]) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            store_split(tile, c / (D / 4), (c % (D / 4)) * 4, reg[u]);
        }
    };

    // ---- K into planes in LDS, the queries into planes in registers
#pragma unroll
    for (int t = 0; t < RES_TILES; t++)
        if (t < n_tiles) store_tile(Kp + t * TILEB, kreg[t]);
    Frag32S<D, 1> f;
    {
        scale_queries<D>(q4, (float)p.D);
        uint32_t qw[3][D / 16][4];
#pragma unroll
        for (int t = 0; t < D / 16; t++)
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    uint32_t w[3];
                    const float x0 = q4[t][half][2 * j], x1 = q4[t][half][2 * j + 1];
                    if (split3_pair(x0, x1, w[0], w[1], w[2])) split3_pair_guarded(x0, x1, w[0], w[1], w[2]);
#pragma unroll
                    for (int q = 0; q < 3; q++) qw[q][t][2 * half + j] = w[q];
                }
#pragma unroll
        for (int q = 0; q < 3; q++)
#pragma unroll
            for (int t = 0; t < D / 16; t++) f.q[0][q][t] = __builtin_bit_cast(plane8, (u32x4_t){qw[q][t][0], qw[q][t][1], qw[q][t][2], qw[q][t][3]});
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++) f.o[0][dvb] = (floatx16_t){0};
        f.m[0] = MI_NEG_INF;
        f.l[0] = 0.0f;
    }
    __syncthreads();

    // ---- scores of every tile (kept raw), V into planes under them, statistics
    floatx16_t keep[RES_TILES][1][2];
    bool active[RES_TILES];
#pragma unroll
    for (int t = 0; t < RES_TILES; t++) {
        active[t] = t < n_tiles && (!CAUSAL || (int64_t)t * BN <= iw + 31);
        if (active[t]) scores32s<D, 1>(f, Kp + t * TILEB, keep[t]);
        if (t < n_tiles && do_pv) store_tile(Vp + t * TILEB, vreg[t]);
    }
#pragma unroll
    for (int t = 0; t < RES_TILES; t++)
        if (active[t]) {
            floatx16_t s[1][2] = {{keep[t][0][0], keep[t][0][1]}};
            flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_STATS, float>(a, s, f.o, f.m, f.l, b, h, iw, (int64_t)t * BN, FlashStaged<1>(), 0, 0u,
                                                                             nullptr, p.Lkv);
        }
    f.l[0] = 1.0f / (f.l[0] + mi_swap32(f.l[0]));
    __syncthreads();

    // ---- weights and output
    const unsigned wlds = lds0 + 2u * RES_TILES * TILEB + wave * FLASH_WSTAGE_BYTES;
#pragma unroll
    for (int t = 0; t < RES_TILES; t++)
        if (active[t]) {
            flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_FINAL, float>(a, keep[t], f.o, f.m, f.l, b, h, iw, (int64_t)t * BN, FlashStaged<1>(), 0, wlds,
                                                                             nullptr, p.Lkv);
            if (do_pv) weights_times_values32s<D, 1>(f, Vp + t * TILEB, keep[t]);
        }
    if (p.weights) flash_zero_skipped_weights<1, float>(a, b, h, iw, n_tiles, CAUSAL);

    if (p.stats && hh == 0) flash_save_stats(p, b, h, qi, f.m[0] * MI_LOG2E, f.l[0]);
    if (do_pv && qi < p.Lq) {
        float *orow = (float *)p.out + p.Ev * (qi + p.Lq * b) + p.Dv * h;
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                floatx4_t o4;
#pragma unroll
                for (int e = 0; e < 4; e++) o4[e] = f.o[0][dvb][4 * g + e];
                if (32 * dvb + 8 * g + 4 * hh < p.Dv) *(floatx4_t *)(orow + 32 * dvb + 8 * g + 4 * hh) = o4;
            }
    }
}

// The same with two wavefronts per 32-query block, one per key tile (128-key problems: C1): eight wavefronts, two per
// SIMD, each with half of the score products, the softmax arithmetic, the weight stores and the value products of a
// block, and half of the K / V split per thread.  The two exchange their row statistics (m, l) after the first
// phase and their partial outputs at the end, through LDS.
template <int D, bool CAUSAL, bool EXTRAS>
__global__ __launch_bounds__(512, 1) void flash32_resident_pair_kernel(FlashArgs a) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB, TILEB = C::TILEB;
    constexpr int NT = 512, CHUNKS = BN * D / 4 / NT;
    constexpr int XT = EXTRAS ? EXTRAS_DIRECT : EXTRAS_NONE;
    static_assert(RES_TILES == 2, "one wavefront of a pair per key tile");
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char flash_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)flash_smem;
    // K tiles (later the partial outputs of the second wavefronts), V tiles, weight staging, exchanged statistics
    const unsigned Kp = lds0, Vp = lds0 + 2 * TILEB;
    float *xstat = (float *)(flash_smem + 4 * TILEB + 8 * FLASH_WSTAGE_BYTES);   // [8 wavefronts][32 rows][2]
    float *xout = (float *)flash_smem;                                           // [4 query blocks][D / 2 registers][64 lanes]
    typedef __attribute__((address_space(3))) u32x2_t *lds8_t;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int qw = wave & 3, tile = wave >> 2;   // query block and key tile of this wavefront
    const int64_t HB = p.H * p.B;
    const int64_t hb = blockIdx.x % HB, qt = a.n_qtiles - 1 - blockIdx.x / HB;
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t i0 = qt * 128, iw = i0 + (int64_t)qw * 32, qi = iw + r;
    int64_t kv_end = p.Lkv;
    if (CAUSAL && i0 + 128 < kv_end) kv_end = i0 + 128;
    const int n_tiles = (int)((kv_end + BN - 1) / BN);   // 1 or 2: checked by the host
    const bool do_pv = p.out != nullptr;

    // ---- every load of the call: K, the wavefront's queries, V
    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    const float *vbase = do_pv ? (const float *)p.v + p.Ev * (p.Lkv * b) + p.Dv * h : nullptr;
    const float *qrow = (const float *)p.q + p.E * (qi + p.Lq * b) + p.D * h;
    const int dqk = (int)p.D, dv = (int)p.Dv;
    floatx4_t kreg[2][CHUNKS], vreg[2][CHUNKS], q4[D / 16][2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + NT * u;
            const int64_t row = (int64_t)t * BN + c / (D / 4);
            const int col = (c % (D / 4)) * 4;
            kreg[t][u] = ldg16f(kbase + p.E * row + col, t < n_tiles && row < p.Lkv && col < dqk);
        }
#pragma unroll
    for (int t = 0; t < D / 16; t++)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int d0 = 16 * t + 8 * hh + 4 * half;
            q4[t][half] = ldg16f(qrow + d0, qi < p.Lq && d0 < dqk);
        }
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + NT * u;
            const int64_t row = (int64_t)t * BN + c / (D / 4);
            const int col = (c % (D / 4)) * 4;
            vreg[t][u] = ldg16f(vbase + p.Ev * row + col, do_pv && t < n_tiles && row < p.Lkv && col < dv);
        }

    auto store_split = [&](unsigned at_tile, int row, int col, const floatx4_t &x) {
        uint32_t pl[3][2];
        const bool odd = split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        if (odd) {   // an Inf or NaN in the chunk (rare)
            split3_pair_guarded(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair_guarded(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        }
        const unsigned at = at_tile + (unsigned)row * ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
        for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * PLANEB) = (u32x2_t){pl[q][0], pl[q][1]};
    };
    auto store_tile = [&](unsigned at_tile, const floatx4_t (&reg)[CHUNKS]) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + NT * u;
            store_split(at_tile, c / (D / 4), (c % (D / 4)) * 4, reg[u]);
        }
    };

    // ---- K into planes in LDS, the queries into planes in registers
#pragma unroll
    for (int t = 0; t < 2; t++)
        if (t < n_tiles) store_tile(Kp + t * TILEB, kreg[t]);
    Frag32S<D, 1> f;
    {
        scale_queries<D>(q4, (float)p.D);
        uint32_t qw3[3][D / 16][4];
#pragma unroll
        for (int t = 0; t < D / 16; t++)
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    uint32_t w[3];
                    const float x0 = q4[t][half][2 * j], x1 = q4[t][half][2 * j + 1];
                    if (split3_pair(x0, x1, w[0], w[1], w[2])) split3_pair_guarded(x0, x1, w[0], w[1], w[2]);
#pragma unroll
                    for (int q = 0; q < 3; q++) qw3[q][t][2 * half + j] = w[q];
                }
#pragma unroll
        for (int q = 0; q < 3; q++)
#pragma unroll
            for (int t = 0; t < D / 16; t++) f.q[0][q][t] = __builtin_bit_cast(plane8, (u32x4_t){qw3[q][t][0], qw3[q][t][1], qw3[q][t][2], qw3[q][t][3]});
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++) f.o[0][dvb] = (floatx16_t){0};
        f.m[0] = MI_NEG_INF;
        f.l[0] = 0.0f;
    }
    __syncthreads();

    // ---- scores of the wavefront's tile (kept raw), V into planes, statistics of the tile
    const int64_t j0 = (int64_t)tile * BN;
    const bool active = tile < n_tiles && (!CAUSAL || j0 <= iw + 31);
    floatx16_t keep[1][2];
    // the two wavefronts of a SIMD (w and w + 4: the two tiles of one query block) take the score products and their
    // half of the V split in opposite order, so that one's matrix instructions run under the other's vector work
    auto split_v = [&]() {
        if (do_pv) {
#pragma unroll
            for (int t = 0; t < 2; t++)
                if (t < n_tiles) store_tile(Vp + t * TILEB, vreg[t]);
        }
    };
    if (tile == 1) split_v();
    if (active) scores32s<D, 1>(f, Kp + tile * TILEB, keep);
    if (tile == 0) split_v();
    if (active) {
        floatx16_t s[1][2] = {{keep[0][0], keep[0][1]}};
        flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_STATS, float>(a, s, f.o, f.m, f.l, b, h, iw, j0, FlashStaged<1>(), 0, 0u, nullptr, p.Lkv);
    }
    // the pair's statistics: (m, l) of both tiles, combined as the online softmax combines tiles (src/softmax.jl:69-79
    // over the whole row): m = max, l = sum of l_i 2^((m_i - m) c); equal maxima (two -Inf or two +Inf included) keep
    // their sums as they are
    const float lsum = f.l[0] + mi_swap32(f.l[0]);
    if (hh == 0) {
        xstat[(wave * 32 + r) * 2] = f.m[0];
        xstat[(wave * 32 + r) * 2 + 1] = lsum;
    }
    __syncthreads();   // statistics exchanged, V in LDS, every wavefront done with the K planes
    {
        const float mp = xstat[((wave ^ 4) * 32 + r) * 2], lp = xstat[((wave ^ 4) * 32 + r) * 2 + 1];
        const float cs = flash_natural_units(XT) ? MI_LOG2E : a.c;
        const float m = fmaxf(f.m[0], mp);
        const float fa = f.m[0] == m ? 1.0f : mi_exp2((f.m[0] - m) * cs), fb = mp == m ? 1.0f : mi_exp2((mp - m) * cs);
        f.m[0] = m;
        f.l[0] = 1.0f / (lsum * fa + lp * fb);
    }

    // ---- weights and the wavefront's share of the output
    const unsigned wlds = lds0 + 4u * TILEB + wave * FLASH_WSTAGE_BYTES;
    if (active) {
        flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_FINAL, float>(a, keep, f.o, f.m, f.l, b, h, iw, j0, FlashStaged<1>(), 0, wlds, nullptr, p.Lkv);
        if (do_pv) weights_times_values32s<D, 1>(f, Vp + tile * TILEB, keep);
    }
    if (tile == 0 && p.weights) flash_zero_skipped_weights<1, float>(a, b, h, iw, n_tiles, CAUSAL);
    if (tile == 0 && p.stats && hh == 0) flash_save_stats(p, b, h, qi, f.m[0] * MI_LOG2E, f.l[0]);

    // the second wavefront's partial output goes through LDS (the K planes' region: nobody reads them any more)
    if (!do_pv) return;
    if (tile == 1) {
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
            for (int v = 0; v < 16; v++) xout[(qw * (D / 2) + 16 * dvb + v) * 64 + lane] = f.o[0][dvb][v];
    }
    __syncthreads();
    if (tile == 0 && qi < p.Lq) {
        float *orow = (float *)p.out + p.Ev * (qi + p.Lq * b) + p.Dv * h;
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                floatx4_t o4;
#pragma unroll
                for (int e = 0; e < 4; e++) o4[e] = f.o[0][dvb][4 * g + e] + xout[(qw * (D / 2) + 16 * dvb + 4 * g + e) * 64 + lane];
                if (32 * dvb + 8 * g + 4 * hh < p.Dv) *(floatx4_t *)(orow + 32 * dvb + 8 * g + 4 * hh) = o4;
            }
    }
}

// The same for calls that leave most of the chip idle (few (head, batch) pairs and queries: C1 has 32 pairs of 128
// queries): one workgroup per 32-query block, four wavefronts, one per 32-key block.  A wavefront has a quarter of a
// query block's score products, softmax arithmetic, weight stores and value products; the price is that every
// workgroup splits K and V of its pair into planes for itself.  The four exchange their row statistics (m, l)
// after the first phase and add up their partial outputs at the end, through LDS.
template <int D, bool CAUSAL, bool EXTRAS>
__global__ __launch_bounds__(256, 1) void flash32_resident_quad_kernel(FlashArgs a) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB, CHUNKS = C::CHUNKS, TILEB = C::TILEB;
    constexpr int XT = EXTRAS ? EXTRAS_DIRECT : EXTRAS_NONE;
    static_assert(RES_TILES == 2, "four 32-key blocks");
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char flash_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)flash_smem;
    // K tiles (later the partial outputs), V tiles, weight staging, exchanged statistics, the query block's planes.
    // Calls with at most 64 keys have one tile per tensor (69 KiB in all: two workgroups per compute unit)
    const unsigned kt = p.Lkv <= BN ? 1u : 2u;
    const unsigned Kp = lds0, Vp = lds0 + kt * TILEB, behind = 2 * kt * TILEB;
    float *xstat = (float *)(flash_smem + behind + 4 * FLASH_WSTAGE_BYTES);   // [4 wavefronts][32 rows][2]
    float *xout = (float *)flash_smem;                                        // [2 kt wavefronts with a key block][D / 2 registers][64 lanes]
    constexpr int QPLANEB = 32 * ROWB, QCHUNKS = 32 * D / 4 / 256;
    const unsigned Qp = lds0 + behind + 4 * FLASH_WSTAGE_BYTES + 4 * 32 * 2 * (unsigned)sizeof(float);
    typedef __attribute__((address_space(3))) const plane8 *lds_plane8_t;
    typedef __attribute__((address_space(3))) u32x2_t *lds8_t;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t n_qblocks = (p.Lq + 31) / 32;
    const int64_t hb = blockIdx.x % HB, qblk = n_qblocks - 1 - blockIdx.x / HB;
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t iw = qblk * 32, qi = iw + r;
    int64_t kv_end = p.Lkv;
    if (CAUSAL && iw + 32 < kv_end) kv_end = iw + 32;
    const int n_tiles = (int)((kv_end + BN - 1) / BN);   // 1 or 2: checked by the host
    const bool do_pv = p.out != nullptr;

    // ---- every load of the call: K, the queries, V
    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    const float *vbase = do_pv ? (const float *)p.v + p.Ev * (p.Lkv * b) + p.Dv * h : nullptr;
    const float *qbase = (const float *)p.q + p.E * (p.Lq * b) + p.D * h;
    const int dqk = (int)p.D, dv = (int)p.Dv;
    floatx4_t kreg[2][CHUNKS], vreg[2][CHUNKS], qreg[QCHUNKS];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int64_t row = (int64_t)t * BN + c / (D / 4);
            const int col = (c % (D / 4)) * 4;
            kreg[t][u] = ldg16f(kbase + p.E * row + col, t < n_tiles && row < p.Lkv && col < dqk);
        }
#pragma unroll
    for (int u = 0; u < QCHUNKS; u++) {   // the four wavefronts share the query block: a quarter each
        const int c = tid + 256 * u;
        const int64_t row = iw + c / (D / 4);
        const int col = (c % (D / 4)) * 4;
        qreg[u] = ldg16f(qbase + p.E * row + col, row < p.Lq && col < dqk);
    }
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            const int64_t row = (int64_t)t * BN + c / (D / 4);
            const int col = (c % (D / 4)) * 4;
            vreg[t][u] = ldg16f(vbase + p.Ev * row + col, do_pv && t < n_tiles && row < p.Lkv && col < dv);
        }

    auto store_split = [&](unsigned at_tile, int row, int col, const floatx4_t &x, int planeb) {
        uint32_t pl[3][2];
        const bool odd = split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        if (odd) {   // an Inf or NaN in the chunk (rare)
            split3_pair_guarded(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair_guarded(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        }
        const unsigned at = at_tile + (unsigned)row * ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
        for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * planeb) = (u32x2_t){pl[q][0], pl[q][1]};
    };
    auto store_tile = [&](unsigned at_tile, const floatx4_t (&reg)[CHUNKS]) {
#pragma unroll
        for (int u = 0; u < CHUNKS; u++) {
            const int c = tid + 256 * u;
            store_split(at_tile, c / (D / 4), (c % (D / 4)) * 4, reg[u], PLANEB);
        }
    };

    // ---- K and the scaled queries into planes in LDS
#pragma unroll
    for (int t = 0; t < 2; t++)
        if (t < n_tiles) store_tile(Kp + t * TILEB, kreg[t]);
    {
        // q / sqrt(D) as the reference has it (see scale_queries)
        const float sq = sqrtf((float)p.D), inv_sq = 1.0f / sq;
        if (sqrt_is_power_of_two(sq)) {
#pragma unroll
            for (int u = 0; u < QCHUNKS; u++) qreg[u] *= inv_sq;
        } else {
#pragma unroll
            for (int u = 0; u < QCHUNKS; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) qreg[u][e] /= sq;
        }
#pragma unroll
        for (int u = 0; u < QCHUNKS; u++) {
            const int c = tid + 256 * u;
            store_split(Qp, c / (D / 4), (c % (D / 4)) * 4, qreg[u], QPLANEB);
        }
    }
    Frag32S<D, 1> f;
#pragma unroll
    for (int dvb = 0; dvb < D / 32; dvb++) f.o[0][dvb] = (floatx16_t){0};
    f.m[0] = MI_NEG_INF;
    f.l[0] = 0.0f;
    __syncthreads();
    // the wavefront's B operand: query row r, features 16t + 8hh .. + 7 of step t, in each plane (read like a K row)
#pragma unroll
    for (int q = 0; q < 3; q++)
#pragma unroll
        for (int t = 0; t < D / 16; t++)
            f.q[0][q][t] = *(lds_plane8_t)(uintptr_t)(Qp + q * QPLANEB + (unsigned)r * ROWB + (((2 * t + hh) ^ C::swz(r)) << 4));

    // ---- scores of the wavefront's block (kept raw), V into planes, statistics of the block
    const int tile = wave >> 1;
    const int64_t j0 = 32 * (int64_t)wave;
    // every block of a tile that some query of the workgroup reaches takes part (a block past the diagonal yields
    // the exact zeros its weights are); tiles nobody reaches are zeroed below
    const bool active = tile < n_tiles;
    const unsigned blk = (unsigned)tile * TILEB + (unsigned)(wave & 1) * 32u * ROWB;
    floatx16_t keep[1][1];
    if (active) scores32s<D, 1, 1>(f, Kp + blk, keep);
    if (do_pv) {
#pragma unroll
        for (int t = 0; t < 2; t++)
            if (t < n_tiles) store_tile(Vp + t * TILEB, vreg[t]);
    }
    if (active) {
        floatx16_t s[1][1] = {{keep[0][0]}};
        flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_STATS, float, 1>(a, s, f.o, f.m, f.l, b, h, iw, j0, FlashStaged<1>(), 0, 0u, nullptr, p.Lkv);
    }
    // the workgroup's statistics: (m, l) of the four blocks, combined as the online softmax combines tiles
    // (src/softmax.jl:69-79 over the whole row): m = max, l = sum of l_i 2^((m_i - m) c); a block whose maximum is the
    // row's keeps its sum as it is (two -Inf or two +Inf included)
    const float lsum = f.l[0] + mi_swap32(f.l[0]);
    if (hh == 0) {
        xstat[(wave * 32 + r) * 2] = f.m[0];
        xstat[(wave * 32 + r) * 2 + 1] = lsum;
    }
    __syncthreads();   // statistics exchanged, V in LDS, every wavefront done with the K planes
    {
        const float cs = flash_natural_units(XT) ? MI_LOG2E : a.c;
        float m = f.m[0];
#pragma unroll
        for (int w = 0; w < 4; w++) m = fmaxf(m, xstat[(w * 32 + r) * 2]);
        float l = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float mw = xstat[(w * 32 + r) * 2], lw = xstat[(w * 32 + r) * 2 + 1];
            l += lw * (mw == m ? 1.0f : mi_exp2((mw - m) * cs));
        }
        f.m[0] = m;
        f.l[0] = 1.0f / l;
    }

    // ---- weights and the wavefront's share of the output
    const unsigned wlds = lds0 + behind + wave * FLASH_WSTAGE_BYTES;
    if (active) {
        flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_FINAL, float, 1>(a, keep, f.o, f.m, f.l, b, h, iw, j0, FlashStaged<1>(), 0, wlds, nullptr, p.Lkv);
        if (do_pv) weights_times_values32s<D, 1, 1>(f, Vp + blk, keep);
    }
    if (wave == 0 && p.weights) flash_zero_skipped_weights<1, float>(a, b, h, iw, n_tiles, false);
    if (wave == 0 && p.stats && hh == 0) flash_save_stats(p, b, h, qi, f.m[0] * MI_LOG2E, f.l[0]);
    if (wave == 1 && p.stats && qblk == n_qblocks - 1) flash_zero_stats_padding(p, b, h, iw + 32);   // rows no query block covers

    // the partial outputs go through LDS (the K planes' region: nobody reads them any more); each wavefront adds up
    // and writes a quarter of the row
    if (!do_pv) return;
    if (wave < (int)(2 * kt)) {
#pragma unroll
        for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
            for (int v = 0; v < 16; v++) xout[(wave * (D / 2) + 16 * dvb + v) * 64 + lane] = f.o[0][dvb][v];
    }
    __syncthreads();
    if (qi < p.Lq) {
        float *orow = (float *)p.out + p.Ev * (qi + p.Lq * b) + p.Dv * h;
        constexpr int PER = D / 32;   // a lane's row share is D / 8 16-byte pieces: a quarter per wavefront
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int piece = wave * PER + i, dvb = piece >> 2, g = piece & 3;
            floatx4_t o4 = (floatx4_t){0};
#pragma unroll
            for (int w = 0; w < 4; w++)
                if (w < (int)(2 * kt)) {
#pragma unroll
                    for (int e = 0; e < 4; e++) o4[e] += xout[(w * (D / 2) + 16 * dvb + 4 * g + e) * 64 + lane];
                }
            if (32 * dvb + 8 * g + 4 * hh < p.Dv) *(floatx4_t *)(orow + 32 * dvb + 8 * g + 4 * hh) = o4;
        }
    }
}

// The workgroup per 32-query block for up to NCH * 128 keys (NCH = 4, or 8 at head dims up to 64): the keys in chunks of 128 (four 32-key blocks, one per
// wavefront), the raw scores of every chunk kept in registers between the statistics and the weights, so the score
// product still runs once.  First phase: K chunks through two LDS buffers (the next chunk's loads in flight, one
// barrier per chunk); second phase: V chunks through the same two buffers.  128-wide tiles have room for one buffer
// (96 KiB): a second barrier per chunk before it is overwritten, and the partial outputs share it at the end.
constexpr int RES_CHUNKS = 4, RES_CHUNKS_NARROW = 8;

template <int D, bool CAUSAL, bool EXTRAS, int NCH>
__global__ __launch_bounds__(256, 1) void flash32_resident_chunks_kernel(FlashArgs a) {
    typedef CfgS<D> C;
    constexpr int ROWB = C::ROWB, PLANEB = C::PLANEB, CHUNKS = C::CHUNKS, TILEB = C::TILEB;
    constexpr int XT = EXTRAS ? EXTRAS_DIRECT : EXTRAS_NONE;
    const AttnParams &p = a.p;
    extern __shared__ __attribute__((aligned(16))) unsigned char flash_smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)flash_smem;
    // chunk buffers of two tiles each, weight staging, exchanged statistics, the query block's planes, partial outputs
    constexpr bool TWO_BUFFERS = D <= 64;
    constexpr int QPLANEB = 32 * ROWB, QCHUNKS = 32 * D / 4 / 256;
    constexpr unsigned OFF_STAGE = (TWO_BUFFERS ? 4 : 2) * TILEB, OFF_STAT = OFF_STAGE + 4 * FLASH_WSTAGE_BYTES, OFF_Q = OFF_STAT + 4 * 32 * 2 * sizeof(float),
                       OFF_OUT = OFF_Q + 3 * QPLANEB;
    float *xstat = (float *)(flash_smem + OFF_STAT);   // [4 wavefronts][32 rows][2]
    float *xout = (float *)(flash_smem + (TWO_BUFFERS ? OFF_OUT : 0));   // [4 wavefronts][D / 2 registers][64 lanes]
    const unsigned Qp = lds0 + OFF_Q;
    typedef __attribute__((address_space(3))) u32x2_t *lds8_t;
    typedef __attribute__((address_space(3))) const plane8 *lds_plane8_t;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hh = lane >> 5;
    const int64_t HB = p.H * p.B;
    const int64_t n_qblocks = (p.Lq + 31) / 32;
    const int64_t hb = blockIdx.x % HB, qblk = n_qblocks - 1 - blockIdx.x / HB;
    const int64_t h = hb % p.H, b = hb / p.H;
    const int64_t iw = qblk * 32, qi = iw + r;
    int64_t kv_end = p.Lkv;
    if (CAUSAL && iw + 32 < kv_end) kv_end = iw + 32;
    const int n_chunks = (int)((kv_end + 127) / 128);   // <= NCH: checked by the host
    const bool do_pv = p.out != nullptr;

    const float *kbase = (const float *)p.k + p.E * (p.Lkv * b) + p.D * h;
    const float *vbase = do_pv ? (const float *)p.v + p.Ev * (p.Lkv * b) + p.Dv * h : nullptr;
    const float *qbase = (const float *)p.q + p.E * (p.Lq * b) + p.D * h;
    const int dqk = (int)p.D, dv = (int)p.Dv;
    auto load_chunk = [&](floatx4_t (&reg)[2][CHUNKS], const float *base, int64_t ld, int dlim, int c, bool on) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int u = 0; u < CHUNKS; u++) {
                const int i = tid + 256 * u;
                const int64_t row = 128 * (int64_t)c + 64 * t + i / (D / 4);
                const int col = (i % (D / 4)) * 4;
                reg[t][u] = ldg16f(base + ld * row + col, on && row < p.Lkv && col < dlim);
            }
    };
    auto store_split = [&](unsigned at_tile, int row, int col, const floatx4_t &x, int planeb) {
        uint32_t pl[3][2];
        const bool odd = split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]) | split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        if (odd) {   // an Inf or NaN in the chunk (rare)
            split3_pair_guarded(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair_guarded(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
        }
        const unsigned at = at_tile + (unsigned)row * ROWB + (unsigned)((((col >> 3) ^ C::swz(row)) << 4) + (col & 7) * 2);
#pragma unroll
        for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(at + q * planeb) = (u32x2_t){pl[q][0], pl[q][1]};
    };
    auto store_chunk = [&](unsigned buf, const floatx4_t (&reg)[2][CHUNKS]) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int u = 0; u < CHUNKS; u++) {
                const int i = tid + 256 * u;
                store_split(buf + t * TILEB, i / (D / 4), (i % (D / 4)) * 4, reg[t][u], PLANEB);
            }
    };

    // ---- the first K chunk and the queries
    floatx4_t reg[2][CHUNKS], nxt[2][CHUNKS], qreg[QCHUNKS];
    load_chunk(reg, kbase, p.E, dqk, 0, true);
#pragma unroll
    for (int u = 0; u < QCHUNKS; u++) {   // the four wavefronts share the query block: a quarter each
        const int i = tid + 256 * u;
        const int64_t row = iw + i / (D / 4);
        const int col = (i % (D / 4)) * 4;
        qreg[u] = ldg16f(qbase + p.E * row + col, row < p.Lq && col < dqk);
    }
    {
        // q / sqrt(D) as the reference has it (see scale_queries)
        const float sq = sqrtf((float)p.D), inv_sq = 1.0f / sq;
        if (sqrt_is_power_of_two(sq)) {
#pragma unroll
            for (int u = 0; u < QCHUNKS; u++) qreg[u] *= inv_sq;
        } else {
#pragma unroll
            for (int u = 0; u < QCHUNKS; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) qreg[u][e] /= sq;
        }
#pragma unroll
        for (int u = 0; u < QCHUNKS; u++) {
            const int i = tid + 256 * u;
            store_split(Qp, i / (D / 4), (i % (D / 4)) * 4, qreg[u], QPLANEB);
        }
    }
    Frag32S<D, 1> f;
#pragma unroll
    for (int dvb = 0; dvb < D / 32; dvb++) f.o[0][dvb] = (floatx16_t){0};
    f.m[0] = MI_NEG_INF;
    f.l[0] = 0.0f;

    // ---- first phase: scores of the wavefront's block of every chunk (kept raw), running statistics
    const unsigned blk = (unsigned)(wave >> 1) * TILEB + (unsigned)(wave & 1) * 32u * ROWB;
    floatx16_t keep[NCH][1][1];
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        if (c < n_chunks) {
            if (c + 1 < n_chunks) load_chunk(nxt, kbase, p.E, dqk, c + 1, true);
            else load_chunk(nxt, vbase, p.Ev, dv, 0, do_pv);   // the first V chunk
            const unsigned buf = lds0 + (TWO_BUFFERS ? (unsigned)(c & 1) * 2u * TILEB : 0u);
            if (!TWO_BUFFERS && c > 0) __syncthreads();   // every wavefront is done with chunk c - 1
            store_chunk(buf, reg);
            __syncthreads();   // chunk c (and the queries) in LDS; with two buffers: every wavefront is done with chunk c - 1
            if (c == 0) {
                // the wavefront's B operand: query row r, features 16t + 8hh .. + 7 of step t, in each plane
#pragma unroll
                for (int q = 0; q < 3; q++)
#pragma unroll
                    for (int t = 0; t < D / 16; t++)
                        f.q[0][q][t] = *(lds_plane8_t)(uintptr_t)(Qp + q * QPLANEB + (unsigned)r * ROWB + (((2 * t + hh) ^ C::swz(r)) << 4));
            }
            scores32s<D, 1, 1>(f, buf + blk, keep[c]);
            floatx16_t s[1][1] = {{keep[c][0][0]}};
            flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_STATS, float, 1>(a, s, f.o, f.m, f.l, b, h, iw, 128 * (int64_t)c + 32 * wave, FlashStaged<1>(), 0,
                                                                                 0u, nullptr, p.Lkv);
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int u = 0; u < CHUNKS; u++) reg[t][u] = nxt[t][u];
        }
    }
    // the workgroup's statistics, combined as the online softmax combines tiles (see flash32_resident_quad_kernel)
    const float lsum = f.l[0] + mi_swap32(f.l[0]);
    if (hh == 0) {
        xstat[(wave * 32 + r) * 2] = f.m[0];
        xstat[(wave * 32 + r) * 2 + 1] = lsum;
    }
    __syncthreads();   // statistics exchanged, every wavefront done with the K chunks
    {
        const float cs = flash_natural_units(XT) ? MI_LOG2E : a.c;
        float m = f.m[0];
#pragma unroll
        for (int w = 0; w < 4; w++) m = fmaxf(m, xstat[(w * 32 + r) * 2]);
        float l = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float mw = xstat[(w * 32 + r) * 2], lw = xstat[(w * 32 + r) * 2 + 1];
            l += lw * (mw == m ? 1.0f : mi_exp2((mw - m) * cs));
        }
        f.m[0] = m;
        f.l[0] = 1.0f / l;
    }

    // ---- second phase: weights and the wavefront's share of the output, V chunks through the same buffers
    const unsigned wlds = lds0 + OFF_STAGE + wave * FLASH_WSTAGE_BYTES;
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        if (c < n_chunks) {
            const unsigned buf = lds0 + (TWO_BUFFERS ? (unsigned)(c & 1) * 2u * TILEB : 0u);
            if (do_pv) {
                if (c + 1 < n_chunks) load_chunk(nxt, vbase, p.Ev, dv, c + 1, true);
                if (!TWO_BUFFERS && c > 0) __syncthreads();   // every wavefront is done with chunk c - 1
                store_chunk(buf, reg);
                __syncthreads();   // V chunk c in LDS; with two buffers: every wavefront is done with chunk c - 1
            }
            flash_softmax_tile<T, 1, D / 32, CAUSAL, XT, PHASE_FINAL, float, 1>(a, keep[c], f.o, f.m, f.l, b, h, iw, 128 * (int64_t)c + 32 * wave, FlashStaged<1>(),
                                                                                 0, wlds, nullptr, p.Lkv);
            if (do_pv) {
                weights_times_values32s<D, 1, 1>(f, buf + blk, keep[c]);
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int u = 0; u < CHUNKS; u++) reg[t][u] = nxt[t][u];
            }
        }
    }
    if (wave == 0 && p.weights) flash_zero_skipped_weights<1, float>(a, b, h, iw, 2 * n_chunks, false);
    if (wave == 0 && p.stats && hh == 0) flash_save_stats(p, b, h, qi, f.m[0] * MI_LOG2E, f.l[0]);
    if (wave == 1 && p.stats && qblk == n_qblocks - 1) flash_zero_stats_padding(p, b, h, iw + 32);   // rows no query block covers

    // the partial outputs go through LDS; each wavefront adds up and writes a quarter of the row
    if (!do_pv) return;
    if (!TWO_BUFFERS) __syncthreads();   // the partial outputs share the chunk buffer: every wavefront is done with the last V chunk
#pragma unroll
    for (int dvb = 0; dvb < D / 32; dvb++)
#pragma unroll
        for (int v = 0; v < 16; v++) xout[(wave * (D / 2) + 16 * dvb + v) * 64 + lane] = f.o[0][dvb][v];
    __syncthreads();
    if (qi < p.Lq) {
        float *orow = (float *)p.out + p.Ev * (qi + p.Lq * b) + p.Dv * h;
        constexpr int PER = D / 32;   // a lane's row share is D / 8 16-byte pieces: a quarter per wavefront
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int piece = wave * PER + i, dvb = piece >> 2, g = piece & 3;
            floatx4_t o4 = (floatx4_t){0};
#pragma unroll
            for (int w = 0; w < 4; w++)
#pragma unroll
                for (int e = 0; e < 4; e++) o4[e] += xout[(w * (D / 2) + 16 * dvb + 4 * g + e) * 64 + lane];
            if (32 * dvb + 8 * g + 4 * hh < p.Dv) *(floatx4_t *)(orow + 32 * dvb + 8 * g + 4 * hh) = o4;
        }
    }
}

template <int D, int NCH>
int32_t launch_resident_chunks(const FlashArgs &a, hipStream_t st, bool extras) {
    constexpr size_t smem = (D <= 64 ? 4 * CfgS<D>::TILEB + 4 * 64 * (D / 2) * sizeof(float) : 2 * CfgS<D>::TILEB) + 4 * FLASH_WSTAGE_BYTES +
                            4 * 32 * 2 * sizeof(float) + 3 * 32 * CfgS<D>::ROWB;
    static_assert(smem <= 160 * 1024, "fits a compute unit's LDS");
    static_assert(4 * 64 * (D / 2) * sizeof(float) <= 2 * CfgS<D>::TILEB, "the partial outputs fit a chunk buffer");
    static bool attr_set = false;
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_chunks_kernel<D, false, false, NCH>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_chunks_kernel<D, false, true, NCH>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_chunks_kernel<D, true, false, NCH>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_chunks_kernel<D, true, true, NCH>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const int64_t total = (a.p.Lq + 31) / 32 * a.p.H * a.p.B;
    auto kern = a.p.causal ? (extras ? flash32_resident_chunks_kernel<D, true, true, NCH> : flash32_resident_chunks_kernel<D, true, false, NCH>)
                           : (extras ? flash32_resident_chunks_kernel<D, false, true, NCH> : flash32_resident_chunks_kernel<D, false, false, NCH>);
    hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(256), smem, st, a);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <int D>
int32_t launch_resident(const FlashArgs &a, hipStream_t st, bool extras) {
    constexpr size_t smem = 2 * RES_TILES * CfgS<D>::TILEB + 4 * FLASH_WSTAGE_BYTES;
    constexpr size_t smem_pair = 2 * RES_TILES * CfgS<D>::TILEB + 8 * FLASH_WSTAGE_BYTES + 8 * 32 * 2 * sizeof(float);
    constexpr size_t smem_quad = 2 * RES_TILES * CfgS<D>::TILEB + 4 * FLASH_WSTAGE_BYTES + 4 * 32 * 2 * sizeof(float) + 3 * 32 * CfgS<D>::ROWB;
    static_assert(4 * 64 * (D / 2) * sizeof(float) <= 2 * CfgS<D>::TILEB, "partial outputs (D / 2 registers of 64 lanes per wavefront) fit the K planes' region");
    static bool attr_set = false;
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_kernel<D, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_kernel<D, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_kernel<D, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_kernel<D, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_pair_kernel<D, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pair));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_pair_kernel<D, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pair));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_pair_kernel<D, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pair));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_pair_kernel<D, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pair));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_quad_kernel<D, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_quad));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_quad_kernel<D, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_quad));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_quad_kernel<D, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_quad));
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)flash32_resident_quad_kernel<D, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_quad));
        attr_set = true;
    }
    const int64_t total = (int64_t)a.n_qtiles * a.p.H * a.p.B;
    const int64_t total_quad = (a.p.Lq + 31) / 32 * a.p.H * a.p.B;
    static const bool no_quad = getenv("MI355ATTN_NO_QUAD") != nullptr;   // the workgroup of eight, for comparisons
    // at most one workgroup per compute unit: a wavefront per 32-key block (with two or four workgroups per unit the
    // workgroups below are faster: 16.7 against 15.0 us at 512, 31.8 against 15.4 us at 1024)
    // (with at most 64 keys two of these workgroups fit a compute unit and it wins at any number of blocks: 2048 pairs of
    // 32 x 32 with the weights 73 -> 33 us, 1024 pairs of 64 x 64 40.6 -> 36.2)
    if ((total_quad <= RESIDENT_QUAD_MAX_BLOCKS || a.p.Lkv <= BN) && !no_quad) {
        auto kern = a.p.causal ? (extras ? flash32_resident_quad_kernel<D, true, true> : flash32_resident_quad_kernel<D, true, false>)
                               : (extras ? flash32_resident_quad_kernel<D, false, true> : flash32_resident_quad_kernel<D, false, false>);
        const size_t smem_q = a.p.Lkv <= BN ? smem_quad - 2 * CfgS<D>::TILEB : smem_quad;   // one tile per tensor
        hipLaunchKernelGGL(kern, dim3((unsigned)total_quad), dim3(256), smem_q, st, a);
    } else if (a.p.Lkv > BN) {   // two key tiles: a wavefront per tile and query block
        auto kern = a.p.causal ? (extras ? flash32_resident_pair_kernel<D, true, true> : flash32_resident_pair_kernel<D, true, false>)
                               : (extras ? flash32_resident_pair_kernel<D, false, true> : flash32_resident_pair_kernel<D, false, false>);
        hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(512), smem_pair, st, a);
    } else {
        auto kern = a.p.causal ? (extras ? flash32_resident_kernel<D, true, true> : flash32_resident_kernel<D, true, false>)
                               : (extras ? flash32_resident_kernel<D, false, true> : flash32_resident_kernel<D, false, false>);
        hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(256), smem, st, a);
    }
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <int D, int QB, bool CAUSAL, bool EXTRAS, bool WEIGHTS, bool SPLIT>
int32_t launch_one(const FlashArgs &a, hipStream_t st) {
    const int64_t total = (int64_t)a.n_qtiles * a.p.H * a.p.B * a.nsplit;
    constexpr size_t smem = (SPLIT ? CfgS<D>::SMEM : Cfg<D>::SMEM) + (WEIGHTS ? 4 * FLASH_WSTAGE_BYTES : 0);
    auto kern = flash32_kernel<D, QB, CAUSAL, EXTRAS, WEIGHTS, SPLIT>;
    static bool attr_set = false;
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(256), smem, st, a);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <int D, int QB, bool SPLIT>
int32_t launch_ds(const FlashArgs &a, hipStream_t st, bool extras) {
    const bool w = a.p.weights != nullptr;
    // The 128-wide plane kernel with bias / mask code and the weights output (512 registers and scratch) once took a
    // memory fault after a change that only touched the plane arithmetic, and no cause was found in the source: such
    // calls run on the Float32 instruction, whose kernel has never failed, until one is.
    constexpr bool SPLIT_XW = SPLIT && D != 128;
    if (a.p.causal) {
        if (extras) return w ? launch_one<D, QB, true, true, true, SPLIT_XW>(a, st) : launch_one<D, QB, true, true, false, SPLIT>(a, st);
        return w ? launch_one<D, QB, true, false, true, SPLIT>(a, st) : launch_one<D, QB, true, false, false, SPLIT>(a, st);
    }
    if (extras) return w ? launch_one<D, QB, false, true, true, SPLIT_XW>(a, st) : launch_one<D, QB, false, true, false, SPLIT>(a, st);
    return w ? launch_one<D, QB, false, false, true, SPLIT>(a, st) : launch_one<D, QB, false, false, false, SPLIT>(a, st);
}

// Products on the 16-bit matrix cores through three bf16 planes (see run_tiles32s) unless the caller's
// environment asks for the Float32 matrix instruction (MI355ATTN_F32_MFMA=1).
bool exact_instruction_wanted() {
    static const bool wanted = [] {
        const char *e = getenv("MI355ATTN_F32_MFMA");
        return e && e[0] == '1';
    }();
    return wanted;
}

template <int D, int QB>
int32_t launch_d(const FlashArgs &a, hipStream_t st, bool extras) {
    if (exact_instruction_wanted()) return launch_ds<D, QB, false>(a, st, extras);
    return launch_ds<D, QB, true>(a, st, extras);
}

}  // namespace

int attention_flash32_nsplit(const AttnParams &p) {
    if (flash_is_query_independent_mask(p) || p.Lq > 65535 || p.B > 65535) return 1;   // context lengths instead / merge kernel's grid limits
    return flash_pick_nsplit(p, 128);
}

// context lengths of a key-padding mask, one per (head, batch) pair: workspace of the calls that take that path
size_t attention_flash32_lengths_bytes(const AttnParams &p) {
    if (!flash_is_query_independent_mask(p) || p.H * p.B > 2147483647LL / 4) return 0;
    return ((size_t)(p.H * p.B) * sizeof(int32_t) + 15) & ~(size_t)15;
}

bool attention_flash32_supports(const AttnParams &p) {
    if (p.dtype != MI_F32) return false;
    // head dims: multiples of 4 (16-byte chunks) up to the 128-wide tiles; smaller ones are zero-padded in flight
    if (p.D < 4 || p.Dv < 4 || p.D > 128 || p.Dv > 128 || (p.D & 3) || (p.Dv & 3)) return false;
    auto al = [](const void *x) { return (((uintptr_t)x) & 15) == 0; };
    if (!al(p.q) || !al(p.k) || (p.out && (!al(p.v) || !al(p.out)))) return false;
    const int64_t tiles = (p.Lq + 127) / 128;
    return tiles * p.H * p.B <= 2147483647LL;
}

int32_t launch_attention_flash32(const AttnParams &p, hipStream_t st) {
    FlashArgs a;
    a.p = p;
    a.nsplit = 1;
    a.tiles_per_split = 0;
    a.c = MI_LOG2E;  // q is pre-divided by sqrt(D); only the change of base remains
    a.cn = 1.0f;
    a.n_qtiles = (int32_t)((p.Lq + 127) / 128);
    flash_fill_vec_flags(a);
    const bool narrow = p.D <= 64 && p.Dv <= 64;
    // split-kv as in the 16-bit kernel: few (query tile, head, batch) workgroups and a long key range (calls that
    // measure context lengths are not split: the planner gives their workspace to the lengths)
    a.nsplit = attention_flash32_nsplit(p);
    if (a.nsplit > 1) {
        const int64_t n_tiles = (p.Lkv + BN - 1) / BN;
        a.tiles_per_split = (int32_t)((n_tiles + a.nsplit - 1) / a.nsplit);
        if ((((uintptr_t)p.workspace) & 15) != 0) return mi_set_error(MI_EWORKSPACE, "attention workspace must be 16-byte aligned");
        const bool extras = p.bias || p.mask;
        const int32_t rc = narrow ? launch_d<64, 1>(a, st, extras) : launch_d<128, 1>(a, st, extras);
        if (rc != MI_OK) return rc;
        return launch_flash_merge(p, a.nsplit, st);
    }
    const bool extras = p.bias || p.mask;
    // few keys and the weights returned: everything resident, one pass (flash32_resident_kernel); without the weights
    // when the call leaves most of the chip idle (the workgroup per 32-query block)
    const bool few_blocks = (p.Lq + 31) / 32 * p.H * p.B <= RESIDENT_QUAD_MAX_BLOCKS;
    // at most 64 keys: the workgroup per query block needs 69 KiB of LDS, two fit a compute unit, and it beats the
    // two-pass kernel on any number of pairs up to 1024 blocks, or when a sequence is one block (2048 pairs of 32 x 32:
    // 48 -> 31 us; 512 pairs of 48 x 48: 18.4 -> 15.7; 1024 pairs of 64 x 64 are 25.6 on the two-pass kernel against 32.1)
    const int64_t q_blocks = (p.Lq + 31) / 32 * p.H * p.B;
    const bool short_keys = p.Lkv <= BN && (q_blocks <= 1024 || p.Lq <= 32);
    const bool resident = narrow && (p.weights || few_blocks || short_keys) && p.Lkv <= RES_TILES * BN && !exact_instruction_wanted();
    static const bool no_quad = getenv("MI355ATTN_NO_QUAD") != nullptr;
    // against the two-pass kernel the workgroup per query block still wins at two workgroups per compute unit when the
    // weights are written or the mask is causal (512 blocks of 512 keys: 43 against 58 us with weights, causal 36 against
    // 62; without weights 40 against 36, causal 28 against 41); beyond that it loses
    const int64_t chunk_max = (p.weights || p.causal) ? 2 * RESIDENT_QUAD_MAX_BLOCKS : RESIDENT_QUAD_MAX_BLOCKS;
    const bool chunks = (p.Lq + 31) / 32 * p.H * p.B <= chunk_max && (!narrow || p.Lkv > RES_TILES * BN) && p.Lkv <= (narrow ? RES_CHUNKS_NARROW : RES_CHUNKS) * 128 &&
                        !exact_instruction_wanted() && !no_quad;
    // (calls on few workgroups take a key-padding mask like any other mask: one launch instead of three)
    if (attention_flash32_lengths_bytes(p) != 0 && !((resident && few_blocks && !no_quad) || chunks)) {
        // key-padding mask: classify the (head, batch) pairs on the device, then launch both variants
        int32_t *lens = (int32_t *)p.workspace;
        int32_t rc = launch_key_mask_lengths(p, lens, st);
        if (rc != MI_OK) return rc;
        a.kv_len = lens;
        rc = narrow ? launch_d<64, 1>(a, st, false) : launch_d<128, 1>(a, st, false);
        if (rc != MI_OK) return rc;
        return narrow ? launch_d<64, 1>(a, st, true) : launch_d<128, 1>(a, st, true);
    }
    if (resident) return launch_resident<64>(a, st, extras);
    if (chunks) {
        if (!narrow) return launch_resident_chunks<128, RES_CHUNKS>(a, st, extras);
        return p.Lkv <= RES_CHUNKS * 128 ? launch_resident_chunks<64, RES_CHUNKS>(a, st, extras) : launch_resident_chunks<64, RES_CHUNKS_NARROW>(a, st, extras);
    }
    return narrow ? launch_d<64, 1>(a, st, extras) : launch_d<128, 1>(a, st, extras);
}
