// Tiled strided batched GEMM for bf16 / f16 on MFMA: the fast path of mi_batched_gemm for operands
// whose rows can be moved in 16-byte pieces (aligned bases, leading dimensions and contiguous extents
// that are multiples of 8).  Stands where the reference calls BLAS gemm per slice
// (src/gemm.jl:141-149, reached through _batched_gemm!, src/batched/batchedmul.jl:298).
//
// Workgroup = 4 wavefronts (2 x 2), output tile 128 (m) x 128 (n), 64 x 64 per wavefront as 2 x 2
// MFMA blocks of 32 x 32; k advances 64 per stage through double-buffered LDS tiles.
// Accumulator rows = m, columns = n: a lane holds runs of 4 consecutive m of one C column, lanes l and
// l + 32 complementary runs; they exchange halves and each lane stores 16 contiguous bytes (C rows that
// cannot be written in aligned 16-byte pieces take element stores).
//
// An operand tile is kept in the orientation its memory has:
//   RMAJ  contiguous along its row index (A with 'N', B with 'T'): tile [64 k][128 rows], chunks
//         XOR-swizzled, MFMA operand through the transposing LDS read (the value tile of the
//         attention kernels has exactly this geometry);
//   KMAJ  contiguous along k (A with 'T', B with 'N'): tile [128 rows][64 k], 128-byte rows with
//         XOR-swizzled chunks; the 8-byte halves of each 16-k group are stored in the order
//         k 0-3, 8-11, 4-7, 12-15, so that the MFMA operand is one 16-byte read per lane (measured:
//         ds_read_b128 moves 1.6x the bytes per second of ds_read_b64 and of the transposing read).
// Both deliver the 16 k of a step in the order {0-3, 8-11 | 4-7, 12-15} per half-wave, which is what
// the transposing read produces; A and B only have to agree.
#include "common.h"
#include "flash_common.h"   // flash_dma_1k, FLASH_WAIT_VMCNT, flash_make_rsrc

namespace {

constexpr int KC = 64;
constexpr int KMAJ_ROWB = 128;                 // bytes per row of a KMAJ tile (64 k x 2 bytes)

// Two shapes: SMALL = 128 x 128 output tile, 4 wavefronts of 64 x 64 (2 x 2 MFMA blocks), two workgroups
// per CU; LARGE = 256 x 256 tile, 8 wavefronts of 128 (m) x 64 (n) (4 x 2 blocks), one workgroup per CU:
// twice the MFMAs per barrier, 3/4 of the LDS operand reads per MFMA and half the global and LDS-store
// traffic per FLOP.  Both tiles are square, so A and B tiles have one size and every thread moves four
// 16-byte pieces per tile and stage in either shape.
template <bool LARGE>
struct Shape {
    static constexpr int TILE = LARGE ? 256 : 128;        // rows of an operand tile (m of A, n of B)
    static constexpr int THREADS = LARGE ? 512 : 256;
    static constexpr int WM = 2, WN = LARGE ? 4 : 2;      // wavefront grid
    static constexpr int BM = LARGE ? 4 : 2, BNB = 2;     // 32 x 32 blocks per wavefront along m and n
    static constexpr int RMAJ_ROWB = TILE * 2;            // bytes per k-row of an RMAJ tile
    static constexpr int TILEB = TILE * KMAJ_ROWB;        // bytes per tile and buffer (an RMAJ tile, 64 * RMAJ_ROWB, has the same size)
};

struct Gemm16Args {
    const void *A, *B;
    void *C;
    int64_t m, n, k, lda, ldb, ldc, sA, sB, sC;
    float alpha, beta;
    int32_t c_vec;   // C base, leading dimension, slice stride and m allow aligned 16-byte stores
};

__device__ inline int rmaj_swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
// 128-byte rows: two rows share a bank span, the row parity picks the half, so the 8 row pairs of 16
// consecutive rows need 8 different values for the 16-byte reads of one row per lane
__device__ inline int kmaj_swz(int row) {
    const int x = (row >> 1) & 7;
    return ((x & 1) << 2) | (x >> 1);
}

template <typename T>
__device__ inline typename T::vec4 lds_tr4(const char *p) {
    s16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t *)p);
    return __builtin_bit_cast(typename T::vec4, r);
}

// One operand tile.  The slice is addressed through a buffer resource with 32-bit byte offsets, so that
// loads need no branches (a piece outside the matrix gets an offset past the end of the resource and
// reads as zeros) and the compiler can count outstanding loads exactly: loads run two stages ahead.
// RM: element (row, kk) at X[row + kk*ld]; else at X[kk + row*ld].
template <typename T, bool RM, bool LARGE>
struct Operand {
    typedef typename T::type t;
    static constexpr int THREADS = Shape<LARGE>::THREADS, RMAJ_ROWB = Shape<LARGE>::RMAJ_ROWB;
    static constexpr int CPR = Shape<LARGE>::TILE / 8;   // 16-byte pieces per k-row of an RMAJ tile
    __amdgpu_buffer_rsrc_t rsrc;
    int off[4];          // byte offset of this thread's four pieces at k0 = 0, or OOB for rows past the edge
    int kstep;           // bytes per unit of k0
    int64_t k;
    u32x4_t regs[2][4];  // two stages in flight
    static constexpr int OOB = 0x7fffffff;

    __device__ void init(const t *X, int64_t ld, int64_t rows, int64_t k_, int64_t row0) {
        k = k_;
        const int64_t extent = RM ? (k_ - 1) * ld + rows : (rows - 1) * ld + k_;   // elements the slice spans
        rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)X, 0, (int)(extent * 2), 0x00020000);
        kstep = RM ? (int)(ld * 2) : 2;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int c = threadIdx.x + THREADS * u;
            if (RM) {
                const int kk = c / CPR, r8 = (c % CPR) * 8;     // kk >= k falls past the extent by itself
                off[u] = row0 + r8 < rows ? (int)(((row0 + r8) + kk * ld) * 2) : OOB;
            } else {
                const int r = c >> 3, k8 = (c & 7) * 8;         // 8 pieces per row
                off[u] = row0 + r < rows ? (int)((k8 + (row0 + r) * ld) * 2) : OOB;
            }
        }
    }
    __device__ void load(int set, int64_t k0) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int o = off[u] == OOB ? OOB : off[u] + (int)k0 * kstep;
            if (!RM) {   // a piece past k in a row-contiguous-in-k matrix would read the next row
                const int k8 = ((threadIdx.x + THREADS * u) & 7) * 8;
                o = k0 + k8 < k ? o : OOB;
            }
            regs[set][u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, o, 0, 0);
        }
    }
    __device__ void store(int set, char *tile) const {
        const u32x4_t (&reg)[4] = regs[set];
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int c = tid + THREADS * u;
            if (RM) {
                const int kk = c / CPR, chunk = c % CPR;
                *(u32x4_t *)(tile + kk * RMAJ_ROWB + ((chunk ^ rmaj_swz(kk)) << 4)) = reg[u];
            } else {
                // piece = k 8*chunk .. +7 = half `chunk & 1` of 16-k group `chunk >> 1`: its first four k go to the
                // group's first 16-byte chunk, its last four to the second, at 8-byte slot `half` of either
                const int r = c >> 3, chunk = c & 7, grp = chunk >> 1, half = chunk & 1, sw = kmaj_swz(r);
                u32x2_t lo = {reg[u][0], reg[u][1]}, hi = {reg[u][2], reg[u][3]};
                *(u32x2_t *)(tile + r * KMAJ_ROWB + (((2 * grp) ^ sw) << 4) + 8 * half) = lo;
                *(u32x2_t *)(tile + r * KMAJ_ROWB + (((2 * grp + 1) ^ sw) << 4) + 8 * half) = hi;
            }
        }
    }
    // MFMA operand of the 32-row block `blk` of the tile for k-step `ks` (0..3)
    __device__ static typename T::vec8 fetch(const char *tile, int blk, int ks, int lane) {
        const int hh = lane >> 5;
        if (RM) {
            const int vrow = 4 * hh + ((lane & 15) >> 2);
            const int vchunk = 4 * blk + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), vsub = 8 * (lane & 1);
            const char *src = tile + (16 * ks + vrow) * RMAJ_ROWB + vsub;
            const typename T::vec4 lo = lds_tr4<T>(src + ((vchunk ^ rmaj_swz(vrow)) << 4));
            const typename T::vec4 hi = lds_tr4<T>(src + 8 * RMAJ_ROWB + ((vchunk ^ rmaj_swz(vrow + 8)) << 4));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            const int row = 32 * blk + (lane & 31);   // k 4hh .. 4hh+3 and 8+4hh .. 8+4hh+3 of the step
            return *(const typename T::vec8 *)(tile + row * KMAJ_ROWB + (((2 * ks + hh) ^ kmaj_swz(row)) << 4));
        }
    }
};

// Writes a workgroup's accumulators: C = alpha * acc + beta * C.  acc[n block][m block] of the wavefront at (wm, wn) of the
// workgroup's grid; the tile starts at (m0, n0) of slice bz.
template <typename T, bool LARGE>
__device__ inline void store_tile(const Gemm16Args &g, const floatx16_t (&acc)[Shape<LARGE>::BNB][Shape<LARGE>::BM], int64_t bz, int64_t m0,
                                  int64_t n0, int wm, int wn, int lane) {
    typedef typename T::type t;
    typedef Shape<LARGE> S;
    constexpr int BM = S::BM, BNB = S::BNB;
    const int r = lane & 31, hh = lane >> 5;
    // accumulator register v of lane (r, hh) of block (i, j): m = 32j + 8*(v/4) + 4*hh + v%4, n = 32i + r
    t *C = (t *)g.C + bz * g.sC;
    const bool vec_ok = g.c_vec != 0;   // C columns can be written in aligned 16-byte pieces
#pragma unroll
    for (int i = 0; i < BNB; i++) {
        const int64_t nj = n0 + 32 * BNB * wn + 32 * i + r;
        t *ccol = C + (nj < g.n ? nj : 0) * g.ldc;
#pragma unroll
        for (int j = 0; j < BM; j++)
#pragma unroll
            for (int gp = 0; gp < 2; gp++) {
                // X: m = mb + 4hh .. +3 (v = 8gp ..), Y: m = mb + 8 + 4hh .. +3 (v = 8gp + 4 ..)
                const int64_t mb = m0 + 32 * BM * wm + 32 * j + 16 * gp;
                float xv[4], yv[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    xv[e] = g.alpha * acc[i][j][8 * gp + e];
                    yv[e] = g.alpha * acc[i][j][8 * gp + 4 + e];
                }
                if (vec_ok) {
                    if (g.beta != 0.0f && nj < g.n) {
                        if (mb + 4 * hh < g.m) {
                            const typename T::vec4 c4 = *(const typename T::vec4 *)(ccol + mb + 4 * hh);
#pragma unroll
                            for (int e = 0; e < 4; e++) xv[e] += g.beta * T::to_f32(c4[e]);
                        }
                        if (mb + 8 + 4 * hh < g.m) {
                            const typename T::vec4 c4 = *(const typename T::vec4 *)(ccol + mb + 8 + 4 * hh);
#pragma unroll
                            for (int e = 0; e < 4; e++) yv[e] += g.beta * T::to_f32(c4[e]);
                        }
                    }
                    typename T::vec4 xe, yo;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        xe[e] = T::from_f32(xv[e]);
                        yo[e] = T::from_f32(yv[e]);
                    }
                    const u32x2_t x = __builtin_bit_cast(u32x2_t, xe), y = __builtin_bit_cast(u32x2_t, yo);
                    uint32_t x0 = x[0], x1 = x[1], y0 = y[0], y1 = y[1];
                    mi_pair_halves(x0, y0);   // every lane takes part; lanes outside C do not store
                    mi_pair_halves(x1, y1);
                    const u32x4_t piece = {x0, x1, y0, y1};
                    if (nj < g.n && mb + 8 * hh < g.m) *(u32x4_t *)(ccol + mb + 8 * hh) = piece;   // m is a multiple of 8 here
                } else if (nj < g.n) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int64_t mx = mb + 4 * hh + e, my = mx + 8;
                        if (mx < g.m) ccol[mx] = T::from_f32(g.beta != 0.0f ? xv[e] + g.beta * T::to_f32(ccol[mx]) : xv[e]);
                        if (my < g.m) ccol[my] = T::from_f32(g.beta != 0.0f ? yv[e] + g.beta * T::to_f32(ccol[my]) : yv[e]);
                    }
                }
            }
    }
}

template <typename T, bool A_RM, bool B_RM, bool LARGE>
__global__ __launch_bounds__(Shape<LARGE>::THREADS, LARGE ? 1 : 2) void gemm16_kernel(Gemm16Args g) {
    typedef typename T::type t;
    typedef Shape<LARGE> S;
    constexpr int TILEB = S::TILEB, BM = S::BM, BNB = S::BNB;
    extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];
    char *As = (char *)gemm_smem, *Bs = As + 2 * TILEB;
    // which tile: an order in which the tiles in flight on one die share operands (mi_gemm_tile_order)
    const MiTile tile = mi_gemm_tile_order(blockIdx.x + (int64_t)gridDim.x * (blockIdx.y + (int64_t)gridDim.y * blockIdx.z), gridDim.x, gridDim.y, gridDim.z);
    const int64_t bx = tile.m, by = tile.n, bz = tile.batch;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave % S::WM, wn = wave / S::WM;
    const int r = lane & 31, hh = lane >> 5;

    Operand<T, A_RM, LARGE> a;
    Operand<T, B_RM, LARGE> b;
    const int64_t m0 = bx * S::TILE, n0 = by * S::TILE;
    a.init((const t *)g.A + bz * g.sA, g.lda, g.m, g.k, m0);
    b.init((const t *)g.B + bz * g.sB, g.ldb, g.n, g.k, n0);

    floatx16_t acc[BNB][BM];   // [n block][m block]
#pragma unroll
    for (int i = 0; i < BNB; i++)
#pragma unroll
        for (int j = 0; j < BM; j++) acc[i][j] = (floatx16_t){0};

    // Loads run two stages ahead of the MFMAs (one stage of MFMAs is shorter than the latency of the loads
    // behind it): stage it+1 sits in LDS or in register set (it+1)&1, stage it+2 is in flight into the
    // other set.
    const int nk = (int)((g.k + KC - 1) / KC);
    a.load(0, 0);
    b.load(0, 0);
    a.store(0, As);
    b.store(0, Bs);
    a.load(1, KC);
    b.load(1, KC);
    __syncthreads();
    auto stage = [&](int it, int set_next) {   // set_next = (it + 1) & 1, a compile-time constant at each call site
        const int buf = it & 1;
        // unconditional: past the last stage every piece is out of range and reads as zeros, and a load that is
        // always issued lets the compiler wait for exactly the older set (vmcnt(8)) before the LDS stores below
        a.load(set_next ^ 1, (int64_t)(it + 2) * KC);
        b.load(set_next ^ 1, (int64_t)(it + 2) * KC);
        const char *at = As + buf * TILEB, *bt = Bs + buf * TILEB;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            typename T::vec8 av[BM], bv[BNB];
#pragma unroll
            for (int j = 0; j < BM; j++) av[j] = Operand<T, A_RM, LARGE>::fetch(at, BM * wm + j, ks, lane);
#pragma unroll
            for (int i = 0; i < BNB; i++) bv[i] = Operand<T, B_RM, LARGE>::fetch(bt, BNB * wn + i, ks, lane);
#pragma unroll
            for (int i = 0; i < BNB; i++)
#pragma unroll
                for (int j = 0; j < BM; j++) acc[i][j] = T::mfma32(av[j], bv[i], acc[i][j]);
        }
        if (it + 1 < nk) {
            a.store(set_next, As + (buf ^ 1) * TILEB);
            b.store(set_next, Bs + (buf ^ 1) * TILEB);
        }
        __syncthreads();
    };
    int it = 0;
    for (; it + 1 < nk; it += 2) {
        stage(it, 1);
        stage(it + 1, 0);
    }
    if (it < nk) stage(it, 1);

    store_tile<T, LARGE>(g, acc, bz, m0, n0, wm, wn, lane);
}

// ---- the 256 x 256 tile with the operand tiles copied global -> LDS by the DMA path ---------------------------------
// Same output tile and wavefront grid as the LARGE shape above; what changes is how the operand tiles arrive: with
// buffer_load ... lds into a ring of four stages of 32 k each (16 KiB per operand and stage, 128 KiB in all), two stages
// ahead of their use, one workgroup barrier per two stages.  No staging registers, no LDS stores issued by the
// wavefronts, and the copies of later stages land while the matrix instructions of the current one run; the
// register-staged kernel above stores a whole stage to LDS between the last matrix instruction of one stage and the
// barrier, which every wavefront of the CU then waits behind.
// Tile layouts (a DMA piece is 16 bytes per lane, 1 KiB per instruction, lane l at byte 16 l of the piece):
//   RMAJ  [32 k][256 rows]: 512-byte k-rows, 16-byte chunks XOR-swizzled by the k-row; operand through the transposing
//         read, here with each half-wave taking 8 consecutive k (rows 8 hh .. 8 hh + 7 of the 16-k step);
//   KMAJ  [256 rows][32 k]: 64-byte rows of four 16-byte chunks (8 consecutive k each), chunk XOR (row / 4) % 4;
//         operand = one 16-byte read per lane.
// Both deliver k 8 hh .. 8 hh + 7 to half-wave hh, so any pair of layouts agrees.
constexpr int RK = 32;                        // k per stage
constexpr int RING = 4;
template <bool LARGE>
struct RingShape {
    static constexpr int TILE = Shape<LARGE>::TILE;
    static constexpr int TILEB = TILE * RK * 2;                // bytes per operand and stage: 16 KiB (8 KiB for the 128 x 128 shape)
    static constexpr int ROWB = TILE * 2;                      // bytes per k-row of an RMAJ tile
    static constexpr size_t SMEM = 2 * RING * TILEB;           // 128 KiB, one workgroup per CU (64 KiB, two)
};

__device__ inline int ring_kswz(int row) { return (row >> 2) & 3; }

template <typename T, bool RM, bool LARGE>
struct RingOperand {
    typedef typename T::type t;
    static constexpr int TILEB = RingShape<LARGE>::TILEB, ROWB = RingShape<LARGE>::ROWB;
    static constexpr int CPR = ROWB / 16;   // 16-byte chunks per k-row of an RMAJ tile; a 1 KiB piece holds 64 / CPR k-rows
    i32x4_t rsrc;
    int voff[2];     // byte offsets of this lane's two pieces of a stage at k0 = 0 (0x80000000: outside the matrix)
    int kpiece[2];   // first k of the piece within the stage (to drop pieces past k)
    int kstep;       // bytes per unit of k0
    int64_t k;
    unsigned lds;    // LDS byte address of this wavefront's first piece in stage 0
    static constexpr int OOB = (int)0x80000000;

    __device__ void init(const t *X, int64_t ld, int64_t rows, int64_t k_, int64_t row0, char *ring, int wave, int lane) {
        k = k_;
        const int64_t extent = RM ? (k_ - 1) * ld + rows : (rows - 1) * ld + k_;
        rsrc = flash_make_rsrc(X, (uint32_t)(extent * 2));
        kstep = RM ? (int)(ld * 2) : 2;
        lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char *)ring + wave * 2048;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int piece = 2 * wave + i;   // TILEB / 1024 pieces per operand and stage, two per wavefront
            if (RM) {
                const int krow = (64 / CPR) * piece + lane / CPR, chunk = (lane % CPR) ^ rmaj_swz(krow);
                kpiece[i] = krow;
                voff[i] = row0 + 8 * chunk < rows ? (int)(((row0 + 8 * chunk) + krow * ld) * 2) : OOB;
            } else {
                const int row = 16 * piece + (lane >> 2), chunk = (lane & 3) ^ ring_kswz(row);
                kpiece[i] = 8 * chunk;
                voff[i] = row0 + row < rows ? (int)((8 * chunk + (row0 + row) * ld) * 2) : OOB;
            }
        }
    }
    // start the copy of the stage whose first k is k0 into ring position `pos`
    __device__ void issue(int pos, int64_t k0) const {
        const unsigned dst = __builtin_amdgcn_readfirstlane(lds + pos * TILEB);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            int o = voff[i] == OOB ? OOB : voff[i] + (int)k0 * kstep;
            o = k0 + kpiece[i] < k ? o : OOB;   // a piece past k would read the next row (KMAJ) or wrap the 32-bit offset (RMAJ)
            flash_dma_1k(rsrc, dst + i * 1024, o);
        }
    }
    // MFMA operand of the 32-row block `blk` of the stage at `tile` for k-step ks (0, 1): k 16 ks + 8 hh .. + 7
    __device__ static typename T::vec8 fetch(const char *tile, int blk, int ks, int lane) {
        const int hh = lane >> 5;
        if (RM) {
            const int vrow = 16 * ks + 8 * hh + ((lane & 15) >> 2);
            const int vchunk = 4 * blk + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), vsub = 8 * (lane & 1);
            const char *src = tile + vrow * ROWB + vsub;
            const typename T::vec4 lo = lds_tr4<T>(src + ((vchunk ^ rmaj_swz(vrow)) << 4));
            const typename T::vec4 hi = lds_tr4<T>(src + 4 * ROWB + ((vchunk ^ rmaj_swz(vrow + 4)) << 4));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            const int row = 32 * blk + (lane & 31);
            return *(const typename T::vec8 *)(tile + row * 64 + (((2 * ks + hh) ^ ring_kswz(row)) << 4));
        }
    }
};

template <typename T, bool A_RM, bool B_RM, bool LARGE>
__global__ __launch_bounds__(Shape<LARGE>::THREADS, LARGE ? 1 : 2) void gemm16_ring_kernel(Gemm16Args g) {
    typedef typename T::type t;
    typedef Shape<LARGE> S;
    constexpr int BM = S::BM, BNB = S::BNB, RTILEB = RingShape<LARGE>::TILEB;
    extern __shared__ __attribute__((aligned(1024))) unsigned char gemm_smem[];
    char *As = (char *)gemm_smem, *Bs = As + RING * RTILEB;
    const MiTile tile = mi_gemm_tile_order(blockIdx.x + (int64_t)gridDim.x * (blockIdx.y + (int64_t)gridDim.y * blockIdx.z), gridDim.x, gridDim.y, gridDim.z);
    const int64_t bz = tile.batch, m0 = tile.m * S::TILE, n0 = tile.n * S::TILE;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wm = wave % S::WM, wn = wave / S::WM;

    RingOperand<T, A_RM, LARGE> a;
    RingOperand<T, B_RM, LARGE> b;
    a.init((const t *)g.A + bz * g.sA, g.lda, g.m, g.k, m0, As, wave, lane);
    b.init((const t *)g.B + bz * g.sB, g.ldb, g.n, g.k, n0, Bs, wave, lane);

    floatx16_t acc[BNB][BM];
#pragma unroll
    for (int i = 0; i < BNB; i++)
#pragma unroll
        for (int j = 0; j < BM; j++) acc[i][j] = (floatx16_t){0};

    // Stage s lives in ring position s % 4.  An even stage starts with "stages s and s + 1 have landed everywhere and
    // stages s - 2 and s - 1 are read by nobody any more"; every stage then requests stage s + 2.
    const int ns = (int)((g.k + RK - 1) / RK);
    a.issue(0, 0);
    b.issue(0, 0);
    a.issue(1, RK);
    b.issue(1, RK);
    for (int st = 0; st < ns; st++) {
        if ((st & 1) == 0) {
            FLASH_WAIT_VMCNT(0);
            asm volatile("" ::: "memory");
            __syncthreads();
        }
        if (st + 2 < ns) {
            a.issue((st + 2) & 3, (int64_t)(st + 2) * RK);
            b.issue((st + 2) & 3, (int64_t)(st + 2) * RK);
        }
        const char *at = As + (st & 3) * RTILEB, *bt = Bs + (st & 3) * RTILEB;
#pragma unroll
        for (int ks = 0; ks < RK / 16; ks++) {
            typename T::vec8 av[BM], bv[BNB];
#pragma unroll
            for (int j = 0; j < BM; j++) av[j] = RingOperand<T, A_RM, LARGE>::fetch(at, BM * wm + j, ks, lane);
#pragma unroll
            for (int i = 0; i < BNB; i++) bv[i] = RingOperand<T, B_RM, LARGE>::fetch(bt, BNB * wn + i, ks, lane);
#pragma unroll
            for (int i = 0; i < BNB; i++)
#pragma unroll
                for (int j = 0; j < BM; j++) acc[i][j] = T::mfma32(av[j], bv[i], acc[i][j]);
        }
    }
    store_tile<T, LARGE>(g, acc, bz, m0, n0, wm, wn, lane);
}

template <typename T, bool A_RM, bool B_RM, bool LARGE>
int32_t launch_ring(const Gemm16Args &g, int64_t nb, hipStream_t st) {
    typedef Shape<LARGE> S;
    auto kern = gemm16_ring_kernel<T, A_RM, B_RM, LARGE>;
    constexpr size_t smem = RingShape<LARGE>::SMEM;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, so a race is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    dim3 grid((unsigned)((g.m + S::TILE - 1) / S::TILE), (unsigned)((g.n + S::TILE - 1) / S::TILE), (unsigned)nb);
    hipLaunchKernelGGL(kern, grid, dim3(S::THREADS), smem, st, g);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <typename T, bool LARGE>
int32_t launch_ring_l(const Gemm16Args &g, int transA, int transB, int64_t nb, hipStream_t st) {
    const bool a_rm = !transA, b_rm = transB != 0;
    if (a_rm) return b_rm ? launch_ring<T, true, true, LARGE>(g, nb, st) : launch_ring<T, true, false, LARGE>(g, nb, st);
    return b_rm ? launch_ring<T, false, true, LARGE>(g, nb, st) : launch_ring<T, false, false, LARGE>(g, nb, st);
}

template <typename T, bool A_RM, bool B_RM, bool LARGE>
int32_t launch_one(const Gemm16Args &g, int64_t nb, hipStream_t st) {
    typedef Shape<LARGE> S;
    auto kern = gemm16_kernel<T, A_RM, B_RM, LARGE>;
    constexpr size_t smem = 4 * S::TILEB;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, so a race is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    dim3 grid((unsigned)((g.m + S::TILE - 1) / S::TILE), (unsigned)((g.n + S::TILE - 1) / S::TILE), (unsigned)nb);
    hipLaunchKernelGGL(kern, grid, dim3(S::THREADS), smem, st, g);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <typename T, bool LARGE>
int32_t launch_l(const Gemm16Args &g, int transA, int transB, int64_t nb, hipStream_t st) {
    const bool a_rm = !transA, b_rm = transB != 0;
    if (a_rm) return b_rm ? launch_one<T, true, true, LARGE>(g, nb, st) : launch_one<T, true, false, LARGE>(g, nb, st);
    return b_rm ? launch_one<T, false, true, LARGE>(g, nb, st) : launch_one<T, false, false, LARGE>(g, nb, st);
}

template <typename T>
int32_t launch_t(const Gemm16Args &g, int transA, int transB, int64_t nb, hipStream_t st) {
    // the large tile when it still gives every CU a workgroup; the small one otherwise
    const int64_t big = ((g.m + 255) / 256) * ((g.n + 255) / 256) * nb;
    static const bool no_ring = getenv("MI355ATTN_GEMM_NO_RING") != nullptr;   // A/B switch: the register-staged kernels
    const bool large = g.m >= 256 && g.n >= 256 && big >= 256;
    // the ring kernel for the large shape only: at 128 x 128 it was measured level or behind the register-staged kernel
    // (128 x 4096 x 4096 x 64: 593 against 637 TFLOP/s, 64 x 2048 x 2048 x 64: 252 / 290, 1024^3 x 4: 607 / 573)
    if (large) return no_ring ? launch_l<T, true>(g, transA, transB, nb, st) : launch_ring_l<T, true>(g, transA, transB, nb, st);
    return launch_l<T, false>(g, transA, transB, nb, st);
}

}  // namespace

// true when every 16-byte piece the kernel moves is aligned and wholly inside or outside its matrix
bool batched_gemm16_supports(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, const void *A, int64_t lda,
                             int64_t sA, const void *B, int64_t ldb, int64_t sB) {
    if (dtype != MI_F16 && dtype != MI_BF16) return false;
    if (k < 1 || m * n < 64 * 64) return false;   // tiny products: the small-tile kernel wastes less
    auto al = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if (!al(A) || !al(B) || (lda & 7) || (ldb & 7) || (sA & 7) || (sB & 7)) return false;
    if ((transA ? k : m) & 7) return false;
    if ((transB ? n : k) & 7) return false;
    // slices are addressed with 32-bit byte offsets
    const int64_t extA = transA ? (m - 1) * lda + k : (k - 1) * lda + m, extB = transB ? (k - 1) * ldb + n : (n - 1) * ldb + k;
    if (extA * 2 >= 2147483647LL || extB * 2 >= 2147483647LL) return false;
    return (n + 127) / 128 <= 65535;
}

int32_t launch_batched_gemm16(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                              int64_t lda, int64_t sA, const void *B, int64_t ldb, int64_t sB, float beta, void *C, int64_t ldc,
                              int64_t sC, int64_t batch, hipStream_t st) {
    const size_t es = 2;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {   // gridDim.z is limited to 65535: issue the batch in slabs
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        Gemm16Args g = {(const char *)A + es * b0 * sA, (const char *)B + es * b0 * sB, (char *)C + es * b0 * sC,
                        m, n, k, lda, ldb, ldc, sA, sB, sC, alpha, beta,
                        (int32_t)((((uintptr_t)C) & 15) == 0 && (ldc & 7) == 0 && (sC & 7) == 0 && (m & 7) == 0)};
        const int32_t rc = dtype == MI_F16 ? launch_t<F16>(g, transA, transB, nb, st) : launch_t<BF16>(g, transA, transB, nb, st);
        if (rc != MI_OK) return rc;
    }
    return MI_OK;
}
