// Tiled strided batched GEMM for Float32 on the fp32 matrix cores (v_mfma_f32_32x32x2_f32): the fast
// path of mi_batched_gemm for operands whose rows can be moved in 16-byte pieces.  Stands where the
// reference calls sgemm per slice (src/gemm.jl:141-149, reached through _batched_gemm!,
// src/batched/batchedmul.jl:298).  Products and sums are true fp32.
//
// Workgroup = 4 wavefronts (2 x 2), output tile 128 (m) x 128 (n), 64 x 64 per wavefront as 2 x 2 MFMA
// blocks; k advances 16 per stage through double-buffered LDS tiles kept as [k][row] (row contiguous),
// so an MFMA operand (one float per lane: row = lane % 32, k = 2*step + lane / 32) is a conflict-free
// 4-byte read whatever the memory layout of the matrix.  As in the other GEMM kernels the MFMA runs on
// the transposed problem so that a half-wave stores 32 consecutive elements of a C column.
#include "common.h"
#include <cstdlib>

namespace {

constexpr int TM = 128, TN = 128, KC = 16;
constexpr int LDT = 128 + 4;   // floats per k-row of a tile (+4: the strided stores of k-contiguous operands spread over banks)

struct Gemm32Args {
    const float *A, *B;
    float *C;
    int64_t m, n, k, lda, ldb, ldc, sA, sB, sC;
    float alpha, beta;
    int32_t c_vec;   // C base, leading dimension, slice stride and m allow aligned 16-byte stores
};

// RM: element (row, kk) at X[row + kk*ld] (contiguous along row); else at X[kk + row*ld]
template <bool RM>
struct Operand32 {
    const float *X;
    int64_t ld, rows, k, row0;
    floatx4_t reg[2];   // 512 pieces of 16 bytes per tile, 2 per thread

    __device__ void load(int64_t k0) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = tid + 256 * u;
            const floatx4_t z = {0.f, 0.f, 0.f, 0.f};
            if (RM) {
                const int kk = c >> 5, r4 = (c & 31) * 4;     // 32 pieces per k-row
                reg[u] = (k0 + kk < k && row0 + r4 < rows) ? *(const floatx4_t *)(X + (row0 + r4) + (k0 + kk) * ld) : z;
            } else {
                const int r = c >> 2, k4 = (c & 3) * 4;       // 4 pieces per row
                reg[u] = (row0 + r < rows && k0 + k4 < k) ? *(const floatx4_t *)(X + (k0 + k4) + (row0 + r) * ld) : z;
            }
        }
    }
    __device__ void store(float *tile) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = tid + 256 * u;
            if (RM) {
                const int kk = c >> 5, r4 = (c & 31) * 4;
                *(floatx4_t *)(tile + kk * LDT + r4) = reg[u];
            } else {
                const int r = c >> 2, k4 = (c & 3) * 4;
#pragma unroll
                for (int e = 0; e < 4; e++) tile[(k4 + e) * LDT + r] = reg[u][e];
            }
        }
    }
};

template <bool A_RM, bool B_RM>
__global__ __launch_bounds__(256, 2) void gemm32_kernel(Gemm32Args g) {
    __shared__ __attribute__((aligned(16))) float As[2][KC * LDT];
    __shared__ __attribute__((aligned(16))) float Bs[2][KC * LDT];
    const int64_t bz = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
    const int r = lane & 31, hh = lane >> 5;

    Operand32<A_RM> a;
    Operand32<B_RM> b;
    a.X = g.A + bz * g.sA;
    a.ld = g.lda;
    a.rows = g.m;
    a.k = g.k;
    a.row0 = (int64_t)blockIdx.x * TM;
    b.X = g.B + bz * g.sB;
    b.ld = g.ldb;
    b.rows = g.n;
    b.k = g.k;
    b.row0 = (int64_t)blockIdx.y * TN;

    floatx16_t acc[2][2];   // [n block][m block]
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = (floatx16_t){0};

    const int nk = (int)((g.k + KC - 1) / KC);
    a.load(0);
    b.load(0);
    a.store(As[0]);
    b.store(Bs[0]);
    __syncthreads();
    for (int it = 0; it < nk; it++) {
        const int buf = it & 1;
        if (it + 1 < nk) {
            a.load((int64_t)(it + 1) * KC);
            b.load((int64_t)(it + 1) * KC);
        }
        const float *at = As[buf] + 64 * wm + r, *bt = Bs[buf] + 64 * wn + r;
#pragma unroll
        for (int ks = 0; ks < KC / 2; ks++) {
            float av[2], bv[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                av[j] = at[(2 * ks + hh) * LDT + 32 * j];
                bv[j] = bt[(2 * ks + hh) * LDT + 32 * j];
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[i], av[j], acc[i][j], 0, 0, 0);
        }
        if (it + 1 < nk) {
            a.store(As[buf ^ 1]);
            b.store(Bs[buf ^ 1]);
        }
        __syncthreads();
    }

    // accumulator register v of lane (r, hh) of block (i, j): n = 32i + 8*(v/4) + 4*hh + v%4, m = 32j + r
    float *C = g.C + bz * g.sC;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int64_t mi = a.row0 + 64 * wm + 32 * j + r;
        if (mi >= g.m) continue;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t nj = b.row0 + 64 * wn + 32 * i + 8 * (v / 4) + 4 * hh + (v % 4);
                if (nj < g.n) {
                    float *c = C + mi + nj * g.ldc;
                    float val = g.alpha * acc[i][j][v];
                    if (g.beta != 0.0f) val += g.beta * *c;
                    *c = val;
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------------
// The same product on the 16-bit matrix cores: both operands as three bf16 planes (see common.h), six
// v_mfma_f32_32x32x16_bf16 per 32x32x16 block.  Same workgroup shape and double-buffered 16-k stages; a tile
// is split when it is stored to LDS and keeps the orientation its memory has, as in the 16-bit kernel:
//   RMAJ (contiguous along its row index): [16 k][rows] per plane, k-rows of 2 bytes per row with swizzled
//        16-byte chunks, MFMA operand through the transposing LDS read;
//   KMAJ (contiguous along k): [rows][16 k] per plane, 32-byte rows whose two 16-byte chunks hold
//        k {0-3, 8-11} and {4-7, 12-15}, the order in which the transposing read delivers a step to the two
//        half-waves; the operand is one 16-byte read.
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef bf16x8_t plane8;
typedef bf16x4_t plane4;
// Two shapes, as in the 16-bit kernel: 128 x 128 output tiles on 4 wavefronts (64 x 64 each, two or three
// workgroups per CU), and 256 x 256 on 8 wavefronts (128 (m) x 64 (n) each, one workgroup per CU), which splits every
// operand element for twice as many products and reads 3/4 of the LDS operands per matrix instruction.
template <bool LARGE>
struct ShapeS {
    static constexpr int TILE = LARGE ? 256 : 128;       // rows of an operand tile (m of A, n of B)
    static constexpr int THREADS = LARGE ? 512 : 256;
    static constexpr int BM = LARGE ? 4 : 2, BNB = 2;     // 32 x 32 blocks per wavefront along m and n
    static constexpr int RMAJ_ROWB = TILE * 2;            // bytes per k-row of an RMAJ plane
    static constexpr int PLANEB = TILE * KC * 2;          // bytes of one plane of one operand tile
    static constexpr int TILE3B = 3 * PLANEB;
};

__device__ inline int rmaj_swz(int kk) { return ((kk & 3) << 2) | ((kk >> 2) & 3); }

template <bool RM, bool LARGE>
struct OperandS {
    typedef ShapeS<LARGE> S;
    static constexpr int ROWB = S::RMAJ_ROWB, PLANEB = S::PLANEB, CPR = S::TILE / 4;   // float4 pieces per k-row
    const float *X;
    int64_t ld, rows, k, row0;
    floatx4_t reg[2];   // TILE * KC / 4 pieces per tile: 2 per thread in either shape

    __device__ void load(int64_t k0) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = tid + S::THREADS * u;
            const floatx4_t z = {0.f, 0.f, 0.f, 0.f};
            if (RM) {
                const int kk = c / CPR, r4 = (c % CPR) * 4;
                reg[u] = (k0 + kk < k && row0 + r4 < rows) ? *(const floatx4_t *)(X + (row0 + r4) + (k0 + kk) * ld) : z;
            } else {
                const int r = c >> 2, k4 = (c & 3) * 4;       // 4 pieces per row
                reg[u] = (row0 + r < rows && k0 + k4 < k) ? *(const floatx4_t *)(X + (k0 + k4) + (row0 + r) * ld) : z;
            }
        }
    }
    // split into planes; `tile` is the LDS byte address of the hi plane
    __device__ void store(unsigned tile) const {
        typedef __attribute__((address_space(3))) u32x2_t *lds8_t;
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = tid + S::THREADS * u;
            const floatx4_t x = reg[u];
            uint32_t pl[3][2];
            split3_pair(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
            split3_pair(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
            if (mi_plane_word_special(pl[0][0]) || mi_plane_word_special(pl[0][1])) {   // an Inf, a NaN or a value beyond the bf16 range among the four (rare)
                split3_pair_wide(x[0], x[1], pl[0][0], pl[1][0], pl[2][0]);
                split3_pair_wide(x[2], x[3], pl[0][1], pl[1][1], pl[2][1]);
            }
            unsigned at;
            if (RM) {
                const int kk = c / CPR, r4 = (c % CPR) * 4;   // rows r4 .. r4+3 of k-row kk
                at = (unsigned)(kk * ROWB + ((((r4 >> 3) ^ rmaj_swz(kk)) << 4) + (r4 & 7) * 2));
            } else {
                const int r = c >> 2, k4 = (c & 3) * 4;       // k k4 .. k4+3 of row r: chunk (k4/4)%2, 8-byte slot k4/8
                at = (unsigned)(r * 32 + (((((k4 >> 2) & 1) ^ ((r >> 3) & 1)) << 4) + 8 * (k4 >> 3)));
            }
#pragma unroll
            for (int q = 0; q < 3; q++) *(lds8_t)(uintptr_t)(tile + at + q * PLANEB) = (u32x2_t){pl[q][0], pl[q][1]};
        }
    }
    // the three planes of the MFMA operand of the 32-row block `blk`
    __device__ static void fetch(unsigned tile, int blk, int lane, plane8 (&out)[3]) {
        const int hh = lane >> 5;
        if (RM) {
            const int vrow = 4 * hh + ((lane & 15) >> 2);
            const int vchunk = 4 * blk + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), vsub = 8 * (lane & 1);
            const unsigned lo_at = tile + (unsigned)(vrow * ROWB + vsub + ((vchunk ^ rmaj_swz(vrow)) << 4));
            const unsigned hi_at = tile + (unsigned)((vrow + 8) * ROWB + vsub + ((vchunk ^ rmaj_swz(vrow + 8)) << 4));
#pragma unroll
            for (int q = 0; q < 3; q++) {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t *)(uintptr_t)(lo_at + q * PLANEB));
                const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t *)(uintptr_t)(hi_at + q * PLANEB));
                out[q] = __builtin_shufflevector(__builtin_bit_cast(plane4, lo), __builtin_bit_cast(plane4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
            }
        } else {
            const int row = 32 * blk + (lane & 31);
            const unsigned at = tile + (unsigned)(row * 32 + ((hh ^ ((row >> 3) & 1)) << 4));
#pragma unroll
            for (int q = 0; q < 3; q++) out[q] = *(__attribute__((address_space(3))) const plane8 *)(uintptr_t)(at + q * PLANEB);
        }
    }
};

template <bool A_RM, bool B_RM, bool LARGE>
__global__ __launch_bounds__(ShapeS<LARGE>::THREADS, LARGE ? 1 : 2) void gemm32s_kernel(Gemm32Args g) {
    typedef ShapeS<LARGE> S;
    constexpr int TILE3B = S::TILE3B, BM = S::BM, BNB = S::BNB;
    extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];   // A and B tiles, two buffers each
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)gemm_smem;
    // which tile: with the large tiles, an order in which the tiles in flight on one die share operands (a few per cent
    // on k >= 1024; the small tiles' calls are bound by their output and lose 1 % to it)
    const int64_t id = blockIdx.x + (int64_t)gridDim.x * (blockIdx.y + (int64_t)gridDim.y * blockIdx.z);
    const MiTile tile = LARGE ? mi_gemm_tile_order(id, gridDim.x, gridDim.y, gridDim.z) : MiTile{blockIdx.x, blockIdx.y, blockIdx.z};
    const int64_t bz = tile.batch;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
    const int r = lane & 31, hh = lane >> 5;

    OperandS<A_RM, LARGE> a;
    OperandS<B_RM, LARGE> b;
    a.X = g.A + bz * g.sA;
    a.ld = g.lda;
    a.rows = g.m;
    a.k = g.k;
    a.row0 = tile.m * S::TILE;
    b.X = g.B + bz * g.sB;
    b.ld = g.ldb;
    b.rows = g.n;
    b.k = g.k;
    b.row0 = tile.n * S::TILE;

    floatx16_t acc[BNB][BM];   // [n block][m block]
#pragma unroll
    for (int i = 0; i < BNB; i++)
#pragma unroll
        for (int j = 0; j < BM; j++) acc[i][j] = (floatx16_t){0};

    // One stage of loads in flight.  Three (two more register sets) measured 0.25 against 0.19 ms on the
    // 1024 x 64 x 1024 x 128 product with the small shape: the registers cost the third workgroup per CU.
    const int nk = (int)((g.k + KC - 1) / KC);
    a.load(0);
    b.load(0);
    a.store(lds0);
    b.store(lds0 + 2 * TILE3B);
    __syncthreads();
    for (int it = 0; it < nk; it++) {
        const int buf = it & 1;
        if (it + 1 < nk) {
            a.load((int64_t)(it + 1) * KC);
            b.load((int64_t)(it + 1) * KC);
        }
        const unsigned at = lds0 + buf * TILE3B, bt = lds0 + (2 + buf) * TILE3B;
        plane8 av[BM][3], bv[BNB][3];
#pragma unroll
        for (int j = 0; j < BM; j++) OperandS<A_RM, LARGE>::fetch(at, BM * wm + j, lane, av[j]);
#pragma unroll
        for (int i = 0; i < BNB; i++) OperandS<B_RM, LARGE>::fetch(bt, BNB * wn + i, lane, bv[i]);
        // the transposed problem (rows = n, columns = m), small terms first
        constexpr int ia[6] = {2, 0, 1, 1, 0, 0}, ib[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
        for (int t = 0; t < 6; t++)
#pragma unroll
            for (int i = 0; i < BNB; i++)
#pragma unroll
                for (int j = 0; j < BM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bv[i][ib[t]], av[j][ia[t]], acc[i][j], 0, 0, 0);
        if (it + 1 < nk) {
            a.store(lds0 + (buf ^ 1) * TILE3B);
            b.store(lds0 + (2 + (buf ^ 1)) * TILE3B);
        }
        __syncthreads();
    }

    // accumulator register v of lane (r, hh) of block (i, j): n = 32i + 8*(v/4) + 4*hh + v%4, m = 32j + r
    float *C = g.C + bz * g.sC;
    if (g.c_vec) {
        // A lane holds single elements of 16 columns of C: stored directly, every instruction moves 4 bytes per lane.
        // Instead each wavefront passes [32 n][64 m] blocks through a private LDS region (the operand buffers are
        // free now) and reads them back as rows of m, so that a store instruction writes four columns of 256
        // contiguous bytes, 16 bytes per lane (C is 512 MiB of the 1024 x 64 x 1024 x 128 product: 0.195 -> 0.178 ms).
        typedef __attribute__((address_space(3))) float *ldsf_t;
        typedef __attribute__((address_space(3))) const floatx4_t *ldsf4_t;
        constexpr int LDW = 64 + 4;   // floats per LDS row
        const unsigned region = lds0 + (unsigned)wave * (32 * LDW * 4);
        const int64_t mw = a.row0 + 32 * BM * wm, nw = b.row0 + 32 * BNB * wn;
#pragma unroll
        for (int i = 0; i < BNB; i++)
#pragma unroll
            for (int jp = 0; jp < BM / 2; jp++) {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int jj = 0; jj < 2; jj++)
#pragma unroll
                    for (int v = 0; v < 16; v++)
                        *(ldsf_t)(uintptr_t)(region + (unsigned)(((8 * (v / 4) + 4 * hh + (v % 4)) * LDW + 32 * jj + r) * 4)) =
                            g.alpha * acc[i][2 * jp + jj][v];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const int nl = 4 * q + (lane >> 4), ml = (lane & 15) * 4;
                    floatx4_t val = *(ldsf4_t)(uintptr_t)(region + (unsigned)((nl * LDW + ml) * 4));
                    const int64_t nj = nw + 32 * i + nl, mi = mw + 64 * jp + ml;
                    if (nj < g.n && mi < g.m) {   // m is a multiple of 4 here
                        floatx4_t *c4 = (floatx4_t *)(C + mi + nj * g.ldc);
                        if (g.beta != 0.0f) {
                            const floatx4_t old = *c4;
#pragma unroll
                            for (int e = 0; e < 4; e++) val[e] += g.beta * old[e];
                        }
                        *c4 = val;
                    }
                }
            }
        return;
    }
#pragma unroll
    for (int j = 0; j < BM; j++) {
        const int64_t mi = a.row0 + 32 * BM * wm + 32 * j + r;
        if (mi >= g.m) continue;
#pragma unroll
        for (int i = 0; i < BNB; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t nj = b.row0 + 32 * BNB * wn + 32 * i + 8 * (v / 4) + 4 * hh + (v % 4);
                if (nj < g.n) {
                    float *c = C + mi + nj * g.ldc;
                    float val = g.alpha * acc[i][j][v];
                    if (g.beta != 0.0f) val += g.beta * *c;
                    *c = val;
                }
            }
    }
}

template <bool A_RM, bool B_RM, bool LARGE>
int32_t launch_planes(const Gemm32Args &g, int64_t nb, hipStream_t st) {
    typedef ShapeS<LARGE> S;
    auto kern = gemm32s_kernel<A_RM, B_RM, LARGE>;
    constexpr size_t smem = 4 * S::TILE3B;
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

template <bool LARGE>
int32_t launch_planes_l(const Gemm32Args &g, bool a_rm, bool b_rm, int64_t nb, hipStream_t st) {
    if (a_rm) return b_rm ? launch_planes<true, true, LARGE>(g, nb, st) : launch_planes<true, false, LARGE>(g, nb, st);
    return b_rm ? launch_planes<false, true, LARGE>(g, nb, st) : launch_planes<false, false, LARGE>(g, nb, st);
}

// the Float32 matrix instruction instead of the bf16 planes (MI355ATTN_F32_MFMA=1 in the environment, read once)
bool exact_instruction_wanted() {
    static const bool wanted = [] {
        const char *e = getenv("MI355ATTN_F32_MFMA");
        return e && e[0] == '1';
    }();
    return wanted;
}

}  // namespace

// true when every 16-byte piece the kernel moves is aligned and wholly inside or outside its matrix
bool batched_gemm32_supports(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, const void *A, int64_t lda,
                             int64_t sA, const void *B, int64_t ldb, int64_t sB) {
    if (dtype != MI_F32) return false;
    if (k < 1 || m * n < 64 * 64) return false;   // tiny products: the small-tile kernel wastes less
    auto al = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if (!al(A) || !al(B) || (lda & 3) || (ldb & 3) || (sA & 3) || (sB & 3)) return false;
    if ((transA ? k : m) & 3) return false;
    if ((transB ? n : k) & 3) return false;
    return (n + TN - 1) / TN <= 65535;
}

int32_t launch_batched_gemm32(int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha, const void *A, int64_t lda,
                              int64_t sA, const void *B, int64_t ldb, int64_t sB, float beta, void *C, int64_t ldc, int64_t sC,
                              int64_t batch, hipStream_t st) {
    const bool a_rm = !transA, b_rm = transB != 0;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {   // gridDim.z is limited to 65535: issue the batch in slabs
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        Gemm32Args g = {(const float *)A + b0 * sA, (const float *)B + b0 * sB, (float *)C + b0 * sC,
                        m, n, k, lda, ldb, ldc, sA, sB, sC, alpha, beta,
                        (int32_t)((((uintptr_t)C) & 15) == 0 && (ldc & 3) == 0 && (sC & 3) == 0 && (m & 3) == 0)};
        dim3 grid((unsigned)((m + TM - 1) / TM), (unsigned)((n + TN - 1) / TN), (unsigned)nb);
        if (exact_instruction_wanted()) {
            if (a_rm && b_rm) hipLaunchKernelGGL((gemm32_kernel<true, true>), grid, dim3(256), 0, st, g);
            else if (a_rm) hipLaunchKernelGGL((gemm32_kernel<true, false>), grid, dim3(256), 0, st, g);
            else if (b_rm) hipLaunchKernelGGL((gemm32_kernel<false, true>), grid, dim3(256), 0, st, g);
            else hipLaunchKernelGGL((gemm32_kernel<false, false>), grid, dim3(256), 0, st, g);
        } else {
            // the large tile when it still gives every CU a workgroup and k is long enough to pay for its longer prologue
            const int64_t big = ((m + 255) / 256) * ((n + 255) / 256) * nb;
            const bool large = m >= 256 && n >= 256 && big >= 256 && k >= 128;
            const int32_t rc = large ? launch_planes_l<true>(g, a_rm, b_rm, nb, st) : launch_planes_l<false>(g, a_rm, b_rm, nb, st);
            if (rc != MI_OK) return rc;
        }
        MI_LAUNCH_CHECK();
    }
    return MI_OK;
}
