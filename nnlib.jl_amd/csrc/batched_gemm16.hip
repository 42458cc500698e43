// Tiled strided batched GEMM for bf16 / f16 on MFMA: the fast path of mi_batched_gemm for operands
// whose rows can be moved in 16-byte pieces (aligned bases, leading dimensions and contiguous extents
// that are multiples of 8).  Stands where the reference calls BLAS gemm per slice
// (src/gemm.jl:141-149, reached through _batched_gemm!, src/batched/batchedmul.jl:298).
//
// Workgroup = 4 wavefronts (2 x 2), output tile 128 (m) x 128 (n), 64 x 64 per wavefront as 2 x 2
// MFMA blocks of 32 x 32; k advances 64 per stage through double-buffered LDS tiles.
// As in batched_gemm.hip the MFMA runs on the transposed problem (accumulator rows = n, columns = m),
// so that the 32 lanes of a half-wave store 32 consecutive elements of a C column.
//
// An operand tile is kept in the orientation its memory has:
//   RMAJ  contiguous along its row index (A with 'N', B with 'T'): tile [64 k][128 rows], chunks
//         XOR-swizzled, MFMA operand through the transposing LDS read (the value tile of the
//         attention kernels has exactly this geometry);
//   KMAJ  contiguous along k (A with 'T', B with 'N'): tile [128 rows][64 k], rows padded to 136
//         bytes, MFMA operand as two 8-byte reads.
// Both deliver the 16 k of a step in the order {0-3, 8-11 | 4-7, 12-15} per half-wave, which is what
// the transposing read produces; A and B only have to agree.
#include "common.h"

namespace {

constexpr int TM = 128, TN = 128, KC = 64;
constexpr int RMAJ_ROWB = 256;                 // bytes per k-row of an RMAJ tile (128 rows x 2 bytes)
constexpr int KMAJ_ROWB = 136;                 // bytes per row of a KMAJ tile (64 k x 2 bytes + 8 pad: conflict-free 8-byte reads)
constexpr int TILEB = 128 * KMAJ_ROWB;         // bytes reserved per tile and buffer (RMAJ needs 64*256 = 16384 <= 17408)

struct Gemm16Args {
    const void *A, *B;
    void *C;
    int64_t m, n, k, lda, ldb, ldc, sA, sB, sC;
    float alpha, beta;
};

__device__ inline int rmaj_swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

template <typename T>
__device__ inline typename T::vec4 lds_tr4(const char *p) {
    s16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t *)p);
    return __builtin_bit_cast(typename T::vec4, r);
}

// One operand tile.  X points at the slice; `rows` = extent along the operand's row index (m or n),
// `ld` = leading dimension.  RM: element (row, kk) at X[row + kk*ld]; else at X[kk + row*ld].
template <typename T, bool RM>
struct Operand {
    typedef typename T::type t;
    const t *X;
    int64_t ld, rows, k, row0;
    u32x4_t reg[4];

    // 1024 chunks of 16 bytes per tile, 4 per thread
    __device__ void load(int64_t k0) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int c = tid + 256 * u;
            u32x4_t z = {0, 0, 0, 0};
            if (RM) {
                const int kk = c >> 4, r8 = (c & 15) * 8;       // 16 chunks per k-row
                const bool ok = k0 + kk < k && row0 + r8 < rows;
                reg[u] = ok ? *(const u32x4_t *)(X + (row0 + r8) + (k0 + kk) * ld) : z;
            } else {
                const int r = c >> 3, k8 = (c & 7) * 8;         // 8 chunks per row
                const bool ok = row0 + r < rows && k0 + k8 < k;
                reg[u] = ok ? *(const u32x4_t *)(X + (k0 + k8) + (row0 + r) * ld) : z;
            }
        }
    }
    __device__ void store(char *tile) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int c = tid + 256 * u;
            if (RM) {
                const int kk = c >> 4, chunk = c & 15;
                *(u32x4_t *)(tile + kk * RMAJ_ROWB + ((chunk ^ rmaj_swz(kk)) << 4)) = reg[u];
            } else {
                const int r = c >> 3, chunk = c & 7;
                u32x2_t lo = {reg[u][0], reg[u][1]}, hi = {reg[u][2], reg[u][3]};   // rows are 8-byte aligned only
                *(u32x2_t *)(tile + r * KMAJ_ROWB + chunk * 16) = lo;
                *(u32x2_t *)(tile + r * KMAJ_ROWB + chunk * 16 + 8) = hi;
            }
        }
    }
    // MFMA operand of the 32-row block `blk` (0..3 within the tile) for k-step `ks` (0..3)
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
            const char *src = tile + (32 * blk + (lane & 31)) * KMAJ_ROWB + 32 * ks + 8 * hh;
            const typename T::vec4 lo = *(const typename T::vec4 *)src;          // k 4hh .. 4hh+3
            const typename T::vec4 hi = *(const typename T::vec4 *)(src + 16);   // k 8+4hh .. 8+4hh+3
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    }
};

template <typename T, bool A_RM, bool B_RM>
__global__ __launch_bounds__(256, 2) void gemm16_kernel(Gemm16Args g) {
    typedef typename T::type t;
    extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];
    char *As = (char *)gemm_smem, *Bs = As + 2 * TILEB;
    const int64_t bz = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
    const int r = lane & 31, hh = lane >> 5;

    Operand<T, A_RM> a;
    Operand<T, B_RM> b;
    a.X = (const t *)g.A + bz * g.sA;
    a.ld = g.lda;
    a.rows = g.m;
    a.k = g.k;
    a.row0 = (int64_t)blockIdx.x * TM;
    b.X = (const t *)g.B + bz * g.sB;
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
    a.store(As);
    b.store(Bs);
    __syncthreads();
    for (int it = 0; it < nk; it++) {
        const int buf = it & 1;
        if (it + 1 < nk) {
            a.load((int64_t)(it + 1) * KC);
            b.load((int64_t)(it + 1) * KC);
        }
        const char *at = As + buf * TILEB, *bt = Bs + buf * TILEB;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            typename T::vec8 av[2], bv[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                av[j] = Operand<T, A_RM>::fetch(at, 2 * wm + j, ks, lane);
                bv[j] = Operand<T, B_RM>::fetch(bt, 2 * wn + j, ks, lane);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = T::mfma32(bv[i], av[j], acc[i][j]);
        }
        if (it + 1 < nk) {
            a.store(As + (buf ^ 1) * TILEB);
            b.store(Bs + (buf ^ 1) * TILEB);
        }
        __syncthreads();
    }

    // accumulator register v of lane (r, hh) of block (i, j): n = 32i + 8*(v/4) + 4*hh + v%4, m = 32j + r
    t *C = (t *)g.C + bz * g.sC;
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
                    t *c = C + mi + nj * g.ldc;
                    float val = g.alpha * acc[i][j][v];
                    if (g.beta != 0.0f) val += g.beta * T::to_f32(*c);
                    *c = T::from_f32(val);
                }
            }
    }
}

template <typename T, bool A_RM, bool B_RM>
int32_t launch_one(const Gemm16Args &g, int64_t nb, hipStream_t st) {
    auto kern = gemm16_kernel<T, A_RM, B_RM>;
    constexpr size_t smem = 4 * TILEB;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, so a race is harmless
    if (!attr_set) {
        MI_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    dim3 grid((unsigned)((g.m + TM - 1) / TM), (unsigned)((g.n + TN - 1) / TN), (unsigned)nb);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, g);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

template <typename T>
int32_t launch_t(const Gemm16Args &g, int transA, int transB, int64_t nb, hipStream_t st) {
    const bool a_rm = !transA, b_rm = transB != 0;
    if (a_rm) return b_rm ? launch_one<T, true, true>(g, nb, st) : launch_one<T, true, false>(g, nb, st);
    return b_rm ? launch_one<T, false, true>(g, nb, st) : launch_one<T, false, false>(g, nb, st);
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
    return (n + TN - 1) / TN <= 65535;
}

int32_t launch_batched_gemm16(int32_t dtype, int transA, int transB, int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                              int64_t lda, int64_t sA, const void *B, int64_t ldb, int64_t sB, float beta, void *C, int64_t ldc,
                              int64_t sC, int64_t batch, hipStream_t st) {
    const size_t es = 2;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {   // gridDim.z is limited to 65535: issue the batch in slabs
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        Gemm16Args g = {(const char *)A + es * b0 * sA, (const char *)B + es * b0 * sB, (char *)C + es * b0 * sC,
                        m, n, k, lda, ldb, ldc, sA, sB, sC, alpha, beta};
        const int32_t rc = dtype == MI_F16 ? launch_t<F16>(g, transA, transB, nb, st) : launch_t<BF16>(g, transA, transB, nb, st);
        if (rc != MI_OK) return rc;
    }
    return MI_OK;
}
