// softmax / logsoftmax / logsumexp and the softmax gradients over any run of adjacent dimensions.
// The array is viewed as (inner, len, outer), element (i, j, o) at i + inner*(j + len*o), and the
// reduction runs over j.  Replaces, for device arrays, NNlib's
//   _softmax!      src/softmax.jl:69-79        (dims other than 1; dims = 1 keeps its own kernels in softmax.hip)
//   _logsoftmax!   src/softmax.jl:137-147
//   logsumexp      src/softmax.jl:200-203
//   _∇softmax!     src/softmax.jl:107-110      dx = dy*y - y*sum(dy*y)
//   _∇logsoftmax!  src/softmax.jl:175-177      dx = dy - sum(dy)*exp(y)
// Arithmetic in fp32.
//
// A workgroup of 256 threads owns TI consecutive `inner` positions of one `outer` slice (TI = a power
// of two <= 64, chosen by the host from `inner`) and splits j over TJ = 256/TI slices; consecutive
// lanes touch consecutive addresses whenever inner >= TI or inner == 1.  Columns of up to CACHE*TJ
// elements stay in registers between the passes (one HBM read, one write); longer ones are re-read.
#include "common.h"

namespace {

enum { OP_SOFTMAX = 0, OP_LOGSOFTMAX = 1, OP_LOGSUMEXP = 2, OP_GRAD_SOFTMAX = 3, OP_GRAD_LOGSOFTMAX = 4 };
constexpr int CACHE = 16;

struct Geometry {
    int64_t inner, len, outer, n_itiles;
    int ti_log2;
};

// reduce over the j-slices of a workgroup: lanes with equal (lane & (TI-1)) within a wavefront by
// butterfly, then the four wavefronts through LDS
template <bool IS_MAX>
__device__ inline float reduce_slices(float v, int ti_log2, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, ti = 1 << ti_log2;
    for (int o = 32; o >= ti; o >>= 1) {
        const float u = __shfl_xor(v, o, 64);
        v = IS_MAX ? fmaxf(v, u) : v + u;
    }
    __syncthreads();  // previous use of `red`
    if (lane < ti) red[wave * 64 + lane] = v;
    __syncthreads();
    const int il = lane & (ti - 1);
    float r = red[il];
#pragma unroll
    for (int w = 1; w < 4; w++) r = IS_MAX ? fmaxf(r, red[w * 64 + il]) : r + red[w * 64 + il];
    return r;
}

// e^x through the hardware 2^x (the reference's own exp is @fastmath, src/softmax.jl:72)
__device__ inline float fast_exp(float x) { return mi_exp2(x * MI_LOG2E); }

// the reference's elementwise rules given the column maximum m
__device__ inline float softmax_term(float x, float m) {   // src/softmax.jl:72-75
    if (m == MI_POS_INF) return x == MI_POS_INF ? 1.0f : 0.0f;
    return fast_exp(x - m);
}
__device__ inline float logsoftmax_shift(float x, float m) {   // src/softmax.jl:140-144
    if (m == MI_POS_INF) return x == MI_POS_INF ? 0.0f : MI_NEG_INF;
    return x - m;
}

template <typename T, int OP>
__global__ __launch_bounds__(256) void softmax_nd_kernel(const typename T::type *x, const typename T::type *x2,
                                                          typename T::type *y, Geometry g) {
    typedef typename T::type t;
    __shared__ float red[256];
    const int ti = 1 << g.ti_log2, tj = 256 >> g.ti_log2;
    const int il = threadIdx.x & (ti - 1), js = threadIdx.x >> g.ti_log2;
    const int64_t n_tiles = g.n_itiles * g.outer;
    const bool cached = g.len <= (int64_t)CACHE * tj;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t o = tile / g.n_itiles, i = (tile % g.n_itiles) * ti + il;
        const bool ok = i < g.inner;
        const int64_t base = i + g.inner * g.len * o;
        const t *xc = x + base;
        const t *x2c = x2 ? x2 + base : nullptr;
        t *yc = y + base;
        float v[CACHE], v2[(OP >= OP_GRAD_SOFTMAX) ? CACHE : 1];

        if constexpr (OP == OP_GRAD_SOFTMAX || OP == OP_GRAD_LOGSOFTMAX) {
            // x = dy, x2 = y (the forward result)
            float s = 0.0f;
            if (cached) {
#pragma unroll
                for (int c = 0; c < CACHE; c++) {
                    const int64_t j = js + (int64_t)tj * c;
                    const bool in = ok && j < g.len;
                    v[c] = in ? T::to_f32(xc[g.inner * j]) : 0.0f;
                    v2[c] = in ? T::to_f32(x2c[g.inner * j]) : 0.0f;
                    s += OP == OP_GRAD_SOFTMAX ? v[c] * v2[c] : v[c];
                }
            } else if (ok) {
                for (int64_t j = js; j < g.len; j += tj) {
                    const float dy = T::to_f32(xc[g.inner * j]);
                    s += OP == OP_GRAD_SOFTMAX ? dy * T::to_f32(x2c[g.inner * j]) : dy;
                }
            }
            s = reduce_slices<false>(s, g.ti_log2, red);
            if (cached) {
#pragma unroll
                for (int c = 0; c < CACHE; c++) {
                    const int64_t j = js + (int64_t)tj * c;
                    if (ok && j < g.len)
                        yc[g.inner * j] = T::from_f32(OP == OP_GRAD_SOFTMAX ? v2[c] * (v[c] - s) : v[c] - s * fast_exp(v2[c]));
                }
            } else if (ok) {
                for (int64_t j = js; j < g.len; j += tj) {
                    const float dy = T::to_f32(xc[g.inner * j]), yy = T::to_f32(x2c[g.inner * j]);
                    yc[g.inner * j] = T::from_f32(OP == OP_GRAD_SOFTMAX ? yy * (dy - s) : dy - s * fast_exp(yy));
                }
            }
            continue;
        }

        // forward ops: maximum, then sum of exponentials, then the result.  fmaxf skips a NaN, but the
        // NaN still reaches every element of its column through the sum, as in the reference.
        float m = MI_NEG_INF;
        if (cached) {
#pragma unroll
            for (int c = 0; c < CACHE; c++) {
                const int64_t j = js + (int64_t)tj * c;
                v[c] = (ok && j < g.len) ? T::to_f32(xc[g.inner * j]) : MI_NEG_INF;
                m = fmaxf(m, v[c]);
            }
        } else if (ok) {
            for (int64_t j = js; j < g.len; j += tj) {
                m = fmaxf(m, T::to_f32(xc[g.inner * j]));
            }
        }
        m = reduce_slices<true>(m, g.ti_log2, red);
        float s = 0.0f;
        auto term = [&](float xv) {
            if (OP == OP_SOFTMAX) return softmax_term(xv, m);
            if (OP == OP_LOGSOFTMAX) return fast_exp(logsoftmax_shift(xv, m));
            return fast_exp(xv - m);   // logsumexp: no special cases (src/softmax.jl:202)
        };
        if (cached) {
#pragma unroll
            for (int c = 0; c < CACHE; c++) {
                const int64_t j = js + (int64_t)tj * c;
                if (ok && j < g.len) s += term(v[c]);
            }
        } else if (ok) {
            for (int64_t j = js; j < g.len; j += tj) s += term(T::to_f32(xc[g.inner * j]));
        }
        s = reduce_slices<false>(s, g.ti_log2, red);
        if (OP == OP_LOGSUMEXP) {
            if (ok && js == 0) y[i + g.inner * o] = T::from_f32(m + logf(s));
            continue;
        }
        const float logs = logf(s);
        auto result = [&](float xv) {
            if (OP == OP_SOFTMAX) return softmax_term(xv, m) / s;
            return logsoftmax_shift(xv, m) - logs;
        };
        if (cached) {
#pragma unroll
            for (int c = 0; c < CACHE; c++) {
                const int64_t j = js + (int64_t)tj * c;
                if (ok && j < g.len) yc[g.inner * j] = T::from_f32(result(v[c]));
            }
        } else if (ok) {
            for (int64_t j = js; j < g.len; j += tj) yc[g.inner * j] = T::from_f32(result(T::to_f32(xc[g.inner * j])));
        }
    }
}

// ---- reductions over a strided dimension with wide rows ----------------------------------------------
// inner is a multiple of VEC (16 bytes of elements) and every row starts 16-byte aligned: a thread owns
// VEC consecutive `inner` positions and walks j in steps of TJ; TI threads side by side cover TI*VEC
// positions, so a wavefront reads 64/TI rows of TI*16 contiguous bytes per load.  Columns of up to 8192
// elements (4096 for the gradients) are held in registers by a 512-thread workgroup: one read, one
// write.  Longer ones are streamed: one pass finds the maximum and the sum together (running maximum,
// sum rescaled when it grows), a second pass writes: two reads and one write per element.
template <typename T, int VEC>
struct VecIO {
    typedef typename T::type t;
    __device__ static void unpack(const u32x4_t &raw, float (&v)[VEC]) {
        if constexpr (VEC == 4) {
            const floatx4_t f = __builtin_bit_cast(floatx4_t, raw);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = f[e];
        } else {
            const typename T::vec8 h = __builtin_bit_cast(typename T::vec8, raw);
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = T::to_f32(h[e]);
        }
    }
    __device__ static u32x4_t pack(const float (&v)[VEC]) {
        if constexpr (VEC == 4) {
            floatx4_t f;
#pragma unroll
            for (int e = 0; e < 4; e++) f[e] = v[e];
            return __builtin_bit_cast(u32x4_t, f);
        } else {
            typename T::vec8 h;
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = T::from_f32(v[e]);
            return __builtin_bit_cast(u32x4_t, h);
        }
    }
    __device__ static void store(t *p, const float (&v)[VEC]) {
        if constexpr (VEC == 4) {
            floatx4_t f;
#pragma unroll
            for (int e = 0; e < 4; e++) f[e] = v[e];
            *(floatx4_t *)p = f;
        } else {
            typename T::vec8 h;
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = T::from_f32(v[e]);
            *(u32x4_t *)p = __builtin_bit_cast(u32x4_t, h);
        }
    }
};

// running (maximum, sum of exponentials against it); the special cases keep the reference's results:
// nothing but -Inf so far contributes no terms, a +Inf maximum counts the +Inf entries (src/softmax.jl:72-75)
// A NaN entry becomes the maximum and stays it (no comparison replaces it), which turns every later term and
// the results of the whole column into NaN, as the reference's maximum does (src/softmax.jl:69-70).
__device__ inline void online_add(float x, float &m, float &s) {
    if (x != x) m = x;
    if (x > m) {
        s = (m == MI_NEG_INF) ? 0.0f : s * fast_exp(m - x);
        m = x;
    }
    if (m != MI_NEG_INF) s += softmax_term(x, m);
}
__device__ inline void online_merge(float m2, float s2, float &m, float &s) {
    if (m2 != m2) m = m2;
    if (m2 > m) {
        s = (m == MI_NEG_INF) ? s2 : s2 + s * fast_exp(m - m2);
        m = m2;
    } else if (m2 != MI_NEG_INF) {
        s += (m2 == m) ? s2 : s2 * fast_exp(m2 - m);
    }
}

// Workgroups go to the 8 XCDs round-robin.  Tiles that are neighbours along `inner` share cache lines
// of every row, so each XCD gets a contiguous range of tiles: a permutation of [0, 8*floor(n/8)), the
// identity on the rest (2.05 -> 2.31 TB/s on a 256 x 4096 x 128 bf16 array reduced over dim 2).
__device__ inline int64_t xcd_order(int64_t tile, int64_t n_tiles) {
    const int64_t n8 = n_tiles >> 3;
    return tile < 8 * n8 ? (tile & 7) * n8 + (tile >> 3) : tile;
}

// lanes with equal (lane & (TI-1)) hold slices of the same positions: butterfly within the wavefront,
// then the NW wavefronts of the workgroup through LDS (red: NW * 64 * VEC floats)
template <bool IS_MAX, int VEC, int NW>
__device__ inline void reduce_slices_vec(float (&v)[VEC], int ti_log2, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, ti = 1 << ti_log2;
    for (int o = 32; o >= ti; o >>= 1) {
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float u = __shfl_xor(v[e], o, 64);
            v[e] = IS_MAX ? fmaxf(v[e], u) : v[e] + u;
        }
    }
    __syncthreads();  // previous use of `red`
    if (lane < ti) {
#pragma unroll
        for (int e = 0; e < VEC; e++) red[(wave * 64 + lane) * VEC + e] = v[e];
    }
    __syncthreads();
    const int il = lane & (ti - 1);
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        float r = red[il * VEC + e];
#pragma unroll
        for (int w = 1; w < NW; w++) {
            const float u = red[(w * 64 + il) * VEC + e];
            r = IS_MAX ? fmaxf(r, u) : r + u;
        }
        v[e] = r;
    }
}

// Keeps a thread's cached pieces in their packed form between the passes: without it the compiler unpacks
// 16-bit pieces once and carries the Float32 values (twice the registers) from pass to pass, which spills.
template <int NP>
__device__ inline void keep_packed(u32x4_t (&raw)[NP]) {
#pragma unroll
    for (int u = 0; u < NP; u++) asm volatile("" : "+v"(raw[u]));
}

// Columns of up to NP * TJ elements (TJ = NT / TI): the NP 16-byte pieces of a thread stay in registers
// between the reduction and the result, so every element is read once and written once.  All loads are
// issued before any arithmetic.  One slab (the inner x len elements of one outer index, below 2 GiB) is
// addressed through a buffer resource: a thread keeps one 32-bit offset, the row of each piece comes from
// a scalar offset, and pieces past the column's end (or columns past `inner`) get an offset outside the
// resource, which reads as zeros.  That leaves the registers to the cached pieces.
template <typename T>
struct CachedTile {
    __amdgpu_buffer_rsrc_t rx, rx2, ry;   // the slab of the tile's outer index in x, x2 (gradients) and y
    int64_t o;                            // outer index
    int col;                              // first column of the tile
    int voff, nrows;                      // this thread's byte offset in the slab; pieces it holds
    bool ok;                              // the thread's columns exist
};

// FULL: every thread holds NP pieces of a valid column (len = NP * TJ, inner a multiple of TI * VEC), so
// the passes are straight-line code.  Columns with infinities take the reference's special cases through
// a branch that is uniform over the wavefront.
template <typename T, int OP, int VEC, int NP, int NT, bool FULL>
__global__ __launch_bounds__(NT, (NP * (OP >= OP_GRAD_SOFTMAX ? 2 : 1) <= 16 && OP != OP_LOGSUMEXP ? 2 : 1) * NT / 256) void softmax_nd_cached_kernel(
        const typename T::type *x, const typename T::type *x2, typename T::type *y, Geometry g) {
    typedef typename T::type t;
    typedef VecIO<T, VEC> IO;
    constexpr bool GRAD = OP >= OP_GRAD_SOFTMAX;
    constexpr int NW = NT / 64, OOB = 0x7fffffff, SZ = (int)sizeof(t);
    __shared__ float red[NW * 64 * VEC];
    const int ti = 1 << g.ti_log2, tj = NT >> g.ti_log2;
    const int il = threadIdx.x & (ti - 1), js = threadIdx.x >> g.ti_log2;
    const int64_t n_tiles = g.n_itiles * g.outer;
    const int inner = (int)g.inner, len = (int)g.len;   // a slab is below 2 GiB (host)
    const int slab_bytes = inner * len * SZ;
    const int step_bytes = inner * tj * SZ;   // between consecutive rows of one thread
    // the thread's offset within a tile whose first column is 0 (threads past the column's end never use it)
    const int thread_off = js < len ? (il * VEC + inner * js) * SZ : 0;
    // scalar offset of a thread's u-th piece; 0 for pieces that lie past the column's end for every thread
    const auto row_off = [&](int u) { return FULL || u * tj < len ? step_bytes * u : 0; };
    const auto locate = [&](int64_t tile0) {
        CachedTile<T> c;
        const int64_t tile = xcd_order(tile0, n_tiles);
        c.o = tile / g.n_itiles;
        c.col = (int)(tile % g.n_itiles) * ti * VEC;
        c.ok = FULL || c.col + il * VEC < inner;
        c.nrows = FULL ? NP : (c.ok && js < len ? (len - js + tj - 1) / tj : 0);   // <= NP (host)
        c.voff = thread_off + c.col * SZ;
        const int64_t slab = g.inner * g.len * c.o;
        c.rx = __builtin_amdgcn_make_buffer_rsrc((void *)(x + slab), 0, slab_bytes, 0x00020000);
        c.rx2 = __builtin_amdgcn_make_buffer_rsrc((void *)((GRAD ? x2 : x) + slab), 0, slab_bytes, 0x00020000);
        c.ry = __builtin_amdgcn_make_buffer_rsrc((void *)(y + (OP == OP_LOGSUMEXP ? 0 : slab)), 0, slab_bytes, 0x00020000);
        return c;
    };
    u32x4_t raw[NP], raw2[GRAD ? NP : 1];
    const auto request = [&](const CachedTile<T> &c, int u) {
        const int vo = FULL || u < c.nrows ? c.voff : OOB;
        raw[u] = __builtin_amdgcn_raw_buffer_load_b128(c.rx, vo, row_off(u), 0);
        if constexpr (GRAD) raw2[u] = __builtin_amdgcn_raw_buffer_load_b128(c.rx2, vo, row_off(u), 0);
    };
    // Stores carry the row in the vector offset, not in the scalar one: the compiler keeps writes to the
    // data registers of a 16-byte buffer store away from the store only when its scalar offset is not a
    // register, and with one the next piece's arithmetic, which reuses those registers at once, now and
    // then overwrote the first of them before the store had read it (a few elements in ten thousand).
    const auto put = [&](const CachedTile<T> &c, int u, const u32x4_t &piece) {
        __builtin_amdgcn_raw_buffer_store_b128(piece, c.ry, c.voff + row_off(u), 0, 0);
    };
    for (int64_t tile0 = blockIdx.x; tile0 < n_tiles; tile0 += gridDim.x) {
        const CachedTile<T> cur = locate(tile0);
#pragma unroll
        for (int u = 0; u < NP; u++) request(cur, u);
        const int nrows = cur.nrows;
        float m[VEC], sum[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            m[e] = MI_NEG_INF;
            sum[e] = 0.0f;
        }
        if constexpr (GRAD) {
#pragma unroll
            for (int u = 0; u < NP; u++) {
                if (FULL || u < nrows) {
                    float v[VEC], v2[VEC];
                    IO::unpack(raw[u], v);
                    if (OP == OP_GRAD_SOFTMAX) IO::unpack(raw2[u], v2);
#pragma unroll
                    for (int e = 0; e < VEC; e++) sum[e] += OP == OP_GRAD_SOFTMAX ? v[e] * v2[e] : v[e];
                }
            }
            reduce_slices_vec<false, VEC, NW>(sum, g.ti_log2, red);
            keep_packed(raw);
            keep_packed(raw2);
#pragma unroll
            for (int u = 0; u < NP; u++) {
                if (FULL || u < nrows) {
                    float v[VEC], v2[VEC], r[VEC];
                    IO::unpack(raw[u], v);
                    IO::unpack(raw2[u], v2);
#pragma unroll
                    for (int e = 0; e < VEC; e++)
                        r[e] = OP == OP_GRAD_SOFTMAX ? v2[e] * (v[e] - sum[e]) : v[e] - sum[e] * fast_exp(v2[e]);
                    put(cur, u, IO::pack(r));
                }
            }
        } else {
            // forward ops: maximum, sum of exponentials, result, all from the registers
#pragma unroll
            for (int u = 0; u < NP; u++) {
                if (FULL || u < nrows) {
                    float v[VEC];
                    IO::unpack(raw[u], v);
#pragma unroll
                    for (int e = 0; e < VEC; e++) m[e] = fmaxf(m[e], v[e]);
                }
            }
            reduce_slices_vec<true, VEC, NW>(m, g.ti_log2, red);
            bool finite = true;   // finite maxima: no special cases
#pragma unroll
            for (int e = 0; e < VEC; e++) finite = finite && m[e] > MI_NEG_INF && m[e] < MI_POS_INF;
            // the same for the whole wavefront; logsumexp has no special cases (src/softmax.jl:202)
            const bool plain = OP == OP_LOGSUMEXP || __builtin_amdgcn_ballot_w64(!finite) == 0;
            keep_packed(raw);
            if (plain) {
                float cm[VEC];
#pragma unroll
                for (int e = 0; e < VEC; e++) cm[e] = -m[e] * MI_LOG2E;
#pragma unroll
                for (int u = 0; u < NP; u++) {
                    if (FULL || u < nrows) {
                        float v[VEC];
                        IO::unpack(raw[u], v);
#pragma unroll
                        for (int e = 0; e < VEC; e++) sum[e] += mi_exp2(fmaf(v[e], MI_LOG2E, cm[e]));
                    }
                }
            } else {
                // an infinite maximum somewhere in the wavefront (rare): the reference's special cases, one
                // piece at a time from memory in a rolled loop, so that this path costs the other no registers
#pragma unroll 1
                for (int u = 0; u < nrows; u++) {
                    float v[VEC];
                    IO::unpack(__builtin_amdgcn_raw_buffer_load_b128(cur.rx, cur.voff + step_bytes * u, 0, 0), v);
#pragma unroll
                    for (int e = 0; e < VEC; e++)
                        sum[e] += OP == OP_SOFTMAX ? softmax_term(v[e], m[e]) : fast_exp(logsoftmax_shift(v[e], m[e]));
                }
            }
            reduce_slices_vec<false, VEC, NW>(sum, g.ti_log2, red);
            keep_packed(raw);
            if constexpr (OP == OP_LOGSUMEXP) {
                if (cur.ok && js == 0) {
                    float r[VEC];
#pragma unroll
                    for (int e = 0; e < VEC; e++) r[e] = m[e] + logf(sum[e]);
                    IO::store(y + cur.col + il * VEC + g.inner * cur.o, r);
                }
            } else if (plain) {
                // m and sum fold into two constants per position
                float c0[VEC], c1[VEC];
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    if (OP == OP_SOFTMAX) {
                        c0[e] = -m[e] * MI_LOG2E;
                        c1[e] = 1.0f / sum[e];
                    } else {
                        c1[e] = -m[e] - logf(sum[e]);
                    }
                }
#pragma unroll
                for (int u = 0; u < NP; u++) {
                    if (FULL || u < nrows) {
                        float v[VEC], r[VEC];
                        IO::unpack(raw[u], v);
#pragma unroll
                        for (int e = 0; e < VEC; e++)
                            r[e] = OP == OP_SOFTMAX ? mi_exp2(fmaf(v[e], MI_LOG2E, c0[e])) * c1[e] : v[e] + c1[e];
                        put(cur, u, IO::pack(r));
                    }
                    }
            } else {
#pragma unroll 1
                for (int u = 0; u < nrows; u++) {
                    float v[VEC], r[VEC];
                    IO::unpack(__builtin_amdgcn_raw_buffer_load_b128(cur.rx, cur.voff + step_bytes * u, 0, 0), v);
#pragma unroll
                    for (int e = 0; e < VEC; e++)
                        r[e] = OP == OP_SOFTMAX ? softmax_term(v[e], m[e]) / sum[e] : logsoftmax_shift(v[e], m[e]) - logf(sum[e]);
                    __builtin_amdgcn_raw_buffer_store_b128(IO::pack(r), cur.ry, cur.voff + step_bytes * u, 0, 0);
                }
            }
        }
    }
}

template <typename T, int OP, int VEC>
__global__ __launch_bounds__(256) void softmax_nd_vec_kernel(const typename T::type *x, const typename T::type *x2,
                                                              typename T::type *y, Geometry g) {
    typedef typename T::type t;
    typedef VecIO<T, VEC> IO;
    constexpr int U = 4;   // rows in flight per thread: all loads of a group are issued before any arithmetic
    constexpr bool GRAD = OP >= OP_GRAD_SOFTMAX;
    __shared__ float red_m[256 * VEC], red_s[256 * VEC];
    const int ti = 1 << g.ti_log2, tj = 256 >> g.ti_log2;
    const int il = threadIdx.x & (ti - 1), js = threadIdx.x >> g.ti_log2;
    const int64_t n_tiles = g.n_itiles * g.outer;
    const int64_t step = g.inner * tj;   // elements between consecutive rows of one thread
    for (int64_t tile0 = blockIdx.x; tile0 < n_tiles; tile0 += gridDim.x) {
        const int64_t tile = xcd_order(tile0, n_tiles);
        const int64_t o = tile / g.n_itiles, i = ((tile % g.n_itiles) * ti + il) * VEC;
        const bool ok = i < g.inner;
        const int64_t base = i + g.inner * g.len * o + g.inner * js;
        const int64_t nrows = ok && js < g.len ? (g.len - js + tj - 1) / tj : 0;   // rows js, js+tj, ... of this thread
        float m[VEC], s[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            m[e] = MI_NEG_INF;
            s[e] = 0.0f;
        }
        for (int64_t r0 = 0; r0 < nrows; r0 += U) {
            u32x4_t raw[U], raw2[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int64_t at = base + step * (r0 + u < nrows ? r0 + u : nrows - 1);   // the tail repeats the last row (ignored below)
                raw[u] = *(const u32x4_t *)(x + at);
                if (OP == OP_GRAD_SOFTMAX) raw2[u] = *(const u32x4_t *)(x2 + at);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (r0 + u >= nrows) break;
                float v[VEC], v2[VEC];
                IO::unpack(raw[u], v);
                if constexpr (GRAD) {
                    if (OP == OP_GRAD_SOFTMAX) IO::unpack(raw2[u], v2);
#pragma unroll
                    for (int e = 0; e < VEC; e++) s[e] += OP == OP_GRAD_SOFTMAX ? v[e] * v2[e] : v[e];
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; e++) online_add(v[e], m[e], s[e]);
                }
            }
        }
        // combine the TJ slices of each position through LDS
        __syncthreads();
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            red_m[(js * ti + il) * VEC + e] = m[e];
            red_s[(js * ti + il) * VEC + e] = s[e];
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            float mm = MI_NEG_INF, ss = 0.0f;
            for (int q = 0; q < tj; q++) {
                const float m2 = red_m[(q * ti + il) * VEC + e], s2 = red_s[(q * ti + il) * VEC + e];
                if constexpr (GRAD) ss += s2;
                else online_merge(m2, s2, mm, ss);
            }
            m[e] = mm;
            s[e] = ss;
        }
        if (!ok) continue;
        if constexpr (OP == OP_LOGSUMEXP) {
            if (js == 0) {
                float r[VEC];
#pragma unroll
                for (int e = 0; e < VEC; e++)   // the reference's x - max is Inf - Inf for an infinite maximum
                    r[e] = (m[e] == MI_POS_INF || m[e] == MI_NEG_INF) ? __builtin_nanf("") : m[e] + logf(s[e]);
                IO::store(y + i + g.inner * o, r);
            }
            continue;
        }
        // per-position constants of the second pass; `plain`: finite maxima, so no special cases
        float c0[VEC], c1[VEC];
        bool plain = true;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            plain = plain && m[e] > MI_NEG_INF && m[e] < MI_POS_INF;
            if (OP == OP_SOFTMAX) {
                c0[e] = -m[e] * MI_LOG2E;
                c1[e] = 1.0f / s[e];
            } else if (OP == OP_LOGSOFTMAX) {
                c0[e] = logf(s[e]);
                c1[e] = -m[e] - c0[e];
            }
        }
        for (int64_t r0 = 0; r0 < nrows; r0 += U) {
            u32x4_t raw[U], raw2[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int64_t at = base + step * (r0 + u < nrows ? r0 + u : nrows - 1);
                raw[u] = *(const u32x4_t *)(x + at);
                if (GRAD) raw2[u] = *(const u32x4_t *)(x2 + at);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (r0 + u >= nrows) break;
                float v[VEC], v2[VEC], r[VEC];
                IO::unpack(raw[u], v);
                if (GRAD) IO::unpack(raw2[u], v2);
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    if (OP == OP_SOFTMAX) r[e] = plain ? mi_exp2(fmaf(v[e], MI_LOG2E, c0[e])) * c1[e] : softmax_term(v[e], m[e]) / s[e];
                    else if (OP == OP_LOGSOFTMAX) r[e] = plain ? v[e] + c1[e] : logsoftmax_shift(v[e], m[e]) - c0[e];
                    else if (OP == OP_GRAD_SOFTMAX) r[e] = v2[e] * (v[e] - s[e]);
                    else r[e] = v[e] - s[e] * fast_exp(v2[e]);
                }
                IO::store(y + base + step * (r0 + u), r);
            }
        }
    }
}

template <typename T, int OP>
void launch_nd(const void *x, const void *x2, void *y, int64_t inner, int64_t len, int64_t outer, hipStream_t st) {
    typedef typename T::type t;
    Geometry g;
    g.inner = inner;
    g.len = len;
    g.outer = outer;
    constexpr int VEC = 16 / (int)sizeof(t);
    const auto al = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if (inner % VEC == 0 && inner >= 4 * VEC && len > 64 && al(x) && al(y) && (!x2 || al(x2))) {
        // wide rows and columns too long for the register cache of the scalar kernel
        const int64_t chunks = inner / VEC;
        // register-cached kernel: a thread holds NP pieces (two workgroups per compute unit) or 2 NP (one);
        // the second is taken when it makes the contiguous pieces of a row wider, which is what the memory
        // system rewards (256 x 4096 x 128 bf16 over dim 2: 0.185 ms with 32-byte pieces, 0.131 with 64)
        constexpr int NP = OP >= OP_GRAD_SOFTMAX ? 8 : 16;   // the gradients hold two arrays
        if (len <= 512 * 2 * NP && inner * len * (int64_t)sizeof(t) < ((int64_t)1 << 31)) {
            // TI as wide as the column length allows (TJ * pieces >= len), but at least 1024 tiles
            const auto widest = [&](int np) {
                int tl = 0;
                while ((1 << tl) < 64 && ((int64_t)1 << tl) < chunks && (int64_t)(512 >> (tl + 1)) * np >= len) tl++;
                while (tl > 0 && ((chunks + (1 << tl) - 1) >> tl) * outer < 1024) tl--;
                return tl;
            };
            const int t1 = len <= 512 * NP ? widest(NP) : -1, t2 = widest(2 * NP);
            const bool wide = t2 > t1;
            g.ti_log2 = wide ? t2 : t1;
            g.n_itiles = (chunks + (1 << g.ti_log2) - 1) >> g.ti_log2;
            int64_t blocks = g.n_itiles * outer;
            if (blocks > 262144) blocks = 262144;
            const bool full = len == (int64_t)(512 >> g.ti_log2) * (wide ? 2 * NP : NP) && chunks % (1 << g.ti_log2) == 0;
#define MI_CACHED_LAUNCH(NP_, FULL_)                                                                                 \
    hipLaunchKernelGGL((softmax_nd_cached_kernel<T, OP, VEC, NP_, 512, FULL_>), dim3((unsigned)blocks), dim3(512), 0, \
                       st, (const t *)x, (const t *)x2, (t *)y, g)
            if (wide) {
                if (full) MI_CACHED_LAUNCH(2 * NP, true);
                else MI_CACHED_LAUNCH(2 * NP, false);
            } else {
                if (full) MI_CACHED_LAUNCH(NP, true);
                else MI_CACHED_LAUNCH(NP, false);
            }
#undef MI_CACHED_LAUNCH
            return;
        }
        g.ti_log2 = 0;
        while ((1 << g.ti_log2) < 64 && ((int64_t)1 << g.ti_log2) < chunks) g.ti_log2++;
        // enough workgroups to fill the chip, but rows of at least 64 contiguous bytes per wavefront load
        while (g.ti_log2 > 2 && ((chunks + (1 << g.ti_log2) - 1) >> g.ti_log2) * outer < 2048) g.ti_log2--;
        g.n_itiles = (chunks + (1 << g.ti_log2) - 1) >> g.ti_log2;
        int64_t blocks = g.n_itiles * outer;
        if (blocks > 262144) blocks = 262144;
        hipLaunchKernelGGL((softmax_nd_vec_kernel<T, OP, VEC>), dim3((unsigned)blocks), dim3(256), 0, st, (const t *)x,
                           (const t *)x2, (t *)y, g);
        return;
    }
    g.ti_log2 = 0;
    while ((1 << g.ti_log2) < 64 && ((int64_t)1 << g.ti_log2) < inner) g.ti_log2++;
    g.n_itiles = (inner + (1 << g.ti_log2) - 1) >> g.ti_log2;
    int64_t blocks = g.n_itiles * outer;
    if (blocks > 262144) blocks = 262144;
    hipLaunchKernelGGL((softmax_nd_kernel<T, OP>), dim3((unsigned)blocks), dim3(256), 0, st, (const t *)x, (const t *)x2,
                       (t *)y, g);
}

template <int OP>
int32_t dispatch(const char *name, int32_t dtype, const void *x, const void *x2, void *y, int64_t inner, int64_t len,
                 int64_t outer, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "%s: unknown dtype %d", name, dtype);
    if (inner < 0 || len < 0 || outer < 0) return mi_set_error(MI_EINVAL, "%s: negative size", name);
    if (inner == 0 || outer == 0 || (len == 0 && OP != OP_LOGSUMEXP)) return MI_OK;
    if (!x || !y || (OP >= OP_GRAD_SOFTMAX && !x2)) return mi_set_error(MI_EINVAL, "%s: null pointer", name);
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F64) return launch_softmax_family_f64(OP, x, x2, y, inner, len, outer, st);
    if (dtype == MI_F32) launch_nd<F32, OP>(x, x2, y, inner, len, outer, st);
    else if (dtype == MI_F16) launch_nd<F16, OP>(x, x2, y, inner, len, outer, st);
    else launch_nd<BF16, OP>(x, x2, y, inner, len, outer, st);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

// pullback of logsumexp given its result: dx[i,j,o] = dy[i,o] * exp(x[i,j,o] - lse[i,o]), which is the
// reference's dy .* tmp ./ sum(tmp) (src/softmax.jl:205-212) with tmp/sum(tmp) = exp(x - logsumexp).  A
// column whose result is not finite gives NaN, as the reference's exp(x - max) does there.
template <typename T>
__global__ __launch_bounds__(256) void logsumexp_bwd_kernel(const typename T::type *dy, const typename T::type *x,
                                                             const typename T::type *lse, typename T::type *dx,
                                                             int64_t inner, int64_t len, int64_t outer) {
    const int64_t n = inner * len * outer;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) {
        const int64_t i = idx % inner, o = idx / (inner * len);
        const float z = T::to_f32(lse[i + inner * o]), g = T::to_f32(dy[i + inner * o]);
        const bool finite = z > MI_NEG_INF && z < MI_POS_INF;   // false for NaN too
        dx[idx] = T::from_f32(finite ? g * fast_exp(T::to_f32(x[idx]) - z) : __builtin_nanf(""));
    }
}

template <typename T>
void launch_logsumexp_bwd(const void *dy, const void *x, const void *lse, void *dx, int64_t inner, int64_t len, int64_t outer,
                          hipStream_t st) {
    typedef typename T::type t;
    int64_t blocks = (inner * len * outer + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(logsumexp_bwd_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, st, (const t *)dy, (const t *)x,
                       (const t *)lse, (t *)dx, inner, len, outer);
}

}  // namespace

MI_API int32_t mi_logsumexp_bwd(int32_t dtype, const void *dy, const void *x, const void *lse, void *dx, int64_t inner,
                                int64_t len, int64_t outer, mi_stream s) {
    if (!mi_dtype_ok_f64(dtype)) return mi_set_error(MI_EDTYPE, "mi_logsumexp_bwd: unknown dtype %d", dtype);
    if (inner < 0 || len < 0 || outer < 0) return mi_set_error(MI_EINVAL, "mi_logsumexp_bwd: negative size");
    if (inner == 0 || len == 0 || outer == 0) return MI_OK;
    if (!dy || !x || !lse || !dx) return mi_set_error(MI_EINVAL, "mi_logsumexp_bwd: null pointer");
    hipStream_t st = (hipStream_t)s;
    if (dtype == MI_F64) return launch_logsumexp_bwd_f64(dy, x, lse, dx, inner, len, outer, st);
    if (dtype == MI_F32) launch_logsumexp_bwd<F32>(dy, x, lse, dx, inner, len, outer, st);
    else if (dtype == MI_F16) launch_logsumexp_bwd<F16>(dy, x, lse, dx, inner, len, outer, st);
    else launch_logsumexp_bwd<BF16>(dy, x, lse, dx, inner, len, outer, st);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_softmax(int32_t op, int32_t dtype, const void *x, void *y, int64_t inner, int64_t len, int64_t outer,
                          mi_stream s) {
    if (op == MI_SOFTMAX) {
        if (inner == 1) return mi_softmax_dim1(dtype, x, y, len, outer, s);
        return dispatch<OP_SOFTMAX>("mi_softmax", dtype, x, nullptr, y, inner, len, outer, s);
    }
    if (op == MI_LOGSOFTMAX) return dispatch<OP_LOGSOFTMAX>("mi_softmax", dtype, x, nullptr, y, inner, len, outer, s);
    return mi_set_error(MI_EINVAL, "mi_softmax: op must be MI_SOFTMAX or MI_LOGSOFTMAX, got %d", op);
}

MI_API int32_t mi_logsumexp(int32_t dtype, const void *x, void *y, int64_t inner, int64_t len, int64_t outer, mi_stream s) {
    return dispatch<OP_LOGSUMEXP>("mi_logsumexp", dtype, x, nullptr, y, inner, len, outer, s);
}

MI_API int32_t mi_softmax_bwd(int32_t op, int32_t dtype, const void *dy, const void *y, void *dx, int64_t inner, int64_t len,
                              int64_t outer, mi_stream s) {
    if (op == MI_SOFTMAX) return dispatch<OP_GRAD_SOFTMAX>("mi_softmax_bwd", dtype, dy, y, dx, inner, len, outer, s);
    if (op == MI_LOGSOFTMAX) return dispatch<OP_GRAD_LOGSOFTMAX>("mi_softmax_bwd", dtype, dy, y, dx, inner, len, outer, s);
    return mi_set_error(MI_EINVAL, "mi_softmax_bwd: op must be MI_SOFTMAX or MI_LOGSOFTMAX, got %d", op);
}
