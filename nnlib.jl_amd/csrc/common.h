// Shared host/device helpers for the gfx950 attention library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <math.h>

#include "../../include/mi355attn.h"

#define MI_API extern "C" __attribute__((visibility("default")))

// ---- error reporting ---------------------------------------------------------------
int32_t mi_set_error(int32_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define MI_HIP_CHECK(expr)                                                                  \
    do {                                                                                    \
        hipError_t _e = (expr);                                                             \
        if (_e != hipSuccess)                                                               \
            return mi_set_error(MI_EHIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                                __FILE__, __LINE__);                                        \
    } while (0)

#define MI_LAUNCH_CHECK()                                                                   \
    do {                                                                                    \
        hipError_t _e = hipGetLastError();                                                  \
        if (_e != hipSuccess)                                                               \
            return mi_set_error(MI_EHIP, "kernel launch failed: %s (%s:%d)",                \
                                hipGetErrorString(_e), __FILE__, __LINE__);                 \
    } while (0)

static inline size_t mi_dtype_size(int32_t dt) { return dt == MI_F64 ? 8 : dt == MI_F32 ? 4 : 2; }
static inline bool mi_dtype_ok(int32_t dt) { return dt == MI_F32 || dt == MI_F16 || dt == MI_BF16; }
// entry points that also take Float64 arrays (the softmax family, the attention forward call)
static inline bool mi_dtype_ok_f64(int32_t dt) { return mi_dtype_ok(dt) || dt == MI_F64; }

// Float64 softmax family (softmax_f64.hip): op 0 softmax, 1 logsoftmax, 2 logsumexp, 3 / 4 the gradients (x = dy, x2 = y)
int32_t launch_softmax_family_f64(int op, const void *x, const void *x2, void *y, int64_t inner, int64_t len, int64_t outer, hipStream_t st);
int32_t launch_logsumexp_bwd_f64(const void *dy, const void *x, const void *lse, void *dx, int64_t inner, int64_t len, int64_t outer, hipStream_t st);

// ---- vector types ------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

// ---- element traits ----------------------------------------------------------------
struct F32 {
    typedef float type;
    typedef floatx4_t vec4;
    static constexpr int id = MI_F32;
    __device__ static inline float to_f32(float x) { return x; }
    __device__ static inline float from_f32(float x) { return x; }
};
struct F16 {
    typedef _Float16 type;
    typedef f16x8_t vec8;
    typedef f16x4_t vec4;
    static constexpr int id = MI_F16;
    __device__ static inline float to_f32(_Float16 x) { return (float)x; }
    __device__ static inline _Float16 from_f32(float x) { return (_Float16)x; }
    __device__ static inline floatx16_t mfma32(vec8 a, vec8 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    // D = A*B + C with D in other registers than C (the builtin always ties D to C, which costs a
    // 16-register copy when C stays live).  The compiler does not know this is an MFMA: the caller
    // keeps VALU reads of the result at least one later MFMA away.
    __device__ static inline floatx16_t mfma32_keep_c(vec8 a, vec8 b, const floatx16_t &c) {
        floatx16_t d;
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
        return d;
    }
};
struct BF16 {
    typedef __bf16 type;
    typedef bf16x8_t vec8;
    typedef bf16x4_t vec4;
    static constexpr int id = MI_BF16;
    __device__ static inline float to_f32(__bf16 x) { return (float)x; }
    __device__ static inline __bf16 from_f32(float x) { return (__bf16)x; }
    __device__ static inline floatx16_t mfma32(vec8 a, vec8 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    __device__ static inline floatx16_t mfma32_keep_c(vec8 a, vec8 b, const floatx16_t &c) {
        floatx16_t d;
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
        return d;
    }
};

#define MI_NEG_INF (-__builtin_huge_valf())
#define MI_POS_INF (__builtin_huge_valf())
#define MI_LOG2E 1.44269504088896340736f

// exchange a value between lane l and lane l^32 of a 64-wide wavefront
__device__ static inline float mi_swap32(float x) {
    return __shfl_xor(x, 32, 64);
}

// Lanes l < 32 and l + 32 of a wavefront hold complementary halves of two 8-byte pieces: in the MFMA
// accumulator layout lane l holds elements 0-3 of piece X and of piece Y, lane l + 32 elements 4-7 of
// both.  After the exchange lane l holds all of X and lane l + 32 all of Y, as (x, y) = (first half,
// second half), so each lane can store 16 contiguous bytes.  One v_permlane32_swap per register.
__device__ static inline void mi_pair_halves(uint32_t &x, uint32_t &y) {
    auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);   // x[32..63] <-> y[0..31]
    x = r[0];
    y = r[1];
}

__device__ static inline float mi_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- Float32 values as three bf16 planes (Float32 products on the 16-bit matrix cores) ----------------
// x = hi + mid + lo to 2^-24 of |x|, each plane the bf16 rounding of what the ones before leave.  A product of
// two bf16 values is exact in Float32 and the matrix cores accumulate in Float32, so
//   a b = a_hi b_hi + (a_hi b_mid + a_mid b_hi) + (a_hi b_lo + a_lo b_hi + a_mid b_mid) + O(2^-24 |a b|):
// six v_mfma_f32_32x32x16_bf16 give a 32x32x16 block of Float32 products at the accuracy of the Float32
// instruction in 2.7 times less matrix-pipe time than eight v_mfma_f32_32x32x2_f32.
// x -> (hi, mid, lo).  An Inf or NaN goes into the lo plane alone: lo only ever multiplies the hi plane of the
// other operand, which has that operand's sign and is zero only if the operand is (to 2^-133), so the product
// is the Inf or NaN that the Float32 instruction would give (Inf x Inf excepted, which gives NaN here).
__device__ static inline void split3(float x, __bf16 &hi, __bf16 &mid, __bf16 &lo, bool guard) {
    hi = (__bf16)x;
    float r = x - (float)hi;
    mid = (__bf16)r;
    lo = (__bf16)(r - (float)mid);
    if (guard && !(__builtin_fabsf(x) < MI_POS_INF)) {
        hi = (__bf16)0.0f;
        mid = (__bf16)0.0f;
        lo = (__bf16)x;
    }
}

// Two values at once, the way the hardware converts (one v_cvt_pk_bf16_f32 per plane and pair): each result word
// holds the plane's bf16 of x0 in its low half and of x1 in its high half.  Returns true if x0 or x1 is Inf or NaN
// (their residual x - hi is NaN then); the caller redoes such values with split3's rule.
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float mi_float2_t;
__device__ static inline uint32_t pack_bf16_pair(float a, float b) {
    const mi_float2_t f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
__device__ static inline bool split3_pair(float x0, float x1, uint32_t &hi, uint32_t &mid, uint32_t &lo) {
    hi = pack_bf16_pair(x0, x1);
    const float r0 = x0 - __builtin_bit_cast(float, hi << 16), r1 = x1 - __builtin_bit_cast(float, hi & 0xffff0000u);
    mid = pack_bf16_pair(r0, r1);
    lo = pack_bf16_pair(r0 - __builtin_bit_cast(float, mid << 16), r1 - __builtin_bit_cast(float, mid & 0xffff0000u));
    return __builtin_isunordered(r0, r1);
}
// the guarded rule of split3 for a pair
__device__ static inline void split3_pair_guarded(float x0, float x1, uint32_t &hi, uint32_t &mid, uint32_t &lo) {
    __bf16 h0, m0, l0, h1, m1, l1;
    split3(x0, h0, m0, l0, true);
    split3(x1, h1, m1, l1, true);
    const bf16x2_t h = {h0, h1}, m = {m0, m1}, l = {l0, l1};
    hi = __builtin_bit_cast(uint32_t, h);
    mid = __builtin_bit_cast(uint32_t, m);
    lo = __builtin_bit_cast(uint32_t, l);
}

// Guarded 16-byte loads without a branch: a lane whose piece of a tile does not exist reads these 16 zero bytes instead.
// (With `ok ? *p : zero` the compiler put a branch around every load and waited for each one before issuing the next:
// a tile's or a query row's loads then cost one memory round trip each instead of one in all.)
__device__ static const uint32_t mi_zero_piece[4] __attribute__((aligned(16))) = {0u, 0u, 0u, 0u};
template <typename V, typename E>
__device__ static inline V mi_load16_or_zero(const E *p, bool ok) {
    static_assert(sizeof(V) == 16, "16-byte pieces");
    // both addresses as global-memory pointers: a select of generic pointers would make this a flat load, which also
    // counts against the LDS counter
    typedef __attribute__((address_space(1))) const V *global_ptr;
    const global_ptr src = ok ? (global_ptr)(uintptr_t)p : (global_ptr)(uintptr_t)mi_zero_piece;
    return *src;
}

// Workgroup order for kernels whose neighbouring workgroups share operands.  The hardware hands workgroup `id` of a
// launch to XCD `id % 8` (eight dies, each with its own L2), so neighbours in launch order never share an L2.
// mi_xcd_order turns the launch id into the id of the work item to take such that every die works through one
// contiguous run of the natural order: die c takes items c*ceil(n/8) ... in the order its workgroups start.  A
// bijection on [0, total) for any total.
constexpr int MI_XCDS = 8;
__device__ static inline int64_t mi_xcd_order(int64_t id, int64_t total) {
    const int64_t chunk = total / MI_XCDS, rem = total % MI_XCDS;
    const int64_t xcd = id % MI_XCDS, slot = id / MI_XCDS;
    return xcd * chunk + (xcd < rem ? xcd : rem) + slot;
}

// Tile of a batched matrix product for workgroup `id` of tiles_m x tiles_n x batches: dies take contiguous runs of
// (tile, batch) items (mi_xcd_order); within a matrix the tiles run in bands of 8 tile rows, n-major inside a band, so
// that the 32 or so tiles a die has in flight form a block of about 8 x 4 tiles that share their A row tiles and B
// column tiles through that die's L2, whatever the matrix's own tile counts.
struct MiTile { int64_t m, n, batch; };
__device__ static inline MiTile mi_gemm_tile_order(int64_t id, int64_t tiles_m, int64_t tiles_n, int64_t batches) {
    constexpr int64_t GROUP_M = 8;
    const int64_t item = mi_xcd_order(id, tiles_m * tiles_n * batches);
    const int64_t pid = item % (tiles_m * tiles_n);
    const int64_t band = pid / (GROUP_M * tiles_n), in_band = pid % (GROUP_M * tiles_n);
    const int64_t band_rows = tiles_m - band * GROUP_M < GROUP_M ? tiles_m - band * GROUP_M : GROUP_M;
    return {band * GROUP_M + in_band % band_rows, in_band / band_rows, item / (tiles_m * tiles_n)};
}


// The same for callers that also keep finite values whose bf16 rounding overflows (|x| above the largest bf16,
// 3.3895e38): split3_pair makes (Inf, -Inf, NaN) of those.  mi_plane_word_special tells whether either half of a hi-plane
// word has an all-ones exponent (Inf, NaN or such an overflow); split3_pair_wide redoes a pair with the first plane
// truncated instead of rounded where the rounding overflows, and with split3's rule for Inf and NaN.
__device__ static inline bool mi_plane_word_special(uint32_t hi) {
    return (hi & 0x7f80u) == 0x7f80u || (hi & 0x7f800000u) == 0x7f800000u;
}
__device__ static inline void split3_wide(float x, __bf16 &hi, __bf16 &mid, __bf16 &lo) {
    if (!(__builtin_fabsf(x) < MI_POS_INF)) {
        hi = (__bf16)0.0f;
        mid = (__bf16)0.0f;
        lo = (__bf16)x;
        return;
    }
    hi = (__bf16)x;
    if (!(__builtin_fabsf((float)hi) < MI_POS_INF))
        hi = __builtin_bit_cast(__bf16, (unsigned short)(__builtin_bit_cast(uint32_t, x) >> 16));   // truncated: finite
    const float r = x - (float)hi;
    mid = (__bf16)r;
    lo = (__bf16)(r - (float)mid);
}
__device__ static inline void split3_pair_wide(float x0, float x1, uint32_t &hi, uint32_t &mid, uint32_t &lo) {
    __bf16 h0, m0, l0, h1, m1, l1;
    split3_wide(x0, h0, m0, l0);
    split3_wide(x1, h1, m1, l1);
    const bf16x2_t h = {h0, h1}, m = {m0, m1}, l = {l0, l1};
    hi = __builtin_bit_cast(uint32_t, h);
    mid = __builtin_bit_cast(uint32_t, m);
    lo = __builtin_bit_cast(uint32_t, l);
}

// max(a, b, c) as one instruction with no quieting of the inputs (fmaxf on MFMA results costs an extra
// v_max x, x per operand); a NaN operand is ignored like fmaxf does.
__device__ static inline float mi_max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// ---- counter-based random bits ------------------------------------------------------------------
// bits(seed, stream, i) = mix64(mix64(seed ^ stream * C) + i * G); one 64-bit word per element index.
__host__ __device__ static inline uint64_t mi_mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__host__ __device__ static inline uint64_t mi_stream_key(uint64_t seed, uint64_t stream_id) {
    return mi_mix64(seed ^ (stream_id * 0xD1342543DE82EF95ull));
}
__host__ __device__ static inline uint64_t mi_counter_bits(uint64_t key, uint64_t i) {
    return mi_mix64(key + i * 0x9E3779B97F4A7C15ull);
}
// Dropout keep decisions: one 64-bit word serves the four elements i = 4g .. 4g+3 (the word of counter g),
// 16 bits each: element i is kept when u = (bits(g) >> 16*(i & 3)) & 0xFFFF reaches thresh = ceil(p * 2^16).
// The hash (two 64-bit multiplies) is by far the dearest part of a decision, and in the MFMA accumulator
// layouts a lane, or a quad of lanes, holds four consecutive elements: one hash per four weights.
#define MI_DROPOUT_STREAM 0x64726F70ull   // stream id reserved for dropout masks
static inline uint32_t mi_dropout_threshold(float p) {
    const double t = ceil((double)p * 65536.0);
    return t <= 0.0 ? 0u : (t >= 65536.0 ? 65536u : (uint32_t)t);
}
__device__ static inline uint64_t mi_dropout_group_bits(uint64_t key, uint64_t group) { return mi_counter_bits(key, group); }
__device__ static inline bool mi_dropout_keep_in(uint64_t bits, int sub, uint32_t thresh) {
    return ((uint32_t)(bits >> (16 * sub)) & 0xFFFFu) >= thresh;
}
__device__ static inline bool mi_dropout_keep(uint64_t key, uint64_t i, uint32_t thresh) {
    return mi_dropout_keep_in(mi_dropout_group_bits(key, i >> 2), (int)(i & 3), thresh);
}

// wavefront (64 lanes) reductions
__device__ static inline float mi_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ static inline float mi_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
