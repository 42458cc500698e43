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
    float c;           // log2(e) * cn
    float cn;          // factor that turns an accumulator into the reference's logit: 1/sqrt(D), or 1 when q is pre-scaled
    int32_t n_qtiles;
    int32_t bias_vec;  // bias rows may be read 4 keys at a time
    int32_t mask_vec;
    int32_t w_vec;     // weight rows may be written 4 keys at a time
    int32_t nsplit;    // key range is cut into this many pieces, one workgroup each (1 = no split)
    int32_t tiles_per_split;
    int32_t bias_lds;  // 16-bit kernels: bias / mask tiles may be staged through LDS with 16-byte DMA pieces
    int32_t mask_lds;
    int32_t w_lds;     // weight rows start 16-byte aligned: tiles may be transposed through LDS and written as full lines
    // gradient kernels only: the launch covers batch elements [b0, b0 + nb), and the bias gradient may be summed
    // without atomics (no two workgroups of one launch add to the same element)
    int32_t b0, nb, dbias_plain;
    // forward kernels, key-padding masks that are context lengths: per (head, batch) pair [b * H + h] the number of
    // leading keys kept when the mask keeps exactly a prefix (the software-pipelined kernel then treats it as that
    // pair's L_kv and the general kernel leaves the pair alone), 0 otherwise (the general kernel applies the mask)
    const int32_t *kv_len = nullptr;
    // software-pipelined forward kernel with a dense mask: the packed mask (AttnMaskWords), strides in 16-byte pieces
    const u32x4_t *mask_words = nullptr;
    int64_t mw_h = 0, mw_b = 0;
    int32_t mw_lqp = 0, mw_groups = 0;
};

// Bytes of LDS per wavefront for the weight staging below: 16 query rows x 128 bytes.
constexpr int FLASH_WSTAGE_BYTES = 2048;

// Row statistics saved for the backward call: planes (maximum in log2 units, 1 / row sum, delta) of
// [B*H][Lq rounded up to 128] floats; the forward kernels fill the first two.  Rows past Lq inside the
// padding get zeros, which make their weights vanish in the backward kernels.
__device__ inline void flash_save_stats(const AttnParams &p, int64_t b, int64_t h, int64_t qi, float m2, float linv) {
    const int64_t pad = attention_stats_lq_pad(p.Lq);
    if (qi >= pad) return;
    const int64_t at = (b * p.H + h) * pad + qi;
    p.stats[at] = qi < p.Lq ? m2 : 0.0f;
    p.stats[p.B * p.H * pad + at] = qi < p.Lq ? linv : 0.0f;
}

// The zeros of the padding rows from `from` on, written by one wavefront: for kernels whose workgroups do not cover
// the padding themselves.
__device__ inline void flash_zero_stats_padding(const AttnParams &p, int64_t b, int64_t h, int64_t from) {
    const int64_t pad = attention_stats_lq_pad(p.Lq);
    for (int64_t qi = from + (threadIdx.x & 63); qi < pad; qi += 64) {
        const int64_t at = (b * p.H + h) * pad + qi;
        p.stats[at] = 0.0f;
        p.stats[p.B * p.H * pad + at] = 0.0f;
    }
}

// Split-kv bookkeeping shared by the planner (workspace size) and the launchers.
// Partials live in the caller's workspace: o as [split][B][Lq][Ev] floats, then (m, l) as
// [split][B][H][Lq][2] floats, m in log2 units.
inline int flash_pick_nsplit(const AttnParams &p, int bm) {
    if (p.weights || !p.out || p.stats) return 1;           // weights need the global maximum up front; saved statistics are per whole row
    const int64_t wgs = ((p.Lq + bm - 1) / bm) * p.H * p.B;
    if (wgs >= 512 || p.Lkv < 2048) return 1;
    // aim at one resident round: two workgroups per CU on 256 CUs (measured best on the f16 cross-attention case)
    int64_t n = (512 + wgs - 1) / wgs;
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
// how a kernel variant reads bias / mask: not at all, straight from global memory with arbitrary
// strides, or from tiles staged through LDS (FlashStaged; every array present must qualify)
// EXTRAS_KEYMASK: no bias and a mask that does not depend on the query (a key-padding mask, query stride 0):
// the scores stay raw dot products as with EXTRAS_NONE and dropped keys are set to -Inf from one mask byte per key.
// EXTRAS_MASKTILE: no bias and a dense mask whose tiles can be staged through LDS: raw dot products as with
// EXTRAS_NONE, dropped entries set to -Inf from the staged mask bytes; only the mask half of the staging is allocated,
// which keeps two workgroups per CU.
enum { EXTRAS_NONE = 0, EXTRAS_DIRECT = 1, EXTRAS_STAGED = 2, EXTRAS_KEYMASK = 3, EXTRAS_MASKTILE = 4 };
// variants that copy bias / mask tiles through LDS (FlashStaged), and the LDS bytes per wavefront they need
constexpr bool flash_uses_staging(int extras) { return extras == EXTRAS_STAGED || extras == EXTRAS_MASKTILE; }
// true when the accumulators hold the reference's logits in natural units (bias added) rather than raw dot products
constexpr bool flash_natural_units(int extras) { return extras == EXTRAS_DIRECT || extras == EXTRAS_STAGED; }
// query-independent mask without bias whose bytes can be read four keys at a time (unit key stride, Lkv a
// multiple of 4, 4-byte aligned slices): eligible for EXTRAS_KEYMASK
// any mask without bias that does not depend on the query (a key-padding mask), whatever its strides: what the
// device-side measurement of context lengths (FlashArgs::kv_len) applies to
inline bool flash_is_query_independent_mask(const AttnParams &p) {
    return p.mask && !p.bias && (p.mask_strides[1] == 0 || p.Lq == 1);
}
inline bool flash_is_key_mask(const AttnParams &p) {
    return p.mask && !p.bias && p.mask_strides[1] == 0 && p.mask_strides[0] == 1 && (p.Lkv & 3) == 0 &&
           ((p.mask_strides[2] | p.mask_strides[3]) & 3) == 0 && (((uintptr_t)p.mask) & 3) == 0;
}

inline void flash_fill_vec_flags(FlashArgs &a) {
    const AttnParams &p = a.p;
    auto mult4 = [](int64_t x) { return (x & 3) == 0; };
    const size_t es = mi_dtype_size(p.dtype);
    a.bias_vec = p.bias && p.bias_strides[0] == 1 && mult4(p.bias_strides[1]) && mult4(p.bias_strides[2]) &&
                 mult4(p.bias_strides[3]) && mult4(p.Lkv) && (((uintptr_t)p.bias) & (4 * es - 1)) == 0;
    a.mask_vec = p.mask && p.mask_strides[0] == 1 && mult4(p.mask_strides[1]) && mult4(p.mask_strides[2]) &&
                 mult4(p.mask_strides[3]) && mult4(p.Lkv) && (((uintptr_t)p.mask) & 3) == 0;
    a.w_vec = p.weights && mult4(p.Lkv) && (((uintptr_t)p.weights) & 15) == 0;
    a.w_lds = p.weights && (p.Lkv * (int64_t)mi_dtype_size(p.weights_dtype)) % 16 == 0 && (((uintptr_t)p.weights) & 15) == 0;
    // LDS staging moves 16-byte pieces addressed with 32-bit byte offsets from the (head, batch) slice:
    // rows must start 16-byte aligned and the slice (plus one query tile of slack) must stay below 2 GiB.
    auto fits = [&](const int64_t *st, size_t elem) {
        const int64_t reach = ((p.Lq + 256) * st[1] + p.Lkv + 128) * (int64_t)elem;   // tiles reach up to 127 keys past Lkv
        const int64_t per16 = 16 / (int64_t)elem;
        return st[0] == 1 && st[1] % per16 == 0 && st[2] % per16 == 0 && st[3] % per16 == 0 && reach < (int64_t)0x7fffffff;
    };
    a.bias_lds = p.bias && es == 2 && fits(p.bias_strides, es) && (((uintptr_t)p.bias) & 15) == 0;
    a.mask_lds = p.mask && es == 2 && fits(p.mask_strides, 1) && (((uintptr_t)p.mask) & 15) == 0;
}

// Encoding of s_waitcnt for "at most N vector memory operations outstanding" (vmcnt[3:0] | expcnt[6:4] |
// lgkmcnt[11:8] | vmcnt[15:14]); the other counters are left unconstrained.
#define FLASH_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 15) | (((N) >> 4) << 14) | (7 << 4) | (15 << 8))

// One 1 KiB piece global -> LDS (64 lanes x 16 bytes, lane l lands at lds_addr + 16*l; lanes whose
// offset is outside the buffer write zeros).  Issued as inline assembly so that the compiler does not
// serialise later LDS reads behind it; completion is tracked by hand with FLASH_WAIT_VMCNT (vector
// memory loads complete in order).
__device__ inline void flash_dma_1k(const i32x4_t &rsrc, unsigned lds_addr, int voffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(voffset), "s"(rsrc)
                 : "memory", "m0");
}

__device__ inline i32x4_t flash_make_rsrc(const void *base, uint32_t bytes) {
    const uint64_t addr = (uint64_t)base;
    i32x4_t rs;
    rs[0] = __builtin_amdgcn_readfirstlane((int)(addr & 0xffffffffu));
    rs[1] = __builtin_amdgcn_readfirstlane((int)((addr >> 32) & 0xffffu));  // stride 0: raw buffer
    rs[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    rs[3] = 0x00020000;
    return rs;
}

// Streams [FLASH_BN][ROWB bytes] tiles of one row-major 16-bit array global -> LDS with 1 KiB DMA pieces: no staging
// registers.  A piece (64 lanes x 16 bytes) covers 1024 / ROWB tile rows; lane l of piece i lands at chunk position
// l % (ROWB / 16) of tile row i * (1024 / ROWB) + l / (ROWB / 16) and fetches the source chunk `position ^ swz(row)`,
// which is how the consumers address the tile.  Each of the four wavefronts moves PIECES pieces per tile.
// The buffer resource is rebuilt per tile with the tile's first row as its base (64-bit scalar arithmetic), so the
// per-lane offsets are tile-local and arrays of any size work; rows past the end of the array lie outside the
// resource and arrive as zeros, and so do chunks past the head dim `dh` (their lanes carry an offset of 2 GiB,
// beyond the 2 GiB - 1 the resource size is clamped to).
template <int ROWB>
struct FlashTileDma {
    static constexpr int TILEB = FLASH_BN * ROWB, RPP = 1024 / ROWB, PIECES = TILEB / 1024 / 4;
    const char *base;          // element (row 0, first feature of the head) of this batch element
    int64_t row_bytes, end;    // end: bytes from `base` to the end of the batch element's last row
    unsigned lds;              // LDS byte address of this wavefront's first piece in buffer 0
    int voff[PIECES];
    template <typename SWZ>
    __device__ void init(const void *base_, int64_t row_elems, int64_t nrows, int64_t head_off_elems, int dh, char *tiles, SWZ swz) {
        const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        base = (const char *)base_;
        row_bytes = row_elems * 2;
        end = (nrows * row_elems - head_off_elems) * 2;
        lds = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) char *)tiles + wave * PIECES * 1024);   // wave-uniform: goes into M0
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int row = (wave * PIECES + i) * RPP + lane / (ROWB / 16);
            const int chunk = (lane % (ROWB / 16)) ^ swz(row);
            voff[i] = 8 * chunk < dh ? row * (int)row_bytes + chunk * 16 : (int)0x80000000;
        }
    }
    // start the copy of the tile whose first row is row0 into buffer `buf`
    __device__ void load(int buf, int64_t row0) const {
        const int64_t skip = row0 * row_bytes;
        int64_t left = end - skip;
        left = left < 0 ? 0 : (left > 0x7fffffffLL ? 0x7fffffffLL : left);
        const i32x4_t rs = flash_make_rsrc(base + skip, (uint32_t)left);
        const unsigned dst = __builtin_amdgcn_readfirstlane(lds + buf * TILEB);
#pragma unroll
        for (int i = 0; i < PIECES; i++) flash_dma_1k(rs, dst + i * 1024, voff[i]);
    }
};

// Bias / mask tiles of one wavefront staged through LDS (16-bit kernels).  A wavefront owns 32*QB query
// rows; per kv tile it needs, for each of them, 64 bias elements (128 bytes) and 64 mask bytes.  Reading
// those straight from global memory in the accumulator layout makes every load instruction touch 32
// different cache lines for 16 (bias) or 8 (mask) bytes each; instead the wavefront copies the
// [rows][64] tile with full-width DMA pieces into a private LDS region, one tile ahead, and reads it
// back in the accumulator layout.  16-byte chunks are XOR-swizzled per row so that those reads spread
// over all banks.  The regions are private to the wavefront: no barrier is involved, only vmcnt.
typedef __attribute__((address_space(3))) const unsigned char flash_lds_cu8;
template <int QB>
struct FlashStaged {
    static constexpr int BIAS_STAGE = 32 * QB * 128, MASK_STAGE = 32 * QB * 64;  // bytes per stage
    static constexpr int BYTES_PER_WAVE = 2 * (BIAS_STAGE + MASK_STAGE);
    static constexpr int BYTES_PER_WAVE_MASK_ONLY = 2 * MASK_STAGE;
    static constexpr int bytes_per_wave(int extras) {
        return extras == EXTRAS_STAGED ? BYTES_PER_WAVE : extras == EXTRAS_MASKTILE ? BYTES_PER_WAVE_MASK_ONLY : 0;
    }
    bool bias = false, mask = false;
    i32x4_t brs, mrs;
    unsigned blds, mlds;                 // LDS byte addresses of the two-stage regions
    int bvoff[4 * QB], mvoff[2 * QB];    // per-lane global byte offsets of the DMA pieces (tile term excluded)

    __device__ static int bias_swz(int row) { return (row >> 1) & 7; }
    __device__ static int mask_swz(int row) { return (row >> 2) & 3; }

    // mask_only: the wavefront's region holds the two mask stages only (EXTRAS_MASKTILE)
    __device__ void init(const FlashArgs &a, unsigned lds_wave_base, int lane, int64_t iw, int64_t h, int64_t b, bool mask_only = false) {
        const AttnParams &p = a.p;
        bias = a.bias_lds && !mask_only;
        mask = a.mask_lds;
        blds = __builtin_amdgcn_readfirstlane(lds_wave_base);  // wave-uniform: goes into M0
        mlds = mask_only ? blds : blds + 2 * BIAS_STAGE;
        {   // set up unconditionally so that the resource words stay in scalar registers
            const int64_t s1 = p.bias_strides[1];
            const char *base = (const char *)p.bias + 2 * (h * p.bias_strides[2] + b * p.bias_strides[3]);
            // sizes are rounded up to whole dwords: the range check is per dword, and a row end that is not a
            // multiple of 4 bytes (rows with stride 0 and any Lkv) would lose its last keys; the dword that
            // holds the last valid byte lies in the same page, and keys past Lkv are dropped by the edge code
            brs = flash_make_rsrc(base, (uint32_t)((2 * ((p.Lq - 1) * s1 + p.Lkv) + 3) & ~(int64_t)3));
#pragma unroll
            for (int i = 0; i < 4 * QB; i++) {
                const int row = 8 * i + (lane >> 3);
                bvoff[i] = (int)(2 * (iw + row) * s1) + (((lane & 7) ^ bias_swz(row)) << 4);
            }
        }
        {
            const int64_t s1 = p.mask_strides[1];
            const char *base = (const char *)p.mask + h * p.mask_strides[2] + b * p.mask_strides[3];
            mrs = flash_make_rsrc(base, (uint32_t)(((p.Lq - 1) * s1 + p.Lkv + 3) & ~(int64_t)3));
#pragma unroll
            for (int i = 0; i < 2 * QB; i++) {
                const int row = 16 * i + (lane >> 2);
                mvoff[i] = (int)((iw + row) * s1) + (((lane & 3) ^ mask_swz(row)) << 4);
            }
        }
    }
    // start the copy of the tile whose first key is j0 into `stage`
    __device__ void issue(int stage, int64_t j0) const {
        if (bias) {
#pragma unroll
            for (int i = 0; i < 4 * QB; i++) flash_dma_1k(brs, blds + stage * BIAS_STAGE + i * 1024, bvoff[i] + (int)(2 * j0));
        }
        if (mask) {
#pragma unroll
            for (int i = 0; i < 2 * QB; i++) flash_dma_1k(mrs, mlds + stage * MASK_STAGE + i * 1024, mvoff[i] + (int)j0);
        }
    }
    // all copies issued so far have landed
    __device__ void wait() const {
        if (bias || mask) {
            FLASH_WAIT_VMCNT(0);
            asm volatile("" ::: "memory");
        }
    }
    // 4 consecutive bias elements (8 bytes) / mask bytes of wavefront row `row`, keys 8*c8 + 4*hh .. +3 of the tile
    template <typename V4>
    __device__ V4 bias4(int stage, int row, int c8, int hh) const {
        const unsigned addr = blds + stage * BIAS_STAGE + row * 128 + ((c8 ^ bias_swz(row)) << 4) + 8 * hh;
        return *(__attribute__((address_space(3))) const V4 *)(uintptr_t)addr;
    }
    __device__ uint32_t mask4(int stage, int row, int c8, int hh) const {
        const unsigned addr = mlds + stage * MASK_STAGE + row * 64 + (((c8 >> 1) ^ mask_swz(row)) << 4) + 8 * (c8 & 1) + 4 * hh;
        return *(__attribute__((address_space(3))) const uint32_t *)(uintptr_t)addr;
    }
};

// On entry s[qb][kb] holds raw dot products k.q of tile rows [j0, j0+64) for the wavefront's query
// blocks; on exit it holds exp2(x - m) (ONLINE / STATS) or the final normalised weights (FINAL),
// with m, l (and, ONLINE only, the output accumulators o) updated.
//   T      element traits of the bias array
//   NDV    number of 32-row blocks of the output accumulator
// Orders a wavefront's LDS stores and loads around a cross-lane exchange: a compiler-level barrier (no instruction
// is emitted; the LDS unit completes the operations of one wavefront in issue order).
__device__ inline void flash_wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Adds a 32-key x 32-query block of Float32 values held in the MFMA accumulator layout (lane (r, hh): query row r
// of the wavefront; register 4g + e: key 8g + 4hh + e of the block) to a Float32 array whose keys are contiguous:
// dst points at (first key of the block, first query row of the wavefront), rows are qstride elements apart (0: every
// query adds to the same row).  Straight from the registers one atomic instruction would touch 64 cache lines; the
// block goes through the wavefront's FLASH_WSTAGE_BYTES LDS region 16 queries at a time and comes back with 8 lanes
// per query row, so an instruction covers 8 rows of 128 contiguous bytes.  Exact zeros are skipped.
// plain: no other workgroup running at the same time adds to these elements (the caller serialises the launches
// that would), so the sum is a load, an add and a store instead of an atomic (Float32 atomics on one array from all
// eight XCDs run at a small fraction of the store rate).
__device__ inline void flash_atomic_add_block(unsigned wlds, const floatx16_t &v, float *dst, int64_t qstride, int nq, int nk, bool plain = false) {
    typedef __attribute__((address_space(3))) u32x4_t *lds16_t;
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        if ((r >> 4) == half) {
            const unsigned rowa = wlds + (unsigned)(r & 15) * 128u;
            const int sw = (r >> 1) & 7;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                floatx4_t t4;
#pragma unroll
                for (int e = 0; e < 4; e++) t4[e] = v[4 * g + e];
                *(lds16_t)(uintptr_t)(rowa + (unsigned)(((2 * g + hh) ^ sw) << 4)) = __builtin_bit_cast(u32x4_t, t4);
            }
        }
        // lanes exchange data through LDS: to the compiler a lane's loads below never alias its own stores above, so
        // the order has to be pinned (the LDS itself completes a wavefront's operations in order)
        flash_wave_lds_fence();
        floatx4_t pieces[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rr = (lane >> 3) + 8 * i, c = lane & 7;
            pieces[i] = __builtin_bit_cast(floatx4_t, *(lds16_t)(uintptr_t)(wlds + (unsigned)rr * 128u + (unsigned)((c ^ ((rr >> 1) & 7)) << 4)));
        }
        flash_wave_lds_fence();
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rr = (lane >> 3) + 8 * i, c = lane & 7;
            const floatx4_t piece = pieces[i];
            const int q = 16 * half + rr;
            if (q < nq) {
                float *row = dst + q * qstride + 4 * c;
                if (plain) {
                    if (4 * c + 3 < nk && (((uintptr_t)row) & 15) == 0) {
                        floatx4_t old = *(const floatx4_t *)row;
#pragma unroll
                        for (int e = 0; e < 4; e++) old[e] += piece[e];
                        *(floatx4_t *)row = old;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (4 * c + e < nk) row[e] += piece[e];
                    }
                    continue;
                }
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (4 * c + e < nk && piece[e] != 0.0f) atomicAdd(row + e, piece[e]);
            }
        }
    }
}

// Key-mask bytes of a 64-key tile in the accumulator layout: word 4*kb + g holds the four bytes of keys
// j0 + 32kb + 8g + 4hh .. +3 (nonzero = keep; keys past Lkv read as kept, the edge code drops them).  All lanes
// of a half-wave read the same bytes.  Callers issue this before the QK^T MFMAs so that the loads are hidden.
__device__ inline void flash_load_key_mask(const FlashArgs &a, int64_t b, int64_t h, int64_t j0, int hh, uint32_t (&w)[8]) {
    const AttnParams &p = a.p;
    const uint8_t *mk = p.mask + h * p.mask_strides[2] + b * p.mask_strides[3] + j0 + 4 * hh;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int off = 32 * (i >> 2) + 8 * (i & 3);
        w[i] = j0 + 4 * hh + off < p.Lkv ? *(const uint32_t *)(mk + off) : 0x01010101u;   // Lkv is a multiple of 4
    }
}

// Mask bytes applied without lane masks (a compare writes a lane mask to scalar registers, which costs the compare, a
// wait state and the select: three issue slots an element).  flash_mask_bits turns the four bytes of a word into "bit 7
// of the byte is set iff the byte is non-zero" (no carry crosses a byte: 0x7f + 0x7f < 0x100); flash_mask_apply
// sign-extends that bit into a word of ones or zeros and picks the score or -Inf with a bit operation, which is not
// arithmetic: a NaN score under a dropped key is dropped like any other, as src/attention.jl:133-138 has it.
__device__ inline uint32_t flash_mask_bits(uint32_t m4) { return ((m4 & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | m4; }
// Written on the bit patterns: the compiler keeps it as a bit-field extract and one three-input bit operation (and, being
// ordinary code, gives a read of a matrix-core result the wait states it needs).
__device__ inline float flash_mask_apply(float s, uint32_t bits, int e) {
    const int keep = __builtin_amdgcn_sbfe((int)bits, 8 * e + 7, 1);   // 0 or -1
    return __builtin_bit_cast(float, (__builtin_bit_cast(int, s) & keep) | ((int)0xFF800000 & ~keep));
}
// elements 4g .. 4g+3 of a 16-element accumulator block against the four mask bytes of m4
__device__ inline void flash_mask_apply4(floatx16_t &v, int g, uint32_t m4) {
    const uint32_t bits = flash_mask_bits(m4);
#pragma unroll
    for (int e = 0; e < 4; e++) v[4 * g + e] = flash_mask_apply(v[4 * g + e], bits, e);
}

// The running maximum of the online softmax only has to bound the exponents: it is raised when a tile's maximum
// exceeds it by more than this many powers of two (and whenever either is infinite), so that the rescaling of the
// row sum and of the output accumulators is skipped for nearly every tile after the first ones.  Weights relative to
// it stay below 2^8, which Float32 sums and 16-bit operands hold without loss.
constexpr float FLASH_LAZY_MAX_LOG2 = 8.0f;

// KBLK: 32-key blocks per tile (2: the 64-key tile of the tile loops; 1: a wavefront that owns a single block)
template <typename T, int QB, int NDV, bool CAUSAL, int EXTRAS, int PHASE, typename TW, int KBLK = 2>
__device__ inline void flash_softmax_tile(const FlashArgs &a, floatx16_t (&s)[QB][KBLK], floatx16_t (&o)[QB][NDV],
                                          float (&fm)[QB], float (&fl)[QB], int64_t b, int64_t h, int64_t iw,
                                          int64_t j0, const FlashStaged<QB> &sg = FlashStaged<QB>(), int stage = 0,
                                          unsigned wlds = 0, const uint32_t *key_mask = nullptr, int64_t kv_len = -1) {
    const AttnParams &p = a.p;
    typedef typename T::type elem_t;
    constexpr int BN = 32 * KBLK;
    static_assert(KBLK == 2 || ((EXTRAS == EXTRAS_NONE || EXTRAS == EXTRAS_DIRECT) && sizeof(TW) == 4), "single blocks: Float32 kernels without staged tiles");
    const int lane = threadIdx.x & 63, r = lane & 31, hh = lane >> 5;
    // kv_len >= 0: keys from kv_len on do not exist for this (head, batch) pair (a context length shorter than L_kv);
    // the weights of such keys come out as exact zeros
    const int64_t lkv = kv_len >= 0 ? kv_len : p.Lkv;
    const bool edge = (j0 + BN > lkv) || (CAUSAL && j0 + BN - 1 > iw);
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
        const int64_t qi = iw + 32 * qb + r;
        const bool qok = qi < p.Lq;
        // ---- scale, bias, mask.  With bias / mask the accumulators end up holding the reference's
        // logits (natural units); without, they keep the raw dot products and the positive factor c
        // is folded into the exponent below (max commutes with a positive scale).
        if (EXTRAS == EXTRAS_STAGED) {
            const int row = 32 * qb + r;
            if (sg.bias) {
#pragma unroll
                for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const typename T::vec4 t4 = sg.template bias4<typename T::vec4>(stage, row, 4 * kb + g, hh);
#pragma unroll
                        for (int e = 0; e < 4; e++) s[qb][kb][4 * g + e] = fmaf(s[qb][kb][4 * g + e], a.cn, T::to_f32(t4[e]));
                    }
            } else {
#pragma unroll
                for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                    for (int v = 0; v < 16; v++) s[qb][kb][v] *= a.cn;
            }
            if (sg.mask) {
#pragma unroll
                for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        flash_mask_apply4(s[qb][kb], g, sg.mask4(stage, row, 4 * kb + g, hh));
                    }
            }
        } else if (EXTRAS == EXTRAS_DIRECT) {
            const elem_t *bias = (const elem_t *)p.bias;
            const int64_t boff = qi * p.bias_strides[1] + h * p.bias_strides[2] + b * p.bias_strides[3];
            const int64_t moff = qi * p.mask_strides[1] + h * p.mask_strides[2] + b * p.mask_strides[3];
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++)
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
                        float x = fmaf(s[qb][kb][4 * g + e], a.cn, bv[e]);
                        s[qb][kb][4 * g + e] = keep[e] ? x : MI_NEG_INF;
                    }
                }
        }
        if (EXTRAS == EXTRAS_MASKTILE) {
            const int row = 32 * qb + r;
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++) {
#pragma unroll
                for (int g = 0; g < 4; g++) flash_mask_apply4(s[qb][kb], g, sg.mask4(stage, row, 4 * kb + g, hh));
            }
        }
        if (EXTRAS == EXTRAS_KEYMASK) {
            // one mask byte per key, shared by every query
            uint32_t own[8];
            if (!key_mask) flash_load_key_mask(a, b, h, j0, hh, own);
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++) {
#pragma unroll
                for (int g = 0; g < 4; g++) flash_mask_apply4(s[qb][kb], g, key_mask ? key_mask[4 * kb + g] : own[4 * kb + g]);
            }
        }
        if (EXTRAS != EXTRAS_DIRECT && edge) {
            // keys past the end of the sequence or, causal, after the query: tile-local limit per lane
            int64_t lim64 = lkv - j0;
            if (CAUSAL && qi - j0 + 1 < lim64) lim64 = qi - j0 + 1;
            const int lim = lim64 > BN ? BN : (lim64 < 0 ? 0 : (int)lim64);
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int kvl = 32 * kb + 8 * (v / 4) + 4 * hh + (v % 4);
                    s[qb][kb][v] = kvl < lim ? s[qb][kb][v] : MI_NEG_INF;
                }
        }
        constexpr bool NAT = flash_natural_units(EXTRAS);
        const float cs = NAT ? MI_LOG2E : a.c;

        float pmul = 1.0f, msafe;
        bool pinf;  // the running maximum is +Inf: weights become the normalised indicator of the +Inf entries
        if (PHASE != PHASE_FINAL) {
            float mx = MI_NEG_INF;
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                for (int v = 0; v < 16; v++) mx = fmaxf(mx, s[qb][kb][v]);
            mx = fmaxf(mx, mi_swap32(mx));
            const float mold = fm[qb];
            // raise the running maximum only when some row of the wavefront outgrows it (see FLASH_LAZY_MAX_LOG2):
            // -Inf before the first kept key and +Inf logits give an infinite difference; a NaN compares false and
            // poisons the row through its own exponential
            if (__builtin_amdgcn_ballot_w64((mx - mold) * cs > FLASH_LAZY_MAX_LOG2) != 0) {
                const float mnew = fmaxf(mold, mx);
                const float ms = mnew == MI_NEG_INF ? 0.0f : mnew;
                float resc = mi_exp2((mold - ms) * cs);
                if (mold == mnew) resc = 1.0f;  // also covers +Inf == +Inf
                fm[qb] = mnew;
                fl[qb] *= resc;
                if (PHASE == PHASE_ONLINE) {
#pragma unroll
                    for (int dvb = 0; dvb < NDV; dvb++)
#pragma unroll
                        for (int v = 0; v < 16; v++) o[qb][dvb][v] *= resc;
                }
            }
            msafe = fm[qb] == MI_NEG_INF ? 0.0f : fm[qb];
            pinf = fm[qb] == MI_POS_INF;
        } else {
            msafe = fm[qb] == MI_NEG_INF ? 0.0f : fm[qb];
            pinf = fm[qb] == MI_POS_INF;
            pmul = fl[qb];  // holds 1 / (row sum) in the final phase
        }
        // src/softmax.jl:74-75.  Only bias or an upstream overflow can produce +Inf logits, so the
        // per-element work sits behind a wavefront-uniform test.
        if (NAT && __builtin_expect(__builtin_amdgcn_ballot_w64(pinf) != 0, 0)) {
            if (pinf) {
#pragma unroll
                for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                    for (int v = 0; v < 16; v++) s[qb][kb][v] = s[qb][kb][v] == MI_POS_INF ? 0.0f : MI_NEG_INF;
                msafe = 0.0f;
            }
        }
        const float moff2 = -msafe * cs;
        float lsum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float x = s[qb][kb][v];
                float e = mi_exp2(fmaf(x, cs, moff2));
                if (PHASE == PHASE_FINAL) e *= pmul;
                lsum += e;
                s[qb][kb][v] = e;
            }
        if (PHASE != PHASE_FINAL) fl[qb] += lsum;

        // fdrop = dropout (src/attention.jl:126): after the softmax, so the row sum above is untouched;
        // before the value product and before the weights are written, which are post-dropout.
        if (PHASE != PHASE_STATS && p.drop_thresh != 0) {
            const uint64_t row0 = (uint64_t)(p.Lkv * (qi + p.Lq * (h + p.H * b)) + j0 + 4 * hh);
            const bool aligned = (p.Lkv & 3) == 0;   // every run of four keys of a lane is one hash group
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float f[4];
                    if (aligned) attention_drop_factors_run4<true>(p, row0 + 32 * kb, g, f);
                    else attention_drop_factors_run4<false>(p, row0 + 32 * kb, g, f);
#pragma unroll
                    for (int e = 0; e < 4; e++) s[qb][kb][4 * g + e] *= f[e];
                }
        }

        if (PHASE == PHASE_FINAL && p.weights && wlds != 0 && a.w_lds) {
            // In the accumulator layout a lane holds runs of 4 keys of ONE query, so a direct store touches 32
            // weight rows with 8 or 16 bytes each.  Instead the tile goes through a wavefront-private LDS region,
            // 16 queries x 128 bytes at a time (64 keys of a 16-bit weight type, 32 keys of Float32), and comes
            // back with 8 lanes per query row: every store instruction writes 8 full 128-byte lines.  Chunks are
            // XOR-swizzled with the row pair (two rows share a bank span).  LDS operations of one wavefront
            // complete in order, so no barrier is needed.
            typedef __attribute__((address_space(3))) u32x4_t *lds16_t;
            typedef __attribute__((address_space(3))) u32x2_t *lds8_t;
            constexpr int EPC = 16 / (int)sizeof(TW);             // weights per 16-byte chunk
            constexpr int NKB = sizeof(TW) == 4 ? KBLK : 1;       // staging rounds per tile along the keys
            TW *wbase = (TW *)p.weights + p.Lkv * (p.Lq * (h + p.H * b));
#pragma unroll
            for (int rk = 0; rk < NKB; rk++)
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    if ((r >> 4) == half) {
                        const unsigned rowa = wlds + (unsigned)(r & 15) * 128u;
                        const int sw = (r >> 1) & 7;
                        if constexpr (sizeof(TW) == 2) {
#pragma unroll
                            for (int kb = 0; kb < KBLK; kb++)
#pragma unroll
                                for (int g = 0; g < 4; g++) {
                                    typedef TW tw4 __attribute__((ext_vector_type(4)));
                                    tw4 t4;
#pragma unroll
                                    for (int e = 0; e < 4; e++) t4[e] = (TW)s[qb][kb][4 * g + e];
                                    *(lds8_t)(uintptr_t)(rowa + (unsigned)(((4 * kb + g) ^ sw) << 4) + 8u * hh) = __builtin_bit_cast(u32x2_t, t4);
                                }
                        } else {
#pragma unroll
                            for (int g = 0; g < 4; g++) {
                                floatx4_t t4;
#pragma unroll
                                for (int e = 0; e < 4; e++) t4[e] = s[qb][rk][4 * g + e];
                                *(lds16_t)(uintptr_t)(rowa + (unsigned)(((2 * g + hh) ^ sw) << 4)) = __builtin_bit_cast(u32x4_t, t4);
                            }
                        }
                    }
                    flash_wave_lds_fence();   // a lane's loads never alias its own stores: the exchange has to be pinned
                    u32x4_t pieces[2];
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const int rr = (lane >> 3) + 8 * i, c = lane & 7;
                        pieces[i] = *(lds16_t)(uintptr_t)(wlds + (unsigned)rr * 128u + (unsigned)((c ^ ((rr >> 1) & 7)) << 4));
                    }
                    flash_wave_lds_fence();
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const int rr = (lane >> 3) + 8 * i, c = lane & 7;
                        const u32x4_t piece = pieces[i];
                        const int64_t qrow = iw + 32 * qb + 16 * half + rr, kv0 = j0 + 32 * rk + (int64_t)c * EPC;
                        if (qrow < p.Lq && kv0 < p.Lkv) *(u32x4_t *)(wbase + p.Lkv * qrow + kv0) = piece;   // Lkv is a multiple of EPC here
                    }
                }
        } else if (PHASE == PHASE_FINAL && p.weights && qok) {
            TW *w = (TW *)p.weights + p.Lkv * (qi + p.Lq * (h + p.H * b));
#pragma unroll
            for (int kb = 0; kb < KBLK; kb++)
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
// from_diag: the wavefront stopped at the tile that holds its last query's diagonal (causal); otherwise it visited
// all n_tiles tiles
__device__ inline void flash_zero_skipped_weights(const FlashArgs &a, int64_t b, int64_t h, int64_t iw, int n_tiles, bool from_diag = true) {
    const AttnParams &p = a.p;
    constexpr int BN = FLASH_BN;
    const int lane = threadIdx.x & 63;
    int64_t kcov = from_diag ? ((iw + 32 * QB - 1) / BN + 1) * BN : (int64_t)n_tiles * BN;
    if (kcov > (int64_t)n_tiles * BN) kcov = (int64_t)n_tiles * BN;
    if (kcov >= p.Lkv) return;
    constexpr int EPC = 16 / (int)sizeof(TW);   // weights per 16-byte store
    if (a.w_lds) {
        // rows start 16-byte aligned and hold a whole number of 16-byte pieces (kcov is a multiple of 64 keys): a
        // store instruction clears 1 KiB of a row
        const u32x4_t z = {0, 0, 0, 0};
        for (int row = 0; row < 32 * QB; row++) {
            const int64_t qi = iw + row;
            if (qi >= p.Lq) break;
            TW *w = (TW *)p.weights + p.Lkv * (qi + p.Lq * (h + p.H * b));
            for (int64_t kv = kcov + (int64_t)lane * EPC; kv < p.Lkv; kv += 64 * EPC) *(u32x4_t *)(w + kv) = z;
        }
        return;
    }
    for (int row = 0; row < 32 * QB; row++) {
        const int64_t qi = iw + row;
        if (qi >= p.Lq) break;
        TW *w = (TW *)p.weights + p.Lkv * (qi + p.Lq * (h + p.H * b));
        for (int64_t kv = kcov + lane; kv < p.Lkv; kv += 64) w[kv] = (TW)0.0f;
    }
}
