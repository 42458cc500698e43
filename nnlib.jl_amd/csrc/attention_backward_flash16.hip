// MFMA attention backward for bf16/f16 inputs: eligibility, workspace size and dispatch to the
// per-(dtype, head dim) instantiations of attention_backward_flash16.inc.
#include "common.h"
#include "attention_params.h"

int32_t launch_bwd_flash16_bf16_d64(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_bf16_d128(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_f16_d64(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_f16_d128(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_bf16_d256(const AttnBwdParams &, hipStream_t);
int32_t launch_bwd_flash16_f16_d256(const AttnBwdParams &, hipStream_t);

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

bool attention_bwd_flash16_supports(const AttnBwdParams &bp) {
    const AttnParams &p = bp.p;
    if (p.dtype != MI_F16 && p.dtype != MI_BF16) return false;
    // one head dim for q, k and v: a multiple of 8 (16-byte chunks) up to the 256-wide tiles
    if (p.D != p.Dv || p.D < 8 || p.D > 256 || (p.D & 7)) return false;
    // the kernels need the forward result (for delta), take no weight cotangent and give no bias gradient
    if (!p.out || bp.dweights) return false;   // a bias gradient is summed with atomics by the dQ kernel
    if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v) || !aligned16(p.out) || !aligned16(bp.dout)) return false;
    if ((bp.dq && !aligned16(bp.dq)) || (bp.dk && !aligned16(bp.dk)) || (bp.dv && !aligned16(bp.dv))) return false;
    // tiles are fetched with 32-bit byte offsets from the (batch, head) slice
    if (p.Lq * p.E * 2 >= 2147483647LL || p.Lkv * p.E * 2 >= 2147483647LL) return false;
    const int64_t tiles = (p.Lq + 127) / 128 > (p.Lkv + 127) / 128 ? (p.Lq + 127) / 128 : (p.Lkv + 127) / 128;
    return tiles * p.H * p.B <= 2147483647LL;
}

// three float planes [B*H][Lq rounded up to 128]: row maximum (log2 units), 1 / row sum, delta
size_t attention_bwd_flash16_workspace(const AttnParams &p) { return attention_stats_bytes(p); }

int32_t launch_attention_bwd_flash16(const AttnBwdParams &bp, hipStream_t st) {
    const AttnParams &p = bp.p;
    if (p.dtype == MI_BF16)
        return p.D <= 64 ? launch_bwd_flash16_bf16_d64(bp, st) : p.D <= 128 ? launch_bwd_flash16_bf16_d128(bp, st) : launch_bwd_flash16_bf16_d256(bp, st);
    return p.D <= 64 ? launch_bwd_flash16_f16_d64(bp, st) : p.D <= 128 ? launch_bwd_flash16_f16_d128(bp, st) : launch_bwd_flash16_f16_d256(bp, st);
}
