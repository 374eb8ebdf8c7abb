// Decoders of the reference's 32-lane layouts, shared by the GEMV / dequant kernels and the batched MoE kernel.
#pragma once

#include "bf16n_c.h"
#include "dev_common.h"

namespace bf16n {
namespace dev {

struct hp_ptrs { const uint8_t * plane; const uint32_t * lut; const uint32_t * ubase; const uint16_t * lrel; const uint32_t * stream; };
struct huf_ptrs { const uint8_t * plane; const uint32_t * lut; const uint32_t * lane_off; const uint32_t * stream; };
struct nib_ptrs { const uint8_t * plane; const uint8_t * codes; const uint8_t * table; const uint32_t * esc_off; const uint32_t * esc; };

__device__ __forceinline__ hp_ptrs hpp(const bf16n_weight & w) {
    return {w.plane, (const uint32_t *) (w.aux + w.off_a), (const uint32_t *) (w.aux + w.off_b),
            (const uint16_t *) (w.aux + w.off_c), (const uint32_t *) (w.aux + w.off_d)};
}
__device__ __forceinline__ huf_ptrs hufp(const bf16n_weight & w) {
    return {w.plane, (const uint32_t *) (w.aux + w.off_a), (const uint32_t *) (w.aux + w.off_b),
            (const uint32_t *) (w.aux + w.off_c)};
}
__device__ __forceinline__ nib_ptrs nibp(const bf16n_weight & w, int64_t shift_rows) {
    // the up half of a merged [gate; up] matrix: every per-row array shifted by shift_rows (escape offsets are absolute)
    return {w.plane + shift_rows * w.K, w.aux + w.off_a + shift_rows * (w.K / 2), w.aux + w.off_b + shift_rows * 16,
            (const uint32_t *) (w.aux + w.off_c) + shift_rows, (const uint32_t *) (w.aux + w.off_d)};
}

// MSB-first bit buffer over one lane stream: `v` valid bits at the top of `buf`, one word of lookahead in `nxt`.
// Two table lookups (<= 24 bits) are always covered because v > 32 after every refill.  The stream buffers end with
// padding words, so the lookahead never leaves the allocation.
struct lane_bits {
    const uint32_t * sp;
    uint64_t buf;
    uint32_t nxt;
    int v;
    __device__ __forceinline__ void begin(const uint32_t * p) {
        sp = p;
        buf = ((uint64_t) sp[0] << 32) | sp[1];
        nxt = sp[2];
        sp += 3;
        v = 64;
    }
    template <int BITS>
    __device__ __forceinline__ uint32_t take(const uint32_t * lut) {
        const uint32_t ent = lut[(uint32_t) (buf >> (64 - BITS))];
        const int len = (int) (ent & 31u);
        buf <<= len;
        v -= len;
        return ent;
    }
    __device__ __forceinline__ void refill() {
        if (v <= 32) {
            buf |= (uint64_t) nxt << (32 - v);
            v += 32;
            nxt = *sp++;
        }
    }
};

// the 16 weights of one lane in one chunk as 8 BF16 pairs: wp[2j], wp[2j+1] = columns 128j + 4l + {0,1}, {2,3}
template <int FORMAT>
__device__ __forceinline__ void decode_chunk(lane_bits & bits, const uint32_t * lut, const uint4 sm, uint32_t (&wp)[8]) {
    const uint32_t smw[4] = {sm.x, sm.y, sm.z, sm.w};
    if (FORMAT == FMT_HUFPAIR) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t e0 = bits.take<HP_LP>(lut);
            const uint32_t e1 = bits.take<HP_LP>(lut);
            bits.refill();
            wp[2 * j] = merge(spread_lo(smw[j]), e0);
            wp[2 * j + 1] = merge(spread_hi(smw[j]), e1);
        }
    } else { // single exponents, entry = len | exponent << 7
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t a = bits.take<HUF_LMAX>(lut), b = bits.take<HUF_LMAX>(lut);
            bits.refill();
            const uint32_t c = bits.take<HUF_LMAX>(lut), d = bits.take<HUF_LMAX>(lut);
            bits.refill();
            wp[2 * j] = merge(spread_lo(smw[j]), (a & 0x7F80u) | ((b & 0x7F80u) << 16));
            wp[2 * j + 1] = merge(spread_hi(smw[j]), (c & 0x7F80u) | ((d & 0x7F80u) << 16));
        }
    }
}

// ---------------------------------------------------------------- NIBBLE (shared by the GEMV / dequant kernels and the batched kernels)

// 4 exponents of 4 adjacent columns from 4 nibble codes (16 bits) and the row's 16-byte table, as bytes e0..e3
__device__ __forceinline__ uint32_t nib_lookup4(const uint4 T, uint32_t codes16) {
    uint32_t s = (codes16 | (codes16 << 8)) & 0x00FF00FFu;
    s = (s | (s << 4)) & 0x0F0F0F0Fu; // one code per byte
    const uint32_t lo = __builtin_amdgcn_perm(T.y, T.x, s & 0x07070707u);
    const uint32_t hi = __builtin_amdgcn_perm(T.w, T.z, s & 0x07070707u);
    const uint32_t pick_hi = ((s >> 3) & 0x01010101u) * 0xFFu;
    return (hi & pick_hi) | (lo & ~pick_hi);
}

// the 16 weights of one lane in one NIBBLE chunk
__device__ __forceinline__ void nib_chunk(const uint4 sm, const uint2 cd, const uint4 T, uint32_t (&wp)[8]) {
    const uint32_t smw[4] = {sm.x, sm.y, sm.z, sm.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t c16 = ((j & 2) ? cd.y : cd.x) >> ((j & 1) * 16) & 0xFFFFu;
        const uint32_t e4 = nib_lookup4(T, c16);
        wp[2 * j] = merge(spread_lo(smw[j]), __builtin_amdgcn_perm(0, e4, 0x0c010c00u) << 7);
        wp[2 * j + 1] = merge(spread_hi(smw[j]), __builtin_amdgcn_perm(0, e4, 0x0c030c02u) << 7);
    }
}

__device__ __forceinline__ uint32_t esc_bits(uint32_t rec) { // BF16 bits of an escape record col | sm << 12 | exponent << 20
    const uint32_t smb = (rec >> 12) & 0xFFu, ex = rec >> 20;
    return ((smb & 0x80u) << 8) | (ex << 7) | (smb & 0x7Fu);
}

} // namespace dev
} // namespace bf16n
