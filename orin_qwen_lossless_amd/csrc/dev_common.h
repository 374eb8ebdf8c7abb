// Device-side helpers shared by the BF16N kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "bf16n/format.h"

namespace bf16n {
namespace dev {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

struct bf16_t { uint16_t bits; }; // activation / output element type tag for BF16

// ---------------------------------------------------------------- column description (reference cols_t, kernels.cuh:93-117)
// One output vector: (token) for a dense product, (token, expert slot) with expert ids.  Strides in bytes.
struct cols {
    const char * x; char * y;
    int64_t x_tok, x_slot, y_tok, y_slot;
    const char * ids; int64_t ids_s0, ids_s1;
    int n_used, x_per_slot;
    int64_t rows_per_matrix, row0, nrows;
    bool y_bf16;
    bool stream_once; // stream blocks with the same hint (small matrices only)
    bool plane_once; // the launch reads every plane byte once: load them with the non-temporal hint
};

struct col_view { const char * x; char * y; int64_t rbase; };

__device__ __forceinline__ col_view col_setup(const cols & p, int col) {
    col_view v;
    if (p.ids) {
        const int t = col / p.n_used, i = col % p.n_used;
        const int e = *(const int32_t *) (p.ids + t * p.ids_s1 + i * p.ids_s0); // int32, or the low word of an int64
        v.x = p.x + t * p.x_tok + (i % p.x_per_slot) * p.x_slot;
        v.y = p.y + t * p.y_tok + i * p.y_slot;
        v.rbase = p.row0 + (int64_t) e * p.rows_per_matrix;
    } else {
        v.x = p.x + col * p.x_tok;
        v.y = p.y + col * p.y_tok;
        v.rbase = p.row0;
    }
    return v;
}

// ---------------------------------------------------------------- numeric helpers
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round to nearest even; NaN stays NaN (quiet)
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return (uint16_t) ((u >> 16) | 0x40);
    }
    return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ void store_y(char * y, bool y_bf16, int64_t i, float v) {
    if (y_bf16) {
        ((uint16_t *) y)[i] = f32_to_bf16_rne(v);
    } else {
        ((float *) y)[i] = v;
    }
}

__device__ __forceinline__ float silu(float x) { return x / (1.0f + __expf(-x)); }

// sum over the 32 lanes of each half-wave; every lane of the half gets the result
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
    for (int o = 16; o; o >>= 1) {
        v += __shfl_xor(v, o, 64);
    }
    return v;
}
// sum over the 64 lanes of the wave; every lane gets the result
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        v += __shfl_xor(v, o, 64);
    }
    return v;
}

// Cross-lane sums on the VALU only (DPP operand swizzles, no LDS traffic).  After the four in-row steps every lane
// holds the sum of its row of 16; row_bcast:15 then leaves the sum of lanes 0..31 in lanes 16..31 and of lanes 32..63
// in lanes 48..63, row_bcast:31 the sum of all 64 in lanes 48..63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float row_sum_dpp(float v) {
    v = dpp_add<0xB1, 0xf>(v);  // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);  // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xf>(v); // row_half_mirror
    v = dpp_add<0x140, 0xf>(v); // row_mirror
    return v;
}
// valid in lanes 31 and 63: the sums of lanes 0..31 and 32..63
__device__ __forceinline__ float half_wave_sum_dpp(float v) {
    return dpp_add<0x142, 0xa>(row_sum_dpp(v)); // row_bcast:15 into rows 1 and 3
}
// valid in lane 63: the sum of all 64 lanes
__device__ __forceinline__ float wave_sum_dpp(float v) {
    return dpp_add<0x143, 0xc>(half_wave_sum_dpp(v)); // row_bcast:31 into rows 2 and 3
}

// wave-wide maximum (float) and minimum (uint32) with the same operand swizzles; valid in lane 63.  Lanes a swizzle
// does not reach keep their own value (the "old" operand), which is neutral for max and min.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_take(uint32_t v) {
    return (uint32_t) __builtin_amdgcn_update_dpp((int) v, (int) v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ float wave_max_dpp(float v) {
#define BF16N_STEP(C, M) v = fmaxf(v, __uint_as_float(dpp_take<C, M>(__float_as_uint(v))))
    BF16N_STEP(0xB1, 0xf); BF16N_STEP(0x4E, 0xf); BF16N_STEP(0x141, 0xf); BF16N_STEP(0x140, 0xf);
    BF16N_STEP(0x142, 0xa); BF16N_STEP(0x143, 0xc);
#undef BF16N_STEP
    return v;
}
__device__ __forceinline__ uint32_t wave_min_dpp(uint32_t v) {
#define BF16N_STEP(C, M) { const uint32_t o = dpp_take<C, M>(v); v = o < v ? o : v; }
    BF16N_STEP(0xB1, 0xf) BF16N_STEP(0x4E, 0xf) BF16N_STEP(0x141, 0xf) BF16N_STEP(0x140, 0xf)
    BF16N_STEP(0x142, 0xa) BF16N_STEP(0x143, 0xc)
#undef BF16N_STEP
    return v;
}
__device__ __forceinline__ float lane63(float v) { return __uint_as_float((uint32_t) __builtin_amdgcn_readlane((int) __float_as_uint(v), 63)); }
__device__ __forceinline__ uint32_t lane63(uint32_t v) { return (uint32_t) __builtin_amdgcn_readlane((int) v, 63); }

// ---------------------------------------------------------------- weight assembly
// Plane word = 4 sign|mantissa bytes of 4 adjacent columns.  spread_lo/hi put bytes (0,1) / (2,3) into 16-bit halves
// with the sign in bit 15 and the mantissa in bits 0..6 (other bits hold copies that merge() masks away); merge takes
// the exponent fields (bits 7..14 and 23..30) from a table entry: the result is two BF16 values, lower column low.
__device__ __forceinline__ uint32_t spread_lo(uint32_t smw) { return __builtin_amdgcn_perm(0, smw, 0x01010000u); }
__device__ __forceinline__ uint32_t spread_hi(uint32_t smw) { return __builtin_amdgcn_perm(0, smw, 0x03030202u); }
__device__ __forceinline__ uint32_t merge(uint32_t spread, uint32_t ent) {
    return (spread & 0x807F807Fu) | (ent & ~0x807F807Fu);
}

// dot of two BF16 pairs with FP32 accumulation
__device__ __forceinline__ float dot2_bf16(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, x), acc, false);
}

} // namespace dev
} // namespace bf16n
