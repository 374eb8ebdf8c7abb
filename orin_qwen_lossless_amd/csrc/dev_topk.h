// The router's selection for one token by one wavefront, shared by the stand-alone top-k kernels (kernels_moe.hip) and
// the routed GEMV that selects in its prologue (kernels_tile.hip).
#pragma once

#include "dev_common.h"

namespace bf16n {
namespace dev {

// softmax over the experts, k largest (ties: lower index), weights renormalised to sum 1 if asked; one wave per token.
// The logits of a token sit in registers (NQ per lane, expert = lane + 64 q); every selection is two wave reductions
// on the VALU: the maximum, then the smallest index that holds it.  NaN logits count as -inf, and a selection only
// ever returns an index below n_experts that was not taken before, whatever the values are: the ids feed address
// arithmetic in the kernels that follow.
// the logits of a token into registers (issued early by callers that have other loads to overlap them with)
template <int NQ>
__device__ __forceinline__ void topk_load(const float * __restrict__ lg, int n_experts, int lane, float (&val)[NQ], bool (&open)[NQ]) {
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        const int i = lane + 64 * q;
        open[q] = i < n_experts;
        val[q] = open[q] ? lg[i] : -INFINITY;
    }
}

// the selection on loaded logits; ids_row / weights_row / ids_copy may be global or LDS rows
template <int NQ>
__device__ __forceinline__ void topk_select(float (&val)[NQ], bool (&open)[NQ], int k, bool renorm, int32_t * ids_row, float * weights_row,
                                            int lane, int * ids_copy = nullptr) {
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        const float v = val[q];
        val[q] = v != v ? -INFINITY : v;
        mx = fmaxf(mx, val[q]);
    }
    mx = lane63(wave_max_dpp(mx));
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        sum += open[q] ? expf(val[q] - mx) : 0.f;
    }
    sum = lane63(wave_sum_dpp(sum));
    float top = 0.f, mine = 0.f; // lane j keeps the j-th weight
    for (int j = 0; j < k; j++) {
        float bv = -INFINITY;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            bv = open[q] ? fmaxf(bv, val[q]) : bv;
        }
        bv = lane63(wave_max_dpp(bv));
        uint32_t bi = 0xFFFFFFFFu;
#pragma unroll
        for (int q = NQ - 1; q >= 0; q--) {
            bi = open[q] && val[q] == bv ? (uint32_t) (lane + 64 * q) : bi; // descending q: the lane's lowest index stays
        }
        bi = lane63(wave_min_dpp(bi)); // k <= n_experts: an open expert holds the maximum of the open ones
        const float pj = expf(bv - mx) / sum;
        top += pj;
        if (lane == (j & 63)) {
            mine = pj; // k <= 64
            ids_row[j] = (int32_t) bi;
            if (ids_copy) {
                ids_copy[j] = (int) bi;
            }
        }
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            open[q] = open[q] && (uint32_t) (lane + 64 * q) != bi;
        }
    }
    if (lane < k) {
        weights_row[lane] = renorm ? mine / top : mine;
    }
}

template <int NQ>
__device__ __forceinline__ void topk_token(const float * __restrict__ lg, int n_experts, int k, bool renorm, int32_t * ids_row,
                                           float * weights_row, int lane, int * ids_copy = nullptr) {
    float val[NQ];
    bool open[NQ]; // a real expert that has not been taken yet
    topk_load<NQ>(lg, n_experts, lane, val, open);
    topk_select<NQ>(val, open, k, renorm, ids_row, weights_row, lane, ids_copy);
}

// what a GEMV needs to select the experts of its token itself: the router's logits and the rows to leave the result in
struct topk_args {
    const float * logits; int64_t stride; // one row of n_experts logits per token
    int n_experts, k;
    bool renorm;
    float * weights; int64_t out_stride;  // weights row of token t at weights + t * out_stride (the ids go to the launch's id rows)
};

} // namespace dev
} // namespace bf16n
