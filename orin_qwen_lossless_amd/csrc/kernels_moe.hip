// MoE glue around the expert GEMVs: SiLU gating, weighted combine, expert-sorted routing lists for the batched kernel,
// and the router's softmax + top-k (on the device so that a decode step has no host round trip and can be captured
// into a HIP graph).  All reductions run in a fixed order: results are bitwise reproducible.
#include "dev_common.h"
#include "launchers.h"

namespace bf16n {
namespace dev {

namespace {

// y = silu(g) * u (reference launch.cu:554-558)
__global__ void __launch_bounds__(256) k_swiglu(const float * __restrict__ g, const float * __restrict__ u, float * __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t) gridDim.x * 256) {
        y[i] = silu(g[i]) * u[i];
    }
}

// y[t, i] = sum_k w[t, k] * ys[t, k, i], slots in order, one fmaf each (reference launch.cu:539-552)
__global__ void __launch_bounds__(256) k_moe_combine(const float * __restrict__ ys, const char * __restrict__ w, bool w_bf16,
                                                     char * __restrict__ y, bool y_bf16, int n_used, int64_t n) {
    const int t = blockIdx.y;
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t) gridDim.x * 256) {
        float acc = 0.f;
        for (int k = 0; k < n_used; k++) {
            const int64_t s = (int64_t) t * n_used + k;
            const float wk = w_bf16 ? bf16_bits_to_f32(((const uint16_t *) w)[s]) : ((const float *) w)[s];
            acc = fmaf(wk, ys[s * n + i], acc);
        }
        store_y(y + (int64_t) t * n * (y_bf16 ? 2 : 4), y_bf16, i, acc);
    }
}

// Routing lists (reference mmid_helper.cu:48-136): block e lists the (token, slot) pairs of expert e in token order at
// positions bounds[e].., where bounds[e] = number of pairs of experts < e.  ids element i of token t at byte
// ids + (t * stride + i) * elem (low 32 bits are read).  Every thread owns a run of consecutive tokens: it counts its
// pairs of lower experts and its own hits, one block-wide scan turns the hit counts into positions, and a second walk
// over the run writes the lists.
__global__ void __launch_bounds__(256) k_route(const char * __restrict__ ids, int elem, int64_t stride, int32_t * __restrict__ ids_src1,
                                               int32_t * __restrict__ ids_dst, int32_t * __restrict__ bounds, int n_tok, int n_used,
                                               int nchannels_y, int sis1) {
    __shared__ int wave_hits[4], wave_lower[4];
    const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per = (n_tok + 255) / 256;
    const int t_begin = tid * per < n_tok ? tid * per : n_tok, t_end = t_begin + per < n_tok ? t_begin + per : n_tok;
    int lower = 0, hits = 0;
    for (int t = t_begin; t < t_end; t++) {
        bool hit = false;
        for (int k = 0; k < n_used; k++) {
            const int v = *(const int32_t *) (ids + ((int64_t) t * stride + k) * elem);
            lower += v < e;
            hit |= v == e;
        }
        hits += hit;
    }
    // inclusive scan of the hit counts and sum of the lower counts inside the wavefront, then over the four wavefronts
    int scan = hits;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(scan, o, 64);
        scan += lane >= o ? up : 0;
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        lower += __shfl_xor(lower, o, 64);
    }
    if (lane == 63) {
        wave_hits[wave] = scan;
        wave_lower[wave] = lower;
    }
    __syncthreads();
    const int base = wave_lower[0] + wave_lower[1] + wave_lower[2] + wave_lower[3];
    int j = base + scan - hits;
    for (int w2 = 0; w2 < wave; w2++) {
        j += wave_hits[w2];
    }
    for (int t = t_begin; t < t_end; t++) {
        int slot = -1;
        for (int k = 0; k < n_used; k++) {
            if (*(const int32_t *) (ids + ((int64_t) t * stride + k) * elem) == e) {
                slot = k; // a token lists an expert once; were it listed twice, the last slot counts
            }
        }
        if (slot >= 0) {
            ids_dst[j] = t * n_used + slot;
            ids_src1[j] = t * sis1 + slot % nchannels_y;
            j++;
        }
    }
    if (tid == 0) {
        bounds[e] = base;
        if (e == (int) gridDim.x - 1) {
            bounds[gridDim.x] = base + wave_hits[0] + wave_hits[1] + wave_hits[2] + wave_hits[3];
        }
    }
}

// softmax over the experts, k largest (ties: lower index), weights renormalised to sum 1 if asked; one wave per token.
// The logits of a token sit in registers (NQ per lane, expert = lane + 64 q); every selection is two wave reductions
// on the VALU: the maximum, then the smallest index that holds it.  NaN logits count as -inf, and a selection only
// ever returns an index below n_experts that was not taken before, whatever the values are: the ids feed address
// arithmetic in the kernels that follow.
template <int NQ>
__global__ void __launch_bounds__(64) k_router_topk(const float * __restrict__ logits, int64_t stride, int n_experts, int k, bool renorm,
                                                    int32_t * __restrict__ ids, float * __restrict__ weights) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float * lg = logits + (int64_t) t * stride;
    float val[NQ];
    bool open[NQ]; // a real expert that has not been taken yet
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        const int i = lane + 64 * q;
        open[q] = i < n_experts;
        const float v = open[q] ? lg[i] : -INFINITY;
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
            ids[(int64_t) t * k + j] = (int32_t) bi;
        }
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            open[q] = open[q] && (uint32_t) (lane + 64 * q) != bi;
        }
    }
    if (lane < k) {
        weights[(int64_t) t * k + lane] = renorm ? mine / top : mine;
    }
}

} // namespace

void launch_swiglu(const float * g, const float * u, float * y, int64_t n, int cus, hipStream_t stream) {
    const int64_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(k_swiglu, dim3((unsigned) (blocks < (int64_t) cus * 8 ? blocks : (int64_t) cus * 8)), dim3(256), 0, stream, g, u, y, n);
}

void launch_moe_combine(const float * ys, const void * w, bool w_bf16, void * y, bool y_bf16, int n_tok, int n_used, int64_t n,
                        hipStream_t stream) {
    const int64_t bx = (n + 255) / 256;
    hipLaunchKernelGGL(k_moe_combine, dim3((unsigned) (bx < 64 ? bx : 64), (unsigned) n_tok), dim3(256), 0, stream, ys, (const char *) w,
                       w_bf16, (char *) y, y_bf16, n_used, n);
}

void launch_route(const void * ids, bool ids_i64, int64_t ids_row_stride, int32_t * ids_src1, int32_t * ids_dst, int32_t * bounds,
                  int n_experts, int n_tok, int n_used, int nchannels_y, int sis1, hipStream_t stream) {
    hipLaunchKernelGGL(k_route, dim3(n_experts), dim3(256), 0, stream, (const char *) ids, ids_i64 ? 8 : 4, ids_row_stride, ids_src1,
                       ids_dst, bounds, n_tok, n_used, nchannels_y, sis1);
}

void launch_router_topk(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                        float * weights, hipStream_t stream) {
    if (n_experts <= 256) {
        hipLaunchKernelGGL(k_router_topk<4>, dim3(n_tok), dim3(64), 0, stream, logits, stride, n_experts, k, renorm, ids, weights);
    } else {
        hipLaunchKernelGGL(k_router_topk<16>, dim3(n_tok), dim3(64), 0, stream, logits, stride, n_experts, k, renorm, ids, weights);
    }
}

} // namespace dev
} // namespace bf16n
