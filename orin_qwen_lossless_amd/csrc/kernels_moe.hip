// MoE glue around the expert GEMVs: SiLU gating, weighted combine, expert-sorted routing lists for the batched kernel,
// and the router's softmax + top-k (on the device so that a decode step has no host round trip and can be captured
// into a HIP graph).  All reductions run in a fixed order: results are bitwise reproducible.
#include "dev_common.h"
#include "dev_topk.h"
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
// ids + (t * stride + i) * elem (low 32 bits are read).  Thread i of a round takes token (round * 1024 + i), so a
// wavefront reads adjacent tokens.  First the pairs of lower experts are counted; then, 64 rounds at a time, every
// wavefront records how many of its tokens of a round use the expert, one wavefront turns the (round, wavefront)
// counts into positions, and the tokens that hit write their pair at position + rank inside the wavefront.
constexpr int ROUTE_THREADS = 1024, ROUTE_WAVES = ROUTE_THREADS / 64, ROUTE_ROUNDS = 64;

// what the ids of one token say about expert e: how many are lower, and the last slot that names e (-1: none).
// NU > 0: NU int32 ids per token in 16-byte aligned rows, read four at a time; NU = 0: any element size and count.
template <int NU>
__device__ __forceinline__ void token_ids(const char * __restrict__ ids, int elem, int64_t stride, int n_used, int t, int e, int & lower,
                                          int & slot) {
    if (NU > 0) {
        const int4 * row = (const int4 *) (ids + (int64_t) t * stride * 4);
#pragma unroll
        for (int q = 0; q < NU / 4; q++) {
            const int4 v = row[q];
            const int a[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                lower += a[i] < e;
                slot = a[i] == e ? 4 * q + i : slot;
            }
        }
    } else {
        for (int k = 0; k < n_used; k++) {
            const int v = *(const int32_t *) (ids + ((int64_t) t * stride + k) * elem);
            lower += v < e;
            slot = v == e ? k : slot;
        }
    }
}

template <int NU>
__global__ void __launch_bounds__(ROUTE_THREADS) k_route(const char * __restrict__ ids, int elem, int64_t stride,
                                                         int32_t * __restrict__ ids_src1, int32_t * __restrict__ ids_dst,
                                                         int32_t * __restrict__ bounds, int n_tok, int n_used, int nchannels_y, int sis1) {
    __shared__ int cnt[ROUTE_ROUNDS][ROUTE_WAVES];
    __shared__ int wave_lower[ROUTE_WAVES];
    __shared__ int chunk_total;
    const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int lower = 0;
#pragma unroll 4
    for (int t = tid; t < n_tok; t += ROUTE_THREADS) {
        int slot = -1;
        token_ids<NU>(ids, elem, stride, n_used, t, e, lower, slot);
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        lower += __shfl_xor(lower, o, 64);
    }
    if (lane == 0) {
        wave_lower[wave] = lower;
    }
    __syncthreads();
    int base = 0;
#pragma unroll
    for (int w2 = 0; w2 < ROUTE_WAVES; w2++) {
        base += wave_lower[w2];
    }
    int done = 0; // pairs of this expert in the chunks before
    for (int c0 = 0; c0 < n_tok; c0 += ROUTE_ROUNDS * ROUTE_THREADS) {
        const int left = n_tok - c0;
        const int rounds = left >= ROUTE_ROUNDS * ROUTE_THREADS ? ROUTE_ROUNDS : (left + ROUTE_THREADS - 1) / ROUTE_THREADS;
        uint64_t mine = 0; // rounds in which this thread's token uses the expert
#pragma unroll 4
        for (int r = 0; r < rounds; r++) {
            const int t = c0 + r * ROUTE_THREADS + tid;
            int slot = -1, unused = 0;
            if (t < n_tok) {
                token_ids<NU>(ids, elem, stride, n_used, t, e, unused, slot);
            }
            const bool hit = slot >= 0;
            mine |= (uint64_t) hit << r;
            const uint64_t m = __ballot(hit);
            if (lane == 0) {
                cnt[r][wave] = (int) __builtin_popcountll(m);
            }
        }
        __syncthreads();
        if (wave == 0) { // exclusive prefix over (round, wavefront) in that order; lane r owns round r
            int row = 0;
            if (lane < rounds) {
                for (int w2 = 0; w2 < ROUTE_WAVES; w2++) {
                    const int v = cnt[lane][w2];
                    cnt[lane][w2] = row;
                    row += v;
                }
            }
            int scan = row;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(scan, o, 64);
                scan += lane >= o ? up : 0;
            }
            if (lane < rounds) {
                for (int w2 = 0; w2 < ROUTE_WAVES; w2++) {
                    cnt[lane][w2] += scan - row;
                }
            }
            if (lane == 63) {
                chunk_total = scan;
            }
        }
        __syncthreads();
        for (int r = 0; r < rounds; r++) {
            const bool hit = (mine >> r) & 1;
            const uint64_t m = __ballot(hit);
            if (hit) {
                const int t = c0 + r * ROUTE_THREADS + tid;
                int slot = -1, unused = 0; // a token lists an expert once; were it listed twice, the last slot counts
                token_ids<NU>(ids, elem, stride, n_used, t, e, unused, slot);
                const int rank = (int) __builtin_amdgcn_mbcnt_hi((uint32_t) (m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t) m, 0u));
                const int j = base + done + cnt[r][wave] + rank;
                ids_dst[j] = t * n_used + slot;
                ids_src1[j] = t * sis1 + slot % nchannels_y;
            }
        }
        done += chunk_total;
        __syncthreads(); // cnt and chunk_total are rewritten by the next chunk
    }
    if (tid == 0) {
        bounds[e] = base;
        if (e == (int) gridDim.x - 1) {
            bounds[gridDim.x] = base + done;
        }
    }
}

template <int NQ>
__global__ void __launch_bounds__(64) k_router_topk(const float * __restrict__ logits, int64_t stride, int n_experts, int k, bool renorm,
                                                    int32_t * __restrict__ ids, float * __restrict__ weights, int64_t out_stride) {
    const int t = blockIdx.x;
    topk_token<NQ>(logits + (int64_t) t * stride, n_experts, k, renorm, ids + (int64_t) t * out_stride, weights + (int64_t) t * out_stride,
                   (int) threadIdx.x);
}

// The router's top-k of up to TOPK_ROUTE_TOKENS tokens and the expert-sorted lists of k_route over the first n_slots
// columns of their id rows (the k chosen here, then columns the caller has filled: experts every token uses), in one
// launch of one block: wavefront t selects for token t, then the block sorts the (token, slot) pairs.  The lists are
// those k_route writes for the same ids (entries of an expert in token order; of an expert that a token names twice
// the last slot counts, and bounds count every naming); ids outside [0, n_listed) are left out.
constexpr int TOPK_ROUTE_TOKENS = 16, TOPK_ROUTE_MAX = 1024; // wavefronts of the block; pairs and listed experts
template <int NQ>
__global__ void __launch_bounds__(TOPK_ROUTE_TOKENS * 64) k_router_topk_route(
        const float * __restrict__ logits, int64_t stride, int n_experts, int k, bool renorm, int32_t * ids, float * __restrict__ weights,
        int64_t out_stride, int n_tok, int n_slots, int n_listed, int32_t * __restrict__ ids_src1, int32_t * __restrict__ ids_dst,
        int32_t * __restrict__ bounds, int nchannels_y, int sis1) {
    __shared__ int named[TOPK_ROUTE_MAX];  // namings of an expert, then the start of its list
    __shared__ int listed[TOPK_ROUTE_MAX]; // entries of its list
    __shared__ int named_by[TOPK_ROUTE_MAX]; // expert a pair names
    __shared__ int key[TOPK_ROUTE_MAX];    // expert of a pair that enters a list, else -1
    __shared__ int wave_total[TOPK_ROUTE_TOKENS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pairs = n_tok * n_slots;
    const int t = tid / n_slots, s = tid - t * n_slots;
    int given = -1; // a column the caller filled
    if (tid < pairs && s >= k) {
        given = ids[(int64_t) t * out_stride + s];
    }
    named[tid] = 0;
    listed[tid] = 0;
    if (wave < n_tok) {
        topk_token<NQ>(logits + (int64_t) wave * stride, n_experts, k, renorm, ids + (int64_t) wave * out_stride,
                       weights + (int64_t) wave * out_stride, lane, named_by + wave * n_slots);
    }
    if (tid < pairs && s >= k) {
        named_by[tid] = given;
    }
    __syncthreads();
    int mine = -1;
    if (tid < pairs) {
        const int v = named_by[tid];
        if (v >= 0 && v < n_listed) {
            bool last = true;
            for (int s2 = s + 1; s2 < n_slots; s2++) {
                last &= named_by[tid - s + s2] != v;
            }
            atomicAdd(&named[v], 1);
            if (last) {
                atomicAdd(&listed[v], 1);
                mine = v;
            }
        }
    }
    key[tid] = mine;
    __syncthreads();
    // exclusive prefix of the namings over the experts
    const int c = named[tid]; // 0 from n_listed on
    int scan = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(scan, o, 64);
        scan += lane >= o ? up : 0;
    }
    if (lane == 63) {
        wave_total[wave] = scan;
    }
    __syncthreads();
    int start = scan - c;
#pragma unroll
    for (int w2 = 0; w2 < TOPK_ROUTE_TOKENS; w2++) {
        start += w2 < wave ? wave_total[w2] : 0;
    }
    named[tid] = start;
    if (tid < n_listed) {
        bounds[tid] = start;
        if (tid == n_listed - 1) {
            bounds[n_listed] = start + listed[tid];
        }
    }
    __syncthreads();
    if (mine >= 0) {
        int rank = 0; // pairs are numbered token by token: the earlier entries of this expert's list
#pragma unroll 8
        for (int j = 0; j < tid; j++) {
            rank += key[j] == mine;
        }
        const int j = named[mine] + rank;
        ids_dst[j] = t * n_slots + s;
        ids_src1[j] = t * sis1 + s % nchannels_y;
    }
}

// Residual add + RMS norm of a decode step in one launch (the engines' glue between the products; llama.cpp fuses the
// same chain in its graph).  Per token: sum = a + b + c + sum_k w_k ys_k in FP32 (every addend but a optional; the
// weighted sum over slots is k_moe_combine's fmaf chain, added last), y_sum = bf16(sum) (optional: the new residual),
// y_norm = bf16(sum * rsqrt(mean(sum^2) + eps) * gamma) (gamma optional).  One block per token; a thread keeps its
// elements in registers between the reduction and the scaling (up to NORM_PER_THREAD * 1024 elements per token, the
// rest is recomputed), and the mean is reduced in a fixed order, so the result does not depend on the launch.
constexpr int NORM_THREADS = 1024, NORM_PER_THREAD = 4;
__device__ __forceinline__ float add_norm_value(const add_norm_args & p, const float * wsm, int64_t base, int64_t tok, int64_t i) {
    float v = bf16_bits_to_f32(p.a[base + i]);
    if (p.b) {
        v += bf16_bits_to_f32(p.b[base + i]);
    }
    if (p.c) {
        v += bf16_bits_to_f32(p.c[base + i]);
    }
    if (p.ys) {
        const float * row = p.ys + tok * p.n_used * p.n + i;
        float acc = 0.f;
        for (int k0 = 0; k0 < p.n_used; k0 += 8) { // the loads of eight slots at once, then their fmaf chain in order
            float yk[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                yk[j] = k0 + j < p.n_used ? row[(int64_t) (k0 + j) * p.n] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (k0 + j < p.n_used) {
                    acc = fmaf(wsm[k0 + j], yk[j], acc);
                }
            }
        }
        v += acc;
    }
    return v;
}
__global__ void __launch_bounds__(NORM_THREADS) k_add_rmsnorm(const add_norm_args p) {
    __shared__ float wave_sq[NORM_THREADS / 64];
    __shared__ float wsm[NORM_THREADS]; // the token's routing weights (n_used < 1024)
    const int64_t tok = blockIdx.x, base = tok * p.n;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (p.ys) {
        if (tid < p.n_used) {
            const int64_t s = tok * p.n_used + tid;
            wsm[tid] = p.wts_bf16 ? bf16_bits_to_f32(((const uint16_t *) p.wts)[s]) : ((const float *) p.wts)[s];
        }
        __syncthreads();
    }
    float keep[NORM_PER_THREAD];
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < NORM_PER_THREAD; j++) {
        const int64_t i = tid + (int64_t) j * NORM_THREADS;
        keep[j] = i < p.n ? add_norm_value(p, wsm, base, tok, i) : 0.f;
        sq = fmaf(keep[j], keep[j], sq);
    }
    for (int64_t i = tid + (int64_t) NORM_PER_THREAD * NORM_THREADS; i < p.n; i += NORM_THREADS) {
        const float v = add_norm_value(p, wsm, base, tok, i);
        sq = fmaf(v, v, sq);
    }
    sq = wave_sum(sq);
    if (lane == 0) {
        wave_sq[wave] = sq;
    }
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < NORM_THREADS / 64; k++) {
        total += wave_sq[k];
    }
    const float scale = 1.0f / sqrtf(total / (float) p.n + p.eps);
#pragma unroll
    for (int j = 0; j < NORM_PER_THREAD; j++) {
        const int64_t i = tid + (int64_t) j * NORM_THREADS;
        if (i < p.n) {
            if (p.y_sum) {
                p.y_sum[base + i] = f32_to_bf16_rne(keep[j]);
            }
            p.y_norm[base + i] = f32_to_bf16_rne(keep[j] * scale * (p.gamma ? bf16_bits_to_f32(p.gamma[i]) : 1.0f));
        }
    }
    for (int64_t i = tid + (int64_t) NORM_PER_THREAD * NORM_THREADS; i < p.n; i += NORM_THREADS) {
        const float v = add_norm_value(p, wsm, base, tok, i);
        if (p.y_sum) {
            p.y_sum[base + i] = f32_to_bf16_rne(v);
        }
        p.y_norm[base + i] = f32_to_bf16_rne(v * scale * (p.gamma ? bf16_bits_to_f32(p.gamma[i]) : 1.0f));
    }
}

// The same glue for rows of 2048 elements (16-byte aligned, at most 16 slots): four wavefronts, every thread eight
// consecutive elements through 16-byte loads (a quarter of the wavefronts to start and to meet at the barrier, an
// eighth of the load instructions).  The slot-ordered fmaf chain per element is k_add_rmsnorm's; the mean of squares
// is summed in another (fixed) order.
constexpr int NORM8_THREADS = 256, NORM8_N = 8 * NORM8_THREADS;
__device__ __forceinline__ void unpack8(const uint4 v, float (&f)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = __uint_as_float(w[i] << 16);
        f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        w[i] = f32_to_bf16_rne(f[2 * i]) | ((uint32_t) f32_to_bf16_rne(f[2 * i + 1]) << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}
__global__ void __launch_bounds__(NORM8_THREADS) k_add_rmsnorm8(const add_norm_args p) {
    __shared__ float wave_sq[NORM8_THREADS / 64];
    __shared__ float wsm[16];
    const int64_t tok = blockIdx.x, base = tok * NORM8_N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i0 = 8 * tid;
    // every load of the thread is requested before anything is waited for
    const uint4 va = *(const uint4 *) (p.a + base + i0);
    const uint4 vb = p.b ? *(const uint4 *) (p.b + base + i0) : make_uint4(0, 0, 0, 0);
    const uint4 vc = p.c ? *(const uint4 *) (p.c + base + i0) : make_uint4(0, 0, 0, 0);
    float4 y0[16], y1[16];
    if (p.ys) {
        const float * row = p.ys + tok * p.n_used * NORM8_N + i0;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            if (k < p.n_used) {
                y0[k] = *(const float4 *) (row + (int64_t) k * NORM8_N);
                y1[k] = *(const float4 *) (row + (int64_t) k * NORM8_N + 4);
            }
        }
        if (tid < p.n_used) {
            const int64_t s = tok * p.n_used + tid;
            wsm[tid] = p.wts_bf16 ? bf16_bits_to_f32(((const uint16_t *) p.wts)[s]) : ((const float *) p.wts)[s];
        }
        __syncthreads();
    }
    float v[8], fb[8], fc[8];
    unpack8(va, v);
    unpack8(vb, fb);
    unpack8(vc, fc);
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if (p.b) {
            v[i] += fb[i];
        }
        if (p.c) {
            v[i] += fc[i];
        }
    }
    if (p.ys) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 16; k++) {
            if (k < p.n_used) {
                const float wk = wsm[k];
                acc[0] = fmaf(wk, y0[k].x, acc[0]); acc[1] = fmaf(wk, y0[k].y, acc[1]);
                acc[2] = fmaf(wk, y0[k].z, acc[2]); acc[3] = fmaf(wk, y0[k].w, acc[3]);
                acc[4] = fmaf(wk, y1[k].x, acc[4]); acc[5] = fmaf(wk, y1[k].y, acc[5]);
                acc[6] = fmaf(wk, y1[k].z, acc[6]); acc[7] = fmaf(wk, y1[k].w, acc[7]);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            v[i] += acc[i];
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        sq = fmaf(v[i], v[i], sq);
    }
    sq = wave_sum(sq);
    if (lane == 0) {
        wave_sq[wave] = sq;
    }
    __syncthreads();
    const float total = ((wave_sq[0] + wave_sq[1]) + wave_sq[2]) + wave_sq[3];
    const float scale = 1.0f / sqrtf(total / (float) NORM8_N + p.eps);
    if (p.y_sum) {
        *(uint4 *) (p.y_sum + base + i0) = pack8(v);
    }
    float g[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
    if (p.gamma) {
        unpack8(*(const uint4 *) (p.gamma + i0), g);
    }
    float o[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        o[i] = v[i] * scale * g[i];
    }
    *(uint4 *) (p.y_norm + base + i0) = pack8(o);
}

} // namespace

void launch_add_rmsnorm(const add_norm_args & a, int n_tok, hipStream_t stream) {
    const auto al = [](const void * q) { return ((uintptr_t) q & 15) == 0; };
    if (a.n == NORM8_N && (!a.ys || a.n_used <= 16) && al(a.a) && al(a.b) && al(a.c) && al(a.ys) && al(a.gamma) && al(a.y_sum) && al(a.y_norm)) {
        hipLaunchKernelGGL(k_add_rmsnorm8, dim3(n_tok), dim3(NORM8_THREADS), 0, stream, a);
        return;
    }
    hipLaunchKernelGGL(k_add_rmsnorm, dim3(n_tok), dim3(NORM_THREADS), 0, stream, a);
}

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
    const bool rows_of_8 = !ids_i64 && n_used == 8 && ids_row_stride % 4 == 0 && ((uintptr_t) ids & 15) == 0;
    if (rows_of_8) { // top-8 routing with int32 ids: vector loads
        hipLaunchKernelGGL(k_route<8>, dim3(n_experts), dim3(ROUTE_THREADS), 0, stream, (const char *) ids, 4, ids_row_stride, ids_src1,
                           ids_dst, bounds, n_tok, n_used, nchannels_y, sis1);
    } else {
        hipLaunchKernelGGL(k_route<0>, dim3(n_experts), dim3(ROUTE_THREADS), 0, stream, (const char *) ids, ids_i64 ? 8 : 4, ids_row_stride,
                           ids_src1, ids_dst, bounds, n_tok, n_used, nchannels_y, sis1);
    }
}

// out_stride: elements between the tokens' rows of ids and weights (k when they are dense)
void launch_router_topk_strided(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                                float * weights, int64_t out_stride, hipStream_t stream) {
    if (n_experts <= 256) {
        hipLaunchKernelGGL(k_router_topk<4>, dim3(n_tok), dim3(64), 0, stream, logits, stride, n_experts, k, renorm, ids, weights, out_stride);
    } else {
        hipLaunchKernelGGL(k_router_topk<16>, dim3(n_tok), dim3(64), 0, stream, logits, stride, n_experts, k, renorm, ids, weights, out_stride);
    }
}
bool router_topk_route_fits(int n_tok, int n_slots, int n_listed) {
    return n_tok <= TOPK_ROUTE_TOKENS && (int64_t) n_tok * n_slots <= TOPK_ROUTE_MAX && n_listed <= TOPK_ROUTE_MAX;
}
void launch_router_topk_route(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                              float * weights, int64_t out_stride, int n_slots, int n_listed, int32_t * ids_src1, int32_t * ids_dst,
                              int32_t * bounds, int nchannels_y, int sis1, hipStream_t stream) {
    if (!router_topk_route_fits(n_tok, n_slots, n_listed)) {
        throw std::invalid_argument("router_topk_route: at most 16 tokens, 1024 (token, slot) pairs and 1024 listed experts");
    }
    if (n_experts <= 256) {
        hipLaunchKernelGGL(k_router_topk_route<4>, dim3(1), dim3(TOPK_ROUTE_TOKENS * 64), 0, stream, logits, stride, n_experts, k, renorm,
                           ids, weights, out_stride, n_tok, n_slots, n_listed, ids_src1, ids_dst, bounds, nchannels_y, sis1);
    } else {
        hipLaunchKernelGGL(k_router_topk_route<16>, dim3(1), dim3(TOPK_ROUTE_TOKENS * 64), 0, stream, logits, stride, n_experts, k, renorm,
                           ids, weights, out_stride, n_tok, n_slots, n_listed, ids_src1, ids_dst, bounds, nchannels_y, sis1);
    }
}
void launch_router_topk(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                        float * weights, hipStream_t stream) {
    launch_router_topk_strided(logits, stride, n_tok, n_experts, k, renorm, ids, weights, k, stream);
}

} // namespace dev
} // namespace bf16n
