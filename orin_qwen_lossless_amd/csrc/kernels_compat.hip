// Kernels for the reference's 32-lane layouts: HUFPAIR row-/chunk-major, HUFFMAN and NIBBLE (GEMV, GLU-GEMV, exact
// dequant, row gather).  Buffers made by the reference encoder decode here unchanged.
//
// A wave64 carries two units (HUFPAIR / HUFFMAN) or two rows (NIBBLE): lanes 0..31 the even one, lanes 32..63 the odd
// one; each half reads its 512-byte plane chunk with one 16-byte load per lane.  Lane streams are per-lane sequential
// reads through the vector cache.  These kernels favour generality (any K, R, layout, expert ids, FP32 or BF16
// activations) over speed; the wave64 layout (kernels_w64.hip) is the fast path.
#include "dev_common.h"
#include "dev_compat.h"
#include "launchers.h"

namespace bf16n {
namespace dev {

namespace {

constexpr int NT = 256;          // threads per block
constexpr int NIB_MM_MIN_COLS = 5; // dense NIBBLE batches of BF16 columns go through the matrix cores from this many on at the earliest
constexpr int HALVES = NT / 32;  // units (rows) per block

template <typename TX>
__device__ __forceinline__ float x_at(const char * x, int i);
template <> __device__ __forceinline__ float x_at<float>(const char * x, int i) { return ((const float *) x)[i]; }
template <> __device__ __forceinline__ float x_at<bf16_t>(const char * x, int i) { return bf16_bits_to_f32(((const uint16_t *) x)[i]); }

__device__ __forceinline__ float dot_chunk(const uint32_t (&wp)[8], const float * xs, int l32) {
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float4 xv = *(const float4 *) (xs + 128 * j + 4 * l32);
        a0 = fmaf(bf16_bits_to_f32(wp[2 * j] & 0xFFFFu), xv.x, a0);
        a1 = fmaf(__uint_as_float(wp[2 * j] & 0xFFFF0000u), xv.y, a1);
        a2 = fmaf(bf16_bits_to_f32(wp[2 * j + 1] & 0xFFFFu), xv.z, a2);
        a3 = fmaf(__uint_as_float(wp[2 * j + 1] & 0xFFFF0000u), xv.w, a3);
    }
    return (a0 + a1) + (a2 + a3);
}

// One unit of R rows: y[rr] (rr < R) ends up in lane rr of the half-wave.  Row-major streams finish a row every C
// chunks; chunk-major streams add one partial sum per (chunk, row).
template <int FORMAT>
__device__ __forceinline__ float unit_dot(const uint8_t * plane, const uint32_t * lut, const uint32_t * sp, int64_t gu, int R,
                                          int C, bool cm, const float * xs, int l32) {
    lane_bits bits;
    bits.begin(sp);
    const uint8_t * up = plane + gu * R * (int64_t) C * CHUNK;
    float mine = 0.f;
    if (cm) {
        for (int c = 0; c < C; c++) {
            for (int rr = 0; rr < R; rr++) {
                uint32_t wp[8];
                decode_chunk<FORMAT>(bits, lut, *((const uint4 *) (up + ((int64_t) c * R + rr) * CHUNK) + l32), wp);
                const float s = half_wave_sum(dot_chunk(wp, xs + c * CHUNK, l32));
                mine += l32 == rr ? s : 0.f;
            }
        }
    } else {
        for (int rr = 0; rr < R; rr++) {
            float acc = 0.f;
            for (int c = 0; c < C; c++) {
                uint32_t wp[8];
                decode_chunk<FORMAT>(bits, lut, *((const uint4 *) (up + ((int64_t) rr * C + c) * CHUNK) + l32), wp);
                acc += dot_chunk(wp, xs + c * CHUNK, l32);
            }
            const float s = half_wave_sum(acc);
            mine = l32 == rr ? s : mine;
        }
    }
    return mine;
}

template <int FORMAT>
__device__ __forceinline__ const uint32_t * lane_stream(const bf16n_weight & w, int64_t gu, int l32) {
    if (FORMAT == FMT_HUFPAIR) {
        const hp_ptrs p = hpp(w);
        return p.stream + p.ubase[gu] + p.lrel[gu * 32 + l32];
    }
    const huf_ptrs p = hufp(w);
    return p.stream + p.lane_off[gu * 32 + l32];
}

// y = W x (GLU: y = silu(gate x) * up x) for HUFPAIR / HUFFMAN in the 32-lane layouts; one half-wave per unit,
// blockIdx.y = column.  Shared memory: x as FP32 [K], then one table per matrix.
template <int FORMAT, typename TX, bool GLU>
__global__ void __launch_bounds__(NT) k_huf_mmv(const bf16n_weight w, const bf16n_weight w_up, const cols p) {
    constexpr int LUT_N = FORMAT == FMT_HUFPAIR ? (1 << HP_LP) : (1 << HUF_LMAX);
    extern __shared__ __align__(16) unsigned char shm_raw[];
    const int K = (int) w.K, C = K / CHUNK, R = w.R;
    float * xs = (float *) shm_raw;
    uint32_t * lut = (uint32_t *) (xs + K);
    uint32_t * lut_up = lut + LUT_N;
    const col_view cv = col_setup(p, blockIdx.y);
    for (int i = threadIdx.x; i < K; i += NT) {
        xs[i] = x_at<TX>(cv.x, i);
    }
    const uint32_t * lut_g = (const uint32_t *) (w.aux + w.off_a);
    for (int i = threadIdx.x; i < LUT_N; i += NT) {
        lut[i] = lut_g[i];
    }
    if (GLU) {
        const uint32_t * lut_ug = (const uint32_t *) (w_up.aux + w_up.off_a);
        for (int i = threadIdx.x; i < LUT_N; i += NT) {
            lut_up[i] = lut_ug[i];
        }
    }
    __syncthreads();
    const int l32 = threadIdx.x & 31, half = threadIdx.x >> 5;
    const bool cm = (w.flags & FLAG_CHUNK_MAJOR) != 0;
    const int64_t units = p.nrows / R;
    for (int64_t u = (int64_t) blockIdx.x * HALVES + half; u < units; u += (int64_t) gridDim.x * HALVES) {
        const int64_t gu = cv.rbase / R + u;
        float v = unit_dot<FORMAT>(w.plane, lut, lane_stream<FORMAT>(w, gu, l32), gu, R, C, cm, xs, l32);
        if (GLU) {
            const float uv = unit_dot<FORMAT>(w_up.plane, lut_up, lane_stream<FORMAT>(w_up, gu, l32), gu, R, C, false, xs, l32);
            v = uv * silu(v);
        }
        if (l32 < R) {
            store_y(cv.y, p.y_bf16, u * R + l32, v);
        }
    }
}

// exact BF16 bits of rows [row0, row0 + nrows) (whole units), row-major; one half-wave per unit
template <int FORMAT>
__global__ void __launch_bounds__(NT) k_huf_dequant(const bf16n_weight w, int64_t row0, int64_t nrows, uint16_t * __restrict__ out) {
    constexpr int LUT_N = FORMAT == FMT_HUFPAIR ? (1 << HP_LP) : (1 << HUF_LMAX);
    __shared__ uint32_t lut[LUT_N];
    const uint32_t * lut_g = (const uint32_t *) (w.aux + w.off_a);
    for (int i = threadIdx.x; i < LUT_N; i += NT) {
        lut[i] = lut_g[i];
    }
    __syncthreads();
    const int K = (int) w.K, C = K / CHUNK, R = w.R;
    const bool cm = (w.flags & FLAG_CHUNK_MAJOR) != 0;
    const int l32 = threadIdx.x & 31, half = threadIdx.x >> 5;
    for (int64_t u = (int64_t) blockIdx.x * HALVES + half; u < nrows / R; u += (int64_t) gridDim.x * HALVES) {
        const int64_t gu = row0 / R + u;
        lane_bits bits;
        bits.begin(lane_stream<FORMAT>(w, gu, l32));
        const uint8_t * up = w.plane + gu * R * (int64_t) K;
        for (int o = 0; o < R * C; o++) {
            const int rr = cm ? o % R : o / C, c = cm ? o / R : o % C;
            uint32_t wp[8];
            decode_chunk<FORMAT>(bits, lut, *((const uint4 *) (up + (int64_t) o * CHUNK) + l32), wp);
            uint16_t * dst = out + (u * R + rr) * K + c * CHUNK;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *(uint2 *) (dst + 128 * j + 4 * l32) = make_uint2(wp[2 * j], wp[2 * j + 1]);
            }
        }
    }
}

// dst[i] = row (row0 + ids[i]) as FP32 or BF16: the half-wave decodes the row's unit from its start and stores only
// the requested row (reference kernels.cuh:840-891)
template <bool BF>
__global__ void __launch_bounds__(NT) k_hp_get_rows(const bf16n_weight w, const char * __restrict__ ids, int64_t ids_s0, int64_t n,
                                                    int64_t row0, char * __restrict__ dst, int64_t dst_s1) {
    __shared__ uint32_t lut[1 << HP_LP];
    const uint32_t * lut_g = (const uint32_t *) (w.aux + w.off_a);
    for (int i = threadIdx.x; i < (1 << HP_LP); i += NT) {
        lut[i] = lut_g[i];
    }
    __syncthreads();
    const int K = (int) w.K, C = K / CHUNK, R = w.R;
    const int l32 = threadIdx.x & 31, half = threadIdx.x >> 5;
    const int64_t i = (int64_t) blockIdx.x * HALVES + half;
    if (i >= n) {
        return;
    }
    const int64_t gr = row0 + *(const int32_t *) (ids + i * ids_s0);
    const int64_t gu = gr / R;
    lane_bits bits;
    bits.begin(lane_stream<FMT_HUFPAIR>(w, gu, l32));
    char * o = dst + i * dst_s1;
    for (int64_t r = gu * R; r <= gr; r++) {
        for (int c = 0; c < C; c++) {
            uint32_t wp[8];
            decode_chunk<FMT_HUFPAIR>(bits, lut, *((const uint4 *) (w.plane + r * K + c * CHUNK) + l32), wp);
            if (r == gr) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int col = c * CHUNK + 128 * j + 4 * l32;
                    if (BF) {
                        *(uint2 *) (o + 2 * col) = make_uint2(wp[2 * j], wp[2 * j + 1]);
                    } else {
                        *(float4 *) (o + 4 * col) = make_float4(bf16_bits_to_f32(wp[2 * j] & 0xFFFFu), __uint_as_float(wp[2 * j] & 0xFFFF0000u),
                                                                bf16_bits_to_f32(wp[2 * j + 1] & 0xFFFFu), __uint_as_float(wp[2 * j + 1] & 0xFFFF0000u));
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- NIBBLE

// the 16 activations one lane meets in a 512-column chunk (columns 128 j + 4 l + 0..3), as FP32
template <typename TX>
__device__ __forceinline__ void x_chunk16(const char * x, int col0, float (&xv)[16]);
template <> __device__ __forceinline__ void x_chunk16<float>(const char * x, int col0, float (&xv)[16]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float4 t = *(const float4 *) (x + 4 * (col0 + 128 * j));
        xv[4 * j] = t.x; xv[4 * j + 1] = t.y; xv[4 * j + 2] = t.z; xv[4 * j + 3] = t.w;
    }
}
template <> __device__ __forceinline__ void x_chunk16<bf16_t>(const char * x, int col0, float (&xv)[16]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint2 t = *(const uint2 *) (x + 2 * (col0 + 128 * j));
        xv[4 * j] = __uint_as_float(t.x << 16); xv[4 * j + 1] = __uint_as_float(t.x & 0xFFFF0000u);
        xv[4 * j + 2] = __uint_as_float(t.y << 16); xv[4 * j + 3] = __uint_as_float(t.y & 0xFFFF0000u);
    }
}

// the 16 weights of one lane in (row gr, chunk c) as 8 BF16 pairs; escaped weights read as +0 here
__device__ __forceinline__ void nib_load_chunk(const nib_ptrs & w, int64_t gr, int C, int c, const uint4 T, int l32, uint32_t (&wp)[8]) {
    const int64_t K = (int64_t) C * CHUNK;
    const uint4 sm = *((const uint4 *) (w.plane + gr * K + c * CHUNK) + l32);
    const uint2 cd = *((const uint2 *) (w.codes + gr * (K / 2) + c * 256) + l32);
    nib_chunk(sm, cd, T, wp);
}

// partial dot of a decoded chunk with x.  The four per-position sums are combined as in the reference
// (kernels.cuh:130-187), then over the 32 lanes on the VALU (DPP, no LDS traffic); result in lane 31 of the half-wave.
__device__ __forceinline__ float nib_dot(const uint32_t (&wp)[8], const float (&xv)[16]) {
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        a0 = fmaf(bf16_bits_to_f32(wp[2 * j] & 0xFFFFu), xv[4 * j], a0);
        a1 = fmaf(__uint_as_float(wp[2 * j] & 0xFFFF0000u), xv[4 * j + 1], a1);
        a2 = fmaf(bf16_bits_to_f32(wp[2 * j + 1] & 0xFFFFu), xv[4 * j + 2], a2);
        a3 = fmaf(__uint_as_float(wp[2 * j + 1] & 0xFFFF0000u), xv[4 * j + 3], a3);
    }
    return half_wave_sum_dpp((a0 + a1) + (a2 + a3));
}

// the same with BF16 activations left as the 8 pairs they arrive in: a pair of weights meets a pair of activations in
// one dot2 instruction (8 instructions where conversions and FMAs took 48)
__device__ __forceinline__ void x_pairs16(const char * x, int col0, uint32_t (&xp)[8]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint2 t = *(const uint2 *) (x + 2 * (col0 + 128 * j));
        xp[2 * j] = t.x;
        xp[2 * j + 1] = t.y;
    }
}
__device__ __forceinline__ float nib_dot_pairs(const uint32_t (&wp)[8], const uint32_t (&xp)[8]) {
    float a01 = 0.f, a23 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        a01 = dot2_bf16(wp[2 * j], xp[2 * j], a01);
        a23 = dot2_bf16(wp[2 * j + 1], xp[2 * j + 1], a23);
    }
    return half_wave_sum_dpp(a01 + a23);
}

// the exact products of a row's escaped weights, summed over the half-wave (result in lane 31)
// (e0, e1: the row's range of escape records, esc_off[gr] and esc_off[gr + 1], which the caller requests together with
// the row's other loads: 3 to 8 % off the four-column launches)
template <typename TX>
__device__ __forceinline__ float nib_escapes(const nib_ptrs & w, uint32_t e0, uint32_t e1, const char * x, int l32) {
    float acc = 0.f;
    for (uint32_t i = e0 + l32; i < e1; i += 32) {
        const uint32_t rec = w.esc[i];
        acc = fmaf(bf16_bits_to_f32(esc_bits(rec)), x_at<TX>(x, (int) (rec & 0xFFFu)), acc);
    }
    return e1 > e0 ? half_wave_sum_dpp(acc) : 0.f;
}

// NIBBLE GEMV; GLU 1: rows_per_matrix = [gate (nrows); up (nrows)] of one matrix; GLU 2: separate gate / up matrices.
// These matrices are small (a few MB at most), so the launch is laid out for latency: one half-wave per (row, chunk)
// pair, every load of a pair issued at once, the C chunk sums of a row combined through LDS in chunk order.
// NC: columns per decode (dense batches: a (row, chunk) is decoded once for NC token columns, each of which gets the
// bits of its single-column launch); columns past the last repeat it and are not stored.
template <typename TX, int GLU, int NC>
__global__ void __launch_bounds__(NT) k_nib_mmv(const bf16n_weight w, const bf16n_weight w_up, const cols p, const int ncols) {
    __shared__ float part[2][NC][HALVES];
    const int K = (int) w.K, C = K / CHUNK; // 1 .. 8
    col_view cv[NC];
#pragma unroll
    for (int j = 0; j < NC; j++) {
        const int col = (int) blockIdx.y * NC + j;
        cv[j] = col_setup(p, col < ncols ? col : ncols - 1);
    }
    const nib_ptrs g = nibp(w, 0);
    const nib_ptrs u = GLU == 1 ? nibp(w, p.nrows) : nibp(w_up, 0);
    const int l32 = threadIdx.x & 31, half = threadIdx.x >> 5;
    const int rpb = HALVES / C; // rows per block: C half-waves per row (C = 3, 5, 6, 7 leave some half-waves idle)
    const int lr = half / C, c = half % C;
    for (int64_t base = (int64_t) blockIdx.x * rpb; base < p.nrows; base += (int64_t) gridDim.x * rpb) {
        const bool live = lr < rpb && base + lr < p.nrows;
        const int64_t r = live ? base + lr : 0;
        const int64_t gr = cv[0].rbase + r; // dense batches share the rows; with expert ids NC is 1
        uint32_t wg[8], wu[8];
        const uint2 eg = make_uint2(g.esc_off[gr], g.esc_off[gr + 1]);
        const uint2 eu = GLU ? make_uint2(u.esc_off[gr], u.esc_off[gr + 1]) : make_uint2(0, 0);
        nib_load_chunk(g, gr, C, c, *(const uint4 *) (g.table + gr * 16), l32, wg);
        if (GLU) {
            nib_load_chunk(u, gr, C, c, *(const uint4 *) (u.table + gr * 16), l32, wu);
        }
#pragma unroll
        for (int j = 0; j < NC; j++) {
            float v, vu = 0.f;
            if constexpr (sizeof(TX) == 2) {
                uint32_t xp[8];
                x_pairs16(cv[j].x, c * CHUNK + 4 * l32, xp);
                v = nib_dot_pairs(wg, xp);
                if (GLU) {
                    vu = nib_dot_pairs(wu, xp);
                }
            } else {
                float xv[16];
                x_chunk16<TX>(cv[j].x, c * CHUNK + 4 * l32, xv);
                v = nib_dot(wg, xv);
                if (GLU) {
                    vu = nib_dot(wu, xv);
                }
            }
            if (c == 0) {
                v += nib_escapes<TX>(g, eg.x, eg.y, cv[j].x, l32);
                if (GLU) {
                    vu += nib_escapes<TX>(u, eu.x, eu.y, cv[j].x, l32);
                }
            }
            if (l32 == 31) {
                part[0][j][half] = v;
                part[1][j][half] = vu;
            }
        }
        __syncthreads();
        if (live && c == 0 && l32 < NC && (int) blockIdx.y * NC + l32 < ncols) {
            float s = part[0][l32][half], su = part[1][l32][half];
            for (int i = 1; i < C; i++) {
                s += part[0][l32][half + i];
                su += part[1][l32][half + i];
            }
            store_y(cv[0].y + l32 * p.y_tok, p.y_bf16, r, GLU ? su * silu(s) : s); // l32 > 0 only in dense batches
        }
        __syncthreads();
    }
}

// Dense NIBBLE products through the matrix cores: y[t] = W x[t] for BF16 token columns, 32 per block (gridDim.y blocks
// of tokens; columns past the last repeat it and are not stored).  The 4-bit code has no decode chain, so one decode of
// the matrix serves 32 tokens at the cost of one.  A block is one group of 32 rows with K / 256 wavefronts; wavefront v
// takes half a chunk: the slots [16 (v & 1), +16) of chunk v / 2.  Lane (row r, half h) decodes two adjacent slots of
// its row per step, 16 (v & 1) + 4n + 2h and the next (n = 0..3): 32 weights, which are eight adjacent columns
// 128 j + 64 (v & 1) + 16 n + 8 h + [0, 8) in each of the chunk's four column blocks j — the A operands of four matrix
// instructions (k positions 8h + [0, 8) of instruction j) — and lane (token t, half h) supplies the same columns of its
// token's activations as B operands, one 16-byte load each: which columns an instruction's k positions stand for is
// free as long as both operands agree.  (The activations staged through LDS by loads that take a token's 128 bytes
// with eight adjacent lanes measured the same for K = 2048 and, in two turns of eight wavefronts, slower for K = 4096:
// a launch is a few serial latencies, not the rate of its loads.)  BF16 products are exact in FP32; the partial sums of
// the wavefronts are added in K order through LDS, the products of escaped weights (decoded as +0) last, and the sum
// is rounded once.
typedef __bf16 nm_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float nm_f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t nm_u32x4_t __attribute__((ext_vector_type(4)));
constexpr int NM_WAVES = 8; // per block: K / 256 half chunks in one turn each, K > 2048 in two
// Words per (wavefront, accumulator register) row of the partial sums in LDS: lane l at l + l / 32.  The threads that add
// the partial sums of one token's 32 rows read 16 registers x 2 half-waves of one lane position: 64 words apart they
// all met one bank (32-way conflicts: 7,900 conflict cycles per block, 3 of a launch's 14 us), 66 apart with the
// upper half-wave shifted by one they spread over all banks, two to a bank.
constexpr int NM_PSTRIDE = 66;
__device__ __forceinline__ int nm_part_at(int wave, int i, int lane) { return (wave * 16 + i) * NM_PSTRIDE + lane + (lane >> 5); }

// TURNS: half chunks per wavefront (wavefront v takes v TURNS + [0, TURNS)).  The loads of a wavefront are written
// ahead of their uses; with one turn the compiler issues them in batches of about nine (68 registers, three blocks per
// CU).  All 28 pinned ahead of the first use (a scheduling barrier; 148 registers) measured 2 to 6 % faster for
// 5120 x 2048 up to 32 columns, 30 % slower at 64 (one block per CU), and with two turns 5 to 7 % slower (256
// registers and spills): left to the compiler.
template <int TURNS>
__global__ void __launch_bounds__(NM_WAVES * 64) k_nib_mm(const bf16n_weight w, const cols p, const int ncols) {
    extern __shared__ __align__(16) float nm_part[]; // [wavefront][accumulator register][lane]
    const nib_ptrs q = nibp(w, 0);
    const int K = (int) w.K;
    const int lane = threadIdx.x & 63, r = lane & 31, h = lane >> 5, wave = (int) (threadIdx.x >> 6), n_waves = (int) (blockDim.x >> 6);
    const int64_t g0 = (int64_t) blockIdx.x * 32;
    const int64_t row = p.row0 + (g0 + r < p.nrows ? g0 + r : p.nrows - 1);
    const int t0 = (int) blockIdx.y * 32;
    const char * x = p.x + (int64_t) (t0 + r < ncols ? t0 + r : ncols - 1) * p.x_tok;
    const uint4 T = *(const uint4 *) (q.table + row * 16);
    // the sums this thread finishes at the end are (token, row) = (e / 32, e % 32) for e = thread, thread + block size:
    // one row (the block size is a multiple of 32), whose escape range is requested now
    const int64_t my_row = g0 + (threadIdx.x & 31);
    const int64_t my_gr = p.row0 + (my_row < p.nrows ? my_row : p.nrows - 1);
    const uint32_t esc0 = q.esc_off[my_gr], esc1 = q.esc_off[my_gr + 1];
    uint4 sm0[TURNS][4], sm1[TURNS][4], cdv[TURNS][4], b[TURNS][4][4];
#pragma unroll
    for (int turn = 0; turn < TURNS; turn++) {
        // a last wavefront with a half chunk too few (K / 256 odd) repeats its first
        const int hc = (wave * TURNS + turn) * 256 < K ? wave * TURNS + turn : wave * TURNS;
        const int c = hc >> 1, s0 = 16 * (hc & 1) + 2 * h; // this lane's first slot
        const uint8_t * pl = q.plane + row * K + c * CHUNK + 16 * s0;
        const uint8_t * cd = q.codes + row * (K / 2) + c * (CHUNK / 2) + 8 * s0;
        const char * xb = x + 2 * (c * CHUNK + 4 * s0);
#pragma unroll
        for (int n = 0; n < 4; n++) {
            sm0[turn][n] = *(const uint4 *) (pl + 64 * n);
            sm1[turn][n] = *(const uint4 *) (pl + 64 * n + 16);
            cdv[turn][n] = *(const uint4 *) (cd + 32 * n);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                b[turn][n][j] = *(const uint4 *) (xb + 32 * n + 256 * j);
            }
        }
    }
    nm_f32x16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        acc[i] = 0.f;
    }
#pragma unroll
    for (int turn = 0; turn < TURNS; turn++) {
        if ((wave * TURNS + turn) * 256 < K) {
#pragma unroll
            for (int n = 0; n < 4; n++) {
                uint32_t w0[8], w1[8];
                nib_chunk(sm0[turn][n], make_uint2(cdv[turn][n].x, cdv[turn][n].y), T, w0);
                nib_chunk(sm1[turn][n], make_uint2(cdv[turn][n].z, cdv[turn][n].w), T, w1);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const nm_u32x4_t a = {w0[2 * j], w0[2 * j + 1], w1[2 * j], w1[2 * j + 1]};
                    const nm_u32x4_t bv = {b[turn][n][j].x, b[turn][n][j].y, b[turn][n][j].z, b[turn][n][j].w};
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(nm_bf16x8_t, a), __builtin_bit_cast(nm_bf16x8_t, bv), acc, 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) {
        nm_part[nm_part_at(wave, i, lane)] = acc[i];
    }
    __syncthreads();
    // accumulator register i of lane l: row 8 (i / 4) + 4 (l / 32) + i % 4 of the group, token l % 32.  A thread per
    // (token, row), rows adjacent in a wavefront: a token's 32 outputs are stored side by side.
    for (int e = (int) threadIdx.x; e < 1024; e += (int) blockDim.x) {
        const int tok = e >> 5, rr = e & 31;
        const int i = 4 * (rr >> 3) + (rr & 3), l = tok + 32 * ((rr >> 2) & 1);
        if (g0 + rr < p.nrows && t0 + tok < ncols) {
            float v = 0.f;
            for (int k = 0; k < n_waves; k++) {
                v += nm_part[nm_part_at(k, i, l)];
            }
            const char * xt = p.x + (int64_t) (t0 + tok) * p.x_tok;
            for (uint32_t k = esc0; k < esc1; k++) {
                const uint32_t rec = q.esc[k];
                v = fmaf(bf16_bits_to_f32(esc_bits(rec)), x_at<bf16_t>(xt, (int) (rec & 0xFFFu)), v);
            }
            store_y(p.y + (int64_t) (t0 + tok) * p.y_tok, p.y_bf16, g0 + rr, v);
        }
    }
}

// The same product for at most 16 token columns per block on 16-row groups (v_mfma_f32_16x16x32_bf16): twice the blocks
// of k_nib_mm, which matters while its groups of 32 rows leave CUs idle (2048 rows: 64 blocks on 256 CUs).  Lane
// (row r of 16, k part q of 4) decodes two adjacent slots of its row per step, 8 n + 2 q and the next: eight adjacent
// columns 128 j + 32 n + 8 q + [0, 8) in each of the chunk's four column blocks j, the A operands of four matrix
// instructions (k positions 8 q + [0, 8) of instruction j); lane (token t of 16, q) supplies the same columns of its
// token as B operands.  A wavefront takes STEPS consecutive steps of a row (a chunk is four steps); the partial sums of
// the wavefronts are added in K order through LDS (rows of 68 words: the 64 threads that add for four tokens meet every
// bank twice), the products of escaped weights last.
typedef float nm_f32x4_t __attribute__((ext_vector_type(4)));
constexpr int NM16_PSTRIDE = 68;
template <int STEPS>
__global__ void __launch_bounds__(NM_WAVES * 64) k_nib_mm16(const bf16n_weight w, const cols p, const int ncols) {
    extern __shared__ __align__(16) float nm_part[]; // [wavefront][accumulator register][lane]
    const nib_ptrs q = nibp(w, 0);
    const int K = (int) w.K;
    const int lane = threadIdx.x & 63, r = lane & 15, kq = lane >> 4, wave = (int) (threadIdx.x >> 6), n_waves = (int) (blockDim.x >> 6);
    const int64_t g0 = (int64_t) blockIdx.x * 16;
    const int64_t row = p.row0 + (g0 + r < p.nrows ? g0 + r : p.nrows - 1);
    const int t0 = (int) blockIdx.y * 16;
    const char * x = p.x + (int64_t) (t0 + r < ncols ? t0 + r : ncols - 1) * p.x_tok;
    const uint4 T = *(const uint4 *) (q.table + row * 16);
    // the sums this thread finishes at the end are (token, row) = (e / 16, e % 16) for e = thread, thread + block size
    const int64_t my_row = g0 + (threadIdx.x & 15);
    const int64_t my_gr = p.row0 + (my_row < p.nrows ? my_row : p.nrows - 1);
    const uint32_t esc0 = q.esc_off[my_gr], esc1 = q.esc_off[my_gr + 1];
    const int first = wave * STEPS, c = first >> 2, s0 = 8 * (first & 3) + 2 * kq; // this lane's first slot
    const uint8_t * pl = q.plane + row * K + c * CHUNK + 16 * s0;
    const uint8_t * cd = q.codes + row * (K / 2) + c * (CHUNK / 2) + 8 * s0;
    const char * xb = x + 2 * (c * CHUNK + 4 * s0);
    uint4 sm0[STEPS], sm1[STEPS], cdv[STEPS], b[STEPS][4];
#pragma unroll
    for (int n = 0; n < STEPS; n++) {
        sm0[n] = *(const uint4 *) (pl + 128 * n);
        sm1[n] = *(const uint4 *) (pl + 128 * n + 16);
        cdv[n] = *(const uint4 *) (cd + 64 * n);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            b[n][j] = *(const uint4 *) (xb + 64 * n + 256 * j);
        }
    }
    nm_f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < STEPS; n++) {
        uint32_t w0[8], w1[8];
        nib_chunk(sm0[n], make_uint2(cdv[n].x, cdv[n].y), T, w0);
        nib_chunk(sm1[n], make_uint2(cdv[n].z, cdv[n].w), T, w1);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const nm_u32x4_t a = {w0[2 * j], w0[2 * j + 1], w1[2 * j], w1[2 * j + 1]};
            const nm_u32x4_t bv = {b[n][j].x, b[n][j].y, b[n][j].z, b[n][j].w};
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(nm_bf16x8_t, a), __builtin_bit_cast(nm_bf16x8_t, bv), acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        nm_part[(wave * 4 + i) * NM16_PSTRIDE + lane] = acc[i];
    }
    __syncthreads();
    // accumulator register i of lane l: row 4 (l / 16) + i of the group, token l % 16
    for (int e = (int) threadIdx.x; e < 256; e += (int) blockDim.x) {
        const int tok = e >> 4, rr = e & 15;
        const int i = rr & 3, l = tok + 16 * (rr >> 2);
        if (g0 + rr < p.nrows && t0 + tok < ncols) {
            float v = 0.f;
            for (int k = 0; k < n_waves; k++) {
                v += nm_part[(k * 4 + i) * NM16_PSTRIDE + l];
            }
            const char * xt = p.x + (int64_t) (t0 + tok) * p.x_tok;
            for (uint32_t k = esc0; k < esc1; k++) {
                const uint32_t rec = q.esc[k];
                v = fmaf(bf16_bits_to_f32(esc_bits(rec)), x_at<bf16_t>(xt, (int) (rec & 0xFFFu)), v);
            }
            store_y(p.y + (int64_t) (t0 + tok) * p.y_tok, p.y_bf16, g0 + rr, v);
        }
    }
}

// exact rows of a NIBBLE matrix: FP32 or BF16, to out + i * stride (bytes); row index from ids (gather) or row0 + i
template <bool BF>
__global__ void __launch_bounds__(NT) k_nib_rows(const bf16n_weight w, const char * __restrict__ ids, int64_t ids_s0, int64_t n,
                                                 int64_t row0, char * __restrict__ dst, int64_t dst_s1) {
    const nib_ptrs q = nibp(w, 0);
    const int K = (int) w.K, C = K / CHUNK;
    const int l32 = threadIdx.x & 31, half = threadIdx.x >> 5;
    for (int64_t i = (int64_t) blockIdx.x * HALVES + half; i < n; i += (int64_t) gridDim.x * HALVES) {
        const int64_t gr = row0 + (ids ? (int64_t) * (const int32_t *) (ids + i * ids_s0) : i);
        char * o = dst + i * dst_s1;
        const uint4 T = *(const uint4 *) (q.table + gr * 16);
        const uint32_t e0 = q.esc_off[gr], e1 = q.esc_off[gr + 1];
        for (int c = 0; c < C; c++) {
            const uint4 sm = *((const uint4 *) (q.plane + gr * K + c * CHUNK) + l32);
            const uint2 cd = *((const uint2 *) (q.codes + gr * (K / 2) + c * 256) + l32);
            uint32_t wp[8];
            nib_chunk(sm, cd, T, wp);
            // the row's escapes go into the registers of the lane that holds their column: every element is stored once
            for (uint32_t e = e0; e < e1; e++) {
                const uint32_t rec = q.esc[e];
                const int rel = (int) (rec & 0xFFFu) - c * CHUNK;
                if (rel >= 0 && rel < CHUNK && ((rel & 127) >> 2) == l32) {
                    const int at = (rel >> 7) * 2 + ((rel & 3) >> 1);
                    const uint32_t b = esc_bits(rec);
#pragma unroll
                    for (int i2 = 0; i2 < 8; i2++) {
                        if (i2 == at) {
                            wp[i2] = (rel & 1) ? (wp[i2] & 0xFFFFu) | (b << 16) : (wp[i2] & 0xFFFF0000u) | b;
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int col = c * CHUNK + 128 * j + 4 * l32;
                if (BF) {
                    *(uint2 *) (o + 2 * col) = make_uint2(wp[2 * j], wp[2 * j + 1]);
                } else {
                    *(float4 *) (o + 4 * col) = make_float4(bf16_bits_to_f32(wp[2 * j] & 0xFFFFu), __uint_as_float(wp[2 * j] & 0xFFFF0000u),
                                                            bf16_bits_to_f32(wp[2 * j + 1] & 0xFFFFu), __uint_as_float(wp[2 * j + 1] & 0xFFFF0000u));
                }
            }
        }
    }
}

// blocks of HALVES units (rows) each, capped so that a launch of several columns stays within a few blocks per CU
int grid_for(int64_t work, int ncols, int cus) {
    const int64_t blocks = (work + HALVES - 1) / HALVES;
    const int64_t cap = (int64_t) cus * 8 / (ncols < 1 ? 1 : ncols > 4 ? 4 : ncols);
    return (int) (blocks < 1 ? 1 : blocks > cap ? cap : blocks);
}

} // namespace

// Steps per wavefront of k_nib_mm16 (a row has K / 128): the fewest for which a block has at most eight wavefronts, or
// four (fewer, longer wavefronts) when the row groups outnumber the CUs anyway; 0: K does not fit the kernel.
int nib_mm16_steps(const bf16n_weight & w, int64_t nrows, int cus) {
    if (w.format != FMT_NIBBLE || w.K % CHUNK != 0 || w.K / 128 > 4 * NM_WAVES) {
        return 0;
    }
    const int steps_all = (int) (w.K / 128);
    const int fewest = steps_all <= NM_WAVES ? 1 : steps_all <= 2 * NM_WAVES ? 2 : 4;
    return fewest == 2 && (nrows + 15) / 16 > cus ? 4 : fewest;
}
// Whether a dense batch of BF16 columns takes the 16-row matrix-core kernel (k_nib_mm16): by the CUs its row groups
// fill, from two columns (a group per CU), three (half of them) or five (a quarter) on; smaller matrices stay with the
// GEMV columns, which run side by side on idle CUs (256 x 2048: 3.2-4.6 us at 2-16 columns against 4.7-5.9; 512 x 4096:
// 4.6-9.3 against 7.4-10.0).  Beyond 16 columns every block of 16 tokens decodes the matrix again, which still wins
// while the launch is at most two blocks per CU (2048 x 4096: 10.5-10.7 us at 17-32 columns and 15.7-17.3 at 40-64
// against 16.5-19.9 in 32-row groups; 1024 x 2048: 6.5-6.8 us up to 64 against 10.7-12.8; 5120 x 2048, 640 blocks at
// 17 columns: 12.4 against 11.2, left to the 32-row groups).  The dispatch below and bf16n_gemv_max_tokens share this
// rule.
bool nib_mm16_pays(const bf16n_weight & w, int64_t nrows, int ncols, int cus) {
    const int64_t groups = (nrows + 15) / 16, token_blocks = (ncols + 15) / 16;
    const bool enough = (ncols >= 2 && groups >= cus) || (ncols >= 3 && groups * 2 >= cus) || (ncols >= 5 && groups * 4 >= cus);
    return enough && (token_blocks == 1 || groups * token_blocks <= 2 * (int64_t) cus) && nib_mm16_steps(w, nrows, cus) != 0;
}

// Whether a dense batch of `ncols` BF16 columns over `nrows` rows of a 4-bit-code matrix goes through the matrix cores
// (k_nib_mm): the row groups of 32 must give enough CUs a block, by column count.  The dispatch below and
// bf16n_gemv_max_tokens share this rule.
bool nib_mm_pays(const bf16n_weight & w, int64_t nrows, int ncols, int cus) {
    const int64_t nm_blocks = (nrows + 31) / 32;
    const bool enough = (ncols >= NIB_MM_MIN_COLS && nm_blocks * 2 >= cus) || (ncols > 8 && nm_blocks * 4 >= cus) ||
                        (ncols > 24 && nm_blocks * 8 >= cus);
    return w.format == FMT_NIBBLE && w.K % CHUNK == 0 && w.K / 256 <= 2 * NM_WAVES && enough;
}

void launch_compat_mmv(const bf16n_weight & w, const bf16n_weight * up, int glu, const cols & p, int ncols, bool x_bf16,
                       int cus, hipStream_t stream, bool matrix_cores) {
    const bf16n_weight & wu = up ? *up : w;
    const int64_t work = w.format == FMT_NIBBLE ? p.nrows : p.nrows / w.R;
    const dim3 grid(grid_for(work, ncols, cus), ncols);
    // the matrix cores where the row groups of 32 give enough CUs a block: from five BF16 columns on with blocks for half
    // of the CUs, from nine with a quarter, from 25 with an eighth (5120 x 2048, 160 blocks: 11.0-13.0 us for 5-32
    // columns against 9.6 / 17.9 us for 4 / 8 GEMV columns and 20 us for dequant + GEMM; 2048 x 4096, 64 blocks: 16.7-20.7
    // us against 8.6 / 15.4 us and 24-28 us; 1024 x 2048, 32 blocks: 10.6-12.8 us against 7.8 / 9.5 / 14.9 / 25.5 us in
    // GEMV columns at 9 / 16 / 32 / 64).  Smaller matrices stay with the GEMV columns, which run side by side on idle CUs
    // (256 x 2048: 4.9-9.5 us for 9-64 columns against 10.5-12.6 us here).
    const int64_t nm_blocks = (p.nrows + 31) / 32;
    if (matrix_cores && !p.ids && glu == 0 && x_bf16 && nib_mm16_pays(w, p.nrows, ncols, cus) && ((uintptr_t) p.x & 15) == 0 &&
        p.x_tok % 16 == 0) {
        // 16-row groups (5120 x 2048: 7.7 / 8.2 / 8.8 / 10.5 us at 2 / 4 / 8 / 16 columns against 8.3 / 11.4
        // in GEMV columns and 9.7 / 10.8 in 32-row groups; 2048 x 4096: 8.0 / 8.2 / 9.0 / 10.3 us at 3 / 4 / 8 / 16
        // against 9.4 / 9.3 / 15.3 / 15.5; 1024 x 2048: 5.6 / 6.5 us at 5 / 16 against 6.8 / 9.1; 2048 x 512: 3.3 / 3.6
        // us at 2 / 16 against 3.5 / 5.5)
        const int steps = nib_mm16_steps(w, p.nrows, cus), waves = (int) (w.K / 128) / steps;
        note_kernel("k_nib_mm16", nullptr, 1, steps);
        const dim3 grid((unsigned) ((p.nrows + 15) / 16), (unsigned) ((ncols + 15) / 16));
        const size_t shm = (size_t) waves * 4 * NM16_PSTRIDE * sizeof(float);
        if (steps == 1)      hipLaunchKernelGGL(k_nib_mm16<1>, grid, dim3(waves * 64), shm, stream, w, p, ncols);
        else if (steps == 2) hipLaunchKernelGGL(k_nib_mm16<2>, grid, dim3(waves * 64), shm, stream, w, p, ncols);
        else                 hipLaunchKernelGGL(k_nib_mm16<4>, grid, dim3(waves * 64), shm, stream, w, p, ncols);
        return;
    }
    if (matrix_cores && !p.ids && glu == 0 && x_bf16 && nib_mm_pays(w, p.nrows, ncols, cus) && ((uintptr_t) p.x & 15) == 0 &&
        p.x_tok % 16 == 0) {
        const int halves = (int) (w.K / 256), turns = halves > NM_WAVES ? 2 : 1, waves = (halves + turns - 1) / turns;
        note_kernel("k_nib_mm", nullptr, 1, turns);
        const dim3 grid((unsigned) nm_blocks, (unsigned) ((ncols + 31) / 32));
        const size_t shm = (size_t) waves * 16 * NM_PSTRIDE * sizeof(float);
        if (turns == 2) {
            hipLaunchKernelGGL(k_nib_mm<2>, grid, dim3(waves * 64), shm, stream, w, p, ncols);
        } else {
            hipLaunchKernelGGL(k_nib_mm<1>, grid, dim3(waves * 64), shm, stream, w, p, ncols);
        }
        return;
    }
    if (w.format == FMT_NIBBLE) {
        const int rpb = HALVES / (int) (w.K / CHUNK);
        // dense batches: four (two) columns share one decode of the matrix once there are columns enough to keep at
        // least four groups of blocks (below that the columns run side by side on the idle CUs, which is faster)
        const int64_t blocks1 = (p.nrows + rpb - 1) / rpb;
        const bool fills = blocks1 >= 4 * (int64_t) cus; // one column's blocks keep every CU busy by themselves
        const int nc = p.ids ? 1 : fills ? (ncols >= 3 ? 4 : ncols == 2 ? 2 : 1) : ncols >= 16 ? 4 : ncols >= 8 ? 2 : 1;
        const int ngroups = (ncols + nc - 1) / nc;
        const dim3 grid(grid_for((p.nrows + rpb - 1) / rpb * HALVES, ngroups, cus), ngroups);
        note_kernel("k_nib_mmv", x_bf16 ? "bf16_t" : "float", 2, glu, nc);
#define NIBC(TX, G, N) hipLaunchKernelGGL((k_nib_mmv<TX, G, N>), grid, dim3(NT), 0, stream, w, wu, p, ncols)
#define NIB(TX, G) do { if (nc == 4) NIBC(TX, G, 4); else if (nc == 2) NIBC(TX, G, 2); else NIBC(TX, G, 1); } while (0)
        if (x_bf16) { if (glu == 0) NIB(bf16_t, 0); else if (glu == 1) NIB(bf16_t, 1); else NIB(bf16_t, 2); }
        else        { if (glu == 0) NIB(float, 0);  else if (glu == 1) NIB(float, 1);  else NIB(float, 2); }
#undef NIB
#undef NIBC
        return;
    }
    const bool hp = w.format == FMT_HUFPAIR;
    const size_t shm = (size_t) w.K * 4 + (size_t) (glu ? 2 : 1) * (hp ? (4u << HP_LP) : (4u << HUF_LMAX));
#define HUF(F, TX, G) hipLaunchKernelGGL((k_huf_mmv<F, TX, G>), grid, dim3(NT), shm, stream, w, wu, p)
    if (hp) {
        if (x_bf16) { if (glu) HUF(FMT_HUFPAIR, bf16_t, true); else HUF(FMT_HUFPAIR, bf16_t, false); }
        else        { if (glu) HUF(FMT_HUFPAIR, float, true);  else HUF(FMT_HUFPAIR, float, false); }
    } else {
        if (x_bf16) { if (glu) HUF(FMT_HUFFMAN, bf16_t, true); else HUF(FMT_HUFFMAN, bf16_t, false); }
        else        { if (glu) HUF(FMT_HUFFMAN, float, true);  else HUF(FMT_HUFFMAN, float, false); }
    }
#undef HUF
}

void launch_compat_dequant(const bf16n_weight & w, int64_t row0, int64_t nrows, uint16_t * out, int cus, hipStream_t stream) {
    const int64_t work = w.format == FMT_NIBBLE ? nrows : nrows / w.R;
    const int64_t blocks = (work + HALVES - 1) / HALVES;
    const dim3 grid((unsigned) (blocks < (int64_t) cus * 16 ? blocks : (int64_t) cus * 16));
    if (w.format == FMT_NIBBLE) {
        hipLaunchKernelGGL((k_nib_rows<true>), grid, dim3(NT), 0, stream, w, (const char *) nullptr, (int64_t) 0, nrows, row0,
                           (char *) out, (int64_t) w.K * 2);
    } else if (w.format == FMT_HUFPAIR) {
        hipLaunchKernelGGL((k_huf_dequant<FMT_HUFPAIR>), grid, dim3(NT), 0, stream, w, row0, nrows, out);
    } else {
        hipLaunchKernelGGL((k_huf_dequant<FMT_HUFFMAN>), grid, dim3(NT), 0, stream, w, row0, nrows, out);
    }
}

void launch_compat_get_rows(const bf16n_weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16,
                            int64_t dst_s1, int64_t row0, hipStream_t stream) {
    const dim3 grid((unsigned) ((n + HALVES - 1) / HALVES));
    if (w.format == FMT_NIBBLE) {
        if (dst_bf16) hipLaunchKernelGGL((k_nib_rows<true>), grid, dim3(NT), 0, stream, w, (const char *) ids, ids_s0, n, row0, (char *) dst, dst_s1);
        else          hipLaunchKernelGGL((k_nib_rows<false>), grid, dim3(NT), 0, stream, w, (const char *) ids, ids_s0, n, row0, (char *) dst, dst_s1);
    } else {
        if (dst_bf16) hipLaunchKernelGGL((k_hp_get_rows<true>), grid, dim3(NT), 0, stream, w, (const char *) ids, ids_s0, n, row0, (char *) dst, dst_s1);
        else          hipLaunchKernelGGL((k_hp_get_rows<false>), grid, dim3(NT), 0, stream, w, (const char *) ids, ids_s0, n, row0, (char *) dst, dst_s1);
    }
}

} // namespace dev
} // namespace bf16n
