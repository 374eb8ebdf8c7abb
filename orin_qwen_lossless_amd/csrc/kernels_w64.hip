// Kernels for the wave64 HUFPAIR layout (FLAG_WAVE64): fused decode + GEMV, exact dequant, row gather.
//
// One 64-lane wavefront decodes one unit at a time and owns a contiguous range of units, so everything it reads is
// sequential in memory:
//   * the sign|mantissa plane: 1024 contiguous bytes per step, one 16-byte load per lane (lanes 0..31 the even,
//     lanes 32..63 the odd 512-column chunk of the step);
//   * the unit streams: one word stream per unit, consumed front to back.  The wave copies it in 1 KiB blocks into a
//     private ring in LDS (coalesced 16-byte loads, one block in flight in registers) and every lane that needs a new
//     word after a pair of codes reads ring[consumed + rank among the refilling lanes] — consecutive addresses, no bank
//     conflicts, no per-lane pointers.  A lane buffers three words, so a requested word is not needed before the next
//     check and its LDS read overlaps the table lookups in between;
//   * the 4096-entry pair table sits in LDS once per block; an entry already holds both exponents in BF16 position, so
//     one v_perm + one v_bfi turn two plane bytes and an entry into two BF16 weights.
// Activations stay in registers for the whole kernel (a lane always meets the same columns), products are accumulated in
// FP32 (v_dot2_f32_bf16 for BF16 activations, v_fma_f32 for FP32 ones) and reduced across the wave once per row.
#include "dev_common.h"
#include "dev_w64.h"
#include "launchers.h"

namespace bf16n {
namespace dev {

namespace {

// ---------------------------------------------------------------- activations in registers

// the 16 activations one lane meets in one 512-column chunk, as the GEMV consumes them
template <typename TX> struct xchunk;
template <> struct xchunk<bf16_t> { // 8 BF16 pairs
    uint32_t v[8];
    __device__ __forceinline__ void load(const char * x, int col0) { // col0 = chunk * 512 + 4 * (lane % 32)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint2 t = *(const uint2 *) (x + 2 * (col0 + 128 * j));
            v[2 * j] = t.x;
            v[2 * j + 1] = t.y;
        }
    }
    __device__ __forceinline__ float dot(const uint32_t (&wp)[8], float acc) const {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            acc = dot2_bf16(wp[q], v[q], acc);
        }
        return acc;
    }
};
template <> struct xchunk<float> {
    float v[16];
    __device__ __forceinline__ void load(const char * x, int col0) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float4 t = *(const float4 *) (x + 4 * (col0 + 128 * j));
            v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
        }
    }
    __device__ __forceinline__ float dot(const uint32_t (&wp)[8], float acc) const {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            acc = fmaf(__uint_as_float(wp[q] << 16), v[2 * q], acc);
            acc = fmaf(__uint_as_float(wp[q] & 0xFFFF0000u), v[2 * q + 1], acc);
        }
        return acc;
    }
};

// ---------------------------------------------------------------- GEMV
//
// C = K / 512 in {1, 2, 4, 8}.  The loop body covers NB steps (2, or 4 for C = 8) so that the plane registers of a step
// are reloaded for the same step of the next body as soon as they are consumed.  A body is 4 rows (C = 1: a step
// holds two rows, one per half-wave), 2 rows (C = 2) or 1 row (C = 4, 8); a unit must hold whole bodies.
template <int C> struct geom {
    static constexpr int NB = C == 8 ? 4 : 2;           // steps per body
    static constexpr int XS = C >= 2 ? C / 2 : 1;       // activation chunk sets per lane
    static constexpr int ROWS = C == 1 ? 4 : C == 2 ? 2 : 1; // rows per body
};

// One decode chain of a wave: a contiguous range of units with its own stream ring, plane pointer and row counter.
// HINT: as in w64_dec_t, for the plane bytes and the stream blocks alike.
template <int NB, int HINT = -1>
struct chain {
    w64_dec_t<HINT> dec;
    range_t plane;         // the plane bytes of the chain's units
    uint32_t off;          // byte offset of this lane's 16 bytes in the next step to load
    uint4 sm[NB];          // plane bytes of the body's steps
    int64_t row;           // output row of the next body, relative to the product
    bool once;             // the launch reads the plane bytes once (see load_once)
    __device__ __forceinline__ uint4 load_step(int) const { // past the end of the chain: dropped, reads as zeros
        if constexpr (HINT < 0) {
            return range_load16(plane, off, once);
        } else {
            return range_load16<HINT == 1>(plane, off);
        }
    }
    // first / end: the stream words of units [gu0, gu0 + n_units) (unit bases, read by the caller ahead of time)
    __device__ __forceinline__ void start(uint32_t * ring, const w64_ptrs & q, int64_t gu0, int64_t n_units, int64_t row0, int R, int K,
                                          int lane, uint32_t first, uint32_t end, bool once_ = false, bool stream_once = false) {
        once = once_;
        plane = make_range(q.plane + uniform64(gu0 * R * K), uniform((uint32_t) (n_units * R * K)));
        off = 16 * (uint32_t) lane;
        row = row0;
#pragma unroll
        for (int s = 0; s < NB; s++) {
            sm[s] = load_step(lane);
            off += 1024;
        }
        dec.start(ring, q.stream, uniform(first), uniform(end), lane, stream_once);
    }
    // plane bytes of step s of the next body, once step s of this body is consumed
    __device__ __forceinline__ void reload(int s, int lane) {
        sm[s] = load_step(lane);
        off += 1024;
    }
};

// N chains advance one unit each, instruction streams interleaved: while one chain waits for a table lookup the
// other one issues.
// GLU (N = 2, NC = 1): chain 0 decodes a unit of the gate matrix, chain 1 the same unit of the up matrix (its table
// LUT_WORDS behind the first), and the rows come out as silu(gate x) * (up x).
template <typename TX, int C, int NC, int N, bool GLU = false, int HINT = -1>
__device__ __forceinline__ void unit_pass(chain<geom<C>::NB, HINT> (&ch)[2], const uint32_t * lut, const xchunk<TX> (&xr)[NC][geom<C>::XS],
                                          const cols & p, const col_view & cv, int R, int lane) {
    using G = geom<C>;
    const int l32 = lane & 31, half = lane >> 5;
#pragma unroll
    for (int k = 0; k < N; k++) {
        ch[k].dec.keep_ahead(); // 256 words ahead cover the 192 of a unit start ...
        ch[k].dec.begin_unit();
        ch[k].dec.keep_ahead(); // ... and then the first step again
    }
    const int bodies = R * C / 2 / G::NB;
    for (int b = 0; b < bodies; b++) {
        // Issue priority by progress: of the wavefronts that share a SIMD, the ones behind go first.  Without it the
        // oldest wavefront wins every tie, runs ahead and ends early, and the launch ends with few wavefronts per SIMD
        // (on the 248320 x 2048 matrix the wavefronts of a compute unit ended between 95 and 127 us); with it they
        // stay within four bodies of each other and end together (115 to 120 us).
        switch (b & 3) { // the instruction takes its level as an immediate
            case 0: __builtin_amdgcn_s_setprio(3); break;
            case 1: __builtin_amdgcn_s_setprio(2); break;
            case 2: __builtin_amdgcn_s_setprio(1); break;
            default: __builtin_amdgcn_s_setprio(0); break;
        }
        float acc[N][NC][G::NB];
#pragma unroll
        for (int s = 0; s < G::NB; s++) {
            uint32_t wp[N][8];
            uint32_t smw[N][4];
#pragma unroll
            for (int k = 0; k < N; k++) {
                smw[k][0] = ch[k].sm[s].x; smw[k][1] = ch[k].sm[s].y; smw[k][2] = ch[k].sm[s].z; smw[k][3] = ch[k].sm[s].w;
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
#pragma unroll
                for (int k = 0; k < N; k++) {
                    uint32_t e0, e1;
                    ch[k].dec.two(GLU ? lut + k * LUT_WORDS : lut, e0, e1);
                    wp[k][2 * j] = merge(spread_lo(smw[k][j]), e0);
                    wp[k][2 * j + 1] = merge(spread_hi(smw[k][j]), e1);
                }
            }
            // all memory traffic of the step in one place, after the decode: the loads waited for here (a stream block
            // about to enter the ring) were issued a whole step ago, and the new ones have a whole step to arrive
#pragma unroll
            for (int k = 0; k < N; k++) {
                ch[k].dec.keep_ahead();
            }
#pragma unroll
            for (int k = 0; k < N; k++) {
                ch[k].reload(s, lane);
#pragma unroll
                for (int n = 0; n < NC; n++) {
                    if (C >= 4) {
                        acc[k][n][0] = xr[n][s].dot(wp[k], s == 0 ? 0.f : acc[k][n][0]);
                    } else {
                        acc[k][n][s] = xr[n][0].dot(wp[k], 0.f);
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < (GLU ? 1 : N); k++) {
            const int64_t row = ch[k].row;
#pragma unroll
            for (int n = 0; n < NC; n++) {
                char * y = cv.y + n * p.y_tok;
                if (GLU) {
                    if (C >= 4) {
                        const float g = wave_sum_dpp(acc[0][n][0]), u = wave_sum_dpp(acc[N - 1][n][0]);
                        if (lane == 63) {
                            store_y(y, p.y_bf16, row, u * silu(g));
                        }
                    } else {
#pragma unroll
                        for (int s = 0; s < 2; s++) {
                            const float g = C == 2 ? wave_sum_dpp(acc[0][n][s]) : half_wave_sum_dpp(acc[0][n][s]);
                            const float u = C == 2 ? wave_sum_dpp(acc[N - 1][n][s]) : half_wave_sum_dpp(acc[N - 1][n][s]);
                            if (C == 2 ? lane == 63 : l32 == 31) {
                                store_y(y, p.y_bf16, C == 2 ? row + s : row + 2 * s + half, u * silu(g));
                            }
                        }
                    }
                } else if (C >= 4) { // a body is one row
                    const float v = wave_sum_dpp(acc[k][n][0]);
                    if (lane == 63) {
                        store_y(y, p.y_bf16, row, v);
                    }
                } else if (C == 2) { // a step is one row
#pragma unroll
                    for (int s = 0; s < 2; s++) {
                        const float v = wave_sum_dpp(acc[k][n][s]);
                        if (lane == 63) {
                            store_y(y, p.y_bf16, row + s, v);
                        }
                    }
                } else { // a step is rows 2s (lanes 0..31) and 2s + 1 (lanes 32..63)
#pragma unroll
                    for (int s = 0; s < 2; s++) {
                        const float v = half_wave_sum_dpp(acc[k][n][s]);
                        if (l32 == 31) {
                            store_y(y, p.y_bf16, row + 2 * s + half, v);
                        }
                    }
                }
            }
            ch[k].row += G::ROWS;
        }
    }
}

// NCH = 2: a wave splits its units into two halves decoded as two interleaved chains (twice the independent work per
// wave to cover LDS latency); NCH = 1 where a wave has a single unit.
// activation registers per lane of an instance (BF16: 8 per 512-column chunk set and column, FP32: 16)
template <typename TX, int C, int NC>
constexpr int x_regs() { return NC * geom<C>::XS * (sizeof(TX) == 2 ? 8 : 16); }

// instances that need more than 128 registers per lane: more than 64 of activations, or 64 with FP32 activations or
// eight chunks per row (they spilled at 128); these run in blocks of at most eight wavefronts
constexpr bool wide_regs(int xr, bool x_bf16, int C) { return xr > 64 || (xr == 64 && (!x_bf16 || C == 8)); }

template <typename TX, int C, int NC, int NCH, int HINT = -1>
__global__ void __launch_bounds__(wide_regs(x_regs<TX, C, NC>(), sizeof(TX) == 2, C) ? 512 : 1024) k_w64_mmv(const bf16n_weight w, const cols p, int units_per_wave) {
    using G = geom<C>;
    constexpr int K = C * CHUNK;
    __shared__ __align__(16) uint32_t lut[LUT_WORDS];          // static: sits at LDS address 0
    extern __shared__ __align__(16) uint32_t rings[];          // per wave and chain: RING + RING_PAD words
    const w64_ptrs q = w64p(w);
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int R = w.R;
    const col_view cv = col_setup(p, blockIdx.y * NC);
    const int64_t units = p.nrows / R;
    const int64_t u_begin = ((int64_t) blockIdx.x * nwaves + wave) * units_per_wave;
    const bool live = u_begin < units;
    const int64_t u_end = u_begin + units_per_wave < units ? u_begin + units_per_wave : units;
    const int64_t n = live ? u_end - u_begin : 0, nA = NCH == 2 ? (n + 1) / 2 : n, nB = n - nA;
    const int64_t gu0 = cv.rbase / R + (live ? u_begin : 0);
    // the unit bases first: the dependent stream loads can then start as soon as the table is staged
    const uint32_t b0 = q.ubase[gu0], b1 = q.ubase[gu0 + nA], b2 = q.ubase[gu0 + n];
    stage_lut(lut, q.lut);
    // activations: chunk 2i + half of the row for i < XS (C = 1: chunk 0 for both halves)
    xchunk<TX> xr[NC][G::XS];
#pragma unroll
    for (int n_ = 0; n_ < NC; n_++) {
#pragma unroll
        for (int i = 0; i < G::XS; i++) {
            xr[n_][i].load(cv.x + n_ * p.x_tok, (C == 1 ? 0 : (2 * i + half) * CHUNK) + 4 * l32);
        }
    }
    __syncthreads();
    if (!live) {
        return;
    }
    chain<G::NB, HINT> ch[2];
    uint32_t * ring = rings + wave * (NCH * WAVE_LDS_WORDS);
    ch[0].start(ring, q, gu0, nA, u_begin * R, R, K, lane, b0, b1, p.plane_once, p.stream_once);
    if (NCH == 2 && nB > 0) {
        ch[1].start(ring + WAVE_LDS_WORDS, q, gu0 + nA, nB, (u_begin + nA) * R, R, K, lane, b1, b2, p.plane_once, p.stream_once);
    }
    for (int64_t i = 0; i < nA; i++) {
        if (NCH == 2 && i < nB) {
            unit_pass<TX, C, NC, 2, false, HINT>(ch, lut, xr, p, cv, R, lane);
        } else {
            unit_pass<TX, C, NC, 1, false, HINT>(ch, lut, xr, p, cv, R, lane);
        }
    }
}

// Fused gate / up + SwiGLU for two matrices of the same shape and unit size: every wave decodes its units of both
// matrices side by side (the two chains) and writes silu(gate x) * (up x).
template <typename TX, int C>
__global__ void __launch_bounds__(1024) k_w64_glu(const bf16n_weight wg, const bf16n_weight wu, const cols p, int units_per_wave) {
    using G = geom<C>;
    constexpr int K = C * CHUNK;
    __shared__ __align__(16) uint32_t lut[2 * LUT_WORDS];
    extern __shared__ __align__(16) uint32_t rings[];
    const w64_ptrs qg = w64p(wg), qu = w64p(wu);
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int R = wg.R;
    const col_view cv = col_setup(p, blockIdx.y);
    const int64_t units = p.nrows / R;
    const int64_t u_begin = ((int64_t) blockIdx.x * nwaves + wave) * units_per_wave;
    const bool live = u_begin < units;
    const int64_t u_end = u_begin + units_per_wave < units ? u_begin + units_per_wave : units;
    const int64_t n = live ? u_end - u_begin : 0;
    const int64_t gu0 = cv.rbase / R + (live ? u_begin : 0);
    const uint32_t g0 = qg.ubase[gu0], g1 = qg.ubase[gu0 + n], u0 = qu.ubase[gu0], u1 = qu.ubase[gu0 + n];
    stage_lut(lut, qg.lut);
    stage_lut(lut + LUT_WORDS, qu.lut);
    xchunk<TX> xr[1][G::XS];
#pragma unroll
    for (int i = 0; i < G::XS; i++) {
        xr[0][i].load(cv.x, (C == 1 ? 0 : (2 * i + half) * CHUNK) + 4 * l32);
    }
    __syncthreads();
    if (!live) {
        return;
    }
    chain<G::NB> ch[2];
    uint32_t * ring = rings + wave * (2 * WAVE_LDS_WORDS);
    ch[0].start(ring, qg, gu0, n, u_begin * R, R, K, lane, g0, g1, p.plane_once, p.stream_once);
    ch[1].start(ring + WAVE_LDS_WORDS, qu, gu0, n, u_begin * R, R, K, lane, u0, u1, p.plane_once, p.stream_once);
    for (int64_t i = 0; i < n; i++) {
        unit_pass<TX, C, 1, 2, true>(ch, lut, xr, p, cv, R, lane);
    }
}

// ---------------------------------------------------------------- dequant / row gather

// exact BF16 bits of rows [row0, row0 + nrows) (whole units) into out (row-major); one wave per range of units.
// only_row >= 0: store just that row (relative to row0) — the row gather decodes its unit from the start.
__device__ __forceinline__ void w64_unit_rows(w64_dec & dec, const uint32_t * lut, const uint8_t * unit_plane, int R, int C,
                                              int lane, int64_t only_row, char * out, int64_t out_row_bytes, bool f32) {
    const int l32 = lane & 31, half = lane >> 5;
    const uint4 * pp = (const uint4 *) unit_plane + lane;
    for (int st = 0; st < R * C / 2; st++) {
        dec.keep_ahead();
        uint32_t wp[8];
        dec.step(lut, pp[64 * st], wp);
        const int o = 2 * st + half, rr = o / C, c = o % C;
        if (only_row >= 0 && (2 * st) / C > only_row) { // same decision in both half-waves
            break;
        }
        if (only_row >= 0 && rr != only_row) {
            continue;
        }
        char * dst = out + (only_row >= 0 ? 0 : rr) * out_row_bytes;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int col = c * CHUNK + 128 * j + 4 * l32;
            if (f32) {
                *(float4 *) (dst + 4 * col) = make_float4(__uint_as_float(wp[2 * j] << 16), __uint_as_float(wp[2 * j] & 0xFFFF0000u),
                                                          __uint_as_float(wp[2 * j + 1] << 16), __uint_as_float(wp[2 * j + 1] & 0xFFFF0000u));
            } else {
                *(uint2 *) (dst + 2 * col) = make_uint2(wp[2 * j], wp[2 * j + 1]);
            }
        }
    }
}

__global__ void __launch_bounds__(256) k_w64_dequant(const bf16n_weight w, int64_t row0, int64_t nrows, uint16_t * __restrict__ out,
                                                     int units_per_wave) {
    __shared__ __align__(16) uint32_t lut[LUT_WORDS];
    extern __shared__ __align__(16) uint32_t rings[];
    const w64_ptrs q = w64p(w);
    stage_lut(lut, q.lut);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int R = w.R, K = (int) w.K, C = K / CHUNK;
    const int64_t units = nrows / R;
    const int64_t u_begin = ((int64_t) blockIdx.x * nwaves + wave) * units_per_wave;
    if (u_begin >= units) {
        return;
    }
    const int64_t u_end = u_begin + units_per_wave < units ? u_begin + units_per_wave : units;
    const int64_t gu0 = row0 / R + u_begin;
    w64_dec dec;
    dec.start(rings + wave * WAVE_LDS_WORDS, q.stream, q.ubase[gu0], q.ubase[gu0 + (u_end - u_begin)], lane);
    for (int64_t u = u_begin; u < u_end; u++) {
        dec.keep_ahead();
        dec.begin_unit();
        w64_unit_rows(dec, lut, q.plane + (row0 / R + u) * R * (int64_t) K, R, C, lane, -1, (char *) (out + u * R * (int64_t) K),
                      (int64_t) K * 2, false);
    }
}

__global__ void __launch_bounds__(256) k_w64_get_rows(const bf16n_weight w, const char * __restrict__ ids, int64_t ids_s0, int64_t n,
                                                      int64_t row0, char * __restrict__ dst, int64_t dst_s1, bool f32) {
    __shared__ __align__(16) uint32_t lut[LUT_WORDS];
    extern __shared__ __align__(16) uint32_t rings[];
    const w64_ptrs q = w64p(w);
    stage_lut(lut, q.lut);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int R = w.R, K = (int) w.K, C = K / CHUNK;
    const int64_t i = (int64_t) blockIdx.x * nwaves + wave;
    if (i >= n) {
        return;
    }
    const int64_t gr = row0 + *(const int32_t *) (ids + i * ids_s0);
    const int64_t gu = gr / R;
    w64_dec dec;
    dec.start(rings + wave * WAVE_LDS_WORDS, q.stream, q.ubase[gu], q.ubase[gu + 1], lane);
    dec.keep_ahead();
    dec.begin_unit();
    w64_unit_rows(dec, lut, q.plane + gu * R * (int64_t) K, R, C, lane, gr - gu * R, dst + i * dst_s1, 0, f32);
}

size_t w64_shm(int waves) { return (size_t) waves * WAVE_LDS_WORDS * 4; } // dynamic part; the table is static

// waves per block and units per wave for `units` units per column: every wave gets the same number of units (but the
// last), and a launch fills the device once when it can
void w64_dims(int64_t units, int ncols, int cus, int & waves_per_block, int & blocks, int & units_per_wave, int waves_per_cu = 16) {
    int64_t max_waves = (int64_t) cus * waves_per_cu / (ncols < 1 ? 1 : ncols);
    max_waves = max_waves < 16 ? 16 : max_waves;
    int64_t upw = (units + max_waves - 1) / max_waves;
    if (upw > 1 && (upw & 1)) {
        upw++; // two chains per wave: an even split
    }
    const int64_t waves = (units + upw - 1) / upw;
    waves_per_block = waves >= 8 * (int64_t) cus && waves_per_cu != 12 ? 8 : 4;
    if (waves < waves_per_block) {
        waves_per_block = (int) waves;
    }
    blocks = (int) ((waves + waves_per_block - 1) / waves_per_block);
    units_per_wave = (int) upw;
}

// columns that share one decode (reference launch.cu:174-193 groups four; its eight-column kernels are
// kernels.cuh:2002-2104).  Up to 64 activation registers per lane an instance runs sixteen wavefronts per CU; up to 128
// (five to eight BF16 columns at K <= 2048, three or four at K = 4096, ...) eight to twelve wavefronts of up to 256
// registers: a lower decode rate, but one pass over the matrix instead of two.
template <typename TX, int C>
constexpr int max_group() {
    constexpr int per_col = x_regs<TX, C, 1>();
    return 128 / per_col < 1 ? 1 : 128 / per_col > 8 ? 8 : 128 / per_col;
}
// two decode chains per wave only where the activations leave room for them in 128 registers (the instances with
// more activation registers would spill; they run one chain per wave)
template <typename TX, int C, int NC>
constexpr bool two_chains() { return x_regs<TX, C, NC>() <= 16; }

// the load policy of plane and stream as a compile-time choice of the instance
template <typename TX, int C, int NC, int HINT>
void mmv_launch_hint(dim3 grid, int nt, int wpb, hipStream_t stream, const bf16n_weight & w, const cols & p, int upw) {
    if constexpr (two_chains<TX, C, NC>()) {
        if (upw >= 2) {
            note_kernel("k_w64_mmv", tx_name<TX>(), 4, C, NC, 2, HINT);
            hipLaunchKernelGGL((k_w64_mmv<TX, C, NC, 2, HINT>), grid, dim3(nt), w64_shm(2 * wpb), stream, w, p, upw);
            return;
        }
    }
    note_kernel("k_w64_mmv", tx_name<TX>(), 4, C, NC, 1, HINT);
    hipLaunchKernelGGL((k_w64_mmv<TX, C, NC, 1, HINT>), grid, dim3(nt), w64_shm(wpb), stream, w, p, upw);
}
template <typename TX, int C, int NC>
void mmv_launch(dim3 grid, int nt, int wpb, hipStream_t stream, const bf16n_weight & w, const cols & p, int upw) {
    if (p.plane_once == p.stream_once) { // (what launch_w64_mmv sets; the run-time form stays for other callers)
        if (p.plane_once) {
            mmv_launch_hint<TX, C, NC, 1>(grid, nt, wpb, stream, w, p, upw);
        } else {
            mmv_launch_hint<TX, C, NC, 0>(grid, nt, wpb, stream, w, p, upw);
        }
        return;
    }
    mmv_launch_hint<TX, C, NC, -1>(grid, nt, wpb, stream, w, p, upw);
}

template <typename TX, int C>
void mmv_nc(int nc, dim3 grid, int nt, int wpb, hipStream_t stream, const bf16n_weight & w, const cols & p, int upw) {
    constexpr int G = max_group<TX, C>();
    if (nc == 1) {
        mmv_launch<TX, C, 1>(grid, nt, wpb, stream, w, p, upw);
    } else if (nc == 2) {
        if constexpr (G >= 2) mmv_launch<TX, C, 2>(grid, nt, wpb, stream, w, p, upw);
    } else if (nc == 3) {
        if constexpr (G >= 3) mmv_launch<TX, C, 3>(grid, nt, wpb, stream, w, p, upw);
    } else if (nc == 4) {
        if constexpr (G >= 4) mmv_launch<TX, C, 4>(grid, nt, wpb, stream, w, p, upw);
    } else if (nc == 5) {
        if constexpr (G >= 8) mmv_launch<TX, C, 5>(grid, nt, wpb, stream, w, p, upw);
    } else if (nc == 6) {
        if constexpr (G >= 8) mmv_launch<TX, C, 6>(grid, nt, wpb, stream, w, p, upw);
    } else if (nc == 7) {
        if constexpr (G >= 8) mmv_launch<TX, C, 7>(grid, nt, wpb, stream, w, p, upw);
    } else {
        if constexpr (G >= 8) mmv_launch<TX, C, 8>(grid, nt, wpb, stream, w, p, upw);
    }
}

template <typename TX>
void mmv_c(int C, int nc, dim3 grid, int nt, int wpb, hipStream_t stream, const bf16n_weight & w, const cols & p, int upw) {
    switch (C) {
        case 1: mmv_nc<TX, 1>(nc, grid, nt, wpb, stream, w, p, upw); break;
        case 2: mmv_nc<TX, 2>(nc, grid, nt, wpb, stream, w, p, upw); break;
        case 4: mmv_nc<TX, 4>(nc, grid, nt, wpb, stream, w, p, upw); break;
        default: mmv_nc<TX, 8>(nc, grid, nt, wpb, stream, w, p, upw); break;
    }
}

template <typename TX>
int group_for(int C) {
    return C == 1 ? max_group<TX, 1>() : C == 2 ? max_group<TX, 2>() : C == 4 ? max_group<TX, 4>() : max_group<TX, 8>();
}

template <typename TX, int C, int NC>
void set_attr() {
    if constexpr (NC <= max_group<TX, C>()) {
        (void) hipFuncSetAttribute((const void *) k_w64_mmv<TX, C, NC, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) w64_shm(16));
        if constexpr (two_chains<TX, C, NC>()) {
            (void) hipFuncSetAttribute((const void *) k_w64_mmv<TX, C, NC, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) w64_shm(32));
        }
    }
}
template <typename TX, int C>
void set_attr_nc() {
    set_attr<TX, C, 1>(); set_attr<TX, C, 2>(); set_attr<TX, C, 3>(); set_attr<TX, C, 4>();
    set_attr<TX, C, 5>(); set_attr<TX, C, 6>(); set_attr<TX, C, 7>(); set_attr<TX, C, 8>();
}
template <typename TX>
void set_attr_c() { set_attr_nc<TX, 1>(); set_attr_nc<TX, 2>(); set_attr_nc<TX, 4>(); set_attr_nc<TX, 8>(); }

} // namespace

template <typename TX>
void set_attr_glu() {
    (void) hipFuncSetAttribute((const void *) k_w64_glu<TX, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) w64_shm(32));
    (void) hipFuncSetAttribute((const void *) k_w64_glu<TX, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) w64_shm(32));
    (void) hipFuncSetAttribute((const void *) k_w64_glu<TX, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) w64_shm(32));
    (void) hipFuncSetAttribute((const void *) k_w64_glu<TX, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) w64_shm(32));
}

void w64_init() {
    set_attr_c<bf16_t>();
    set_attr_c<float>();
    set_attr_glu<bf16_t>();
    set_attr_glu<float>();
}

// shapes with a fused wave64 GEMV: K in {512, 1024, 2048, 4096} and units that hold whole loop bodies
bool w64_mmv_supported(const bf16n_weight & w, bool) {
    const int64_t C = w.K / CHUNK;
    if (C != 1 && C != 2 && C != 4 && C != 8) {
        return false;
    }
    const int nb = C == 8 ? 4 : 2;
    return (w.R * C / 2) % nb == 0;
}

void launch_w64_mmv(const bf16n_weight & w, const cols & p, int ncols, bool x_bf16, bool multi_col, int cus, hipStream_t stream) {
    const int C = (int) (w.K / CHUNK);
    const int64_t units = p.nrows / w.R;
    // dense batches: groups of columns share one decode (max_group)
    const int group_max = !multi_col || p.ids ? 1 : x_bf16 ? group_for<bf16_t>(C) : group_for<float>(C);
    for (int c0 = 0; c0 < (group_max == 1 ? 1 : ncols); c0 += group_max) {
        const int nc = group_max == 1 ? 1 : (ncols - c0 < group_max ? ncols - c0 : group_max);
        const int ny = group_max == 1 ? ncols : 1;
        cols q = p;
        // a dense product whose columns all fit one launch reads each plane byte once, and a matrix of 2^27 weights
        // or more outlasts the caches between two launches: keep such planes out of the way of the activations.
        // One routed token names each of its experts once. Routed batches and column loops over smaller matrices read
        // words again and keep the default policy.
        q.plane_once = p.ids ? ncols <= p.n_used
                              : (group_max == 1 ? ncols == 1 : ncols <= group_max) || p.nrows * w.K >= ((int64_t) 1 << 27);
        q.stream_once = q.plane_once;
        if (group_max > 1) {
            q.x += c0 * p.x_tok;
            q.y += c0 * p.y_tok;
        }
        int wpb, blocks, upw;
        // wavefronts per CU the instance is sized for, by its activation registers (x_regs): 16 up to 64 registers,
        // then three per SIMD in blocks of four, two per SIMD beyond 112
        const int xr = nc * (C >= 2 ? C / 2 : 1) * (x_bf16 ? 8 : 16);
        w64_dims(units, ny, cus, wpb, blocks, upw, !wide_regs(xr, x_bf16, C) ? 16 : xr <= 112 ? 12 : 8);
        const dim3 grid(blocks, ny);
        if (x_bf16) {
            mmv_c<bf16_t>(C, nc, grid, wpb * 64, wpb, stream, w, q, upw);
        } else {
            mmv_c<float>(C, nc, grid, wpb * 64, wpb, stream, w, q, upw);
        }
    }
}

template <typename TX>
void glu_c(int C, dim3 grid, int nt, int wpb, hipStream_t stream, const bf16n_weight & g, const bf16n_weight & u, const cols & p, int upw) {
    const size_t shm = w64_shm(2 * wpb);
    switch (C) {
        case 1: hipLaunchKernelGGL((k_w64_glu<TX, 1>), grid, dim3(nt), shm, stream, g, u, p, upw); break;
        case 2: hipLaunchKernelGGL((k_w64_glu<TX, 2>), grid, dim3(nt), shm, stream, g, u, p, upw); break;
        case 4: hipLaunchKernelGGL((k_w64_glu<TX, 4>), grid, dim3(nt), shm, stream, g, u, p, upw); break;
        default: hipLaunchKernelGGL((k_w64_glu<TX, 8>), grid, dim3(nt), shm, stream, g, u, p, upw); break;
    }
}

// y = silu(gate x) * (up x), one column per launch row (dense tokens or (token, slot) pairs with expert ids)
void launch_w64_glu(const bf16n_weight & gate, const bf16n_weight & up, const cols & p, int ncols, bool x_bf16, int cus,
                    hipStream_t stream) {
    const int C = (int) (gate.K / CHUNK);
    const int64_t units = p.nrows / gate.R;
    const int64_t max_waves = (int64_t) cus * 16 / (ncols < 1 ? 1 : ncols) < 16 ? 16 : (int64_t) cus * 16 / (ncols < 1 ? 1 : ncols);
    const int64_t upw = (units + max_waves - 1) / max_waves;
    const int64_t waves = (units + upw - 1) / upw;
    const int wpb = (int) (waves < 4 ? waves : 4);
    const dim3 grid((unsigned) ((waves + wpb - 1) / wpb), ncols);
    cols q = p;
    q.plane_once = p.ids ? ncols <= p.n_used : ncols == 1; // one token: every plane byte is read once
    q.stream_once = q.plane_once;
    if (x_bf16) {
        glu_c<bf16_t>(C, grid, wpb * 64, wpb, stream, gate, up, q, (int) upw);
    } else {
        glu_c<float>(C, grid, wpb * 64, wpb, stream, gate, up, q, (int) upw);
    }
}

void launch_w64_dequant(const bf16n_weight & w, int64_t row0, int64_t nrows, uint16_t * out, int cus, hipStream_t stream) {
    const int64_t units = nrows / w.R;
    const int64_t max_waves = (int64_t) cus * 16;
    const int64_t upw = (units + max_waves - 1) / max_waves;
    const int64_t waves = (units + upw - 1) / upw;
    const int wpb = 4;
    hipLaunchKernelGGL(k_w64_dequant, dim3((unsigned) ((waves + wpb - 1) / wpb)), dim3(wpb * 64), w64_shm(wpb), stream, w, row0, nrows,
                       out, (int) upw);
}

void launch_w64_get_rows(const bf16n_weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16,
                         int64_t dst_s1, int64_t row0, hipStream_t stream) {
    const int wpb = 4;
    hipLaunchKernelGGL(k_w64_get_rows, dim3((unsigned) ((n + wpb - 1) / wpb)), dim3(wpb * 64), w64_shm(wpb), stream, w, (const char *) ids,
                       ids_s0, n, row0, (char *) dst, dst_s1, !dst_bf16);
}

} // namespace dev
} // namespace bf16n
