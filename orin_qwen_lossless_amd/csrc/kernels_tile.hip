// Kernels for the tile form of the wave64 layout (FLAG_WAVE64 with R = 32; include/bf16n/format.h): units are 32-row x
// 256-column tiles whose decode order is the A-operand order of v_mfma_f32_32x32x16_bf16.  In step s (of 8) of a tile,
// lane 32 h + l holds, in slot order, columns 32 s + 8 h + [0, 8) and 32 s + 16 + 8 h + [0, 8) of row l: the eight
// BF16 pairs that the decoder produces are, as they stand, the A operands of two matrix instructions.  The tiles of a
// row group are consecutive units, so a wavefront decodes them as one run of its stream.
//
//   * k_mm_tile: batched MoE prefill (reference mm_ids / k_hp_mm_ids, core/src/launch.cu:473-535,
//     core/src/kernels.cuh:1162-1505).  Weights go from the decoder's registers into the matrix cores; the activations
//     of up to 128 tokens are staged in LDS, 128 columns at a time, and shared by the eight wavefronts of a block.
//   * k_tile_mmv: GEMV / fused gate-up GEMV at decode (reference mmv / mmv_glu, launch.cu:313-365): a lane accumulates
//     one row over the whole tile, so a tile ends with one cross-half add instead of a reduction per row.
//   * k_tile_dequant, k_tile_get_rows: exact BF16 rows (launch.cu:367-443).
#include "dev_common.h"
#include "dev_compat.h"
#include "dev_topk.h"
#include "dev_w64.h"
#include "launchers.h"

#include <algorithm>
#include <cmath>

#include <stdexcept>

namespace bf16n {
namespace dev {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int T_STEPS = 8;                      // steps per tile
constexpr int T_BYTES = TILE_R * TILE_K;        // plane bytes per tile
constexpr int STEP_BYTES = 1024;

// column (inside the tile) of the first of the four weights that plane word j of a lane holds in step s
__device__ __forceinline__ int tile_col(int s, int j, int half) { return 32 * s + 16 * (j >> 1) + 8 * half + 4 * (j & 1); }

// One decode chain: the tiles [first unit, first unit + n) of one matrix, with the plane bytes of the next D steps
// in registers (reloaded as soon as a step is consumed).
// ONCE: the plane bytes are read by this launch only and are loaded with the non-temporal hint; stream_once (start)
// asks the same for the stream blocks, which pays for routed experts and not for a large dense matrix
template <int D, bool ONCE = false> struct tchain_t {
    w64_dec dec;
    range_t plane;   // the plane bytes of the chain's tiles
    uint32_t off;    // byte offset of this lane's 16 bytes in the next step to load
    uint4 sm[D];
    __device__ __forceinline__ uint4 load_step(int) const { // past the end of the chain: dropped, reads as zeros
        return range_load16<ONCE>(plane, off);
    }
    __device__ __forceinline__ void start(uint32_t * ring, const w64_ptrs & q, int64_t unit0, int n_units, int lane, bool stream_once = false) {
        start(ring, q, unit0, n_units, lane, q.ubase[unit0], q.ubase[unit0 + n_units], stream_once);
    }
    // first / end: the stream words of the units (their unit bases, read by the caller ahead of time)
    __device__ __forceinline__ void start(uint32_t * ring, const w64_ptrs & q, int64_t unit0, int n_units, int lane, uint32_t first,
                                          uint32_t end, bool stream_once = false, bool split = false) {
        plane = make_range(q.plane + uniform64(unit0 * T_BYTES), uniform((uint32_t) (n_units * T_BYTES)));
        off = 16 * (uint32_t) lane;
#pragma unroll
        for (int s = 0; s < D; s++) {
            sm[s] = load_step(lane);
            off += STEP_BYTES;
        }
        dec.start(ring, q.stream, uniform(first), uniform(end), lane, stream_once, split);
    }
    // s: the step just consumed (a compile-time value at every call)
    __device__ __forceinline__ void reload(int s, int lane) {
        sm[s % D] = load_step(lane);
        off += STEP_BYTES;
    }
    __device__ __forceinline__ void begin_tile() {
        dec.keep_ahead();
        dec.begin_unit();
        dec.keep_ahead();
    }
};
typedef tchain_t<4> tchain;

// one step of N chains, instruction streams interleaved; lut of chain k at lut + k * lut_stride
// ABS: the tables sit at the start of the kernel's LDS (address 0): see w64_dec_t::two_at
template <int N, int D, bool ONCE = false, bool ABS = false>
__device__ __forceinline__ void tile_step(tchain_t<D, ONCE> * ch, const uint32_t * lut, int lut_stride, int s, uint32_t (&wp)[N][8]) {
    uint32_t smw[N][4];
#pragma unroll
    for (int k = 0; k < N; k++) {
        smw[k][0] = ch[k].sm[s % D].x; smw[k][1] = ch[k].sm[s % D].y; smw[k][2] = ch[k].sm[s % D].z; smw[k][3] = ch[k].sm[s % D].w;
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int k = 0; k < N; k++) {
            uint32_t e0, e1;
            if constexpr (ABS) {
                ch[k].dec.two_at((uint32_t) (k * lut_stride * 4), e0, e1);
            } else {
                ch[k].dec.two(lut + k * lut_stride, e0, e1);
            }
            wp[k][2 * j] = merge(spread_lo(smw[k][j]), e0);
            wp[k][2 * j + 1] = merge(spread_hi(smw[k][j]), e1);
        }
    }
#pragma unroll
    for (int k = 0; k < N; k++) {
        ch[k].dec.keep_ahead();
    }
}

// One step of two chains against one block of 32 tokens on the matrix cores.  The two matrix instructions of a
// 16-column block are issued right behind its decode and run while the next block is decoded (2 to 5 % faster than all
// four at the end of the step, and some registers fewer: no spills at 128).  b(kb): the B operand of 16-column block kb.
template <int D, bool ONCE, typename B>
__device__ __forceinline__ void tile_step_mm(tchain_t<D, ONCE> * ch, const uint32_t * lut, int lut_stride, int s, int lane, B b,
                                             f32x16_t & acc0, f32x16_t & acc1) {
    uint32_t smw[2][4];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const uint4 v = ch[k].sm[s % D];
        smw[k][0] = v.x; smw[k][1] = v.y; smw[k][2] = v.z; smw[k][3] = v.w;
    }
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {
        bf16x8_t av[2];
#pragma unroll
        for (int k = 0; k < 2; k++) {
            uint32_t wq[4];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint32_t e0, e1;
                ch[k].dec.two_at((uint32_t) (k * lut_stride * 4), e0, e1); // (its callers keep the tables at LDS address 0)
                wq[2 * j] = merge(spread_lo(smw[k][2 * kb + j]), e0);
                wq[2 * j + 1] = merge(spread_hi(smw[k][2 * kb + j]), e1);
            }
            const u32x4_t v = {wq[0], wq[1], wq[2], wq[3]};
            av[k] = __builtin_bit_cast(bf16x8_t, v);
        }
        const bf16x8_t bv = b(kb);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv, acc1, 0, 0, 0);
    }
    ch[0].dec.keep_ahead();
    ch[1].dec.keep_ahead();
    ch[0].reload(s, lane);
    ch[1].reload(s, lane);
}

// ---------------------------------------------------------------- batched MoE prefill

constexpr int MT_SMALL_PAIRS = 16;  // routed pairs per expert up to which the 32-token shape is used
constexpr int MT_MAX_LISTED = 1024; // experts up to which a block lists the active ones
constexpr int MT_MAX_UNITS = 2 * MT_MAX_LISTED; // listed (expert, pass of 32 tokens) units: one per active expert and one
                                                // more per 32 routed pairs, of which the 32-token shape takes 16 per expert
constexpr int MT_HK = 128;         // activation columns staged at a time (half a tile)
constexpr int MT_BSTRIDE = 136;    // BF16 elements per staged token row: 272 bytes spread 16 lanes over all banks

// Three shapes of the kernel.  NT = 4: passes of 128 tokens, eight wavefronts per block (the 2 x 4 accumulator blocks
// take 128 registers: two wavefronts per SIMD).  NT = 1: passes of 32 tokens for experts, or dense matrices, with few
// tokens, where the decode is all that counts: sixteen wavefronts per block (32 accumulator registers: four wavefronts
// per SIMD, twice the decode chains per CU), or four per block, two blocks per CU, when so few experts are active that
// whole experts per block would leave most of the CUs idle.
template <int NT, int W> struct mt_shape {
    static constexpr int WAVES = W, THREADS = WAVES * 64, TOK = 32 * NT;
    static constexpr int STAGERS = TOK * MT_HK / 8 < THREADS ? TOK * MT_HK / 8 : THREADS; // threads that stage activations
    static constexpr int TPT = STAGERS / TOK;                      // of them per token
    static constexpr int CPT = MT_HK / TPT;                        // columns each: 8 per uint4
    static constexpr int VPT = CPT / 8;
    // steps of plane bytes held ahead per chain: two in every shape (a step of the 128-token shape takes about 2 us,
    // longer than a load; four ahead took 18 more registers and ran the down product 6 % slower at 2048 tokens)
    static constexpr int DEPTH = 2;
};

// the V uint4s a thread stages per block of activations, in named registers (under this kernel's register pressure
// an array, or a struct of them, stays in scratch, and every load into it is waited for at once)
#define MT_STAGE_LOAD(V, r0, r1, r2, r3, p)  \
    do {                                      \
        r0 = (p)[0];                          \
        if constexpr ((V) >= 2) r1 = (p)[1];  \
        if constexpr ((V) >= 4) {             \
            r2 = (p)[2];                      \
            r3 = (p)[3];                      \
        }                                     \
    } while (0)
#define MT_STAGE_STORE(V, r0, r1, r2, r3, p) \
    do {                                      \
        (p)[0] = r0;                          \
        if constexpr ((V) >= 2) (p)[1] = r1;  \
        if constexpr ((V) >= 4) {             \
            (p)[2] = r2;                      \
            (p)[3] = r3;                      \
        }                                     \
    } while (0)

// Component c (0, 1, 2) of eight FP32 activations as BF16: x = hi + mid + lo exactly (three times eight significant
// bits cover the 24 of an FP32 value), each the nearest BF16 of what the previous ones leave.  A product of FP32
// activations becomes three columns of BF16 products, exact in FP32, added at the end.
__device__ __forceinline__ uint4 split_bf16(const uint4 a, const uint4 b, int c) {
    const uint32_t in[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t out[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float x = __uint_as_float(in[i]);
        const uint32_t hi = f32_to_bf16_rne(x);
        const float hf = __uint_as_float(hi << 16);
        const bool fin = (hi & 0x7F80u) != 0x7F80u;               // infinities and NaNs stay in the first component alone
        const float r1 = fin ? x - hf : 0.f;
        const uint32_t mid = f32_to_bf16_rne(r1);
        const float r2 = r1 - __uint_as_float(mid << 16);
        const uint32_t lo = f32_to_bf16_rne(r2);
        out[i] = c == 0 ? hi : c == 1 ? mid : lo;
    }
    return make_uint4(out[0] | (out[1] << 16), out[2] | (out[3] << 16), out[4] | (out[5] << 16), out[6] | (out[7] << 16));
}

struct mm_args {
    const uint16_t * x; int64_t x_row;
    const int32_t * ids_src1, * ids_dst, * bounds; // all null: one dense matrix, token j reads row j of x and writes column j
    char * dst; int64_t dst_col; bool dst_bf16;
    int64_t rows;   // per expert
    int n_experts, n_tok;
};

// The work of a call with routing lists, listed in LDS: one unit per active expert and pass of 32 of its tokens, in
// expert order (unit[MT_MAX_UNITS]: expert | pass << 16; their number is returned).  The blocks share out the work
// items of these only, so that a call with few active experts keeps its blocks equally loaded instead of leaving some
// with several items and others with none, and the passes of an expert with more than 32 tokens (one that every token
// uses, say) run side by side on different blocks instead of one after the other on one.  Every wavefront of the block
// takes 64 experts at a time (one read of their bounds for the whole block), the counts meet in LDS behind the list.
// Ends with a barrier.  span (optional, [MT_MAX_UNITS]): first routed pair and number of pairs of every unit.
template <int TOK = 32>
__device__ __forceinline__ int list_units(uint32_t * unit, const mm_args & a, int wave, int lane, int n_waves, int2 * span = nullptr) {
    int * cnt = (int *) (unit + MT_MAX_UNITS); // [n_waves], n_waves <= 16
    int total = 0;
    for (int e0 = 0; e0 < a.n_experts; e0 += 64 * n_waves) {
        const int e = e0 + 64 * wave + lane;
        const int b0 = e < a.n_experts ? a.bounds[e] : 0, b1 = e < a.n_experts ? a.bounds[e + 1] : 0;
        const int np = b1 > b0 ? (b1 - b0 + TOK - 1) / TOK : 0;
        int scan; // inclusive prefix of the passes over the lanes
        if (__ballot(np > 1) == 0) { // (nearly always: no expert of these 64 has more than a pass of tokens)
            const uint64_t m = __ballot(np > 0);
            scan = (int) __builtin_amdgcn_mbcnt_hi((uint32_t) (m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t) m, 0u)) + np;
        } else {
            scan = np;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(scan, o, 64);
                scan += lane >= o ? up : 0;
            }
        }
        if (lane == 63) {
            cnt[wave] = scan;
        }
        __syncthreads();
        int before = total, all = 0;
        for (int k = 0; k < n_waves; k++) {
            const int c = cnt[k];
            before += k < wave ? c : 0;
            all += c;
        }
        const int at = before + scan - np;
        for (int k = 0; k < np && at + k < MT_MAX_UNITS; k++) {
            unit[at + k] = (uint32_t) e | ((uint32_t) k << 16);
            if (span) {
                span[at + k] = make_int2(b0 + TOK * k, b1 - b0 - TOK * k < TOK ? b1 - b0 - TOK * k : TOK);
            }
        }
        total += all;
        __syncthreads();
    }
    return (int) uniform((uint32_t) (total < MT_MAX_UNITS ? total : MT_MAX_UNITS));
}

// A work item is (expert, slab of row groups): every wavefront owns two decode chains, gate and up of one row group
// (GLU) or two row groups of the matrix, and keeps their 2 x NT accumulator blocks (32 rows x 32 tokens each) for
// the whole pass over the expert's K columns.  Per step a chain yields two A operands (32 rows x 16 columns); the B
// operands (16 columns x 32 tokens) come from the staged activations and are used by both chains.
// XF32 (dense products of up to ten FP32 activation columns, 32-token shape): a.x holds FP32 rows and token 3 j + c of
// the pass is component c of column j (split_bf16); the three accumulator columns of a token are added before the store.
template <bool GLU, int NT, int W, bool XF32 = false>
__global__ void __launch_bounds__((mt_shape<NT, W>::THREADS)) k_mm_tile(const bf16n_weight w, const bf16n_weight w_up, const mm_args a) {
    using S = mt_shape<NT, W>;
    static_assert(!XF32 || (NT == 1 && W == 16 && !GLU), "FP32 activations: the dense 32-token shape only");
    constexpr int XB = XF32 ? 4 : 2;                          // bytes per activation
    constexpr int NM = GLU ? 2 : 1;
    extern __shared__ __align__(16) uint32_t shm[];
    uint32_t * lut = shm;
    uint32_t * rings = shm + NM * LUT_WORDS;
    uint16_t * bbuf = (uint16_t *) (rings + S::WAVES * 2 * WAVE_LDS_WORDS); // two buffers of TOK x MT_BSTRIDE
    const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31, half = lane >> 5, wave = (int) uniform(tid >> 6);
    stage_lut(lut, (const uint32_t *) (w.aux + w.off_a));
    if (GLU) {
        stage_lut(lut + LUT_WORDS, (const uint32_t *) (w_up.aux + w_up.off_a));
    }
    const int slabs = (int) (w.K / TILE_K), halves = 2 * slabs;
    const int groups = (int) (a.rows / TILE_R);               // row groups per expert
    constexpr int GPI = GLU ? S::WAVES : 2 * S::WAVES;        // row groups per work item
    const int slabs_per_expert = (groups + GPI - 1) / GPI;
    const w64_ptrs q0 = w64p(w), q1 = w64p(GLU ? w_up : w);
    // this thread's share of a staged block: CPT columns of one token (NT = 1: the upper wavefronts stage nothing)
    const bool stager = S::STAGERS == S::THREADS || wave < S::STAGERS / 64;
    const int b_tok = stager ? tid / S::TPT : 0, b_part = tid % S::TPT;
    uint32_t * unit = (uint32_t *) (bbuf + 2 * S::TOK * MT_BSTRIDE);
    // (passes of 128 tokens are for calls with many tokens per expert: every expert is active)
    const bool listed = NT == 1 && a.bounds != nullptr && a.n_experts <= MT_MAX_LISTED;
    const int n_act = listed ? list_units(unit, a, wave, lane, S::WAVES) : a.n_experts;
    __syncthreads();
    for (int item = blockIdx.x; item < n_act * slabs_per_expert; item += gridDim.x) {
        // (read from LDS: the same in every lane, and kept in a scalar register like the arithmetic form)
        const uint32_t un = listed ? uniform(unit[item / slabs_per_expert]) : (uint32_t) (item / slabs_per_expert);
        const int e = listed ? (int) (un & 0xFFFFu) : (int) un, sl = item % slabs_per_expert;
        // a listed unit is one pass of 32 tokens of its expert
        const int first = a.bounds ? a.bounds[e] : 0, j0 = listed ? first + 32 * (int) (un >> 16) : first;
        const int left_e = a.bounds ? a.bounds[e + 1] - j0 : a.n_tok, n = listed && left_e > 32 ? 32 : left_e;
        // this wavefront's row groups (inside the expert); a missing second group repeats the first and is dropped
        const int g0 = GLU ? sl * GPI + wave : sl * GPI + 2 * wave;
        const bool live = g0 < groups, has1 = GLU || g0 + 1 < groups;
        const int g1 = GLU ? g0 : (has1 ? g0 + 1 : g0);
        for (int tp = 0; tp < n; tp += S::TOK) {
            const int left = n - tp, nt = NT == 1 ? 1 : left >= S::TOK ? NT : (left + 31) >> 5;
            const int btk = tp + b_tok;
            const int bj = j0 + (btk < n ? btk : 0);
            const int bcomp = XF32 ? bj % 3 : 0;
            // (element pointers, not bytes: the byte form costs the BF16 instances five more spilled registers)
            const uint16_t * xsrc = a.x + ((int64_t) (XF32 ? bj / 3 : a.ids_src1 ? a.ids_src1[bj] : bj) * a.x_row + S::CPT * b_part) * (XB / 2);
            uint16_t * bdst = bbuf + b_tok * MT_BSTRIDE + S::CPT * b_part;
            constexpr int VLD = XF32 ? 2 * S::VPT : S::VPT;       // uint4 loads per thread and block
            uint4 f0, f1, f2, f3;
            if (stager) {
                MT_STAGE_LOAD(VLD, f0, f1, f2, f3, (const uint4 *) xsrc);
            }
            // 32-token shape: (nearly) every tile of a launch is decoded once, so its loads are read-once; the 128-token
            // shape serves long token lists, whose passes share tiles
            tchain_t<S::DEPTH, NT == 1> ch[2];
            if (live) {
                uint32_t * ring = rings + wave * (2 * WAVE_LDS_WORDS);
                ch[0].start(ring, q0, ((int64_t) e * groups + g0) * slabs, slabs, lane, NT == 1 && a.bounds != nullptr);
                ch[1].start(ring + WAVE_LDS_WORDS, q1, ((int64_t) e * groups + g1) * slabs, slabs, lane, NT == 1 && a.bounds != nullptr);
            }
            f32x16_t acc[2][NT];
#pragma unroll
            for (int c = 0; c < 2; c++) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        acc[c][t][i] = 0.f;
                    }
                }
            }
            if (stager) {
                if constexpr (XF32) {
                    *(uint4 *) bdst = split_bf16(f0, f1, bcomp);
                } else {
                    MT_STAGE_STORE(S::VPT, f0, f1, f2, f3, (uint4 *) bdst);
                }
            }
            __syncthreads();
#pragma unroll 1
            for (int hs = 0; hs < halves; hs++) {
                const uint16_t * bcur = bbuf + (hs & 1) * (S::TOK * MT_BSTRIDE);
                // the next block of activations: requested now, staged after this block's steps.  Unconditional and
                // local to the iteration (after the last block the same block goes into the buffer nobody reads any
                // more): registers that are loaded under a condition and live around the loop are filled through a
                // temporary with a full wait per load.
                const int nxt = hs + 1 < halves ? hs + 1 : hs;
                uint4 b0, b1, b2, b3;
                if (stager) {
                    MT_STAGE_LOAD(VLD, b0, b1, b2, b3, (const uint4 *) (xsrc + nxt * MT_HK * (XB / 2)));
                }
                if (live) {
                    if ((hs & 1) == 0) {
                        ch[0].begin_tile();
                        ch[1].begin_tile();
                    }
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        const uint16_t * bp = bcur + l32 * MT_BSTRIDE + 32 * s + 8 * half;
                        if constexpr (NT == 1) {
                            // (with four token blocks the same order measured 3 to 4 % slower than the whole step's
                            // matrix instructions together)
                            tile_step_mm(ch, lut, GLU ? LUT_WORDS : 0, s, lane,
                                         [&](int kb) { return *(const bf16x8_t *) (bp + 16 * kb); }, acc[0][0], acc[1][0]);
                        } else {
                            uint32_t wp[2][8];
                            tile_step<2, S::DEPTH, NT == 1, true>(ch, lut, GLU ? LUT_WORDS : 0, s, wp);
                            ch[0].reload(s, lane);
                            ch[1].reload(s, lane);
                            bf16x8_t av[2][2]; // [chain][16-column block]
#pragma unroll
                            for (int c = 0; c < 2; c++) {
#pragma unroll
                                for (int kb = 0; kb < 2; kb++) {
                                    const u32x4_t v = {wp[c][4 * kb], wp[c][4 * kb + 1], wp[c][4 * kb + 2], wp[c][4 * kb + 3]};
                                    av[c][kb] = __builtin_bit_cast(bf16x8_t, v);
                                }
                            }
                            // token blocks beyond the first are there only for experts with that many tokens (one
                            // branch per block: both B operands are read together, then four matrix instructions)
#pragma unroll
                            for (int t = 0; t < NT; t++) {
                                if (t == 0 || t < nt) {
                                    const bf16x8_t bv0 = *(const bf16x8_t *) (bp + t * 32 * MT_BSTRIDE);
                                    const bf16x8_t bv1 = *(const bf16x8_t *) (bp + t * 32 * MT_BSTRIDE + 16);
                                    acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0][0], bv0, acc[0][t], 0, 0, 0);
                                    acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1][0], bv0, acc[1][t], 0, 0, 0);
                                    acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0][1], bv1, acc[0][t], 0, 0, 0);
                                    acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1][1], bv1, acc[1][t], 0, 0, 0);
                                }
                            }
                        }
                    }
                }
                if (stager) {
                    uint4 * bn = (uint4 *) (bdst + ((hs + 1) & 1) * (S::TOK * MT_BSTRIDE));
                    if constexpr (XF32) {
                        *bn = split_bf16(b0, b1, bcomp);
                    } else {
                        MT_STAGE_STORE(S::VPT, b0, b1, b2, b3, bn);
                    }
                }
                __syncthreads();
            }
            if constexpr (XF32) {
                // the three components of a token sit in adjacent lanes of a half: their sum lands in the first
#pragma unroll
                for (int c = 0; c < 2; c++) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const float v = acc[c][0][i];
                        acc[c][0][i] = (v + __shfl_down(v, 1, 32)) + __shfl_down(v, 2, 32);
                    }
                }
            }
            // accumulator element i of a lane: row 8 (i / 4) + 4 (lane / 32) + i % 4 of the group, token lane % 32
            if (live) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int tk = tp + 32 * t + l32;
                    if (t < nt && tk < n && (!XF32 || tk % 3 == 0)) {
                        const int64_t col = (int64_t) (XF32 ? tk / 3 : a.ids_dst ? a.ids_dst[j0 + tk] : tk) * a.dst_col;
#pragma unroll
                        for (int c = 0; c < (GLU ? 1 : 2); c++) {
                            if (c == 1 && !has1) {
                                continue;
                            }
                            const int64_t row0 = (int64_t) (c ? g1 : g0) * TILE_R + 4 * half;
#pragma unroll
                            for (int g = 0; g < 4; g++) {
                                float v[4];
#pragma unroll
                                for (int i = 0; i < 4; i++) {
                                    const float p = acc[c][t][4 * g + i];
                                    v[i] = GLU ? acc[1][t][4 * g + i] * silu(p) : p;
                                }
                                const int64_t o = col + row0 + 8 * g;
                                if (a.dst_bf16) {
                                    *(uint2 *) ((uint16_t *) a.dst + o) =
                                        make_uint2(f32_to_bf16_rne(v[0]) | ((uint32_t) f32_to_bf16_rne(v[1]) << 16),
                                                   f32_to_bf16_rne(v[2]) | ((uint32_t) f32_to_bf16_rne(v[3]) << 16));
                                } else {
                                    *(float4 *) ((float *) a.dst + o) = make_float4(v[0], v[1], v[2], v[3]);
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- batched MoE prefill in two phases (many tokens per expert)
//
// With a few hundred tokens per expert the fused kernel above decodes every expert once per pass of 128 tokens, at
// half the decode chains per CU of the GEMV (its accumulators take the registers), and the decode is what it waits
// for.  The two-phase form decodes a group of experts once, at the GEMV's chain count, into a scratch buffer of the
// caller's (k_tile_expand), and multiplies from there with a kernel that has no decoder in its registers (k_mm_raw).
// The scratch keeps the tiles in the decoder's own order, the A-operand order of the matrix instruction: tile u of
// the group, step s, 16-column block kb, lane l -> 16 bytes at ((u * 8 + s) * 2 + kb) * 1024 + 16 l, so that both
// kernels move whole 1 KiB rows per wavefront and instruction.  A group is sized to stay in the last-level cache
// between the two kernels.
constexpr int TILE_RAW_BYTES = TILE_R * TILE_K * 2;   // one tile as BF16
constexpr int EXPAND_WAVES = 16;

// chain c of the launch decodes tiles [c * tpc, (c + 1) * tpc) of matrix blockIdx.y (0: w, 1: w_up) from unit
// unit_first on; two chains per wavefront.  Experts without tokens are skipped (bounds, tiles_per_expert).
__global__ void __launch_bounds__(EXPAND_WAVES * 64) k_tile_expand(const bf16n_weight w, const bf16n_weight w_up, int64_t unit_first, int n_units,
                                                                   int tpc, int tiles_per_expert, const int32_t * __restrict__ bounds,
                                                                   uint4 * __restrict__ out) {
    __shared__ __align__(16) uint32_t lut[LUT_WORDS];
    extern __shared__ __align__(16) uint32_t rings[];
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6);
    const bool second = blockIdx.y != 0;
    const w64_ptrs q = w64p(second ? w_up : w);
    stage_lut(lut, q.lut);
    const int n_chains = (n_units + tpc - 1) / tpc;
    const int c0 = ((int) blockIdx.x * EXPAND_WAVES + wave) * 2;
    __syncthreads();
    if (c0 >= n_chains) {
        return;
    }
    const bool two = c0 + 1 < n_chains;
    int u0[2], n[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int c = two || k == 0 ? c0 + k : c0;  // a missing second chain repeats the first and stores nothing
        u0[k] = c * tpc;
        n[k] = n_units - u0[k] < tpc ? n_units - u0[k] : tpc;
        if (bounds) {
            const int e = (int) ((unit_first + u0[k]) / tiles_per_expert);
            if (bounds[e + 1] == bounds[e]) {
                n[k] = 0;
            }
        }
    }
    if (n[0] == 0 && (!two || n[1] == 0)) {
        return;
    }
    // (a chain of an expert without tokens rides along with its neighbour and stores nothing)
    const bool st0 = n[0] > 0, st1 = two && n[1] > 0;
    if (!st0) { u0[0] = u0[1]; n[0] = n[1]; }
    if (!st1) { u0[1] = u0[0]; n[1] = n[0]; }
    const int steps = n[0] < n[1] ? n[1] : n[0];
    tchain_t<4, true> ch[2];
    uint32_t * ring = rings + wave * (2 * WAVE_LDS_WORDS);
    ch[0].start(ring, q, unit_first + u0[0], n[0], lane, true);
    ch[1].start(ring + WAVE_LDS_WORDS, q, unit_first + u0[1], n[1], lane, true);
    uint4 * o0 = out + ((int64_t) (second ? n_units : 0) + u0[0]) * (TILE_RAW_BYTES / 16) + lane;
    uint4 * o1 = out + ((int64_t) (second ? n_units : 0) + u0[1]) * (TILE_RAW_BYTES / 16) + lane;
    for (int u = 0; u < steps; u++) { // (n[0] == n[1] except for the last chain of the launch, whose partner runs past its own end harmlessly: see below)
        ch[0].begin_tile();
        ch[1].begin_tile();
#pragma unroll 1
        for (int hh = 0; hh < 2; hh++) {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                uint32_t wp[2][8];
                tile_step<2, 4, true>(ch, lut, 0, s, wp);
                ch[0].reload(s, lane);
                ch[1].reload(s, lane);
                const int so = ((4 * hh + s) * 2) * 64;
                if (st0 && u < n[0]) {
                    o0[so] = make_uint4(wp[0][0], wp[0][1], wp[0][2], wp[0][3]);
                    o0[so + 64] = make_uint4(wp[0][4], wp[0][5], wp[0][6], wp[0][7]);
                }
                if (st1 && u < n[1]) {
                    o1[so] = make_uint4(wp[1][0], wp[1][1], wp[1][2], wp[1][3]);
                    o1[so + 64] = make_uint4(wp[1][4], wp[1][5], wp[1][6], wp[1][7]);
                }
            }
        }
        o0 += TILE_RAW_BYTES / 16;
        o1 += TILE_RAW_BYTES / 16;
    }
}

// The product from expanded tiles.  Work items, passes, staging of the activations and the stores are those of
// k_mm_tile's 128-token shape; the A operands are loaded, two steps ahead, from the scratch (t0: tiles of w for the
// experts [e0, e0 + n_e), t1: of w_up, or t0 again).
template <bool GLU, int NT, int W>
__global__ void __launch_bounds__((mt_shape<NT, W>::THREADS)) k_mm_raw(const uint4 * __restrict__ t0, const uint4 * __restrict__ t1, const mm_args a,
                                                                       int e0, int n_e, int slabs) {
    using S = mt_shape<NT, W>;
    constexpr int D = 2; // steps of A operands in flight (four take 64 registers and spill)
    extern __shared__ __align__(16) uint32_t shm[];
    uint16_t * bbuf = (uint16_t *) shm; // two buffers of TOK x MT_BSTRIDE
    const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31, half = lane >> 5, wave = (int) uniform(tid >> 6);
    const int halves = 2 * slabs;
    const int groups = (int) (a.rows / TILE_R);
    constexpr int GPI = GLU ? S::WAVES : 2 * S::WAVES;
    const int slabs_per_expert = (groups + GPI - 1) / GPI;
    const bool stager = S::STAGERS == S::THREADS || wave < S::STAGERS / 64;
    const int b_tok = stager ? tid / S::TPT : 0, b_part = tid % S::TPT;
    constexpr int TU = TILE_RAW_BYTES / 16; // uint4 per tile
    for (int item = blockIdx.x; item < n_e * slabs_per_expert; item += gridDim.x) {
        const int el = item / slabs_per_expert, e = e0 + el, sl = item % slabs_per_expert;
        const int j0 = a.bounds[e], n = a.bounds[e + 1] - j0;
        const int g0 = GLU ? sl * GPI + wave : sl * GPI + 2 * wave;
        const bool live = g0 < groups, has1 = GLU || g0 + 1 < groups;
        const int g1 = GLU ? g0 : (has1 ? g0 + 1 : g0);
        const uint4 * pa0 = t0 + ((int64_t) el * groups + (live ? g0 : 0)) * slabs * TU + lane;
        const uint4 * pa1 = t1 + ((int64_t) el * groups + (live ? g1 : 0)) * slabs * TU + lane;
        const int n_steps = T_STEPS * slabs;
        for (int tp = 0; tp < n; tp += S::TOK) {
            const int left = n - tp, nt = left >= S::TOK ? NT : (left + 31) >> 5;
            const int btk = tp + b_tok;
            const int bj = j0 + (btk < n ? btk : 0);
            const uint16_t * xsrc = a.x + ((int64_t) (a.ids_src1 ? a.ids_src1[bj] : bj) * a.x_row + S::CPT * b_part);
            uint16_t * bdst = bbuf + b_tok * MT_BSTRIDE + S::CPT * b_part;
            uint4 f0, f1, f2, f3;
            if (stager) {
                MT_STAGE_LOAD(S::VPT, f0, f1, f2, f3, (const uint4 *) xsrc);
            }
            // A operands of the first D steps: [step][chain][16-column block]
            uint4 av[D][2][2];
#pragma unroll
            for (int s = 0; s < D; s++) {
                av[s][0][0] = pa0[(s * 2) * 64];
                av[s][0][1] = pa0[(s * 2 + 1) * 64];
                av[s][1][0] = pa1[(s * 2) * 64];
                av[s][1][1] = pa1[(s * 2 + 1) * 64];
            }
            f32x16_t acc[2][NT];
#pragma unroll
            for (int c = 0; c < 2; c++) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        acc[c][t][i] = 0.f;
                    }
                }
            }
            if (stager) {
                MT_STAGE_STORE(S::VPT, f0, f1, f2, f3, (uint4 *) bdst);
            }
            __syncthreads();
#pragma unroll 1
            for (int hs = 0; hs < halves; hs++) {
                const uint16_t * bcur = bbuf + (hs & 1) * (S::TOK * MT_BSTRIDE);
                const int nxt = hs + 1 < halves ? hs + 1 : hs;
                uint4 b0, b1, b2, b3;
                if (stager) {
                    MT_STAGE_LOAD(S::VPT, b0, b1, b2, b3, (const uint4 *) (xsrc + nxt * MT_HK));
                }
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    const uint16_t * bp = bcur + l32 * MT_BSTRIDE + 32 * s + 8 * half;
                    const int sd = s % D;
                    const bf16x8_t a00 = __builtin_bit_cast(bf16x8_t, av[sd][0][0]), a01 = __builtin_bit_cast(bf16x8_t, av[sd][0][1]);
                    const bf16x8_t a10 = __builtin_bit_cast(bf16x8_t, av[sd][1][0]), a11 = __builtin_bit_cast(bf16x8_t, av[sd][1][1]);
                    // the same slot's operands D steps on (the last steps of a pass ask for the pass's last step again)
                    const int st = 4 * hs + s + D, sn = st < n_steps ? st : n_steps - 1;
                    av[sd][0][0] = pa0[(sn * 2) * 64];
                    av[sd][0][1] = pa0[(sn * 2 + 1) * 64];
                    av[sd][1][0] = pa1[(sn * 2) * 64];
                    av[sd][1][1] = pa1[(sn * 2 + 1) * 64];
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        if (t == 0 || t < nt) {
                            const bf16x8_t bv0 = *(const bf16x8_t *) (bp + t * 32 * MT_BSTRIDE);
                            const bf16x8_t bv1 = *(const bf16x8_t *) (bp + t * 32 * MT_BSTRIDE + 16);
                            acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a00, bv0, acc[0][t], 0, 0, 0);
                            acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a10, bv0, acc[1][t], 0, 0, 0);
                            acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a01, bv1, acc[0][t], 0, 0, 0);
                            acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a11, bv1, acc[1][t], 0, 0, 0);
                        }
                    }
                }
                if (stager) {
                    MT_STAGE_STORE(S::VPT, b0, b1, b2, b3, (uint4 *) (bdst + ((hs + 1) & 1) * (S::TOK * MT_BSTRIDE)));
                }
                __syncthreads();
            }
            if (live) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int tk = tp + 32 * t + l32;
                    if (t < nt && tk < n) {
                        const int64_t col = (int64_t) (a.ids_dst ? a.ids_dst[j0 + tk] : tk) * a.dst_col;
#pragma unroll
                        for (int c = 0; c < (GLU ? 1 : 2); c++) {
                            if (c == 1 && !has1) {
                                continue;
                            }
                            const int64_t row0 = (int64_t) (c ? g1 : g0) * TILE_R + 4 * half;
#pragma unroll
                            for (int g = 0; g < 4; g++) {
                                float v[4];
#pragma unroll
                                for (int i = 0; i < 4; i++) {
                                    const float p = acc[c][t][4 * g + i];
                                    v[i] = GLU ? acc[1][t][4 * g + i] * silu(p) : p;
                                }
                                const int64_t o = col + row0 + 8 * g;
                                if (a.dst_bf16) {
                                    *(uint2 *) ((uint16_t *) a.dst + o) =
                                        make_uint2(f32_to_bf16_rne(v[0]) | ((uint32_t) f32_to_bf16_rne(v[1]) << 16),
                                                   f32_to_bf16_rne(v[2]) | ((uint32_t) f32_to_bf16_rne(v[3]) << 16));
                                } else {
                                    *(float4 *) ((float *) a.dst + o) = make_float4(v[0], v[1], v[2], v[3]);
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}

// Few active experts (decode at small batch): a pass over an expert is one decode chain per wavefront, K / 32 steps
// long, and nothing runs beside it, so the chain is cut instead: WPI wavefronts share a work item (expert, pair of row
// groups, or gate and up of one group), each decodes K / 256 / WPI tiles per chain against its columns of the
// activations, read straight from memory (16 bytes per lane and matrix instruction, one step ahead: no staging, no
// barrier inside the chain), and the partial accumulators are added in K order through LDS (the rings, idle by then).
// Sixteen wavefronts per block: 16 / WPI items.  Passes of 32 tokens; the block runs as many as its busiest item needs.
// WPI is chosen by the block itself once it has listed the active experts: the most wavefronts per item (the
// shortest chains) for which every item of the call runs at once.  The host only knows the routed pairs, an upper
// bound of the active experts that is up to a third too high (tokens share experts), and an item count just above
// what the GPU holds at once doubles the time (a second round of blocks) where the next split down would not.
constexpr int KS_WAVES = 16;

struct ks_ctx {
    uint32_t * lut, * rings, * unit; const int2 * span;
    int n_items, per_expert, groups, slabs;
};

template <bool GLU, int WPI>
__device__ __forceinline__ void ks_items(const bf16n_weight & w, const bf16n_weight & w_up, const mm_args & a, const ks_ctx & c) {
    constexpr int IPB = KS_WAVES / WPI, RPW = 16 / WPI; // items per block; accumulator registers a wavefront adds up
    uint32_t * lut = c.lut;
    uint32_t * rings = c.rings;
    float * part = (float *) rings;                           // [wavefront][register][lane], 6 KB apart
    const uint32_t * unit = c.unit;
    const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31, half = lane >> 5, wave = (int) uniform(tid >> 6);
    const int is = wave / WPI, kw = wave % WPI;               // item of the block, K part
    const int groups = c.groups, per_expert = c.per_expert, n_items = c.n_items, spw = c.slabs / WPI;
    const w64_ptrs q0 = w64p(w), q1 = w64p(GLU ? w_up : w);
    uint32_t * ring = rings + wave * (2 * WAVE_LDS_WORDS);
    // When the launch holds every item at once (always, unless WPI is 1) the items are dealt out evenly over all
    // blocks, fewer than IPB to a block if need be: a block's wavefronts share its SIMDs, and the decode is VALU work
    // (33 active experts: 2 or 3 items on each of 256 CUs instead of 4 on 132 of them).  Else IPB per block, in rounds.
    const int64_t per_round = (int64_t) gridDim.x * IPB;
    // More items than one round holds: dealt out evenly as well, every block taking its share IPB at a time, so that
    // the last round has a few items on every CU rather than full blocks on a few CUs.
    const bool dealt = n_items <= per_round - gridDim.x || n_items > per_round; // (only where that lowers the most items of a block)
    const int first = (int) ((int64_t) blockIdx.x * n_items / gridDim.x);
    const int share = (int) ((int64_t) (blockIdx.x + 1) * n_items / gridDim.x) - first;
    for (int64_t r0 = 0, r = 0; r0 < n_items; r0 += per_round, r++) {
        int base, cnt;
        if (dealt) {
            base = first + (int) r * IPB;
            cnt = share - (int) r * IPB < IPB ? share - (int) r * IPB : IPB;
        } else {
            base = (int) (r0 + (int64_t) blockIdx.x * IPB);
            cnt = n_items - base < IPB ? n_items - base : IPB;
        }
        if (cnt <= 0) { // (the same in every thread of the block)
            continue;
        }
        int maxn = 0;
#pragma unroll
        for (int k = 0; k < IPB; k++) {
            if (k < cnt) {
                const int nk = (int) uniform((uint32_t) c.span[(base + k) / per_expert].y);
                maxn = nk > maxn ? nk : maxn;
            }
        }
        const int item = base + is;
        const bool valid = is < cnt;
        const int at = valid ? item / per_expert : 0, p = valid ? item % per_expert : 0;
        const int e = (int) (uniform(unit[at]) & 0xFFFFu);
        const int j0 = (int) uniform((uint32_t) c.span[at].x), n = valid ? (int) uniform((uint32_t) c.span[at].y) : 0;
        const int g0 = GLU ? p : 2 * p;
        const bool has1 = GLU || g0 + 1 < groups;
        const int g1 = has1 && !GLU ? g0 + 1 : g0;
        for (int tp = 0; tp < maxn; tp += 32) {
            const int tk = tp + l32;
            f32x16_t acc[2];
#pragma unroll
            for (int m = 0; m < 2; m++) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    acc[m][i] = 0.f;
                }
            }
            if (tp < n) {
                // this lane's token (past the item's last: that one again, dropped at the store), its K part and half
                const char * xr = (const char *) (a.x + (int64_t) a.ids_src1[j0 + (tk < n ? tk : n - 1)] * a.x_row + kw * spw * TILE_K) + 16 * half;
                tchain_t<2, true> ch[2];
                // the unit bases of both chains, then the first stream and plane loads of both, then the first
                // activations, and only then the waits: one chain after the other is four memory latencies in a row
                // before the first step (7.4 of a launch's 30 us at four tokens), this order two
                const int64_t u0 = ((int64_t) e * groups + g0) * (WPI * spw) + kw * spw, u1 = ((int64_t) e * groups + g1) * (WPI * spw) + kw * spw;
                const uint32_t f0 = q0.ubase[u0], e0 = q0.ubase[u0 + spw], f1 = q1.ubase[u1], e1 = q1.ubase[u1 + spw];
                ch[0].start(ring, q0, u0, spw, lane, f0, e0, true, true);
                ch[1].start(ring + WAVE_LDS_WORDS, q1, u1, spw, lane, f1, e1, true, true);
                // B operands of a step: columns 32 s + 8 half + [0, 8) and 16 further on
                bf16x8_t nb0 = *(const bf16x8_t *) xr, nb1 = *(const bf16x8_t *) (xr + 32);
                ch[0].dec.start_finish();
                ch[1].dec.start_finish();
#pragma unroll 1
                for (int t = 0; t < spw; t++) {
                ch[0].begin_tile();
                ch[1].begin_tile();
#pragma unroll
                for (int s = 0; s < T_STEPS; s++) {
                    const bf16x8_t bv0 = nb0, bv1 = nb1;
                    const int nq = t * T_STEPS + s + 1;
                    const char * xn = xr + (nq < spw * T_STEPS ? nq : 0) * 64; // after the last step: the first again, unused
                    nb0 = *(const bf16x8_t *) xn;
                    nb1 = *(const bf16x8_t *) (xn + 32);
                    tile_step_mm(ch, lut, GLU ? LUT_WORDS : 0, s, lane, [&](int kb) { return kb ? bv1 : bv0; }, acc[0], acc[1]);
                }
                }
            }
            float r[2][RPW];
            if constexpr (WPI == 1) { // a wavefront has the whole sums
#pragma unroll
                for (int m = 0; m < 2; m++) {
#pragma unroll
                    for (int q = 0; q < RPW; q++) {
                        r[m][q] = acc[m][q];
                    }
                }
            } else {
                __syncthreads(); // every ring is idle: they hold the partial sums now
#pragma unroll
                for (int m = 0; m < 2; m++) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        part[(wave * (2 * WAVE_LDS_WORDS)) + i * 64 + lane] = acc[m][i];
                    }
                    __syncthreads();
#pragma unroll
                    for (int q = 0; q < RPW; q++) {
                        float sum = 0.f;
#pragma unroll
                        for (int k = 0; k < WPI; k++) {
                            sum += part[((is * WPI + k) * (2 * WAVE_LDS_WORDS)) + (kw * RPW + q) * 64 + lane];
                        }
                        r[m][q] = sum;
                    }
                    __syncthreads();
                }
            }
            // accumulator element i of a lane: row 8 (i / 4) + 4 (lane / 32) + i % 4 of the group, token lane % 32
            if (tk < n) {
                const int64_t col = (int64_t) a.ids_dst[j0 + tk] * a.dst_col;
#pragma unroll
                for (int m = 0; m < (GLU ? 1 : 2); m++) {
                    if (m == 1 && !has1) {
                        continue;
                    }
#pragma unroll
                    for (int q = 0; q < RPW; q++) {
                        const int i = kw * RPW + q;
                        const int64_t o = col + (int64_t) (m ? g1 : g0) * TILE_R + 8 * (i >> 2) + 4 * half + (i & 3);
                        const float v = GLU ? r[1][q] * silu(r[0][q]) : r[m][q];
                        if (a.dst_bf16) {
                            ((uint16_t *) a.dst)[o] = f32_to_bf16_rne(v);
                        } else {
                            ((float *) a.dst)[o] = v;
                        }
                    }
                }
            }
        }
    }
}

template <bool GLU>
__global__ void __launch_bounds__(KS_WAVES * 64) k_mm_tile_ks(const bf16n_weight w, const bf16n_weight w_up, const mm_args a) {
    constexpr int NM = GLU ? 2 : 1;
    extern __shared__ __align__(16) uint32_t shm[];
    ks_ctx c;
    c.lut = shm;
    c.rings = shm + NM * LUT_WORDS;
    c.unit = c.rings + KS_WAVES * 2 * WAVE_LDS_WORDS;
    int2 * span = (int2 *) (c.unit + MT_MAX_UNITS + 16); // behind the list and its 16 counters
    c.span = span;
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6);
    // the tables are requested first (one 16-byte load per thread and table) and stored once the block knows that it
    // has work: their way from memory overlaps the listing of the active experts
    static_assert(LUT_WORDS / 4 == KS_WAVES * 64, "one uint4 of a table per thread");
    const uint4 t0 = ((const uint4 *) (w.aux + w.off_a))[threadIdx.x];
    const uint4 t1 = GLU ? ((const uint4 *) (w_up.aux + w_up.off_a))[threadIdx.x] : make_uint4(0, 0, 0, 0);
    c.groups = (int) (a.rows / TILE_R);
    c.per_expert = GLU ? c.groups : (c.groups + 1) / 2;       // items per expert
    c.slabs = (int) (w.K / TILE_K);
    c.n_items = list_units(c.unit, a, wave, lane, KS_WAVES, span) * c.per_expert;
    // the most wavefronts per item for which the launch's blocks hold every item at once
    int wpi = KS_WAVES;
    while (wpi > 1 && (c.slabs % wpi != 0 || (int64_t) c.n_items * wpi > (int64_t) gridDim.x * KS_WAVES)) {
        wpi >>= 1;
    }
    const int ipb = KS_WAVES / wpi;
    if (c.n_items <= (int) gridDim.x * (ipb - 1) ? (int64_t) (blockIdx.x + 1) * c.n_items / gridDim.x == (int64_t) blockIdx.x * c.n_items / gridDim.x
                                                  : (int64_t) blockIdx.x * ipb >= c.n_items) {
        return; // no item for this block (the same in every thread of the block)
    }
    ((uint4 *) c.lut)[threadIdx.x] = t0;
    if (GLU) {
        ((uint4 *) (c.lut + LUT_WORDS))[threadIdx.x] = t1;
    }
    __syncthreads();
    switch (wpi) {
        case 16: ks_items<GLU, 16>(w, w_up, a, c); break;
        case 8: ks_items<GLU, 8>(w, w_up, a, c); break;
        case 4: ks_items<GLU, 4>(w, w_up, a, c); break;
        case 2: ks_items<GLU, 2>(w, w_up, a, c); break;
        default: ks_items<GLU, 1>(w, w_up, a, c); break;
    }
}

// ---------------------------------------------------------------- batched products of experts in the 4-bit code
//
// Experts stored in the reference's NIBBLE layout (rows of all experts stacked) have no decode chain: a wavefront decodes
// any 32 rows x 256 columns it likes, which makes the batched product a plain tiled one.  A block of eight wavefronts
// takes a work item (expert, pass of 32 NT of its tokens, slab of row groups: eight groups with the fused gate / up
// product, sixteen without) and walks K in half chunks of 256 columns.  Wavefront v owns one row group of gate and the
// same of up (or two row groups of the matrix) and their 2 x NT accumulator blocks; per step lane (row r, half h)
// decodes two adjacent slots of its row in each matrix — eight adjacent columns in each of the chunk's four column
// blocks, the A operands of four matrix instructions (k_nib_mm explains the order; here a lane owns four adjacent
// slots, two steps' worth, so that a row's cache line is used up at once) — and the B operands come from the
// pass's activations of these 256 columns, staged in LDS by the whole block (double buffered: one barrier per half
// chunk) in a token-major layout padded so that sixteen tokens meet all banks.  No table and no ring in LDS, so the
// staged activations may take it all.  Escaped weights (decoded as +0) add their exact products before the SwiGLU.
constexpr int NB_WAVES = 8;
constexpr int NB_PAIRS_32 = 12, NB_PAIRS_64 = 40; // routed pairs per expert up to which passes are 32 / 64 tokens long
constexpr int NB_TOK_BYTES = 4 * 128 + 16; // a staged token: four runs of 64 columns, padded
template <int NT> constexpr int nb_stage_bytes() { return 32 * NT * NB_TOK_BYTES; }
template <int NT> size_t nb_shm() { return (size_t) 2 * nb_stage_bytes<NT>() + (size_t) 32 * NT * 4 + (MT_MAX_UNITS + 16) * 4; }

template <bool GLU, int NT>
__global__ void __launch_bounds__(NB_WAVES * 64, NT == 1 ? 2 : 1) k_nib_mm_ids(const bf16n_weight w, const bf16n_weight w_up, const mm_args a) {
    constexpr int TOK = 32 * NT, STAGE = nb_stage_bytes<NT>();
    constexpr int GPI = GLU ? NB_WAVES : 2 * NB_WAVES; // row groups per work item
    constexpr int SV = TOK * 32 / (NB_WAVES * 64);      // uint4 a thread stages per half chunk: 32 per token
    extern __shared__ __align__(16) char nb_lds[];
    char * stage = nb_lds;                              // [2][TOK][NB_TOK_BYTES]
    int * tok_row = (int *) (nb_lds + 2 * STAGE);       // [TOK]: the activation row of every token of the pass
    uint32_t * unit = (uint32_t *) (tok_row + TOK);
    const nib_ptrs q0 = nibp(w, 0), q1 = nibp(GLU ? w_up : w, 0);
    const int K = (int) w.K, halves = K / 256;
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, h = lane >> 5, wave = (int) uniform(tid >> 6);
    const int groups = (int) (a.rows / 32), slabs = (groups + GPI - 1) / GPI;
    const int n_units = list_units<TOK>(unit, a, wave, lane, NB_WAVES);
    for (int item = blockIdx.x; item < n_units * slabs; item += gridDim.x) {
        const uint32_t un = uniform(unit[item / slabs]);
        const int e = (int) (un & 0xFFFFu), sl = item % slabs;
        const int j0 = a.bounds[e] + TOK * (int) (un >> 16);
        const int left = a.bounds[e + 1] - j0, n = left < TOK ? left : TOK, nt = (n + 31) >> 5;
        __syncthreads(); // the item before is done with tok_row and the staging buffers
        if (tid < TOK) {
            tok_row[tid] = a.ids_src1[j0 + (tid < n ? tid : n - 1)];
        }
        __syncthreads();
        const int g0 = GLU ? sl * GPI + wave : sl * GPI + 2 * wave;
        const bool live = g0 < groups, has1 = GLU || g0 + 1 < groups;
        const int g1 = GLU || !has1 ? g0 : g0 + 1;
        const int64_t row0 = (int64_t) e * a.rows + (live ? g0 : 0) * 32 + r, row1 = (int64_t) e * a.rows + (live ? g1 : 0) * 32 + r;
        const uint4 T0 = *(const uint4 *) (q0.table + row0 * 16), T1 = *(const uint4 *) (q1.table + row1 * 16);
        // a lane takes four adjacent slots of its row at a time, 64 plane bytes and 32 code bytes, the two halves of a
        // row's 128-byte line in the same load instructions: taken 32 bytes at a time, a step apart, every line came from
        // HBM twice at 2,048 tokens (FETCH_SIZE 1.92 GB for 0.83 GB of weights: neither L1 nor L2 kept it that long)
        const uint8_t * pl0 = q0.plane + row0 * K + 64 * h, * pl1 = q1.plane + row1 * K + 64 * h;
        const uint8_t * cd0 = q0.codes + row0 * (K / 2) + 32 * h, * cd1 = q1.codes + row1 * (K / 2) + 32 * h;
        // staging: uint4 v of this thread is part (index % 8) of column block (index / 8 % 4) of token index / 32
        const char * sx[SV];
        int so[SV];
#pragma unroll
        for (int v = 0; v < SV; v++) {
            const int idx = tid + NB_WAVES * 64 * v, tok = idx >> 5, jb = (idx >> 3) & 3, part = idx & 7;
            sx[v] = (const char *) (a.x + (int64_t) tok_row[tok] * a.x_row) + 256 * jb + 16 * part;
            so[v] = tok * NB_TOK_BYTES + 128 * jb + 16 * part;
        }
        f32x16_t acc[2][NT];
#pragma unroll
        for (int m = 0; m < 2; m++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    acc[m][t][i] = 0.f;
                }
            }
        }
        // the weights of the first pair of steps: per matrix four slots of 16 plane bytes and their 32 code bytes
        uint4 pa[12];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            pa[k] = *(const uint4 *) (pl0 + 16 * k);
            pa[6 + k] = *(const uint4 *) (pl1 + 16 * k);
        }
#pragma unroll
        for (int k = 0; k < 2; k++) {
            pa[4 + k] = *(const uint4 *) (cd0 + 16 * k);
            pa[10 + k] = *(const uint4 *) (cd1 + 16 * k);
        }
        {   // the first half chunk's activations
            uint4 f[SV];
#pragma unroll
            for (int v = 0; v < SV; v++) {
                f[v] = *(const uint4 *) sx[v];
            }
#pragma unroll
            for (int v = 0; v < SV; v++) {
                *(uint4 *) (stage + so[v]) = f[v];
            }
        }
        __syncthreads();
#pragma unroll 1
        for (int hc = 0; hc < halves; hc++) {
            const char * bcur = stage + (hc & 1) * STAGE;
            // the next half chunk's activations: requested now, stored after this one's steps (after the last half
            // chunk the same one again, into the buffer nobody reads any more)
            const int nx = hc + 1 < halves ? hc + 1 : hc;
            uint4 f[SV];
#pragma unroll
            for (int v = 0; v < SV; v++) {
                f[v] = *(const uint4 *) (sx[v] + 2 * ((nx >> 1) * 512 + 64 * (nx & 1)));
            }
            if (live) {
#pragma unroll
                for (int d = 0; d < 2; d++) {
                    // pair p = 2 hc + d of steps takes the plane bytes [128 p, +128) and the code bytes [64 p, +64) of the
                    // row (two lanes); its loads were issued a pair ago, and those of pair p + 1 go out now
                    // (128-token passes have no registers for a pair ahead: they load the pair they are at, and the
                    // matrix instructions of the pair before cover the wait)
                    const int p = 2 * hc + d;
                    uint4 cur[12];
                    if constexpr (NT != 4) {
#pragma unroll
                        for (int k = 0; k < 12; k++) {
                            cur[k] = pa[k];
                        }
                    }
                    const int pn = NT == 4 ? p : p + 1 < 2 * halves ? p + 1 : p; // past the end: this pair's again, unused
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        pa[k] = *(const uint4 *) (pl0 + 128 * pn + 16 * k);
                        pa[6 + k] = *(const uint4 *) (pl1 + 128 * pn + 16 * k);
                    }
#pragma unroll
                    for (int k = 0; k < 2; k++) {
                        pa[4 + k] = *(const uint4 *) (cd0 + 64 * pn + 16 * k);
                        pa[10 + k] = *(const uint4 *) (cd1 + 64 * pn + 16 * k);
                    }
                    if constexpr (NT == 4) {
#pragma unroll
                        for (int k = 0; k < 12; k++) {
                            cur[k] = pa[k];
                        }
                    }
#pragma unroll
                    for (int st = 0; st < 2; st++) { // the pair's steps: slots 2 st, 2 st + 1 of the lane's four
                        uint32_t wa[2][8], wb[2][8]; // [matrix]: the step's first and second slot
#pragma unroll
                        for (int m = 0; m < 2; m++) {
                            const uint4 ck = cur[6 * m + 4 + st];
                            nib_chunk(cur[6 * m + 2 * st], make_uint2(ck.x, ck.y), m ? T1 : T0, wa[m]);
                            nib_chunk(cur[6 * m + 2 * st + 1], make_uint2(ck.z, ck.w), m ? T1 : T0, wb[m]);
                        }
#pragma unroll
                        for (int jb = 0; jb < 4; jb++) {
                            const u32x4_t a0 = {wa[0][2 * jb], wa[0][2 * jb + 1], wb[0][2 * jb], wb[0][2 * jb + 1]};
                            const u32x4_t a1 = {wa[1][2 * jb], wa[1][2 * jb + 1], wb[1][2 * jb], wb[1][2 * jb + 1]};
#pragma unroll
                            for (int t = 0; t < NT; t++) {
                                if (t == 0 || t < nt) {
                                    const bf16x8_t bv = *(const bf16x8_t *) (bcur + (32 * t + r) * NB_TOK_BYTES + 128 * jb + 64 * d + 32 * h + 16 * st);
                                    acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a0), bv, acc[0][t], 0, 0, 0);
                                    acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a1), bv, acc[1][t], 0, 0, 0);
                                }
                            }
                        }
                    }
                }
            }
            char * bn = stage + ((hc + 1) & 1) * STAGE;
#pragma unroll
            for (int v = 0; v < SV; v++) {
                *(uint4 *) (bn + so[v]) = f[v];
            }
            __syncthreads();
        }
        if (!live) {
            continue;
        }
        // the exact products of escaped weights; accumulator element i of a lane: row 8 (i / 4) + 4 h + i % 4, token 32 t + r
#pragma unroll
        for (int m = 0; m < 2; m++) {
            const nib_ptrs & q = m ? q1 : q0;
            const int64_t gr0 = (int64_t) e * a.rows + (m && !GLU ? g1 : g0) * 32;
            if (uniform(q.esc_off[gr0 + 32] - q.esc_off[gr0]) == 0) {
                continue;
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t gr = gr0 + 8 * (i >> 2) + 4 * h + (i & 3);
                for (uint32_t k = q.esc_off[gr]; k < q.esc_off[gr + 1]; k++) {
                    const uint32_t rec = q.esc[k];
                    const float wv = bf16_bits_to_f32(esc_bits(rec));
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        if (t < nt) {
                            const uint16_t xv = a.x[(int64_t) tok_row[32 * t + r] * a.x_row + (rec & 0xFFFu)];
                            acc[m][t][i] = fmaf(wv, bf16_bits_to_f32(xv), acc[m][t][i]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int tk = 32 * t + r;
            if (t < nt && tk < n) {
                const int64_t col = (int64_t) a.ids_dst[j0 + tk] * a.dst_col;
#pragma unroll
                for (int m = 0; m < (GLU ? 1 : 2); m++) {
                    if (m == 1 && !has1) {
                        continue;
                    }
                    const int64_t rbase = (int64_t) (m ? g1 : g0) * 32 + 4 * h;
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        float v[4];
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float pv = acc[m][t][4 * g + i];
                            v[i] = GLU ? acc[1][t][4 * g + i] * silu(pv) : pv;
                        }
                        const int64_t o = col + rbase + 8 * g;
                        if (a.dst_bf16) {
                            *(uint2 *) ((uint16_t *) a.dst + o) =
                                make_uint2(f32_to_bf16_rne(v[0]) | ((uint32_t) f32_to_bf16_rne(v[1]) << 16),
                                           f32_to_bf16_rne(v[2]) | ((uint32_t) f32_to_bf16_rne(v[3]) << 16));
                        } else {
                            *(float4 *) ((float *) a.dst + o) = make_float4(v[0], v[1], v[2], v[3]);
                        }
                    }
                }
            }
        }
    }
}

size_t ks_shm(bool glu) { // tables, rings, list of active experts + counters, their spans
    return (size_t) (glu ? 2 : 1) * LUT_WORDS * 4 + (size_t) KS_WAVES * 2 * WAVE_LDS_WORDS * 4 + (MT_MAX_UNITS + 16) * 4 +
           (size_t) MT_MAX_UNITS * 8;
}

template <int NT, int W> size_t mt_shm(bool glu) {
    using S = mt_shape<NT, W>;
    return (size_t) (glu ? 2 : 1) * LUT_WORDS * 4 + (size_t) S::WAVES * 2 * WAVE_LDS_WORDS * 4 + (size_t) 2 * S::TOK * MT_BSTRIDE * 2 +
           (MT_MAX_UNITS + 16) * 4;
}

// ---------------------------------------------------------------- GEMV

// 8 consecutive activations as FP32
template <typename TX> struct x8;
template <> struct x8<bf16_t> {
    uint4 r;
    __device__ __forceinline__ void load(const char * x, int k) { r = *(const uint4 *) (x + 2 * (int64_t) k); }
    __device__ __forceinline__ float dot(const uint32_t * wp, float acc) const {
        const uint32_t xw[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            acc = dot2_bf16(wp[i], xw[i], acc);
        }
        return acc;
    }
};
template <> struct x8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const char * x, int k) {
        a = *(const float4 *) (x + 4 * (int64_t) k);
        b = *(const float4 *) (x + 4 * (int64_t) k + 16);
    }
    __device__ __forceinline__ float dot(const uint32_t * wp, float acc) const {
        const float xv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            acc = fmaf(__uint_as_float(wp[i] << 16), xv[2 * i], acc);
            acc = fmaf(__uint_as_float(wp[i] & 0xFFFF0000u), xv[2 * i + 1], acc);
        }
        return acc;
    }
};

constexpr int TV_WAVES = 16;
// wavefronts per block: 16 (128 registers each) where gate and up run on separate wavefronts with BF16 activations,
// else 8 (FP32 activations take twice the registers)
template <typename TX, bool GLU>
constexpr int tv_max_waves() { return GLU && sizeof(TX) == 2 ? TV_WAVES : TV_WAVES / 2; }

// A block covers `gpb` row groups of one column.  Each wavefront runs one decode chain — `upw` consecutive tiles of
// one matrix (at decode a launch is a few hundred tiles and its time is the length of a chain: one short chain per
// wavefront, many wavefronts) — and the partial sums (one per lane and row) of a group's `wpg` wavefronts per matrix
// are added in tile order.  GLU: the group has wpg wavefronts on the gate matrix and wpg on the up matrix, and the
// block writes silu(gate x) * (up x).
// TOPK: the launch selects the experts itself (the router's softmax + top-k would otherwise be a launch of one
// wavefront between the router's GEMV and this one).  Wavefront 0 of every block selects for the block's token from the
// logits while the block stages its tables, and leaves the k ids in LDS; slots from k on (experts every token uses)
// come from the id rows as before.  The first block of every token also writes the ids and weights to the rows that
// the following launches read.  Every block of a token computes the same selection: the same function on the same
// logits as k_router_topk.
template <typename TX, bool GLU, bool ONCE, bool TOPK = false>
__global__ void __launch_bounds__((tv_max_waves<TX, GLU>()) * 64) k_tile_mmv(const bf16n_weight w, const bf16n_weight w_up, const cols p, int wpg, int upw,
                                                                             const topk_args ta = {}) {
    constexpr int NM = GLU ? 2 : 1;
    constexpr int NQ = 4; // the fused selection takes up to 256 experts
    __shared__ __align__(16) uint32_t lut[NM * LUT_WORDS];
    __shared__ float part[TV_WAVES][32];
    __shared__ int32_t sel_id[64];
    __shared__ float sel_w[64];
    extern __shared__ __align__(16) uint32_t rings[];
    const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31, half = lane >> 5, wave = (int) uniform(tid >> 6);
    const int slabs = (int) (w.K / TILE_K), wpgm = NM * wpg, gpb = (int) (blockDim.x >> 6) / wpgm;
    const int gi = wave / wpgm, m = (wave % wpgm) / wpg, wi = wave % wpg; // group in the block, matrix, position in K
    col_view cv;
    if constexpr (TOPK) {
        const int t = (int) blockIdx.y / p.n_used, slot = (int) blockIdx.y % p.n_used;
        float val[NQ];
        bool open[NQ];
        int32_t given = 0;
        if (wave == 0) {
            topk_load<NQ>(ta.logits + (int64_t) t * ta.stride, ta.n_experts, lane, val, open); // in flight beside the tables
        }
        if (slot >= ta.k) {
            given = *(const int32_t *) (p.ids + t * p.ids_s1 + slot * p.ids_s0);
        }
        stage_lut(lut, (const uint32_t *) (w.aux + w.off_a));
        if (GLU) {
            stage_lut(lut + LUT_WORDS, (const uint32_t *) (w_up.aux + w_up.off_a));
        }
        if (wave == 0) {
            topk_select<NQ>(val, open, ta.k, ta.renorm, sel_id, sel_w, lane);
        }
        __syncthreads();
        if (blockIdx.x == 0 && slot == 0 && tid < ta.k) { // the rows the next launches read
            *(int32_t *) (const_cast<char *>(p.ids) + t * p.ids_s1 + tid * p.ids_s0) = sel_id[tid];
            ta.weights[(int64_t) t * ta.out_stride + tid] = sel_w[tid];
        }
        const int e = slot < ta.k ? sel_id[slot] : given;
        cv.x = p.x + t * p.x_tok + (slot % p.x_per_slot) * p.x_slot;
        cv.y = p.y + t * p.y_tok + slot * p.y_slot;
        cv.rbase = p.row0 + (int64_t) e * p.rows_per_matrix;
    } else {
        cv = col_setup(p, blockIdx.y);
    }
    const int64_t groups = p.nrows / TILE_R, g = (int64_t) blockIdx.x * gpb + gi;
    const bool live = gi < gpb && g < groups;
    const w64_ptrs q = w64p(GLU && m ? w_up : w);
    const int64_t unit0 = live ? (cv.rbase / TILE_R + g) * slabs + wi * upw : 0;
    // the unit bases first: the stream loads that depend on them can start as soon as the tables are requested
    const uint32_t first = q.ubase[unit0], end = q.ubase[unit0 + upw];
    tchain_t<4, ONCE> ch[1];
    if (live) {
        ch[0].start(rings + wave * WAVE_LDS_WORDS, q, unit0, upw, lane, first, end, ONCE, !TOPK);
    }
    if constexpr (!TOPK) {
        // the chain's first stream and plane loads travel while the tables are staged
        stage_lut(lut, (const uint32_t *) (w.aux + w.off_a));
        if (GLU) {
            stage_lut(lut + LUT_WORDS, (const uint32_t *) (w_up.aux + w_up.off_a));
        }
        if (live) {
            ch[0].dec.start_finish();
        }
        __syncthreads();
    }
    if (live) {
        const uint32_t * my_lut = lut + m * LUT_WORDS;
        float acc = 0.f;
        for (int u = 0; u < upw; u++) {
            const int k0 = (wi * upw + u) * TILE_K + 8 * half;
            ch[0].begin_tile();
#pragma unroll 1
            for (int hh = 0; hh < 2; hh++) { // two halves of four steps: the step index into the plane registers stays static
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    const int kk = k0 + 32 * (4 * hh + s);
                    // BF16 activations (8 registers a step) are requested before the decode, FP32 ones (16) after it
                    x8<TX> xa, xb;
                    if (sizeof(TX) == 2) {
                        xa.load(cv.x, kk);
                        xb.load(cv.x, kk + 16);
                    }
                    uint32_t wp[1][8];
                    tile_step<1, 4, ONCE>(ch, my_lut, 0, s, wp);
                    ch[0].reload(s, lane);
                    if (sizeof(TX) != 2) {
                        xa.load(cv.x, kk);
                        xb.load(cv.x, kk + 16);
                    }
                    acc = xb.dot(wp[0] + 4, xa.dot(wp[0], acc));
                }
            }
        }
        const float v = acc + __shfl_xor(acc, 32, 64);
        if (half == 0) {
            part[wave][l32] = v;
        }
    }
    __syncthreads();
    if (live && m == 0 && wi == 0 && half == 0) {
        float s[NM];
#pragma unroll
        for (int k = 0; k < NM; k++) {
            s[k] = part[wave + k * wpg][l32];
            for (int i = 1; i < wpg; i++) {
                s[k] += part[wave + k * wpg + i][l32];
            }
        }
        store_y(cv.y, p.y_bf16, g * TILE_R + l32, GLU ? s[NM - 1] * silu(s[0]) : s[0]);
    }
}

// ---------------------------------------------------------------- dequant / row gather

// one step of a tile as exact BF16 (or FP32) values; only_l >= 0: just that row of the tile, to `out`
__device__ __forceinline__ void tile_store_step(const uint32_t (&wp)[8], int s, int l32, int half, int only_l, char * out,
                                                int64_t row_bytes, bool f32) {
    if (only_l >= 0 && l32 != only_l) {
        return;
    }
    char * dst = out + (only_l >= 0 ? 0 : l32) * row_bytes;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int col = tile_col(s, j, half);
        if (f32) {
            *(float4 *) (dst + 4 * col) = make_float4(__uint_as_float(wp[2 * j] << 16), __uint_as_float(wp[2 * j] & 0xFFFF0000u),
                                                      __uint_as_float(wp[2 * j + 1] << 16), __uint_as_float(wp[2 * j + 1] & 0xFFFF0000u));
        } else {
            *(uint2 *) (dst + 2 * col) = make_uint2(wp[2 * j], wp[2 * j + 1]);
        }
    }
}

// decode the `n` tiles from unit0 on (one row group: consecutive column slabs from slab t0) and store them
__device__ __forceinline__ void tile_run(const bf16n_weight & w, const uint32_t * lut, uint32_t * ring, int64_t unit0, int n, int t0,
                                         int lane, int only_l, char * out, int64_t row_bytes, bool f32) {
    const w64_ptrs q = w64p(w);
    tchain ch[1];
    ch[0].start(ring, q, unit0, n, lane);
    for (int u = 0; u < n; u++) {
        ch[0].begin_tile();
#pragma unroll 1
        for (int hh = 0; hh < 2; hh++) {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                uint32_t wp[1][8];
                tile_step<1, 4>(ch, lut, 0, s, wp);
                ch[0].reload(s, lane);
                tile_store_step(wp[0], 4 * hh + s, lane & 31, lane >> 5, only_l, out + (int64_t) (t0 + u) * TILE_K * (f32 ? 4 : 2), row_bytes,
                                f32);
            }
        }
    }
}

// rows [row0, row0 + nrows) (whole row groups) as BF16, row-major; one wavefront per (row group, run of slabs)
__global__ void __launch_bounds__(256) k_tile_dequant(const bf16n_weight w, int64_t row0, int64_t nrows, uint16_t * __restrict__ out) {
    __shared__ __align__(16) uint32_t lut[LUT_WORDS];
    extern __shared__ __align__(16) uint32_t rings[];
    stage_lut(lut, (const uint32_t *) (w.aux + w.off_a));
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int slabs = (int) (w.K / TILE_K);
    const int64_t g = (int64_t) blockIdx.x * nwaves + wave;
    if (g >= nrows / TILE_R) {
        return;
    }
    tile_run(w, lut, rings + wave * WAVE_LDS_WORDS, (row0 / TILE_R + g) * slabs, slabs, 0, lane, -1,
             (char *) (out + g * TILE_R * w.K), w.K * 2, false);
}

__global__ void __launch_bounds__(256) k_tile_get_rows(const bf16n_weight w, const char * __restrict__ ids, int64_t ids_s0, int64_t n,
                                                       int64_t row0, char * __restrict__ dst, int64_t dst_s1, bool f32) {
    __shared__ __align__(16) uint32_t lut[LUT_WORDS];
    extern __shared__ __align__(16) uint32_t rings[];
    stage_lut(lut, (const uint32_t *) (w.aux + w.off_a));
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = (int) uniform(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int slabs = (int) (w.K / TILE_K);
    const int64_t i = (int64_t) blockIdx.x * nwaves + wave;
    if (i >= n) {
        return;
    }
    const int64_t gr = row0 + *(const int32_t *) (ids + i * ids_s0);
    tile_run(w, lut, rings + wave * WAVE_LDS_WORDS, gr / TILE_R * slabs, slabs, 0, lane, (int) (gr % TILE_R), dst + i * dst_s1, 0, f32);
}

} // namespace

bool is_tile_layout(const bf16n_weight & w) {
    return w.format == FMT_HUFPAIR && (w.flags & FLAG_WAVE64) && !(w.flags & FLAG_CHUNK_MAJOR) && w.R == TILE_R;
}

// The batched kernels address their tables by LDS address (two_at), which holds as long as the dynamic segment, whose
// first words the tables are, starts at address 0: the kernel must have no static LDS.  Checked once per kernel here.
void lds_attr(const void * kernel, size_t dynamic_bytes) {
    hipFuncAttributes fa;
    if (hipFuncGetAttributes(&fa, kernel) == hipSuccess && fa.sharedSizeBytes != 0) {
        throw std::logic_error("bf16n: a batched tile kernel has static LDS in front of its tables");
    }
    (void) hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) dynamic_bytes);
}
template <bool GLU, int NT, int W> void mt_attr() { lds_attr((const void *) k_mm_tile<GLU, NT, W>, mt_shm<NT, W>(GLU)); }
template <bool GLU> void ks_attr() { lds_attr((const void *) k_mm_tile_ks<GLU>, ks_shm(GLU)); }

template <bool GLU, int NT> void nb_attr() {
    (void) hipFuncSetAttribute((const void *) k_nib_mm_ids<GLU, NT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) nb_shm<NT>());
}

void tile_init() {
    nb_attr<true, 1>(); nb_attr<false, 1>(); nb_attr<true, 2>(); nb_attr<false, 2>(); nb_attr<true, 4>(); nb_attr<false, 4>();
    mt_attr<true, 4, 8>();
    mt_attr<false, 4, 8>();
    mt_attr<true, 1, 16>();
    mt_attr<false, 1, 16>();
    lds_attr((const void *) k_mm_tile<false, 1, 16, true>, mt_shm<1, 16>(false));
    ks_attr<true>(); ks_attr<false>();
    (void) hipFuncSetAttribute((const void *) k_tile_expand, hipFuncAttributeMaxDynamicSharedMemorySize, EXPAND_WAVES * 2 * WAVE_LDS_WORDS * 4);
    (void) hipFuncSetAttribute((const void *) k_mm_raw<true, 4, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 128 * MT_BSTRIDE * 2);
    (void) hipFuncSetAttribute((const void *) k_mm_raw<false, 4, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 128 * MT_BSTRIDE * 2);
}

template <int W> int64_t mt_items(const mm_args & a, bool glu) {
    const int groups = (int) (a.rows / TILE_R), gpi = glu ? W : 2 * W;
    return (int64_t) a.n_experts * ((groups + gpi - 1) / gpi);
}

template <int NT, int W>
void mt_launch(const bf16n_weight & w, const bf16n_weight * up, const mm_args & a, int cus, hipStream_t stream) {
    using S = mt_shape<NT, W>;
    const int64_t items = mt_items<W>(a, up != nullptr), slots = cus; // the LDS of a CU holds one block
    const dim3 grid((unsigned) (items < slots ? items : slots));
    note_kernel("k_mm_tile", up ? "true" : "false", 2, NT, W);
    if (up) {
        hipLaunchKernelGGL((k_mm_tile<true, NT, W>), grid, dim3(S::THREADS), (mt_shm<NT, W>(true)), stream, w, *up, a);
    } else {
        hipLaunchKernelGGL((k_mm_tile<false, NT, W>), grid, dim3(S::THREADS), (mt_shm<NT, W>(false)), stream, w, w, a);
    }
}

// Passes of 32 tokens.  While the experts that can be active give at most a round of items to the kernel that may
// split K over wavefronts (k_mm_tile_ks: one block per CU, the split chosen on the device from the experts that are
// active), that kernel; else whole experts (or 32 row groups) per block of sixteen wavefronts with the activations
// staged in LDS, which keeps only as many CUs busy as experts are active.  The estimate of the active experts is the
// expectation for uniform routing; when it is too low the K-split kernel runs further rounds, dealt out evenly.
void mt_launch_small(const bf16n_weight & w, const bf16n_weight * up, const mm_args & a, int64_t n_pairs, int cus, hipStream_t stream) {
    const int slabs = (int) (w.K / TILE_K), groups = (int) (a.rows / TILE_R);
    const double e = (double) a.n_experts;
    const double active = std::min((double) n_pairs, e * (1.0 - std::pow(1.0 - 1.0 / e, (double) n_pairs)));
    const double items = active * (up ? groups : (groups + 1) / 2);
    // (a product without the fusion has short items, K / 256 = 2 tiles in the MoE down product, and runs a second
    // round of them well: 130 / 159 / 203 / 227 active experts of 256 took 56 / 60 / 74 / 85 us against 70 / 74 / 80 /
    // 84 us of the staged kernel; the fused gate / up product at one wavefront per item, eight tiles per chain, is ahead
    // of it up to two thirds of a round, level at 0.8 and far behind at 0.9: 107 / 294 us at 173 / 230 active experts)
    const double rounds = up ? 0.75 : 1.5;
    const bool split = a.bounds && a.n_experts <= MT_MAX_LISTED && slabs % 2 == 0 && items <= rounds * (double) cus * KS_WAVES;
    if (split) {
        if (up) {
            hipLaunchKernelGGL((k_mm_tile_ks<true>), dim3((unsigned) cus), dim3(KS_WAVES * 64), ks_shm(true), stream, w, *up, a);
        } else {
            hipLaunchKernelGGL((k_mm_tile_ks<false>), dim3((unsigned) cus), dim3(KS_WAVES * 64), ks_shm(false), stream, w, w, a);
        }
    } else {
        mt_launch<1, 16>(w, up, a, cus, stream);
    }
}

// n_pairs: routed (token, slot) pairs of the call
void launch_tile_mm_ids(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                        const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                        int64_t n_pairs, int cus, hipStream_t stream) {
    mm_args a;
    a.x = (const uint16_t *) x_bf16; a.x_row = x_row;
    a.ids_src1 = ids_src1; a.ids_dst = ids_dst; a.bounds = bounds;
    a.dst = (char *) dst; a.dst_col = dst_col; a.dst_bf16 = dst_bf16;
    a.rows = w.rows / n_experts; a.n_experts = n_experts; a.n_tok = 0;
    if (a.rows % TILE_R != 0) {
        throw std::invalid_argument("bf16n: rows per expert must be a multiple of 32 for the tile layout");
    }
    // passes of 32 tokens while few experts can hold more than 32 (every further pass decodes the expert again)
    if (n_pairs <= (int64_t) MT_SMALL_PAIRS * n_experts) {
        mt_launch_small(w, up, a, n_pairs, cus, stream);
    } else {
        mt_launch<4, 8>(w, up, a, cus, stream);
    }
}

// The two-phase form of launch_tile_mm_ids for calls with many tokens per expert: groups of experts are expanded into
// `scratch` (bytes: at least one expert's tiles of w and up) and multiplied from there, group after group.
uint64_t tile_mm_ids_scratch_per_expert(const bf16n_weight & w, const bf16n_weight * up, int n_experts) {
    return (uint64_t) (w.rows / n_experts) * w.K * 2 * (up ? 2 : 1);
}
void launch_tile_mm_ids_expand(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                               const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                               void * scratch, uint64_t scratch_bytes, int cus, hipStream_t stream) {
    mm_args a;
    a.x = (const uint16_t *) x_bf16; a.x_row = x_row;
    a.ids_src1 = ids_src1; a.ids_dst = ids_dst; a.bounds = bounds;
    a.dst = (char *) dst; a.dst_col = dst_col; a.dst_bf16 = dst_bf16;
    a.rows = w.rows / n_experts; a.n_experts = n_experts; a.n_tok = 0;
    const uint64_t per_expert = tile_mm_ids_scratch_per_expert(w, up, n_experts);
    if (a.rows % TILE_R != 0 || !scratch || ((uintptr_t) scratch & 15) != 0 || scratch_bytes < per_expert) {
        throw std::invalid_argument("bf16n: the two-phase batched product needs rows per expert in multiples of 32 and a 16-byte "
                                    "aligned scratch buffer for at least one expert's tiles as BF16");
    }
    const int slabs = (int) (w.K / TILE_K), groups = (int) (a.rows / TILE_R), tpe = groups * slabs;
    int64_t G = (int64_t) (scratch_bytes / per_expert);
    G = G < n_experts ? G : n_experts;
    // groups of equal size (the last one is not a small remainder)
    const int64_t n_groups = (n_experts + G - 1) / G;
    G = (n_experts + n_groups - 1) / n_groups;
    using S = mt_shape<4, 8>;
    const size_t shm = (size_t) 2 * S::TOK * MT_BSTRIDE * 2;
    for (int64_t e0 = 0; e0 < n_experts; e0 += G) {
        const int n_e = (int) (n_experts - e0 < G ? n_experts - e0 : G);
        const int n_units = n_e * tpe;
        // chains enough for every CU's 32 slots where the group has them; a chain stays inside one expert
        int tpc = 1;
        const int64_t all_tiles = (int64_t) n_units * (up ? 2 : 1), slots = (int64_t) cus * 2 * EXPAND_WAVES;
        while (all_tiles / (tpc * 2) >= slots && tpe % (tpc * 2) == 0) {
            tpc *= 2;
        }
        const int n_chains = (n_units + tpc - 1) / tpc;
        const dim3 grid((unsigned) ((n_chains + 2 * EXPAND_WAVES - 1) / (2 * EXPAND_WAVES)), up ? 2 : 1);
        hipLaunchKernelGGL(k_tile_expand, grid, dim3(EXPAND_WAVES * 64), (size_t) EXPAND_WAVES * 2 * WAVE_LDS_WORDS * 4, stream, w, up ? *up : w,
                           (int64_t) e0 * tpe, n_units, tpc, tpe, bounds, (uint4 *) scratch);
        const uint4 * t0 = (const uint4 *) scratch;
        const uint4 * t1 = up ? t0 + (int64_t) n_units * (TILE_RAW_BYTES / 16) : t0;
        const int64_t items = (int64_t) n_e * ((groups + (up ? 8 : 16) - 1) / (up ? 8 : 16));
        const dim3 g2((unsigned) (items < cus ? items : cus));
        if (up) {
            hipLaunchKernelGGL((k_mm_raw<true, 4, 8>), g2, dim3(S::THREADS), shm, stream, t0, t1, a, (int) e0, n_e, slabs);
        } else {
            hipLaunchKernelGGL((k_mm_raw<false, 4, 8>), g2, dim3(S::THREADS), shm, stream, t0, t1, a, (int) e0, n_e, slabs);
        }
    }
}

// Experts in the 4-bit code (NIBBLE, the rows of all experts stacked): passes of 32, 64 or 128 tokens by the routed pairs
// per expert; blocks stay on their CU and take items in turn (how many there are is known on the device only).
bool nib_mm_ids_ok(const bf16n_weight & w, const bf16n_weight * up) {
    return w.format == FMT_NIBBLE && w.K % 512 == 0 && (!up || (up->format == FMT_NIBBLE && up->rows == w.rows && up->K == w.K));
}

// upper bound of the (expert, pass) units a call lists: one per expert and one per full pass
int64_t nib_mm_ids_units_bound(int n_experts, int64_t n_pairs, int pass_tokens) { return n_experts + n_pairs / pass_tokens; }

template <int NT>
void nb_launch(const bf16n_weight & w, const bf16n_weight * up, const mm_args & a, int cus, hipStream_t stream) {
    const int per_cu = (int) (160 * 1024 / nb_shm<NT>()) < 3 ? (int) (160 * 1024 / nb_shm<NT>()) : 3;
    const dim3 grid((unsigned) (cus * (per_cu < 1 ? 1 : per_cu)));
    if (up) {
        hipLaunchKernelGGL((k_nib_mm_ids<true, NT>), grid, dim3(NB_WAVES * 64), nb_shm<NT>(), stream, w, *up, a);
    } else {
        hipLaunchKernelGGL((k_nib_mm_ids<false, NT>), grid, dim3(NB_WAVES * 64), nb_shm<NT>(), stream, w, w, a);
    }
}

void launch_nib_mm_ids(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                       const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                       int64_t n_pairs, int cus, hipStream_t stream) {
    mm_args a;
    a.x = (const uint16_t *) x_bf16; a.x_row = x_row;
    a.ids_src1 = ids_src1; a.ids_dst = ids_dst; a.bounds = bounds;
    a.dst = (char *) dst; a.dst_col = dst_col; a.dst_bf16 = dst_bf16;
    a.rows = w.rows / n_experts; a.n_experts = n_experts; a.n_tok = 0;
    if (a.rows % 32 != 0 || n_experts > MT_MAX_LISTED) {
        throw std::invalid_argument("bf16n: batched 4-bit-code experts need rows per expert in multiples of 32 and at most 1024 experts");
    }
    // a pass decodes the expert's rows again: long passes where the experts have many tokens.  The units listed are at
    // most one per expert and one per full pass: within MT_MAX_UNITS for up to 32 pairs per expert with the shortest;
    // with the longest the bound depends on the call, and a list that does not fit would leave experts uncomputed.
    const int pass = n_pairs <= (int64_t) NB_PAIRS_32 * n_experts ? 32 : n_pairs <= (int64_t) NB_PAIRS_64 * n_experts ? 64 : 128;
    if (nib_mm_ids_units_bound(n_experts, n_pairs, pass) > MT_MAX_UNITS) {
        throw std::invalid_argument("bf16n: too many routed pairs for one batched call on 4-bit-code experts (experts + pairs / 128 "
                                    "must stay within 2048): split the tokens over several calls");
    }
    if (n_pairs <= (int64_t) NB_PAIRS_32 * n_experts) {
        nb_launch<1>(w, up, a, cus, stream);
    } else if (n_pairs <= (int64_t) NB_PAIRS_64 * n_experts) {
        nb_launch<2>(w, up, a, cus, stream);
    } else {
        nb_launch<4>(w, up, a, cus, stream);
    }
}

// Dense product through the matrix cores: y[j] = W[row0, row0 + nrows) x[j] for ncols BF16 columns (the products of BF16
// values are exact in FP32, the accumulation is FP32).  Strides in elements of x (BF16) and of y.
bool tile_mm_dense_pays(const bf16n_weight & w, int64_t nrows, int cus) {
    // a block takes 32 row groups at a time: worth it when that gives at least half of the CUs a block
    return nrows / (TILE_R * 2 * 16) >= cus / 2 && w.K >= 1024;
}

void launch_tile_mm_dense(const bf16n_weight & w, int64_t row0, int64_t nrows, const void * x, bool x_bf16, int64_t x_row, int ncols,
                          void * y, bool y_bf16, int64_t y_col, int cus, hipStream_t stream) {
    mm_args a;
    a.x = (const uint16_t *) x; a.x_row = x_row;
    a.ids_src1 = a.ids_dst = a.bounds = nullptr;
    a.dst = (char *) y; a.dst_col = y_col; a.dst_bf16 = y_bf16;
    a.rows = nrows; a.n_experts = 1; a.n_tok = x_bf16 ? ncols : 3 * ncols;
    // a view of the row range: the plane bytes and the unit bases of its first tile onwards
    bf16n_weight v = w;
    const int64_t tile0 = row0 / TILE_R * (w.K / TILE_K);
    v.plane += tile0 * T_BYTES;
    v.off_b += (uint64_t) tile0 * 4;
    if (!x_bf16) {
        if (ncols > TILE_DENSE_F32_COLS) {
            throw std::invalid_argument("bf16n: at most 10 FP32 columns per dense tile product");
        }
        using S = mt_shape<1, 16>;
        const int64_t items = mt_items<16>(a, false);
        hipLaunchKernelGGL((k_mm_tile<false, 1, 16, true>), dim3((unsigned) (items < cus ? items : cus)), dim3(S::THREADS),
                           (mt_shm<1, 16>(false)), stream, v, v, a);
    } else if (ncols <= 32) {
        mt_launch<1, 16>(v, nullptr, a, cus, stream);
    } else {
        mt_launch<4, 8>(v, nullptr, a, cus, stream);
    }
}

// y = W x (up == nullptr) or silu(gate x) * (up x), one column per launch row
void launch_tile_mmv(const bf16n_weight & w, const bf16n_weight * up, const cols & p, int ncols, bool x_bf16, hipStream_t stream,
                     const topk_args * topk) {
    if (topk && !(up && x_bf16 && p.ids && p.ids_s0 == 4 && topk->n_experts <= 256 && topk->k <= p.n_used && topk->k <= 64)) {
        throw std::invalid_argument("bf16n: the GEMV that selects its experts takes gate / up tiles, BF16 activations, int32 id rows, "
                                    "at most 256 experts and k <= min(slots, 64)");
    }
    const int slabs = (int) (w.K / TILE_K);
    // wavefronts per row group and matrix: one per tile where the block has room for them, else the fewest tiles per
    // wavefront that fit
    const int nm = up ? 2 : 1, max_waves = up && x_bf16 ? TV_WAVES : TV_WAVES / 2;
    int upw = 1;
    while (slabs % upw != 0 || slabs / upw * nm > max_waves) {
        upw++;
    }
    const int wpg = slabs / upw, wpgm = wpg * nm;
    // blocks of four wavefronts where a row group takes at most four: more, smaller blocks spread a routed GEMV (a
    // few hundred tiles) over more compute units
    const int waves = wpgm <= 4 ? 4 : wpgm <= 8 ? 8 : TV_WAVES, gpb = waves / wpgm;
    const int64_t groups = p.nrows / TILE_R;
    const dim3 grid((unsigned) ((groups + gpb - 1) / gpb), ncols);
    const size_t shm = (size_t) waves * WAVE_LDS_WORDS * 4;
    // one token, or few routed pairs over many experts: (nearly) every tile is read once, by this launch only
    const int64_t n_experts = p.rows_per_matrix > 0 ? w.rows / p.rows_per_matrix : 1;
    const bool once = p.ids ? ncols <= p.n_used || (int64_t) ncols * 4 <= n_experts : ncols == 1;
    const dim3 nt(waves * 64);
#define TILE_MMV(TX, GLU, UP)                                                                                   \
    if (once) {                                                                                                 \
        hipLaunchKernelGGL((k_tile_mmv<TX, GLU, true>), grid, nt, shm, stream, w, UP, p, wpg, upw, topk_args{});  \
    } else {                                                                                                    \
        hipLaunchKernelGGL((k_tile_mmv<TX, GLU, false>), grid, nt, shm, stream, w, UP, p, wpg, upw, topk_args{}); \
    }
    if (topk) { // (every expert of a token is read once: the non-temporal loads)
        hipLaunchKernelGGL((k_tile_mmv<bf16_t, true, true, true>), grid, nt, shm, stream, w, *up, p, wpg, upw, *topk);
    } else if (up) {
        if (x_bf16) {
            TILE_MMV(bf16_t, true, *up)
        } else {
            TILE_MMV(float, true, *up)
        }
    } else if (x_bf16) {
        TILE_MMV(bf16_t, false, w)
    } else {
        TILE_MMV(float, false, w)
    }
#undef TILE_MMV
}

void launch_tile_dequant(const bf16n_weight & w, int64_t row0, int64_t nrows, uint16_t * out, hipStream_t stream) {
    const int64_t groups = nrows / TILE_R;
    hipLaunchKernelGGL(k_tile_dequant, dim3((unsigned) ((groups + 3) / 4)), dim3(256), 4 * WAVE_LDS_WORDS * 4, stream, w, row0, nrows, out);
}

void launch_tile_get_rows(const bf16n_weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16,
                          int64_t dst_s1, int64_t row0, hipStream_t stream) {
    hipLaunchKernelGGL(k_tile_get_rows, dim3((unsigned) ((n + 3) / 4)), dim3(256), 4 * WAVE_LDS_WORDS * 4, stream, w,
                       (const char *) ids, ids_s0, n, row0, (char *) dst, dst_s1, !dst_bf16);
}

} // namespace dev
} // namespace bf16n
