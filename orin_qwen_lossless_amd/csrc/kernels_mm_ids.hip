// Batched MoE prefill: dst[ids_dst[j], row] = sum_k W[e, row, k] * x[ids_src1[j], k] for the routed pairs j of every
// expert e (bounds[e] <= j < bounds[e + 1]), optionally dst = silu(gate x) * (up x).  Reference: mm_ids / k_hp_mm_ids,
// core/src/launch.cu:473-535, core/src/kernels.cuh:1162-1505 (BF16 activations, FP32 accumulation on the matrix units).
//
// One block of four wavefronts works on one (expert, slab of 64 rows) at a time and passes over the expert's tokens
// 128 at a time.  For each 512-column chunk the block decodes 32 rows of the slab into a BF16 tile in LDS (the exact
// weights, as in the GEMV kernels: table lookups + v_perm / v_bfi), then every wavefront multiplies the tile with the
// activations of its 32 tokens on the matrix cores (v_mfma_f32_32x32x16_bf16: A = tile rows x 16 columns from LDS,
// B = 16 columns x 32 tokens straight from global memory, 16 bytes per lane).  Decoding happens once per 128 tokens.
//
// Layouts with a batched kernel (the shapes the MoE layers use):
//   * reference chunk-major HUFPAIR, R = 8, K = 2048 (gate / up; also fused gate + up + SwiGLU): a half-wavefront per
//     unit, 8 units per slab;
//   * reference row-major HUFPAIR, R = 16, K = 512 (down): a half-wavefront per unit, 4 units per slab;
//   * wave64 HUFPAIR, R = 4, 8 or 16, K = 512 (down under the mi355x policy): a wavefront per 16 rows, 64 rows per slab;
//   * wave64 HUFPAIR, R = 2, 4 or 8, K = 2048 (gate / up under the mi355x policy): k_mm_ids_w64k below.
#include "dev_common.h"
#include "dev_compat.h"
#include "dev_w64.h"
#include "launchers.h"

#include <stdexcept>

namespace bf16n {
namespace dev {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int MM_THREADS = 256;
constexpr int SLAB_ROWS = 64;     // rows of one expert per work item
constexpr int TILE_ROWS = 32;     // rows decoded per phase: one MFMA block of rows
constexpr int TILE_STRIDE = 520;  // BF16 elements per tile row: 512 + 8 (row stride 1040 bytes spreads rows over banks)
constexpr int TOK_PASS = 128;     // tokens per pass: 32 per wavefront

enum { L_CM8 = 0, L_RM16 = 1, L_W64 = 2, L_W64K = 3 };

struct mm_args {
    const uint16_t * x; int64_t x_row;
    const int32_t * ids_src1, * ids_dst, * bounds;
    char * dst; int64_t dst_col; bool dst_bf16;
    int64_t rows; // per expert
    int n_experts;
};

template <int LAYOUT> struct lay;
template <> struct lay<L_CM8>  { static constexpr int C = 4, R = 8,  UNITS = 8, ROWS_PER_PHASE = 4; };
template <> struct lay<L_RM16> { static constexpr int C = 1, R = 16, UNITS = 4, ROWS_PER_PHASE = 8; };
template <> struct lay<L_W64>  { static constexpr int C = 1, R = 16, UNITS = 4, ROWS_PER_PHASE = 8; };

// 16 weights of one lane (8 BF16 pairs: columns 128 j + 4 l + {0,1}, {2,3}) into row t of the tile
__device__ __forceinline__ void tile_put(uint16_t * tile, int t, int l32, const uint32_t (&wp)[8]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        *(uint2 *) (tile + t * TILE_STRIDE + 128 * j + 4 * l32) = make_uint2(wp[2 * j], wp[2 * j + 1]);
    }
}

// decoder of one matrix inside a work item: the state that persists from phase to phase
template <int LAYOUT>
struct slab_dec {
    lane_bits bits;        // 32-lane layouts
    w64_dec w64;           // wave64 layout
    const uint8_t * plane; // first plane byte of this thread's unit (wave64: of its run of units)
    bool active;
    int unit_steps;        // wave64: steps per unit

    __device__ __forceinline__ void begin(const bf16n_weight & w, int64_t gu0, uint32_t * ring, int tid) {
        using L = lay<LAYOUT>;
        const int lane = tid & 63, l32 = tid & 31;
        if (LAYOUT == L_W64) { // 16 rows per wavefront: a run of 16 / R consecutive units (R = 4, 8 or 16)
            const int run = L::R / w.R;
            const int64_t gu = (gu0 + (tid >> 6)) * run;
            const w64_ptrs q = w64p(w);
            active = true;
            unit_steps = w.R / 2;
            plane = q.plane + gu * w.R * (int64_t) (L::C * CHUNK);
            w64.start(ring + (tid >> 6) * WAVE_LDS_WORDS, q.stream, uniform(q.ubase[gu]), uniform(q.ubase[gu + run]), lane);
        } else {
            const int u = tid >> 5;
            active = u < L::UNITS;
            const int64_t gu = gu0 + (active ? u : 0);
            const hp_ptrs q = hpp(w);
            plane = q.plane + gu * L::R * (int64_t) (L::C * CHUNK);
            bits.begin(q.stream + q.ubase[gu] + q.lrel[gu * 32 + l32]);
        }
    }
    // phase (c, h): the next ROWS_PER_PHASE rows of every unit for chunk c -> 32 tile rows
    __device__ __forceinline__ void phase(const uint32_t * lut, uint16_t * tile, int c, int h, int tid) {
        using L = lay<LAYOUT>;
        const int lane = tid & 63, l32 = tid & 31;
        // the plane words of the whole phase are requested first: the decode below then waits for table lookups only
        if (LAYOUT == L_W64) {
            const int wv = tid >> 6;
            uint4 sm[4];
#pragma unroll
            for (int st = 0; st < 4; st++) {
                sm[st] = *((const uint4 *) (plane + (4 * h + st) * 1024) + lane);
            }
#pragma unroll
            for (int st = 0; st < 4; st++) { // a step holds rows 2 step (lanes 0..31) and 2 step + 1 (lanes 32..63)
                const int step = 4 * h + st;
                uint32_t wp[8];
                w64.keep_ahead();
                if (step % unit_steps == 0) {
                    w64.begin_unit();
                    w64.keep_ahead();
                }
                w64.step(lut, sm[st], wp);
                tile_put(tile, wv * 8 + 2 * st + (lane >> 5), l32, wp);
            }
        } else if (active) {
            const int u = tid >> 5;
            uint4 sm[L::ROWS_PER_PHASE];
#pragma unroll
            for (int i = 0; i < L::ROWS_PER_PHASE; i++) {
                const int rr = L::ROWS_PER_PHASE * h + i;
                const int64_t o = LAYOUT == L_CM8 ? (int64_t) c * L::R + rr : rr; // position of (row, chunk) in the unit
                sm[i] = *((const uint4 *) (plane + o * CHUNK) + l32);
            }
#pragma unroll
            for (int i = 0; i < L::ROWS_PER_PHASE; i++) {
                uint32_t wp[8];
                decode_chunk<FMT_HUFPAIR>(bits, lut, sm[i], wp);
                tile_put(tile, u * L::ROWS_PER_PHASE + i, l32, wp);
            }
        }
    }
};

// row of the slab that tile row t holds in row half h
template <int LAYOUT>
__device__ __forceinline__ int slab_row(int t, int h) {
    using L = lay<LAYOUT>;
    return (t / L::ROWS_PER_PHASE) * L::R + L::ROWS_PER_PHASE * h + t % L::ROWS_PER_PHASE;
}

template <int LAYOUT, bool GLU>
__global__ void __launch_bounds__(MM_THREADS, 2) k_mm_ids(const bf16n_weight w, const bf16n_weight w_up, const mm_args a) {
    using L = lay<LAYOUT>;
    constexpr int NM = GLU ? 2 : 1;
    extern __shared__ __align__(16) uint32_t shm[];
    uint32_t * lut = shm;                                   // NM tables
    uint16_t * tile = (uint16_t *) (shm + NM * LUT_WORDS);  // TILE_ROWS x TILE_STRIDE
    uint32_t * rings = shm + NM * LUT_WORDS + TILE_ROWS * TILE_STRIDE / 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < LUT_WORDS / 4; i += MM_THREADS) {
        ((uint4 *) lut)[i] = ((const uint4 *) (w.aux + w.off_a))[i];
        if (GLU) {
            ((uint4 *) (lut + LUT_WORDS))[i] = ((const uint4 *) (w_up.aux + w_up.off_a))[i];
        }
    }
    const int slabs = (int) (a.rows / SLAB_ROWS);
    const int64_t units_per_expert = a.rows / L::R; // wave64: runs of units that make 16 rows
    for (int item = blockIdx.x; item < a.n_experts * slabs; item += gridDim.x) {
        const int e = item / slabs, sl = item % slabs;
        const int j0 = a.bounds[e], n = a.bounds[e + 1] - j0;
        for (int tp = 0; tp < n; tp += TOK_PASS) {
            // this wavefront's 32 tokens; lanes past the end take the expert's first pair and drop the result
            const int tk = tp + wave * 32 + (lane & 31);
            const bool wave_has = tp + wave * 32 < n, valid = tk < n;
            const int jj = j0 + (valid ? tk : 0);
            const uint16_t * xrow = a.x + (int64_t) a.ids_src1[jj] * a.x_row + 8 * (lane >> 5);
            slab_dec<LAYOUT> dec[NM];
            const int64_t gu0 = e * units_per_expert + (int64_t) sl * L::UNITS;
            dec[0].begin(w, gu0, rings, tid);
            if (GLU) {
                dec[1].begin(w_up, gu0, rings, tid);
            }
            f32x16_t acc[NM][2];
#pragma unroll
            for (int m = 0; m < NM; m++) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        acc[m][h][i] = 0.f;
                    }
                }
            }
#pragma unroll 1
            for (int c = 0; c < L::C; c++) {
                // the activations of this chunk (B operands of its 32 matrix instructions) are requested before the
                // decode and stay in registers for the chunk's phases
                bf16x8_t bv[CHUNK / 16];
#pragma unroll
                for (int ks = 0; ks < CHUNK / 16; ks++) {
                    bv[ks] = *(const bf16x8_t *) (xrow + c * CHUNK + 16 * ks);
                }
#pragma unroll
                for (int h = 0; h < 2; h++) {
#pragma unroll
                    for (int m = 0; m < NM; m++) {
                        __syncthreads(); // the tile is free (and the tables are staged)
                        dec[m].phase(lut + m * LUT_WORDS, tile, c, h, tid);
                        __syncthreads();
                        if (wave_has) {
                            const uint16_t * ap = tile + (lane & 31) * TILE_STRIDE + 8 * (lane >> 5);
#pragma unroll
                            for (int ks = 0; ks < CHUNK / 16; ks++) {
                                const bf16x8_t av = *(const bf16x8_t *) (ap + 16 * ks);
                                acc[m][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv[ks], acc[m][h], 0, 0, 0);
                            }
                        }
                    }
                }
            }
            // accumulator element i of a lane: tile row 8 (i / 4) + 4 (lane / 32) + i % 4, token lane % 32
            if (valid) {
                const int64_t col = (int64_t) a.ids_dst[jj] * a.dst_col + (int64_t) sl * SLAB_ROWS;
#pragma unroll
                for (int h = 0; h < 2; h++) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        float v[4];
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float p = acc[0][h][4 * g + i];
                            v[i] = GLU ? acc[NM - 1][h][4 * g + i] * silu(p) : p;
                        }
                        const int row = slab_row<LAYOUT>(8 * g + 4 * (lane >> 5), h); // four consecutive rows from here
                        if (a.dst_bf16) {
                            uint16_t * d = (uint16_t *) a.dst + col + row;
                            *(uint2 *) d = make_uint2(f32_to_bf16_rne(v[0]) | ((uint32_t) f32_to_bf16_rne(v[1]) << 16),
                                                      f32_to_bf16_rne(v[2]) | ((uint32_t) f32_to_bf16_rne(v[3]) << 16));
                        } else {
                            *(float4 *) ((float *) a.dst + col + row) = make_float4(v[0], v[1], v[2], v[3]);
                        }
                    }
                }
            }
        }
    }
}

// wave64 row-major units of 8 rows, K = 2048 (gate / up under the mi355x policy).  A row-major unit stream yields whole
// rows, so the tile holds 32 full rows (4 units, one per wavefront; 128.5 KiB) and a work item is one decode phase and
// one product phase per matrix; the table in LDS is swapped between gate and up.  One block per CU.
constexpr int WK_ROWS = 32, WK_K = 2048, WK_STRIDE = WK_K + 8, WK_WAVE_ROWS = 8;

// one matrix of a work item: stage its table if needed, decode this wavefront's 8 rows into the tile, multiply
__device__ __forceinline__ void wk_matrix(const bf16n_weight & wm, int m, int & staged, uint32_t * lut, uint16_t * tile, uint32_t * rings,
                                          int64_t gu, int run, int unit_steps, const uint16_t * xrow, bool wave_has, f32x16_t & acc) {
    const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31, wave = tid >> 6;
    __syncthreads(); // tile and table are free
    if (staged != m) {
        stage_lut(lut, (const uint32_t *) (wm.aux + wm.off_a));
        staged = m;
        __syncthreads();
    }
    {   // this wavefront's 8 rows = 16 steps of (row, chunk pair)
        const w64_ptrs q = w64p(wm);
        const uint8_t * plane = q.plane + gu * wm.R * (int64_t) WK_K;
        w64_dec dec;
        dec.start(rings + wave * WAVE_LDS_WORDS, q.stream, uniform(q.ubase[gu]), uniform(q.ubase[gu + run]), lane);
#pragma unroll 1
        for (int s0 = 0; s0 < 2 * WK_WAVE_ROWS; s0 += 4) {
            uint4 sm[4]; // the plane words of four steps, requested before their decode
#pragma unroll
            for (int i = 0; i < 4; i++) {
                sm[i] = *((const uint4 *) (plane + (s0 + i) * 1024) + lane);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int st = s0 + i;
                uint32_t wp[8];
                dec.keep_ahead();
                if (st % unit_steps == 0) {
                    dec.begin_unit();
                    dec.keep_ahead();
                }
                dec.step(lut, sm[i], wp);
                // chunk 2 (st % 2) + lane / 32 of row st / 2
                uint16_t * trow = tile + (wave * WK_WAVE_ROWS + st / 2) * WK_STRIDE + (2 * (st & 1) + (lane >> 5)) * CHUNK;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    *(uint2 *) (trow + 128 * j + 4 * l32) = make_uint2(wp[2 * j], wp[2 * j + 1]);
                }
            }
        }
    }
    __syncthreads();
    if (wave_has) {
        // B operands (activations, 16 bytes per lane and instruction) in two register sets of 8: the next set is
        // requested before the current one is multiplied
        const uint16_t * ap = tile + l32 * WK_STRIDE + 8 * (lane >> 5);
        constexpr int G = 8;
        bf16x8_t bv[2][G];
#pragma unroll
        for (int i = 0; i < G; i++) {
            bv[0][i] = *(const bf16x8_t *) (xrow + 16 * i);
        }
#pragma unroll 2
        for (int g = 0; g < WK_K / 16 / G; g += 2) {
#pragma unroll
            for (int i = 0; i < G; i++) {
                bv[1][i] = *(const bf16x8_t *) (xrow + 16 * ((g + 1) * G + i));
            }
#pragma unroll
            for (int i = 0; i < G; i++) {
                const bf16x8_t av = *(const bf16x8_t *) (ap + 16 * (g * G + i));
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv[0][i], acc, 0, 0, 0);
            }
            if (g + 2 < WK_K / 16 / G) {
#pragma unroll
                for (int i = 0; i < G; i++) {
                    bv[0][i] = *(const bf16x8_t *) (xrow + 16 * ((g + 2) * G + i));
                }
            }
#pragma unroll
            for (int i = 0; i < G; i++) {
                const bf16x8_t av = *(const bf16x8_t *) (ap + 16 * ((g + 1) * G + i));
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv[1][i], acc, 0, 0, 0);
            }
        }
    }
}

template <bool GLU>
__global__ void __launch_bounds__(MM_THREADS) k_mm_ids_w64k(const bf16n_weight w, const bf16n_weight w_up, const mm_args a) {
    extern __shared__ __align__(16) uint32_t shm[];
    uint32_t * lut = shm;
    uint16_t * tile = (uint16_t *) (shm + LUT_WORDS);
    uint32_t * rings = shm + LUT_WORDS + WK_ROWS * WK_STRIDE / 2;
    const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31, wave = tid >> 6;
    const int slabs = (int) (a.rows / WK_ROWS);
    const int run = WK_WAVE_ROWS / w.R, unit_steps = 2 * w.R; // a wavefront decodes 8 rows: a run of 8 / R units (R = 2, 4, 8)
    const int64_t units_per_expert = a.rows / w.R;
    int staged = -1; // which matrix's table is in LDS
    for (int item = blockIdx.x; item < a.n_experts * slabs; item += gridDim.x) {
        const int e = item / slabs, sl = item % slabs;
        const int j0 = a.bounds[e], n = a.bounds[e + 1] - j0;
        for (int tp = 0; tp < n; tp += TOK_PASS) {
            const int tk = tp + wave * 32 + l32;
            const bool wave_has = tp + wave * 32 < n, valid = tk < n;
            const int jj = j0 + (valid ? tk : 0);
            const uint16_t * xrow = a.x + (int64_t) a.ids_src1[jj] * a.x_row + 8 * (lane >> 5);
            const int64_t gu = e * units_per_expert + ((int64_t) sl * (WK_ROWS / WK_WAVE_ROWS) + wave) * run;
            f32x16_t acc_g, acc_u;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                acc_g[i] = 0.f;
                acc_u[i] = 0.f;
            }
            wk_matrix(w, 0, staged, lut, tile, rings, gu, run, unit_steps, xrow, wave_has, acc_g);
            if (GLU) {
                wk_matrix(w_up, 1, staged, lut, tile, rings, gu, run, unit_steps, xrow, wave_has, acc_u);
            }
            if (valid) { // accumulator element i: tile row 8 (i / 4) + 4 (lane / 32) + i % 4 = row of the slab
                const int64_t col = (int64_t) a.ids_dst[jj] * a.dst_col + (int64_t) sl * WK_ROWS;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float v[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float p = acc_g[4 * g + i];
                        v[i] = GLU ? acc_u[4 * g + i] * silu(p) : p;
                    }
                    const int row = 8 * g + 4 * (lane >> 5);
                    if (a.dst_bf16) {
                        *(uint2 *) ((uint16_t *) a.dst + col + row) =
                            make_uint2(f32_to_bf16_rne(v[0]) | ((uint32_t) f32_to_bf16_rne(v[1]) << 16),
                                       f32_to_bf16_rne(v[2]) | ((uint32_t) f32_to_bf16_rne(v[3]) << 16));
                    } else {
                        *(float4 *) ((float *) a.dst + col + row) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                }
            }
        }
    }
}

size_t wk_shm() { return (size_t) LUT_WORDS * 4 + (size_t) WK_ROWS * WK_STRIDE * 2 + 4 * WAVE_LDS_WORDS * 4; }

int layout_of(const bf16n_weight & w) {
    if (w.format != FMT_HUFPAIR || (w.flags & FLAG_FRAG_ORDER)) {
        return -1;
    }
    const bool cm = (w.flags & FLAG_CHUNK_MAJOR) != 0, w64 = (w.flags & FLAG_WAVE64) != 0;
    if (cm && !w64 && w.K == 2048 && w.R == 8) {
        return L_CM8;
    }
    if (!cm && w.K == 512 && (w.R == 16 || (w64 && (w.R == 8 || w.R == 4)))) {
        return w64 ? L_W64 : L_RM16;
    }
    if (!cm && w64 && w.K == WK_K && (w.R == 8 || w.R == 4 || w.R == 2)) {
        return L_W64K;
    }
    return -1;
}

template <int LAYOUT, bool GLU>
size_t mm_shm() {
    return (size_t) (GLU ? 2 : 1) * LUT_WORDS * 4 + (size_t) TILE_ROWS * TILE_STRIDE * 2 + (LAYOUT == L_W64 ? 4 * WAVE_LDS_WORDS * 4 : 0);
}

template <int LAYOUT, bool GLU>
void mm_launch(const bf16n_weight & w, const bf16n_weight * up, const mm_args & a, int blocks, hipStream_t stream) {
    const size_t shm = mm_shm<LAYOUT, GLU>();
    hipLaunchKernelGGL((k_mm_ids<LAYOUT, GLU>), dim3(blocks), dim3(MM_THREADS), shm, stream, w, up ? *up : w, a);
}

} // namespace

void mm_ids_init() {
    (void) hipFuncSetAttribute((const void *) k_mm_ids<L_CM8, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) mm_shm<L_CM8, true>());
    (void) hipFuncSetAttribute((const void *) k_mm_ids<L_CM8, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) mm_shm<L_CM8, false>());
    (void) hipFuncSetAttribute((const void *) k_mm_ids<L_RM16, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) mm_shm<L_RM16, false>());
    (void) hipFuncSetAttribute((const void *) k_mm_ids<L_W64, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) mm_shm<L_W64, false>());
    (void) hipFuncSetAttribute((const void *) k_mm_ids_w64k<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) wk_shm());
    (void) hipFuncSetAttribute((const void *) k_mm_ids_w64k<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) wk_shm());
}

// the reference's rule (launch.cu:446-456) restated for the layouts this build encodes: gate / up in chunk-major
// R = 8 units of K = 2048 (alone or fused with SwiGLU), down in row-major R = 16 units of K = 512
bool mm_ids_shape_ok(const bf16n_weight & w, const bf16n_weight * up) {
    if (w.format == FMT_NIBBLE) { // kernels_tile.hip: experts in the 4-bit code
        return nib_mm_ids_ok(w, up);
    }
    if (is_tile_layout(w)) { // kernels_tile.hip: any K, gate / up of the same shape
        return !up || (is_tile_layout(*up) && up->rows == w.rows && up->K == w.K);
    }
    const int l = layout_of(w);
    if (l < 0) {
        return false;
    }
    if (!up) {
        return true;
    }
    return (l == L_CM8 || l == L_W64K) && layout_of(*up) == l && up->rows == w.rows && up->R == w.R;
}

void launch_mm_ids(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                   const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                   int n_tok, int n_used, int cus, hipStream_t stream) {
    (void) n_tok; (void) n_used;
    mm_args a;
    a.x = (const uint16_t *) x_bf16; a.x_row = x_row;
    a.ids_src1 = ids_src1; a.ids_dst = ids_dst; a.bounds = bounds;
    a.dst = (char *) dst; a.dst_col = dst_col; a.dst_bf16 = dst_bf16;
    a.rows = w.rows / n_experts; a.n_experts = n_experts;
    const int layout = layout_of(w);
    if (a.rows % (layout == L_W64K ? WK_ROWS : SLAB_ROWS) != 0) {
        throw std::invalid_argument("bf16n: no batched kernel for this matrix (rows per expert must be a multiple of 64)");
    }
    if (layout == L_W64K) {
        const int64_t items = (int64_t) n_experts * (a.rows / WK_ROWS);
        const dim3 grid((unsigned) (items < (int64_t) cus ? items : (int64_t) cus));
        const size_t shm = wk_shm();
        if (up) {
            hipLaunchKernelGGL(k_mm_ids_w64k<true>, grid, dim3(MM_THREADS), shm, stream, w, *up, a);
        } else {
            hipLaunchKernelGGL(k_mm_ids_w64k<false>, grid, dim3(MM_THREADS), shm, stream, w, w, a);
        }
        return;
    }
    const int64_t items = (int64_t) n_experts * (a.rows / SLAB_ROWS);
    const int blocks = (int) (items < 2 * (int64_t) cus ? items : 2 * (int64_t) cus);
    switch (layout) {
        case L_CM8:
            if (up) {
                mm_launch<L_CM8, true>(w, up, a, blocks, stream);
            } else {
                mm_launch<L_CM8, false>(w, nullptr, a, blocks, stream);
            }
            break;
        case L_RM16: mm_launch<L_RM16, false>(w, nullptr, a, blocks, stream); break;
        case L_W64:  mm_launch<L_W64, false>(w, nullptr, a, blocks, stream); break;
        default: throw std::invalid_argument("bf16n: no batched kernel for this matrix");
    }
}

} // namespace dev
} // namespace bf16n
