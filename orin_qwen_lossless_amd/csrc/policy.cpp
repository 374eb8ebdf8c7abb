// Shape policy: which format, unit size and layout a weight matrix gets (reference core/src/policy.cpp:9-69).
// The llama and vllm engines reproduce the reference's decisions; mi355x is this build's tuning for 256 CUs of wave64.
#include "encode_impl.h"

namespace bf16n {
namespace impl {

namespace {

// dense matrices: rows per unit.  llama: the largest R in {16, 8, 4, 2} that divides rows and leaves >= 512 units.
// vllm: start from that R and move to a smaller one whenever its cost — waves of 512 units times R — is at least 5 %
// lower (policy.cpp:9-31; the 0.95 comparison is done in double precision there as well).
int dense_unit_rows(int64_t rows, int engine) noexcept {
    int chosen = 1;
    int64_t chosen_cost = 0;
    const int candidates[] = {16, 8, 4, 2};
    for (int r : candidates) {
        if (rows % r != 0 || rows / r < 512) {
            continue;
        }
        const int64_t units = rows / r;
        const int64_t waves = units / 512 + (units % 512 != 0);
        const int64_t cost = waves * r;
        if (chosen == 1) {
            chosen = r;
            chosen_cost = cost;
            if (engine == 0) {
                return chosen;
            }
        } else if ((double) cost <= 0.95 * (double) chosen_cost) {
            chosen = r;
            chosen_cost = cost;
        }
    }
    return chosen;
}

// rows * K * n >= threshold without forming the product (policy.cpp:34-41)
bool reaches(int64_t rows, int64_t K, int64_t n, int64_t threshold) noexcept {
    if (threshold <= 0) {
        return true;
    }
    const int64_t per_matrix = threshold / n + (threshold % n != 0);
    const int64_t rows_needed = per_matrix / K + (per_matrix % K != 0);
    return rows >= rows_needed;
}

// mi355x dense: one wavefront decodes one unit, and 256 CUs hold 4096 wavefronts at once.  A matrix with more rows than
// that streams: it takes the longest units (16 rows: fewest unit starts, fewest bytes).  A smaller one is a single
// round of wavefronts whose time is the length of one unit's decode chain, so it takes the shortest units that still
// fit the round, i.e. the smallest R with rows / R <= 4096 (in hybrid mode the smallest of these units, 4096 weights,
// give way to the 4-bit code: see choose) (measured, K = 2048: 5120 rows 7.9 us with R = 2 against
// 9.2 with R = 4 and 8.9 with R = 1; 2048 x 4096: 6.7 us with R = 1 against 7.7 with R = 2), at 6 % more bytes per
// halving.  Units of at least 4096 weights: every unit ends with about 512 bytes of stream words that were requested
// and never used, one bit per weight at that size (units of 2048 weights compress to 0.82 of BF16 instead of 0.70-0.74).
// The wave64 layout needs whole loop bodies per unit: R a multiple of 4 for K = 512, of 2 for K = 1024.
int mi355x_dense_unit_rows(int64_t rows, int64_t K) noexcept {
    const int64_t C = K / CHUNK;
    const int step = C == 1 ? 4 : C == 2 ? 2 : 1;
    for (int r : {1, 2, 4, 8, 16}) {
        if (r % step == 0 && rows % r == 0 && rows / r <= 4096 && r * K >= 4096) {
            return r;
        }
    }
    for (int r : {16, 8, 4, 2}) {
        if (rows % r == 0) {
            return r;
        }
    }
    return 1;
}

constexpr int64_t MI355X_DENSE_TILE_ROWS = 128 * 1024; // 128 blocks of 32 row groups: half of the CUs

} // namespace

bool choose(int64_t rows, int64_t K, int64_t n, int engine, int mode, int64_t dense_min, bool expert_flag,
            bool dense_frag_order, choice & out) noexcept {
    if (rows <= 0 || n <= 0 || K <= 0 || K % CHUNK != 0 || K > K_MAX) {
        return false;
    }
    const bool vllm = engine == 1, mi355x = engine == 2;
    // llama classifies by the caller's flag, vllm by the stack size (policy.cpp:49); mi355x takes either: a stack of
    // several matrices is an expert stack whatever the caller says, as in every later decision of its branch
    const bool expert = vllm ? n > 1 : mi355x ? (expert_flag || n > 1) : expert_flag;
    if (mode == 2 || (mode == 0 && !expert && !reaches(rows, K, n, dense_min))) {
        out = {FMT_NIBBLE, 0, false, false, false};
        return true;
    }
    const int64_t C = K / CHUNK;
    if (mi355x) {
        int R;
        if (n > 1 && rows % TILE_R == 0) {
            // experts whose row count allows it: 32-row x 256-column tiles in matrix-core operand order.  The batched
            // kernel (more than 8 tokens: prefill, and decode at serving batch sizes) decodes them straight into MFMA
            // operands, about 2x faster than through a tile in LDS; a tile is 8 decode steps, as short a chain for the
            // routed GEMV at decode as the 4-row units below (measured: +2 us on a 47 us MoE layer at batch 1).
            out = {FMT_HUFPAIR, TILE_R, false, false, true};
            return true;
        }
        if (n > 1) {
            // other experts: the reference's rule (policy.cpp:59-61), except that matrices with long rows take units
            // of 4 rows: at decode only top-k experts are read, a routed GEMV is a few hundred units, and its time is
            // the length of one unit's decode chain (8 steps instead of 16; +1.9 % bytes on a 35B-A3B layer)
            R = rows % 16 == 0 && rows >= 2048 ? 16 : rows % 8 == 0 ? 8 : rows % 4 == 0 ? 4 : 1;
            if ((C == 2 || C == 4 || C == 8) && rows % 4 == 0) { // the shapes that get the wave64 layout below
                R = 4;
            }
        } else if (dense_frag_order && rows % TILE_R == 0 && rows >= MI355X_DENSE_TILE_ROWS && K >= 2 * CHUNK) {
            // dense matrices with enough rows to give every CU whole blocks of row groups, when the caller asks for
            // the matrix-core order (the counterpart of the reference's fragment order for dense tensors): products
            // then run on the matrix cores for any batch, 1 to 32 BF16 tokens (10 FP32 tokens, as three BF16
            // components each) in the time of one decode of the matrix.  At batch 1 that is a few per cent behind the
            // 16-row units below with BF16 activations (the tiles are 4 % more bytes), hence on request.
            out = {FMT_HUFPAIR, TILE_R, false, false, true};
            return true;
        } else {
            R = mi355x_dense_unit_rows(rows, K);
            if (mode == 0 && (int64_t) R * K <= 4096 && !reaches(rows, K, 1, dense_min + dense_min / 2)) {
                // a matrix up to half as large again as the dense minimum that fits one round of wavefronts only in
                // units of 4096 weights: such units compress to 0.74 of BF16 (a quarter of their stream is the three
                // start words per lane), the 4-bit code to 0.75, and its GEMV has no decode chain (5120 x 2048 from
                // HBM: 7.3 us against 8.9, 12.7 against 12.6 at four tokens; a 40-layer decode step with qkv and o this
                // way: 55.1 us per layer against 59.7 at one token, 100.7 against 103.5 at four).  Twice the dense
                // minimum is too large for it: 8192 x 2048 takes 10.6 against 10.2 us, 17.4 against 13.5 at four tokens.
                out = {FMT_NIBBLE, 0, false, false, false};
                return true;
            }
        }
        // the wave64 layout where the fused GEMV has an instance (K in {512, 1024, 2048, 4096}, units of whole loop
        // bodies); it is row-major: the batched kernel decodes whole rows per step and needs no chunk-major order.
        // Other shapes keep the reference layout and its rules.
        const bool w64 = (C == 1 && R % 4 == 0) || (C == 2 && R % 2 == 0) || C == 4 || C == 8;
        const bool cm = !w64 && n > 1 && K > CHUNK && (R == 4 || R == 8 || R == 16);
        out = {FMT_HUFPAIR, R, cm, false, w64};
        return true;
    }
    const bool fo_dense = vllm && dense_frag_order && n == 1 && rows % 16 == 0;
    const bool fo_gate_up = vllm && n > 1 && K == 4 * CHUNK && rows % 16 == 0;
    int R;
    if (n > 1) {
        R = fo_gate_up || (rows % 16 == 0 && rows >= 2048) ? 16 : rows % 8 == 0 ? 8 : rows % 4 == 0 ? 4 : 1;
    } else {
        R = fo_dense ? 16 : dense_unit_rows(rows, engine);
    }
    const bool fo_experts = fo_gate_up || (vllm && n > 1 && K == CHUNK && R == 16);
    out = {FMT_HUFPAIR, R, n > 1 && K > CHUNK && !fo_experts, fo_experts || fo_dense, false};
    return true;
}

} // namespace impl
} // namespace bf16n
