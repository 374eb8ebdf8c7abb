// Kernel launchers (defined in the .hip files), called by the C ABI after argument checks.  They only enqueue work.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "bf16n_c.h"
#include "dev_common.h"

namespace bf16n {
namespace dev {

// The kernel instance the calling thread's last product launcher chose: template name and its integer arguments, set
// by the dispatch code itself (the benchmark names the kernel it timed from here instead of from a string of its own).
struct kernel_note { const char * name; const char * tx; int n_args; int arg[5]; };
extern thread_local kernel_note g_last_kernel;
inline void note_kernel(const char * name, const char * tx, int n_args, int a0 = 0, int a1 = 0, int a2 = 0, int a3 = 0, int a4 = 0) {
    g_last_kernel = {name, tx, n_args, {a0, a1, a2, a3, a4}};
}
template <typename TX> constexpr const char * tx_name() { return sizeof(TX) == 2 ? "bf16_t" : "float"; }

// 32-lane layouts (kernels_compat.hip). glu: 0 plain, 1 merged [gate; up] NIBBLE matrix, 2 separate gate / up matrices
bool nib_mm_pays(const bf16n_weight & w, int64_t nrows, int ncols, int cus);
bool nib_mm16_pays(const bf16n_weight & w, int64_t nrows, int ncols, int cus);
void launch_compat_mmv(const bf16n_weight & w, const bf16n_weight * up, int glu, const cols & p, int ncols, bool x_bf16,
                       int cus, hipStream_t stream, bool matrix_cores = true);
void launch_compat_dequant(const bf16n_weight & w, int64_t row0, int64_t nrows, uint16_t * out, int cus, hipStream_t stream);
void launch_compat_get_rows(const bf16n_weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16,
                            int64_t dst_s1, int64_t row0, hipStream_t stream);

// wave64 layout (kernels_w64.hip)
void w64_init();
bool w64_mmv_supported(const bf16n_weight & w, bool x_bf16);
void launch_w64_mmv(const bf16n_weight & w, const cols & p, int ncols, bool x_bf16, bool multi_col, int cus, hipStream_t stream);
void launch_w64_glu(const bf16n_weight & gate, const bf16n_weight & up, const cols & p, int ncols, bool x_bf16, int cus,
                    hipStream_t stream);
void launch_w64_dequant(const bf16n_weight & w, int64_t row0, int64_t nrows, uint16_t * out, int cus, hipStream_t stream);
void launch_w64_get_rows(const bf16n_weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16,
                         int64_t dst_s1, int64_t row0, hipStream_t stream);

// tile form of the wave64 layout: R = 32, units of 32 rows x 256 columns in matrix-core operand order (kernels_tile.hip)
void tile_init();
bool is_tile_layout(const bf16n_weight & w);
// experts in the 4-bit code through the matrix cores
bool nib_mm_ids_ok(const bf16n_weight & w, const bf16n_weight * up);
void launch_nib_mm_ids(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                       const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                       int64_t n_pairs, int cus, hipStream_t stream);
struct topk_args;
void launch_tile_mmv(const bf16n_weight & w, const bf16n_weight * up, const cols & p, int ncols, bool x_bf16, hipStream_t stream,
                     const topk_args * topk = nullptr);
void launch_tile_dequant(const bf16n_weight & w, int64_t row0, int64_t nrows, uint16_t * out, hipStream_t stream);
void launch_tile_get_rows(const bf16n_weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16,
                          int64_t dst_s1, int64_t row0, hipStream_t stream);
void launch_tile_mm_ids(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                        const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                        int64_t n_pairs, int cus, hipStream_t stream);
uint64_t tile_mm_ids_scratch_per_expert(const bf16n_weight & w, const bf16n_weight * up, int n_experts);
void launch_tile_mm_ids_expand(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                               const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                               void * scratch, uint64_t scratch_bytes, int cus, hipStream_t stream);

bool tile_mm_dense_pays(const bf16n_weight & w, int64_t nrows, int cus);
constexpr int TILE_DENSE_F32_COLS = 10; // FP32 columns per dense tile product: three BF16 components each, 32 per pass
void launch_tile_mm_dense(const bf16n_weight & w, int64_t row0, int64_t nrows, const void * x, bool x_bf16, int64_t x_row, int ncols,
                          void * y, bool y_bf16, int64_t y_col, int cus, hipStream_t stream);

// MoE glue (kernels_moe.hip)
void launch_swiglu(const float * g, const float * u, float * y, int64_t n, int cus, hipStream_t stream);
void launch_moe_combine(const float * ys, const void * w, bool w_bf16, void * y, bool y_bf16, int n_tok, int n_used, int64_t n,
                        hipStream_t stream);
void launch_route(const void * ids, bool ids_i64, int64_t ids_row_stride, int32_t * ids_src1, int32_t * ids_dst, int32_t * bounds,
                  int n_experts, int n_tok, int n_used, int nchannels_y, int sis1, hipStream_t stream);
void launch_router_topk(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                        float * weights, hipStream_t stream);
struct add_norm_args {
    const uint16_t * a, * b, * c;         // [n_tok, n] BF16; b, c may be null
    const float * ys; const void * wts;   // [n_tok, n_used, n] FP32 rows and [n_tok, n_used] weights to combine, or null
    bool wts_bf16; int n_used;
    const uint16_t * gamma;               // [n] BF16 or null
    uint16_t * y_sum, * y_norm;           // [n_tok, n] BF16; y_sum may be null
    int64_t n; float eps;
};
void launch_add_rmsnorm(const add_norm_args & a, int n_tok, hipStream_t stream);
void launch_router_topk_strided(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                                float * weights, int64_t out_stride, hipStream_t stream);
// top-k and the routing lists of launch_route over the first n_slots columns of the id rows in one launch (few tokens)
bool router_topk_route_fits(int n_tok, int n_slots, int n_listed);
void launch_router_topk_route(const float * logits, int64_t stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                              float * weights, int64_t out_stride, int n_slots, int n_listed, int32_t * ids_src1, int32_t * ids_dst,
                              int32_t * bounds, int nchannels_y, int sis1, hipStream_t stream);


// batched MoE prefill (kernels_mm_ids.hip)
void mm_ids_init();
bool mm_ids_shape_ok(const bf16n_weight & w, const bf16n_weight * up);
void launch_mm_ids(const bf16n_weight & w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                   const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                   int n_tok, int n_used, int cus, hipStream_t stream);

} // namespace dev
} // namespace bf16n
