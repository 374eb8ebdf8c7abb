// Launchers of the BF16N kernels: the reference's C++ interface (core/include/bf16n/launch.h:15-85) over the C ABI of
// libbf16n_hip.so, with hipStream_t where the reference has cudaStream_t.  Every call only enqueues kernels on the
// given stream (no allocation, no host synchronisation), so after init() all of them can be captured into HIP graphs.
// Contract violations throw std::invalid_argument("bf16n: ..."), driver errors std::runtime_error.
#pragma once

#include "bf16n/detail.h"
#include "bf16n/format.h"

#include <hip/hip_runtime_api.h>

#include <cstdint>

namespace bf16n {

// device view of one encoded matrix; the metadata comes from the aux header, parsed once on the host
struct weight {
    const uint8_t * plane = nullptr;
    const uint8_t * aux   = nullptr;
    int     format = 0;
    int64_t K = 0, rows = 0;
    int     R = 0;
    bool    cm = false;     // FLAG_CHUNK_MAJOR
    bool    fo = false;     // FLAG_FRAG_ORDER: always refused by this build's launchers
    uint64_t off_a = 0, off_b = 0, off_c = 0, off_d = 0;
    bool    wave64 = false; // FLAG_WAVE64 (this build)
};

// One product per column; see bf16n_mmv_args in bf16n_c.h.  Dense: column = token.  With ids: column = (token, slot),
// expert = ids[token, slot], rows [row0 + expert * rows_per_matrix, + nrows).  Strides are signed bytes.
struct mmv_args {
    const void * x = nullptr; bool x_bf16 = false;
    void * y = nullptr;       bool y_bf16 = false;
    int ncols = 0;
    int64_t x_tok = 0, y_tok = 0;
    const void * ids = nullptr; int64_t ids_s0 = 0, ids_s1 = 0;
    int n_used = 1, x_per_slot = 1;
    int64_t x_slot = 0, y_slot = 0;
    int64_t rows_per_matrix = 0, row0 = 0, nrows = 0;
};

namespace detail {
inline bf16n_weight c_view(const weight & w) {
    bf16n_weight v{};
    v.plane = w.plane; v.aux = w.aux; v.format = w.format; v.R = w.R; v.K = w.K; v.rows = w.rows;
    v.flags = (w.cm ? FLAG_CHUNK_MAJOR : 0u) | (w.fo ? FLAG_FRAG_ORDER : 0u) | (w.wave64 ? FLAG_WAVE64 : 0u);
    v.off_a = w.off_a; v.off_b = w.off_b; v.off_c = w.off_c; v.off_d = w.off_d;
    return v;
}
inline bf16n_mmv_args c_args(const mmv_args & a) {
    bf16n_mmv_args v{};
    v.x = a.x; v.y = a.y; v.ids = a.ids;
    v.x_tok = a.x_tok; v.y_tok = a.y_tok; v.ids_s0 = a.ids_s0; v.ids_s1 = a.ids_s1; v.x_slot = a.x_slot; v.y_slot = a.y_slot;
    v.rows_per_matrix = a.rows_per_matrix; v.row0 = a.row0; v.nrows = a.nrows;
    v.ncols = a.ncols; v.n_used = a.n_used; v.x_per_slot = a.x_per_slot;
    v.x_bf16 = a.x_bf16; v.y_bf16 = a.y_bf16;
    return v;
}
} // namespace detail

// once per process before any launch and before graph capture
inline void init() { detail::check(bf16n_init()); }
inline int sm_count() { int n = 0; detail::check(bf16n_cu_count(&n)); return n; } // compute units of the device
inline int cu_count() { return sm_count(); }

// BF16 token columns up to which mmv is the faster dense path for this matrix; beyond it: dequant + a stock GEMM.
// (8 in the reference, fixed: core/torch/torch_bindings.cpp:195.)
inline int gemv_max_tokens(const weight & w) {
    const bf16n_weight cw = detail::c_view(w);
    int n = 0;
    detail::check(bf16n_gemv_max_tokens(&cw, &n));
    return n;
}

inline void mmv(const weight & w, const mmv_args & a, hipStream_t stream, bool multi_col = true) {
    const bf16n_weight cw = detail::c_view(w);
    const bf16n_mmv_args ca = detail::c_args(a);
    detail::check(bf16n_mmv(&cw, &ca, (void *) stream, multi_col ? 1 : 0));
}
// NIBBLE matrices whose rows_per_matrix rows are [gate (nrows); up (nrows)]: y = silu(gate x) * up x
inline void mmv_glu(const weight & w, const mmv_args & a, hipStream_t stream) {
    const bf16n_weight cw = detail::c_view(w);
    const bf16n_mmv_args ca = detail::c_args(a);
    detail::check(bf16n_mmv_glu(&cw, &ca, (void *) stream));
}
// separate gate and up matrices of the same shape, format and layout; nrows == 0 enqueues nothing
inline void mmv_glu(const weight & gate, const weight & up, const mmv_args & a, hipStream_t stream) {
    const bf16n_weight cg = detail::c_view(gate), cu = detail::c_view(up);
    const bf16n_mmv_args ca = detail::c_args(a);
    detail::check(bf16n_mmv_glu2(&cg, &cu, &ca, (void *) stream));
}
// exact BF16 bits of rows [row0, row0 + nrows) (whole units), row-major
inline void dequant(const weight & w, int64_t row0, int64_t nrows, uint16_t * out, hipStream_t stream) {
    const bf16n_weight cw = detail::c_view(w);
    detail::check(bf16n_dequant(&cw, row0, nrows, out, (void *) stream));
}
// dst[i] = W[row0 + ids[i]], FP32 or BF16, dst_s1 bytes between rows
inline void get_rows(const weight & w, const void * ids, int64_t ids_s0, int64_t n, void * dst, bool dst_bf16, int64_t dst_s1,
                     hipStream_t stream, int64_t row0 = 0) {
    const bf16n_weight cw = detail::c_view(w);
    detail::check(bf16n_get_rows(&cw, ids, ids_s0, n, dst, dst_bf16 ? 1 : 0, dst_s1, (void *) stream, row0));
}

// batched MUL_MAT_ID (prefill): routing lists by mm_ids_route, then one grouped product per launch of mm_ids
inline bool mm_ids_supported(const weight & w, const weight * up) {
    const bf16n_weight cw = detail::c_view(w);
    bf16n_weight cu{};
    if (up) {
        cu = detail::c_view(*up);
    }
    return bf16n_mm_ids_supported(&cw, up ? &cu : nullptr) != 0;
}
inline void mm_ids_route(const void * ids, bool ids_i64, int64_t ids_row_stride, int32_t * ids_src1, int32_t * ids_dst,
                         int32_t * bounds, int n_experts, int n_tok, int n_used, int nchannels_y, int sis1, hipStream_t stream) {
    detail::check(bf16n_mm_ids_route(ids, ids_i64 ? 1 : 0, ids_row_stride, ids_src1, ids_dst, bounds, n_experts, n_tok, n_used,
                                     nchannels_y, sis1, (void *) stream));
}
inline void mm_ids(const weight & w, const weight * up, const void * x_bf16, int64_t x_row, const int32_t * ids_src1,
                   const int32_t * ids_dst, const int32_t * bounds, void * dst, bool dst_bf16, int64_t dst_col, int n_experts,
                   int n_tok, int n_used, hipStream_t stream) {
    const bf16n_weight cw = detail::c_view(w);
    bf16n_weight cu{};
    if (up) {
        cu = detail::c_view(*up);
    }
    detail::check(bf16n_mm_ids(&cw, up ? &cu : nullptr, x_bf16, x_row, ids_src1, ids_dst, bounds, dst, dst_bf16 ? 1 : 0, dst_col,
                               n_experts, n_tok, n_used, (void *) stream));
}

inline void moe_combine(const float * ys, const void * w, bool w_bf16, void * y, bool y_bf16, int n_tok, int n_used, int64_t n,
                        hipStream_t stream) {
    detail::check(bf16n_moe_combine(ys, w, w_bf16 ? 1 : 0, y, y_bf16 ? 1 : 0, n_tok, n_used, n, (void *) stream));
}
inline void swiglu(const float * g, const float * u, float * y, int64_t n, hipStream_t stream) {
    detail::check(bf16n_swiglu(g, u, y, n, (void *) stream));
}
// this build: router softmax + top-k on the device (the reference leaves it to the engines)
inline void router_topk(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, bool renorm, int32_t * ids,
                        float * weights, hipStream_t stream) {
    detail::check(bf16n_router_topk(logits, logits_stride, n_tok, n_experts, k, renorm ? 1 : 0, ids, weights, (void *) stream));
}

} // namespace bf16n
