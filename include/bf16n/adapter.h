// Load-time conversion and the registry of resident tensors: the C++ face of the reference's llama.cpp adapter
// (engines/llamacpp/patches/0002-ggml-cuda-thin-BF16N-adapter-over-the-shared-core.patch) over the C ABI, without ggml
// types.  An engine's glue turns its tensor into (data address, rows, K, matrices) and calls these; the launchers of
// bf16n/launch.h then take the weight that lookup() returns.  convert / release allocate and synchronise: load time only.
#pragma once

#include "bf16n/detail.h"
#include "bf16n/launch.h"
#include "bf16n/policy.h"

#include <cstdint>
#include <optional>

namespace bf16n {
namespace adapter {

enum class tag { stay_bf16 = 0, nibble = 1, huffman = 2 }; // the conversion tags of ggml's ABI (GGML_BF16N_*)

// ggml_backend_cuda_bf16n_choose (patch 0002:258-268)
inline tag choose(int64_t rows, int64_t K, int64_t n_matrices, const char * mode, int64_t dense_min, bool expert,
                  policy_engine engine = policy_engine::mi355x) noexcept {
    return (tag) bf16n_adapter_choose(rows, K, n_matrices, mode, dense_min, expert ? 1 : 0, (int) engine);
}

namespace detail {
inline weight cpp_view(const bf16n_weight & c) {
    weight w;
    w.plane = c.plane; w.aux = c.aux; w.format = c.format; w.K = c.K; w.rows = c.rows; w.R = c.R;
    w.cm = (c.flags & FLAG_CHUNK_MAJOR) != 0; w.fo = (c.flags & FLAG_FRAG_ORDER) != 0; w.wave64 = (c.flags & FLAG_WAVE64) != 0;
    w.off_a = c.off_a; w.off_b = c.off_b; w.off_c = c.off_c; w.off_d = c.off_d;
    return w;
}
} // namespace detail

// ggml_backend_cuda_bf16n_convert (patch 0002:271-329): encode, upload (plane into tensor_data, aux into a buffer owned
// by the registry), register under `owner`, decode on the device and compare with the source; the round-trip result
inline bool convert(void * tensor_data, const void * bf16_host, int64_t rows_per_matrix, int64_t K, int64_t n_matrices, tag format,
                    const void * owner, const char * name = "", policy_engine engine = policy_engine::mi355x,
                    bool matrix_core_order = false, bool verbose = true) {
    int ok = 0;
    bf16n::detail::check(bf16n_adapter_convert(tensor_data, bf16_host, rows_per_matrix, K, n_matrices, (int) format, (int) engine,
                                               matrix_core_order ? 1 : 0, owner, name, verbose ? 1 : 0, &ok));
    return ok != 0;
}

struct found {
    weight w;
    int64_t row0; // the row of the tensor that the address is the start of (views of whole rows)
};

// lookup (patch 0002:73-92); nullopt: the address belongs to no registered tensor
inline std::optional<found> lookup(const void * p) {
    bf16n_weight c{};
    int64_t row0 = 0;
    int hit = 0;
    bf16n::detail::check(bf16n_adapter_lookup(p, &c, &row0, &hit));
    if (!hit) {
        return std::nullopt;
    }
    return found{detail::cpp_view(c), row0};
}

inline bool is_registered(const void * p) { return lookup(p).has_value(); } // ggml_cuda_bf16n_is_registered

// ggml_cuda_bf16n_free (patch 0002:121-132): before the owning buffer is freed; the number of tensors dropped
inline int release(const void * owner) {
    int n = 0;
    bf16n::detail::check(bf16n_adapter_release(owner, &n));
    return n;
}

// The dense path above gemv_max_tokens(w) tokens (patch 0002:423-437: exact BF16 reconstruction, then the stock BF16
// GEMM): y (n_tok x rows) = x (n_tok x K) W^T, BF16 in and out, FP32 accumulation; row strides in elements.  Scratch for
// the decoded rows and the GEMM's workspace are the caller's (dense_sizes says how much; also to be called once before
// the first capture), so the call itself allocates nothing.
struct dense_sizes_t { uint64_t scratch_bytes, gemm_workspace_bytes; };
inline dense_sizes_t dense_sizes(const weight & w) {
    const bf16n_weight c = bf16n::detail::c_view(w);
    dense_sizes_t s{};
    bf16n::detail::check(bf16n_linear_dense_sizes(&c, &s.scratch_bytes, &s.gemm_workspace_bytes));
    return s;
}
inline void linear_dense(const weight & w, const uint16_t * x, int64_t x_row, int n_tok, uint16_t * y, int64_t y_row, void * scratch,
                         uint64_t scratch_bytes, void * gemm_workspace, uint64_t gemm_workspace_bytes, hipStream_t stream) {
    const bf16n_weight c = bf16n::detail::c_view(w);
    bf16n::detail::check(bf16n_linear_dense(&c, x, x_row, n_tok, y, y_row, scratch, scratch_bytes, gemm_workspace, gemm_workspace_bytes, stream));
}

inline bool verify_roundtrip(const weight & w, const uint16_t * bf16_host) {
    const bf16n_weight c = bf16n::detail::c_view(w);
    int ok = 0;
    bf16n::detail::check(bf16n_verify_roundtrip(&c, bf16_host, &ok));
    return ok != 0;
}

} // namespace adapter
} // namespace bf16n
