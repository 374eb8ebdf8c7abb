// Shape policy: the reference's C++ interface (core/include/bf16n/policy.h:12-38) over the C ABI.  The llama and vllm
// engines give the reference's answers; `mi355x` is this build's engine (unit sizes for 256 CUs of wave64, the wave64
// stream layout where the shape allows it).
#pragma once

#include "bf16n/detail.h"
#include "bf16n/format.h"

#include <cstdint>
#include <optional>

namespace bf16n {

enum class policy_engine { llama = BF16N_ENGINE_LLAMA, vllm = BF16N_ENGINE_VLLM, mi355x = BF16N_ENGINE_MI355X };
enum class policy_mode { hybrid = BF16N_MODE_HYBRID, huffman = BF16N_MODE_HUFFMAN, nibble = BF16N_MODE_NIBBLE };

struct policy_options {
    policy_engine engine = policy_engine::vllm;
    policy_mode mode = policy_mode::hybrid;
    int64_t dense_min = 8ll << 20;  // dense tensors below this many weights take NIBBLE in hybrid mode
    bool expert = false;            // llama: the loader's "_exps" classification; vllm uses n_matrices > 1 instead;
                                    // mi355x: experts are n_matrices > 1 or this flag
    bool dense_frag_order = false;  // vllm: fragment order for dense tensors; mi355x: matrix-core tiles (R = 32) for
                                    // dense matrices of at least 131072 rows (BF16-activation callers)
};

struct policy_choice {
    int format;
    int R;                   // 0 for NIBBLE
    bool chunk_major;
    bool frag_order = false; // only ever set by the vllm engine
    bool wave64 = false;     // only ever set by the mi355x engine
};

// nullopt: the shape stays BF16 (non-positive sizes, K not a multiple of 512 or above 4096)
inline std::optional<policy_choice> choose(int64_t rows, int64_t K, int64_t n_matrices = 1, policy_options opts = {}) noexcept {
    int out[5] = {0, 0, 0, 0, 0};
    if (!bf16n_choose(rows, K, n_matrices, (int) opts.engine, (int) opts.mode, opts.dense_min, opts.expert ? 1 : 0,
                      opts.dense_frag_order ? 1 : 0, out)) {
        return std::nullopt;
    }
    return policy_choice{out[0], out[1], out[2] != 0, out[3] != 0, out[4] != 0};
}

} // namespace bf16n
