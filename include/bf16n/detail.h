// Status code -> exception translation shared by the C++ wrappers over the C ABI.
#pragma once

#include "bf16n_c.h"

#include <stdexcept>
#include <string>

namespace bf16n {
namespace detail {

// BF16N_EINVAL -> std::invalid_argument, anything else non-zero -> std::runtime_error, with the library's message
// (the reference throws the same types with the same texts: core/src/compat.cuh:11-25, core/src/encode.cpp:15-20)
inline void check(int status) {
    if (status == BF16N_OK) {
        return;
    }
    const char * msg = bf16n_last_error();
    if (status == BF16N_EINVAL) {
        throw std::invalid_argument(msg ? msg : "bf16n: invalid argument");
    }
    throw std::runtime_error(msg ? msg : "bf16n: runtime error");
}

} // namespace detail
} // namespace bf16n
