// Internal interface between the host encoder / policy and the C ABI (capi.cpp).
#pragma once

#include "bf16n/format.h"

#include <cstdint>
#include <memory>
#include <new>
#include <utility>
#include <vector>

namespace bf16n {
namespace impl {

// std::allocator whose value-less construct leaves the bytes as they are: a vector of these can be sized without the
// single-threaded zero fill (and page faults) of hundreds of megabytes that the encoder's threads overwrite anyway
template <typename T>
struct uninit_allocator : std::allocator<T> {
    template <typename U> struct rebind { using other = uninit_allocator<U>; };
    template <typename U> void construct(U * p) noexcept { ::new ((void *) p) U; }
    template <typename U, typename... A> void construct(U * p, A &&... a) { ::new ((void *) p) U(std::forward<A>(a)...); }
};
using bytes = std::vector<uint8_t, uninit_allocator<uint8_t>>;

struct encoded_buffers {
    bytes plane; // rows * K sign|mantissa bytes
    bytes aux;   // header + exponent data
    int format = 0;             // format actually produced
    int R = 0;                  // rows per unit, 0 for NIBBLE
};

// throws std::invalid_argument("bf16n encode: ...") on contract violations, std::runtime_error on encoder invariants
encoded_buffers encode(const uint16_t * w, int64_t rows, int64_t K, int format, int R, uint32_t flags);
void set_threads(int n);

struct choice { int format, R; bool chunk_major, frag_order, wave64; };
// false: the shape stays BF16.  engine: 0 llama, 1 vllm, 2 mi355x; mode: 0 hybrid, 1 huffman, 2 nibble
bool choose(int64_t rows, int64_t K, int64_t n_matrices, int engine, int mode, int64_t dense_min, bool expert,
            bool dense_frag_order, choice & out) noexcept;

} // namespace impl
} // namespace bf16n
