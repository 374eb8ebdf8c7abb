// Host-side BF16N encoder: the reference's C++ interface (core/include/bf16n/encode.h:12-26) over the C ABI of
// libbf16n_hip.so.  Same struct, same argument rules, same exceptions; `wave64` is this build's extra layout request.
#pragma once

#include "bf16n/detail.h"
#include "bf16n/format.h"

#include <cstdint>
#include <vector>

namespace bf16n {

struct encoded {
    std::vector<uint8_t> plane; // one sign|mantissa byte per weight
    std::vector<uint8_t> aux;   // 256-byte header, then the exponent data
    int format;                 // what was produced: a HUFPAIR request may come back as FMT_HUFFMAN
    int R;                      // rows per unit; 0 for FMT_NIBBLE
};

// rows x K BF16 bit patterns, row-major.  K a multiple of 512 in [512, 4096]; NIBBLE takes R = 0 and no layout;
// the Huffman formats take R in {1, 2, 4, 8, 16} dividing rows; chunk_major needs HUFPAIR, K > 512, R in {4, 8, 16};
// frag_order is the reference's NVIDIA operand order and is refused; wave64 (HUFPAIR, row-major, R * K / 512 even)
// asks for the 64-lane stream layout; with it R = 32 (rows a multiple of 32) asks for 32-row x 256-column tiles in the
// operand order of the matrix cores (format.h: TILE_R, TILE_K).  std::invalid_argument on a broken rule,
// std::runtime_error on an encoder invariant.
inline encoded encode(const uint16_t * w, int64_t rows, int64_t K, int format, int R, bool chunk_major, bool frag_order = false,
                      bool wave64 = false) {
    const uint32_t flags = (chunk_major ? FLAG_CHUNK_MAJOR : 0u) | (frag_order ? FLAG_FRAG_ORDER : 0u) | (wave64 ? FLAG_WAVE64 : 0u);
    bf16n_encoded * h = nullptr;
    detail::check(bf16n_encode(w, rows, K, format, R, flags, &h));
    struct guard { bf16n_encoded * p; ~guard() { bf16n_encoded_free(p); } } g{h};
    uint64_t np = 0, na = 0;
    const uint8_t * p = bf16n_encoded_plane(h, &np);
    const uint8_t * a = bf16n_encoded_aux(h, &na);
    return encoded{std::vector<uint8_t>(p, p + np), std::vector<uint8_t>(a, a + na), bf16n_encoded_format(h), bf16n_encoded_R(h)};
}

} // namespace bf16n
