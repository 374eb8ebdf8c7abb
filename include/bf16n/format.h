// BF16N byte layout: constants and the aux header shared by the host encoder, the HIP kernels and the Python header
// parser.  Values and field order are those of the reference (core/include/bf16n/format.h:12-51) so that buffers made
// by either implementation are interchangeable; FLAG_WAVE64 and the mi355x policy are additions of this build.
#pragma once

#include <cstdint>

namespace bf16n {

// aux_header::format
constexpr int FMT_NIBBLE  = 1; // 4-bit code per weight into a 16-entry exponent table per row, escape list per row
constexpr int FMT_HUFFMAN = 2; // canonical Huffman over single exponents (fallback: more than 4096 distinct pairs)
constexpr int FMT_HUFPAIR = 3; // canonical Huffman over pairs of adjacent exponents

constexpr uint32_t MAGIC   = 0x4e363142; // bytes "B16N"
constexpr int HUF_LMAX     = 10;         // longest single-exponent code: 1024-entry table
constexpr int HP_LP        = 12;         // longest pair code: 4096-entry table, two codes fit in 32 bits with room to spare
constexpr int HP_MAX_PAIRS = 1 << HP_LP;
constexpr int CHUNK        = 512;        // weights per lane-major chunk; K is a multiple of it
constexpr int K_MAX        = 4096;       // NIBBLE escape records keep the column in 12 bits
constexpr int HEADER_BYTES = 256;
constexpr int LANES        = 32;         // lanes per unit of the reference layouts (16 weights per lane and chunk)

// aux_header::flags
constexpr uint32_t FLAG_CHUNK_MAJOR = 1; // HUFPAIR: a unit's streams and plane go chunk by chunk over its rows
constexpr uint32_t FLAG_FRAG_ORDER  = 2; // reference only (NVIDIA mma fragment order); this build rejects it
// HUFPAIR, this build: 64 lanes per unit, one word-interleaved stream per unit consumed front to back by a wave64.
// The plane is unchanged.  Lanes 0..31 own the even, lanes 32..63 the odd 512-column chunks of the unit in stream
// order (so R * K / 512 must be even); see encode_w64() in csrc/encode.cpp for the stream definition.
constexpr uint32_t FLAG_WAVE64      = 4;
// FLAG_WAVE64 with R = 32: the units are tiles of TILE_R rows x TILE_K columns in the operand order of the 32x32x16
// matrix instruction (lane l: row l % 32, two runs of 8 consecutive columns per step); unit g * (K / 256) + t is the
// tile of row group g and column slab t.  Each tile is stored as a wave64 unit of 16 rows of 512 columns; the element
// mapping is tile32_index() in csrc/encode.cpp.
constexpr int TILE_R = 32, TILE_K = 256;

// First bytes of every aux buffer (the header occupies HEADER_BYTES); offsets are bytes from the aux start.
//   NIBBLE : off_a codes (rows*K/2), off_b row tables (rows*16), off_c u32 esc_off[rows+1], off_d u32 escapes; n_a escapes
//   HUFFMAN: off_a u32 lut[1024], off_b u32 lane_off[units*32] (absolute word), off_c words; n_a units, n_b words
//   HUFPAIR: off_a u32 lut[4096], off_b u32 unit_base[units], off_c u16 lane_rel[units*32], off_d words (16-byte
//            aligned); n_a units, n_b words
//   HUFPAIR + FLAG_WAVE64: off_a u32 lut[4096] indexed by the next 12 stream bits, first bit lowest; off_b u32
//            unit_base[units+1]; off_c unused (= off_d); off_d words; n_a units, n_b words
struct aux_header {
    uint32_t magic, format, K, R;
    uint64_t rows;
    uint64_t off_a, off_b, off_c, off_d;
    uint64_t n_a, n_b;
    uint32_t flags, pad_;
};
static_assert(sizeof(aux_header) == 80, "aux_header is read with struct '<IIIIQQQQQQQII'");

// column inside a chunk of slot s (0..15) of lane l (0..31); the plane keeps it at byte 16*l + s of the chunk
inline constexpr int pos_of(int l, int s) { return 128 * (s >> 2) + 4 * l + (s & 3); }

} // namespace bf16n
