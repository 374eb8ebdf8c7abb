// Host-side BF16N encoder (C++17, std::thread).  Produces the byte layout of the reference encoder
// (core/src/encode.cpp) for NIBBLE, HUFFMAN and HUFPAIR row-/chunk-major, and this build's wave64 stream layout.
//
// Structure: every format is written in two parallel passes straight into the final aux buffer — pass 1 sizes each
// row / unit, a prefix sum places it, pass 2 writes it — so no per-unit buffers are kept and the passes scale over
// all host cores.
#include "encode_impl.h"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>

namespace bf16n {
namespace impl {

namespace {

std::atomic<int> g_threads{0};

int worker_count() {
    const int want = g_threads.load();
    const int hw = (int) std::max(1u, std::thread::hardware_concurrency());
    return want > 0 ? want : std::min(16, hw);
}

// f(begin, end) over [0, n) in blocks handed out dynamically
template <typename F>
void parallel_blocks(int64_t n, int64_t block, F && f) {
    if (n <= 0) {
        return;
    }
    const int64_t nblk = (n + block - 1) / block;
    const int nt = (int) std::min<int64_t>(worker_count(), nblk);
    if (nt <= 1) {
        f(0, n);
        return;
    }
    std::atomic<int64_t> next{0};
    std::vector<std::thread> pool;
    std::exception_ptr err;
    std::atomic<bool> failed{false};
    for (int t = 0; t < nt; t++) {
        pool.emplace_back([&] {
            try {
                for (int64_t b; (b = next.fetch_add(1)) < nblk;) {
                    f(b * block, std::min(n, (b + 1) * block));
                }
            } catch (...) {
                if (!failed.exchange(true)) {
                    err = std::current_exception();
                }
            }
        });
    }
    for (auto & t : pool) {
        t.join();
    }
    if (failed) {
        std::rethrow_exception(err);
    }
}

inline int exp_of(uint16_t v) { return (v >> 7) & 0xFF; }
inline uint8_t sm_of(uint16_t v) { return (uint8_t) (((v >> 15) << 7) | (v & 0x7F)); }

[[noreturn]] void invariant(const char * what) { throw std::runtime_error(std::string("bf16n encode: check failed: ") + what); }

// ---------------------------------------------------------------------------------------------- code construction

// Length-limited Huffman lengths (package-merge, reference core/src/encode.cpp:182-218) by counting instead of symbol
// sets: at each level the chosen items are a prefix of the merged list, the packages among them a prefix of the
// package list, which in turn selects twice as many items one level down; a leaf gains a bit for every level whose
// chosen prefix contains it.  The leaf order for equal weights is whatever std::sort yields for a weight-only
// comparison on the symbols in ascending order, which is what the reference's sort sees.
struct leaf { uint64_t w; int sym; };

std::vector<int> limited_lengths(const std::vector<uint64_t> & freq, int L) {
    std::vector<leaf> leaves;
    for (int s = 0; s < (int) freq.size(); s++) {
        if (freq[s]) {
            leaves.push_back({freq[s], s});
        }
    }
    std::vector<int> len(freq.size(), 0);
    const int n = (int) leaves.size();
    if (n == 0) {
        return len;
    }
    if (n == 1) {
        len[leaves[0].sym] = 1;
        return len;
    }
    std::sort(leaves.begin(), leaves.end(), [](const leaf & a, const leaf & b) { return a.w < b.w; });
    std::vector<std::vector<uint64_t>> wt(L);
    std::vector<std::vector<uint8_t>> is_pk(L);
    wt[0].resize(n);
    is_pk[0].assign(n, 0);
    for (int i = 0; i < n; i++) {
        wt[0][i] = leaves[i].w;
    }
    for (int d = 1; d < L; d++) {
        const auto & prev = wt[d - 1];
        const int np = (int) prev.size() / 2;
        wt[d].reserve(np + n);
        is_pk[d].reserve(np + n);
        int i = 0, j = 0;
        while (i < np || j < n) {
            const bool take_pk = i < np && (j >= n || !(leaves[j].w < prev[2 * i] + prev[2 * i + 1]));
            if (take_pk) {
                wt[d].push_back(prev[2 * i] + prev[2 * i + 1]);
                is_pk[d].push_back(1);
                i++;
            } else {
                wt[d].push_back(leaves[j].w);
                is_pk[d].push_back(0);
                j++;
            }
        }
    }
    int64_t m = 2 * (int64_t) n - 2;
    for (int d = L - 1; d >= 0; d--) {
        m = std::min<int64_t>(m, (int64_t) wt[d].size());
        int64_t p = 0;
        for (int64_t i = 0; i < m; i++) {
            p += is_pk[d][i];
        }
        for (int64_t i = 0; i < m - p; i++) {
            len[leaves[i].sym]++;
        }
        m = 2 * p;
    }
    return len;
}

// canonical code: shorter codes first, equal lengths by ascending symbol (encode.cpp:239-250, 348-358)
std::vector<uint32_t> canonical_codes(const std::vector<int> & len, int L) {
    std::vector<uint32_t> code(len.size(), 0);
    uint32_t c = 0;
    for (int l = 1; l <= L; l++) {
        for (size_t s = 0; s < len.size(); s++) {
            if (len[s] == l) {
                code[s] = c++;
            }
        }
        c <<= 1;
    }
    return code;
}

uint32_t bitrev(uint32_t v, int bits) {
    uint32_t r = 0;
    for (int i = 0; i < bits; i++) {
        r |= ((v >> i) & 1u) << (bits - 1 - i);
    }
    return r;
}

// MSB-first writer into a preallocated word range
struct msb_writer {
    uint32_t * out;
    uint64_t acc = 0;
    int nb = 0;
    void put(uint32_t code, int len) {
        acc = (acc << len) | code;
        nb += len;
        if (nb >= 32) {
            *out++ = (uint32_t) (acc >> (nb - 32));
            nb -= 32;
            acc &= nb ? ((1ull << nb) - 1) : 0;
        }
    }
    void flush() {
        if (nb) {
            *out++ = (uint32_t) (acc << (32 - nb));
        }
    }
};

struct pair_code {
    std::vector<uint8_t> len;   // [65536]
    std::vector<uint16_t> code; // [65536]
    std::vector<uint32_t> lut;  // [4096], entry = e_odd << 23 | e_even << 7 | len
};

// false: more than HP_MAX_PAIRS distinct pairs
bool build_pair_code(const uint16_t * w, int64_t rows, int64_t K, pair_code & pc) {
    std::vector<uint64_t> freq(65536, 0);
    {
        std::mutex mu;
        // at most 64 blocks: every block zeroes and merges a 65536-entry histogram of its own (a block holds fewer
        // than 2^32 pairs: rows * K < 2^37 / 64)
        const int64_t per_block = std::max<int64_t>(256, (rows + 63) / 64);
        parallel_blocks(rows, per_block, [&](int64_t r0, int64_t r1) {
            std::vector<uint32_t> h(65536, 0);
            for (int64_t i = r0 * K; i < r1 * K; i += 2) {
                h[exp_of(w[i]) | exp_of(w[i + 1]) << 8]++;
            }
            std::lock_guard<std::mutex> lk(mu);
            for (int s = 0; s < 65536; s++) {
                freq[s] += h[s];
            }
        });
    }
    int nsym = 0;
    for (uint64_t f : freq) {
        nsym += f != 0;
    }
    if (nsym > HP_MAX_PAIRS) {
        return false;
    }
    const std::vector<int> len = limited_lengths(freq, HP_LP);
    const std::vector<uint32_t> code = canonical_codes(len, HP_LP);
    pc.len.assign(65536, 0);
    pc.code.assign(65536, 0);
    pc.lut.assign(1 << HP_LP, 0);
    for (int s = 0; s < 65536; s++) {
        if (!len[s]) {
            continue;
        }
        pc.len[s] = (uint8_t) len[s];
        pc.code[s] = (uint16_t) code[s];
        const uint32_t ent = ((uint32_t) (s >> 8) << 23) | ((uint32_t) (s & 0xFF) << 7) | (uint32_t) len[s];
        const uint32_t lo = code[s] << (HP_LP - len[s]), hi = (code[s] + 1) << (HP_LP - len[s]);
        std::fill(pc.lut.begin() + lo, pc.lut.begin() + hi, ent);
    }
    return true;
}

// stream order of a unit: o-th 512-column chunk -> (row within the unit, chunk)
inline void chunk_of(int64_t o, int R, int64_t C, bool cm, int & rr, int64_t & c) {
    if (cm) {
        rr = (int) (o % R);
        c = o / R;
    } else {
        rr = (int) (o / C);
        c = o % C;
    }
}

} // namespace

void set_threads(int n) { g_threads.store(n); }

// ---------------------------------------------------------------------------------------------- plane

// byte 16*l + s of a chunk = sign|mantissa of column pos_of(l, s) (encode.cpp:48-62); chunk-major units keep chunk c
// of unit row r at (c*R + r)*512 (encode.cpp:511-524)
void write_plane(const uint16_t * w, int64_t rows, int64_t K, int R, bool cm, uint8_t * plane) {
    const int64_t C = K / CHUNK;
    parallel_blocks(rows, 64, [&](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; r++) {
            for (int64_t c = 0; c < C; c++) {
                const uint16_t * src = w + r * K + c * CHUNK;
                uint8_t * dst = cm ? plane + (r / R) * R * K + (c * R + r % R) * CHUNK : plane + r * K + c * CHUNK;
                for (int j = 0; j < 4; j++) {
                    for (int l = 0; l < 32; l++) {
                        const uint16_t * q = src + 128 * j + 4 * l;
                        uint8_t * o = dst + 16 * l + 4 * j;
                        o[0] = sm_of(q[0]); o[1] = sm_of(q[1]); o[2] = sm_of(q[2]); o[3] = sm_of(q[3]);
                    }
                }
            }
        }
    });
}

// ---------------------------------------------------------------------------------------------- NIBBLE

// per row: table entry 0 = exponent 0, then up to 15 exponents in (0, 128) by falling count, ties to the smaller
// exponent; anything else is an escape record col | sm << 12 | exponent << 20 whose plane byte and code read as +0
// (encode.cpp:94-180, 482-493)
bytes encode_nibble(const uint16_t * w, int64_t rows, int64_t K, uint8_t * plane) {
    const int64_t C = K / CHUNK;
    aux_header h = {};
    h.magic = MAGIC; h.format = FMT_NIBBLE; h.K = (uint32_t) K; h.rows = (uint64_t) rows;
    h.off_a = HEADER_BYTES;
    h.off_b = h.off_a + (uint64_t) (rows * K / 2);
    h.off_c = h.off_b + (uint64_t) rows * 16;
    h.off_d = h.off_c + ((uint64_t) rows + 1) * 4;
    bytes aux(h.off_d, 0);
    std::vector<uint32_t> n_esc(rows + 1, 0);
    auto row_table = [&](const uint16_t * row, uint8_t * table, int8_t * code_of) {
        int hist[256] = {0};
        for (int64_t k = 0; k < K; k++) {
            hist[exp_of(row[k])]++;
        }
        std::fill(code_of, code_of + 256, (int8_t) -1);
        std::fill(table, table + 16, (uint8_t) 0);
        code_of[0] = 0;
        for (int n = 1; n < 16; n++) { // next best unused exponent in (0, 128)
            int best = -1;
            for (int e = 1; e < 128; e++) {
                if (code_of[e] < 0 && hist[e] > 0 && (best < 0 || hist[e] > hist[best])) {
                    best = e;
                }
            }
            if (best < 0) {
                break;
            }
            table[n] = (uint8_t) best;
            code_of[best] = (int8_t) n;
        }
    };
    // pass 1: tables, codes, escape counts
    parallel_blocks(rows, 32, [&](int64_t r0, int64_t r1) {
        int8_t code_of[256];
        for (int64_t r = r0; r < r1; r++) {
            const uint16_t * row = w + r * K;
            row_table(row, aux.data() + h.off_b + r * 16, code_of);
            uint32_t ne = 0;
            for (int64_t c = 0; c < C; c++) {
                uint8_t * nb = aux.data() + h.off_a + (r * C + c) * 256;
                for (int l = 0; l < 32; l++) {
                    uint64_t codes = 0;
                    for (int s = 0; s < 16; s++) {
                        int code = code_of[exp_of(row[c * CHUNK + pos_of(l, s)])];
                        if (code < 0) {
                            ne++;
                            code = 0;
                        }
                        codes |= (uint64_t) code << (4 * s);
                    }
                    std::memcpy(nb + 8 * l, &codes, 8);
                }
            }
            n_esc[r + 1] = ne;
        }
    });
    for (int64_t r = 0; r < rows; r++) {
        n_esc[r + 1] += n_esc[r];
    }
    const uint64_t total_esc = n_esc[rows];
    h.n_a = total_esc;
    aux.resize(h.off_d + std::max<uint64_t>(total_esc, 1) * 4, 0);
    std::memcpy(aux.data(), &h, sizeof(h));
    std::memcpy(aux.data() + h.off_c, n_esc.data(), (size_t) (rows + 1) * 4);
    // pass 2: escape records in (chunk, lane, slot) order, and their plane bytes cleared
    if (total_esc) {
        parallel_blocks(rows, 32, [&](int64_t r0, int64_t r1) {
            for (int64_t r = r0; r < r1; r++) {
                if (n_esc[r + 1] == n_esc[r]) {
                    continue;
                }
                const uint16_t * row = w + r * K;
                const uint8_t * table = aux.data() + h.off_b + r * 16;
                bool in_table[256] = {false};
                in_table[0] = true;
                for (int n = 1; n < 16; n++) {
                    in_table[table[n]] = true; // unused entries are 0
                }
                uint32_t * rec = (uint32_t *) (aux.data() + h.off_d) + n_esc[r];
                for (int64_t c = 0; c < C; c++) {
                    for (int l = 0; l < 32; l++) {
                        for (int s = 0; s < 16; s++) {
                            const int col = (int) (c * CHUNK + pos_of(l, s));
                            const uint16_t v = row[col];
                            if (!in_table[exp_of(v)]) {
                                *rec++ = (uint32_t) col | ((uint32_t) sm_of(v) << 12) | ((uint32_t) exp_of(v) << 20);
                                plane[r * K + c * CHUNK + 16 * l + s] = 0;
                            }
                        }
                    }
                }
            }
        });
    }
    return aux;
}

// ---------------------------------------------------------------------------------------------- HUFFMAN (fallback)

// single-exponent code, 16 symbols per (row, chunk, lane) in slot order, row-major units (encode.cpp:220-312)
bytes encode_huffman(const uint16_t * w, int64_t rows, int64_t K, int R) {
    const int64_t C = K / CHUNK, units = rows / R;
    std::vector<uint64_t> freq(256, 0);
    {
        std::mutex mu;
        parallel_blocks(rows, 256, [&](int64_t r0, int64_t r1) {
            uint64_t hloc[256] = {0};
            for (int64_t i = r0 * K; i < r1 * K; i++) {
                hloc[exp_of(w[i])]++;
            }
            std::lock_guard<std::mutex> lk(mu);
            for (int s = 0; s < 256; s++) {
                freq[s] += hloc[s];
            }
        });
    }
    const std::vector<int> len = limited_lengths(freq, HUF_LMAX);
    const std::vector<uint32_t> code = canonical_codes(len, HUF_LMAX);
    std::vector<uint32_t> lane_words(units * 32);
    parallel_blocks(units, 8, [&](int64_t u0, int64_t u1) {
        for (int64_t u = u0; u < u1; u++) {
            for (int l = 0; l < 32; l++) {
                uint64_t bits = 0;
                for (int64_t r = u * R; r < (u + 1) * R; r++) {
                    for (int64_t c = 0; c < C; c++) {
                        for (int s = 0; s < 16; s++) {
                            bits += len[exp_of(w[r * K + c * CHUNK + pos_of(l, s)])];
                        }
                    }
                }
                lane_words[u * 32 + l] = (uint32_t) ((bits + 31) / 32);
            }
        }
    });
    aux_header h = {};
    h.magic = MAGIC; h.format = FMT_HUFFMAN; h.K = (uint32_t) K; h.R = (uint32_t) R; h.rows = (uint64_t) rows;
    h.off_a = HEADER_BYTES;
    h.off_b = h.off_a + (4u << HUF_LMAX);
    h.off_c = h.off_b + (uint64_t) units * 32 * 4;
    uint64_t n_words = 0;
    std::vector<uint64_t> start(units * 32);
    for (int64_t i = 0; i < units * 32; i++) {
        start[i] = n_words;
        n_words += lane_words[i];
    }
    if (!(n_words + 16 < (1ull << 32))) {
        invariant("n_words + 16 < 2^32");
    }
    h.n_a = (uint64_t) units; h.n_b = n_words;
    bytes aux(h.off_c + (n_words + 16) * 4, 0); // 16 words of decoder lookahead
    std::memcpy(aux.data(), &h, sizeof(h));
    uint32_t * lut = (uint32_t *) (aux.data() + h.off_a);
    for (int s = 0; s < 256; s++) {
        if (len[s]) {
            std::fill(lut + (code[s] << (HUF_LMAX - len[s])), lut + ((code[s] + 1) << (HUF_LMAX - len[s])),
                      (uint32_t) len[s] | ((uint32_t) s << 7));
        }
    }
    uint32_t * lane_off = (uint32_t *) (aux.data() + h.off_b);
    uint32_t * stream = (uint32_t *) (aux.data() + h.off_c);
    parallel_blocks(units, 8, [&](int64_t u0, int64_t u1) {
        for (int64_t u = u0; u < u1; u++) {
            for (int l = 0; l < 32; l++) {
                lane_off[u * 32 + l] = (uint32_t) start[u * 32 + l];
                msb_writer bw{stream + start[u * 32 + l]};
                for (int64_t r = u * R; r < (u + 1) * R; r++) {
                    for (int64_t c = 0; c < C; c++) {
                        for (int s = 0; s < 16; s++) {
                            const int e = exp_of(w[r * K + c * CHUNK + pos_of(l, s)]);
                            bw.put(code[e], len[e]);
                        }
                    }
                }
                bw.flush();
            }
        }
    });
    return aux;
}

// ---------------------------------------------------------------------------------------------- HUFPAIR, 32-lane units

// per unit and lane an MSB-first stream of pair codes, chunks in stream order, slots 0,2,..,14 (encode.cpp:321-439).
// Empty result: too many distinct pairs.
bytes encode_hufpair(const uint16_t * w, int64_t rows, int64_t K, int R, bool cm) {
    pair_code pc;
    if (!build_pair_code(w, rows, K, pc)) {
        return {};
    }
    const int64_t C = K / CHUNK, units = rows / R;
    auto sym_at = [&](int64_t i) { return exp_of(w[i]) | exp_of(w[i + 1]) << 8; };
    std::vector<uint32_t> lane_words(units * 32);
    parallel_blocks(units, 8, [&](int64_t u0, int64_t u1) {
        for (int64_t u = u0; u < u1; u++) {
            uint64_t bits[32] = {0};
            for (int64_t o = 0; o < R * C; o++) {
                int rr; int64_t c;
                chunk_of(o, R, C, cm, rr, c);
                const int64_t base = (u * R + rr) * K + c * CHUNK;
                for (int l = 0; l < 32; l++) {
                    for (int s = 0; s < 16; s += 2) {
                        bits[l] += pc.len[sym_at(base + pos_of(l, s))];
                    }
                }
            }
            for (int l = 0; l < 32; l++) {
                lane_words[u * 32 + l] = (uint32_t) ((bits[l] + 31) / 32);
            }
        }
    });
    aux_header h = {};
    h.magic = MAGIC; h.format = FMT_HUFPAIR; h.K = (uint32_t) K; h.R = (uint32_t) R; h.rows = (uint64_t) rows;
    h.off_a = HEADER_BYTES;
    h.off_b = h.off_a + (4u << HP_LP);
    h.off_c = h.off_b + (uint64_t) units * 4;
    h.off_d = (h.off_c + (uint64_t) units * 32 * 2 + 15) & ~15ull;
    std::vector<uint64_t> ubase(units + 1);
    uint64_t n_words = 0;
    for (int64_t u = 0; u < units; u++) {
        ubase[u] = n_words;
        uint64_t rel = 0;
        for (int l = 0; l < 32; l++) {
            if (rel > 0xFFFF) {
                invariant("lane offset <= 0xFFFF");
            }
            rel += lane_words[u * 32 + l];
        }
        n_words += rel;
    }
    ubase[units] = n_words;
    if (!(n_words + 32 < (1ull << 32))) {
        invariant("n_words + 32 < 2^32");
    }
    h.n_a = (uint64_t) units; h.n_b = n_words; h.flags = cm ? FLAG_CHUNK_MAJOR : 0;
    bytes aux(h.off_d + (n_words + 32) * 4, 0); // 32 words of decoder lookahead
    std::memcpy(aux.data(), &h, sizeof(h));
    std::memcpy(aux.data() + h.off_a, pc.lut.data(), 4u << HP_LP);
    uint32_t * unit_base = (uint32_t *) (aux.data() + h.off_b);
    uint16_t * lane_rel = (uint16_t *) (aux.data() + h.off_c);
    uint32_t * stream = (uint32_t *) (aux.data() + h.off_d);
    parallel_blocks(units, 8, [&](int64_t u0, int64_t u1) {
        for (int64_t u = u0; u < u1; u++) {
            unit_base[u] = (uint32_t) ubase[u];
            uint32_t rel = 0;
            for (int l = 0; l < 32; l++) {
                lane_rel[u * 32 + l] = (uint16_t) rel;
                msb_writer bw{stream + ubase[u] + rel};
                for (int64_t o = 0; o < R * C; o++) {
                    int rr; int64_t c;
                    chunk_of(o, R, C, cm, rr, c);
                    const int64_t base = (u * R + rr) * K + c * CHUNK;
                    for (int s = 0; s < 16; s += 2) {
                        const int sym = sym_at(base + pos_of(l, s));
                        bw.put(pc.code[sym], pc.len[sym]);
                    }
                }
                bw.flush();
                rel += lane_words[u * 32 + l];
            }
        }
    });
    return aux;
}

// ---------------------------------------------------------------------------------------------- HUFPAIR, wave64 units
//
// A unit is R rows decoded by one 64-lane wavefront.  Step i of a unit covers the chunks o = 2i (lanes 0..31) and
// o = 2i + 1 (lanes 32..63) of the unit's stream order, each lane with the (lane % 32, slot) ownership of the plane,
// so the plane bytes do not change and a wave reads 1024 contiguous plane bytes per step.
//
// Every lane has a bit sequence: 2 zero bits, then its pair codes in order, each written with its first (most
// significant) code bit lowest.  Word k of the lane holds sequence bits [32k, 32k + 32), sequence bit 32k + j in bit
// j.  The decoder keeps three words per lane (w0, w1, w2) and a position P < 32 into w0; the next code's table index
// is bits [P + 2, P + 14) of w1:w0.  After every second pair it adds the two code lengths to P; every lane with
// P >= 32 then takes the next word of the unit's stream (lanes in ascending order) as its new w2, the old w2 becomes
// w1, the old w1 becomes w0, and P drops by 32 (the word taken is not needed before the next such check, so its read
// overlaps the table lookups in between).  The unit's stream is therefore: words 0, 1, 2 of lane 0, of lane 1, ... of
// lane 63, then the refill words in exactly the order the decoder takes them — a wave reads it front to back with
// coalesced loads, and the lane of a refill word is its rank among the refilling lanes.  The table at off_a is
// indexed by those 12 bits as they sit in the word (first code bit = index bit 0), i.e. the canonical table with
// bit-reversed index.  unit_base has units + 1 entries (word index of each unit's first word and the end).
bytes encode_hufpair_w64(const uint16_t * w, int64_t rows, int64_t K, int R, bool cm) {
    pair_code pc;
    if (!build_pair_code(w, rows, K, pc)) {
        return {};
    }
    const int64_t C = K / CHUNK, units = rows / R, steps = R * C / 2;
    auto sym_at = [&](int64_t i) { return exp_of(w[i]) | exp_of(w[i + 1]) << 8; };
    // first element of the chunk that half-wave `half` decodes in step st of unit u
    auto chunk_base = [&](int64_t u, int64_t st, int half) {
        int rr; int64_t c;
        chunk_of(2 * st + half, R, C, cm, rr, c);
        return (u * R + rr) * K + c * CHUNK;
    };
    // the two pairs of lane l at check t (pairs 2t, 2t+1) of a chunk
    auto pair_syms = [&](int64_t base, int l, int t, int & s0, int & s1) {
        s0 = sym_at(base + pos_of(l & 31, 4 * t));
        s1 = sym_at(base + pos_of(l & 31, 4 * t + 2));
    };
    std::vector<uint16_t> rcode(65536, 0); // codes with their first bit lowest, as the stream holds them
    for (int sidx = 0; sidx < 65536; sidx++) {
        if (pc.len[sidx]) {
            rcode[sidx] = (uint16_t) bitrev(pc.code[sidx], pc.len[sidx]);
        }
    }
    // pass 1: words per unit = 192 + number of refills
    std::vector<uint64_t> ubase(units + 1, 0);
    parallel_blocks(units, 8, [&](int64_t u0, int64_t u1) {
        for (int64_t u = u0; u < u1; u++) {
            uint32_t P[64] = {0};
            uint64_t refills = 0;
            for (int64_t st = 0; st < steps; st++) {
                const int64_t base[2] = {chunk_base(u, st, 0), chunk_base(u, st, 1)};
                for (int t = 0; t < 4; t++) {
                    for (int l = 0; l < 64; l++) {
                        int s0, s1;
                        pair_syms(base[l >> 5], l, t, s0, s1);
                        P[l] += pc.len[s0] + pc.len[s1];
                        if (P[l] >= 32) {
                            P[l] -= 32;
                            refills++;
                        }
                    }
                }
            }
            ubase[u + 1] = 192 + refills;
        }
    });
    for (int64_t u = 0; u < units; u++) {
        ubase[u + 1] += ubase[u];
    }
    const uint64_t n_words = ubase[units];
    if (!(n_words + 1024 < (1ull << 32))) {
        invariant("n_words + 1024 < 2^32");
    }
    aux_header h = {};
    h.magic = MAGIC; h.format = FMT_HUFPAIR; h.K = (uint32_t) K; h.R = (uint32_t) R; h.rows = (uint64_t) rows;
    h.off_a = HEADER_BYTES;
    h.off_b = h.off_a + (4u << HP_LP);
    h.off_d = (h.off_b + ((uint64_t) units + 1) * 4 + 15) & ~15ull;
    h.off_c = h.off_d;
    h.n_a = (uint64_t) units; h.n_b = n_words; h.flags = FLAG_WAVE64 | (cm ? FLAG_CHUNK_MAJOR : 0);
    // 1024 words of padding: a wave prefetches its stream in 1 KiB blocks and may run up to three blocks ahead
    // not zeroed as a whole: pass 2 writes every stream word; zero what it does not write (header padding, the gap
    // before the stream, the padding behind it)
    bytes aux(h.off_d + (n_words + 1024) * 4);
    std::memset(aux.data(), 0, h.off_d);
    std::memset(aux.data() + h.off_d + n_words * 4, 0, 1024 * 4);
    std::memcpy(aux.data(), &h, sizeof(h));
    uint32_t * lut = (uint32_t *) (aux.data() + h.off_a);
    for (uint32_t i = 0; i < (1u << HP_LP); i++) {
        lut[bitrev(i, HP_LP)] = pc.lut[i];
    }
    uint32_t * unit_base = (uint32_t *) (aux.data() + h.off_b);
    for (int64_t u = 0; u <= units; u++) {
        unit_base[u] = (uint32_t) ubase[u];
    }
    uint32_t * stream = (uint32_t *) (aux.data() + h.off_d);
    // pass 2: build each lane's words, then lay them out in the order the decoder takes them
    // a lane takes at most 24 bits per pair of codes: steps * 4 * 24 bits and the two leading ones, + the zero words behind
    const int64_t maxw = (steps * 4 * 24 + 2 + 31) / 32 + 5;
    parallel_blocks(units, 8, [&](int64_t u0, int64_t u1) {
        std::vector<uint32_t> lane_words((size_t) (64 * maxw));
        std::vector<uint8_t> order; // lane of every refill, in decoder order
        order.reserve((size_t) (steps * 4 * 64));
        for (int64_t u = u0; u < u1; u++) {
            order.clear();
            uint64_t acc[64];
            int nb[64], nw[64];
            uint32_t P[64];
            for (int l = 0; l < 64; l++) {
                acc[l] = 0; nb[l] = 2; nw[l] = 0; P[l] = 0; // two leading zero bits
            }
            auto put = [&](int l, uint32_t code, int len) { // code: first bit lowest
                acc[l] |= (uint64_t) code << nb[l];
                nb[l] += len;
                if (nb[l] >= 32) {
                    lane_words[(size_t) (l * maxw + nw[l]++)] = (uint32_t) acc[l];
                    acc[l] >>= 32;
                    nb[l] -= 32;
                }
            };
            for (int64_t st = 0; st < steps; st++) {
                const int64_t base[2] = {chunk_base(u, st, 0), chunk_base(u, st, 1)};
                for (int t = 0; t < 4; t++) {
                    for (int l = 0; l < 64; l++) {
                        int s0, s1;
                        pair_syms(base[l >> 5], l, t, s0, s1);
                        put(l, rcode[s0], pc.len[s0]);
                        put(l, rcode[s1], pc.len[s1]);
                        P[l] += pc.len[s0] + pc.len[s1];
                        if (P[l] >= 32) {
                            P[l] -= 32;
                            order.push_back((uint8_t) l);
                        }
                    }
                }
            }
            uint32_t taken[64];
            uint32_t * out = stream + ubase[u];
            for (int l = 0; l < 64; l++) {
                uint32_t * lw = lane_words.data() + l * maxw;
                lw[nw[l]++] = (uint32_t) acc[l]; // partial last word, zero-filled
                for (int z = 0; z < 4; z++) {
                    lw[nw[l]++] = 0;             // the words a lane requests past its last code
                }
                *out++ = lw[0];
                *out++ = lw[1];
                *out++ = lw[2];
                taken[l] = 3;
            }
            for (uint8_t l : order) {
                *out++ = lane_words[(size_t) (l * maxw + taken[l]++)];
            }
            if ((uint64_t) (out - stream) != ubase[u + 1]) {
                invariant("wave64 unit size");
            }
        }
    });
    return aux;
}

// ---------------------------------------------------------------------------------------------- HUFPAIR, wave64 tiles
//
// R = 32 with the wave64 layout: units are tiles of 32 rows x 256 columns in the operand order of the 32x32x16 matrix
// instruction, so that a wavefront decodes straight into A operands (lane l holds row l % 32; its 16 weights of a
// step are two runs of 8 consecutive columns, 8 (l / 32) into each 16-column block of the step's 32 columns).
// Unit u = g * (K / 256) + t is the tile of rows [32 g, 32 g + 32), columns [256 t, 256 t + 256): the tiles of a row
// group are consecutive units, a wavefront can decode them as one run.  A tile is stored exactly as a wave64 unit
// of 16 rows of the 512-column matrix V (same plane and stream rules), with
//   V[16 u + 2 s + h][128 j + 4 l + q] = W[32 g + l][256 t + 32 s + 16 (j / 2) + 8 h + 4 (j % 2) + q]
// for step s < 8, half-wave h < 2, j < 4, l < 32, q < 4.  The header keeps the matrix's own K and rows, R = 32.
int64_t tile32_index(int64_t vrow, int64_t vcol, int64_t K) {
    const int64_t u = vrow / 16, s = (vrow % 16) / 2, h = vrow % 2;
    const int64_t j = vcol / 128, l = (vcol % 128) / 4, q = vcol % 4;
    const int64_t slabs = K / TILE_K, g = u / slabs, t = u % slabs;
    return (TILE_R * g + l) * K + TILE_K * t + 32 * s + 16 * (j / 2) + 8 * h + 4 * (j % 2) + q;
}

bool encode_tile32(const uint16_t * w, int64_t rows, int64_t K, encoded_buffers & out) {
    const int64_t vrows = rows * K / CHUNK;
    const std::unique_ptr<uint16_t[]> v_mem(new uint16_t[(size_t) (rows * K)]); // not zeroed: every element is written below
    uint16_t * const v = v_mem.get();
    // tile32_index() row by row: the four weights of a (j, l) cell are adjacent in W
    const int64_t slabs = K / TILE_K;
    parallel_blocks(vrows, 64, [&](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; r++) {
            const int64_t u = r / 16, s = (r % 16) / 2, h = r % 2, g = u / slabs, t = u % slabs;
            const uint16_t * src = w + TILE_R * g * K + TILE_K * t + 32 * s + 8 * h;
            uint16_t * dst = v + r * CHUNK;
            for (int64_t j = 0; j < 4; j++) {
                const uint16_t * sj = src + 16 * (j / 2) + 4 * (j % 2);
                for (int64_t l = 0; l < 32; l++) {
                    std::memcpy(dst + 128 * j + 4 * l, sj + l * K, 4 * sizeof(uint16_t));
                }
            }
        }
    });
    out.aux = encode_hufpair_w64(v, vrows, CHUNK, 16, false);
    if (out.aux.empty()) {
        return false;
    }
    aux_header h;
    std::memcpy(&h, out.aux.data(), sizeof(h));
    h.K = (uint32_t) K; h.R = TILE_R; h.rows = (uint64_t) rows;
    std::memcpy(out.aux.data(), &h, sizeof(h));
    write_plane(v, vrows, CHUNK, 16, false, out.plane.data());
    out.format = FMT_HUFPAIR;
    out.R = TILE_R;
    return true;
}

// ---------------------------------------------------------------------------------------------- entry point

// argument contract of the reference (encode.cpp:443-474) plus the wave64 layout of this build
encoded_buffers encode(const uint16_t * w, int64_t rows, int64_t K, int format, int R, uint32_t flags) {
    auto bad = [](const std::string & m) { throw std::invalid_argument("bf16n encode: " + m); };
    const bool cm = flags & FLAG_CHUNK_MAJOR, fo = flags & FLAG_FRAG_ORDER, w64 = flags & FLAG_WAVE64;
    if (flags & ~(FLAG_CHUNK_MAJOR | FLAG_FRAG_ORDER | FLAG_WAVE64)) {
        bad("unknown layout flags " + std::to_string(flags));
    }
    if (K % CHUNK != 0 || K < CHUNK || K > K_MAX) {
        bad("K must be a multiple of 512 in [512, 4096], got " + std::to_string(K));
    }
    if (rows <= 0) {
        bad("rows must be positive");
    }
    if (format == FMT_NIBBLE) {
        if (R != 0 || cm || fo || w64) {
            bad("NIBBLE takes R = 0 and no chunk-major or fragment-order layout");
        }
    } else if (format == FMT_HUFFMAN || format == FMT_HUFPAIR) {
        const bool tiles = R == TILE_R && w64 && format == FMT_HUFPAIR; // matrix-core tiles, see encode_tile32()
        if (R != 1 && R != 2 && R != 4 && R != 8 && R != 16 && !tiles) {
            bad("R must be one of 1, 2, 4, 8, 16 (or 32 for wave64 HUFPAIR tiles), got " + std::to_string(R));
        }
        if (rows % R != 0) {
            bad("rows (" + std::to_string(rows) + ") must be a multiple of R (" + std::to_string(R) + ")");
        }
        if (format == FMT_HUFFMAN && cm) {
            bad("chunk-major units exist only for HUFPAIR");
        }
        if (cm && (K == CHUNK || (R != 4 && R != 8 && R != 16))) {
            bad("chunk-major units need K > 512 and R in {4, 8, 16} (the chunk-major kernels' instances)");
        }
        if (fo && (format != FMT_HUFPAIR || cm || R != 16)) {
            bad("fragment order exists only for HUFPAIR with R = 16, without chunk-major units");
        }
        if (fo) {
            bad("fragment order is the NVIDIA mma register layout and is not available in the MI355X build");
        }
        if (w64 && (format != FMT_HUFPAIR || cm)) {
            bad("the wave64 layout exists only for row-major HUFPAIR (no chunk-major units)");
        }
        if (w64 && (R * (K / CHUNK)) % 2 != 0) {
            bad("the wave64 layout needs an even number of 512-column chunks per unit (R * K / 512)");
        }
    } else {
        bad("unknown format " + std::to_string(format));
    }

    encoded_buffers out;
    out.plane.resize((size_t) (rows * K));
    out.R = format == FMT_NIBBLE ? 0 : R;
    if (format == FMT_NIBBLE) {
        write_plane(w, rows, K, 1, false, out.plane.data());
        out.aux = encode_nibble(w, rows, K, out.plane.data());
        out.format = FMT_NIBBLE;
        return out;
    }
    if (format == FMT_HUFPAIR && R == TILE_R) {
        if (encode_tile32(w, rows, K, out)) {
            return out;
        }
        R = 16; // more than 4096 distinct pairs: single-symbol fallback below, which has no special layouts
        out.R = R;
    } else if (format == FMT_HUFPAIR) {
        out.aux = w64 ? encode_hufpair_w64(w, rows, K, R, cm) : encode_hufpair(w, rows, K, R, cm);
    }
    if (!out.aux.empty()) {
        out.format = FMT_HUFPAIR;
        write_plane(w, rows, K, R, cm, out.plane.data());
    } else { // too many distinct pairs (or HUFFMAN requested): the single-symbol format has no special layouts
        out.aux = encode_huffman(w, rows, K, R);
        out.format = FMT_HUFFMAN;
        write_plane(w, rows, K, R, false, out.plane.data());
    }
    return out;
}

} // namespace impl
} // namespace bf16n
