// Host encoder and policy under AddressSanitizer / UBSan (no GPU code involved): every format and layout on small
// tensors with all special BF16 classes, the pair-alphabet fallback, the argument contract, many policy queries.
#include "encode_impl.h"

#include <cstdio>
#include <stdexcept>
#include <vector>

using namespace bf16n;

int main() {
    uint64_t s = 0x2545F4914F6CDD1Dull;
    auto rnd = [&]() { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return s; };
    const uint16_t special[] = {0x0000, 0x8000, 0x0001, 0x807F, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7FC1, 0xFFFF, 0x3F80};
    int done = 0;
    for (int K : {512, 1024, 2048, 4096}) {
        const int64_t rows = 32;
        std::vector<uint16_t> w(rows * K);
        for (auto & v : w) {
            const uint64_t r = rnd();
            v = (uint16_t) (((r & 1) << 15) | ((118 + (r >> 1) % 10) << 7) | ((r >> 8) & 0x7F));
        }
        for (size_t i = 0; i < sizeof special / 2; i++) {
            w[(rnd() % rows) * K + rnd() % K] = special[i];
        }
        impl::encode(w.data(), rows, K, FMT_NIBBLE, 0, 0);
        impl::encode(w.data(), rows, K, FMT_HUFPAIR, 32, FLAG_WAVE64); // 32 x 256 tiles
        done += 2;
        for (int R : {1, 2, 4, 8, 16}) {
            impl::encode(w.data(), rows, K, FMT_HUFFMAN, R, 0);
            impl::encode(w.data(), rows, K, FMT_HUFPAIR, R, 0);
            done += 2;
            if (K > 512 && R >= 4) {
                impl::encode(w.data(), rows, K, FMT_HUFPAIR, R, FLAG_CHUNK_MAJOR);
                done++;
            }
            if ((R * K / 512) % 2 == 0) {
                impl::encode(w.data(), rows, K, FMT_HUFPAIR, R, FLAG_WAVE64);
                done++;
            }
        }
    }
    {   // more than 4096 distinct pairs: the single-exponent fallback
        std::vector<uint16_t> w(16 * 1024);
        for (size_t i = 0; i < w.size(); i += 2) {
            const size_t p = (i / 2) % 4200;
            w[i] = (uint16_t) ((60 + p % 70) << 7);
            w[i + 1] = (uint16_t) ((60 + p / 70) << 7);
        }
        const auto e = impl::encode(w.data(), 16, 1024, FMT_HUFPAIR, 8, 0);
        std::vector<uint16_t> w2(w);
        w2.insert(w2.end(), w.begin(), w.end());
        const auto t = impl::encode(w2.data(), 32, 1024, FMT_HUFPAIR, 32, FLAG_WAVE64); // tiles fall back the same way
        std::printf("fallback format %d, tiles %d R %d\n", e.format, t.format, t.R);
    }
    int thrown = 0;
    const std::vector<uint16_t> w(16 * 512);
    for (int variant = 0; variant < 6; variant++) {
        try {
            switch (variant) {
                case 0: impl::encode(w.data(), 16, 500, FMT_HUFPAIR, 4, 0); break;
                case 1: impl::encode(w.data(), 16, 512, FMT_HUFPAIR, 3, 0); break;
                case 2: impl::encode(w.data(), 15, 512, FMT_HUFPAIR, 4, 0); break;
                case 3: impl::encode(w.data(), 16, 512, FMT_HUFPAIR, 4, FLAG_CHUNK_MAJOR); break;
                case 4: impl::encode(w.data(), 16, 512, FMT_NIBBLE, 4, 0); break;
                default: impl::encode(w.data(), 16, 512, FMT_HUFPAIR, 16, FLAG_FRAG_ORDER); break;
            }
        } catch (const std::invalid_argument &) {
            thrown++;
        }
    }
    int chosen = 0;
    impl::choice c;
    for (int64_t rows : {1ll, 7ll, 512ll, 5120ll, 248320ll, (1ll << 40)}) {
        for (int64_t K : {512ll, 1536ll, 4096ll, 4608ll}) {
            for (int engine = 0; engine < 3; engine++) {
                chosen += impl::choose(rows, K, 1 + (rows % 3) * 127, engine, 0, 8ll << 20, rows % 2 == 0, true, c) ? 1 : 0;
            }
        }
    }
    std::printf("encoded %d thrown %d chosen %d\n", done, thrown, chosen);
    return 0;
}
