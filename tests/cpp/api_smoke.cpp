// Host-only use of the C++ API headers (include/bf16n/*.h): policy, encoder, exception translation.  Prints lines the
// Python test checks.  No GPU call is made; launch.h is only compiled.
#include "bf16n/encode.h"
#include "bf16n/launch.h"
#include "bf16n/policy.h"

#include <cstdio>
#include <cstring>

int main() {
    const auto none = bf16n::choose(100, 500);
    std::printf("choose_bad_k %d\n", none.has_value() ? 1 : 0);
    bf16n::policy_options llama;
    llama.engine = bf16n::policy_engine::llama;
    const auto c = bf16n::choose(248320, 2048, 1, llama);
    std::printf("choose_llama %d %d %d %d\n", c->format, c->R, (int) c->chunk_major, (int) c->frag_order);
    bf16n::policy_options mi;
    mi.engine = bf16n::policy_engine::mi355x;
    const auto m = bf16n::choose(248320, 2048, 1, mi);
    std::printf("choose_mi355x %d %d %d %d\n", m->format, m->R, (int) m->chunk_major, (int) m->wave64);

    std::vector<uint16_t> w(16 * 1024);
    for (size_t i = 0; i < w.size(); i++) {
        w[i] = (uint16_t) (0x3c00 + (i * 2654435761u >> 24));
    }
    const bf16n::encoded e = bf16n::encode(w.data(), 16, 1024, bf16n::FMT_HUFPAIR, 4, false);
    bf16n::aux_header h;
    std::memcpy(&h, e.aux.data(), sizeof h);
    std::printf("encode %zu %d %d %u %u %u\n", e.plane.size(), e.format, e.R, h.magic == bf16n::MAGIC ? 1u : 0u, h.K, h.flags);
    const bf16n::encoded e64 = bf16n::encode(w.data(), 16, 1024, bf16n::FMT_HUFPAIR, 4, false, false, true);
    std::memcpy(&h, e64.aux.data(), sizeof h);
    std::printf("encode_wave64 %u\n", h.flags);
    try {
        bf16n::encode(w.data(), 16, 1024, bf16n::FMT_HUFPAIR, 3, false);
        std::printf("no_throw\n");
    } catch (const std::invalid_argument & ex) {
        std::printf("invalid_argument %s\n", ex.what());
    }
    try {
        bf16n::encode(w.data(), 16, 512, bf16n::FMT_HUFPAIR, 16, false, true);
        std::printf("no_throw\n");
    } catch (const std::invalid_argument & ex) {
        std::printf("invalid_argument %s\n", ex.what());
    }
    bf16n::weight view;
    bf16n::mmv_args args;
    std::printf("views %d %d\n", (int) sizeof(view.off_a), args.n_used);
    return 0;
}
