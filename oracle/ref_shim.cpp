// TEST INFRASTRUCTURE ONLY.  C-callable shim around the reference's own host encoder and shape policy, compiled
// together with the reference sources where they lie (see Makefile, target _ref/libbf16n_ref.so).  Used to validate the
// C restatement in bf16n_oracle.c and to generate the golden fixtures under tests/golden/.
#include "bf16n/encode.h"
#include "bf16n/policy.h"

#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>

static thread_local std::string g_err;

extern "C" {

const char * ref_last_error() { return g_err.c_str(); }

// 0 ok, 1 std::invalid_argument, 2 any other exception. plane: rows*K bytes (caller). *aux: malloc'ed.
int ref_encode(const uint16_t * w, int64_t rows, int64_t K, int format, int R, int chunk_major, int frag_order,
               uint8_t * plane, uint8_t ** aux, uint64_t * aux_bytes, int * format_out, int * R_out) {
    try {
        bf16n::encoded e = bf16n::encode(w, rows, K, format, R, chunk_major != 0, frag_order != 0);
        std::memcpy(plane, e.plane.data(), e.plane.size());
        *aux = (uint8_t *) std::malloc(e.aux.size());
        std::memcpy(*aux, e.aux.data(), e.aux.size());
        *aux_bytes = e.aux.size();
        *format_out = e.format;
        *R_out = e.R;
        return 0;
    } catch (const std::invalid_argument & ex) {
        g_err = ex.what();
        return 1;
    } catch (const std::exception & ex) {
        g_err = ex.what();
        return 2;
    }
}

void ref_free(void * p) { std::free(p); }

// engine: 0 llama, 1 vllm; mode: 0 hybrid, 1 huffman, 2 nibble. Returns 0 for nullopt, else 1 and fills out[4] =
// {format, R, chunk_major, frag_order}.
int ref_choose(int64_t rows, int64_t K, int64_t n, int engine, int mode, int64_t dense_min, int expert,
               int dense_frag_order, int * out) {
    bf16n::policy_options o;
    o.engine = engine == 0 ? bf16n::policy_engine::llama : bf16n::policy_engine::vllm;
    o.mode = mode == 0 ? bf16n::policy_mode::hybrid : mode == 1 ? bf16n::policy_mode::huffman : bf16n::policy_mode::nibble;
    o.dense_min = dense_min;
    o.expert = expert != 0;
    o.dense_frag_order = dense_frag_order != 0;
    const auto c = bf16n::choose(rows, K, n, o);
    if (!c) {
        return 0;
    }
    out[0] = c->format; out[1] = c->R; out[2] = c->chunk_major; out[3] = c->frag_order;
    return 1;
}

}
