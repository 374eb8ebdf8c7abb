// The load-time path the way the reference's llama.cpp adapter drives it (patch 0002: choose -> convert -> lookup by
// tensor address -> launch -> free): three tensors of one "buffer" are converted into their own device storage, found
// again by base and interior addresses, multiplied through the looked-up weights, and dropped with their owner.
// Prints "ok" lines the Python test reads.
#include "bf16n/adapter.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("hip error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)

static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t) b << 16; float f; std::memcpy(&f, &u, 4); return f; }
static uint16_t f32_to_bf16(float f) { uint32_t u; std::memcpy(&u, &f, 4); return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }

static uint64_t s = 0x9E3779B97F4A7C15ull;
static double rnd() { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return (double) (s >> 11) / 9007199254740992.0; }
static double gauss() { return std::sqrt(-2.0 * std::log(rnd() + 1e-300)) * std::cos(6.283185307179586 * rnd()); }

struct tensor {
    const char * name;
    int64_t rows_per_matrix, K, n;
    std::vector<uint16_t> host;
    uint8_t * data = nullptr; // device: rows * K bytes
};

int main() {
    namespace ad = bf16n::adapter;
    tensor ts[3] = {{"output.weight", 8192, 2048, 1, {}}, {"blk.0.ffn_gate_exps.weight", 64, 2048, 8, {}}, {"blk.0.ffn_down_shexp.weight", 2048, 512, 1, {}}};
    int owner_a = 0, owner_b = 0; // two "buffers"
    for (auto & t : ts) {
        t.host.resize(t.rows_per_matrix * t.n * t.K);
        for (auto & v : t.host) { v = f32_to_bf16((float) (0.02 * gauss())); }
        HIP_OK(hipMalloc(&t.data, t.host.size()));
    }
    // the loader's decision per tensor (hybrid: small dense tensors take NIBBLE), then the conversion
    const ad::tag want[3] = {ad::tag::huffman, ad::tag::huffman, ad::tag::nibble};
    for (int i = 0; i < 3; i++) {
        tensor & t = ts[i];
        const ad::tag tg = ad::choose(t.rows_per_matrix, t.K, t.n, "hybrid", 8ll << 20, t.n > 1);
        if (tg != want[i]) { std::printf("choose %s: tag %d\n", t.name, (int) tg); return 1; }
        const bool ok = ad::convert(t.data, t.host.data(), t.rows_per_matrix, t.K, t.n, tg, i < 2 ? (void *) &owner_a : (void *) &owner_b, t.name);
        std::printf("convert %s %s\n", t.name, ok ? "ok" : "ROUNDTRIP FAILED");
    }
    std::printf("registered %d\n", bf16n_adapter_count());
    if (ad::choose(7, 500, 1, "hybrid", 0, false) != ad::tag::stay_bf16) { std::printf("choose accepted K = 500\n"); return 1; }

    // lookups: base address, an interior row (a view), just past the end, an unaligned address
    const auto base = ad::lookup(ts[0].data);
    const auto view = ad::lookup(ts[0].data + 96 * ts[0].K);
    const auto expert3 = ad::lookup(ts[1].data + 3 * 64 * ts[1].K);
    const auto past = ad::lookup(ts[2].data + ts[2].host.size());
    std::printf("lookup %s\n", base && base->row0 == 0 && view && view->row0 == 96 && view->w.aux == base->w.aux && expert3 &&
                                       expert3->row0 == 192 && expert3->w.R == 32 && (!past || past->w.plane != ts[2].data) ? "ok" : "WRONG");
    try {
        ad::lookup(ts[0].data + 5);
        std::printf("no throw\n");
    } catch (const std::invalid_argument & ex) {
        std::printf("invalid_argument %s\n", ex.what());
    }
    // a tensor must not be converted twice into the same storage, and the refused call leaves the resident tensor as
    // it was (the source here is another one: the verify step below would notice its plane bytes)
    try {
        const std::vector<uint16_t> other(ts[2].host.size(), (uint16_t) 0x3F80);
        ad::convert(ts[2].data, other.data(), 2048, 512, 1, ad::tag::nibble, &owner_b, "again", bf16n::policy_engine::mi355x, false, false);
        std::printf("no throw\n");
    } catch (const std::invalid_argument & ex) {
        std::printf("invalid_argument %s\n", ex.what());
    }
    // the verify step notices one flipped mantissa bit in the source it is given
    std::vector<uint16_t> bad = ts[2].host;
    bad[bad.size() / 2] ^= 1;
    const auto sh = ad::lookup(ts[2].data);
    std::printf("verify %s\n", ad::verify_roundtrip(sh->w, ts[2].host.data()) && !ad::verify_roundtrip(sh->w, bad.data()) ? "ok" : "WRONG");

    // products through the looked-up weights: rows [96, 96 + 256) of the dense tensor, and expert 3 of the stacked one
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    const int64_t K = 2048;
    std::vector<uint16_t> x(K);
    for (auto & v : x) { v = f32_to_bf16((float) gauss()); }
    uint16_t * d_x; float * d_y;
    HIP_OK(hipMalloc(&d_x, K * 2)); HIP_OK(hipMalloc(&d_y, 256 * 4));
    HIP_OK(hipMemcpy(d_x, x.data(), K * 2, hipMemcpyHostToDevice));
    bool all_ok = true;
    struct prod { const bf16n::adapter::found * f; const tensor * t; int64_t nrows; } prods[2] = {{&*view, &ts[0], 256}, {&*expert3, &ts[1], 64}};
    for (const auto & p : prods) {
        bf16n::mmv_args a;
        a.x = d_x; a.x_bf16 = true; a.y = d_y; a.ncols = 1; a.x_tok = K * 2; a.y_tok = p.nrows * 4;
        a.rows_per_matrix = p.t->rows_per_matrix; a.row0 = p.f->row0; a.nrows = p.nrows;
        bf16n::mmv(p.f->w, a, stream);
        std::vector<float> y(p.nrows);
        HIP_OK(hipMemcpyAsync(y.data(), d_y, p.nrows * 4, hipMemcpyDeviceToHost, stream));
        HIP_OK(hipStreamSynchronize(stream));
        for (int64_t r = 0; r < p.nrows; r++) {
            double ref = 0, bound = 0;
            for (int64_t k = 0; k < K; k++) {
                const double q = (double) bf16_to_f32(p.t->host[(p.f->row0 + r) * K + k]) * (double) bf16_to_f32(x[k]);
                ref += q; bound += std::fabs(q);
            }
            all_ok = all_ok && std::fabs(y[r] - ref) <= 1e-5 * bound;
        }
    }
    std::printf("mmv %s\n", all_ok ? "ok" : "OUT OF BOUND");

    // more tokens than the GEMV serves: the dense path (exact dequant into caller-owned scratch + the stock BF16 GEMM)
    {
        const int T = 12;
        const int64_t rows = ts[0].rows_per_matrix;
        std::vector<uint16_t> xs((size_t) T * K);
        for (auto & v : xs) { v = f32_to_bf16((float) gauss()); }
        const auto sizes = ad::dense_sizes(base->w);
        uint16_t * d_xs, * d_ys; void * d_scratch, * d_ws;
        HIP_OK(hipMalloc(&d_xs, xs.size() * 2)); HIP_OK(hipMalloc(&d_ys, (size_t) T * rows * 2));
        HIP_OK(hipMalloc(&d_scratch, sizes.scratch_bytes)); HIP_OK(hipMalloc(&d_ws, sizes.gemm_workspace_bytes));
        HIP_OK(hipMemcpy(d_xs, xs.data(), xs.size() * 2, hipMemcpyHostToDevice));
        ad::linear_dense(base->w, d_xs, K, T, d_ys, rows, d_scratch, sizes.scratch_bytes, d_ws, sizes.gemm_workspace_bytes, stream);
        std::vector<uint16_t> ys((size_t) T * rows);
        HIP_OK(hipMemcpyAsync(ys.data(), d_ys, ys.size() * 2, hipMemcpyDeviceToHost, stream));
        HIP_OK(hipStreamSynchronize(stream));
        bool dense_ok = true;
        for (int t = 0; t < T; t++) {
            for (int64_t r = 0; r < rows; r += 37) {
                double ref = 0, bound = 0;
                for (int64_t k = 0; k < K; k++) {
                    const double q = (double) bf16_to_f32(ts[0].host[r * K + k]) * (double) bf16_to_f32(xs[(size_t) t * K + k]);
                    ref += q; bound += std::fabs(q);
                }
                dense_ok = dense_ok && std::fabs(bf16_to_f32(ys[(size_t) t * rows + r]) - ref) <= std::fabs(ref) / 256 + 1e-5 * bound;
            }
        }
        std::printf("linear_dense %s\n", dense_ok ? "ok" : "OUT OF BOUND");
    }

    // freeing a buffer drops its tensors and their aux storage; the other buffer's tensor stays
    const int dropped = ad::release(&owner_a);
    std::printf("release %s\n", dropped == 2 && !ad::is_registered(ts[0].data) && !ad::is_registered(ts[1].data) && ad::is_registered(ts[2].data) &&
                                        ad::release(&owner_b) == 1 && bf16n_adapter_count() == 0 ? "ok" : "WRONG");
    return 0;
}
