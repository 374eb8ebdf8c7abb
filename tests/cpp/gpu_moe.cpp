// One small MoE layer through the C++ API on the device, both token regimes of the reference's engines: expert GEMVs
// (mmv_glu(gate, up) with ids, mmv with ids, moe_combine) and the batched kernels (mm_ids_route, mm_ids fused gate/up,
// mm_ids down, moe_combine), experts encoded under the mi355x policy.  Both are compared with an FP64 product of the
// exact weights.  Prints lines the Python test reads.
#include "bf16n/encode.h"
#include "bf16n/launch.h"
#include "bf16n/policy.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("hip error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)

static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t) b << 16; float f; std::memcpy(&f, &u, 4); return f; }
static uint16_t f32_to_bf16(float f) { uint32_t u; std::memcpy(&u, &f, 4); return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }

struct dev_weight {
    bf16n::weight w;
    int R = 0;
    uint32_t flags = 0;
};

static int upload(const std::vector<uint16_t> & bits, int64_t rows_per, int64_t K, int n, dev_weight & out) {
    bf16n::policy_options po;
    po.engine = bf16n::policy_engine::mi355x;
    po.expert = true;
    const auto ch = bf16n::choose(rows_per, K, n, po);
    if (!ch) { return 1; }
    const bf16n::encoded e = bf16n::encode(bits.data(), rows_per * n, K, ch->format, ch->R, ch->chunk_major, ch->frag_order, ch->wave64);
    bf16n::aux_header h;
    std::memcpy(&h, e.aux.data(), sizeof h);
    uint8_t * d_plane, * d_aux;
    HIP_OK(hipMalloc(&d_plane, e.plane.size())); HIP_OK(hipMalloc(&d_aux, e.aux.size()));
    HIP_OK(hipMemcpy(d_plane, e.plane.data(), e.plane.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_aux, e.aux.data(), e.aux.size(), hipMemcpyHostToDevice));
    out.w.plane = d_plane; out.w.aux = d_aux; out.w.format = (int) h.format; out.w.K = h.K; out.w.rows = (int64_t) h.rows; out.w.R = (int) h.R;
    out.w.cm = h.flags & bf16n::FLAG_CHUNK_MAJOR; out.w.wave64 = h.flags & bf16n::FLAG_WAVE64;
    out.w.off_a = h.off_a; out.w.off_b = h.off_b; out.w.off_c = h.off_c; out.w.off_d = h.off_d;
    out.R = (int) h.R; out.flags = h.flags;
    return 0;
}

int main() {
    const int E = 8, topk = 2, T = 40, Tdec = 4; // 40 tokens through the batched kernels, the first 4 also through the GEMVs
    const int64_t K = 1024, N = 512;              // gate, up: E x N x K; down: E x K x N
    uint64_t s = 0x2545F4914F6CDD1Dull;
    auto rnd = [&]() { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return (double) (s >> 11) / 9007199254740992.0; };
    auto gauss = [&](double sd) { return (float) (sd * std::sqrt(-2.0 * std::log(rnd() + 1e-300)) * std::cos(6.283185307179586 * rnd())); };
    std::vector<uint16_t> gate(E * N * K), up(E * N * K), down(E * K * N), x(T * K);
    for (auto & v : gate) { v = f32_to_bf16(gauss(0.05)); }
    for (auto & v : up) { v = f32_to_bf16(gauss(0.05)); }
    for (auto & v : down) { v = f32_to_bf16(gauss(0.05)); }
    for (auto & v : x) { v = f32_to_bf16(gauss(1.0)); }

    bf16n::init();
    dev_weight wg, wu, wd;
    if (upload(gate, N, K, E, wg) || upload(up, N, K, E, wu) || upload(down, K, N, E, wd)) { std::printf("setup failed\n"); return 1; }
    std::printf("experts R %d %d flags %u %u\n", wg.R, wd.R, wg.flags, wd.flags);

    // router logits -> top-k on the device
    std::vector<float> logits(T * E);
    for (auto & v : logits) { v = gauss(1.0); }
    float * d_logits, * d_wts, * d_act, * d_ys, * d_ys2; int32_t * d_ids, * d_src1, * d_dst, * d_bounds; uint16_t * d_x, * d_a16, * d_out, * d_out2;
    HIP_OK(hipMalloc(&d_logits, logits.size() * 4)); HIP_OK(hipMalloc(&d_wts, T * topk * 4)); HIP_OK(hipMalloc(&d_ids, T * topk * 4));
    HIP_OK(hipMalloc(&d_x, x.size() * 2)); HIP_OK(hipMalloc(&d_act, T * topk * N * 4)); HIP_OK(hipMalloc(&d_a16, T * topk * N * 2));
    HIP_OK(hipMalloc(&d_ys, T * topk * K * 4)); HIP_OK(hipMalloc(&d_ys2, T * topk * K * 4));
    HIP_OK(hipMalloc(&d_out, T * K * 2)); HIP_OK(hipMalloc(&d_out2, T * K * 2));
    HIP_OK(hipMalloc(&d_src1, T * topk * 4)); HIP_OK(hipMalloc(&d_dst, T * topk * 4)); HIP_OK(hipMalloc(&d_bounds, (E + 1) * 4));
    HIP_OK(hipMemcpy(d_logits, logits.data(), logits.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_x, x.data(), x.size() * 2, hipMemcpyHostToDevice));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    bf16n::router_topk(d_logits, E, T, E, topk, true, d_ids, d_wts, stream);

    // batched path, all T tokens
    std::printf("mm_ids_supported %d %d\n", (int) bf16n::mm_ids_supported(wg.w, &wu.w), (int) bf16n::mm_ids_supported(wd.w, nullptr));
    bf16n::mm_ids_route(d_ids, false, topk, d_src1, d_dst, d_bounds, E, T, topk, 1, 1, stream);
    bf16n::mm_ids(wg.w, &wu.w, d_x, K, d_src1, d_dst, d_bounds, d_a16, true, N, E, T, topk, stream);
    bf16n::mm_ids(wd.w, nullptr, d_a16, N, d_dst, d_dst, d_bounds, d_ys, false, K, E, T, topk, stream); // source row = destination row
    bf16n::moe_combine(d_ys, d_wts, false, d_out, true, T, topk, K, stream);

    // decode path, the first Tdec tokens: FP32 activations between the GEMVs
    bf16n::mmv_args a;
    a.x = d_x; a.x_bf16 = true; a.y = d_act; a.ncols = Tdec * topk; a.x_tok = K * 2; a.y_tok = topk * N * 4; a.y_slot = N * 4;
    a.ids = d_ids; a.ids_s0 = 4; a.ids_s1 = topk * 4; a.n_used = topk; a.x_per_slot = 1; a.rows_per_matrix = N; a.nrows = N;
    bf16n::mmv_glu(wg.w, wu.w, a, stream);
    bf16n::mmv_args b;
    b.x = d_act; b.x_bf16 = false; b.y = d_ys2; b.ncols = Tdec * topk; b.x_tok = topk * N * 4; b.x_slot = N * 4; b.x_per_slot = topk;
    b.y_tok = topk * K * 4; b.y_slot = K * 4; b.ids = d_ids; b.ids_s0 = 4; b.ids_s1 = topk * 4; b.n_used = topk; b.rows_per_matrix = K; b.nrows = K;
    bf16n::mmv(wd.w, b, stream);
    bf16n::moe_combine(d_ys2, d_wts, false, d_out2, true, Tdec, topk, K, stream);

    std::vector<uint16_t> out(T * K), out2(Tdec * K);
    std::vector<int32_t> ids(T * topk);
    std::vector<float> wts(T * topk);
    HIP_OK(hipMemcpyAsync(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(out2.data(), d_out2, out2.size() * 2, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(ids.data(), d_ids, ids.size() * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(wts.data(), d_wts, wts.size() * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));

    // FP64 reference with the exact weights (activations between gate/up and down kept in FP64)
    double worst = 0, worst2 = 0, scale = 0;
    std::vector<double> ref(T * K, 0.0), act(N);
    for (int t = 0; t < T; t++) {
        for (int k = 0; k < topk; k++) {
            const int e = ids[t * topk + k];
            if (e < 0 || e >= E) { std::printf("bad expert id %d\n", e); return 1; }
            for (int64_t r = 0; r < N; r++) {
                double g = 0, u = 0;
                for (int64_t c = 0; c < K; c++) {
                    const double xv = bf16_to_f32(x[t * K + c]);
                    g += (double) bf16_to_f32(gate[(e * N + r) * K + c]) * xv;
                    u += (double) bf16_to_f32(up[(e * N + r) * K + c]) * xv;
                }
                act[r] = u * (g / (1.0 + std::exp(-g)));
            }
            for (int64_t r = 0; r < K; r++) {
                double d = 0;
                for (int64_t c = 0; c < N; c++) { d += (double) bf16_to_f32(down[(e * K + r) * N + c]) * act[c]; }
                ref[t * K + r] += wts[t * topk + k] * d;
            }
        }
    }
    for (double v : ref) { scale = std::max(scale, std::fabs(v)); }
    for (int64_t i = 0; i < T * K; i++) { worst = std::max(worst, std::fabs(bf16_to_f32(out[i]) - ref[i])); }
    for (int64_t i = 0; i < Tdec * K; i++) { worst2 = std::max(worst2, std::fabs(bf16_to_f32(out2[i]) - ref[i])); }
    // the results are BF16 (half a step of 2^-8 relative = 0.2 % of the largest value); the batched kernels also round
    // the activations between gate/up and down to BF16
    std::printf("batched %s worst %.3g of %.3g\n", worst <= 0.008 * scale ? "ok" : "OUT OF BOUND", worst, scale);
    std::printf("gemv %s worst %.3g of %.3g\n", worst2 <= 0.005 * scale ? "ok" : "OUT OF BOUND", worst2, scale);
    return 0;
}
