// The C++ API end to end on the device, the way the reference's core/bench/standalone_mmv.cu uses it: policy, encode,
// upload, bit-exact dequant, one fused decode+GEMV on a stream, an error path.  Prints "ok" lines the Python test reads.
#include "bf16n/encode.h"
#include "bf16n/launch.h"
#include "bf16n/policy.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("hip error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)

static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t) b << 16; float f; std::memcpy(&f, &u, 4); return f; }
static uint16_t f32_to_bf16(float f) { uint32_t u; std::memcpy(&u, &f, 4); return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }

int main() {
    const int64_t rows = 8192, K = 2048;
    std::vector<uint16_t> w(rows * K), x(K);
    uint64_t s = 0x9E3779B97F4A7C15ull;
    auto rnd = [&]() { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return (double) (s >> 11) / 9007199254740992.0; };
    for (auto & v : w) { v = f32_to_bf16((float) (0.02 * std::sqrt(-2.0 * std::log(rnd() + 1e-300)) * std::cos(6.283185307179586 * rnd()))); }
    for (auto & v : x) { v = f32_to_bf16((float) (std::sqrt(-2.0 * std::log(rnd() + 1e-300)) * std::cos(6.283185307179586 * rnd()))); }

    bf16n::init();
    bf16n::policy_options po;
    po.engine = bf16n::policy_engine::mi355x;
    po.dense_min = 0;
    const auto ch = bf16n::choose(rows, K, 1, po);
    if (!ch) { std::printf("no choice\n"); return 1; }
    const bf16n::encoded e = bf16n::encode(w.data(), rows, K, ch->format, ch->R, ch->chunk_major, ch->frag_order, ch->wave64);
    bf16n::aux_header h;
    std::memcpy(&h, e.aux.data(), sizeof h);
    std::printf("encoded format %d R %d flags %u ratio %.4f\n", e.format, e.R, h.flags, (double) (e.plane.size() + e.aux.size()) / (2.0 * rows * K));

    uint8_t * d_plane, * d_aux; uint16_t * d_x, * d_w; float * d_y;
    HIP_OK(hipMalloc(&d_plane, e.plane.size())); HIP_OK(hipMalloc(&d_aux, e.aux.size()));
    HIP_OK(hipMalloc(&d_x, K * 2)); HIP_OK(hipMalloc(&d_w, rows * K * 2)); HIP_OK(hipMalloc(&d_y, rows * 4));
    HIP_OK(hipMemcpy(d_plane, e.plane.data(), e.plane.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_aux, e.aux.data(), e.aux.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_x, x.data(), K * 2, hipMemcpyHostToDevice));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    bf16n::weight wt;
    wt.plane = d_plane; wt.aux = d_aux; wt.format = (int) h.format; wt.K = h.K; wt.rows = (int64_t) h.rows; wt.R = (int) h.R;
    wt.cm = h.flags & bf16n::FLAG_CHUNK_MAJOR; wt.wave64 = h.flags & bf16n::FLAG_WAVE64;
    wt.off_a = h.off_a; wt.off_b = h.off_b; wt.off_c = h.off_c; wt.off_d = h.off_d;

    bf16n::dequant(wt, 0, rows, d_w, stream);
    std::vector<uint16_t> back(rows * K);
    HIP_OK(hipMemcpyAsync(back.data(), d_w, rows * K * 2, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::printf("dequant %s\n", std::memcmp(back.data(), w.data(), rows * K * 2) == 0 ? "ok" : "MISMATCH");

    bf16n::mmv_args a;
    a.x = d_x; a.x_bf16 = true; a.y = d_y; a.ncols = 1; a.x_tok = K * 2; a.y_tok = rows * 4; a.rows_per_matrix = rows; a.nrows = rows;
    bf16n::mmv(wt, a, stream);
    std::vector<float> y(rows);
    HIP_OK(hipMemcpyAsync(y.data(), d_y, rows * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    double worst = 0;
    for (int64_t r = 0; r < rows; r++) {
        double ref = 0, bound = 0;
        for (int64_t k = 0; k < K; k++) {
            const double p = (double) bf16_to_f32(w[r * K + k]) * (double) bf16_to_f32(x[k]);
            ref += p; bound += std::fabs(p);
        }
        worst = std::fmax(worst, std::fabs(y[r] - ref) / bound);
    }
    std::printf("mmv %s worst %.3g\n", worst <= 1e-5 ? "ok" : "OUT OF BOUND", worst);

    try {
        bf16n::dequant(wt, 1, 16, d_w, stream); // not whole units
        std::printf("no throw\n");
    } catch (const std::invalid_argument & ex) {
        std::printf("invalid_argument %s\n", ex.what());
    }
    return 0;
}
