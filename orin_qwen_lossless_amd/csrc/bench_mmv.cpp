// Stand-alone timing of the fused decode+GEMV through the C++ API, without Python or torch in the process: the
// counterpart of the reference's core/bench/standalone_mmv.cu:21-84 (encode, upload, warm up for a fixed time, then the
// median of individually synchronised launches between events on a non-blocking stream).  It is also the program to put
// behind `rocprofv3 ... --` when only this kernel is to be profiled.
//
//   bf16n_bench [--rows N] [--K K] [--batch T] [--reps R] [--warm-ms MS] [--tiles] [--f32] [--probe] [--copies C]
//
// Weights: N(0, 0.02) rounded to BF16 from the counter-based generator of orin_qwen_lossless_amd/synth.py (splitmix64 on
// (seed, index) + Box-Muller), activations N(0, 1); `copies` copies of the encoded matrix at different addresses are
// used in turn so that the last-level cache does not serve the stream.  Prints one JSON line.
#include "bf16n/encode.h"
#include "bf16n/launch.h"
#include "bf16n/policy.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

// the read probe of libbf16n_probe.so (bench_probe.hip): measurement only, not part of the product library
extern "C" int bf16n_probe_read(const void * src, uint64_t bytes, int pattern, int waves_per_cu, uint32_t * sink, void * stream);

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "hip error %s at line %d\n", hipGetErrorString(e_), __LINE__); std::exit(2); } } while (0)

namespace {

uint64_t splitmix64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
double uniform01(uint64_t i, uint64_t seed, uint64_t stream) {
    return ((double) (splitmix64(i + (seed << 32) + (stream << 56)) >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}
uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
float bf16_to_f32(uint16_t b) {
    const uint32_t u = (uint32_t) b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// element 2i, 2i + 1 of stream `seed`: r cos(2 pi u2), r sin(2 pi u2) with r = sqrt(-2 ln u1)
void normals_bf16(uint16_t * out, size_t n, uint64_t seed, float scale) {
    const unsigned nt = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    const size_t pairs = (n + 1) / 2;
    std::vector<std::thread> pool;
    for (unsigned t = 0; t < nt; t++) {
        pool.emplace_back([=] {
            for (size_t i = pairs * t / nt; i < pairs * (t + 1) / nt; i++) {
                const double r = std::sqrt(-2.0 * std::log(uniform01(i, seed, 1)));
                const double a = 6.283185307179586 * uniform01(i, seed, 2);
                out[2 * i] = f32_to_bf16((float) (r * std::cos(a)) * scale);
                if (2 * i + 1 < n) {
                    out[2 * i + 1] = f32_to_bf16((float) (r * std::sin(a)) * scale);
                }
            }
        });
    }
    for (auto & th : pool) {
        th.join();
    }
}

struct stats { double median_us, mean_us, best_us; };
stats summarise(std::vector<float> ms) {
    std::sort(ms.begin(), ms.end());
    double sum = 0;
    for (float v : ms) {
        sum += v;
    }
    return {ms[ms.size() / 2] * 1e3, sum / ms.size() * 1e3, ms[0] * 1e3};
}

} // namespace

int main(int argc, char ** argv) {
    int64_t rows = 248320, K = 2048;
    int batch = 1, reps = 200, copies = 2;
    double warm_ms = 500;
    bool tiles = false, x_f32 = false, probe = false;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        auto val = [&]() { return i + 1 < argc ? argv[++i] : "0"; };
        if (a == "--rows") rows = std::atoll(val());
        else if (a == "--K") K = std::atoll(val());
        else if (a == "--batch") batch = std::atoi(val());
        else if (a == "--reps") reps = std::atoi(val());
        else if (a == "--warm-ms") warm_ms = std::atof(val());
        else if (a == "--copies") copies = std::atoi(val());
        else if (a == "--tiles") tiles = true;
        else if (a == "--f32") x_f32 = true;
        else if (a == "--probe") probe = true;
        else { std::fprintf(stderr, "unknown argument %s\n", a.c_str()); return 1; }
    }
    bf16n::init();
    int cus = 0;
    bf16n::detail::check(bf16n_cu_count(&cus));

    std::vector<uint16_t> w((size_t) rows * K), x((size_t) batch * K);
    normals_bf16(w.data(), w.size(), 1, 0.02f);
    normals_bf16(x.data(), x.size(), 2, 1.0f);
    bf16n::policy_options po;
    po.engine = bf16n::policy_engine::mi355x;
    po.dense_frag_order = tiles;
    const auto ch = bf16n::choose(rows, K, 1, po);
    if (!ch) { std::fprintf(stderr, "the policy leaves this shape in BF16\n"); return 1; }
    const auto t_enc = std::chrono::steady_clock::now();
    const bf16n::encoded e = bf16n::encode(w.data(), rows, K, ch->format, ch->R, ch->chunk_major, ch->frag_order, ch->wave64);
    const double enc_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_enc).count();
    bf16n::aux_header h;
    std::memcpy(&h, e.aux.data(), sizeof h);

    hipStream_t stream;
    HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    std::vector<bf16n::weight> wt(copies);
    for (auto & v : wt) {
        uint8_t * d_plane, * d_aux;
        HIP_OK(hipMalloc(&d_plane, e.plane.size()));
        HIP_OK(hipMalloc(&d_aux, e.aux.size()));
        HIP_OK(hipMemcpy(d_plane, e.plane.data(), e.plane.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(d_aux, e.aux.data(), e.aux.size(), hipMemcpyHostToDevice));
        v.plane = d_plane; v.aux = d_aux; v.format = (int) h.format; v.K = h.K; v.rows = (int64_t) h.rows; v.R = (int) h.R;
        v.cm = h.flags & bf16n::FLAG_CHUNK_MAJOR; v.wave64 = h.flags & bf16n::FLAG_WAVE64;
        v.off_a = h.off_a; v.off_b = h.off_b; v.off_c = h.off_c; v.off_d = h.off_d;
    }
    // the load-time verify: the device decode reproduces every source bit
    int same = 0;
    const bf16n_weight cw = bf16n::detail::c_view(wt[0]);
    bf16n::detail::check(bf16n_verify_roundtrip(&cw, w.data(), &same));
    if (!same) { std::fprintf(stderr, "device decode is not bit-exact\n"); return 3; }

    void * d_x; float * d_y;
    std::vector<float> xf(x.size());
    for (size_t i = 0; i < x.size(); i++) {
        xf[i] = bf16_to_f32(x[i]);
    }
    const size_t xsz = x_f32 ? 4 : 2;
    HIP_OK(hipMalloc(&d_x, x.size() * xsz));
    HIP_OK(hipMalloc(&d_y, (size_t) batch * rows * 4));
    HIP_OK(hipMemcpy(d_x, x_f32 ? (const void *) xf.data() : (const void *) x.data(), x.size() * xsz, hipMemcpyHostToDevice));
    bf16n::mmv_args a;
    a.x = d_x; a.x_bf16 = !x_f32; a.y = d_y; a.ncols = batch; a.x_tok = K * (int64_t) xsz; a.y_tok = rows * 4;
    a.rows_per_matrix = rows; a.nrows = rows;

    // one product checked against FP64 on a sample of rows (bound of the reference's tests: 1e-5 * sum |w x|)
    bf16n::mmv(wt[0], a, stream);
    std::vector<float> y((size_t) batch * rows);
    HIP_OK(hipMemcpyAsync(y.data(), d_y, y.size() * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    double worst = 0;
    for (int64_t r = 0; r < rows; r += 997) {
        for (int t = 0; t < batch; t++) {
            double ref = 0, bound = 0;
            for (int64_t k = 0; k < K; k++) {
                const double q = (double) bf16_to_f32(w[r * K + k]) * (double) xf[t * K + k];
                ref += q;
                bound += std::fabs(q);
            }
            worst = std::max(worst, std::fabs(y[t * rows + r] - ref) / bound);
        }
    }
    if (!(worst <= 1e-5)) { std::fprintf(stderr, "product out of bound: %g\n", worst); return 4; }

    int it = 0;
    for (const auto t0 = std::chrono::steady_clock::now();
         std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() < warm_ms;) {
        for (int k = 0; k < 8; k++) {
            bf16n::mmv(wt[it++ % copies], a, stream);
        }
        HIP_OK(hipStreamSynchronize(stream));
    }
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    std::vector<float> ms(reps);
    // back to back: the whole block between two events (what a decode loop sees) ...
    HIP_OK(hipEventRecord(e0, stream));
    for (int r = 0; r < reps; r++) {
        bf16n::mmv(wt[it++ % copies], a, stream);
    }
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    float block_ms = 0;
    HIP_OK(hipEventElapsedTime(&block_ms, e0, e1));
    // ... and launch by launch, each synchronised (standalone_mmv.cu:78-83)
    for (int r = 0; r < reps; r++) {
        HIP_OK(hipEventRecord(e0, stream));
        bf16n::mmv(wt[it++ % copies], a, stream);
        HIP_OK(hipEventRecord(e1, stream));
        HIP_OK(hipEventSynchronize(e1));
        HIP_OK(hipEventElapsedTime(&ms[r], e0, e1));
    }
    const stats st = summarise(ms);
    const double comp = (double) (e.plane.size() + e.aux.size());
    const double algo = comp + (double) batch * K * xsz + (double) batch * rows * 4;
    std::printf("{\"workload\": \"%lldx%lld batch %d %s activations, format %d R %d flags %u\", \"cus\": %d, \"compressed_bytes\": %.0f, "
                "\"algorithmic_bytes\": %.0f, \"encode_s\": %.2f, \"max_err_over_sum_abs\": %.3g, \"reps\": %d, "
                "\"back_to_back_us\": %.2f, \"median_us\": %.2f, \"mean_us\": %.2f, \"best_us\": %.2f, \"GBps\": %.1f, "
                "\"frac_of_hbm_peak\": %.4f",
                (long long) rows, (long long) K, batch, x_f32 ? "FP32" : "BF16", e.format, e.R, h.flags, cus, comp, algo, enc_s, worst, reps,
                block_ms * 1e3 / reps, st.median_us, st.mean_us, st.best_us, algo / (block_ms * 1e-3 / reps) / 1e9,
                algo / (block_ms * 1e-3 / reps) / 1e9 / 8000.0);
    if (probe) {
        // a kernel that only reads as many bytes, from buffers of its own (two, alternated), in the four patterns
        const uint64_t nbytes = (uint64_t) comp / 1024 * 1024;
        uint8_t * buf[2];
        uint32_t * sink;
        HIP_OK(hipMalloc(&sink, 4));
        for (auto & b : buf) {
            HIP_OK(hipMalloc(&b, nbytes));
            HIP_OK(hipMemset(b, 0x5A, nbytes));
        }
        const char * names[4] = {"ranges_nt", "ranges_plain", "stride_nt", "stride_plain"};
        for (int p = 0; p < 4; p++) {
            for (int wpc : {8, 16, 32}) {
                for (int r = 0; r < 10; r++) {
                    if (bf16n_probe_read(buf[r & 1], nbytes, p, wpc, sink, stream) != 0) { std::fprintf(stderr, "read probe failed\n"); return 2; }
                }
                HIP_OK(hipStreamSynchronize(stream));
                std::vector<float> pm(30);
                for (int r = 0; r < 30; r++) {
                    HIP_OK(hipEventRecord(e0, stream));
                    if (bf16n_probe_read(buf[r & 1], nbytes, p, wpc, sink, stream) != 0) { std::fprintf(stderr, "read probe failed\n"); return 2; }
                    HIP_OK(hipEventRecord(e1, stream));
                    HIP_OK(hipEventSynchronize(e1));
                    HIP_OK(hipEventElapsedTime(&pm[r], e0, e1));
                }
                const stats ps = summarise(pm);
                std::printf(", \"read_%s_w%d_GBps\": %.1f", names[p], wpc, nbytes / (ps.median_us * 1e-6) / 1e9);
            }
        }
    }
    std::printf("}\n");
    return 0;
}
