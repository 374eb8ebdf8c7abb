// Load-time conversion, bit-exact verify on the device, and the registry that finds a resident tensor by the address of
// its plane bytes: what the reference's llama.cpp adapter adds on top of the core (patch
// engines/llamacpp/patches/0002-ggml-cuda-thin-BF16N-adapter-over-the-shared-core.patch: entry and lookup :64-92, free
// :121-132, choose :258-268, convert :271-329), restated without ggml types.  An engine keeps its tensor object; what
// this layer sees is the device address of the tensor's data (which holds the plane), the shape, and an owner token
// (the buffer that will be freed as a whole).
#include "bf16n_c.h"

#include "bf16n/format.h"
#include "launchers.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <functional>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

using namespace bf16n;

namespace bf16n {
namespace impl {
int report(const std::function<void()> & f); // capi.cpp: runs f, maps exceptions to a status and the thread's message
void check_weight(const bf16n_weight & w);   // capi.cpp: the launchers' contract on a weight (throws std::invalid_argument)
}
} // namespace bf16n

namespace {

struct entry {
    bf16n_weight w;
    size_t nbytes;      // plane bytes: the address range that belongs to this tensor
    const void * owner;
    bool owns_aux;      // aux was allocated by convert and is freed by release
};

std::mutex g_mutex;
std::vector<entry> g_entries; // sorted by plane address

void require(bool cond, const char * msg) {
    if (!cond) {
        throw std::invalid_argument(std::string("bf16n: ") + msg);
    }
}

void hip_check(hipError_t e, const char * what) {
    if (e != hipSuccess) {
        throw std::runtime_error(std::string("bf16n: HIP error ") + hipGetErrorString(e) + " in " + what);
    }
}

// where [plane, plane + nbytes) goes in the sorted registry; throws when the range overlaps a registered tensor.
// The caller holds g_mutex.
std::vector<entry>::iterator free_slot(const uint8_t * plane, size_t nbytes) {
    const auto less = std::less<const uint8_t *>{};
    auto it = std::upper_bound(g_entries.begin(), g_entries.end(), plane,
                               [&](const uint8_t * p, const entry & v) { return less(p, v.w.plane); });
    if (it != g_entries.begin()) {
        const entry & prev = *(it - 1);
        require(!less(plane, prev.w.plane + prev.nbytes), "adapter: the tensor overlaps a registered one");
    }
    if (it != g_entries.end()) {
        require(!less(it->w.plane, plane + nbytes), "adapter: the tensor overlaps a registered one");
    }
    return it;
}

void insert(const entry & e) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_entries.insert(free_slot(e.w.plane, e.nbytes), e);
}

// one flag for the whole comparison: any differing 16-byte piece sets it (plain stores of the same value)
__global__ void k_differs(const uint4 * a, const uint4 * b, int64_t n16, int * flag) {
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) {
        const uint4 x = a[i], y = b[i];
        if (x.x != y.x || x.y != y.y || x.z != y.z || x.w != y.w) {
            *flag = 1;
        }
    }
}

struct device_buffer {
    void * p = nullptr;
    explicit device_buffer(size_t bytes, const char * what) { hip_check(hipMalloc(&p, bytes), what); }
    ~device_buffer() { (void) hipFree(p); }
    device_buffer(const device_buffer &) = delete;
    device_buffer & operator=(const device_buffer &) = delete;
};

// decode(encoded) == source for every weight: the tensor is decoded on the device in pieces of at most 64 MiB of BF16
// (whole units), each piece compared there with the same rows of the source
bool verify_on_device(const bf16n_weight & w, const uint16_t * host) {
    impl::check_weight(w); // K, format and R are divisors below
    require(w.rows > 0, "verify: empty tensor");
    const int64_t unit = w.format == FMT_NIBBLE ? 1 : w.R;
    int64_t chunk_rows = std::max<int64_t>((64ll << 20) / (w.K * 2) / unit * unit, unit);
    chunk_rows = std::min<int64_t>(chunk_rows, w.rows);
    const size_t chunk_bytes = (size_t) chunk_rows * w.K * 2;
    device_buffer out(chunk_bytes, "hipMalloc (verify)"), src(chunk_bytes, "hipMalloc (verify)"), flag(sizeof(int), "hipMalloc (verify)");
    hip_check(hipMemset(flag.p, 0, sizeof(int)), "hipMemset");
    for (int64_t r0 = 0; r0 < w.rows; r0 += chunk_rows) {
        const int64_t nr = std::min(chunk_rows, w.rows - r0);
        const size_t bytes = (size_t) nr * w.K * 2;
        hip_check(hipMemcpy(src.p, host + r0 * w.K, bytes, hipMemcpyHostToDevice), "hipMemcpy (verify)");
        if (bf16n_dequant(&w, r0, nr, (uint16_t *) out.p, nullptr) != BF16N_OK) {
            throw std::runtime_error(bf16n_last_error());
        }
        const int64_t n16 = (int64_t) (bytes / 16); // K is a multiple of 512: rows are whole 16-byte pieces
        hipLaunchKernelGGL(k_differs, dim3((unsigned) ((n16 + 255) / 256)), dim3(256), 0, nullptr, (const uint4 *) out.p,
                           (const uint4 *) src.p, n16, (int *) flag.p);
        hip_check(hipGetLastError(), "verify");
    }
    int differs = 0;
    hip_check(hipMemcpy(&differs, flag.p, sizeof(int), hipMemcpyDeviceToHost), "hipMemcpy (verify)");
    return differs == 0;
}

bf16n_weight view_of(const uint8_t * plane, const uint8_t * aux_dev, const aux_header & h, int format, int R) {
    bf16n_weight w = {};
    w.plane = plane;
    w.aux = aux_dev;
    w.format = format;
    w.R = R;
    w.K = h.K;
    w.rows = (int64_t) h.rows;
    w.flags = h.flags;
    w.off_a = h.off_a; w.off_b = h.off_b; w.off_c = h.off_c; w.off_d = h.off_d;
    return w;
}

} // namespace

extern "C" {

// patch 0002:258-268: 0 = the tensor stays BF16, 1 = NIBBLE, 2 = the Huffman family (pairs, single-symbol fallback)
int bf16n_adapter_choose(int64_t rows, int64_t K, int64_t n_matrices, const char * mode, int64_t dense_min, int expert, int engine) {
    const int m = mode && strcmp(mode, "nibble") == 0 ? BF16N_MODE_NIBBLE : mode && strcmp(mode, "huffman") == 0 ? BF16N_MODE_HUFFMAN
                                                                                                                   : BF16N_MODE_HYBRID;
    int out[5] = {0, 0, 0, 0, 0};
    if (!bf16n_choose(rows, K, n_matrices, engine, m, dense_min, expert, 0, out)) {
        return 0;
    }
    return out[0] == BF16N_FMT_NIBBLE ? 1 : 2;
}

// patch 0002:271-329
int bf16n_adapter_convert(void * tensor_data, const void * bf16_host, int64_t rows_per_matrix, int64_t K, int64_t n_matrices,
                          int format_tag, int engine, int matrix_core_order, const void * owner, const char * name, int verbose,
                          int * roundtrip_ok) {
    return impl::report([&] {
        require(tensor_data && bf16_host && roundtrip_ok, "adapter: null pointer");
        require(format_tag == 1 || format_tag == 2, "adapter: format tag must be 1 (NIBBLE) or 2 (Huffman family)");
        require(rows_per_matrix > 0 && n_matrices > 0, "adapter: empty tensor");
        require(((uintptr_t) tensor_data & 15) == 0, "adapter: tensor data must be 16-byte aligned");
        *roundtrip_ok = 0;
        if (bf16n_init() != BF16N_OK) {
            throw std::runtime_error(bf16n_last_error());
        }
        // the explicit format is the caller's decision (its own choose call); the shape policy tunes units and layout
        int c[5] = {0, 0, 0, 0, 0};
        require(bf16n_choose(rows_per_matrix, K, n_matrices, engine, format_tag == 1 ? BF16N_MODE_NIBBLE : BF16N_MODE_HUFFMAN, 0,
                             n_matrices > 1, matrix_core_order, c) != 0,
                "adapter: K must be a multiple of 512 in [512, 4096]");
        const int64_t rows = rows_per_matrix * n_matrices;
        {
            // a tensor that overlaps a registered one is refused before anything is written into it
            std::lock_guard<std::mutex> lock(g_mutex);
            (void) free_slot((const uint8_t *) tensor_data, (size_t) (rows * K));
        }
        const uint32_t flags = (c[2] ? FLAG_CHUNK_MAJOR : 0) | (c[3] ? FLAG_FRAG_ORDER : 0) | (c[4] ? FLAG_WAVE64 : 0);
        bf16n_encoded * enc = nullptr;
        if (bf16n_encode((const uint16_t *) bf16_host, rows, K, c[0], c[1], flags, &enc) != BF16N_OK) {
            throw std::invalid_argument(bf16n_last_error());
        }
        struct guard {
            bf16n_encoded * e;
            ~guard() { bf16n_encoded_free(e); }
        } g{enc};
        uint64_t plane_bytes = 0, aux_bytes = 0;
        const uint8_t * plane = bf16n_encoded_plane(enc, &plane_bytes);
        const uint8_t * aux = bf16n_encoded_aux(enc, &aux_bytes);
        hip_check(hipMemcpy(tensor_data, plane, plane_bytes, hipMemcpyHostToDevice), "hipMemcpy (plane)");
        void * aux_dev = nullptr;
        hip_check(hipMalloc(&aux_dev, aux_bytes), "hipMalloc (aux)");
        entry e;
        try {
            hip_check(hipMemcpy(aux_dev, aux, aux_bytes, hipMemcpyHostToDevice), "hipMemcpy (aux)");
            aux_header h;
            memcpy(&h, aux, sizeof(h));
            e.w = view_of((const uint8_t *) tensor_data, (const uint8_t *) aux_dev, h, bf16n_encoded_format(enc), bf16n_encoded_R(enc));
            e.nbytes = (size_t) plane_bytes;
            e.owner = owner;
            e.owns_aux = true;
            insert(e);
        } catch (...) {
            (void) hipFree(aux_dev);
            throw;
        }
        const bool ok = verify_on_device(e.w, (const uint16_t *) bf16_host);
        *roundtrip_ok = ok ? 1 : 0;
        if (verbose) {
            fprintf(stderr, "bf16n: %-32s %s K=%5lld rows=%7lld R=%2d%s ratio=%.4f roundtrip=%s\n", name ? name : "",
                    e.w.format == FMT_HUFPAIR ? "hufpair" : e.w.format == FMT_HUFFMAN ? "huffman" : "nibble ", (long long) K,
                    (long long) rows, e.w.R, (e.w.flags & FLAG_WAVE64) ? (e.w.R == TILE_R ? " tiles " : " wave64") : "",
                    double(plane_bytes + aux_bytes) / double(rows * K * 2), ok ? "OK" : "FAIL");
        }
    });
}

// decode(encoded) == host source, compared on the device (the load-time verify on its own)
int bf16n_verify_roundtrip(const bf16n_weight * w, const uint16_t * bf16_host, int * ok) {
    return impl::report([&] {
        require(w && bf16_host && ok, "verify: null pointer");
        *ok = verify_on_device(*w, bf16_host) ? 1 : 0;
    });
}

// a tensor encoded and uploaded by the caller joins the registry; its aux buffer stays the caller's
int bf16n_adapter_register(const bf16n_weight * w, const void * owner) {
    return impl::report([&] {
        require(w && w->plane && w->aux && w->rows > 0 && w->K > 0, "adapter: incomplete weight");
        entry e;
        e.w = *w;
        e.nbytes = (size_t) (w->rows * w->K);
        e.owner = owner;
        e.owns_aux = false;
        insert(e);
    });
}

// patch 0002:73-92: the tensor whose plane holds address p (a view of whole rows: p may point at any row start);
// *found = 0 when no registered tensor does.  The weight is returned by value: entries move when tensors come and go.
int bf16n_adapter_lookup(const void * p, bf16n_weight * out, int64_t * row0, int * found) {
    return impl::report([&] {
        require(out && row0 && found, "adapter: null pointer");
        *found = 0;
        std::lock_guard<std::mutex> lock(g_mutex);
        const auto q = static_cast<const uint8_t *>(p);
        const auto less = std::less<const uint8_t *>{};
        auto it = std::upper_bound(g_entries.begin(), g_entries.end(), q,
                                   [&](const uint8_t * a, const entry & e) { return less(a, e.w.plane); });
        if (it == g_entries.begin()) {
            return;
        }
        --it;
        if (!less(q, it->w.plane + it->nbytes)) {
            return;
        }
        const size_t off = (size_t) (q - it->w.plane);
        require(off % (size_t) it->w.K == 0, "adapter: the address is not the start of a row");
        *out = it->w;
        *row0 = (int64_t) (off / (size_t) it->w.K);
        *found = 1;
    });
}

// patch 0002:121-132: before the owning buffer is freed; returns the number of tensors dropped through *n
int bf16n_adapter_release(const void * owner, int * n) {
    return impl::report([&] {
        int dropped = 0;
        std::lock_guard<std::mutex> lock(g_mutex);
        for (auto it = g_entries.begin(); it != g_entries.end();) {
            if (it->owner == owner) {
                if (it->owns_aux) {
                    hip_check(hipFree(const_cast<uint8_t *>(it->w.aux)), "hipFree (aux)");
                }
                it = g_entries.erase(it);
                dropped++;
            } else {
                ++it;
            }
        }
        if (n) {
            *n = dropped;
        }
    });
}

int bf16n_adapter_count(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    return (int) g_entries.size();
}

} // extern "C"
