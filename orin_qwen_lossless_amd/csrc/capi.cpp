// C ABI of libbf16n_hip.so (include/bf16n_c.h): argument checks, dispatch and error reporting.  Contract checks and
// messages follow the reference launchers (core/src/launch.cu:261-582) so that callers and tests written against the
// reference see the same failures.  This file and the .hip files are the only places that call HIP.
#include "bf16n_c.h"

#include "encode_impl.h"
#include "dev_topk.h"
#include "launchers.h"

#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <functional>
#include <mutex>
#include <stdexcept>
#include <string>

using namespace bf16n;

struct bf16n_encoded {
    impl::encoded_buffers b;
};

namespace {

thread_local std::string g_error;
thread_local std::string g_kernel_text;

int g_cus = 0;
int g_lds_max = 0;
std::once_flag g_once;

// Routing lists of bf16n_moe_mm_ids_static: device memory that belongs to the library, so that the call allocates
// nothing.  Every GPU holds its own copy of the array for the life of the process (about 516 KiB).  In host code the
// array's name is not a device address; the address on a device comes from hipGetSymbolAddress with that device
// current, once per device (route_lists_of_current_device), and only that pointer is handed to kernels.
constexpr int STATIC_MAX_PAIRS = 1 << 16;   // routed (token, slot) pairs per call: 8192 tokens of top-8
constexpr int STATIC_MAX_EXPERTS = 1024;
struct route_lists {
    int32_t src1[STATIC_MAX_PAIRS];
    int32_t dst[STATIC_MAX_PAIRS];
    int32_t bounds[STATIC_MAX_EXPERTS + 64];
};
static __device__ __align__(256) unsigned char scratch[sizeof(route_lists)];

constexpr int MAX_DEVICES = 64;
route_lists * g_route_lists[MAX_DEVICES] = {};
std::mutex g_route_lists_mutex;

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

route_lists * route_lists_of_current_device() {
    int dev = 0;
    hip_check(hipGetDevice(&dev), "hipGetDevice");
    if (dev < 0 || dev >= MAX_DEVICES) {
        throw std::runtime_error("bf16n: device ordinal beyond the library's per-device tables");
    }
    std::lock_guard<std::mutex> lock(g_route_lists_mutex);
    if (!g_route_lists[dev]) {
        void * p = nullptr;
        hip_check(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress (routing lists)");
        g_route_lists[dev] = static_cast<route_lists *>(p);
    }
    return g_route_lists[dev];
}

void ensure_init() {
    std::call_once(g_once, [] {
        int dev = 0;
        hip_check(hipGetDevice(&dev), "hipGetDevice");
        hip_check(hipDeviceGetAttribute(&g_cus, hipDeviceAttributeMultiprocessorCount, dev), "hipDeviceGetAttribute");
        hip_check(hipDeviceGetAttribute(&g_lds_max, hipDeviceAttributeMaxSharedMemoryPerBlock, dev), "hipDeviceGetAttribute");
        dev::w64_init();
        dev::mm_ids_init();
        dev::tile_init();
    });
    (void) route_lists_of_current_device(); // per device; after the first call on a device this is a table lookup
}

template <typename F>
int guarded(F && f) {
    try {
        f();
        return BF16N_OK;
    } catch (const std::invalid_argument & e) {
        g_error = e.what();
        return BF16N_EINVAL;
    } catch (const std::exception & e) {
        g_error = e.what();
        return BF16N_ERUNTIME;
    }
}

} // namespace

namespace bf16n {
namespace impl {
// for the other translation units of the C ABI: run f, map exceptions to a status and the calling thread's message
int report(const std::function<void()> & f) { return guarded(f); }
} // namespace impl
} // namespace bf16n

namespace {

void check_weight(const bf16n_weight & w);

} // namespace

namespace bf16n {
namespace impl {
void check_weight(const bf16n_weight & w) { ::check_weight(w); }
} // namespace impl
} // namespace bf16n

namespace {

// launch.cu:261-268
void check_weight(const bf16n_weight & w) {
    require(w.K % 512 == 0 && w.K >= 512 && w.K <= K_MAX, "K must be a multiple of 512 in [512, 4096]");
    require(w.format == FMT_NIBBLE || w.format == FMT_HUFFMAN || w.format == FMT_HUFPAIR, "unknown format");
    require(w.rows >= 0, "rows must be nonnegative");
    require(w.format == FMT_NIBBLE || (w.R > 0 && w.rows % w.R == 0), "rows must be a multiple of R");
    require(!(w.flags & FLAG_CHUNK_MAJOR) || w.format == FMT_HUFPAIR, "chunk-major units exist only for HUFPAIR");
    require(!(w.flags & FLAG_FRAG_ORDER), "fragment-order weights are not supported by the MI355X build");
    require(!(w.flags & FLAG_WAVE64) || (w.format == FMT_HUFPAIR && !(w.flags & FLAG_CHUNK_MAJOR)),
            "the wave64 layout exists only for row-major HUFPAIR");
    require(!(w.flags & ~(FLAG_CHUNK_MAJOR | FLAG_FRAG_ORDER | FLAG_WAVE64)), "unknown layout flags");
    require(w.format == FMT_NIBBLE || w.R <= 16 || dev::is_tile_layout(w), "R = 32 exists only as wave64 HUFPAIR tiles");
}

bool is_w64(const bf16n_weight & w) { return (w.flags & FLAG_WAVE64) != 0; }

dev::cols make_cols(const bf16n_mmv_args & a) { // launch.cu:69-84
    dev::cols p = {};
    p.x = (const char *) a.x;
    p.y = (char *) a.y;
    p.x_tok = a.x_tok; p.y_tok = a.y_tok;
    p.ids = (const char *) a.ids;
    p.ids_s0 = a.ids_s0; p.ids_s1 = a.ids_s1;
    p.n_used = a.ids ? a.n_used : 1;
    p.x_per_slot = a.x_per_slot > 0 ? a.x_per_slot : 1;
    p.x_slot = a.x_slot; p.y_slot = a.y_slot;
    p.rows_per_matrix = a.rows_per_matrix;
    p.row0 = a.row0;
    p.nrows = a.nrows;
    p.y_bf16 = a.y_bf16 != 0;
    return p;
}

// dense products of a tile-layout matrix that go through the matrix cores: BF16 activations (or a few FP32 columns),
// rows enough to fill the GPU, and the 16-byte alignment of x rows and y columns that the kernel's vector accesses need
bool tile_dense_mm(const bf16n_weight & w, const bf16n_mmv_args & a) {
    if (a.ids || !dev::tile_mm_dense_pays(w, a.nrows, g_cus)) {
        return false;
    }
    const int64_t ya = a.y_bf16 ? 8 : 16;
    return ((uintptr_t) a.x & 15) == 0 && ((uintptr_t) a.y & 15) == 0 && (a.ncols == 1 || (a.x_tok % 16 == 0 && a.y_tok % ya == 0));
}

void launch_check(const char * what) { hip_check(hipGetLastError(), what); }

} // namespace

namespace bf16n {
namespace dev {
thread_local kernel_note g_last_kernel = {nullptr, nullptr, 0, {0, 0, 0, 0, 0}};
} // namespace dev
} // namespace bf16n

extern "C" {

const char * bf16n_last_error(void) { return g_error.c_str(); }

// ---------------------------------------------------------------- encoder / policy

int bf16n_encode(const uint16_t * w, int64_t rows, int64_t K, int format, int R, uint32_t flags, bf16n_encoded ** out) {
    return guarded([&] {
        require(out != nullptr, "encode: null output");
        *out = nullptr;
        auto * e = new bf16n_encoded;
        try {
            e->b = impl::encode(w, rows, K, format, R, flags);
        } catch (...) {
            delete e;
            throw;
        }
        *out = e;
    });
}

const uint8_t * bf16n_encoded_plane(const bf16n_encoded * e, uint64_t * bytes) {
    if (bytes) {
        *bytes = e->b.plane.size();
    }
    return e->b.plane.data();
}
const uint8_t * bf16n_encoded_aux(const bf16n_encoded * e, uint64_t * bytes) {
    if (bytes) {
        *bytes = e->b.aux.size();
    }
    return e->b.aux.data();
}
int bf16n_encoded_format(const bf16n_encoded * e) { return e->b.format; }
int bf16n_encoded_R(const bf16n_encoded * e) { return e->b.R; }
void bf16n_encoded_free(bf16n_encoded * e) { delete e; }
void bf16n_set_encode_threads(int n) { impl::set_threads(n); }

int bf16n_choose(int64_t rows, int64_t K, int64_t n_matrices, int engine, int mode, int64_t dense_min, int expert,
                 int dense_frag_order, int * out) {
    impl::choice c;
    if (!impl::choose(rows, K, n_matrices, engine, mode, dense_min, expert != 0, dense_frag_order != 0, c)) {
        return 0;
    }
    out[0] = c.format; out[1] = c.R; out[2] = c.chunk_major; out[3] = c.frag_order; out[4] = c.wave64;
    return 1;
}

// ---------------------------------------------------------------- launchers

int bf16n_init(void) {
    return guarded([] { ensure_init(); });
}

int bf16n_cu_count(int * out) {
    return guarded([&] {
        ensure_init();
        *out = g_cus;
    });
}

// launch.cu:313-325
int bf16n_mmv(const bf16n_weight * w, const bf16n_mmv_args * a, void * stream, int multi_col) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(a->ncols > 0 && a->ncols <= 65535, "ncols out of range");
        require(w->format == FMT_NIBBLE || (a->nrows % w->R == 0 && a->row0 % w->R == 0 && a->rows_per_matrix % w->R == 0),
                "rows of a product must be whole units");
        if (a->nrows == 0) {
            return;
        }
        const dev::cols p = make_cols(*a);
        if (dev::is_tile_layout(*w) && tile_dense_mm(*w, *a)) {
            // a large dense matrix through the matrix cores: any number of BF16 columns, or up to ten FP32 columns as
            // three BF16 components each
            const int per_launch = a->x_bf16 ? a->ncols : dev::TILE_DENSE_F32_COLS;
            for (int c0 = 0; c0 < a->ncols; c0 += per_launch) {
                const int nc = a->ncols - c0 < per_launch ? a->ncols - c0 : per_launch;
                dev::launch_tile_mm_dense(*w, a->row0, a->nrows, (const char *) a->x + c0 * a->x_tok, a->x_bf16 != 0,
                                          a->x_tok / (a->x_bf16 ? 2 : 4), nc, (char *) a->y + c0 * a->y_tok, a->y_bf16 != 0,
                                          a->y_tok / (a->y_bf16 ? 2 : 4), g_cus, (hipStream_t) stream);
            }
        } else if (dev::is_tile_layout(*w)) {
            dev::launch_tile_mmv(*w, nullptr, p, a->ncols, a->x_bf16 != 0, (hipStream_t) stream);
        } else if (is_w64(*w)) {
            require(dev::w64_mmv_supported(*w, a->x_bf16 != 0), "no wave64 GEMV kernel for this K / R (K in {512, 1024, 2048, 4096})");
            dev::launch_w64_mmv(*w, p, a->ncols, a->x_bf16 != 0, multi_col != 0, g_cus, (hipStream_t) stream);
        } else {
            dev::launch_compat_mmv(*w, nullptr, 0, p, a->ncols, a->x_bf16 != 0, g_cus, (hipStream_t) stream, multi_col != 0);
        }
        launch_check("mmv");
    });
}

// The kernel instance that the calling thread's last bf16n_mmv / bf16n_mmv_glu2 launch chose, as the profiler prints it
// ("k_w64_mmv<bf16_t, 4, 1, 2, 1>"); an empty string before the first launch or after a launch on a path that leaves
// no note.  The pointer stays valid until the thread's next call of this function.
const char * bf16n_last_kernel(void) {
    const dev::kernel_note & k = dev::g_last_kernel;
    g_kernel_text.clear();
    if (k.name) {
        g_kernel_text = std::string(k.name) + "<" + (k.tx ? k.tx : "");
        for (int i = 0; i < k.n_args; i++) {
            g_kernel_text += (i || k.tx ? ", " : "") + std::to_string(k.arg[i]);
        }
        g_kernel_text += ">";
    }
    return g_kernel_text.c_str();
}

// The number of BF16 token columns up to which bf16n_mmv is the faster dense path; beyond it dequant + a stock GEMM is.
// 8 is the reference's fixed rule (core/torch/torch_bindings.cpp:195); matrices whose products run on the matrix cores
// stay ahead for far longer (every pass of up to 128 columns decodes the matrix once).
int bf16n_gemv_max_tokens(const bf16n_weight * w, int * out) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(out != nullptr, "null output");
        if (dev::is_tile_layout(*w) && dev::tile_mm_dense_pays(*w, w->rows, g_cus)) {
            *out = 512;
        } else if (is_w64(*w) && !dev::is_tile_layout(*w) && dev::w64_mmv_supported(*w, true) && w->K <= 2048 &&
                   w->rows * w->K >= ((int64_t) 1 << 27)) {
            // a large matrix in wave64 units: two launches of eight columns per decode (2 x 302 us on 248320 x 2048)
            // still beat writing and re-reading the whole matrix as BF16 (dequant + GEMM: 820 us)
            *out = 16;
        } else if (w->format == FMT_NIBBLE) {
            // the 4-bit code has no decode chain: batches go through the matrix cores, 32 tokens per decode of the
            // matrix (5120 x 2048: 11-13 us up to 32 tokens, 20 us up to 64, where dequant + GEMM takes 20-21 us;
            // 2048 x 4096: 17-21 us against 22-28 us), where the dispatch takes that kernel for every count from 9 to
            // 64; matrices of up to 256 rows run their GEMV columns side by side on idle CUs (4.9-9.5 us for 9-64
            // columns); between the two the GEMV columns lose to dequant + GEMM beyond the reference's 8
            // (the 16-row kernel takes over where its launch is at most two blocks per CU: 1024 x 2048 6.5-6.8 us up to
            // 64 columns against 15.4 us for dequant + GEMM)
            bool all_counts = true;
            for (int n = 9; n <= 64 && all_counts; n++) {
                all_counts = dev::nib_mm_pays(*w, w->rows, n, g_cus) || dev::nib_mm16_pays(*w, w->rows, n, g_cus);
            }
            *out = all_counts || w->rows <= 256 ? 64 : dev::nib_mm16_pays(*w, w->rows, 16, g_cus) ? 16 : 8;
        } else {
            *out = 8;
        }
    });
}

// launch.cu:327-339
int bf16n_mmv_glu(const bf16n_weight * w, const bf16n_mmv_args * a, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(w->format == FMT_NIBBLE, "mmv_glu supports NIBBLE matrices only");
        require(a->rows_per_matrix == 2 * a->nrows, "mmv_glu: rows per matrix must be [gate; up] of nrows each");
        require(a->ncols > 0 && a->ncols <= 65535, "ncols out of range");
        if (a->nrows == 0) {
            return;
        }
        dev::launch_compat_mmv(*w, nullptr, 1, make_cols(*a), a->ncols, a->x_bf16 != 0, g_cus, (hipStream_t) stream);
        launch_check("mmv_glu");
    });
}

// launch.cu:341-365
int bf16n_mmv_glu2(const bf16n_weight * gate, const bf16n_weight * up, const bf16n_mmv_args * a, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*gate);
        check_weight(*up);
        require(gate->format == up->format && gate->K == up->K, "mmv_glu: gate/up format and K must match");
        require(gate->rows == up->rows, "mmv_glu: gate/up row counts must match");
        require(a->row0 >= 0 && a->nrows >= 0 && a->row0 <= gate->rows && a->nrows <= gate->rows - a->row0,
                "mmv_glu: product rows out of range");
        require(!(gate->flags & FLAG_CHUNK_MAJOR) && !(up->flags & FLAG_CHUNK_MAJOR),
                "mmv_glu: chunk-major weights require separate mmv launches");
        require(is_w64(*gate) == is_w64(*up), "mmv_glu: gate/up layouts must match");
        require(gate->format == FMT_NIBBLE || gate->R == up->R, "mmv_glu: gate/up R must match");
        require(!is_w64(*gate) || dev::is_tile_layout(*gate) || dev::w64_mmv_supported(*gate, a->x_bf16 != 0),
                "mmv_glu: no fused kernel for this wave64 shape");
        require(a->ncols > 0 && a->ncols <= 65535, "ncols out of range");
        require(gate->format == FMT_NIBBLE || (a->nrows % gate->R == 0 && a->row0 % gate->R == 0 && a->rows_per_matrix % gate->R == 0),
                "rows of a product must be whole units");
        if (a->nrows == 0) {
            return;
        }
        if (dev::is_tile_layout(*gate)) {
            dev::launch_tile_mmv(*gate, up, make_cols(*a), a->ncols, a->x_bf16 != 0, (hipStream_t) stream);
        } else if (is_w64(*gate)) {
            dev::launch_w64_glu(*gate, *up, make_cols(*a), a->ncols, a->x_bf16 != 0, g_cus, (hipStream_t) stream);
        } else {
            dev::launch_compat_mmv(*gate, up, 2, make_cols(*a), a->ncols, a->x_bf16 != 0, g_cus, (hipStream_t) stream);
        }
        launch_check("mmv_glu");
    });
}

// No counterpart in the reference (whose engines run the router's top-k as a launch of their own): bf16n_mmv_glu2 over
// routed experts that selects the experts in its own prologue.
int bf16n_mmv_glu2_topk(const bf16n_weight * gate, const bf16n_weight * up, const bf16n_mmv_args * a, const float * logits,
                        int64_t logits_stride, int n_experts, int k, int renorm, float * weights, int64_t weights_stride, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*gate);
        check_weight(*up);
        require(dev::is_tile_layout(*gate) && dev::is_tile_layout(*up) && gate->K == up->K && gate->rows == up->rows,
                "mmv_glu2_topk: gate / up must be expert stacks of the same shape in the tile layout");
        require(logits && weights && a->ids, "mmv_glu2_topk: null pointer");
        require(n_experts > 0 && n_experts <= 256 && k > 0 && k <= n_experts && k <= 64 && k <= a->n_used,
                "mmv_glu2_topk: need 0 < k <= min(n_experts, slots, 64) and at most 256 experts");
        require(a->ids_s0 == 4 && a->x_bf16, "mmv_glu2_topk: int32 id rows and BF16 activations");
        require(a->ncols > 0 && a->ncols <= 65535 && a->ncols % a->n_used == 0, "ncols must be tokens x slots");
        require(a->nrows > 0 && a->nrows % gate->R == 0 && a->row0 % gate->R == 0 && a->rows_per_matrix % gate->R == 0,
                "rows of a product must be whole units");
        require(a->row0 >= 0 && a->row0 + a->nrows <= a->rows_per_matrix && (int64_t) n_experts * a->rows_per_matrix <= gate->rows,
                "mmv_glu2_topk: product rows out of range");
        const dev::topk_args ta = {logits, logits_stride, n_experts, k, renorm != 0, weights, weights_stride};
        dev::launch_tile_mmv(*gate, up, make_cols(*a), a->ncols, true, (hipStream_t) stream, &ta);
        launch_check("mmv_glu2_topk");
    });
}

// launch.cu:367-402
int bf16n_dequant(const bf16n_weight * w, int64_t row0, int64_t nrows, uint16_t * out, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(row0 >= 0 && nrows >= 0 && row0 + nrows <= w->rows, "dequant rows out of range");
        if (nrows == 0) {
            return;
        }
        if (w->format != FMT_NIBBLE) {
            require(nrows % w->R == 0 && row0 % w->R == 0, "dequant rows must be whole units");
        }
        if (dev::is_tile_layout(*w)) {
            dev::launch_tile_dequant(*w, row0, nrows, out, (hipStream_t) stream);
        } else if (is_w64(*w)) {
            dev::launch_w64_dequant(*w, row0, nrows, out, g_cus, (hipStream_t) stream);
        } else {
            dev::launch_compat_dequant(*w, row0, nrows, out, g_cus, (hipStream_t) stream);
        }
        launch_check("dequant");
    });
}

// launch.cu:404-443
int bf16n_get_rows(const bf16n_weight * w, const void * ids, int64_t ids_s0, int64_t n, void * dst, int dst_bf16,
                   int64_t dst_s1, void * stream, int64_t row0) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(n >= 0, "get_rows: n must be nonnegative");
        require(row0 >= 0 && (n == 0 ? row0 <= w->rows : row0 < w->rows), "get_rows: row0 out of range");
        require(!(w->flags & FLAG_CHUNK_MAJOR), "get_rows of a chunk-major (expert) matrix");
        require(w->format != FMT_HUFFMAN, "get_rows is not implemented for the single-symbol Huffman format");
        if (n == 0) {
            return;
        }
        if (dev::is_tile_layout(*w)) {
            dev::launch_tile_get_rows(*w, ids, ids_s0, n, dst, dst_bf16 != 0, dst_s1, row0, (hipStream_t) stream);
        } else if (is_w64(*w)) {
            dev::launch_w64_get_rows(*w, ids, ids_s0, n, dst, dst_bf16 != 0, dst_s1, row0, (hipStream_t) stream);
        } else {
            dev::launch_compat_get_rows(*w, ids, ids_s0, n, dst, dst_bf16 != 0, dst_s1, row0, (hipStream_t) stream);
        }
        launch_check("get_rows");
    });
}

int bf16n_mm_ids_supported(const bf16n_weight * w, const bf16n_weight * up) { return dev::mm_ids_shape_ok(*w, up) ? 1 : 0; }

// launch.cu:458-471
int bf16n_mm_ids_route(const void * ids, int ids_i64, int64_t ids_row_stride, int32_t * ids_src1, int32_t * ids_dst,
                       int32_t * bounds, int n_experts, int n_tok, int n_used, int nchannels_y, int sis1, void * stream) {
    return guarded([&] {
        ensure_init();
        require(n_tok > 0 && n_tok < (1 << 22) && n_used > 0 && n_used < (1 << 10), "routing sizes out of range");
        require(n_experts > 0, "routing sizes out of range");
        require((int64_t) n_tok * ids_row_stride < INT32_MAX, "routing ids too large for 32-bit indexing");
        dev::launch_route(ids, ids_i64 != 0, ids_row_stride, ids_src1, ids_dst, bounds, n_experts, n_tok, n_used, nchannels_y, sis1,
                          (hipStream_t) stream);
        launch_check("mm_ids_route");
    });
}

// launch.cu:473-535
int bf16n_mm_ids(const bf16n_weight * w, const bf16n_weight * up, const void * x_bf16, int64_t x_row,
                 const int32_t * ids_src1, const int32_t * ids_dst, const int32_t * bounds, void * dst, int dst_bf16,
                 int64_t dst_col, int n_experts, int n_tok, int n_used, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(dev::mm_ids_shape_ok(*w, up), "no batched kernel for this matrix");
        require(n_experts > 0 && w->rows % n_experts == 0, "rows must split evenly into experts");
        if (up) {
            check_weight(*up);
        }
        require(x_bf16 && dst && ids_src1 && ids_dst && bounds, "null pointer");
        require(((uintptr_t) x_bf16 & 15) == 0 && x_row % 8 == 0, "activations must be 16-byte aligned with 16-byte row strides");
        require(((uintptr_t) dst & 15) == 0 && dst_col % 4 == 0, "dst must be 16-byte aligned with a column stride that is a multiple of 4");
        if (w->format == FMT_NIBBLE) {
            dev::launch_nib_mm_ids(*w, up, x_bf16, x_row, ids_src1, ids_dst, bounds, dst, dst_bf16 != 0, dst_col, n_experts,
                                   (int64_t) n_tok * n_used, g_cus, (hipStream_t) stream);
        } else if (dev::is_tile_layout(*w)) {
            dev::launch_tile_mm_ids(*w, up, x_bf16, x_row, ids_src1, ids_dst, bounds, dst, dst_bf16 != 0, dst_col, n_experts,
                                    (int64_t) n_tok * n_used, g_cus, (hipStream_t) stream);
        } else {
            dev::launch_mm_ids(*w, up, x_bf16, x_row, ids_src1, ids_dst, bounds, dst, dst_bf16 != 0, dst_col, n_experts, n_tok, n_used,
                               g_cus, (hipStream_t) stream);
        }
        launch_check("mm_ids");
    });
}

// No counterpart in the reference.  bf16n_mm_ids for calls with many tokens per expert, in two phases through a scratch
// buffer of the caller's: groups of experts are decoded once into the scratch (as BF16, in matrix-core operand order)
// and multiplied from there.  The result is the one of bf16n_mm_ids up to the order of the FP32 sums, which is the same
// here (the same instruction sequence per output element).
int bf16n_mm_ids_scratch_bytes(const bf16n_weight * w, const bf16n_weight * up, int n_experts, uint64_t * per_expert, uint64_t * advised) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(per_expert && advised, "null output");
        require(dev::is_tile_layout(*w) && (!up || dev::is_tile_layout(*up)), "the two-phase batched product takes the tile layout only");
        require(n_experts > 0 && w->rows % n_experts == 0, "rows must split evenly into experts");
        *per_expert = dev::tile_mm_ids_scratch_per_expert(*w, up, n_experts);
        // a group of experts should stay in the 256 MB last-level cache between its two kernels: about half of it
        const uint64_t want = (uint64_t) 128 << 20;
        uint64_t g = want / *per_expert;
        g = g < 1 ? 1 : g > (uint64_t) n_experts ? (uint64_t) n_experts : g;
        *advised = g * *per_expert;
    });
}

int bf16n_mm_ids_scratch(const bf16n_weight * w, const bf16n_weight * up, const void * x_bf16, int64_t x_row,
                         const int32_t * ids_src1, const int32_t * ids_dst, const int32_t * bounds, void * dst, int dst_bf16,
                         int64_t dst_col, int n_experts, void * scratch, uint64_t scratch_bytes, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        if (up) {
            check_weight(*up);
        }
        require(dev::is_tile_layout(*w) && (!up || (dev::is_tile_layout(*up) && up->rows == w->rows && up->K == w->K)),
                "the two-phase batched product takes the tile layout only");
        require(n_experts > 0 && w->rows % n_experts == 0, "rows must split evenly into experts");
        require(x_bf16 && dst && ids_dst && bounds && scratch, "null pointer");
        require(((uintptr_t) x_bf16 & 15) == 0 && x_row % 8 == 0, "activations must be 16-byte aligned with 16-byte row strides");
        require(((uintptr_t) dst & 15) == 0 && dst_col % 4 == 0, "dst must be 16-byte aligned with a column stride that is a multiple of 4");
        dev::launch_tile_mm_ids_expand(*w, up, x_bf16, x_row, ids_src1, ids_dst, bounds, dst, dst_bf16 != 0, dst_col, n_experts, scratch,
                                       scratch_bytes, g_cus, (hipStream_t) stream);
        launch_check("mm_ids_scratch");
    });
}

// Routing lists + batched product in one call that allocates nothing: the lists live in the library's own device array
// (see `scratch` above).  No counterpart in the reference, whose callers allocate the lists per call.
int bf16n_moe_mm_ids_static(const bf16n_weight * w, const bf16n_weight * up, const void * x_bf16, int64_t x_row, const void * ids,
                            int ids_i64, int64_t ids_row_stride, int per_slot, void * dst, int dst_bf16, int64_t dst_col,
                            int n_experts, int n_tok, int n_used, void * stream) {
    return guarded([&] {
        ensure_init();
        check_weight(*w);
        require(dev::mm_ids_shape_ok(*w, up), "no batched kernel for this matrix");
        require(n_experts > 0 && w->rows % n_experts == 0, "rows must split evenly into experts");
        if (up) {
            check_weight(*up);
        }
        require(x_bf16 && dst && ids, "null pointer");
        require(n_tok > 0 && n_used > 0 && n_used < (1 << 10), "routing sizes out of range");
        require(n_experts <= STATIC_MAX_EXPERTS && (int64_t) n_tok * n_used <= STATIC_MAX_PAIRS,
                "moe_mm_ids_static: at most 65536 routed pairs and 1024 experts per call (use mm_ids_route + mm_ids beyond)");
        require((int64_t) n_tok * ids_row_stride < INT32_MAX, "routing ids too large for 32-bit indexing");
        require(((uintptr_t) x_bf16 & 15) == 0 && x_row % 8 == 0, "activations must be 16-byte aligned with 16-byte row strides");
        require(((uintptr_t) dst & 15) == 0 && dst_col % 4 == 0, "dst must be 16-byte aligned with a column stride that is a multiple of 4");
        route_lists * r = route_lists_of_current_device();
        const int nch = per_slot ? n_used : 1; // activations per (token, slot), as the down product takes them, or per token
        // every list entry and every bound the product reads is rewritten by the routing kernel: nothing to clear
        dev::launch_route(ids, ids_i64 != 0, ids_row_stride, r->src1, r->dst, r->bounds, n_experts, n_tok, n_used, nch, nch,
                          (hipStream_t) stream);
        launch_check("mm_ids_route");
        if (w->format == FMT_NIBBLE) {
            dev::launch_nib_mm_ids(*w, up, x_bf16, x_row, r->src1, r->dst, r->bounds, dst, dst_bf16 != 0, dst_col, n_experts,
                                   (int64_t) n_tok * n_used, g_cus, (hipStream_t) stream);
        } else if (dev::is_tile_layout(*w)) {
            dev::launch_tile_mm_ids(*w, up, x_bf16, x_row, r->src1, r->dst, r->bounds, dst, dst_bf16 != 0, dst_col, n_experts,
                                    (int64_t) n_tok * n_used, g_cus, (hipStream_t) stream);
        } else {
            dev::launch_mm_ids(*w, up, x_bf16, x_row, r->src1, r->dst, r->bounds, dst, dst_bf16 != 0, dst_col, n_experts, n_tok, n_used,
                               g_cus, (hipStream_t) stream);
        }
        launch_check("mm_ids");
    });
}

// launch.cu:562-572
int bf16n_moe_combine(const float * ys, const void * w, int w_bf16, void * y, int y_bf16, int n_tok, int n_used, int64_t n,
                      void * stream) {
    return guarded([&] {
        ensure_init();
        if (n_tok == 0 || n == 0) {
            return;
        }
        require(n_tok <= 65535, "moe_combine: too many tokens for one launch");
        dev::launch_moe_combine(ys, w, w_bf16 != 0, y, y_bf16 != 0, n_tok, n_used, n, (hipStream_t) stream);
        launch_check("moe_combine");
    });
}

// Residual add + weighted combine + RMS norm between the products of a decode step, one launch (engine glue; no
// counterpart in the reference's core, whose engines bring their own)
int bf16n_add_rmsnorm(const uint16_t * a, const uint16_t * b, const uint16_t * c, const float * ys, const void * wts, int wts_bf16,
                      int n_used, const uint16_t * gamma, uint16_t * y_sum, uint16_t * y_norm, int n_tok, int64_t n, float eps,
                      void * stream) {
    return guarded([&] {
        ensure_init();
        require(a && y_norm && n_tok > 0 && n_tok <= 65535 && n > 0, "add_rmsnorm: null pointer or empty input");
        require(!ys || (wts && n_used > 0 && n_used < 1024), "add_rmsnorm: rows to combine need weights and a slot count below 1024");
        dev::add_norm_args p;
        p.a = a; p.b = b; p.c = c; p.ys = ys; p.wts = wts; p.wts_bf16 = wts_bf16 != 0; p.n_used = n_used;
        p.gamma = gamma; p.y_sum = y_sum; p.y_norm = y_norm; p.n = n; p.eps = eps;
        dev::launch_add_rmsnorm(p, n_tok, (hipStream_t) stream);
        launch_check("add_rmsnorm");
    });
}

// launch.cu:574-582
int bf16n_swiglu(const float * g, const float * u, float * y, int64_t n, void * stream) {
    return guarded([&] {
        ensure_init();
        if (n == 0) {
            return;
        }
        dev::launch_swiglu(g, u, y, n, g_cus, (hipStream_t) stream);
        launch_check("swiglu");
    });
}

int bf16n_router_topk_strided(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, int renorm,
                              int32_t * ids, float * weights, int64_t out_stride, void * stream) {
    return guarded([&] {
        ensure_init();
        require(n_tok > 0 && n_experts > 0 && k > 0 && k <= n_experts && k <= 64, "router_topk: need 0 < k <= min(n_experts, 64)");
        require(n_experts <= 1024, "router_topk: at most 1024 experts");
        require(out_stride >= k, "router_topk: the output row stride must be at least k");
        dev::launch_router_topk_strided(logits, logits_stride, n_tok, n_experts, k, renorm != 0, ids, weights, out_stride,
                                        (hipStream_t) stream);
        launch_check("router_topk");
    });
}

int bf16n_router_topk_route_fits(int n_tok, int n_slots, int n_listed) {
    return n_tok > 0 && n_slots > 0 && n_listed > 0 && dev::router_topk_route_fits(n_tok, n_slots, n_listed) ? 1 : 0;
}

int bf16n_router_topk_route(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, int renorm,
                            int32_t * ids, float * weights, int64_t out_stride, int n_slots, int n_listed,
                            int32_t * ids_src1, int32_t * ids_dst, int32_t * bounds, int nchannels_y, int sis1, void * stream) {
    return guarded([&] {
        ensure_init();
        require(n_tok > 0 && n_experts > 0 && k > 0 && k <= n_experts && k <= 64, "router_topk: need 0 < k <= min(n_experts, 64)");
        require(n_experts <= 1024, "router_topk: at most 1024 experts");
        require(n_slots >= k && out_stride >= n_slots, "router_topk_route: need k <= n_slots <= out_stride");
        require(n_listed >= n_experts, "router_topk_route: the lists must cover the router's experts");
        require(bf16n_router_topk_route_fits(n_tok, n_slots, n_listed) != 0,
                "router_topk_route: at most 16 tokens, 1024 (token, slot) pairs and 1024 listed experts");
        require(logits && ids && weights && ids_src1 && ids_dst && bounds, "null pointer");
        require(nchannels_y > 0, "routing sizes out of range");
        dev::launch_router_topk_route(logits, logits_stride, n_tok, n_experts, k, renorm != 0, ids, weights, out_stride, n_slots,
                                      n_listed, ids_src1, ids_dst, bounds, nchannels_y, sis1, (hipStream_t) stream);
        launch_check("router_topk_route");
    });
}

int bf16n_router_topk(const float * logits, int64_t logits_stride, int n_tok, int n_experts, int k, int renorm,
                      int32_t * ids, float * weights, void * stream) {
    return bf16n_router_topk_strided(logits, logits_stride, n_tok, n_experts, k, renorm, ids, weights, k, stream);
}

} // extern "C"
