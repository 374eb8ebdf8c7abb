// The dense path for more tokens than the decode GEMV serves: exact dequant of the matrix, in pieces, into scratch memory
// of the caller, and a stock BF16 GEMM (hipBLASLt, FP32 accumulation) on each piece.  The reference does the same above
// 8 tokens: its llama.cpp adapter with a pool allocation and cuBLAS (engines/llamacpp/patches/0002-...patch:423-437,
// the switch at :157), its torch binding with at::mm per 64 MiB piece (core/torch/torch_bindings.cpp:195-239).
// Here nothing is allocated in the call (scratch and GEMM workspace are arguments), so it can be captured into a HIP
// graph after bf16n_linear_dense_sizes() has been called once (that call creates the BLAS handle).
// hipBLASLt is opened with dlopen at first use: the library proper does not depend on it.
#include "bf16n_c.h"

#include "bf16n/format.h"

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <dlfcn.h>

#include <algorithm>
#include <functional>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>

using namespace bf16n;

namespace bf16n {
namespace impl {
int report(const std::function<void()> & f);
void check_weight(const bf16n_weight & w);
} // namespace impl
} // namespace bf16n

namespace {

constexpr uint64_t PIECE_BYTES = 64ull << 20;     // decoded BF16 per piece (torch_bindings.cpp:213)
constexpr uint64_t GEMM_WORKSPACE = 32ull << 20;  // what the GEMM heuristic may ask for

void require(bool cond, const char * msg) {
    if (!cond) {
        throw std::invalid_argument(std::string("bf16n: ") + msg);
    }
}

struct lt_api {
    decltype(&hipblasLtCreate) create;
    decltype(&hipblasLtMatmulDescCreate) desc_create;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic;
    decltype(&hipblasLtMatmul) matmul;
    hipblasLtHandle_t handle = nullptr;
};

std::mutex g_mutex;
lt_api * g_lt = nullptr;
// the GEMM plans by shape: (rows of the piece, tokens, K, ld of x, ld of y)
std::map<std::tuple<int64_t, int64_t, int64_t, int64_t, int64_t>, hipblasLtMatmulHeuristicResult_t> g_plans;

template <typename F>
void bind(void * lib, F & fn, const char * name) {
    fn = reinterpret_cast<F>(dlsym(lib, name));
    if (!fn) {
        throw std::runtime_error(std::string("bf16n: hipBLASLt lacks ") + name);
    }
}

void lt_ok(hipblasStatus_t s, const char * what) {
    if (s != HIPBLAS_STATUS_SUCCESS) {
        throw std::runtime_error(std::string("bf16n: hipBLASLt error ") + std::to_string((int) s) + " in " + what);
    }
}

lt_api & lt() { // the caller holds g_mutex
    if (!g_lt) {
        void * lib = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
        if (!lib) {
            lib = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
        }
        if (!lib) {
            throw std::runtime_error(std::string("bf16n: cannot load hipBLASLt: ") + dlerror());
        }
        auto * a = new lt_api;
        bind(lib, a->create, "hipblasLtCreate");
        bind(lib, a->desc_create, "hipblasLtMatmulDescCreate");
        bind(lib, a->desc_destroy, "hipblasLtMatmulDescDestroy");
        bind(lib, a->desc_set, "hipblasLtMatmulDescSetAttribute");
        bind(lib, a->layout_create, "hipblasLtMatrixLayoutCreate");
        bind(lib, a->layout_destroy, "hipblasLtMatrixLayoutDestroy");
        bind(lib, a->pref_create, "hipblasLtMatmulPreferenceCreate");
        bind(lib, a->pref_destroy, "hipblasLtMatmulPreferenceDestroy");
        bind(lib, a->pref_set, "hipblasLtMatmulPreferenceSetAttribute");
        bind(lib, a->heuristic, "hipblasLtMatmulAlgoGetHeuristic");
        bind(lib, a->matmul, "hipblasLtMatmul");
        lt_ok(a->create(&a->handle), "hipblasLtCreate");
        g_lt = a;
    }
    return *g_lt;
}

int64_t unit_rows(const bf16n_weight & w) { return w.format == FMT_NIBBLE ? 1 : w.R; }

// rows per piece: whole units and a multiple of 8 (every piece's slice of y then starts on a 16-byte boundary), at most
// PIECE_BYTES of BF16 and at most what the scratch holds
int64_t piece_rows(const bf16n_weight & w, uint64_t scratch_bytes) {
    const int64_t step = std::max<int64_t>(unit_rows(w), 8);
    const uint64_t budget = std::min<uint64_t>(PIECE_BYTES, scratch_bytes);
    const int64_t all = (int64_t) (budget / (uint64_t) (w.K * 2));
    return all >= w.rows ? w.rows : all / step * step;
}

// y[:, r0 : r0 + nr] = x (n_tok x K, BF16) times piece^T (piece: nr x K BF16, row-major): column-major C (nr x n_tok,
// ld y_row) = A^T B with A = the piece seen as K x nr (ld K), B = x seen as K x n_tok (ld x_row)
void gemm_piece(lt_api & L, const uint16_t * piece, int64_t nr, int64_t K, const uint16_t * x, int64_t x_row, int64_t n_tok, uint16_t * y,
                int64_t y_row, void * workspace, uint64_t workspace_bytes, hipStream_t stream) {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    lt_ok(L.desc_create(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "MatmulDescCreate");
    struct cleanup {
        lt_api & L; hipblasLtMatmulDesc_t & d; hipblasLtMatrixLayout_t & a, & b, & c;
        ~cleanup() {
            if (a) L.layout_destroy(a);
            if (b) L.layout_destroy(b);
            if (c) L.layout_destroy(c);
            if (d) L.desc_destroy(d);
        }
    } guard{L, desc, la, lb, lc};
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    lt_ok(L.desc_set(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "MatmulDescSetAttribute");
    lt_ok(L.desc_set(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "MatmulDescSetAttribute");
    lt_ok(L.layout_create(&la, HIP_R_16BF, (uint64_t) K, (uint64_t) nr, K), "MatrixLayoutCreate");
    lt_ok(L.layout_create(&lb, HIP_R_16BF, (uint64_t) K, (uint64_t) n_tok, x_row), "MatrixLayoutCreate");
    lt_ok(L.layout_create(&lc, HIP_R_16BF, (uint64_t) nr, (uint64_t) n_tok, y_row), "MatrixLayoutCreate");
    const auto key = std::make_tuple(nr, n_tok, K, x_row, y_row);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        hipblasLtMatmulPreference_t pref = nullptr;
        lt_ok(L.pref_create(&pref), "MatmulPreferenceCreate");
        hipblasLtMatmulHeuristicResult_t res = {};
        int found = 0;
        const hipblasStatus_t s1 = L.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes, sizeof(workspace_bytes));
        const hipblasStatus_t s2 = s1 == HIPBLAS_STATUS_SUCCESS ? L.heuristic(L.handle, desc, la, lb, lc, lc, pref, 1, &res, &found) : s1;
        L.pref_destroy(pref);
        lt_ok(s2, "MatmulAlgoGetHeuristic");
        if (found < 1) {
            throw std::runtime_error("bf16n: hipBLASLt has no BF16 GEMM for this shape");
        }
        it = g_plans.emplace(key, res).first;
    }
    if (it->second.workspaceSize > workspace_bytes) {
        throw std::invalid_argument("bf16n: linear_dense: the GEMM workspace is smaller than bf16n_linear_dense_sizes() asks for");
    }
    const float alpha = 1.0f, beta = 0.0f;
    lt_ok(L.matmul(L.handle, desc, &alpha, piece, la, x, lb, &beta, y, lc, y, lc, &it->second.algo, workspace, workspace_bytes, stream),
          "Matmul");
}

} // namespace

extern "C" {

int bf16n_linear_dense_sizes(const bf16n_weight * w, uint64_t * scratch_bytes, uint64_t * gemm_workspace_bytes) {
    return impl::report([&] {
        require(w && scratch_bytes && gemm_workspace_bytes, "linear_dense: null pointer");
        impl::check_weight(*w);
        require(w->rows > 0, "linear_dense: empty matrix");
        *scratch_bytes = (uint64_t) piece_rows(*w, PIECE_BYTES) * (uint64_t) w->K * 2; // never zero: 32 rows x 4096 x 2 bytes fit a piece
        *gemm_workspace_bytes = GEMM_WORKSPACE;
        std::lock_guard<std::mutex> lock(g_mutex);
        (void) lt(); // loads the BLAS and creates its handle now, outside any capture
    });
}

int bf16n_linear_dense(const bf16n_weight * w, const uint16_t * x, int64_t x_row, int n_tok, uint16_t * y, int64_t y_row,
                       void * scratch, uint64_t scratch_bytes, void * gemm_workspace, uint64_t gemm_workspace_bytes, void * stream) {
    return impl::report([&] {
        require(w && x && y && scratch, "linear_dense: null pointer");
        impl::check_weight(*w);
        require(n_tok > 0, "linear_dense: no tokens");
        require(x_row >= w->K && y_row >= w->rows, "linear_dense: row strides shorter than the rows");
        require(((uintptr_t) x & 15) == 0 && ((uintptr_t) y & 15) == 0 && ((uintptr_t) scratch & 15) == 0 && x_row % 8 == 0 && y_row % 8 == 0,
                "linear_dense: x, y and scratch must be 16-byte aligned with 16-byte row strides");
        const int64_t pr = piece_rows(*w, scratch_bytes);
        require(pr > 0, "linear_dense: the scratch buffer is too small (it must hold max(8, rows per unit) decoded rows at least)");
        std::lock_guard<std::mutex> lock(g_mutex);
        lt_api & L = lt();
        for (int64_t r0 = 0; r0 < w->rows; r0 += pr) {
            const int64_t nr = std::min(pr, w->rows - r0);
            if (bf16n_dequant(w, r0, nr, (uint16_t *) scratch, stream) != BF16N_OK) {
                throw std::invalid_argument(bf16n_last_error());
            }
            // pieces share the scratch buffer: the stream orders the decode of a piece behind the GEMM of the one before
            gemm_piece(L, (const uint16_t *) scratch, nr, w->K, x, x_row, n_tok, y + r0, y_row, gemm_workspace, gemm_workspace_bytes,
                       (hipStream_t) stream);
        }
    });
}

} // extern "C"
