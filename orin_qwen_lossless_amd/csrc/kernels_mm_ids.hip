// Batched MoE prefill (grouped GEMM over the routing lists): placeholder until the MFMA kernel lands.
#include "dev_common.h"
#include "launchers.h"

#include <stdexcept>

namespace bf16n {
namespace dev {

bool mm_ids_shape_ok(const bf16n_weight &, const bf16n_weight *) { return false; }

void launch_mm_ids(const bf16n_weight &, const bf16n_weight *, const void *, int64_t, const int32_t *, const int32_t *, const int32_t *,
                   void *, bool, int64_t, int, int, int, int, hipStream_t) {
    throw std::invalid_argument("bf16n: no batched kernel for this matrix");
}

} // namespace dev
} // namespace bf16n
