// MFMA GEMM for M >= 16 (prefill chunks, batched decode).  Placeholder until the tiled kernel lands:
// reports every shape as unsupported so callers stream the weights through the GEMV kernel instead.
#include "ops.h"

namespace rwkv {

bool linear_mfma_supported(int, int, int, int) { return false; }

int linear_mfma(hipStream_t, int, int, int, int, const half_t*, const void*, const half_t*, const uint8_t*, int, int,
                void*) {
  set_error("linear_mfma: not available");
  return RWKV_E_INVALID;
}

}  // namespace rwkv
