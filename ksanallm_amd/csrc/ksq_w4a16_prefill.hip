// W4A16 prefill kernel (large M, MFMA-bound): LDS-tiled activations, weights dequantised in registers.
#include "ksq_internal.h"

namespace ksq {

bool w4a16_prefill_supported(size_t, size_t, size_t, size_t) { return false; }

int w4a16_launch_prefill(int, void*, const void*, const void*, const void*, size_t, size_t, size_t, size_t,
                         hipStream_t) {
  return fail(KSQ_ERR_UNSUPPORTED, "prefill kernel not built");
}

}  // namespace ksq
