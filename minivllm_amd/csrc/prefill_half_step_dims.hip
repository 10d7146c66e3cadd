// The LDS-tiled MFMA prefill kernel for head dimensions 40, 56 (in the tile layout of 64), 72, 88, 104 and 120 (in that
// of 128): multiples of 8 whose last 16-dim step of the first product holds 8 dims (prefill_mfma.h: kHalfStep).  The
// reference's kernel takes any head_dim by tile table (src/myvllm/layers/attention.py:249-257).  A translation unit of
// its own so that its instances compile next to the others.
#include "prefill_mfma.h"

namespace mvllm {

template <typename T, bool PAGED>
static int launch_half_step(const PrefillArgs& a, hipStream_t stream) {
  switch (a.head_dim) {
    case 40: return launch_prefill_mfma_as<T, PAGED, false, 64, 40>(a, stream);
    case 56: return launch_prefill_mfma_as<T, PAGED, false, 64, 56>(a, stream);
    case 72: return launch_prefill_mfma_as<T, PAGED, false, 128, 72>(a, stream);
    case 88: return launch_prefill_mfma_as<T, PAGED, false, 128, 88>(a, stream);
    case 104: return launch_prefill_mfma_as<T, PAGED, false, 128, 104>(a, stream);
    case 120: return launch_prefill_mfma_as<T, PAGED, false, 128, 120>(a, stream);
    default: return MVLLM_ERR_UNSUPPORTED;
  }
}

int launch_prefill_mfma_half_step(const PrefillArgs& a, int dtype, bool paged, hipStream_t stream) {
  if (dtype == MVLLM_BF16) return paged ? launch_half_step<bf16_t, true>(a, stream) : launch_half_step<bf16_t, false>(a, stream);
  if (dtype == MVLLM_F16) return paged ? launch_half_step<f16_t, true>(a, stream) : launch_half_step<f16_t, false>(a, stream);
  return MVLLM_ERR_UNSUPPORTED;
}

}  // namespace mvllm
