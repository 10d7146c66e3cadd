// The LDS-tiled MFMA prefill kernel for head dimensions 32, 48, 80, 96 and 112 (the same kernel as for 64 and 128, in
// the tile layout of the next of those two) and 256 (a layout of its own); 40, 56, 72, 88, 104 and 120, whose last
// 16-dim step is half empty, are instantiated in prefill_half_step_dims.hip.  The reference picks its tile sizes by
// head_dim and covers every size (src/myvllm/layers/attention.py:249-257).  A translation unit of its own so that
// its instances compile next to the others.
#include "prefill_mfma.h"

namespace mvllm {

bool prefill_mfma_other_dim(int head_dim) {
  return (head_dim >= 32 && head_dim < 128 && head_dim % 8 == 0 && head_dim != 64) || head_dim == 256;
}

template <typename T, bool PAGED>
static int launch_other(const PrefillArgs& a, hipStream_t stream) {
  switch (a.head_dim) {
    case 32: return launch_prefill_mfma_as<T, PAGED, false, 64, 32>(a, stream);
    case 48: return launch_prefill_mfma_as<T, PAGED, false, 64, 48>(a, stream);
    case 80: return launch_prefill_mfma_as<T, PAGED, false, 128, 80>(a, stream);
    case 96: return launch_prefill_mfma_as<T, PAGED, false, 128, 96>(a, stream);
    case 112: return launch_prefill_mfma_as<T, PAGED, false, 128, 112>(a, stream);
    case 256: return launch_prefill_mfma_as<T, PAGED, false, 256, 256>(a, stream);
    default: return MVLLM_ERR_UNSUPPORTED;
  }
}

int launch_prefill_mfma_half_step(const PrefillArgs& a, int dtype, bool paged, hipStream_t stream);   // prefill_half_step_dims.hip

int launch_prefill_mfma_other(const PrefillArgs& a, int dtype, bool paged, hipStream_t stream) {
  if (a.head_dim % 16 == 8) return launch_prefill_mfma_half_step(a, dtype, paged, stream);
  if (dtype == MVLLM_BF16) return paged ? launch_other<bf16_t, true>(a, stream) : launch_other<bf16_t, false>(a, stream);
  if (dtype == MVLLM_F16) return paged ? launch_other<f16_t, true>(a, stream) : launch_other<f16_t, false>(a, stream);
  return MVLLM_ERR_UNSUPPORTED;
}

}  // namespace mvllm
