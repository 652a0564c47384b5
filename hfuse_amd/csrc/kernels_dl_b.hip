// Tensor kernels, second translation unit: the fused pairs whose first kernel is the
// batch-norm statistics or the nearest-neighbour upsampling.
#include "kernels_dl_common.h"

namespace hfuse {

hipError_t launch_fused_dl_b(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                             const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s) {
  switch (k1) {
    case K_BNSTATS: return dl_second<BnStatsBody>(k2, mode, waves, a1, a2, g, grid, lds, s);
    case K_UPSAMPLE_NEAREST: return dl_second<UpsampleNearestBody>(k2, mode, waves, a1, a2, g, grid, lds, s);
    default: return hipErrorNotSupported;
  }
}

}  // namespace hfuse
