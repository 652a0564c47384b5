// Tensor kernels, third translation unit: the fused pairs whose first kernel is the
// bilinear upsampling or the histogram.
#include "kernels_dl_common.h"

namespace hfuse {

hipError_t launch_fused_dl_c(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                             const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s) {
  switch (k1) {
    case K_UPSAMPLE_BILINEAR: return dl_second<UpsampleBilinearBody>(k2, mode, waves, a1, a2, g, grid, lds, s);
    case K_HISTC: return dl_second<HistcBody>(k2, mode, waves, a1, a2, g, grid, lds, s);
    default: return hipErrorNotSupported;
  }
}

}  // namespace hfuse
