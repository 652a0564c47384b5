// Tensor kernels, fourth translation unit: the three-kernel fusions of the reference's lists
// (configs/im2col_maxpool_norm.yaml, configs/maxpool_summary_norm.yaml), built in their listed order; the host
// maps a list that names the same kernels in another order onto the same instantiation.
#include "kernels_dl_common.h"

namespace hfuse {
namespace {

template <class K0, class K1, class K2>
hipError_t triple(bool vertical, bool bounded, const void *const a[3], const FuseGeom3 &g, unsigned grid, unsigned block,
                  size_t lds, hipStream_t s) {
  const auto &x0 = *static_cast<const typename K0::Args *>(a[0]);
  const auto &x1 = *static_cast<const typename K1::Args *>(a[1]);
  const auto &x2 = *static_cast<const typename K2::Args *>(a[2]);
  if (vertical && bounded)
    hipLaunchKernelGGL((vertical_kernel3_lb<K0, K1, K2, kDlBlock>), dim3(grid), dim3(block), lds, s, x0, x1, x2, g);
  else if (vertical)
    hipLaunchKernelGGL((vertical_kernel3<K0, K1, K2, kDlBlock>), dim3(grid), dim3(block), lds, s, x0, x1, x2, g);
  else if (bounded)
    hipLaunchKernelGGL((fused_kernel3_lb<K0, K1, K2, kDlBlock>), dim3(grid), dim3(block), lds, s, x0, x1, x2, g);
  else
    hipLaunchKernelGGL((fused_kernel3<K0, K1, K2, kDlBlock>), dim3(grid), dim3(block), lds, s, x0, x1, x2, g);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_fused3_dl(const KernelId k[3], bool vertical, bool bounded, const void *const a[3], const FuseGeom3 &g,
                            unsigned grid, unsigned block, size_t lds, hipStream_t s) {
  if (k[0] == K_IM2COL && k[1] == K_MAXPOOL && k[2] == K_BNSTATS)
    return triple<Im2colBody, MaxPoolBody, BnStatsBody>(vertical, bounded, a, g, grid, block, lds, s);
  if (k[0] == K_MAXPOOL && k[1] == K_HISTC && k[2] == K_BNSTATS)
    return triple<MaxPoolBody, HistcBody, BnStatsBody>(vertical, bounded, a, g, grid, block, lds, s);
  return hipErrorNotSupported;
}

}  // namespace hfuse
