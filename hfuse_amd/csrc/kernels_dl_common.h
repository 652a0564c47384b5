// Launch templates shared by the tensor-kernel translation units.  The 36 ordered pairs of
// the six tensor kernels are split over two units by their first kernel so they compile in
// parallel (both orders are built because the fused argument list follows the YAML order,
// lib/KernelFuser/KernelPrinter.cpp:107-115).
#pragma once
#include "device/dl_bodies.h"
#include "launch.h"

namespace hfuse {

constexpr int kDlBlock = 1024;  // launch bound: any split with d1 + d2 <= 1024

template <class K>
hipError_t dl_native(const void *args, unsigned hint, unsigned grid, unsigned block, size_t lds, hipStream_t s) {
  constexpr int kWaves = NativeWaves<K>::value;
  if constexpr (kWaves != 0)
    hipLaunchKernelGGL((native_kernel_capped<K, kDlBlock, kWaves>), dim3(grid), dim3(block), lds, s,
                       *static_cast<const typename K::Args *>(args), hint);
  else
    hipLaunchKernelGGL((native_kernel<K, kDlBlock>), dim3(grid), dim3(block), lds, s,
                       *static_cast<const typename K::Args *>(args), hint);
  return hipGetLastError();
}

template <class K1, class K2>
hipError_t dl_pair(FuseMode mode, int waves, const void *a1, const void *a2, const FuseGeom &g, unsigned grid, size_t lds,
                   hipStream_t s) {
  const auto &x1 = *static_cast<const typename K1::Args *>(a1);
  const auto &x2 = *static_cast<const typename K2::Args *>(a2);
  const unsigned wide = g.d1 > g.d2 ? g.d1 : g.d2;
  constexpr int kExtra = pair_extra_waves(K1::kId, K2::kId);   // a second bounded build of this pair, or 0
  const int build = built_bound_waves(K1::kId, K2::kId, waves);
  switch (mode) {
    case MODE_HFUSE:
      if constexpr (pair_has_wave_set(K1::kId, K2::kId)) {
        // one build per bound a block shape of this pair can ask for
        switch (build) {
          case 0: hipLaunchKernelGGL((fused_kernel<K1, K2, kDlBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          case 5: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, false, 5>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          case 6: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, false, 6>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          case 7: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, false, 7>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          default: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, false, 8>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
        }
        break;
      }
      if constexpr (kExtra != 0) {
        if (build == kExtra) {
          hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, false, kExtra>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
          break;
        }
      }
      if (build)
        hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      else
        hipLaunchKernelGGL((fused_kernel<K1, K2, kDlBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      break;
    case MODE_MATCHED:
      if constexpr (K1::kBarriers && K2::kBarriers) {
        if (build)
          hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kDlBlock, true>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
        else
          hipLaunchKernelGGL((fused_kernel<K1, K2, kDlBlock, true>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      } else {
        return hipErrorNotSupported;
      }
      break;
    case MODE_VERTICAL:
      if (build)   // the vertical baseline has the 8-wave bounded build only
        hipLaunchKernelGGL((vertical_kernel_lb<K1, K2, kDlBlock>), dim3(grid), dim3(wide), lds, s, x1, x2, g);
      else
        hipLaunchKernelGGL((vertical_kernel<K1, K2, kDlBlock>), dim3(grid), dim3(wide), lds, s, x1, x2, g);
      break;
    case MODE_BLOCKIDX:
      hipLaunchKernelGGL((blockidx_kernel<K1, K2, kDlBlock>), dim3(grid), dim3(wide), lds, s, x1, x2, g);
      break;
  }
  return hipGetLastError();
}

template <class K1>
hipError_t dl_second(KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2, const FuseGeom &g, unsigned grid,
                     size_t lds, hipStream_t s) {
  switch (k2) {
    case K_IM2COL: return dl_pair<K1, Im2colBody>(mode, waves, a1, a2, g, grid, lds, s);
    case K_MAXPOOL: return dl_pair<K1, MaxPoolBody>(mode, waves, a1, a2, g, grid, lds, s);
    case K_BNSTATS: return dl_pair<K1, BnStatsBody>(mode, waves, a1, a2, g, grid, lds, s);
    case K_UPSAMPLE_NEAREST: return dl_pair<K1, UpsampleNearestBody>(mode, waves, a1, a2, g, grid, lds, s);
    case K_UPSAMPLE_BILINEAR: return dl_pair<K1, UpsampleBilinearBody>(mode, waves, a1, a2, g, grid, lds, s);
    case K_HISTC: return dl_pair<K1, HistcBody>(mode, waves, a1, a2, g, grid, lds, s);
    default: return hipErrorNotSupported;
  }
}

// first kernel in {im2col, max-pool, batch-norm} / {upsample nearest, upsample bilinear, histogram}
hipError_t launch_fused_dl_a(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                             const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s);
hipError_t launch_fused_dl_b(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                             const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s);
hipError_t launch_fused_dl_c(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                             const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s);

}  // namespace hfuse
