// Instantiations of the tensor kernels: five native kernels and every ordered
// pair of them as a horizontally fused kernel (the reference's ml_fusion.yaml
// lists ten of these pairs; both orders are built because the fused argument
// list follows the YAML order, lib/KernelFuser/KernelPrinter.cpp:107-115).
#include "device/dl_bodies.h"
#include "launch.h"

namespace hfuse {
namespace {

constexpr int kDlBlock = 1024;  // launch bound: any split with d1 + d2 <= 1024

template <class K>
hipError_t native(const void *args, unsigned hint, unsigned grid, unsigned block, size_t lds, hipStream_t s) {
  hipLaunchKernelGGL((native_kernel<K, kDlBlock>), dim3(grid), dim3(block), lds, s,
                     *static_cast<const typename K::Args *>(args), hint);
  return hipGetLastError();
}

template <class K1, class K2>
hipError_t pair(FuseMode mode, const void *a1, const void *a2, const FuseGeom &g, unsigned grid, size_t lds,
                hipStream_t s) {
  const auto &x1 = *static_cast<const typename K1::Args *>(a1);
  const auto &x2 = *static_cast<const typename K2::Args *>(a2);
  switch (mode) {
    case MODE_HFUSE:
      hipLaunchKernelGGL((fused_kernel<K1, K2, kDlBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      break;
    case MODE_MATCHED:
      if constexpr (K1::kBarriers && K2::kBarriers) {
        hipLaunchKernelGGL((fused_kernel<K1, K2, kDlBlock, true>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      } else {
        return hipErrorNotSupported;
      }
      break;
    case MODE_VERTICAL:
      hipLaunchKernelGGL((vertical_kernel<K1, K2, kDlBlock>), dim3(grid), dim3(g.d1 > g.d2 ? g.d1 : g.d2), lds, s, x1, x2, g);
      break;
    case MODE_BLOCKIDX:
      hipLaunchKernelGGL((blockidx_kernel<K1, K2, kDlBlock>), dim3(grid), dim3(g.d1 > g.d2 ? g.d1 : g.d2), lds, s, x1,
                         x2, g);
      break;
  }
  return hipGetLastError();
}

template <class K1>
hipError_t second(KernelId k2, FuseMode mode, const void *a1, const void *a2, const FuseGeom &g, unsigned grid,
                  size_t lds, hipStream_t s) {
  switch (k2) {
    case K_IM2COL: return pair<K1, Im2colBody>(mode, a1, a2, g, grid, lds, s);
    case K_MAXPOOL: return pair<K1, MaxPoolBody>(mode, a1, a2, g, grid, lds, s);
    case K_BNSTATS: return pair<K1, BnStatsBody>(mode, a1, a2, g, grid, lds, s);
    case K_UPSAMPLE_NEAREST: return pair<K1, UpsampleNearestBody>(mode, a1, a2, g, grid, lds, s);
    case K_HISTC: return pair<K1, HistcBody>(mode, a1, a2, g, grid, lds, s);
    default: return hipErrorNotSupported;
  }
}

__global__ __launch_bounds__(256) void fill_splitmix64_kernel(unsigned long long *dst, unsigned long long n,
                                                              unsigned long long seed) {
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    unsigned long long z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    dst[i] = z ^ (z >> 31);
  }
}

__global__ __launch_bounds__(256) void copy_f32_kernel(const float *src, float *dst, unsigned long long n) {
  const unsigned long long n4 = n >> 2;
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
    reinterpret_cast<f32x4 *>(dst)[i] = reinterpret_cast<const f32x4 *>(src)[i];
  if (blockIdx.x == 0)
    for (unsigned long long i = (n4 << 2) + threadIdx.x; i < n; i += blockDim.x) dst[i] = src[i];
}

}  // namespace

hipError_t launch_native_dl(KernelId k, const void *args, unsigned hint, unsigned grid, unsigned block, size_t lds,
                            hipStream_t s) {
  switch (k) {
    case K_IM2COL: return native<Im2colBody>(args, hint, grid, block, lds, s);
    case K_MAXPOOL: return native<MaxPoolBody>(args, hint, grid, block, lds, s);
    case K_BNSTATS: return native<BnStatsBody>(args, hint, grid, block, lds, s);
    case K_UPSAMPLE_NEAREST: return native<UpsampleNearestBody>(args, hint, grid, block, lds, s);
    case K_HISTC: return native<HistcBody>(args, hint, grid, block, lds, s);
    default: return hipErrorNotSupported;
  }
}

hipError_t launch_fused_dl(KernelId k1, KernelId k2, FuseMode mode, const void *a1, const void *a2, const FuseGeom &g,
                           unsigned grid, size_t lds, hipStream_t s) {
  switch (k1) {
    case K_IM2COL: return second<Im2colBody>(k2, mode, a1, a2, g, grid, lds, s);
    case K_MAXPOOL: return second<MaxPoolBody>(k2, mode, a1, a2, g, grid, lds, s);
    case K_BNSTATS: return second<BnStatsBody>(k2, mode, a1, a2, g, grid, lds, s);
    case K_UPSAMPLE_NEAREST: return second<UpsampleNearestBody>(k2, mode, a1, a2, g, grid, lds, s);
    case K_HISTC: return second<HistcBody>(k2, mode, a1, a2, g, grid, lds, s);
    default: return hipErrorNotSupported;
  }
}

hipError_t launch_fill_splitmix64(unsigned long long *dst, unsigned long long n, unsigned long long seed,
                                  hipStream_t s) {
  if (n == 0) return hipSuccess;
  unsigned long long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_splitmix64_kernel, dim3((unsigned)blocks), dim3(256), 0, s, dst, n, seed);
  return hipGetLastError();
}

hipError_t launch_copy_f32(const float *src, float *dst, unsigned long long n, hipStream_t s) {
  if (n == 0) return hipSuccess;
  unsigned long long blocks = (n / 4 + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(copy_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, s, src, dst, n);
  return hipGetLastError();
}

}  // namespace hfuse
