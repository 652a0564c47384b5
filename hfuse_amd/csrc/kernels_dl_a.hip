// Tensor kernels, first translation unit: the six native kernels, the fused pairs whose first
// kernel is im2col or max-pool, and the two support kernels.
#include "kernels_dl_common.h"

namespace hfuse {
namespace {

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
    case K_IM2COL: return dl_native<Im2colBody>(args, hint, grid, block, lds, s);
    case K_MAXPOOL: return dl_native<MaxPoolBody>(args, hint, grid, block, lds, s);
    case K_BNSTATS: return dl_native<BnStatsBody>(args, hint, grid, block, lds, s);
    case K_UPSAMPLE_NEAREST: return dl_native<UpsampleNearestBody>(args, hint, grid, block, lds, s);
    case K_UPSAMPLE_BILINEAR: return dl_native<UpsampleBilinearBody>(args, hint, grid, block, lds, s);
    case K_HISTC: return dl_native<HistcBody>(args, hint, grid, block, lds, s);
    default: return hipErrorNotSupported;
  }
}

hipError_t launch_fused_dl_a(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                             const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s) {
  switch (k1) {
    case K_IM2COL: return dl_second<Im2colBody>(k2, mode, waves, a1, a2, g, grid, lds, s);
    case K_MAXPOOL: return dl_second<MaxPoolBody>(k2, mode, waves, a1, a2, g, grid, lds, s);
    default: return hipErrorNotSupported;
  }
}

hipError_t launch_fused_dl(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2, const FuseGeom &g,
                           unsigned grid, size_t lds, hipStream_t s) {
  switch (k1) {
    case K_IM2COL:
    case K_MAXPOOL: return launch_fused_dl_a(k1, k2, mode, waves, a1, a2, g, grid, lds, s);
    case K_BNSTATS:
    case K_UPSAMPLE_NEAREST: return launch_fused_dl_b(k1, k2, mode, waves, a1, a2, g, grid, lds, s);
    default: return launch_fused_dl_c(k1, k2, mode, waves, a1, a2, g, grid, lds, s);
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
