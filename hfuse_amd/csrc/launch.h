// Internal launch interface between the C-ABI layer and the kernel TUs.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>

#include "device/subblock.h"

namespace hfuse {

enum KernelId {
  K_IM2COL = 0,
  K_MAXPOOL,
  K_BNSTATS,
  K_UPSAMPLE_NEAREST,
  K_HISTC,
  K_ETHASH,
  K_SHA256D,
  K_SIA_BLAKE2B,
  K_BLAKE2B,
  K_UPSAMPLE_BILINEAR,
  K_COUNT
};

enum FuseMode { MODE_HFUSE = 0, MODE_MATCHED = 1, MODE_BLOCKIDX = 2, MODE_VERTICAL = 3 };

inline bool is_crypto(KernelId k) { return k >= K_ETHASH && k <= K_BLAKE2B; }

// `dev_args` points at the device-side argument struct of kernel `k`
// (hf_*_args for the tensor kernels, *DevArgs for the searches).
hipError_t launch_native_dl(KernelId k, const void *dev_args, unsigned hint, unsigned grid, unsigned block,
                            size_t lds, hipStream_t stream);
hipError_t launch_native_crypto(KernelId k, const void *dev_args, unsigned hint, unsigned grid, unsigned block,
                                size_t lds, hipStream_t stream);

// Returns hipErrorNotSupported when the pair is not instantiated.  `bounded` selects the
// register-bounded build of the fused / vertical kernel (the launch-bound presets).
hipError_t launch_fused_dl(KernelId k1, KernelId k2, FuseMode mode, bool bounded, const void *a1, const void *a2,
                           const FuseGeom &g, unsigned grid, size_t lds, hipStream_t stream);
hipError_t launch_fused_crypto(KernelId k1, KernelId k2, FuseMode mode, bool bounded, const void *a1, const void *a2,
                               const FuseGeom &g, unsigned grid, size_t lds, hipStream_t stream);

hipError_t launch_fill_splitmix64(unsigned long long *dst, unsigned long long nwords, unsigned long long seed,
                                  hipStream_t stream);
hipError_t launch_copy_f32(const float *src, float *dst, unsigned long long n, hipStream_t stream);

}  // namespace hfuse
