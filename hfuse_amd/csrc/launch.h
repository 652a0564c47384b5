// Internal launch interface between the C-ABI layer and the kernel TUs.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>

#include "device/subblock.h"

namespace hfuse {

enum FuseMode { MODE_HFUSE = 0, MODE_MATCHED = 1, MODE_BLOCKIDX = 2, MODE_VERTICAL = 3 };

inline bool is_crypto(KernelId k) { return k >= K_ETHASH && k <= K_BLAKE2B; }

// `dev_args` points at the device-side argument struct of kernel `k`
// (hf_*_args for the tensor kernels, *DevArgs for the searches).
hipError_t launch_native_dl(KernelId k, const void *dev_args, unsigned hint, unsigned grid, unsigned block,
                            size_t lds, hipStream_t stream);
hipError_t launch_native_crypto(KernelId k, const void *dev_args, unsigned hint, unsigned grid, unsigned block,
                                size_t lds, hipStream_t stream);

// Returns hipErrorNotSupported when the pair is not instantiated.  `waves` selects the build of the
// fused / vertical kernel: 0 the plain one, otherwise the register-bounded build for that many
// waves per SIMD as built_bound_waves(k1, k2, waves) resolves it (the launch-bound presets).
hipError_t launch_fused_dl(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                           const FuseGeom &g, unsigned grid, size_t lds, hipStream_t stream);
hipError_t launch_fused_crypto(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                               const FuseGeom &g, unsigned grid, size_t lds, hipStream_t stream);

// Three-kernel fusions (vertical = the baseline preset).  hipErrorNotSupported when the list is not instantiated.
// `bounded`: the build compiled for 8 waves per SIMD (the launch-bound presets).
hipError_t launch_fused3_dl(const KernelId k[3], bool vertical, bool bounded, const void *const a[3], const FuseGeom3 &g,
                            unsigned grid, unsigned block, size_t lds, hipStream_t stream);
hipError_t launch_fused3_crypto(const KernelId k[3], bool vertical, bool bounded, const void *const a[3], const FuseGeom3 &g,
                                unsigned grid, unsigned block, size_t lds, hipStream_t stream);

hipError_t launch_fill_splitmix64(unsigned long long *dst, unsigned long long nwords, unsigned long long seed,
                                  hipStream_t stream);
hipError_t launch_copy_f32(const float *src, float *dst, unsigned long long n, hipStream_t stream);
// The bare stream kernels (HF_STREAM_* patterns) over n4 16-byte vectors.
hipError_t launch_stream_probe(int pattern, const void *src, void *dst, unsigned long long n4, unsigned grid, unsigned block,
                               hipStream_t stream);

}  // namespace hfuse
