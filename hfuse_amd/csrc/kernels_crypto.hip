// Instantiations of the nonce-search kernels: four native kernels and the
// ordered pairs of the reference's crypto_fusion.yaml (both orders).
#include "device/crypto_bodies.h"
#include "launch.h"

namespace hfuse {
namespace {

// The searches run 128+128 threads in the reference's YAML; 512 leaves room for
// every 64-lane re-split of up to 512 threads.  Four waves per SIMD keeps each
// wave under 128 VGPRs so a memory-bound half still has waves to hide latency.
constexpr int kCryptoBlock = 512;

template <class K>
hipError_t native(const void *args, unsigned hint, unsigned grid, unsigned block, size_t lds, hipStream_t s) {
  hipLaunchKernelGGL((native_kernel<K, kCryptoBlock>), dim3(grid), dim3(block), lds, s,
                     *static_cast<const typename K::Args *>(args), hint);
  return hipGetLastError();
}

template <class K1, class K2>
hipError_t pair(FuseMode mode, int waves, const void *a1, const void *a2, const FuseGeom &g, unsigned grid, size_t lds,
                hipStream_t s) {
  const auto &x1 = *static_cast<const typename K1::Args *>(a1);
  const auto &x2 = *static_cast<const typename K2::Args *>(a2);
  if (g.d1 + g.d2 > (unsigned)kCryptoBlock) return hipErrorNotSupported;
  constexpr int kExtra = pair_extra_waves(K1::kId, K2::kId);   // a second bounded build of this pair, or 0
  const int build = built_bound_waves(K1::kId, K2::kId, waves);
  const bool bounded = build != 0;
  switch (mode) {
    case MODE_HFUSE:
      if constexpr (pair_has_wave_set(K1::kId, K2::kId)) {
        // one build per bound a block shape of this pair can ask for
        switch (build) {
          case 0: hipLaunchKernelGGL((fused_kernel<K1, K2, kCryptoBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          case 5: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kCryptoBlock, false, 5>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          case 6: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kCryptoBlock, false, 6>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          case 7: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kCryptoBlock, false, 7>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
          default: hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kCryptoBlock, false, 8>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g); break;
        }
        break;
      }
      if constexpr (kExtra != 0) {
        if (build == kExtra) {
          hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kCryptoBlock, false, kExtra>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
          break;
        }
      }
      if (build)
        hipLaunchKernelGGL((fused_kernel_lb<K1, K2, kCryptoBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      else
        hipLaunchKernelGGL((fused_kernel<K1, K2, kCryptoBlock, false>), dim3(grid), dim3(g.d1 + g.d2), lds, s, x1, x2, g);
      break;
    case MODE_MATCHED:
      return hipErrorNotSupported;  // none of the searches has a barrier
    case MODE_VERTICAL:
      if (bounded)
        hipLaunchKernelGGL((vertical_kernel_lb<K1, K2, kCryptoBlock>), dim3(grid), dim3(g.d1 > g.d2 ? g.d1 : g.d2), lds,
                           s, x1, x2, g);
      else
        hipLaunchKernelGGL((vertical_kernel<K1, K2, kCryptoBlock>), dim3(grid), dim3(g.d1 > g.d2 ? g.d1 : g.d2), lds, s,
                           x1, x2, g);
      break;
    case MODE_BLOCKIDX:
      hipLaunchKernelGGL((blockidx_kernel<K1, K2, kCryptoBlock>), dim3(grid), dim3(g.d1 > g.d2 ? g.d1 : g.d2), lds,
                         s, x1, x2, g);
      break;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_native_crypto(KernelId k, const void *args, unsigned hint, unsigned grid, unsigned block, size_t lds,
                                hipStream_t s) {
  switch (k) {
    case K_ETHASH: return native<EthashBody>(args, hint, grid, block, lds, s);
    case K_SHA256D: return native<Sha256dBody>(args, hint, grid, block, lds, s);
    case K_SIA_BLAKE2B: return native<SiaBlake2bBody>(args, hint, grid, block, lds, s);
    case K_BLAKE2B: return native<CcminerBlake2bBody>(args, hint, grid, block, lds, s);
    default: return hipErrorNotSupported;
  }
}

// The three-kernel list of configs/crypt_four.yaml, in its listed order.
hipError_t launch_fused3_crypto(const KernelId k[3], bool vertical, bool bounded, const void *const a[3], const FuseGeom3 &g,
                                unsigned grid, unsigned block, size_t lds, hipStream_t s) {
  if (!(k[0] == K_BLAKE2B && k[1] == K_SHA256D && k[2] == K_ETHASH)) return hipErrorNotSupported;
  if (block > (unsigned)kCryptoBlock) return hipErrorNotSupported;
  const auto &x0 = *static_cast<const Blake2bDevArgs *>(a[0]);
  const auto &x1 = *static_cast<const Sha256dDevArgs *>(a[1]);
  const auto &x2 = *static_cast<const EthashDevArgs *>(a[2]);
  if (vertical && bounded)
    hipLaunchKernelGGL((vertical_kernel3_lb<CcminerBlake2bBody, Sha256dBody, EthashBody, kCryptoBlock>), dim3(grid), dim3(block),
                       lds, s, x0, x1, x2, g);
  else if (vertical)
    hipLaunchKernelGGL((vertical_kernel3<CcminerBlake2bBody, Sha256dBody, EthashBody, kCryptoBlock>), dim3(grid), dim3(block),
                       lds, s, x0, x1, x2, g);
  else if (bounded)
    hipLaunchKernelGGL((fused_kernel3_lb<CcminerBlake2bBody, Sha256dBody, EthashBody, kCryptoBlock>), dim3(grid), dim3(block), lds,
                       s, x0, x1, x2, g);
  else
    hipLaunchKernelGGL((fused_kernel3<CcminerBlake2bBody, Sha256dBody, EthashBody, kCryptoBlock>), dim3(grid), dim3(block), lds,
                       s, x0, x1, x2, g);
  return hipGetLastError();
}

#define HF_PAIR(A, KA, B, KB)                                                     \
  if (k1 == A && k2 == B) return pair<KA, KB>(mode, waves, a1, a2, g, grid, lds, s);     \
  if (k1 == B && k2 == A) return pair<KB, KA>(mode, waves, a1, a2, g, grid, lds, s);

hipError_t launch_fused_crypto(KernelId k1, KernelId k2, FuseMode mode, int waves, const void *a1, const void *a2,
                               const FuseGeom &g, unsigned grid, size_t lds, hipStream_t s) {
  HF_PAIR(K_ETHASH, EthashBody, K_BLAKE2B, CcminerBlake2bBody)
  HF_PAIR(K_SHA256D, Sha256dBody, K_ETHASH, EthashBody)
  HF_PAIR(K_SIA_BLAKE2B, SiaBlake2bBody, K_ETHASH, EthashBody)
  HF_PAIR(K_BLAKE2B, CcminerBlake2bBody, K_SHA256D, Sha256dBody)
  HF_PAIR(K_BLAKE2B, CcminerBlake2bBody, K_SIA_BLAKE2B, SiaBlake2bBody)
  HF_PAIR(K_SHA256D, Sha256dBody, K_SIA_BLAKE2B, SiaBlake2bBody)
  return hipErrorNotSupported;
}

}  // namespace hfuse
