// The view a kernel body has of "its" threads, whether it owns the whole
// workgroup (native launch) or a wavefront-aligned slice of it (fused launch).
//
// The reference rewrites threadIdx/blockDim of each original kernel into
// per-kernel locals computed from (flat tid - lower bound)
// (lib/KernelFuser/ThreadInfoRewriter.cpp:38-58) and leaves blockIdx/gridDim
// alone (include/ThreadInfoRewriter.h:29-31).  A body here is written once
// against SubBlock and never touches threadIdx/blockDim itself.
//
// Barriers.  The reference turns __syncthreads() into the PTX named barrier
// `bar.sync id,count` (lib/KernelFuser/BarrierRewriter.cpp:12-16) so a half
// only waits for itself.  gfx950 has one barrier per workgroup (s_barrier
// waits for every wave that has not ended), so a half that synchronises next to
// a half that streams uses an LDS arrival counter instead: lane 0 of each wave
// of the half adds 1 and spins (s_sleep) until the counter reaches
// phase * waves_in_half.  The counter only grows, so no reset race exists; the
// fused kernel zeroes it before one workgroup-wide s_barrier that every wave of
// both halves executes exactly once on entry.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

namespace hfuse {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef long long i64x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

enum { BAR_WORKGROUP = 0, BAR_SUBSET = 1 };

#ifndef HF_SYNC_BACKOFF
#define HF_SYNC_BACKOFF 1  // 0: a parked wave polls its arrival counter every 64 cycles (experiment switch)
#endif

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

// Register-bounded builds.  The reference prints `__launch_bounds__(T, B)` with B = min over the kernels of
// regfile / Reg / threads, capped by the resident threads (lib/KernelFuser/KernelPrinter.cpp:44-66): B blocks of T
// threads are to fit a multiprocessor.  With this part's 128 K registers and 2048 threads per CU that is a bound of
// ceil(B * T / 64 / 4) waves per SIMD.  Every pair has a build for kBoundedWaves waves per SIMD.  The five benchmarked
// pairs have one for each of 5, 6, 7 and 8, so that whatever block shape a plan of theirs is given, the build a
// launch-bound preset runs is bounded at exactly the formula's value (up to four waves per SIMD the plain build's
// launch bound already holds); three more pairs of the shipped list have a second build at the value of their
// shipped shape.
constexpr int kBoundedWaves = 8;
constexpr int kMinSetWaves = 5;
constexpr bool pair_has_wave_set(KernelId k1, KernelId k2) {
  return (k1 == K_IM2COL && k2 == K_MAXPOOL) || (k1 == K_BNSTATS && k2 == K_UPSAMPLE_NEAREST) ||
         (k1 == K_HISTC && k2 == K_MAXPOOL) || (k1 == K_SHA256D && k2 == K_SIA_BLAKE2B) ||
         (k1 == K_ETHASH && k2 == K_SIA_BLAKE2B);
}
constexpr int pair_extra_waves(KernelId k1, KernelId k2) {
  return (k1 == K_IM2COL && k2 == K_HISTC) ? 7                  // 2 blocks of 640 + 256 threads
         : (k1 == K_IM2COL && k2 == K_UPSAMPLE_NEAREST) ? 6     // 2 blocks of 256 + 512
         : (k1 == K_IM2COL && k2 == K_UPSAMPLE_BILINEAR) ? 6    // 2 blocks of 256 + 512
                                                         : 0;
}
// The bound of the build that runs when `waves` waves per SIMD are asked for (0: the plain build): the smallest
// built bound that is not below the request.
constexpr int built_bound_waves(KernelId k1, KernelId k2, int waves) {
  return waves <= 0 ? 0
         : pair_has_wave_set(k1, k2) ? (waves < kMinSetWaves ? kMinSetWaves : waves > kBoundedWaves ? kBoundedWaves : waves)
         : (pair_extra_waves(k1, k2) != 0 && waves <= pair_extra_waves(k1, k2)) ? pair_extra_waves(k1, k2)
                                                                                : kBoundedWaves;
}


template <int BAR>
struct SubBlock {
  unsigned tid;       // thread index inside this half
  unsigned nthreads;  // threads of this half (a multiple of 64)
  unsigned bid;       // block index the body strides from
  unsigned nblocks;   // grid size the body strides by
  unsigned *bar;      // LDS arrival counter of this half (BAR_SUBSET only)
  unsigned phase;     // barriers this thread has passed
  unsigned gbase;     // index of this half's thread 0 among all threads that run this kernel
  unsigned gthreads;  // number of threads that run this kernel in the whole launch
  bool whole = false; // BAR_SUBSET only: this body runs on every wave of the workgroup, so the hardware barrier serves it

  // Flat work-item index and stride of a body that walks a 1-D range.  Equal to
  // bid * nthreads + tid and nblocks * nthreads except where a block lends the idle
  // half's waves to the partner (see fused_kernel), which makes blocks unequal in size.
  __device__ __forceinline__ unsigned gtid() const { return gbase + tid; }
  __device__ __forceinline__ unsigned gstride() const { return gthreads; }

  __device__ __forceinline__ unsigned lane() const { return tid & 63u; }
  __device__ __forceinline__ unsigned wave() const { return tid >> 6; }
  __device__ __forceinline__ unsigned nwaves() const { return nthreads >> 6; }

  __device__ __forceinline__ void sync() {
    if constexpr (BAR == BAR_WORKGROUP) {
      __syncthreads();
    } else {
      if (whole) {  // wave-uniform: every wave of the workgroup runs this body and reaches this barrier
        __syncthreads();
        return;
      }
      phase++;
      // Release this wave's LDS/global writes to the workgroup, arrive, wait, acquire.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane() == 0) {
        __hip_atomic_fetch_add(bar, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        const unsigned target = phase * nwaves();
        // A parked wave polls the LDS its working siblings add into: the naps grow (64, 128, 256, then 512
        // cycles) so that a long wait costs a handful of LDS reads instead of one every 64 cycles.
        unsigned polls = 0;
        while (__hip_atomic_load(bar, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
          if (!HF_SYNC_BACKOFF || polls < 2) __builtin_amdgcn_s_sleep(1);
          else if (polls < 4) __builtin_amdgcn_s_sleep(2);
          else if (polls < 8) __builtin_amdgcn_s_sleep(4);
          else __builtin_amdgcn_s_sleep(8);
          polls++;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
  }
};

// Launch geometry the host passes next to the two argument lists.
struct FuseGeom {
  unsigned d1, d2;          // threads of each half
  unsigned lds1, lds2;      // LDS bytes of each half
  unsigned hint1, hint2;    // fast-path selector the host derived from each argument list
  unsigned grid1, grid2;    // workgroups each kernel strides over: in the fused kernel half k works in
                            // blocks [0, grid_k) only; in blockIdx mode kernel 2 starts at block grid1
  unsigned lend;            // 1: in a block beyond its own grid a half's waves run the partner's body
};

constexpr unsigned kBarrierWords = 4;  // 16 bytes reserved at the base of LDS for arrival counters

// Native launch: the body owns the whole workgroup.
template <class K, int T>
__global__ __launch_bounds__(T) void native_kernel(typename K::Args a, unsigned hint) {
  extern __shared__ __align__(16) unsigned char smem[];
  const unsigned bid = blockIdx.x;
  SubBlock<BAR_WORKGROUP> sb{threadIdx.x, blockDim.x, bid, gridDim.x, nullptr, 0,
                             bid * blockDim.x, gridDim.x * blockDim.x};
  K::run(a, sb, smem, hint);
}

// The same with residency capped at W waves per SIMD (the register allocation is padded so that no
// more fit).  A body asks for it with `kNativeWaves`: a kernel that writes many separate streams per
// work item runs faster when fewer of its waves write at once.
template <class K, int T, int W>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(W, W))) void native_kernel_capped(typename K::Args a,
                                                                                                   unsigned hint) {
  extern __shared__ __align__(16) unsigned char smem[];
  const unsigned bid = blockIdx.x;
  SubBlock<BAR_WORKGROUP> sb{threadIdx.x, blockDim.x, bid, gridDim.x, nullptr, 0,
                             bid * blockDim.x, gridDim.x * blockDim.x};
  K::run(a, sb, smem, hint);
}

template <class K, class = void>
struct NativeWaves {
  static constexpr int value = 0;  // no cap
};
template <class K>
struct NativeWaves<K, std::void_t<decltype(K::kNativeWaves)>> {
  static constexpr int value = K::kNativeWaves;
};

// Horizontal fusion: waves [0, d1/64) run kernel 1, the rest run kernel 2.  The
// selector is a scalar (readfirstlane) so each wave takes one side without
// divergence.  MATCHED: both bodies execute the same number of barriers, so
// they may share the hardware barrier; otherwise a body that synchronises
// uses its own LDS counter.
template <class K1, class K2, bool MATCHED>
__device__ __forceinline__ void fused_block(const typename K1::Args &a1, const typename K2::Args &a2,
                                            const FuseGeom &g) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned *bars = reinterpret_cast<unsigned *>(smem);
  const unsigned tid = threadIdx.x;
  constexpr bool kSubset = !MATCHED && (K1::kBarriers || K2::kBarriers);
  if constexpr (kSubset) {
    if (tid < kBarrierWords) bars[tid] = 0;
    __syncthreads();
  }
  const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int B1 = (kSubset && K1::kBarriers) ? BAR_SUBSET : BAR_WORKGROUP;
  constexpr int B2 = (kSubset && K2::kBarriers) ? BAR_SUBSET : BAR_WORKGROUP;
  // Both halves see the launch's blockIdx (the reference leaves blockIdx/gridDim alone,
  // include/ThreadInfoRewriter.h:29-31).  A half whose kernel wants fewer workgroups than the
  // launch has would idle in the surplus blocks; there its waves either end at once (freeing
  // their slots) or, when the partner walks a flat 1-D range (K::kFlat) and lending is on,
  // run the partner's body, so a surplus block is one whole block of the partner.  The
  // partner's flat index then counts d_partner threads in shared blocks and d1+d2 in lent ones.
  const unsigned bid = blockIdx.x, dd = g.d1 + g.d2;
  const bool in1 = bid < g.grid1, in2 = bid < g.grid2;
  const bool lend1 = K1::kFlat && g.lend && g.grid1 > g.grid2;  // kernel 1 borrows kernel 2's waves
  const bool lend2 = K2::kFlat && g.lend && g.grid2 > g.grid1;  // kernel 2 borrows kernel 1's waves
  const unsigned total1 = lend1 ? g.grid2 * g.d1 + (g.grid1 - g.grid2) * dd : g.grid1 * g.d1;
  const unsigned total2 = lend2 ? g.grid1 * g.d2 + (g.grid2 - g.grid1) * dd : g.grid2 * g.d2;
  unsigned char *lds1 = smem + 4 * kBarrierWords, *lds2 = lds1 + g.lds1;
  if (in1 && in2) {  // a shared block
    if (wave < (g.d1 >> 6)) {
      SubBlock<B1> sb{tid, g.d1, bid, g.grid1, bars + 0, 0, bid * g.d1, total1};
      K1::run(a1, sb, lds1, g.hint1);
    } else {
      SubBlock<B2> sb{tid - g.d1, g.d2, bid, g.grid2, bars + 1, 0, bid * g.d2, total2};
      K2::run(a2, sb, lds2, g.hint2);
    }
  } else if (in1) {  // kernel 2 has no work here
    if (lend1) {
      SubBlock<BAR_WORKGROUP> sb{tid, dd, bid, g.grid1, nullptr, 0, g.grid2 * g.d1 + (bid - g.grid2) * dd, total1};
      K1::run(a1, sb, lds1, g.hint1);
    } else if (wave < (g.d1 >> 6)) {
      SubBlock<B1> sb{tid, g.d1, bid, g.grid1, bars + 0, 0, bid * g.d1, total1};
      K1::run(a1, sb, lds1, g.hint1);
    }
  } else if (in2) {  // kernel 1 has no work here
    if (lend2) {
      SubBlock<BAR_WORKGROUP> sb{tid, dd, bid, g.grid2, nullptr, 0, g.grid1 * g.d2 + (bid - g.grid1) * dd, total2};
      K2::run(a2, sb, lds2, g.hint2);
    } else if (wave >= (g.d1 >> 6)) {
      SubBlock<B2> sb{tid - g.d1, g.d2, bid, g.grid2, bars + 1, 0, bid * g.d2, total2};
      K2::run(a2, sb, lds2, g.hint2);
    }
  }
}

template <class K1, class K2, int T, bool MATCHED>
__global__ __launch_bounds__(T) void fused_kernel(typename K1::Args a1, typename K2::Args a2, FuseGeom g) {
  fused_block<K1, K2, MATCHED>(a1, a2, g);
}

// The launch-bound presets (hfuse_lb, vfuse_lb).  The reference prints
// `__launch_bounds__(T, B)` with B = min_k(regfile / Reg_k / size_k) capped by the resident
// thread limit (lib/KernelFuser/KernelPrinter.cpp:44-66), i.e. it makes the compiler keep the
// fused kernel's registers low enough for the occupancy the natives had.  The gfx950 form of
// that request is a waves-per-SIMD bound: this build of each fused kernel is compiled for
// W waves per SIMD (at most 512 / W vector registers: 64 for the default of 8), spilling if it must.
template <class K1, class K2, int T, bool MATCHED, int W = kBoundedWaves>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(W, W)))
void fused_kernel_lb(typename K1::Args a1, typename K2::Args a2, FuseGeom g) {
  fused_block<K1, K2, MATCHED>(a1, a2, g);
}

// Fallback when the halves cannot share a workgroup: workgroups [0, grid1) run
// kernel 1 and [grid1, grid1+grid2) run kernel 2, each with the whole
// workgroup's hardware barrier.  The block is max(d1, d2) threads; waves beyond
// a kernel's own size end at once (ended waves do not count at s_barrier).
template <class K1, class K2, int T>
__global__ __launch_bounds__(T) void blockidx_kernel(typename K1::Args a1, typename K2::Args a2, FuseGeom g) {
  extern __shared__ __align__(16) unsigned char smem[];
  const unsigned tid = threadIdx.x;
  if (blockIdx.x < g.grid1) {
    if (tid >= g.d1) return;
    SubBlock<BAR_WORKGROUP> sb{tid, g.d1, blockIdx.x, g.grid1, nullptr, 0, blockIdx.x * g.d1, g.grid1 * g.d1};
    K1::run(a1, sb, smem, g.hint1);
  } else {
    if (tid >= g.d2) return;
    const unsigned b2 = blockIdx.x - g.grid1;
    SubBlock<BAR_WORKGROUP> sb{tid, g.d2, b2, g.grid2, nullptr, 0, b2 * g.d2, g.grid2 * g.d2};
    K2::run(a2, sb, smem, g.hint2);
  }
}

// Vertical fusion, the reference's baseline presets (vfuse, vfuse_lb: main.cpp:183-184,
// KernelFusion.h:76-78 -- both kernels start at thread 0): the block is max(d1, d2) threads
// and the same threads run kernel 1's body and then kernel 2's.  A body that synchronises
// uses its LDS arrival counter, because the threads beyond its own size are still alive
// (they wait for, or already run, the other body) and must not be waited for.
template <class K1, class K2>
__device__ __forceinline__ void vertical_block(const typename K1::Args &a1, const typename K2::Args &a2,
                                               const FuseGeom &g) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned *bars = reinterpret_cast<unsigned *>(smem);
  const unsigned tid = threadIdx.x, bid = blockIdx.x;
  if constexpr (K1::kBarriers || K2::kBarriers) {
    if (tid < kBarrierWords) bars[tid] = 0;
    __syncthreads();
  }
  constexpr int B1 = K1::kBarriers ? BAR_SUBSET : BAR_WORKGROUP;
  constexpr int B2 = K2::kBarriers ? BAR_SUBSET : BAR_WORKGROUP;
  const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // A body as wide as the block runs on every wave, so its barriers are the workgroup's own.
  if (wave < (g.d1 >> 6) && bid < g.grid1) {
    SubBlock<B1> sb{tid, g.d1, bid, g.grid1, bars + 0, 0, bid * g.d1, g.grid1 * g.d1, g.d1 == blockDim.x};
    K1::run(a1, sb, smem + 4 * kBarrierWords, g.hint1);
  }
  if (wave < (g.d2 >> 6) && bid < g.grid2) {
    SubBlock<B2> sb{tid, g.d2, bid, g.grid2, bars + 1, 0, bid * g.d2, g.grid2 * g.d2, g.d2 == blockDim.x};
    K2::run(a2, sb, smem + 4 * kBarrierWords + g.lds1, g.hint2);
  }
}

template <class K1, class K2, int T>
__global__ __launch_bounds__(T) void vertical_kernel(typename K1::Args a1, typename K2::Args a2, FuseGeom g) {
  vertical_block<K1, K2>(a1, a2, g);
}

template <class K1, class K2, int T, int W = kBoundedWaves>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(W, W)))
void vertical_kernel_lb(typename K1::Args a1, typename K2::Args a2, FuseGeom g) {
  vertical_block<K1, K2>(a1, a2, g);
}

// ----------------------------------------------------------------------------
// Three kernels in one workgroup (the reference's Context partitions a block among any number of
// kernels, include/KernelFusion.h:45-80; configs/crypt_four.yaml and im2col_maxpool_norm.yaml
// list three).  Kernel k runs on threads [lo[k], lo[k] + d[k]): in the order a list is built in that is waves
// [0, d0/64), the next d1/64 and the rest; a list that names the same kernels in another order is the same
// instantiation with other bounds and the arguments in the built order.  Each
// kernel strides over its own number of workgroups; in a block beyond that number its waves end at
// once (no lending here).  A body that synchronises uses its own LDS arrival counter.
// ----------------------------------------------------------------------------
struct FuseGeom3 {
  unsigned lo[3];    // first thread of each part (the parts follow the fusion list's order, the kernels the built order)
  unsigned d[3];     // threads of each part
  unsigned lds[3];   // LDS bytes of each part
  unsigned hint[3];  // fast-path selectors
  unsigned grid[3];  // workgroups each kernel strides over
};

template <class K, int BAR>
__device__ __forceinline__ void run_part(const typename K::Args &a, unsigned tid, unsigned d, unsigned bid, unsigned grid,
                                         unsigned *bar, unsigned char *lds, unsigned hint) {
  if (bid >= grid) return;
  SubBlock<BAR> sb{tid, d, bid, grid, bar, 0, bid * d, grid * d};
  K::run(a, sb, lds, hint);
}

template <class K0, class K1, class K2>
__device__ __forceinline__ void fused_block3(const typename K0::Args &a0, const typename K1::Args &a1,
                                             const typename K2::Args &a2, const FuseGeom3 &g) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned *bars = reinterpret_cast<unsigned *>(smem);
  const unsigned tid = threadIdx.x, bid = blockIdx.x;
  constexpr bool kAny = K0::kBarriers || K1::kBarriers || K2::kBarriers;
  if constexpr (kAny) {
    if (tid < kBarrierWords) bars[tid] = 0;
    __syncthreads();
  }
  const unsigned first = __builtin_amdgcn_readfirstlane(tid & ~63u);   // this wave's first thread: the selector is a scalar
  unsigned char *l0 = smem + 4 * kBarrierWords, *l1 = l0 + g.lds[0], *l2 = l1 + g.lds[1];
  if (first - g.lo[0] < g.d[0])
    run_part<K0, K0::kBarriers ? BAR_SUBSET : BAR_WORKGROUP>(a0, tid - g.lo[0], g.d[0], bid, g.grid[0], bars + 0, l0, g.hint[0]);
  else if (first - g.lo[1] < g.d[1])
    run_part<K1, K1::kBarriers ? BAR_SUBSET : BAR_WORKGROUP>(a1, tid - g.lo[1], g.d[1], bid, g.grid[1], bars + 1, l1, g.hint[1]);
  else if (first - g.lo[2] < g.d[2])
    run_part<K2, K2::kBarriers ? BAR_SUBSET : BAR_WORKGROUP>(a2, tid - g.lo[2], g.d[2], bid, g.grid[2], bars + 2, l2,
                                                             g.hint[2]);
}

template <class K0, class K1, class K2, int T>
__global__ __launch_bounds__(T) void fused_kernel3(typename K0::Args a0, typename K1::Args a1, typename K2::Args a2,
                                                   FuseGeom3 g) {
  fused_block3<K0, K1, K2>(a0, a1, a2, g);
}

// The launch-bound presets of a three-kernel list: the same kernel compiled for kBoundedWaves waves per SIMD.
template <class K0, class K1, class K2, int T>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(kBoundedWaves, kBoundedWaves)))
void fused_kernel3_lb(typename K0::Args a0, typename K1::Args a1, typename K2::Args a2, FuseGeom3 g) {
  fused_block3<K0, K1, K2>(a0, a1, a2, g);
}

// The vertical baseline of a three-kernel list: a block of max(d) threads runs the bodies one after the other.
template <class K0, class K1, class K2>
__device__ __forceinline__ void vertical_block3(const typename K0::Args &a0, const typename K1::Args &a1,
                                                const typename K2::Args &a2, const FuseGeom3 &g) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned *bars = reinterpret_cast<unsigned *>(smem);
  const unsigned tid = threadIdx.x, bid = blockIdx.x;
  constexpr bool kAny = K0::kBarriers || K1::kBarriers || K2::kBarriers;
  if constexpr (kAny) {
    if (tid < kBarrierWords) bars[tid] = 0;
    __syncthreads();
  }
  const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char *l0 = smem + 4 * kBarrierWords, *l1 = l0 + g.lds[0], *l2 = l1 + g.lds[1];
  if (wave < (g.d[0] >> 6))
    run_part<K0, K0::kBarriers ? BAR_SUBSET : BAR_WORKGROUP>(a0, tid, g.d[0], bid, g.grid[0], bars + 0, l0, g.hint[0]);
  if (wave < (g.d[1] >> 6))
    run_part<K1, K1::kBarriers ? BAR_SUBSET : BAR_WORKGROUP>(a1, tid, g.d[1], bid, g.grid[1], bars + 1, l1, g.hint[1]);
  if (wave < (g.d[2] >> 6))
    run_part<K2, K2::kBarriers ? BAR_SUBSET : BAR_WORKGROUP>(a2, tid, g.d[2], bid, g.grid[2], bars + 2, l2, g.hint[2]);
}

template <class K0, class K1, class K2, int T>
__global__ __launch_bounds__(T) void vertical_kernel3(typename K0::Args a0, typename K1::Args a1, typename K2::Args a2,
                                                      FuseGeom3 g) {
  vertical_block3<K0, K1, K2>(a0, a1, a2, g);
}

template <class K0, class K1, class K2, int T>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(kBoundedWaves, kBoundedWaves)))
void vertical_kernel3_lb(typename K0::Args a0, typename K1::Args a1, typename K2::Args a2, FuseGeom3 g) {
  vertical_block3<K0, K1, K2>(a0, a1, a2, g);
}

}  // namespace hfuse
