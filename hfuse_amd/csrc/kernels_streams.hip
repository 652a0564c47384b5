// Bare stream kernels: what this part's memory system delivers for the access patterns the library's kernels have,
// so that each kernel can be judged against the ceiling of its own pattern in the same run.  16-byte accesses per
// lane, non-temporal, every load or store instruction of a wave one contiguous KiB (except the random-line pattern).
#include "launch.h"

namespace hfuse {
namespace {

__device__ __forceinline__ unsigned mix32(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

__global__ void stream_empty_kernel() {}

// Each workgroup reads one contiguous region, eight loads in flight per lane.
__global__ __launch_bounds__(1024) void stream_read_kernel(const f32x4 *__restrict__ p, unsigned long long n4, float *sink) {
  constexpr int U = 8;
  const unsigned tid = threadIdx.x, nt = blockDim.x;
  const unsigned long long per = n4 / gridDim.x;   // the host passes a size the grid divides
  const f32x4 *q = p + (unsigned long long)blockIdx.x * per;
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  unsigned long long i = tid;
  for (; i + (U - 1) * nt < per; i += U * nt) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = __builtin_nontemporal_load(q + i + u * nt);
#pragma unroll
    for (int u = 0; u < U; u++) acc += v[u];
  }
  for (; i < per; i += nt) acc += __builtin_nontemporal_load(q + i);
  const float s = acc.x + acc.y + acc.z + acc.w;
  if (s == 12345.678f) *sink = s;   // keeps the loads alive; never true for the probe's fill
}

// Each workgroup writes one contiguous region.  XCD: the workgroups are renumbered so that each of the eight XCDs
// (workgroups are dealt to them round-robin) owns one contiguous eighth of the buffer.
template <bool XCD>
__global__ __launch_bounds__(1024) void stream_write_kernel(f32x4 *__restrict__ p, unsigned long long n4) {
  const unsigned tid = threadIdx.x, nt = blockDim.x;
  unsigned bid = blockIdx.x;
  if (XCD) bid = (bid & 7u) * (gridDim.x >> 3) + (bid >> 3);
  const unsigned long long per = n4 / gridDim.x;
  f32x4 *q = p + (unsigned long long)bid * per;
  const f32x4 v = {1.0f, 2.0f, 3.0f, (float)tid};
  for (unsigned long long i = tid; i < per; i += nt) __builtin_nontemporal_store(v, q + i);
}

// The whole grid writes one window of the buffer at a time (a grid-stride loop).
__global__ __launch_bounds__(1024) void stream_write_strided_kernel(f32x4 *__restrict__ p, unsigned long long n4) {
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  const f32x4 v = {1.0f, 2.0f, 3.0f, (float)threadIdx.x};
  for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
    __builtin_nontemporal_store(v, p + i);
}

// Uniformly random 128-byte lines out of the whole buffer, eight lanes a line, four lines in flight per lane
// (the DAG reads of Ethash); n4 vectors are read in total.
__global__ __launch_bounds__(1024) void stream_read_lines_kernel(const f32x4 *__restrict__ p, unsigned long long n4,
                                                                 float *sink) {
  constexpr int U = 4;
  const unsigned tid = threadIdx.x, nt = blockDim.x;
  const unsigned long long per_thread = n4 / ((unsigned long long)gridDim.x * nt);
  const unsigned group = (blockIdx.x * nt + tid) >> 3, within = tid & 7u;
  const unsigned nlines = (unsigned)(n4 >> 3);
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (unsigned long long k = 0; k + U <= per_thread; k += U) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const unsigned line = mix32(group * 2654435761u + (unsigned)(k + u) * 40503u + 12345u) % nlines;
      v[u] = __builtin_nontemporal_load(p + (unsigned long long)line * 8u + within);
    }
#pragma unroll
    for (int u = 0; u < U; u++) acc += v[u];
  }
  const float s = acc.x + acc.y + acc.z + acc.w;
  if (s == 12345.678f) *sink = s;
}

// One vector read, four written (to four planes of n4 vectors each): the shape of nearest-neighbour upsampling.
__global__ __launch_bounds__(1024) void stream_copy_1_4_kernel(const f32x4 *__restrict__ src, f32x4 *__restrict__ dst,
                                                               unsigned long long n4) {
  constexpr int U = 2;
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + (U - 1) * stride < n4; i += U * stride) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = src[i + u * stride];
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int r = 0; r < 4; r++) __builtin_nontemporal_store(v[u], dst + (unsigned long long)r * n4 + i + u * stride);
  }
  for (; i < n4; i += stride) {
    const f32x4 v = src[i];
#pragma unroll
    for (int r = 0; r < 4; r++) __builtin_nontemporal_store(v, dst + (unsigned long long)r * n4 + i);
  }
}

}  // namespace

hipError_t launch_stream_probe(int pattern, const void *src, void *dst, unsigned long long n4, unsigned grid, unsigned block,
                               hipStream_t s) {
  const f32x4 *in = static_cast<const f32x4 *>(src);
  switch (pattern) {
    case 0: hipLaunchKernelGGL(stream_empty_kernel, dim3(1), dim3(64), 0, s); break;
    case 1: hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(block), 0, s, in, n4, static_cast<float *>(dst)); break;
    case 2: hipLaunchKernelGGL(stream_write_kernel<false>, dim3(grid), dim3(block), 0, s, static_cast<f32x4 *>(dst), n4); break;
    case 5: hipLaunchKernelGGL(stream_write_strided_kernel, dim3(grid), dim3(block), 0, s, static_cast<f32x4 *>(dst), n4); break;
    case 6: hipLaunchKernelGGL(stream_write_kernel<true>, dim3(grid), dim3(block), 0, s, static_cast<f32x4 *>(dst), n4); break;
    case 3: hipLaunchKernelGGL(stream_read_lines_kernel, dim3(grid), dim3(block), 0, s, in, n4, static_cast<float *>(dst)); break;
    case 4: hipLaunchKernelGGL(stream_copy_1_4_kernel, dim3(grid), dim3(block), 0, s, in, static_cast<f32x4 *>(dst), n4); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace hfuse
