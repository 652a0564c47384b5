// Device bodies of the five tensor kernels.  Each body is written once against
// SubBlock and is instantiated both as a native kernel and as one half of a
// fused kernel.  Every body has a general path that follows the original
// kernel's semantics for any argument list, and a vectorised path (selected by
// a host-validated hint) for the layouts that matter: 16-byte aligned rows,
// stride-1 3x3 im2col, stride-2 pooling, exact 2x nearest upsampling.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../../include/hfuse_gfx950.h"
#include "subblock.h"

namespace hfuse {

// Hints (0 always means the general path).
enum { HINT_GENERIC = 0, HINT_IM2COL_3X3_S1P1 = 1, HINT_POOL_K3S2P1 = 1, HINT_POOL_K2S2P0 = 2, HINT_UP_2X = 1, HINT_BN_VEC4 = 1, HINT_HIST_VEC4 = 1, HINT_HIST_POW2 = 2, HINT_HIST_GLOBAL = 8 /* more bins than the LDS budget: count straight into global memory */, HINT_HIST_HEAD_SHIFT = 4 /* bits 4-5: elements before the first 16-byte boundary */, HINT_BILINEAR_VEC4 = 1, HINT_BILINEAR_2X = 2, HINT_BILINEAR_2X_ALIGN = 3,
       // general path with 32-bit index arithmetic: every tensor of the call has fewer than 2^31 elements
       HINT_IDX32 = 0x100 };

__device__ __forceinline__ f32x4 ld4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
// The same load with the non-temporal hint, for streams whose every byte is read once (the histogram's
// input, batch-norm planes, 2x2 pooling windows): they then leave the caches to whoever re-reads.  Kernels that do re-read
// through the cache (im2col's taps, overlapping 3x3 windows) lose 10-30 % with it.
#ifndef HF_NT_LOADS
#define HF_NT_LOADS 1
#endif
__device__ __forceinline__ f32x4 ld4_stream(const float *p) {
#if HF_NT_LOADS
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
#else
  return *reinterpret_cast<const f32x4 *>(p);
#endif
}

// One DPP move of a float.  0x138 = wave_shr:1 (lane i receives lane i-1's value),
// 0x130 = wave_shl:1 (lane i receives lane i+1's); the lane without a source keeps 0.
// The first active lane's value of a 64-bit quantity, as a wave-uniform value.
__device__ __forceinline__ size_t uniform_u64(size_t x) {
  return ((size_t)__builtin_amdgcn_readfirstlane((unsigned)(x >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((unsigned)x);
}
// Lane 63's value of a 64-bit quantity, as a wave-uniform value (every lane of the wavefront must be active).
__device__ __forceinline__ size_t uniform_last_u64(size_t x) {
  return ((size_t)(unsigned)__builtin_amdgcn_readlane((int)(unsigned)(x >> 32), 63) << 32) |
         (unsigned)__builtin_amdgcn_readlane((int)(unsigned)x, 63);
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
#ifndef HF_NT_STORES
#define HF_NT_STORES 1
#endif
// Timing-only builds that take a fused pair apart (any bit set gives wrong results; the default 0 is the product):
//   1  max-pooling 2x2: stores off      2  max-pooling 2x2: loads off (window values made up from the index)
//   4  histogram: LDS atomics off       8  histogram: loads off (element values made up from the index)
#ifndef HF_TAKEAPART
#define HF_TAKEAPART 0
#endif
__device__ __forceinline__ void st4(float *p, f32x4 v) {
#if HF_NT_STORES
  __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
#else
  *reinterpret_cast<f32x4 *>(p) = v;
#endif
}

// ----------------------------------------------------------------------------
// im2col_kernel<float>  (argument list: scripts/data/ml-event.csv:17)
// One work item per (channel_in, h_out, w_out): kernel_h*kernel_w taps go to
// rows channel_in*kh*kw + i*kw + j of the column matrix, zero outside the image.
// ----------------------------------------------------------------------------
struct Im2colBody {
  static constexpr KernelId kId = K_IM2COL;
  using Args = hf_im2col_args;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = true;  // walks one flat index range: may borrow a partner's idle waves
  // Every work item writes kernel_h*kernel_w separate rows of the column matrix.  With all 32 waves of a CU
  // resident the chip writes into so many places at once that HBM takes the stores at 5.4 TB/s; with 16 waves
  // per CU (4 per SIMD) the same launch reaches 5.9-6.0 TB/s (47.2 -> 43.0 us at [32,64,56,56], 3x3).
  static constexpr int kNativeWaves = 4;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned hint) {
    if (hint == HINT_IM2COL_3X3_S1P1) {
      vec4_3x3(a, sb);
      return;
    }
    if (hint == HINT_IDX32) general<unsigned, int>(a, sb);
    else general<int64_t, int64_t>(a, sb);
  }

  // The original per-element loop, any geometry.  I indexes work items and elements (64-bit
  // division is a long instruction sequence on this part, so tensors below 2^31 elements use
  // 32-bit indices), S is the signed type of image coordinates.
  template <class I, class S, class SB>
  static __device__ __forceinline__ void general(const Args &a, SB &sb) {
    const I stride = (I)sb.gstride(), n = (I)a.n;
    const I width_col = (I)a.width_col, height_col = (I)a.height_col, plane_col = height_col * width_col;
    const I kh = (I)a.kernel_h, kw = (I)a.kernel_w;
    const S height = (S)a.height, width = (S)a.width, dil_h = (S)a.dilation_h, dil_w = (S)a.dilation_w;
    for (I index = (I)sb.gtid(); index < n; index += stride) {
      const I w_out = index % width_col;
      const I idx = index / width_col;
      const I h_out = idx % height_col;
      const I channel_in = idx / height_col;
      const I channel_out = channel_in * kh * kw;
      const S h_in = (S)h_out * (S)a.stride_h - (S)a.pad_h;
      const S w_in = (S)w_out * (S)a.stride_w - (S)a.pad_w;
      float *col = a.data_col + (size_t)((channel_out * height_col + h_out) * width_col + w_out);
      const float *im = a.data_im + (ptrdiff_t)((S)channel_in * height + h_in) * (ptrdiff_t)width + (ptrdiff_t)w_in;
      for (I i = 0; i < kh; ++i) {
        for (I j = 0; j < kw; ++j) {
          const S h = h_in + (S)i * dil_h, w = w_in + (S)j * dil_w;
          *col = (h >= 0 && w >= 0 && h < height && w < width) ? im[(ptrdiff_t)((S)i * dil_h * width + (S)j * dil_w)] : 0.0f;
          col += plane_col;
        }
      }
    }
  }

  // 3x3, stride 1, pad 1, dilation 1, width % 4 == 0: a work item owns four
  // neighbouring output columns.  Per input row it needs columns w0-1 .. w0+4:
  // one aligned 16-byte load; the two edge columns are the neighbouring lanes'
  // outer elements, moved with a wavefront-wide DPP shift (lanes 0 and 63 fetch
  // theirs from memory with one single-lane load each; taking them from a
  // wave-uniform address instead, as the bilinear kernel does, costs this kernel
  // 8-9 %: it writes fastest with a slow front end).  Each of the nine taps is
  // then one 16-byte store.  The trip count is wave-uniform so every lane's
  // neighbour is live.
  template <class SB>
  static __device__ __forceinline__ void vec4_3x3(const Args &a, SB &sb) {
    const unsigned W = (unsigned)a.width, H = (unsigned)a.height;
    const unsigned wq = W >> 2;
    const unsigned plane = H * W;
    const unsigned n4 = (unsigned)(a.n >> 2);
    const unsigned stride = sb.gstride();
    const unsigned lane = sb.lane();
    for (unsigned first = sb.gtid() - lane; first < n4; first += stride) {
      const bool valid = first + lane < n4;
      const unsigned idx4 = valid ? first + lane : n4 - 1;
      const unsigned w4 = idx4 % wq;
      const unsigned t = idx4 / wq;
      const unsigned h_out = t % H;
      const unsigned c = t / H;
      const unsigned w0 = w4 << 2;
      const float *im = a.data_im + (size_t)c * plane;
      float *col = a.data_col + (size_t)c * 9u * plane + (size_t)h_out * W + w0;
      const bool has_left = w0 > 0, has_right = w0 + 4 < W;
      float r[3][6];
#pragma unroll
      for (int i = 0; i < 3; i++) {
        const int h = (int)h_out - 1 + i;
        const bool in = h >= 0 && h < (int)H;
        const float *row = im + (unsigned)(in ? h : (int)h_out) * W + w0;
        f32x4 m = ld4(row);
        if (!in) m = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        float left = dpp_f32<0x138>(m.w);   // wave_shr:1 -- lane-1's last column
        float right = dpp_f32<0x130>(m.x);  // wave_shl:1 -- lane+1's first column
        if (lane == 0 && has_left) left = in ? row[-1] : 0.0f;
        if (lane == 63 && has_right) right = in ? row[4] : 0.0f;
        r[i][0] = has_left ? left : 0.0f;
        r[i][1] = m.x; r[i][2] = m.y; r[i][3] = m.z; r[i][4] = m.w;
        r[i][5] = has_right ? right : 0.0f;
      }
      if (valid) {
#pragma unroll
        for (int i = 0; i < 3; i++)
#pragma unroll
          for (int j = 0; j < 3; j++) {
            f32x4 v = {r[i][j], r[i][j + 1], r[i][j + 2], r[i][j + 3]};
            st4(col + (size_t)(i * 3 + j) * plane, v);
          }
      }
    }
  }
};

// ----------------------------------------------------------------------------
// MaxPoolForward<float,float>  (argument list: scripts/data/ml-event.csv:5)
// One work item per output; the window is scanned in (h, w) order and replaced
// on `v > max || isnan(v)`, so ties keep the first index; the mask is h*W+w.
// ----------------------------------------------------------------------------
struct MaxPoolBody {
  static constexpr KernelId kId = K_MAXPOOL;
  using Args = hf_maxpool_args;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = true;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned hint) {
    if (hint == HINT_POOL_K3S2P1) { vec2_s2<3, 1>(a, sb); return; }
    if (hint == HINT_POOL_K2S2P0) { vec2_s2<2, 0>(a, sb); return; }
    if (hint == HINT_IDX32) general<unsigned>(a, sb);
    else general<int64_t>(a, sb);
  }

  // The original loop: any window, stride, padding and dilation.  I is the index type
  // (32-bit when input and output have fewer than 2^31 elements).
  template <class I, class SB>
  static __device__ __forceinline__ void general(const Args &a, SB &sb) {
    const I stride = (I)sb.gstride(), n = (I)a.nthreads;
    const I pw_n = (I)a.pooled_width, ph_n = (I)a.pooled_height, ch_n = (I)a.channels;
    for (I index = (I)sb.gtid(); index < n; index += stride) {
      const I t0 = index / pw_n, t1 = t0 / ph_n;
      const int pw = (int)(index - t0 * pw_n);
      const int ph = (int)(t0 - t1 * ph_n);
      const I nn = t1 / ch_n;
      const int c = (int)(t1 - nn * ch_n);
      int hstart = ph * a.stride_h - a.pad_h;
      int wstart = pw * a.stride_w - a.pad_w;
      const int hend = min(hstart + (a.kernel_h - 1) * a.dilation_h + 1, a.height);
      const int wend = min(wstart + (a.kernel_w - 1) * a.dilation_w + 1, a.width);
      while (hstart < 0) hstart += a.dilation_h;
      while (wstart < 0) wstart += a.dilation_w;
      float maxval = -INFINITY;
      int maxidx = hstart * a.width + wstart;
      const float *plane = a.bottom_data + (size_t)((nn * ch_n + (I)c) * (I)a.height) * (size_t)a.width;
      for (int h = hstart; h < hend; h += a.dilation_h)
        for (int w = wstart; w < wend; w += a.dilation_w) {
          const float v = plane[h * a.width + w];
          if ((v > maxval) || isnan(v)) {
            maxidx = h * a.width + w;
            maxval = v;
          }
        }
      a.top_data[index] = maxval;
      a.top_mask[index] = maxidx;
    }
  }

  // K x K window, stride 2, pad P (K=3,P=1 or K=2,P=0), width % 4 == 0 and
  // pooled_width == width/2: a work item owns two neighbouring outputs and reads,
  // per window row, one aligned 16-byte vector (+ the left edge for P=1).  Two
  // outputs per lane make every store instruction of the wave one contiguous
  // run (8 B of values, 16 B of int64 indices per lane): write-once streams
  // leave the chip as whole lines.
  template <int K, int P, class SB>
  static __device__ __forceinline__ void vec2_s2(const Args &a, SB &sb) {
    const unsigned W = (unsigned)a.width, H = (unsigned)a.height;
    const unsigned PW = (unsigned)a.pooled_width, PH = (unsigned)a.pooled_height;
    const unsigned ph2 = PW >> 1;
    const unsigned n2 = (unsigned)a.nthreads >> 1;
    const unsigned stride = sb.gstride();
    // One work item: its K window rows are loaded first (`load_item`), compared and stored later (`finish_item`), so
    // that a thread which loops over several items has the loads of two of them in flight at a time.
    auto load_item = [&](unsigned idx2, f32x4 (&v)[K], float (&left)[K]) __attribute__((always_inline)) {
      const unsigned pw2 = idx2 % ph2;
      const unsigned t = idx2 / ph2;
      const unsigned ph = t % PH;
      const unsigned nc = t / PH;
      const float *plane = a.bottom_data + (size_t)nc * H * W;
      const int hstart = (int)ph * 2 - P;
      const unsigned wbase = pw2 << 2;
      const int h0 = hstart < 0 ? 0 : hstart;
#pragma unroll
      for (int i = 0; i < K; i++) {
        const int h = hstart + i;
        const bool in = h >= 0 && h < (int)H;
        const float *row = plane + (unsigned)(in ? h : h0) * W + wbase;
        if ((HF_TAKEAPART & 2) && K == 2) {
          const float f = __builtin_bit_cast(float, (idx2 * 2654435761u + (unsigned)i) >> 9 | 0x3f800000u);
          v[i] = f32x4{f, f + 0.25f, f + 0.5f, f + 0.125f};
        } else {
          v[i] = (K == 2 && P == 0) ? ld4_stream(row) : ld4(row);
        }
        left[i] = 0.0f;
        if constexpr (P == 1) {
          // Lane 0 has nobody to its left in this wavefront: its column wbase - 1 is loaded from an
          // address every lane agrees on (one cache line, no divergence).  In column 0 it is padding.
          const size_t off = (size_t)(row - a.bottom_data);
          left[i] = a.bottom_data[uniform_u64(wbase > 0 ? off - 1 : off)];
        }
      }
      if constexpr (P == 1) {
        // Column wbase - 1 is the last column of the lane to the left (neighbouring lanes hold
        // neighbouring work items; with wbase > 0 they sit in the same output row and loaded the
        // same input rows), so it comes by a wavefront shift instead of a second load per row.
#pragma unroll
        for (int i = 0; i < K; i++) {
          const float from_left = dpp_f32<0x138>(v[i].w);
          if (sb.lane() != 0) left[i] = from_left;
        }
      }
    };
    auto finish_item = [&](unsigned idx2, const f32x4 (&v)[K], const float (&left)[K]) __attribute__((always_inline)) {
      const unsigned pw2 = idx2 % ph2;
      const unsigned ph = (idx2 / ph2) % PH;
      const int hstart = (int)ph * 2 - P;
      const unsigned wbase = pw2 << 2;
      const int h0 = hstart < 0 ? 0 : hstart;
      float maxv[2];
      int maxi[2];
#pragma unroll
      for (int o = 0; o < 2; o++) {
        const int ws = (int)wbase + 2 * o - P;
        maxv[o] = -INFINITY;
        maxi[o] = h0 * (int)W + (ws < 0 ? 0 : ws);
      }
#pragma unroll
      for (int i = 0; i < K; i++) {
        const int h = hstart + i;
        if (h < 0 || h >= (int)H) continue;
        // vals[k] is input column wbase - P + k
        float vals[5];
        if (P == 1) {
          vals[0] = left[i]; vals[1] = v[i].x; vals[2] = v[i].y; vals[3] = v[i].z; vals[4] = v[i].w;
        } else {
          vals[0] = v[i].x; vals[1] = v[i].y; vals[2] = v[i].z; vals[3] = v[i].w; vals[4] = 0.0f;
        }
        const int base_idx = h * (int)W + (int)wbase - P;
#pragma unroll
        for (int o = 0; o < 2; o++)
#pragma unroll
          for (int j = 0; j < K; j++) {
            const int k = 2 * o + j;
            if (P == 1 && k == 0 && wbase == 0) continue;  // column -1 is padding
            const float x = vals[k];
            if ((x > maxv[o]) || isnan(x)) {
              maxv[o] = x;
              maxi[o] = base_idx + k;
            }
          }
      }
      const f32x2 ov = {maxv[0], maxv[1]};
      const i64x2 om = {maxi[0], maxi[1]};
      f32x2 *vp = reinterpret_cast<f32x2 *>(a.top_data + (size_t)idx2 * 2);
      i64x2 *mp = reinterpret_cast<i64x2 *>(a.top_mask + (size_t)idx2 * 2);
      if ((HF_TAKEAPART & 1) && K == 2 && !(maxv[0] == 12345.678f && maxi[1] == -7)) return;  // keeps the loads alive
#if HF_NT_STORES
      __builtin_nontemporal_store(ov, vp);
      __builtin_nontemporal_store(om, mp);
#else
      *vp = ov;
      *mp = om;
#endif
    };
    // Two items per trip (the second one `stride` further on; the lanes that have one are a prefix of the wave, so
    // every lane that shifts a halo column in still has its left neighbour).  A launch in which every thread
    // has one item -- the native one -- never enters the second half.
    for (unsigned idx2 = sb.gtid(); idx2 < n2; idx2 += 2 * stride) {
      const unsigned idx_b = idx2 + stride;
      const bool has_b = idx_b < n2;
      f32x4 va[K], vb[K];
      float la[K], lb[K];
      load_item(idx2, va, la);
      if (has_b) load_item(idx_b, vb, lb);
      finish_item(idx2, va, la);
      if (has_b) finish_item(idx_b, vb, lb);
    }
  }
};

// ----------------------------------------------------------------------------
// upsample_nearest2d_out_frame<float>: src = min((int)floorf(dst * scale), in - 1)
// ----------------------------------------------------------------------------
struct UpsampleNearestBody {
  static constexpr KernelId kId = K_UPSAMPLE_NEAREST;
  using Args = hf_upsample_nearest_args;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = true;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned hint) {
    if (hint == HINT_UP_2X) {
      // Exact 2x: a lane loads two neighbouring input pixels (8 B) and stores the four
      // output pixels they expand to (16 B) into both output rows, so each load and each
      // store instruction of the wave covers one contiguous run.  Two items per trip keep
      // two loads in flight.
      const unsigned w1h = (unsigned)a.width1 >> 1;
      const unsigned w2 = (unsigned)a.width2;
      const unsigned n2 = (unsigned)(a.nc * a.height1) * w1h;
      const unsigned stride = sb.gstride();
      const f32x2 *in = reinterpret_cast<const f32x2 *>(a.idata);
      for (unsigned idx = sb.gtid(); idx < n2; idx += 2 * stride) {
        const unsigned idx_b = idx + stride;
        const bool has_b = idx_b < n2;
        const f32x2 va = in[idx];
        const f32x2 vb = has_b ? in[idx_b] : f32x2{0.0f, 0.0f};
        {
          const unsigned xh = idx % w1h, row = idx / w1h;  // row = c * h1 + y1; output row = 2 * row
          float *o = a.odata + (size_t)row * 2u * w2 + (size_t)xh * 4u;
          const f32x4 e = {va.x, va.x, va.y, va.y};
          st4(o, e);
          st4(o + w2, e);
        }
        if (has_b) {
          const unsigned xh = idx_b % w1h, row = idx_b / w1h;
          float *o = a.odata + (size_t)row * 2u * w2 + (size_t)xh * 4u;
          const f32x4 e = {vb.x, vb.x, vb.y, vb.y};
          st4(o, e);
          st4(o + w2, e);
        }
      }
      return;
    }
    if (hint == HINT_IDX32) general<unsigned>(a, sb);
    else general<size_t>(a, sb);
  }

  // The original per-pixel loop, any sizes and scales: src = min(floor(dst * scale), in - 1).
  template <class I, class SB>
  static __device__ __forceinline__ void general(const Args &a, SB &sb) {
    const I w2 = (I)a.width2, h2 = (I)a.height2, w1 = (I)a.width1, h1 = (I)a.height1;
    const I total = (I)a.nc * h2 * w2;
    const I stride = (I)sb.gstride();
    for (I index = (I)sb.gtid(); index < total; index += stride) {
      const I t = index / w2;
      const I x2 = index - t * w2;
      const I c = t / h2;
      const I y2 = t - c * h2;
      const int y1 = min((int)floorf((float)y2 * a.height_scale), (int)a.height1 - 1);
      const int x1 = min((int)floorf((float)x2 * a.width_scale), (int)a.width1 - 1);
      a.odata[index] = a.idata[(c * h1 + (I)y1) * w1 + (I)x1];
    }
  }
};

// ----------------------------------------------------------------------------
// upsample_bilinear2d_out_frame<float,float>  (argument list: scripts/data/ml-event.csv:9)
//   src = align_corners ? scale*dst : max(scale*(dst+0.5)-0.5, 0); i1 = (int)src; l1 = src-i1
//   out = h0*(w0*a + w1*b) + h1*(w0*c + w1*d)
// Every product and sum is rounded on its own (rn_mul / rn_add below keep the compiler from
// contracting them into FMAs), so results are the same bits as a plain fp32 CPU evaluation.
// The original runs one thread per output pixel and loops over batch and channels; here the
// flat range is all outputs, four neighbouring columns per work item where the output is
// contiguous, which keeps the stores 16 bytes per lane and contiguous across the wave.
// ----------------------------------------------------------------------------
// Singly rounded fp32 operations: the pragma keeps the compiler from contracting a
// product and the sum that uses it into one fused multiply-add (HIP's __fmul_rn and
// __fadd_rn are plain operators, which the default -ffp-contract=fast may fuse).
__device__ __forceinline__ float rn_mul(float x, float y) {
#pragma clang fp contract(off)
  return x * y;
}
__device__ __forceinline__ float rn_add(float x, float y) {
#pragma clang fp contract(off)
  return x + y;
}
__device__ __forceinline__ float rn_sub(float x, float y) {
#pragma clang fp contract(off)
  return x - y;
}

struct UpsampleBilinearBody {
  static constexpr KernelId kId = K_UPSAMPLE_BILINEAR;
  using Args = hf_upsample_bilinear_args;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = true;

  static __device__ __forceinline__ float src_index(float scale, int dst, bool align) {
    if (align) return rn_mul(scale, (float)dst);
    const float s = rn_sub(rn_mul(scale, rn_add((float)dst, 0.5f)), 0.5f);
    return s < 0.0f ? 0.0f : s;
  }

  static __device__ __forceinline__ float blend(float h0, float h1, float w0, float w1, float a, float b, float c,
                                                float d) {
    const float top = rn_add(rn_mul(w0, a), rn_mul(w1, b));
    const float bot = rn_add(rn_mul(w0, c), rn_mul(w1, d));
    return rn_add(rn_mul(h0, top), rn_mul(h1, bot));
  }

  // Exact 2x, contiguous NCHW, even input width.  A work item owns input rows 2p, 2p+1, columns 2q, 2q+1 and
  // writes output rows 4p..4p+3, columns 4q..4q+3: those sixteen outputs read input rows 2p-1..2p+2 (clamped)
  // at columns 2q-1..2q+2.  Each row is one 8-byte load; the two outer columns are the neighbouring lanes'
  // elements, moved with a wavefront-wide DPP shift (lanes 0 and 63 fetch theirs from memory).  At twice the
  // size the source of output d starts at input (d - 1) >> 1 (0 for d = 0), with or without align_corners, so
  // which rows and columns an output blends is fixed and only the weights differ: without align_corners
  // 0.5 * (d + 0.5) - 0.5 is exact and the weights are the constants 0.25 / 0.75 (1 / 0 at the clamped first
  // column and row); with align_corners the weights come from the general path's expressions, and the host
  // takes this path only after checking, in the same fp32 steps, that every output's source index is the one
  // above.  Either way the bits are those of the general path.  The trip count is wave-uniform so every
  // lane's neighbour is live.
  template <bool ALIGN, class SB>
  static __device__ __forceinline__ void exact2x(const Args &a, SB &sb) {
    const unsigned H1 = (unsigned)a.idata.sizes[2], W1 = (unsigned)a.idata.sizes[3];
    const unsigned W2 = W1 * 2u;
    const unsigned wq = W1 >> 1, hp = (H1 + 1u) >> 1;
    const unsigned NC = (unsigned)(a.idata.sizes[0] * a.idata.sizes[1]);
    const unsigned n = NC * hp * wq;
    const unsigned stride = sb.gstride();
    const unsigned lane = sb.lane();
    for (unsigned first = sb.gtid() - lane; first < n; first += stride) {
      const bool valid = first + lane < n;
      const unsigned idx = valid ? first + lane : n - 1;
      const unsigned q = idx % wq;
      const unsigned t = idx / wq;
      const unsigned p = t % hp;
      const unsigned nc = t / hp;
      const unsigned j0 = 2u * p;
      const bool second = j0 + 1u < H1;  // an odd height leaves the last work item of a plane one input row
      const float *pl = a.idata.data + (size_t)nc * H1 * W1 + 2u * q;
      const unsigned jr[4] = {j0 > 0 ? j0 - 1 : 0u, j0, second ? j0 + 1 : j0, j0 + 2 < H1 ? j0 + 2 : H1 - 1};
      const bool has_left = q > 0, has_right = q + 1 < wq;
      float wl[4], wr[4];  // weight of the left / right source column of output 4q+k
#pragma unroll
      for (int k = 0; k < 4; k++) {
        if (ALIGN) {
          const float w1r = src_index(a.rwidth, (int)(4u * q) + k, true);
          wr[k] = rn_sub(w1r, (float)(int)w1r);
        } else {
          wr[k] = (k & 1) ? 0.25f : (k == 0 && !has_left) ? 0.0f : 0.75f;
        }
        wl[k] = rn_sub(1.0f, wr[k]);
      }
      // All loads of the work item are issued before the first use.  Lane 0 has nobody to its left in this
      // wavefront and lane 63 nobody to its right: their outer columns are loaded from addresses every lane agrees
      // on (one cache line each, no divergence, nothing to wait for in turn).
      float2 mm[4];
      float edge_l[4], edge_r[4];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float *row = pl + (size_t)jr[r] * W1;
        mm[r] = *reinterpret_cast<const float2 *>(row);
        const size_t off = (size_t)(row - a.idata.data);
        edge_l[r] = a.idata.data[uniform_u64(has_left ? off - 1 : off)];
        edge_r[r] = a.idata.data[uniform_last_u64(has_right ? off + 2 : off)];
      }
      float hl[4][4];  // horizontally interpolated rows 2p-1 .. 2p+2
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float2 m = mm[r];
        float left = dpp_f32<0x138>(m.y);   // wave_shr:1 -- lane-1's second column
        float right = dpp_f32<0x130>(m.x);  // wave_shl:1 -- lane+1's first column
        if (lane == 0) left = edge_l[r];
        if (lane == 63) right = edge_r[r];
        // output 4q: source columns (2q-1, 2q), or (0, 1) with weights (1, 0) at the left edge
        hl[r][0] = rn_add(rn_mul(wl[0], has_left ? left : m.x), rn_mul(wr[0], has_left ? m.x : m.y));
        hl[r][1] = rn_add(rn_mul(wl[1], m.x), rn_mul(wr[1], m.y));
        hl[r][2] = rn_add(rn_mul(wl[2], m.x), rn_mul(wr[2], m.y));
        // output 4q+3: source columns (2q+1, 2q+2); the last column pairs with itself
        hl[r][3] = rn_add(rn_mul(wl[3], m.y), rn_mul(wr[3], has_right ? right : m.y));
      }
      // Output row 2j blends input rows (j-1, j), or (0, 1) with weights (1, 0) at the top edge; output row 2j+1
      // blends (j, j+1), the last row with itself.  hl[0..3] are rows 2p-1, 2p, 2p+1, 2p+2, clamped to the plane.
      float *out = a.odata.data + ((size_t)nc * (2u * H1) + 2u * j0) * W2 + 4u * q;
#pragma unroll
      for (int s = 0; s < 4; s++) {
        float bw;
        if (ALIGN) {
          const float h1r = src_index(a.rheight, (int)(2u * j0) + s, true);
          bw = rn_sub(h1r, (float)(int)h1r);
        } else {
          bw = (s & 1) ? 0.25f : (s == 0 && j0 == 0) ? 0.0f : 0.75f;
        }
        const float tw = rn_sub(1.0f, bw);
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const float top = s == 0 ? hl[0][k] : s == 3 ? hl[2][k] : hl[1][k];
          const float bot = s == 0 ? (j0 > 0 ? hl[1][k] : hl[2][k]) : s == 3 ? hl[3][k] : hl[2][k];
          o[k] = rn_add(rn_mul(tw, top), rn_mul(bw, bot));
        }
        if (valid && (s < 2 || second)) st4(out + (size_t)s * W2, f32x4{o[0], o[1], o[2], o[3]});
      }
    }
  }

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned hint) {
    const int H1 = (int)a.idata.sizes[2], W1 = (int)a.idata.sizes[3];
    const int H2 = (int)a.odata.sizes[2], W2 = (int)a.odata.sizes[3];
    const unsigned NC = (unsigned)(a.idata.sizes[0] * a.idata.sizes[1]);
    const unsigned C = (unsigned)a.idata.sizes[1];
    const bool align = a.align_corners != 0;
    const bool same = H1 == H2 && W1 == W2;
    if (hint == HINT_BILINEAR_2X) {
      exact2x<false>(a, sb);
      return;
    }
    if (hint == HINT_BILINEAR_2X_ALIGN) {
      exact2x<true>(a, sb);
      return;
    }
    if (hint == HINT_BILINEAR_VEC4) {
      // contiguous NCHW on both sides, W2 % 4 == 0, 16-byte aligned output
      const unsigned wq = (unsigned)W2 >> 2;
      const unsigned n4 = NC * (unsigned)H2 * wq;
      const unsigned stride = sb.gstride();
      for (unsigned idx = sb.gtid(); idx < n4; idx += stride) {
        const unsigned xq = idx % wq;
        const unsigned t = idx / wq;
        const int y2 = (int)(t % (unsigned)H2);
        const unsigned nc = t / (unsigned)H2;
        const float *in = a.idata.data + (size_t)nc * H1 * W1;
        f32x4 o;
        if (same) {
          o = ld4(in + (size_t)y2 * W1 + xq * 4);
        } else {
          const float h1r = src_index(a.rheight, y2, align);
          const int y1 = (int)h1r;
          const int y1p = (y1 < H1 - 1) ? 1 : 0;
          const float h1l = rn_sub(h1r, (float)y1), h0l = rn_sub(1.0f, h1l);
          const float *r0 = in + (size_t)y1 * W1, *r1 = r0 + (size_t)y1p * W1;
          float v[4];
#pragma unroll
          for (int k = 0; k < 4; k++) {
            const float w1r = src_index(a.rwidth, (int)(xq * 4) + k, align);
            const int x1 = (int)w1r;
            const int x1p = (x1 < W1 - 1) ? 1 : 0;
            const float w1l = rn_sub(w1r, (float)x1), w0l = rn_sub(1.0f, w1l);
            v[k] = blend(h0l, h1l, w0l, w1l, r0[x1], r0[x1 + x1p], r1[x1], r1[x1 + x1p]);
          }
          o = f32x4{v[0], v[1], v[2], v[3]};
        }
        st4(a.odata.data + (size_t)idx * 4, o);
      }
      return;
    }
    const unsigned total = NC * (unsigned)H2 * (unsigned)W2;
    const unsigned stride = sb.gstride();
    for (unsigned idx = sb.gtid(); idx < total; idx += stride) {
      const int x2 = (int)(idx % (unsigned)W2);
      const unsigned t = idx / (unsigned)W2;
      const int y2 = (int)(t % (unsigned)H2);
      const unsigned nc = t / (unsigned)H2;
      const unsigned n = nc / C, c = nc - n * C;
      const float *in = a.idata.data + (int64_t)n * a.idata.strides[0] + (int64_t)c * a.idata.strides[1];
      float *out = a.odata.data + (int64_t)n * a.odata.strides[0] + (int64_t)c * a.odata.strides[1] +
                   (int64_t)y2 * a.odata.strides[2] + (int64_t)x2 * a.odata.strides[3];
      const int64_t sh = a.idata.strides[2], sw = a.idata.strides[3];
      if (same) {
        *out = in[y2 * sh + x2 * sw];
        continue;
      }
      const float h1r = src_index(a.rheight, y2, align);
      const int y1 = (int)h1r;
      const int y1p = (y1 < H1 - 1) ? 1 : 0;
      const float h1l = rn_sub(h1r, (float)y1), h0l = rn_sub(1.0f, h1l);
      const float w1r = src_index(a.rwidth, x2, align);
      const int x1 = (int)w1r;
      const int x1p = (x1 < W1 - 1) ? 1 : 0;
      const float w1l = rn_sub(w1r, (float)x1), w0l = rn_sub(1.0f, w1l);
      *out = blend(h0l, h1l, w0l, w1l, in[y1 * sh + x1 * sw], in[y1 * sh + (x1 + x1p) * sw],
                   in[(y1 + y1p) * sh + x1 * sw], in[(y1 + y1p) * sh + (x1 + x1p) * sw]);
    }
  }
};

// ----------------------------------------------------------------------------
// batch_norm_collect_statistics_kernel<InvStd,float,float,float,int>
// (argument list: scripts/data/ml-event.csv:14).  One plane (channel) per block
// iteration: per-thread Welford, Chan merges across the wavefront with DPP /
// permute shuffles, one barrier, then a second wave-level merge.
// ----------------------------------------------------------------------------
struct Welford {
  float n, mean, m2;
};

__device__ __forceinline__ Welford chan_merge(const Welford &a, const Welford &b) {
  Welford r;
  r.n = a.n + b.n;
  const float f = r.n > 0.0f ? b.n * __frcp_rn(r.n) : 0.0f;
  const float d = b.mean - a.mean;
  r.mean = a.mean + d * f;
  r.m2 = a.m2 + b.m2 + d * d * a.n * f;
  return r;
}

// Butterfly over the 64 lanes.  The first four steps stay inside a row of 16
// lanes and use DPP (quad permutes, half-row and row mirrors: the merge is
// symmetric, so a mirror is as good as an xor); the last two cross rows.
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ Welford dpp(const Welford &w) {
  return Welford{dpp<CTRL>(w.n), dpp<CTRL>(w.mean), dpp<CTRL>(w.m2)};
}
__device__ __forceinline__ Welford shfl_xor(const Welford &w, int m) {
  return Welford{__shfl_xor(w.n, m), __shfl_xor(w.mean, m), __shfl_xor(w.m2, m)};
}
__device__ __forceinline__ Welford wave_merge(Welford w) {
  w = chan_merge(w, dpp<0xB1>(w));   // quad_perm [1,0,3,2]
  w = chan_merge(w, dpp<0x4E>(w));   // quad_perm [2,3,0,1]
  w = chan_merge(w, dpp<0x141>(w));  // row_half_mirror
  w = chan_merge(w, dpp<0x140>(w));  // row_mirror
  w = chan_merge(w, shfl_xor(w, 16));
  w = chan_merge(w, shfl_xor(w, 32));
  return w;
}

struct BnStatsBody {
  static constexpr KernelId kId = K_BNSTATS;
  using Args = hf_bn_stats_args;
  static constexpr bool kBarriers = true;
  static constexpr bool kFlat = false;  // one plane per block: the block index is part of the work mapping
  static constexpr unsigned kLdsBytes = 16 * sizeof(Welford) + 16;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *lds, unsigned hint) {
    Welford *part = reinterpret_cast<Welford *>(lds);
    const int N = a.input.sizes[0], C = a.input.sizes[1], L = a.input.sizes[2];
    for (int plane = (int)sb.bid; plane < C; plane += (int)sb.nblocks) {
      Welford acc{0.0f, 0.0f, 0.0f};
      if (hint == HINT_BN_VEC4) {
        // stride[2] == 1, L % 4 == 0, 16-byte aligned rows: chunks of four.
        const unsigned lq = (unsigned)L >> 2;
        const unsigned chunks = (unsigned)N * lq;
        const float *base = a.input.data + (size_t)plane * a.input.strides[1];
        float k = 0.0f;
        // Welford of a chunk of four, then merge (4, m4, s4) into the running triple.
        auto merge4 = [&](const f32x4 v) {
          const float m4 = (v.x + v.y + v.z + v.w) * 0.25f;
          const float dx = v.x - m4, dy = v.y - m4, dz = v.z - m4, dw = v.w - m4;
          const float s4 = dx * dx + dy * dy + dz * dz + dw * dw;
          k += 1.0f;
          const float inv = __frcp_rn(k);  // 4 / (4k)
          const float d = m4 - acc.mean;
          acc.mean += d * inv;
          acc.m2 += s4 + d * d * (4.0f * (k - 1.0f)) * inv;
        };
        auto chunk = [&](unsigned ch) {
          const unsigned b = ch / lq, q = ch - b * lq;
          return ld4_stream(base + (size_t)b * a.input.strides[0] + (size_t)q * 4);
        };
#ifndef HF_BN_U
#define HF_BN_U 4
#endif
        unsigned ch = sb.tid;
        for (; ch + (HF_BN_U - 1) * sb.nthreads < chunks; ch += HF_BN_U * sb.nthreads) {  // loads in flight
          f32x4 v[HF_BN_U];
#pragma unroll
          for (int u = 0; u < HF_BN_U; u++) v[u] = chunk(ch + u * sb.nthreads);
#pragma unroll
          for (int u = 0; u < HF_BN_U; u++) merge4(v[u]);
        }
        for (; ch < chunks; ch += sb.nthreads) merge4(chunk(ch));
        acc.n = 4.0f * k;
      } else {
        const int total = N * L;
        for (int e = (int)sb.tid; e < total; e += (int)sb.nthreads) {
          const int b = e / L, x = e - b * L;
          const float v = a.input.data[(size_t)b * a.input.strides[0] + (size_t)plane * a.input.strides[1] +
                                       (size_t)x * a.input.strides[2]];
          const float d1 = v - acc.mean;
          acc.n += 1.0f;
          acc.mean += d1 * __frcp_rn(acc.n);
          acc.m2 += d1 * (v - acc.mean);
        }
      }
      acc = wave_merge(acc);
      if (sb.lane() == 0) part[sb.wave()] = acc;
      sb.sync();
      if (sb.wave() == 0) {
        Welford w = sb.lane() < sb.nwaves() ? part[sb.lane()] : Welford{0.0f, 0.0f, 0.0f};
        w = wave_merge(w);
        if (sb.lane() == 0) {
          a.save_mean.data[(size_t)plane * a.save_mean.strides[0]] = w.mean;
          a.save_transformed_var.data[(size_t)plane * a.save_transformed_var.strides[0]] =
              1.0f / sqrtf(w.m2 / w.n + a.epsilon);
        }
      }
      sb.sync();  // the partial slots are reused by the next plane
    }
  }
};

// ----------------------------------------------------------------------------
// kernelHistogram1D<..., SHARED, ...>  (argument list: scripts/data/ml-event.csv:2)
// LDS bins, zero -> barrier -> grid-stride atomic accumulation -> barrier ->
// flush to the fp32 counts with global atomics.
// ----------------------------------------------------------------------------
struct HistcBody {
  static constexpr KernelId kId = K_HISTC;
  using Args = hf_histc_args;
  static constexpr bool kBarriers = true;
  static constexpr bool kFlat = false;  // block-private LDS bins

  // LDS words the bins take: one spare word after the last bin collects the elements outside [min, max].
  static constexpr unsigned lds_bytes(unsigned nbins) { return (nbins + 1u) * 4u; }

  // bin = (int)((v - min) * nbins / (max - min)) in fp32, bin == nbins -> nbins - 1.
  // POW2: max - min is a power of two, so the correctly rounded division equals the
  // multiplication by its (exact) reciprocal and the IEEE division sequence is not needed.
  // LDS bins are counted without a branch: an element outside the range (or NaN) adds to the spare
  // word behind the last bin, so the four elements of a vector are four independent instruction
  // chains the compiler interleaves (with the range test as a branch a wave walks them one after
  // the other: 49 -> 43 us for 2^26 elements with eight wavefronts per CU, 41.7 -> 41.0 with twelve).
  template <bool POW2, bool GLOBAL>
  static __device__ __forceinline__ void count(unsigned *bins, float v, float lo, float hi, float scale_n, float range,
                                               float inv_lo, float inv_hi, int nbins) {
    // v >= lo && v <= hi as one comparison (a NaN fails it, as it fails the two): the median of (v, lo, hi) is v
    // itself exactly when v lies between them -- one lane mask per element instead of three
    const bool in = GLOBAL ? (v >= lo && v <= hi) : (__builtin_amdgcn_fmed3f(v, lo, hi) == v);
    if constexpr (GLOBAL) {
      if (!in) return;
    }
    const float t = (v - lo) * scale_n;
    int bin;
    if constexpr (POW2) {
      // scale_n already holds nbins / range: scaling by a power of two commutes with rounding.  Clamped as a
      // float (v == max lands on nbins: the original's `if (bin == nbins) bin -= 1`; nbins - 0.5 truncates to
      // nbins - 1 and is exact below 2^23 bins), which also keeps the conversion defined for elements out of range.
      bin = (int)__builtin_amdgcn_fmed3f(t, 0.0f, (float)nbins - 0.5f);
    } else {
      // (int)(t / range) without the division where that is safe.  t times two reciprocals that
      // bracket 1 / range by a relative 2^-21 brackets the correctly rounded quotient; when both
      // products truncate to the same integer so does the quotient.  Only a wavefront in which some
      // lane's products disagree does the IEEE division (its reciprocal sequence runs at a quarter
      // of the multiply rate); the empty asm keeps the compiler from hoisting it out of the branch.
      const float tc = in ? t : 0.0f;
      bin = (int)(tc * inv_lo);
      const bool unsure = bin != (int)(tc * inv_hi);
      if (__builtin_amdgcn_ballot_w64(unsure) != 0) {
        asm volatile("" ::: "memory");
        if (unsure) bin = (int)(tc / range);
      }
      bin = min(bin, nbins - 1);  // v == max lands in bin nbins
    }
    if ((HF_TAKEAPART & 4) && bin != -12345) return;  // the bin arithmetic stays, the atomic goes
    if constexpr (GLOBAL) unsafeAtomicAdd(reinterpret_cast<float *>(bins) + bin, 1.0f);
    else __hip_atomic_fetch_add(bins + (in ? bin : nbins), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }

  // The input stream: 16-byte non-temporal loads (values made up from the address in the loads-off timing build).
  static __device__ __forceinline__ f32x4 ldh(const float *p) {
    if (HF_TAKEAPART & 8) {
      const float f = __builtin_amdgcn_fractf((float)(((unsigned)(size_t)p >> 4) & 0xFFFFu) * 0.6180339887f);  // full-rate ops only
      return f32x4{f, __builtin_amdgcn_fractf(f + 0.3819f), __builtin_amdgcn_fractf(f + 0.7071f), __builtin_amdgcn_fractf(f + 0.1234f)};
    }
    return ld4_stream(p);
  }

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *lds, unsigned hint) {
    // The original picks shared or global memory for the bins by what fits; so does the host here.
    // (one global-memory instantiation, with the general bin formula: three copies of the loop
    // keep the body small enough to be inlined at every call site of the fused kernel)
    if (hint & HINT_HIST_GLOBAL) {
      body<false, true>(a, sb, lds, hint);
    } else if (hint & HINT_HIST_POW2) {
      body<true, false>(a, sb, lds, hint);
    } else {
      body<false, false>(a, sb, lds, hint);
    }
  }

  // GLOBAL: every element adds 1.0f to its bin of the (contiguous) output directly; the two
  // synchronisation points stay, so a partner that shares the hardware barrier still matches.
  template <bool POW2, bool GLOBAL, class SB>
  static __device__ __forceinline__ void body(const Args &a, SB &sb, unsigned char *lds, unsigned hint) {
    unsigned *bins = GLOBAL ? reinterpret_cast<unsigned *>(a.a.data) : reinterpret_cast<unsigned *>(lds);
    const int nbins = a.nbins;
    if constexpr (!GLOBAL)
      for (int i = (int)sb.tid; i <= nbins; i += (int)sb.nthreads) bins[i] = 0;
    sb.sync();
    const float lo = a.minvalue, hi = a.maxvalue, range = hi - lo;
    const float inv_range = 1.0f / range;
    // (v - lo) * nbins / range: with a power-of-two range the division is an exact scaling, folded into the factor
    const float fn = POW2 ? (float)nbins * inv_range : (float)nbins;
    const float inv_lo = inv_range * (1.0f - 0x1p-21f), inv_hi = inv_range * (1.0f + 0x1p-21f);
    const float *b = a.b.data;
    const int64_t total = a.total_elements;
    auto count4 = [&](const f32x4 v) __attribute__((always_inline)) {
      count<POW2, GLOBAL>(bins, v.x, lo, hi, fn, range, inv_lo, inv_hi, nbins);
      count<POW2, GLOBAL>(bins, v.y, lo, hi, fn, range, inv_lo, inv_hi, nbins);
      count<POW2, GLOBAL>(bins, v.z, lo, hi, fn, range, inv_lo, inv_hi, nbins);
      count<POW2, GLOBAL>(bins, v.w, lo, hi, fn, range, inv_lo, inv_hi, nbins);
      // four chains at a time: interleaving all sixteen of a batch would keep sixteen lane masks alive in scalar registers
      __builtin_amdgcn_sched_barrier(0);
    };
    if (hint & HINT_HIST_VEC4) {
      // `head` elements (0..3) precede the first 16-byte boundary; block 0 counts them and the
      // tail with scalar loads, everyone streams the aligned middle.
      const int64_t head = min((int64_t)((hint >> HINT_HIST_HEAD_SHIFT) & 3u), total);
      if (sb.bid == 0 && (int64_t)sb.tid < head) count<POW2, GLOBAL>(bins, b[sb.tid], lo, hi, fn, range, inv_lo, inv_hi, nbins);
      b += head;
      const int64_t rest = total - head;
      const int64_t n4 = rest >> 2;
      // The aligned middle goes in chunks of U KiB, one chunk per wavefront and trip: U loads of 16 bytes per
      // lane, each load instruction of the wave one contiguous KiB and the U of them consecutive, all in flight
      // before the dependent LDS atomics.  Chunk (k * waves + w) * blocks + b is wave w's k-th in block b, so at
      // any moment the chip reads one narrow window of the input (2^26 elements natively: 41 us against 43.7 us
      // with the same loads spread a grid stride apart).  Eight loads in flight with up to eight wavefronts,
      // four with more: about 48-64 KB per CU either way; beyond that the memory system gets slower.
      const unsigned wave = (unsigned)__builtin_amdgcn_readfirstlane((int)sb.wave());
      const unsigned lane = sb.lane(), nw = sb.nwaves();
      int64_t done4 = 0;  // vectors the chunks cover
      // (chunk numbers fit 32 bits: the host takes this path for inputs below 2^40 elements only)
      auto chunks = [&](auto unroll) __attribute__((always_inline)) {
        constexpr int U = decltype(unroll)::value;
        const unsigned nchunks = (unsigned)(n4 / (64 * U));
        const unsigned step = nw * sb.nblocks;
        for (unsigned c = wave * sb.nblocks + sb.bid; c < nchunks; c += step) {
          const float *p = b + ((size_t)c * (64 * U) + lane) * 4;
          f32x4 v[U];
#pragma unroll
          for (int u = 0; u < U; u++) v[u] = ldh(p + u * 256);
#pragma unroll
          for (int u = 0; u < U; u++) count4(v[u]);
        }
        done4 = (int64_t)nchunks * (64 * U);
      };
      if (sb.nthreads > 512) chunks(std::integral_constant<int, 4>());
      else chunks(std::integral_constant<int, 8>());
      // what no whole chunk covers (fewer than 64 * U vectors), then the up to three elements behind the last vector
      for (int64_t i = done4 + (int64_t)sb.gtid(); i < n4; i += (int64_t)sb.gstride()) count4(ldh(b + i * 4));
      if (sb.bid == 0)
        for (int64_t k = (n4 << 2) + sb.tid; k < rest; k += sb.nthreads)
          count<POW2, GLOBAL>(bins, b[k], lo, hi, fn, range, inv_lo, inv_hi, nbins);
    } else {
      const int64_t stride = (int64_t)sb.gstride();
      const int64_t bs = a.b.strides[0];
      for (int64_t i = (int64_t)sb.gtid(); i < total; i += stride)
        count<POW2, GLOBAL>(bins, b[i * bs], lo, hi, fn, range, inv_lo, inv_hi, nbins);
    }
    sb.sync();
    if constexpr (GLOBAL) return;
    const int64_t as = a.a.strides[0];
    for (int i = (int)sb.tid; i < nbins; i += (int)sb.nthreads) {
      const unsigned c = bins[i];
      if (c) unsafeAtomicAdd(a.a.data + i * as, (float)c);
    }
  }
};

}  // namespace hfuse
