// C-ABI of libhfuse_gfx950: configuration, plans, argument validation and the
// host launcher.  Compiled as HIP host code; no kernels live in this file.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>
#include <initializer_list>
#include <memory>
#include <mutex>
#include <new>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/hfuse_gfx950.h"
#include "device/crypto_bodies.h"
#include "device/dl_bodies.h"
#include "fusion_model.h"
#include "launch.h"

using namespace hfuse;

// ---------------------------------------------------------------- error state
namespace {

thread_local std::string g_error;

int fail(int code, const std::string &msg) {
  g_error = msg;
  return code;
}

int hip_fail(hipError_t e, const char *what) {
  return fail(HF_EHIP, std::string(what) + ": " + hipGetErrorString(e));
}

// No exception leaves the library: every entry point is a function-try-block that ends here.
// (What can throw is host allocation: strings and vectors of the YAML model, plan objects.)
int trap_exception() noexcept {
  try {
    throw;
  } catch (const std::bad_alloc &) {
    try { g_error.assign("out of memory"); } catch (...) {}   // fits the small-string buffer
    return HF_ENOMEM;
  } catch (const std::exception &e) {
    try { g_error.assign(e.what()); } catch (...) {}
    return HF_ENOMEM;
  } catch (...) {
    try { g_error.assign("unknown error"); } catch (...) {}
    return HF_ENOMEM;
  }
}

struct KernelName {
  const char *name;
  KernelId id;
};
const KernelName kNames[] = {
    {"im2col_kernel", K_IM2COL},
    {"MaxPoolForward", K_MAXPOOL},
    {"batch_norm_collect_statistics_kernel", K_BNSTATS},
    {"upsample_nearest2d_out_frame", K_UPSAMPLE_NEAREST},
    {"upsample_bilinear2d_out_frame", K_UPSAMPLE_BILINEAR},
    {"kernelHistogram1D", K_HISTC},
    {"ethash_search", K_ETHASH},
    // the reference clones ethash_search so each pair has its own symbol (configs/ethash_sha256.yaml:7)
    {"ethash_search2", K_ETHASH},
    {"ethash_search3", K_ETHASH},
    {"ethash_search4", K_ETHASH},
    {"sha256d_gpu_hash_shared", K_SHA256D},
    {"sia_blake2b_gpu_hash", K_SIA_BLAKE2B},
    {"blake2b_gpu_hash", K_BLAKE2B},
};

bool lookup_kernel(const std::string &name, KernelId &id) {
  for (auto &k : kNames)
    if (name == k.name) {
      id = k.id;
      return true;
    }
  return false;
}

// Barriers each built body executes (the YAML's HasBarriers is informational in the
// reference as well: BarrierRewriter rewrites whatever __syncthreads it finds).
bool body_has_barriers(KernelId id) { return id == K_BNSTATS || id == K_HISTC; }

// Bodies that walk one flat index range (K::kFlat): they can run on a partner's idle waves.
bool body_is_flat(KernelId id) { return id != K_BNSTATS && id != K_HISTC && id != K_ETHASH; }

// ------------------------------------------------ constants of the searches
// What the original kernels read from __constant__ symbols.  One process-wide set mirrors those
// symbols (hf_*_set_*); an hf_constants object is a caller-owned set that a plan can be bound to
// or a native launch can name, so that host threads working on different headers never share state.
struct SearchConstants {
  // ethash
  const void *dag = nullptr;
  uint32_t dag_items = 0;
  uint64_t eth_header[4] = {0, 0, 0, 0};
  uint64_t eth_target = 0;
  bool eth_set = false;
  // sha256d
  uint32_t sha_mid[8] = {0};
  uint32_t sha_tail[3] = {0};
  uint64_t sha_target = 0;
  bool sha_set = false;
  // blake2b headers
  uint64_t sia_m[10] = {0};
  bool sia_set = false;
  uint64_t b2_m[10] = {0};
  bool b2_set = false;
};
std::mutex g_const_mu;      // guards g_const only
SearchConstants g_const;    // the process-wide set

SearchConstants snapshot_process_constants() {
  std::lock_guard<std::mutex> lock(g_const_mu);
  return g_const;
}

uint32_t load_be32(const uint8_t *p) {
  return ((uint32_t)p[0] << 24) | ((uint32_t)p[1] << 16) | ((uint32_t)p[2] << 8) | p[3];
}
uint64_t load_le64(const uint8_t *p) {
  uint64_t v = 0;
  for (int i = 7; i >= 0; i--) v = (v << 8) | p[i];
  return v;
}
uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

// Host SHA-256 compression, used once per header for the midstate.
void host_sha256_compress(uint32_t st[8], const uint32_t blk[16]) {
  static const uint32_t K[64] = {
      0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5,
      0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
      0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
      0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
      0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
      0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
      0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3,
      0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
  uint32_t w[64];
  for (int i = 0; i < 16; i++) w[i] = blk[i];
  for (int i = 16; i < 64; i++)
    w[i] = w[i - 16] + (rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3)) + w[i - 7] +
           (rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10));
  uint32_t v[8];
  for (int i = 0; i < 8; i++) v[i] = st[i];
  for (int i = 0; i < 64; i++) {
    uint32_t t1 = v[7] + (rotr(v[4], 6) ^ rotr(v[4], 11) ^ rotr(v[4], 25)) + ((v[4] & v[5]) ^ (~v[4] & v[6])) + K[i] + w[i];
    uint32_t t2 = (rotr(v[0], 2) ^ rotr(v[0], 13) ^ rotr(v[0], 22)) + ((v[0] & v[1]) ^ (v[0] & v[2]) ^ (v[1] & v[2]));
    for (int j = 7; j > 0; j--) v[j] = v[j - 1];
    v[4] += t1;
    v[0] = t1 + t2;
  }
  for (int i = 0; i < 8; i++) st[i] += v[i];
}

// ------------------------------------------------------------ device facts
// Compute units of the current device, asked once (function-local static: thread-safe).
int cu_count() {
  static const int count = [] {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        prop.multiProcessorCount > 0)
      return prop.multiProcessorCount;
    return 256;  // MI355X
  }();
  return count;
}

// ------------------------------------------------------- argument validation
struct Prepared {
  KernelId id = K_COUNT;
  alignas(16) unsigned char blob[512];  // device-side argument struct
  unsigned hint = 0;
  unsigned lds = 0;
  bool exact_grid = false;  // the grid decides the amount of work (ethash)
  bool idx32 = false;       // the chosen path walks its work items with a 32-bit counter
  unsigned long long items = 0;  // work items of one pass at the chosen hint
};

static_assert(sizeof(hf_im2col_args) <= 512 && sizeof(hf_maxpool_args) <= 512 && sizeof(hf_bn_stats_args) <= 512 &&
                  sizeof(hf_upsample_nearest_args) <= 512 && sizeof(hf_histc_args) <= 512 &&
                  sizeof(hf_upsample_bilinear_args) <= 512 &&
                  sizeof(EthashDevArgs) <= 512 && sizeof(Sha256dDevArgs) <= 512 && sizeof(Blake2bDevArgs) <= 512,
              "argument blob too small");

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Every extent, stride and geometry value a caller passes is bounded before it is multiplied:
// one value below 2^31, products through checked multiplication, so no validator can overflow
// or divide by a wrapped zero whatever the argument struct holds.
constexpr int64_t kMaxExtent = (int64_t)1 << 31;
constexpr int64_t kMaxOffset = (int64_t)1 << 46;  // elements; far beyond 288 GB of fp32
bool extent_ok(int64_t v) { return v > 0 && v < kMaxExtent; }
bool pad_ok(int64_t v) { return v >= 0 && v < kMaxExtent; }
// out = product of the arguments, false on overflow of int64 or beyond kMaxOffset
bool product(int64_t &out, std::initializer_list<int64_t> factors) {
  out = 1;
  for (int64_t f : factors)
    if (f < 0 || __builtin_mul_overflow(out, f, &out) || out > kMaxOffset) return false;
  return true;
}

int prepare_im2col(const hf_im2col_args &a, Prepared &p) {
  if (!a.data_im || !a.data_col) return fail(HF_EINVAL, "im2col_kernel: null data pointer");
  if (a.n < 0 || a.n > kMaxOffset || !extent_ok(a.height) || !extent_ok(a.width) || !extent_ok(a.kernel_h) ||
      !extent_ok(a.kernel_w) || !extent_ok(a.stride_h) || !extent_ok(a.stride_w) || !extent_ok(a.dilation_h) ||
      !extent_ok(a.dilation_w) || !extent_ok(a.height_col) || !extent_ok(a.width_col) || !pad_ok(a.pad_h) ||
      !pad_ok(a.pad_w))
    return fail(HF_EINVAL, "im2col_kernel: non-positive or oversized geometry");
  const int64_t plane_col = a.height_col * a.width_col;  // both below 2^31
  if (a.n % plane_col != 0) return fail(HF_EINVAL, "im2col_kernel: n is not channels * height_col * width_col");
  const int64_t hc = (a.height + 2 * a.pad_h - (a.dilation_h * (a.kernel_h - 1) + 1)) / a.stride_h + 1;
  const int64_t wc = (a.width + 2 * a.pad_w - (a.dilation_w * (a.kernel_w - 1) + 1)) / a.stride_w + 1;
  if (hc != a.height_col || wc != a.width_col)
    return fail(HF_EINVAL, "im2col_kernel: height_col/width_col do not follow from the geometry");
  const int64_t channels = a.n / plane_col;
  int64_t in_elems, out_elems;
  if (!product(in_elems, {channels, a.height, a.width}) || !product(out_elems, {a.n, a.kernel_h, a.kernel_w}))
    return fail(HF_EINVAL, "im2col_kernel: tensor sizes overflow");
  std::memcpy(p.blob, &a, sizeof a);
  const bool fast = a.kernel_h == 3 && a.kernel_w == 3 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 1 &&
                    a.pad_w == 1 && a.dilation_h == 1 && a.dilation_w == 1 && a.width % 4 == 0 &&
                    aligned16(a.data_im) && aligned16(a.data_col) && out_elems < (int64_t)1 << 31;
  // 32-bit index arithmetic in the general loop: every element offset, and the window reach
  // (effective kernel + padding) times the row length, stays below 2^31
  const int64_t lim = (int64_t)1 << 31;
  const bool idx32 = in_elems < lim && out_elems < lim &&
                     (a.dilation_h * (a.kernel_h - 1) + 1 + a.pad_h + a.height) * a.width < lim &&
                     a.dilation_w * (a.kernel_w - 1) + 1 + a.pad_w + a.width < lim &&
                     a.height_col * a.stride_h < lim && a.width_col * a.stride_w < lim;
  p.hint = fast ? HINT_IM2COL_3X3_S1P1 : idx32 ? HINT_IDX32 : HINT_GENERIC;
  p.items = fast ? (unsigned long long)a.n / 4 : (unsigned long long)a.n;
  p.idx32 = p.hint != HINT_GENERIC;
  return HF_OK;
}

int prepare_maxpool(const hf_maxpool_args &a, Prepared &p) {
  if (!a.bottom_data || !a.top_data || !a.top_mask) return fail(HF_EINVAL, "MaxPoolForward: null data pointer");
  if (a.nthreads < 0 || a.num <= 0 || a.channels <= 0 || a.height <= 0 || a.width <= 0 || a.pooled_height <= 0 ||
      a.pooled_width <= 0 || a.kernel_h <= 0 || a.kernel_w <= 0 || a.stride_h <= 0 || a.stride_w <= 0 ||
      a.pad_h < 0 || a.pad_w < 0 || a.dilation_h <= 0 || a.dilation_w <= 0)
    return fail(HF_EINVAL, "MaxPoolForward: non-positive geometry");
  int64_t out_elems, in_elems;
  if (!product(out_elems, {a.num, a.channels, a.pooled_height, a.pooled_width}) || out_elems != (int64_t)a.nthreads)
    return fail(HF_EINVAL, "MaxPoolForward: nthreads is not num * channels * pooled_height * pooled_width");
  if (!product(in_elems, {a.num, a.channels, a.height, a.width}))
    return fail(HF_EINVAL, "MaxPoolForward: input size overflows");
  const int64_t eff_h = ((int64_t)a.kernel_h - 1) * a.dilation_h + 1, eff_w = ((int64_t)a.kernel_w - 1) * a.dilation_w + 1;
  if (eff_h >= kMaxExtent || eff_w >= kMaxExtent) return fail(HF_EINVAL, "MaxPoolForward: effective kernel size overflows");
  if ((int64_t)a.pad_h * 2 > eff_h || (int64_t)a.pad_w * 2 > eff_w)
    return fail(HF_EINVAL, "MaxPoolForward: pad should be at most half of the effective kernel size");
  if (((int64_t)a.pooled_height - 1) * a.stride_h - a.pad_h >= a.height ||
      ((int64_t)a.pooled_width - 1) * a.stride_w - a.pad_w >= a.width)
    return fail(HF_EINVAL, "MaxPoolForward: last window starts outside the input");
  std::memcpy(p.blob, &a, sizeof a);
  const bool common = a.stride_h == 2 && a.stride_w == 2 && a.dilation_h == 1 && a.dilation_w == 1 &&
                      a.width % 4 == 0 && (int64_t)a.pooled_width * 2 == a.width && a.pooled_width % 2 == 0 &&
                      aligned16(a.bottom_data) && aligned16(a.top_data) && aligned16(a.top_mask) &&
                      in_elems < (int64_t)1 << 31;
  p.hint = (in_elems < (int64_t)1 << 31 && out_elems < (int64_t)1 << 31) ? HINT_IDX32 : HINT_GENERIC;
  if (common && a.kernel_h == 3 && a.kernel_w == 3 && a.pad_h == 1 && a.pad_w == 1 &&
      a.pooled_height == (a.height + 2 - 3) / 2 + 1)
    p.hint = HINT_POOL_K3S2P1;
  if (common && a.kernel_h == 2 && a.kernel_w == 2 && a.pad_h == 0 && a.pad_w == 0 &&
      a.pooled_height == (a.height - 2) / 2 + 1)
    p.hint = HINT_POOL_K2S2P0;
  p.items = (p.hint == HINT_POOL_K3S2P1 || p.hint == HINT_POOL_K2S2P0) ? (unsigned long long)a.nthreads / 2
                                                                         : (unsigned long long)a.nthreads;
  p.idx32 = p.hint != HINT_GENERIC;
  return HF_OK;
}

int prepare_bn(const hf_bn_stats_args &a, Prepared &p) {
  const char *who = "batch_norm_collect_statistics_kernel: ";
  if (!a.input.data || !a.save_mean.data || !a.save_transformed_var.data)
    return fail(HF_EINVAL, std::string(who) + "null data pointer");
  if (a.input.sizes[0] <= 0 || a.input.sizes[1] <= 0 || a.input.sizes[2] <= 0)
    return fail(HF_EINVAL, std::string(who) + "empty input");
  if (a.save_mean.sizes[0] != a.input.sizes[1] || a.save_transformed_var.sizes[0] != a.input.sizes[1])
    return fail(HF_EINVAL, std::string(who) + "output length is not the channel count");
  // one plane's N * L elements are walked with 32-bit counters; the farthest element of the
  // (possibly strided) input and outputs must be addressable
  int64_t plane, reach = 0;
  if (!extent_ok(a.input.sizes[0]) || !extent_ok(a.input.sizes[1]) || !extent_ok(a.input.sizes[2]) ||
      !product(plane, {a.input.sizes[0], a.input.sizes[2]}) || plane >= kMaxExtent)
    return fail(HF_EUNSUPPORTED, std::string(who) + "planes of 2^31 elements or more are not built");
  for (int i = 0; i < 3; i++) {
    int64_t far;
    if (a.input.strides[i] < 0 || !product(far, {a.input.sizes[i] - 1, a.input.strides[i]}) ||
        __builtin_add_overflow(reach, far, &reach) || reach > kMaxOffset)
      return fail(HF_EINVAL, std::string(who) + "negative or oversized stride");
  }
  int64_t far;
  if (!product(far, {a.input.sizes[1] - 1, a.save_mean.strides[0]}) ||
      !product(far, {a.input.sizes[1] - 1, a.save_transformed_var.strides[0]}))
    return fail(HF_EINVAL, std::string(who) + "negative or oversized output stride");
  std::memcpy(p.blob, &a, sizeof a);
  const bool fast = a.input.strides[2] == 1 && a.input.sizes[2] % 4 == 0 && a.input.strides[0] % 4 == 0 &&
                    a.input.strides[1] % 4 == 0 && aligned16(a.input.data);
  p.hint = fast ? HINT_BN_VEC4 : HINT_GENERIC;
  p.lds = BnStatsBody::kLdsBytes;
  p.items = (unsigned long long)a.input.sizes[1];  // planes
  return HF_OK;
}

int prepare_upsample(const hf_upsample_nearest_args &a, Prepared &p) {
  if (!a.idata || !a.odata) return fail(HF_EINVAL, "upsample_nearest2d_out_frame: null data pointer");
  if (a.nc == 0 || a.height1 == 0 || a.width1 == 0 || a.height2 == 0 || a.width2 == 0)
    return fail(HF_EINVAL, "upsample_nearest2d_out_frame: empty tensor");
  if (!(a.height_scale > 0.0f) || !(a.width_scale > 0.0f))
    return fail(HF_EINVAL, "upsample_nearest2d_out_frame: scale must be positive");
  int64_t in_elems, out_elems;
  if (a.nc >= (size_t)kMaxExtent || a.height1 >= (size_t)kMaxExtent || a.width1 >= (size_t)kMaxExtent ||
      a.height2 >= (size_t)kMaxExtent || a.width2 >= (size_t)kMaxExtent ||
      !product(in_elems, {(int64_t)a.nc, (int64_t)a.height1, (int64_t)a.width1}) ||
      !product(out_elems, {(int64_t)a.nc, (int64_t)a.height2, (int64_t)a.width2}))
    return fail(HF_EINVAL, "upsample_nearest2d_out_frame: tensor sizes overflow");
  std::memcpy(p.blob, &a, sizeof a);
  const bool fast = a.height2 == 2 * a.height1 && a.width2 == 2 * a.width1 && a.height_scale == 0.5f &&
                    a.width_scale == 0.5f && a.width1 % 2 == 0 && aligned16(a.idata) && aligned16(a.odata) &&
                    out_elems < (int64_t)1 << 32;
  p.hint = fast ? HINT_UP_2X : (in_elems < (int64_t)1 << 31 && out_elems < (int64_t)1 << 31) ? HINT_IDX32 : HINT_GENERIC;
  p.items = fast ? (unsigned long long)in_elems / 2 : (unsigned long long)out_elems;
  p.idx32 = p.hint != HINT_GENERIC;
  return HF_OK;
}

int prepare_bilinear(const hf_upsample_bilinear_args &a, Prepared &p) {
  const char *who = "upsample_bilinear2d_out_frame: ";
  if (!a.idata.data || !a.odata.data) return fail(HF_EINVAL, std::string(who) + "null data pointer");
  for (int i = 0; i < 4; i++)
    if (a.idata.sizes[i] <= 0 || a.odata.sizes[i] <= 0) return fail(HF_EINVAL, std::string(who) + "empty tensor");
  if (a.idata.sizes[0] != a.odata.sizes[0] || a.idata.sizes[1] != a.odata.sizes[1])
    return fail(HF_EINVAL, std::string(who) + "batch / channel counts of input and output differ");
  int64_t total, in_total, hw;
  if (!product(total, {a.odata.sizes[0], a.odata.sizes[1], a.odata.sizes[2], a.odata.sizes[3]}) ||
      !product(in_total, {a.idata.sizes[0], a.idata.sizes[1], a.idata.sizes[2], a.idata.sizes[3]}) ||
      total >= (int64_t)1 << 32 || in_total >= (int64_t)1 << 32)
    return fail(HF_EUNSUPPORTED, std::string(who) + "tensors of 2^32 elements or more are not built");
  if (!product(hw, {a.odata.sizes[2], a.odata.sizes[3]}) || (int64_t)a.n != hw)
    return fail(HF_EINVAL, std::string(who) + "n is not height2 * width2");
  if (!(a.rheight >= 0.0f) || !(a.rwidth >= 0.0f) || !std::isfinite(a.rheight) || !std::isfinite(a.rwidth))
    return fail(HF_EINVAL, std::string(who) + "scales must be finite and not negative");
  // The kernel reads input row (int)src and column (int)src of every output pixel without a clamp,
  // as the original does: the source index of the last output row / column, evaluated in the
  // kernel's own fp32 steps (it grows with the destination index), must lie inside the input.
  auto last_source = [&](float scale, int64_t out_size) {
    const volatile float dst = (float)(out_size - 1);
    if (a.align_corners) {
      const volatile float s = scale * dst;
      return (double)s;
    }
    const volatile float t0 = dst + 0.5f;
    const volatile float t1 = scale * t0;
    const volatile float t2 = t1 - 0.5f;
    return (double)(t2 < 0.0f ? 0.0f : t2);
  };
  const bool same_size = a.idata.sizes[2] == a.odata.sizes[2] && a.idata.sizes[3] == a.odata.sizes[3];  // a plain copy
  if (!same_size && (last_source(a.rheight, a.odata.sizes[2]) >= (double)a.idata.sizes[2] ||
                     last_source(a.rwidth, a.odata.sizes[3]) >= (double)a.idata.sizes[3]))
    return fail(HF_EINVAL, std::string(who) + "scale maps the last output row or column beyond the input");
  for (const hf_accessor4 *t : {&a.idata, &a.odata}) {
    int64_t reach = 0;
    for (int i = 0; i < 4; i++) {
      int64_t far;
      if (t->strides[i] < 0 || !product(far, {t->sizes[i] - 1, t->strides[i]}) ||
          __builtin_add_overflow(reach, far, &reach) || reach > kMaxOffset)
        return fail(HF_EINVAL, std::string(who) + "negative or oversized stride");
    }
  }
  std::memcpy(p.blob, &a, sizeof a);
  auto contiguous = [](const hf_accessor4 &t) {
    return t.strides[3] == 1 && t.strides[2] == t.sizes[3] && t.strides[1] == t.sizes[2] * t.sizes[3] &&
           t.strides[0] == t.sizes[1] * t.sizes[2] * t.sizes[3];
  };
  const bool fast = contiguous(a.idata) && contiguous(a.odata) && a.odata.sizes[3] % 4 == 0 && aligned16(a.odata.data) &&
                    (a.idata.sizes[2] != a.odata.sizes[2] || a.idata.sizes[3] != a.odata.sizes[3] || aligned16(a.idata.data));
  // exact 2x without align_corners: 0.5 * (dst + 0.5) - 0.5 is exact below 2^22 output columns / rows
  const bool twice = fast && !a.align_corners && a.rheight == 0.5f && a.rwidth == 0.5f &&
                     a.odata.sizes[2] == 2 * a.idata.sizes[2] && a.odata.sizes[3] == 2 * a.idata.sizes[3] &&
                     a.idata.sizes[3] % 2 == 0 && ((uintptr_t)a.idata.data & 7) == 0 &&
                     a.odata.sizes[2] < (1 << 22) && a.odata.sizes[3] < (1 << 22);
  // the same work-item shape with align_corners: there src = dst * (in - 1) / (out - 1) drifts from dst / 2 - 1/2 to
  // dst / 2 across the image, and as long as its integer part is (dst - 1) >> 1 (0 for dst = 0), as it is without
  // align_corners, every output blends the same rows and columns of its work item's window and only the weights differ.
  // Checked here with the kernel's own fp32 steps, one pass over the output's width and height (rounding breaks the
  // rule near the far edge of images a few thousand pixels wide; those take the gathered path).
  bool twice_align = fast && a.align_corners && a.odata.sizes[2] == 2 * a.idata.sizes[2] &&
                     a.odata.sizes[3] == 2 * a.idata.sizes[3] && a.idata.sizes[3] % 2 == 0 &&
                     ((uintptr_t)a.idata.data & 7) == 0 && a.odata.sizes[2] <= (1 << 16) && a.odata.sizes[3] <= (1 << 16);
  if (twice_align) {
    auto fixed_sources = [](float scale, int64_t out_size) {
      for (int64_t dst = 0; dst < out_size; dst++) {
        const volatile float src = scale * (float)dst;
        if ((int64_t)(float)src != (dst ? (dst - 1) >> 1 : 0)) return false;
      }
      return true;
    };
    twice_align = fixed_sources(a.rwidth, a.odata.sizes[3]) && fixed_sources(a.rheight, a.odata.sizes[2]);
  }
  p.hint = twice ? HINT_BILINEAR_2X : twice_align ? HINT_BILINEAR_2X_ALIGN : fast ? HINT_BILINEAR_VEC4 : HINT_GENERIC;
  // exact 2x: one work item per two input rows and two input columns
  const unsigned long long row_pairs = ((unsigned long long)a.idata.sizes[2] + 1) / 2;
  p.items = (twice || twice_align) ? (unsigned long long)a.idata.sizes[0] * a.idata.sizes[1] * row_pairs * (a.idata.sizes[3] / 2) : fast ? (unsigned long long)total / 4 : (unsigned long long)total;
  p.idx32 = true;  // every bilinear path counts in 32 bits (tensors below 2^32 elements)
  return HF_OK;
}

int prepare_histc(const hf_histc_args &a, Prepared &p) {
  if (!a.a.data || !a.b.data) return fail(HF_EINVAL, "kernelHistogram1D: null data pointer");
  if (a.nbins <= 0) return fail(HF_EINVAL, "kernelHistogram1D: bins must be > 0");
  if (!(a.minvalue < a.maxvalue)) return fail(HF_EINVAL, "kernelHistogram1D: max must be larger than min");
  if (a.total_elements < 0 || a.total_elements > kMaxOffset)
    return fail(HF_EINVAL, "kernelHistogram1D: negative or oversized element count");
  if (a.a.dims != 1 || a.b.dims != 1)
    return fail(HF_EUNSUPPORTED, "kernelHistogram1D: only 1-D tensors are built");
  if (a.a.sizes[0] != a.nbins) return fail(HF_EINVAL, "kernelHistogram1D: output length is not nbins");
  if (a.b.sizes[0] != a.total_elements) return fail(HF_EINVAL, "kernelHistogram1D: totalElements is not the input length");
  if (a.a.strides[0] != 1) return fail(HF_EUNSUPPORTED, "kernelHistogram1D: output must be contiguous");
  const bool global_bins = a.nbins > 15360;  // beyond the LDS budget the bins are counted in global memory
  int64_t far;
  if (a.b.strides[0] < 0 || !product(far, {a.total_elements > 0 ? a.total_elements - 1 : 0, a.b.strides[0]}))
    return fail(HF_EINVAL, "kernelHistogram1D: negative or oversized input stride");
  std::memcpy(p.blob, &a, sizeof a);
  // contiguous input: 16-byte loads from the first aligned element on; the up to three elements
  // before it (HINT_HIST_HEAD bits) and the tail go through scalar loads
  // (the vector path numbers its 1-2 KiB chunks in 32 bits: inputs below 2^40 elements, far more than HBM holds)
  const bool fast = a.b.strides[0] == 1 && (reinterpret_cast<uintptr_t>(a.b.data) & 3u) == 0 &&
                    a.total_elements < ((int64_t)1 << 40);
  const unsigned head = fast ? (unsigned)(((16u - (reinterpret_cast<uintptr_t>(a.b.data) & 15u)) & 15u) >> 2) : 0u;
  // max - min a power of two (exact reciprocal): the division in the bin formula can be a multiply
  int exp2 = 0;
  const float range = a.maxvalue - a.minvalue;
  const bool pow2 = std::frexp(range, &exp2) == 0.5f && exp2 > -100 && exp2 < 100;
  p.hint = (fast ? HINT_HIST_VEC4 : HINT_GENERIC) | (pow2 ? HINT_HIST_POW2 : 0) | (head << HINT_HIST_HEAD_SHIFT) |
           (global_bins ? HINT_HIST_GLOBAL : 0);
  p.lds = global_bins ? 0u : HistcBody::lds_bytes((unsigned)a.nbins);
  p.items = fast ? (unsigned long long)(a.total_elements + 3) / 4 : (unsigned long long)a.total_elements;
  return HF_OK;
}

int prepare_ethash(const hf_ethash_args &a, const SearchConstants &c, Prepared &p) {
  if (!a.g_output) return fail(HF_EINVAL, "ethash_search: null result pointer");
  if (!c.eth_set) return fail(HF_EINVAL, "ethash_search: hf_ethash_set_constants has not been called");
  EthashDevArgs d;
  d.out = a.g_output;
  d.start_nonce = a.start_nonce;
  d.dag = static_cast<const u32x4 *>(c.dag);
  d.n_items = c.dag_items;
  d.pow2_mask = (d.n_items & (d.n_items - 1)) == 0 ? d.n_items - 1 : 0;
  d.target = c.eth_target;
  std::memcpy(d.header, c.eth_header, sizeof d.header);
  std::memcpy(p.blob, &d, sizeof d);
  p.exact_grid = true;
  return HF_OK;
}

int prepare_sha256d(const hf_sha256d_args &a, const SearchConstants &c, Prepared &p) {
  if (!a.res_nonces) return fail(HF_EINVAL, "sha256d_gpu_hash_shared: null result pointer");
  if (!c.sha_set) return fail(HF_EINVAL, "sha256d_gpu_hash_shared: hf_sha256d_set_block has not been called");
  Sha256dDevArgs d;
  d.threads = a.threads;
  d.start_nonce = a.start_nonce;
  d.out = reinterpret_cast<hf_search_results *>(a.res_nonces);
  std::memcpy(d.midstate, c.sha_mid, sizeof d.midstate);
  std::memcpy(d.tail, c.sha_tail, sizeof d.tail);
  d.pad = 0;
  d.target64 = c.sha_target;
  std::memcpy(p.blob, &d, sizeof d);
  p.items = a.threads;
  return HF_OK;
}

int prepare_blake2b(const hf_blake2b_args &a, bool sia, const SearchConstants &c, Prepared &p) {
  const char *who = sia ? "sia_blake2b_gpu_hash" : "blake2b_gpu_hash";
  if (!a.res_nonce) return fail(HF_EINVAL, std::string(who) + ": null result pointer");
  if (!(sia ? c.sia_set : c.b2_set))
    return fail(HF_EINVAL, std::string(who) + ": the header block has not been set");
  Blake2bDevArgs d;
  d.threads = a.threads;
  d.start_nonce = a.start_nonce;
  d.out = reinterpret_cast<hf_search_results *>(a.res_nonce);
  d.target64 = ((uint64_t)a.target2[1] << 32) | a.target2[0];
  std::memcpy(d.m, sia ? c.sia_m : c.b2_m, sizeof d.m);
  std::memcpy(p.blob, &d, sizeof d);
  p.items = a.threads;
  return HF_OK;
}

// `consts`: the constants a search kernel is launched with; null = the process-wide set as it is now.
int prepare(KernelId id, const void *args, Prepared &p, const SearchConstants *consts = nullptr) {
  if (!args) return fail(HF_EINVAL, "null argument list");
  p = Prepared();
  p.id = id;
  SearchConstants process;
  if (is_crypto(id) && !consts) {
    process = snapshot_process_constants();
    consts = &process;
  }
  switch (id) {
    case K_IM2COL: return prepare_im2col(*static_cast<const hf_im2col_args *>(args), p);
    case K_MAXPOOL: return prepare_maxpool(*static_cast<const hf_maxpool_args *>(args), p);
    case K_BNSTATS: return prepare_bn(*static_cast<const hf_bn_stats_args *>(args), p);
    case K_UPSAMPLE_NEAREST: return prepare_upsample(*static_cast<const hf_upsample_nearest_args *>(args), p);
    case K_HISTC: return prepare_histc(*static_cast<const hf_histc_args *>(args), p);
    case K_UPSAMPLE_BILINEAR: return prepare_bilinear(*static_cast<const hf_upsample_bilinear_args *>(args), p);
    case K_ETHASH: return prepare_ethash(*static_cast<const hf_ethash_args *>(args), *consts, p);
    case K_SHA256D: return prepare_sha256d(*static_cast<const hf_sha256d_args *>(args), *consts, p);
    case K_SIA_BLAKE2B: return prepare_blake2b(*static_cast<const hf_blake2b_args *>(args), true, *consts, p);
    case K_BLAKE2B: return prepare_blake2b(*static_cast<const hf_blake2b_args *>(args), false, *consts, p);
    default: return fail(HF_ENOTFOUND, "unknown kernel id");
  }
}

// Blocks one pass of `p` wants when it owns `threads` threads per block.
unsigned long long wanted_blocks(const Prepared &p, unsigned threads) {
  if (p.id == K_BNSTATS) return p.items;
  return (p.items + threads - 1) / threads;
}

// Default grid of one kernel inside a block of `block_threads` threads: enough workgroups
// to fill every CU sixteen times over, never more than the work asks for.  The streaming
// bodies stride over the rest; a larger grid evens out their tail.  The histogram is the
// exception: every block flushes its LDS bins with one global atomic per bin, and its input
// stream runs fastest with about twelve wavefronts per CU (four 16-byte loads in flight per lane:
// 48 KB per CU; twice that is slower), so it gets as many blocks per CU as make up twelve
// wavefronts, within what fits next to each other.
unsigned default_grid(const Prepared &p, unsigned own_threads, unsigned block_threads) {
  const unsigned long long want = wanted_blocks(p, own_threads);
  const unsigned per_cu = std::max(1u, 2048u / block_threads);
  const unsigned hist_per_cu = std::min(per_cu, std::max(1u, 768u / own_threads));
  const unsigned long long cap = p.id == K_HISTC ? (unsigned long long)cu_count() * hist_per_cu
                                                 : (unsigned long long)cu_count() * per_cu * 16ull;
  return (unsigned)std::min(std::max(want, 1ull), cap);
}

constexpr unsigned kDefaultEthashGrid = 8192;  // the authors' launches: scripts/data/ethminer_event.csv

// A body that counts its work items in 32 bits steps its index past the last item once before the
// loop test ends it (twice in the exact-2x upsampling path, which takes two items per trip): with
// `threads` threads striding over `p.items` items the counter reaches items + 2 * threads at most,
// which must not wrap.  (The searches and the 64-bit paths count in 64 bits.)
bool counter_fits(const Prepared &p, unsigned long long threads) {
  return !p.idx32 || p.items + 2ull * threads <= (1ull << 32);
}
const char *const kCounterMsg =
    "work items + 2 * grid_blocks * block threads must fit 32 bits (this path indexes its work items with a 32-bit counter)";

int do_launch_native(KernelId id, const Prepared &p, int grid_blocks, unsigned block, hipStream_t stream) {
  if (block == 0 || block % kWave != 0 || block > (is_crypto(id) ? 512u : kMaxBlock))
    return fail(HF_EINVAL, "block size must be a multiple of 64 within the kernel's launch bound");
  unsigned grid;
  if (grid_blocks > 0) grid = (unsigned)grid_blocks;
  else if (p.exact_grid) grid = kDefaultEthashGrid;
  else grid = default_grid(p, block, block);
  if (!p.exact_grid && p.items == 0) return HF_OK;  // nothing to do
  if ((unsigned long long)grid * block > 0xFFFFFFFFull)
    return fail(HF_EINVAL, "grid_blocks * block threads must fit 32 bits (the bodies index work items with 32-bit counters)");
  if (!counter_fits(p, (unsigned long long)grid * block)) return fail(HF_EINVAL, kCounterMsg);
  hipError_t e = is_crypto(id) ? launch_native_crypto(id, p.blob, p.hint, grid, block, p.lds, stream)
                               : launch_native_dl(id, p.blob, p.hint, grid, block, p.lds, stream);
  if (e != hipSuccess) return hip_fail(e, "native launch");
  return HF_OK;
}

}  // namespace

// ------------------------------------------------------------------ opaque types
struct hf_config {
  Config cfg;
};

struct hf_constants {
  SearchConstants c;
};

struct hf_plan {
  bool has_consts = false;             // hf_plan_bind_constants: launches of this plan use `consts`
  SearchConstants consts;
  int n = 2;                           // kernels of the fusion: 2, or 3 for the reference's three-kernel lists
  KernelRow rows[kMaxFuse];
  KernelId ids[kMaxFuse] = {K_COUNT, K_COUNT, K_COUNT};
  const Preset *preset;
  Partition part;
  int barrier_mode;
  unsigned grid_override[2] = {0, 0};  // hf_plan_set_grids
  bool lending = true;                 // hf_plan_set_lending
  int bounded = -1;                    // hf_plan_set_launch_bound: 0 / 1, -1 = by the preset
  int bound_waves = 0;                 // hf_plan_set_launch_waves: waves per SIMD of the bounded build, 0 = by the formula
};

namespace {
// Waves per SIMD the occupancy formula of the reference's printer asks for with this part's constants:
// B = min_k(regfile / Reg_k / threads_k) blocks per CU, capped by the resident threads
// (lib/KernelFuser/KernelPrinter.cpp:44-66), times the block's waves, spread over four SIMDs.
// Rounded up: B blocks of T threads are B * T / 64 waves, and all of them have to fit (5.5 waves per SIMD need 6).
int formula_waves(const hf_plan *plan) {
  const unsigned long long waves = (unsigned long long)plan->part.bound_blocks * (plan->part.launch_threads / kWave);
  const unsigned long long w = (waves + 3) / 4;
  return (int)std::min<unsigned long long>(std::max<unsigned long long>(w, 1), (unsigned long long)kBoundedWaves);
}

// The build a launch of this plan runs: 0 = plain, otherwise the wave bound of a register-bounded build.
// The launch-bound presets ask for a bounded build when the formula wants more waves per SIMD than the
// plain build's launch bound of 1024 threads already guarantees (four).
int plan_build_waves(const hf_plan *plan) {
  if (plan->n != 2) return plan->preset->launch_bound ? kBoundedWaves : 0;  // three-kernel fusions: plain, or bounded for 8 waves
  if (!plan->preset->base_line && plan->barrier_mode == HF_BARRIER_BLOCKIDX) return 0;  // no bounded build
  const int formula = formula_waves(plan);
  const bool want = plan->bounded >= 0 ? plan->bounded != 0 : plan->preset->launch_bound && formula > 4;
  if (!want) return 0;
  const int built = built_bound_waves(plan->ids[0], plan->ids[1], plan->bound_waves ? plan->bound_waves : formula);
  return plan->preset->base_line ? kBoundedWaves : built;   // the vertical baseline has the 8-wave build only
}

// The three-kernel lists that are instantiated, in the order they are built in (the reference's configs/
// im2col_maxpool_norm.yaml, maxpool_summary_norm.yaml, crypt_four.yaml).  A list that names the same three
// kernels in another order runs the same instantiation: perm[c] = position in the list of built kernel c.
constexpr KernelId kBuiltTriples[3][3] = {{K_IM2COL, K_MAXPOOL, K_BNSTATS}, {K_MAXPOOL, K_HISTC, K_BNSTATS},
                                          {K_BLAKE2B, K_SHA256D, K_ETHASH}};
bool built_triple(const KernelId ids[3], int perm[3]) {
  for (const auto &t : kBuiltTriples) {
    bool all = true;
    for (int c = 0; c < 3 && all; c++) {
      perm[c] = -1;
      for (int i = 0; i < 3; i++)
        if (ids[i] == t[c]) perm[c] = i;
      all = perm[c] >= 0;
    }
    if (all) return true;
  }
  return false;
}

// The reference's Context partitions a block among any number of kernels (include/KernelFusion.h:45-80);
// its lists hold pairs and three-kernel entries (configs/crypt_four.yaml), which is what is built here.
int unsupported_size(const FusionRow &f) {
  return fail(HF_EUNSUPPORTED, "fusion '" + f.file + "' names " + std::to_string(f.kernels.size()) +
                                   " kernels: fused kernels are built for two or three");
}
// Calls that shape a pair's launch (block shape, per-half grids, lending, barrier design, bounded builds).
int pair_call_only(const hf_plan *plan) {
  if (plan->n != 2) return fail(HF_EINVAL, "this call is for pairs; the plan fuses three kernels (see the *_n calls)");
  return HF_OK;
}
}  // namespace

// ------------------------------------------------------------------ C-ABI
extern "C" {

HF_API const char *hf_last_error(void) { return g_error.c_str(); }
HF_API int hf_version(void) { return 300; }

HF_API int hf_config_load_text(const char *fusion_yaml, const char *kernels_yaml, hf_config **out) try {
  if (!out) return fail(HF_EINVAL, "null output pointer");
  *out = nullptr;
  if (!kernels_yaml) return fail(HF_EINVAL, "null kernel table");
  auto *c = new hf_config();
  std::string err;
  if (!parse_config(fusion_yaml, kernels_yaml, c->cfg, err)) {
    delete c;
    return fail(HF_EPARSE, err);
  }
  *out = c;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_config_load_files(const char *fusion_path, const char *kernels_path, hf_config **out) try {
  if (!out) return fail(HF_EINVAL, "null output pointer");
  *out = nullptr;
  if (!kernels_path) return fail(HF_EINVAL, "null kernel table path");
  auto slurp = [](const char *path, std::string &dst) {
    std::ifstream in(path, std::ios::binary);
    if (!in) return false;
    std::ostringstream ss;
    ss << in.rdbuf();
    dst = ss.str();
    return true;
  };
  std::string f, k;
  if (!slurp(kernels_path, k)) return fail(HF_EIO, std::string("failed to read configs: ") + kernels_path);
  if (fusion_path && !slurp(fusion_path, f)) return fail(HF_EIO, std::string("failed to read configs: ") + fusion_path);
  return hf_config_load_text(fusion_path ? f.c_str() : nullptr, k.c_str(), out);
} catch (...) {
  return trap_exception();
}

HF_API void hf_config_free(hf_config *cfg) { delete cfg; }

HF_API int hf_config_num_fusions(const hf_config *cfg) { return cfg ? (int)cfg->cfg.fusions.size() : fail(HF_EINVAL, "null config"); }
HF_API int hf_config_num_kernels(const hf_config *cfg) { return cfg ? (int)cfg->cfg.rows.size() : fail(HF_EINVAL, "null config"); }

HF_API int hf_config_fusion(const hf_config *cfg, int i, const char **file, const char **k1, const char **k2) try {
  if (!cfg) return fail(HF_EINVAL, "null config");
  if (i < 0 || i >= (int)cfg->cfg.fusions.size()) return fail(HF_EINVAL, "fusion index out of range");
  const FusionRow &f = cfg->cfg.fusions[i];
  if (file) *file = f.file.c_str();
  if (k1) *k1 = f.kernels[0].c_str();
  if (k2) *k2 = f.kernels.size() > 1 ? f.kernels[1].c_str() : "";
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_config_fusion_size(const hf_config *cfg, int i) {
  if (!cfg) return fail(HF_EINVAL, "null config");
  if (i < 0 || i >= (int)cfg->cfg.fusions.size()) return fail(HF_EINVAL, "fusion index out of range");
  return (int)cfg->cfg.fusions[i].kernels.size();
}

HF_API int hf_config_fusion_kernel(const hf_config *cfg, int i, int k, const char **name) {
  if (!cfg || !name) return fail(HF_EINVAL, "null argument");
  if (i < 0 || i >= (int)cfg->cfg.fusions.size()) return fail(HF_EINVAL, "fusion index out of range");
  const FusionRow &f = cfg->cfg.fusions[i];
  if (k < 0 || k >= (int)f.kernels.size()) return fail(HF_EINVAL, "kernel index out of range");
  *name = f.kernels[k].c_str();
  return HF_OK;
}

HF_API int hf_config_kernel(const hf_config *cfg, const char *name, hf_kernel_info *out) try {
  if (!cfg || !name || !out) return fail(HF_EINVAL, "null argument");
  const KernelRow *r = cfg->cfg.find(name);
  if (!r) return fail(HF_ENOTFOUND, std::string("kernel '") + name + "' is not in the kernel table");
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->kernel_name, r->name.c_str(), sizeof out->kernel_name - 1);
  out->has_barriers = r->has_barriers;
  out->block_dim = {r->block_dim.x, r->block_dim.y, r->block_dim.z};
  out->reg = r->reg;
  out->exec_time = r->exec_time;
  out->native_threads = r->native_block();
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_num_splits(const hf_config *cfg, int fusion_index) try {
  if (!cfg) return fail(HF_EINVAL, "null config");
  if (fusion_index < 0 || fusion_index >= (int)cfg->cfg.fusions.size()) return fail(HF_EINVAL, "fusion index out of range");
  const FusionRow &f = cfg->cfg.fusions[fusion_index];
  if (f.kernels.size() != 2 && f.kernels.size() != 3) return unsupported_size(f);
  // (the driver's split loop varies the first two kernels only, main.cpp:219-225)
  return num_splits(*cfg->cfg.find(f.kernels[0]), *cfg->cfg.find(f.kernels[1]));
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_create(const hf_config *cfg, int fusion_index, const char *preset, int split_idx, int split_threads,
                          hf_plan **out) try {
  if (!out) return fail(HF_EINVAL, "null output pointer");
  *out = nullptr;
  if (!cfg || !preset) return fail(HF_EINVAL, "null argument");
  if (fusion_index < 0 || fusion_index >= (int)cfg->cfg.fusions.size()) return fail(HF_EINVAL, "fusion index out of range");
  const FusionRow &f = cfg->cfg.fusions[fusion_index];
  // "shipped": the preset the entry names with its `Preset:` key, the thread partition without one
  const std::string entry_preset = f.preset.empty() ? "hfuse" : f.preset;
  const std::string asked = std::strcmp(preset, "shipped") == 0 ? entry_preset : std::string(preset);
  const Preset *p = find_preset(asked);
  if (!p) return fail(HF_ENOTFOUND, std::string("unknown preset '") + preset + "' (vfuse_lb, vfuse, hfuse, hfuse_lb, or shipped)");
  if (split_threads > 0 && split_threads % (int)kWave != 0)
    return fail(HF_EINVAL, "split_threads must be a multiple of the 64-lane wavefront");
  if (f.kernels.size() != 2 && f.kernels.size() != 3) return unsupported_size(f);
  std::unique_ptr<hf_plan> plan(new hf_plan());  // freed on every early return and on an exception
  plan->preset = p;
  plan->n = (int)f.kernels.size();
  for (int i = 0; i < plan->n; i++) {
    plan->rows[i] = *cfg->cfg.find(f.kernels[i]);
    if (!lookup_kernel(plan->rows[i].name, plan->ids[i]))
      return fail(HF_ENOTFOUND, "kernel '" + plan->rows[i].name + "' has no gfx950 implementation in this library");
  }
  if (plan->n == 3) {
    // A three-kernel list: the Context's partition among three, no tuned keys, no lending, every
    // synchronising body on its own LDS arrival counter.
    if (is_crypto(plan->ids[0]) != is_crypto(plan->ids[1]) || is_crypto(plan->ids[0]) != is_crypto(plan->ids[2])) {
      return fail(HF_EUNSUPPORTED, "fusions mixing tensor kernels with search kernels are not built");
    }
    if (split_threads > 0) {
      return fail(HF_EINVAL, "split_threads shapes a pair; give a three-kernel plan its block with hf_plan_set_block_n");
    }
    int perm[3];
    if (!built_triple(plan->ids, perm)) {
      return fail(HF_EUNSUPPORTED, "three-kernel fusions are built for im2col + max-pool + bn-stats, max-pool + histogram + "
                                   "bn-stats and ccminer-Blake2b + SHA-256d + Ethash (in any order); this list is none of them");
    }
    if (f.split || f.threads || f.lending >= 0 || f.barrier >= 0 || f.launch_bound >= 0) {
      return fail(HF_EINVAL, "fusion '" + f.file + "': Split / Threads / Lending / Barrier / LaunchBound shape a pair; a three-kernel entry takes 'Blocks'");
    }
    // the entry's own block shape (`Blocks:`), applied like a pair's Split / Threads: to the table split of a horizontal preset
    KernelRow shaped[kMaxFuse] = {plan->rows[0], plan->rows[1], plan->rows[2]};
    const bool own_shape = split_idx == HF_SPLIT_TABLE && f.blocks.size() == 3 && !p->base_line;
    std::string label;
    for (int i = 0; own_shape && i < 3; i++) {
      if (shaped[i].block_dim.z != 1 || f.blocks[i] % shaped[i].block_dim.y) {
        std::string msg = "'Blocks' entry does not divide by BlockDim.Y of '" + shaped[i].name + "'";
        return fail(HF_EINVAL, msg);
      }
      shaped[i].block_dim.x = f.blocks[i] / shaped[i].block_dim.y;
      label += "_" + std::to_string(f.blocks[i]);
    }
    const KernelRow *rows[kMaxFuse] = {&shaped[0], &shaped[1], &shaped[2]};
    std::string err3;
    int rc3 = make_partition_n(rows, 3, *p, split_idx, plan->part, err3);
    if (rc3 == HF_OK && own_shape)
      plan->part.name = plan->rows[0].name + "_" + plan->rows[1].name + "_" + plan->rows[2].name + "_fused_kernel_" +
                        p->name + "_block" + label;
    if (rc3 == HF_OK && is_crypto(plan->ids[0]) && plan->part.launch_threads > 512) {
      rc3 = HF_EINVAL;
      err3 = "search kernels are built for fused blocks of at most 512 threads";
    }
    if (rc3 != HF_OK) {
      return fail(rc3, err3);
    }
    plan->lending = false;
    plan->barrier_mode = (body_has_barriers(plan->ids[0]) || body_has_barriers(plan->ids[1]) || body_has_barriers(plan->ids[2]))
                             ? HF_BARRIER_SUBSET : HF_BARRIER_NONE;
    *out = plan.release();
    return HF_OK;
  }
  if (is_crypto(plan->ids[0]) != is_crypto(plan->ids[1])) {
    return fail(HF_EUNSUPPORTED, "pairs mixing a tensor kernel with a search kernel are not built");
  }
  std::string err;
  // The pair's tuned default from the fusion list: `Split` alone re-splits the table's block,
  // `Split` + `Threads` give the fused block its own shape (applied below).
  const bool tuned = split_idx == HF_SPLIT_TABLE && split_threads <= 0 && f.split > 0 && !p->base_line;
  if (tuned && f.threads == 0) split_threads = (int)f.split;
  int rc = make_partition(plan->rows[0], plan->rows[1], *p, split_idx, split_threads, plan->part, err);
  if (rc != HF_OK) {
    return fail(rc, err);
  }
  if (tuned && f.threads > 0) {
    // the pair's tuned block shape from the fusion list: Split threads of kernel 1 in a block of Threads
    rc = hf_plan_set_block(plan.get(), (int)f.split, (int)(f.threads - f.split));
    if (rc != HF_OK) {
      return rc;
    }
  }
  if (split_idx == HF_SPLIT_TABLE && split_threads <= 0 && p->base_line && f.blocks.size() == 2) {
    // the pair's tuned vertical shape: `Blocks` threads run each body, both from thread 0
    rc = hf_plan_set_block(plan.get(), (int)f.blocks[0], (int)f.blocks[1]);
    if (rc != HF_OK) {
      return rc;
    }
  }
  if (split_idx == HF_SPLIT_TABLE && split_threads <= 0 && asked == entry_preset) {
    plan->grid_override[0] = f.grids[0];   // `Grids:` belongs to the entry's own preset
    plan->grid_override[1] = f.grids[1];
  }
  if (is_crypto(plan->ids[0]) && !p->base_line && plan->part.launch_threads > 512) {
    return fail(HF_EINVAL, "search kernels are built for fused blocks of at most 512 threads");
  }
  // the entry's tuned keys belong to its tuned shape: a plan of an explicit split or variant starts from the library's defaults
  const bool table_shape = split_idx == HF_SPLIT_TABLE && split_threads <= 0;
  if (f.lending >= 0 && table_shape) plan->lending = f.lending != 0;
  if (f.launch_bound >= 0 && table_shape) plan->bounded = f.launch_bound;
  const bool b1 = body_has_barriers(plan->ids[0]), b2 = body_has_barriers(plan->ids[1]);
  // One barrier policy per pair: nothing to do when neither body synchronises;
  // an LDS-counter barrier scoped to the synchronising half otherwise.  (Both
  // tensor bodies that synchronise do so twice per block, so a pair of them may
  // also share the hardware barrier: HF_BARRIER_MATCHED via hf_plan_set_barrier_mode.)
  plan->barrier_mode = (b1 || b2) ? HF_BARRIER_SUBSET : HF_BARRIER_NONE;
  if (f.barrier >= 0 && !p->base_line && table_shape) {
    rc = hf_plan_set_barrier_mode(plan.get(), f.barrier);
    if (rc != HF_OK) {
      return rc;
    }
  }
  *out = plan.release();
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_barrier_mode(hf_plan *plan, int mode) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  const bool b1 = body_has_barriers(plan->ids[0]), b2 = body_has_barriers(plan->ids[1]);
  switch (mode) {
    case HF_BARRIER_NONE:
      if (b1 || b2) return fail(HF_EINVAL, "this pair synchronises; HF_BARRIER_NONE is not legal");
      break;
    case HF_BARRIER_SUBSET:
      if (!b1 && !b2) return fail(HF_EINVAL, "neither kernel synchronises; nothing to scope");
      break;
    case HF_BARRIER_MATCHED:
      if (!(b1 && b2)) return fail(HF_EINVAL, "matched s_barrier needs both halves to synchronise equally often");
      break;
    case HF_BARRIER_BLOCKIDX:
      break;
    default:
      return fail(HF_EINVAL, "unknown barrier mode");
  }
  plan->barrier_mode = mode;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_grids(hf_plan *plan, int grid1, int grid2) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  if (grid1 < 0 || grid2 < 0) return fail(HF_EINVAL, "negative grid");
  plan->grid_override[0] = (unsigned)grid1;
  plan->grid_override[1] = (unsigned)grid2;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_block(hf_plan *plan, int threads1, int threads2) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  // (under a vertical preset both bodies start at thread 0: the two counts are the threads that run each body)
  if (threads1 <= 0 || threads2 <= 0 || threads1 % (int)kWave || threads2 % (int)kWave)
    return fail(HF_EINVAL, "both parts must be positive multiples of the 64-lane wavefront");
  // Same rule as the re-split of the reference's Context (KernelFusion.h:72): BlockDim.X = threads / BlockDim.Y.
  KernelRow rows[2] = {plan->rows[0], plan->rows[1]};
  const int want[2] = {threads1, threads2};
  for (int i = 0; i < 2; i++) {
    if (rows[i].block_dim.z != 1 || want[i] % (int)rows[i].block_dim.y)
      return fail(HF_EINVAL, "thread count does not divide by BlockDim.Y of '" + rows[i].name + "'");
    rows[i].block_dim.x = (uint32_t)want[i] / rows[i].block_dim.y;
  }
  if (is_crypto(plan->ids[0]) && (plan->preset->base_line ? std::max(threads1, threads2) : threads1 + threads2) > 512)
    return fail(HF_EINVAL, "search kernels are built for fused blocks of at most 512 threads");
  Partition part;
  std::string err;
  int rc = make_partition(rows[0], rows[1], *plan->preset, HF_SPLIT_TABLE, 0, part, err);
  if (rc != HF_OK) return fail(rc, err);
  part.name = plan->rows[0].name + "_" + plan->rows[1].name + "_fused_kernel_" + plan->preset->name + "_block_" +
              std::to_string(threads1) + "_" + std::to_string(threads2);
  plan->part = part;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_lending(hf_plan *plan, int on) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  plan->lending = on != 0;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_launch_bound(hf_plan *plan, int on) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  plan->bounded = on < 0 ? -1 : (on != 0);
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_launch_waves(hf_plan *plan, int waves) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  if (waves < 0 || waves > kBoundedWaves) return fail(HF_EINVAL, "waves per SIMD must be 0 (by the formula) or 1..8");
  plan->bound_waves = waves;
  if (waves > 0) plan->bounded = 1;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_launch_waves(const hf_plan *plan, int *formula, int *built) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (formula) *formula = formula_waves(plan);
  if (built) *built = plan_build_waves(plan);
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API void hf_plan_free(hf_plan *plan) { delete plan; }

HF_API int hf_plan_partition(const hf_plan *plan, hf_partition *out) try {
  if (!plan || !out) return fail(HF_EINVAL, "null argument");
  if (int prc = pair_call_only(plan)) return prc;
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->name, plan->part.name.c_str(), sizeof out->name - 1);
  for (int i = 0; i < 2; i++) {
    out->lo[i] = plan->part.lo[i];
    out->hi[i] = plan->part.hi[i];
    out->block_dim[i] = {plan->part.block_dim[i].x, plan->part.block_dim[i].y, plan->part.block_dim[i].z};
  }
  out->launch_threads = plan->part.launch_threads;
  out->launch_blocks = plan->part.launch_blocks;
  out->barrier_mode = plan->barrier_mode;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_num_kernels(const hf_plan *plan) { return plan ? plan->n : fail(HF_EINVAL, "null plan"); }

HF_API int hf_plan_partition_n(const hf_plan *plan, hf_partition_n *out) try {
  if (!plan || !out) return fail(HF_EINVAL, "null argument");
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->name, plan->part.name.c_str(), sizeof out->name - 1);
  out->n = plan->n;
  for (int i = 0; i < plan->n; i++) {
    out->lo[i] = plan->part.lo[i];
    out->hi[i] = plan->part.hi[i];
    out->block_dim[i] = {plan->part.block_dim[i].x, plan->part.block_dim[i].y, plan->part.block_dim[i].z};
  }
  out->launch_threads = plan->part.launch_threads;
  out->launch_blocks = plan->part.launch_blocks;
  out->barrier_mode = plan->barrier_mode;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_set_block_n(hf_plan *plan, const int *threads, int n) try {
  if (!plan || !threads) return fail(HF_EINVAL, "null argument");
  if (n != plan->n) return fail(HF_EINVAL, "one thread count per kernel of the plan");
  if (plan->n == 2) return hf_plan_set_block(plan, threads[0], threads[1]);
  if (plan->preset->base_line) return fail(HF_EINVAL, "vertical presets have no thread partition to set");
  KernelRow rows[kMaxFuse] = {plan->rows[0], plan->rows[1], plan->rows[2]};
  int total = 0;
  std::string label;
  for (int i = 0; i < n; i++) {
    if (threads[i] <= 0 || threads[i] % (int)kWave)
      return fail(HF_EINVAL, "every part must be a positive multiple of the 64-lane wavefront");
    if (rows[i].block_dim.z != 1 || threads[i] % (int)rows[i].block_dim.y)
      return fail(HF_EINVAL, "thread count does not divide by BlockDim.Y of '" + rows[i].name + "'");
    rows[i].block_dim.x = (uint32_t)threads[i] / rows[i].block_dim.y;  // KernelFusion.h:72
    total += threads[i];
    label += "_" + std::to_string(threads[i]);
  }
  if (is_crypto(plan->ids[0]) && total > 512) return fail(HF_EINVAL, "search kernels are built for fused blocks of at most 512 threads");
  const KernelRow *ptrs[kMaxFuse] = {&rows[0], &rows[1], &rows[2]};
  Partition part;
  std::string err;
  int rc = make_partition_n(ptrs, n, *plan->preset, HF_SPLIT_TABLE, part, err);
  if (rc != HF_OK) return fail(rc, err);
  part.name = plan->rows[0].name + "_" + plan->rows[1].name + "_" + plan->rows[2].name + "_fused_kernel_" +
              plan->preset->name + "_block" + label;
  plan->part = part;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_local_index(const hf_plan *plan, int half, uint32_t tid, hf_dim3 *out) try {
  if (!plan || !out) return fail(HF_EINVAL, "null argument");
  if (half < 0 || half >= plan->n) return fail(HF_EINVAL, "kernel index outside the plan");
  if (tid < plan->part.lo[half] || tid >= plan->part.hi[half])
    return fail(HF_EINVAL, "thread is outside this kernel's bounds");
  Dim3 d = local_index(tid, plan->part.lo[half], plan->part.block_dim[half]);
  *out = {d.x, d.y, d.z};
  return HF_OK;
} catch (...) {
  return trap_exception();
}

// ------------------------------------------------------------- constants
namespace {
int store_ethash(SearchConstants &c, const void *dag, uint32_t dag_items, const uint8_t *header, uint64_t target) {
  if (!dag || !header) return fail(HF_EINVAL, "ethash: null dag or header");
  if (dag_items == 0) return fail(HF_EINVAL, "ethash: empty dag");
  if (!aligned16(dag)) return fail(HF_EINVAL, "ethash: dag must be 16-byte aligned");
  c.dag = dag;
  c.dag_items = dag_items;
  for (int i = 0; i < 4; i++) c.eth_header[i] = load_le64(header + 8 * i);
  c.eth_target = target;
  c.eth_set = true;
  return HF_OK;
}
int store_sha256d(SearchConstants &c, const uint8_t *header, uint64_t target64) {
  if (!header) return fail(HF_EINVAL, "sha256d: null header");
  uint32_t st[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
  uint32_t blk[16];
  for (int i = 0; i < 16; i++) blk[i] = load_be32(header + 4 * i);
  host_sha256_compress(st, blk);
  std::memcpy(c.sha_mid, st, sizeof st);
  for (int i = 0; i < 3; i++) c.sha_tail[i] = load_be32(header + 64 + 4 * i);
  c.sha_target = target64;
  c.sha_set = true;
  return HF_OK;
}
int store_blake2b(SearchConstants &c, bool sia, const uint8_t *header) {
  if (!header) return fail(HF_EINVAL, sia ? "sia_blake2b: null header" : "blake2b: null header");
  uint64_t *m = sia ? c.sia_m : c.b2_m;
  for (int i = 0; i < 10; i++) m[i] = load_le64(header + 8 * i);
  (sia ? c.sia_set : c.b2_set) = true;
  return HF_OK;
}
}  // namespace

// The process-wide set: each call builds the new values aside and swaps them in under the lock.
HF_API int hf_ethash_set_constants(const void *dag, uint32_t dag_items, const uint8_t header[32], uint64_t target,
                                   void *) try {
  SearchConstants c;
  int rc = store_ethash(c, dag, dag_items, header, target);
  if (rc != HF_OK) return rc;
  std::lock_guard<std::mutex> lock(g_const_mu);
  g_const.dag = c.dag;
  g_const.dag_items = c.dag_items;
  std::memcpy(g_const.eth_header, c.eth_header, sizeof c.eth_header);
  g_const.eth_target = c.eth_target;
  g_const.eth_set = true;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_sha256d_set_block(const uint8_t header[80], uint64_t target64, void *) try {
  SearchConstants c;
  int rc = store_sha256d(c, header, target64);
  if (rc != HF_OK) return rc;
  std::lock_guard<std::mutex> lock(g_const_mu);
  std::memcpy(g_const.sha_mid, c.sha_mid, sizeof c.sha_mid);
  std::memcpy(g_const.sha_tail, c.sha_tail, sizeof c.sha_tail);
  g_const.sha_target = c.sha_target;
  g_const.sha_set = true;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_sia_blake2b_set_block(const uint8_t header[80], void *) try {
  SearchConstants c;
  int rc = store_blake2b(c, true, header);
  if (rc != HF_OK) return rc;
  std::lock_guard<std::mutex> lock(g_const_mu);
  std::memcpy(g_const.sia_m, c.sia_m, sizeof c.sia_m);
  g_const.sia_set = true;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_blake2b_set_block(const uint8_t header[80], void *) try {
  SearchConstants c;
  int rc = store_blake2b(c, false, header);
  if (rc != HF_OK) return rc;
  std::lock_guard<std::mutex> lock(g_const_mu);
  std::memcpy(g_const.b2_m, c.b2_m, sizeof c.b2_m);
  g_const.b2_set = true;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

// Caller-owned sets.
HF_API int hf_constants_create(hf_constants **out) try {
  if (!out) return fail(HF_EINVAL, "null output pointer");
  *out = new hf_constants();
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API void hf_constants_free(hf_constants *c) { delete c; }

HF_API int hf_constants_set_ethash(hf_constants *c, const void *dag, uint32_t dag_items, const uint8_t header[32],
                                   uint64_t target) try {
  if (!c) return fail(HF_EINVAL, "null constants");
  return store_ethash(c->c, dag, dag_items, header, target);
} catch (...) {
  return trap_exception();
}

HF_API int hf_constants_set_sha256d(hf_constants *c, const uint8_t header[80], uint64_t target64) try {
  if (!c) return fail(HF_EINVAL, "null constants");
  return store_sha256d(c->c, header, target64);
} catch (...) {
  return trap_exception();
}

HF_API int hf_constants_set_sia_blake2b(hf_constants *c, const uint8_t header[80]) try {
  if (!c) return fail(HF_EINVAL, "null constants");
  return store_blake2b(c->c, true, header);
} catch (...) {
  return trap_exception();
}

HF_API int hf_constants_set_blake2b(hf_constants *c, const uint8_t header[80]) try {
  if (!c) return fail(HF_EINVAL, "null constants");
  return store_blake2b(c->c, false, header);
} catch (...) {
  return trap_exception();
}

HF_API int hf_plan_bind_constants(hf_plan *plan, const hf_constants *c) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  plan->has_consts = c != nullptr;
  if (c) plan->consts = c->c;
  return HF_OK;
} catch (...) {
  return trap_exception();
}

// ---------------------------------------------------------------- launches
namespace {
int launch_native_named(const char *kernel_name, const void *args, const SearchConstants *consts, int grid_blocks,
                        int block_threads, void *stream) {
  if (!kernel_name) return fail(HF_EINVAL, "null kernel name");
  KernelId id;
  if (!lookup_kernel(kernel_name, id))
    return fail(HF_ENOTFOUND, std::string("kernel '") + kernel_name + "' has no gfx950 implementation in this library");
  Prepared p;
  int rc = prepare(id, args, p, consts);
  if (rc != HF_OK) return rc;
  unsigned block = block_threads > 0 ? (unsigned)block_threads
                                     : (is_crypto(id) ? 128u : (id == K_MAXPOOL ? 256u : (id == K_HISTC ? 768u : 512u)));
  return do_launch_native(id, p, grid_blocks, block, static_cast<hipStream_t>(stream));
}
}  // namespace

HF_API int hf_launch_native(const char *kernel_name, const void *args, int grid_blocks, int block_threads,
                            void *stream) try {
  return launch_native_named(kernel_name, args, nullptr, grid_blocks, block_threads, stream);
} catch (...) {
  return trap_exception();
}

HF_API int hf_launch_native_with(const char *kernel_name, const void *args, const hf_constants *constants,
                                 int grid_blocks, int block_threads, void *stream) try {
  if (!constants) return fail(HF_EINVAL, "null constants");
  return launch_native_named(kernel_name, args, &constants->c, grid_blocks, block_threads, stream);
} catch (...) {
  return trap_exception();
}

namespace {

int do_launch_fused(const hf_plan *plan, const Prepared &p1, const Prepared &p2, int grid_blocks, hipStream_t stream) {
  FuseGeom g;
  g.d1 = plan->part.hi[0] - plan->part.lo[0];
  g.d2 = plan->part.hi[1] - plan->part.lo[1];
  g.lds1 = (p1.lds + 15u) & ~15u;
  g.lds2 = (p2.lds + 15u) & ~15u;
  g.hint1 = p1.hint;
  g.hint2 = p2.hint;
  g.grid1 = g.grid2 = 0;
  g.lend = 0;
  const bool crypto = is_crypto(plan->ids[0]);
  const unsigned exact = grid_blocks > 0 ? (unsigned)grid_blocks : kDefaultEthashGrid;
  if ((unsigned long long)std::max(exact, std::max(plan->grid_override[0], plan->grid_override[1])) * (g.d1 + g.d2) >
      0xFFFFFFFFull)
    return fail(HF_EINVAL, "grid_blocks * block threads must fit 32 bits (the bodies index work items with 32-bit counters)");
  const int waves = plan_build_waves(plan);  // 0: the plain build
  // every thread of the launch may run either body (lending), so each 32-bit counter is checked against all of them
  auto counters_fit = [&](unsigned grid, unsigned block) {
    const unsigned long long threads = (unsigned long long)grid * block;
    return threads <= 0xFFFFFFFFull && counter_fits(p1, threads) && counter_fits(p2, threads);
  };
  hipError_t e;
  if (plan->preset->base_line) {
    // Vertical baseline: both kernels start at thread 0 of a block of max(d1, d2) threads.
    const unsigned block = std::max(g.d1, g.d2);
    g.grid1 = p1.exact_grid ? exact : (grid_blocks > 0 ? (unsigned)grid_blocks : default_grid(p1, g.d1, block));
    g.grid2 = p2.exact_grid ? exact : (grid_blocks > 0 ? (unsigned)grid_blocks : default_grid(p2, g.d2, block));
    // hf_plan_set_grids / the entry's `Grids:`: a few resident blocks whose threads stride over each body's work in turn
    if (grid_blocks <= 0 && plan->grid_override[0] && !p1.exact_grid) g.grid1 = plan->grid_override[0];
    if (grid_blocks <= 0 && plan->grid_override[1] && !p2.exact_grid) g.grid2 = plan->grid_override[1];
    const size_t lds = 4 * kBarrierWords + g.lds1 + g.lds2;
    const unsigned grid = std::max(g.grid1, g.grid2);
    if (!counters_fit(grid, block)) return fail(HF_EINVAL, kCounterMsg);
    e = crypto ? launch_fused_crypto(plan->ids[0], plan->ids[1], MODE_VERTICAL, waves, p1.blob, p2.blob, g, grid, lds, stream)
               : launch_fused_dl(plan->ids[0], plan->ids[1], MODE_VERTICAL, waves, p1.blob, p2.blob, g, grid, lds, stream);
  } else if (plan->barrier_mode == HF_BARRIER_BLOCKIDX) {
    // Each kernel gets its own workgroups inside one launch.
    const unsigned block = std::max(g.d1, g.d2);
    g.grid1 = p1.exact_grid ? exact : default_grid(p1, g.d1, block);
    g.grid2 = p2.exact_grid ? exact : default_grid(p2, g.d2, block);
    if (!p1.exact_grid && !p2.exact_grid && grid_blocks > 0) {
      g.grid1 = std::max(1u, (unsigned)grid_blocks / 2);
      g.grid2 = std::max(1u, (unsigned)grid_blocks - g.grid1);
    }
    const size_t lds = std::max(g.lds1, g.lds2);
    if ((unsigned long long)g.grid1 + g.grid2 > 0xFFFFFFFFull || !counters_fit(g.grid1 + g.grid2, block))
      return fail(HF_EINVAL, kCounterMsg);
    e = crypto ? launch_fused_crypto(plan->ids[0], plan->ids[1], MODE_BLOCKIDX, 0, p1.blob, p2.blob, g, g.grid1 + g.grid2, lds, stream)
               : launch_fused_dl(plan->ids[0], plan->ids[1], MODE_BLOCKIDX, 0, p1.blob, p2.blob, g, g.grid1 + g.grid2, lds, stream);
  } else {
    // One grid for both halves.  When the caller names it, both halves stride over all of it
    // (a kernel whose grid fixes its work, ethash, always does); otherwise each half strides
    // over its own preferred number of blocks and the launch covers the larger of the two.
    const unsigned block = g.d1 + g.d2;
    if (grid_blocks > 0) {
      g.grid1 = g.grid2 = (unsigned)grid_blocks;
    } else {
      g.grid1 = p1.exact_grid ? exact : default_grid(p1, g.d1, block);
      g.grid2 = p2.exact_grid ? exact : default_grid(p2, g.d2, block);
      if (plan->grid_override[0] && !p1.exact_grid) g.grid1 = plan->grid_override[0];
      if (plan->grid_override[1] && !p2.exact_grid) g.grid2 = plan->grid_override[1];
    }
    // Wave lending: in the blocks only one kernel strides over, the other half's waves run
    // that kernel too, so those blocks are d1+d2 threads wide for it and it needs fewer of them.
    g.lend = plan->lending && grid_blocks <= 0;
    if (g.lend) {
      const unsigned dd = g.d1 + g.d2;
      if (g.grid2 > g.grid1 && body_is_flat(plan->ids[1]) && !p2.exact_grid)
        g.grid2 = g.grid1 + (unsigned)(((unsigned long long)(g.grid2 - g.grid1) * g.d2 + dd - 1) / dd);
      else if (g.grid1 > g.grid2 && body_is_flat(plan->ids[0]) && !p1.exact_grid)
        g.grid1 = g.grid2 + (unsigned)(((unsigned long long)(g.grid1 - g.grid2) * g.d1 + dd - 1) / dd);
    }
    const unsigned grid = std::max(g.grid1, g.grid2);
    if (!counters_fit(grid, block)) return fail(HF_EINVAL, kCounterMsg);
    const size_t lds = 4 * kBarrierWords + g.lds1 + g.lds2;
    const FuseMode mode = plan->barrier_mode == HF_BARRIER_MATCHED ? MODE_MATCHED : MODE_HFUSE;
    e = crypto ? launch_fused_crypto(plan->ids[0], plan->ids[1], mode, waves, p1.blob, p2.blob, g, grid, lds, stream)
               : launch_fused_dl(plan->ids[0], plan->ids[1], mode, waves, p1.blob, p2.blob, g, grid, lds, stream);
  }
  if (e == hipErrorNotSupported) return fail(HF_EUNSUPPORTED, "this pair / barrier mode is not built");
  if (e != hipSuccess) return hip_fail(e, "fused launch");
  return HF_OK;
}

}  // namespace

HF_API int hf_launch_fused(const hf_plan *plan, const void *args1, const void *args2, int grid_blocks, void *stream) try {
  if (!plan) return fail(HF_EINVAL, "null plan");
  if (int prc = pair_call_only(plan)) return prc;
  Prepared p1, p2;
  const SearchConstants *consts = plan->has_consts ? &plan->consts : nullptr;
  int rc = prepare(plan->ids[0], args1, p1, consts);
  if (rc != HF_OK) return rc;
  rc = prepare(plan->ids[1], args2, p2, consts);
  if (rc != HF_OK) return rc;
  return do_launch_fused(plan, p1, p2, grid_blocks, static_cast<hipStream_t>(stream));
} catch (...) {
  return trap_exception();
}

extern "C++" {
namespace {
// `warmup` untimed repetitions of once(r), then `iters` timed ones between two HIP events recorded on `stream`.
template <class Once>
int time_repetitions(hipStream_t stream, int warmup, int iters, Once once, float *elapsed_ms) {
  for (int r = 0; r < warmup; r++) {
    int rc = once(r);
    if (rc != HF_OK) return rc;
  }
  hipEvent_t t0, t1;
  hipError_t e = hipEventCreate(&t0);
  if (e != hipSuccess) return hip_fail(e, "hipEventCreate");
  e = hipEventCreate(&t1);
  if (e != hipSuccess) { (void)hipEventDestroy(t0); return hip_fail(e, "hipEventCreate"); }
  int rc = HF_OK;
  e = hipEventRecord(t0, stream);
  for (int r = 0; r < iters && rc == HF_OK && e == hipSuccess; r++) rc = once(warmup + r);
  if (e == hipSuccess) e = hipEventRecord(t1, stream);
  if (e == hipSuccess) e = hipEventSynchronize(t1);
  if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, t0, t1);
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc != HF_OK) return rc;
  if (e != hipSuccess) return hip_fail(e, "timing");
  return HF_OK;
}
}  // namespace
}  // extern "C++"

HF_API int hf_time_pair(const hf_plan *plan, int mode, const void *const *args1, const void *const *args2, int nsets,
                        int first_set, int warmup, int iters, int grid_blocks, void *stream_, float *elapsed_ms) try {
  if (!plan || !args1 || !args2 || !elapsed_ms) return fail(HF_EINVAL, "null argument");
  if (int prc = pair_call_only(plan)) return prc;
  if (nsets <= 0 || iters <= 0 || warmup < 0 || mode < 0 || mode > 4 || first_set < 0 || first_set >= nsets)
    return fail(HF_EINVAL, "bad repetition arguments");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  // mode 4: a second stream (default priority) and a fork / join event pair per repetition
  hipStream_t side = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  struct SideGuard {
    hipStream_t &s;
    hipEvent_t &a, &b;
    ~SideGuard() {
      if (a) (void)hipEventDestroy(a);
      if (b) (void)hipEventDestroy(b);
      if (s) (void)hipStreamDestroy(s);
    }
  } side_guard{side, fork, join};
  if (mode == 4) {
    hipError_t se = hipStreamCreateWithFlags(&side, hipStreamNonBlocking);
    if (se == hipSuccess) se = hipEventCreateWithFlags(&fork, hipEventDisableTiming);
    if (se == hipSuccess) se = hipEventCreateWithFlags(&join, hipEventDisableTiming);
    if (se != hipSuccess) return hip_fail(se, "second stream");
  }
  std::vector<Prepared> p1(nsets), p2(nsets);
  const SearchConstants *consts = plan->has_consts ? &plan->consts : nullptr;
  for (int i = 0; i < nsets; i++) {
    int rc = prepare(plan->ids[0], args1[i], p1[i], consts);
    if (rc != HF_OK) return rc;
    rc = prepare(plan->ids[1], args2[i], p2[i], consts);
    if (rc != HF_OK) return rc;
  }
  const unsigned b1 = plan->rows[0].native_block(), b2 = plan->rows[1].native_block();
  auto once = [&](int i) -> int {
    const int s = (int)(((long long)first_set + i) % nsets);
    int rc = HF_OK;
    // A kernel whose grid fixes its amount of work (ethash) always gets grid_blocks; the
    // others size their own grid in the back-to-back mode.
    const int g1 = (mode == 2 && !p1[s].exact_grid) ? 0 : grid_blocks;
    const int g2 = (mode == 2 && !p2[s].exact_grid) ? 0 : grid_blocks;
    if (mode == 0 || mode == 2) rc = do_launch_native(plan->ids[0], p1[s], g1, b1, stream);
    if (rc != HF_OK) return rc;
    if (mode == 1 || mode == 2) rc = do_launch_native(plan->ids[1], p2[s], g2, b2, stream);
    if (rc != HF_OK) return rc;
    if (mode == 3) rc = do_launch_fused(plan, p1[s], p2[s], grid_blocks, stream);
    if (mode == 4) {
      hipError_t se = hipEventRecord(fork, stream);
      if (se == hipSuccess) se = hipStreamWaitEvent(side, fork, 0);
      if (se != hipSuccess) return hip_fail(se, "fork");
      rc = do_launch_native(plan->ids[0], p1[s], p1[s].exact_grid ? grid_blocks : 0, b1, stream);
      if (rc != HF_OK) return rc;
      rc = do_launch_native(plan->ids[1], p2[s], p2[s].exact_grid ? grid_blocks : 0, b2, side);
      if (rc != HF_OK) return rc;
      se = hipEventRecord(join, side);
      if (se == hipSuccess) se = hipStreamWaitEvent(stream, join, 0);
      if (se != hipSuccess) return hip_fail(se, "join");
    }
    return rc;
  };
  return time_repetitions(stream, warmup, iters, once, elapsed_ms);
} catch (...) {
  return trap_exception();
}

namespace {

int do_launch_fused3(const hf_plan *plan, const Prepared *p, int grid_blocks, hipStream_t stream) {
  FuseGeom3 g;
  const bool vertical = plan->preset->base_line;
  unsigned block = 0, grid = 0;
  size_t lds = 4 * kBarrierWords;
  for (int i = 0; i < 3; i++) {
    g.d[i] = plan->part.hi[i] - plan->part.lo[i];
    g.lds[i] = (p[i].lds + 15u) & ~15u;
    g.hint[i] = p[i].hint;
    lds += g.lds[i];
    block = vertical ? std::max(block, g.d[i]) : block + g.d[i];
  }
  for (int i = 0; i < 3; i++) {
    if (grid_blocks > 0) g.grid[i] = (unsigned)grid_blocks;
    else g.grid[i] = p[i].exact_grid ? kDefaultEthashGrid : (p[i].items == 0 ? 0u : default_grid(p[i], g.d[i], block));
    grid = std::max(grid, g.grid[i]);
  }
  if (grid == 0) return HF_OK;  // nothing to do
  const unsigned long long threads = (unsigned long long)grid * block;
  if (threads > 0xFFFFFFFFull || !counter_fits(p[0], threads) || !counter_fits(p[1], threads) || !counter_fits(p[2], threads))
    return fail(HF_EINVAL, kCounterMsg);
  // into the order the instantiation is built in: kernel c of it is the list's kernel perm[c]
  int perm[3];
  if (!built_triple(plan->ids, perm)) return fail(HF_EUNSUPPORTED, "this three-kernel list is not built");
  FuseGeom3 b;
  KernelId ids[3];
  const void *blobs[3];
  for (int c = 0; c < 3; c++) {
    const int i = perm[c];
    ids[c] = plan->ids[i];
    blobs[c] = p[i].blob;
    b.lo[c] = vertical ? 0u : plan->part.lo[i];
    b.d[c] = g.d[i];
    b.lds[c] = g.lds[i];
    b.hint[c] = g.hint[i];
    b.grid[c] = g.grid[i];
  }
  const bool bounded = plan_build_waves(plan) != 0;   // the launch-bound presets: the build bounded for 8 waves per SIMD
  const hipError_t e = is_crypto(ids[0]) ? launch_fused3_crypto(ids, vertical, bounded, blobs, b, grid, block, lds, stream)
                                         : launch_fused3_dl(ids, vertical, bounded, blobs, b, grid, block, lds, stream);
  if (e == hipErrorNotSupported) return fail(HF_EUNSUPPORTED, "this three-kernel list is not built (built: the reference's lists, in their order)");
  if (e != hipSuccess) return hip_fail(e, "fused launch");
  return HF_OK;
}

}  // namespace

HF_API int hf_launch_fused_n(const hf_plan *plan, const void *const *args, int n, int grid_blocks, void *stream) try {
  if (!plan || !args) return fail(HF_EINVAL, "null argument");
  if (n != plan->n) return fail(HF_EINVAL, "one argument list per kernel of the plan");
  if (n == 2) return hf_launch_fused(plan, args[0], args[1], grid_blocks, stream);
  Prepared p[3];
  const SearchConstants *consts = plan->has_consts ? &plan->consts : nullptr;
  for (int i = 0; i < 3; i++) {
    int rc = prepare(plan->ids[i], args[i], p[i], consts);
    if (rc != HF_OK) return rc;
  }
  return do_launch_fused3(plan, p, grid_blocks, static_cast<hipStream_t>(stream));
} catch (...) {
  return trap_exception();
}

HF_API int hf_time_fused_n(const hf_plan *plan, int mode, const void *const *args, int n, int nsets, int first_set,
                           int warmup, int iters, int grid_blocks, void *stream_, float *elapsed_ms) try {
  if (!plan || !args || !elapsed_ms) return fail(HF_EINVAL, "null argument");
  if (n != plan->n || n != 3) return fail(HF_EINVAL, "hf_time_fused_n times three-kernel plans (pairs: hf_time_pair)");
  if (nsets <= 0 || iters <= 0 || warmup < 0 || (mode != 2 && mode != 3) || first_set < 0 || first_set >= nsets)
    return fail(HF_EINVAL, "bad repetition arguments");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const SearchConstants *consts = plan->has_consts ? &plan->consts : nullptr;
  std::vector<Prepared> p((size_t)nsets * 3);
  for (int s = 0; s < nsets; s++)
    for (int i = 0; i < 3; i++) {
      int rc = prepare(plan->ids[i], args[(size_t)s * 3 + i], p[(size_t)s * 3 + i], consts);
      if (rc != HF_OK) return rc;
    }
  auto once = [&](int r) -> int {
    const Prepared *q = &p[(size_t)(((long long)first_set + r) % nsets) * 3];
    if (mode == 3) return do_launch_fused3(plan, q, grid_blocks, stream);
    for (int i = 0; i < 3; i++) {
      int rc = do_launch_native(plan->ids[i], q[i], q[i].exact_grid ? grid_blocks : 0, plan->rows[i].native_block(), stream);
      if (rc != HF_OK) return rc;
    }
    return HF_OK;
  };
  return time_repetitions(stream, warmup, iters, once, elapsed_ms);
} catch (...) {
  return trap_exception();
}

HF_API int hf_fill_splitmix64(uint64_t *dst, uint64_t nwords, uint64_t seed, void *stream) try {
  if (!dst && nwords) return fail(HF_EINVAL, "null destination");
  hipError_t e = launch_fill_splitmix64(reinterpret_cast<unsigned long long *>(dst), nwords, seed, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "fill launch");
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_copy_f32(const float *src, float *dst, uint64_t n, void *stream) try {
  if ((!src || !dst) && n) return fail(HF_EINVAL, "null pointer");
  hipError_t e = launch_copy_f32(src, dst, n, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "copy launch");
  return HF_OK;
} catch (...) {
  return trap_exception();
}

namespace {
int check_stream_probe(int pattern, const void *src, void *dst, uint64_t bytes, int grid_blocks, int block_threads) {
  if (pattern < HF_STREAM_EMPTY || pattern > HF_STREAM_WRITE_XCD) return fail(HF_EINVAL, "unknown stream pattern");
  if (pattern == HF_STREAM_EMPTY) return HF_OK;
  const bool writes_only = pattern == HF_STREAM_WRITE || pattern == HF_STREAM_WRITE_STRIDED || pattern == HF_STREAM_WRITE_XCD;
  const bool reads_only = pattern == HF_STREAM_READ || pattern == HF_STREAM_READ_LINES;
  if ((!writes_only && !src) || !dst) return fail(HF_EINVAL, "null pointer");
  if ((!writes_only && !aligned16(src)) || (!reads_only && !aligned16(dst))) return fail(HF_EINVAL, "buffers must be 16-byte aligned");
  if (grid_blocks <= 0 || block_threads <= 0 || block_threads % (int)kWave || block_threads > (int)kMaxBlock)
    return fail(HF_EINVAL, "grid must be positive and the block a multiple of 64 up to 1024");
  if (pattern == HF_STREAM_WRITE_XCD && grid_blocks % 8) return fail(HF_EINVAL, "the XCD-ordered pattern needs a multiple of eight workgroups");
  const uint64_t threads = (uint64_t)grid_blocks * (uint64_t)block_threads;
  // whole vectors, shared out evenly: every workgroup (every thread, for the random lines) gets the same share
  const uint64_t unit = 16ull * (pattern == HF_STREAM_READ_LINES ? threads * 4ull : (uint64_t)grid_blocks);
  if (bytes == 0 || bytes % unit)
    return fail(HF_EINVAL, "bytes must be a positive multiple of 16 * grid (64 * grid * block for the random lines)");
  if (pattern == HF_STREAM_READ_LINES && (bytes >> 7) > 0xFFFFFFFFull) return fail(HF_EINVAL, "more than 2^32 lines");
  return HF_OK;
}
}  // namespace

HF_API int hf_stream_probe(int pattern, const void *src, void *dst, uint64_t bytes, int grid_blocks, int block_threads,
                           void *stream) try {
  if (int rc = check_stream_probe(pattern, src, dst, bytes, grid_blocks, block_threads)) return rc;
  hipError_t e = launch_stream_probe(pattern, src, dst, bytes / 16, (unsigned)grid_blocks, (unsigned)block_threads,
                                     static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "stream probe launch");
  return HF_OK;
} catch (...) {
  return trap_exception();
}

HF_API int hf_time_stream_probe(int pattern, const void *src, void *dst, uint64_t bytes, uint64_t src_stride,
                                uint64_t dst_stride, int nbuf, int grid_blocks, int block_threads, int warmup, int iters,
                                void *stream_, float *elapsed_ms) try {
  if (!elapsed_ms) return fail(HF_EINVAL, "null argument");
  if (nbuf <= 0 || iters <= 0 || warmup < 0 || src_stride % 16 || dst_stride % 16) return fail(HF_EINVAL, "bad repetition arguments");
  if (int rc = check_stream_probe(pattern, src, dst, bytes, grid_blocks, block_threads)) return rc;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  auto once = [&](int r) -> int {
    const uint64_t k = (uint64_t)(r % nbuf);
    const void *s = src ? static_cast<const char *>(src) + k * src_stride : nullptr;
    void *d = dst ? static_cast<char *>(dst) + k * dst_stride : nullptr;
    hipError_t e = launch_stream_probe(pattern, s, d, bytes / 16, (unsigned)grid_blocks, (unsigned)block_threads, stream);
    return e == hipSuccess ? HF_OK : hip_fail(e, "stream probe launch");
  };
  return time_repetitions(stream, warmup, iters, once, elapsed_ms);
} catch (...) {
  return trap_exception();
}

}  // extern "C"
