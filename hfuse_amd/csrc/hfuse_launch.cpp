// hfuse-launch: a C++ host program over the C-ABI, the shape of the callers the reference's
// kernels were generated for (its README's TorchKernel extension and ethminer's fuse/fuser):
// for one pair (or three-kernel entry) of the fusion list it launches native kernel 1, native kernel 2,
// both back to back and the fused kernel on identical synthetic inputs, several times in one process,
// prints the per-launch durations, and checks that the fused launch produced the same bytes
// as the two native launches (batch-norm statistics: the same values to 1e-5 relative).
//
//   hfuse-launch <fusion.yaml> <kernels.yaml> <File name | index | all> [--preset P] [--split N]
//                [--iters N] [--small]
//
// Inputs are the benchmark shapes (--small: shapes a thousand times smaller), filled from
// a SplitMix64 counter stream.  Uses only include/hfuse_gfx950.h and the HIP runtime.
// One input set is reused by every repetition, so kernels whose inputs fit the 256 MB
// memory-side cache time faster here than in the benchmark, which rotates input sets.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/hfuse_gfx950.h"

namespace {

void hip_check(hipError_t e, const char *what) {
  if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
void hf_check(int rc) {
  if (rc != HF_OK) throw std::runtime_error(hf_last_error());
}

uint64_t splitmix64(uint64_t seed, uint64_t i) {
  uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// A device buffer with a host mirror for filling and comparing.
struct Buffer {
  void *dev = nullptr;
  size_t bytes = 0;
  explicit Buffer(size_t n) : bytes(n) { hip_check(hipMalloc(&dev, n ? n : 16), "hipMalloc"); }
  ~Buffer() { (void)hipFree(dev); }
  Buffer(const Buffer &) = delete;
  Buffer &operator=(const Buffer &) = delete;
  void fill_uniform(uint64_t seed, float lo, float hi) {
    std::vector<float> h(bytes / 4);
    for (size_t i = 0; i < h.size(); i++) h[i] = lo + (hi - lo) * (float)(splitmix64(seed, i) >> 40) * (1.0f / 16777216.0f);
    hip_check(hipMemcpy(dev, h.data(), bytes, hipMemcpyHostToDevice), "upload");
  }
  void fill_byte(int v) { hip_check(hipMemset(dev, v, bytes), "hipMemset"); }
  std::vector<unsigned char> download() const {
    std::vector<unsigned char> h(bytes);
    hip_check(hipMemcpy(h.data(), dev, bytes, hipMemcpyDeviceToHost), "download");
    return h;
  }
};

// One original kernel bound to synthetic inputs: its argument struct, its outputs (two sets:
// one for native launches, one for fused ones) and how to reset accumulating outputs.
struct Workload {
  std::string kernel;
  std::vector<std::unique_ptr<Buffer>> inputs;
  std::vector<std::unique_ptr<Buffer>> out_native, out_fused;
  std::vector<unsigned char> args_native, args_fused;  // the hf_*_args struct, pointing at either output set
  bool accumulates = false;                            // outputs must be zeroed before a compared launch
  float tolerance = 0.0f;                              // relative tolerance of fp32 outputs, 0 = same bytes
  int grid = 0;                                        // exact grid (ethash) or 0
  double bytes = 0;                                    // algorithmic bytes per launch (0 for the searches)
  double hashes = 0;                                   // nonces per launch (0 for tensor kernels)

  template <class A>
  void set_args(const A &native, const A &fused) {
    args_native.assign(reinterpret_cast<const unsigned char *>(&native), reinterpret_cast<const unsigned char *>(&native) + sizeof native);
    args_fused.assign(reinterpret_cast<const unsigned char *>(&fused), reinterpret_cast<const unsigned char *>(&fused) + sizeof fused);
  }
  void reset() {
    for (auto *set : {&out_native, &out_fused})
      for (auto &b : *set) b->fill_byte(accumulates ? 0 : 0xFF);
  }
};

Buffer *add(std::vector<std::unique_ptr<Buffer>> &v, size_t bytes) {
  v.emplace_back(new Buffer(bytes));
  return v.back().get();
}

std::unique_ptr<Workload> make_workload(const std::string &k, bool second_of_hist_pair, bool small, uint64_t seed) {
  auto w = std::make_unique<Workload>();
  w->kernel = k;
  const int64_t N = small ? 2 : 32;
  if (k == "im2col_kernel") {
    const int64_t C = small ? 4 : 64, H = small ? 12 : 56, W = H;
    Buffer *x = add(w->inputs, N * C * H * W * 4);
    x->fill_uniform(seed, -1.0f, 1.0f);
    hf_im2col_args a[2] = {};
    for (int s = 0; s < 2; s++) {
      Buffer *col = add(s ? w->out_fused : w->out_native, N * C * 9 * H * W * 4);
      a[s].n = N * C * H * W;
      a[s].data_im = static_cast<const float *>(x->dev);
      a[s].height = H; a[s].width = W; a[s].kernel_h = a[s].kernel_w = 3; a[s].pad_h = a[s].pad_w = 1;
      a[s].stride_h = a[s].stride_w = 1; a[s].dilation_h = a[s].dilation_w = 1; a[s].height_col = H; a[s].width_col = W;
      a[s].data_col = static_cast<float *>(col->dev);
    }
    w->set_args(a[0], a[1]);
    w->bytes = 4.0 * N * C * H * W * 10;
  } else if (k == "MaxPoolForward") {
    // benchmark config 1 (3x3, stride 2, pad 1 over 112x112) or, next to the histogram, config 3 (2x2 over 64x64)
    const bool k2 = second_of_hist_pair;
    const int n = small ? 2 : (k2 ? 16 : 32), c = small ? 4 : (k2 ? 128 : 64), h = small ? 16 : (k2 ? 64 : 112);
    const int ks = k2 ? 2 : 3, pad = k2 ? 0 : 1, ph = (h + 2 * pad - ks) / 2 + 1;
    Buffer *x = add(w->inputs, (size_t)n * c * h * h * 4);
    x->fill_uniform(seed, -1.0f, 1.0f);
    hf_maxpool_args a[2] = {};
    for (int s = 0; s < 2; s++) {
      Buffer *val = add(s ? w->out_fused : w->out_native, (size_t)n * c * ph * ph * 4);
      Buffer *idx = add(s ? w->out_fused : w->out_native, (size_t)n * c * ph * ph * 8);
      a[s].nthreads = n * c * ph * ph; a[s].bottom_data = static_cast<const float *>(x->dev);
      a[s].num = n; a[s].channels = c; a[s].height = a[s].width = h; a[s].pooled_height = a[s].pooled_width = ph;
      a[s].kernel_h = a[s].kernel_w = ks; a[s].stride_h = a[s].stride_w = 2; a[s].pad_h = a[s].pad_w = pad;
      a[s].dilation_h = a[s].dilation_w = 1;
      a[s].top_data = static_cast<float *>(val->dev); a[s].top_mask = static_cast<int64_t *>(idx->dev);
    }
    w->set_args(a[0], a[1]);
    w->bytes = 4.0 * n * c * h * h + 12.0 * n * c * ph * ph;
  } else if (k == "batch_norm_collect_statistics_kernel") {
    const int C = small ? 9 : 256, L = small ? 36 : 784;
    Buffer *x = add(w->inputs, (size_t)N * C * L * 4);
    x->fill_uniform(seed, -3.0f, 4.0f);
    hf_bn_stats_args a[2] = {};
    for (int s = 0; s < 2; s++) {
      Buffer *mean = add(s ? w->out_fused : w->out_native, C * 4), *inv = add(s ? w->out_fused : w->out_native, C * 4);
      a[s].input.data = static_cast<float *>(x->dev);
      a[s].input.sizes[0] = (int)N; a[s].input.sizes[1] = C; a[s].input.sizes[2] = L;
      a[s].input.strides[0] = C * L; a[s].input.strides[1] = L; a[s].input.strides[2] = 1;
      a[s].epsilon = 1e-5f;
      a[s].save_mean.data = static_cast<float *>(mean->dev); a[s].save_mean.sizes[0] = C; a[s].save_mean.strides[0] = 1;
      a[s].save_transformed_var.data = static_cast<float *>(inv->dev); a[s].save_transformed_var.sizes[0] = C;
      a[s].save_transformed_var.strides[0] = 1;
    }
    w->set_args(a[0], a[1]);
    w->bytes = 4.0 * N * C * L + 8.0 * C;
    // the Welford merge tree follows the number of threads, which differs between a native block and
    // a share of a fused block: equal to rounding, not to the bit
    w->tolerance = 1e-5f;
  } else if (k == "upsample_nearest2d_out_frame" || k == "upsample_bilinear2d_out_frame") {
    const int64_t C = small ? 3 : 64, H = small ? 8 : 56, W = H;
    Buffer *x = add(w->inputs, N * C * H * W * 4);
    x->fill_uniform(seed, -1.0f, 1.0f);
    if (k == "upsample_nearest2d_out_frame") {
      hf_upsample_nearest_args a[2] = {};
      for (int s = 0; s < 2; s++) {
        Buffer *o = add(s ? w->out_fused : w->out_native, N * C * H * W * 16);
        a[s].idata = static_cast<const float *>(x->dev); a[s].odata = static_cast<float *>(o->dev);
        a[s].nc = N * C; a[s].height1 = H; a[s].width1 = W; a[s].height2 = 2 * H; a[s].width2 = 2 * W;
        a[s].height_scale = a[s].width_scale = 0.5f;
      }
      w->set_args(a[0], a[1]);
    } else {
      hf_upsample_bilinear_args a[2] = {};
      for (int s = 0; s < 2; s++) {
        Buffer *o = add(s ? w->out_fused : w->out_native, N * C * H * W * 16);
        a[s].n = (int)(4 * H * W); a[s].rheight = a[s].rwidth = 0.5f; a[s].align_corners = 0;
        const int64_t si[4] = {N, C, H, W}, so[4] = {N, C, 2 * H, 2 * W};
        for (int d = 0; d < 4; d++) { a[s].idata.sizes[d] = si[d]; a[s].odata.sizes[d] = so[d]; }
        a[s].idata.strides[3] = 1; a[s].idata.strides[2] = W; a[s].idata.strides[1] = H * W; a[s].idata.strides[0] = C * H * W;
        a[s].odata.strides[3] = 1; a[s].odata.strides[2] = 2 * W; a[s].odata.strides[1] = 4 * H * W; a[s].odata.strides[0] = 4 * C * H * W;
        a[s].idata.data = static_cast<float *>(x->dev); a[s].odata.data = static_cast<float *>(o->dev);
      }
      w->set_args(a[0], a[1]);
    }
    w->bytes = 4.0 * N * C * H * W * 5;
  } else if (k == "kernelHistogram1D") {
    const int64_t n = small ? 50000 : (int64_t)1 << 26;
    Buffer *x = add(w->inputs, n * 4);
    x->fill_uniform(seed, 0.0f, 1.0f);
    hf_histc_args a[2] = {};
    for (int s = 0; s < 2; s++) {
      Buffer *bins = add(s ? w->out_fused : w->out_native, 1024 * 4);
      a[s].a.data = static_cast<float *>(bins->dev); a[s].a.dims = 1; a[s].a.sizes[0] = 1024; a[s].a.strides[0] = 1;
      a[s].b.data = static_cast<float *>(x->dev); a[s].b.dims = 1; a[s].b.sizes[0] = n; a[s].b.strides[0] = 1;
      a[s].nbins = 1024; a[s].minvalue = 0.0f; a[s].maxvalue = 1.0f; a[s].total_elements = n;
    }
    w->set_args(a[0], a[1]);
    w->accumulates = true;
    w->bytes = 4.0 * n + 4096;
  } else {
    // the searches: a result record per output set; constants uploaded here
    const uint32_t threads = small ? 1u << 14 : 1u << 24;
    uint8_t header[80];
    for (int i = 0; i < 80; i++) header[i] = (uint8_t)(splitmix64(seed, i / 8) >> (8 * (i % 8)));
    const uint64_t target = small ? (1ull << 52) - 1 : (1ull << 40) - 1;
    Buffer *res[2] = {add(w->out_native, sizeof(hf_search_results)), add(w->out_fused, sizeof(hf_search_results))};
    w->accumulates = true;
    w->hashes = threads;
    if (k == "ethash_search" || k == "ethash_search2" || k == "ethash_search3" || k == "ethash_search4") {
      const uint32_t items = small ? 1u << 12 : 1u << 22;   // 512 MiB of DAG unless --small
      Buffer *dag = add(w->inputs, (size_t)items * 128);
      hf_check(hf_fill_splitmix64(static_cast<uint64_t *>(dag->dev), (uint64_t)items * 16, seed, nullptr));
      hip_check(hipDeviceSynchronize(), "dag fill");
      hf_check(hf_ethash_set_constants(dag->dev, items, header, small ? (1ull << 54) - 1 : (1ull << 44) - 1, nullptr));   // about 16 hits either way: well under the record's 64 slots
      hf_ethash_args a[2] = {{static_cast<hf_search_results *>(res[0]->dev), 0}, {static_cast<hf_search_results *>(res[1]->dev), 0}};
      w->set_args(a[0], a[1]);
      w->grid = (int)(threads / 128);
    } else if (k == "sha256d_gpu_hash_shared") {
      hf_check(hf_sha256d_set_block(header, target, nullptr));
      hf_sha256d_args a[2] = {{threads, 0, static_cast<uint32_t *>(res[0]->dev)}, {threads, 0, static_cast<uint32_t *>(res[1]->dev)}};
      w->set_args(a[0], a[1]);
    } else if (k == "sia_blake2b_gpu_hash" || k == "blake2b_gpu_hash") {
      hf_check(k[0] == 's' ? hf_sia_blake2b_set_block(header, nullptr) : hf_blake2b_set_block(header, nullptr));
      hf_blake2b_args a[2] = {};
      for (int s = 0; s < 2; s++) {
        a[s].threads = threads; a[s].start_nonce = 0; a[s].res_nonce = static_cast<uint32_t *>(res[s]->dev);
        a[s].target2[0] = (uint32_t)target; a[s].target2[1] = (uint32_t)(target >> 32);
      }
      w->set_args(a[0], a[1]);
    } else {
      throw std::runtime_error("no synthetic workload for kernel '" + k + "'");
    }
  }
  return w;
}

// Search records are appended in arrival order: compare them as sets (sorted by nonce).
bool same_outputs(const Workload &w) {
  for (size_t i = 0; i < w.out_native.size(); i++) {
    auto a = w.out_native[i]->download(), b = w.out_fused[i]->download();
    if (w.hashes > 0) {
      auto sort_hits = [](std::vector<unsigned char> &raw) {
        auto *r = reinterpret_cast<hf_search_results *>(raw.data());
        const uint32_t n = r->count < HF_MAX_SEARCH_RESULTS ? r->count : HF_MAX_SEARCH_RESULTS;
        for (uint32_t x = 1; x < n; x++)
          for (uint32_t y = x; y > 0 && r->hit[y].nonce < r->hit[y - 1].nonce; y--) std::swap(r->hit[y], r->hit[y - 1]);
        std::memset(static_cast<void *>(r->hit + n), 0, sizeof(hf_search_hit) * (HF_MAX_SEARCH_RESULTS - n));
      };
      sort_hits(a);
      sort_hits(b);
    }
    if (w.tolerance > 0.0f) {
      const float *fa = reinterpret_cast<const float *>(a.data()), *fb = reinterpret_cast<const float *>(b.data());
      for (size_t k = 0; k < a.size() / 4; k++)
        if (!(std::fabs(fa[k] - fb[k]) <= w.tolerance * std::fmax(std::fabs(fa[k]), std::fabs(fb[k])))) return false;
    } else if (a != b) {
      return false;
    }
  }
  return true;
}

// One pair: a compared launch of each form on identical inputs, then timed repetitions.
// Returns the speedup of the fused kernel over back to back in percent; `ok` = outputs agree.
double run_pair(hf_config *cfg, int index, const std::string &preset, int split, int iters, bool small, bool &ok) {
  const char *file = "", *k1 = "", *k2 = "";
  hf_check(hf_config_fusion(cfg, index, &file, &k1, &k2));
  hf_plan *plan = nullptr;
  hf_check(hf_plan_create(cfg, index, preset.c_str(), split, 0, &plan));
  hf_partition part;
  hf_check(hf_plan_partition(plan, &part));
  std::printf("%s: %s + %s as %s (%u threads: [%u,%u) + [%u,%u))\n", file, k1, k2, part.name, part.launch_threads,
              part.lo[0], part.hi[0], part.lo[1], part.hi[1]);

  const bool hist_pair = std::string(k1) == "kernelHistogram1D";
  auto w1 = make_workload(k1, false, small, 0x48467573ull);
  auto w2 = make_workload(k2, hist_pair, small, 0x48467574ull);
  // ethash scans grid * (its block) nonces: natively 128-thread blocks, fused its share of the block
  const int native_grid = w1->grid ? w1->grid : w2->grid;
  int fused_grid = 0;
  if (w1->grid) fused_grid = (int)(w1->hashes / (part.hi[0] - part.lo[0]));
  if (w2->grid) fused_grid = (int)(w2->hashes / (part.hi[1] - part.lo[1]));

  w1->reset();
  w2->reset();
  hip_check(hipDeviceSynchronize(), "reset");
  hf_check(hf_launch_native(k1, w1->args_native.data(), w1->grid, 0, nullptr));
  hf_check(hf_launch_native(k2, w2->args_native.data(), w2->grid, 0, nullptr));
  hf_check(hf_launch_fused(plan, w1->args_fused.data(), w2->args_fused.data(), fused_grid, nullptr));
  hip_check(hipDeviceSynchronize(), "compared launches");
  const bool ok1 = same_outputs(*w1), ok2 = same_outputs(*w2);
  std::printf("fused == native: %s %s, %s %s\n", k1, ok1 ? "yes" : "NO", k2, ok2 ? "yes" : "NO");  // batch-norm: to 1e-5 relative

  // timed repetitions: A, B, A then B, fused
  const void *a1[1] = {w1->args_native.data()}, *a2[1] = {w2->args_native.data()};
  const char *label[4] = {k1, k2, "back to back", part.name};
  float ms[4];
  for (int mode = 0; mode < 4; mode++) {
    hf_check(hf_time_pair(plan, mode, a1, a2, 1, 0, 2, iters, mode == 3 ? fused_grid : native_grid, nullptr, &ms[mode]));
    std::printf("%-60s %10.3f us per launch\n", label[mode], 1e3 * ms[mode] / iters);
  }
  const double speedup = (ms[2] / ms[3] - 1.0) * 100.0;
  std::printf("speedup of the fused kernel over back to back: %+.1f %%\n", speedup);
  hf_plan_free(plan);
  ok = ok1 && ok2;
  return speedup;
}

// A three-kernel entry (the reference's configs/crypt_four.yaml, im2col_maxpool_norm.yaml, maxpool_summary_norm.yaml):
// the three native kernels, then the one fused kernel, on identical inputs; outputs compared; both forms timed.
double run_triple(hf_config *cfg, int index, const std::string &preset, int split, int iters, bool small, bool &ok) {
  const char *names[3] = {"", "", ""};
  for (int k = 0; k < 3; k++) hf_check(hf_config_fusion_kernel(cfg, index, k, &names[k]));
  hf_plan *plan = nullptr;
  hf_check(hf_plan_create(cfg, index, preset.c_str(), split, 0, &plan));
  hf_partition_n part;
  hf_check(hf_plan_partition_n(plan, &part));
  std::printf("%s + %s + %s as %s (%u threads: [%u,%u) + [%u,%u) + [%u,%u))\n", names[0], names[1], names[2], part.name,
              part.launch_threads, part.lo[0], part.hi[0], part.lo[1], part.hi[1], part.lo[2], part.hi[2]);
  bool with_hist = false;
  for (int k = 0; k < 3; k++) with_hist = with_hist || std::string(names[k]) == "kernelHistogram1D";
  std::unique_ptr<Workload> w[3];
  int native_grid = 0, fused_grid = 0;
  for (int k = 0; k < 3; k++) {
    w[k] = make_workload(names[k], with_hist && std::string(names[k]) == "MaxPoolForward", small, 0x48467573ull + k);
    if (w[k]->grid) {   // ethash scans grid * (its block) nonces: natively 128-thread blocks, fused its share of the block
      native_grid = w[k]->grid;
      fused_grid = (int)(w[k]->hashes / (part.hi[k] - part.lo[k]));
    }
    w[k]->reset();
  }
  hip_check(hipDeviceSynchronize(), "reset");
  const void *fused_args[3], *native_args[3];
  for (int k = 0; k < 3; k++) {
    hf_check(hf_launch_native(names[k], w[k]->args_native.data(), w[k]->grid, 0, nullptr));
    fused_args[k] = w[k]->args_fused.data();
    native_args[k] = w[k]->args_native.data();
  }
  hf_check(hf_launch_fused_n(plan, fused_args, 3, fused_grid, nullptr));
  hip_check(hipDeviceSynchronize(), "compared launches");
  ok = true;
  for (int k = 0; k < 3; k++) {
    const bool same = same_outputs(*w[k]);
    std::printf("fused == native: %s %s\n", names[k], same ? "yes" : "NO");
    ok = ok && same;
  }
  float ms[2];
  hf_check(hf_time_fused_n(plan, 2, native_args, 3, 1, 0, 2, iters, native_grid, nullptr, &ms[0]));
  hf_check(hf_time_fused_n(plan, 3, native_args, 3, 1, 0, 2, iters, fused_grid, nullptr, &ms[1]));
  std::printf("%-60s %10.3f us per launch\n", "three native launches back to back", 1e3 * ms[0] / iters);
  std::printf("%-60s %10.3f us per launch\n", part.name, 1e3 * ms[1] / iters);
  const double speedup = (ms[0] / ms[1] - 1.0) * 100.0;
  std::printf("speedup of the fused kernel over back to back: %+.1f %%\n", speedup);
  hf_plan_free(plan);
  return speedup;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc < 4) {
    std::fprintf(stderr, "usage: %s <fusion.yaml> <kernels.yaml> <File name | index | all> [--preset P] [--split N] [--iters N] [--small]\n", argv[0]);
    return 2;
  }
  std::string preset = "hfuse";
  int split = HF_SPLIT_TABLE, iters = 20;
  bool small = false;
  for (int i = 4; i < argc; i++) {
    const std::string o = argv[i];
    if (o == "--small") small = true;
    else if (o == "--preset" && i + 1 < argc) preset = argv[++i];
    else if (o == "--split" && i + 1 < argc) split = std::atoi(argv[++i]);
    else if (o == "--iters" && i + 1 < argc) iters = std::atoi(argv[++i]);
    else { std::fprintf(stderr, "unknown option %s\n", o.c_str()); return 2; }
  }
  try {
    hf_config *cfg = nullptr;
    hf_check(hf_config_load_files(argv[1], argv[2], &cfg));
    const std::string which = argv[3];
    const int n = hf_config_num_fusions(cfg);
    std::vector<int> todo;
    for (int i = 0; i < n; i++) {
      const char *file = "", *k1 = "", *k2 = "";
      hf_check(hf_config_fusion(cfg, i, &file, &k1, &k2));
      const int size = hf_config_fusion_size(cfg, i);
      if (which == "all" ? (size == 2 || size == 3) : (which == file || std::to_string(i) == which)) {
        todo.push_back(i);
        if (which != "all") break;
      }
    }
    if (todo.empty()) throw std::runtime_error("no fusion '" + which + "' in " + argv[1]);
    bool all_ok = true;
    std::vector<std::pair<std::string, double>> summary;
    for (int index : todo) {
      bool ok = false;
      const double speedup = hf_config_fusion_size(cfg, index) == 3 ? run_triple(cfg, index, preset, split, iters, small, ok)
                                                                   : run_pair(cfg, index, preset, split, iters, small, ok);
      all_ok = all_ok && ok;
      const char *file = "", *k1 = "", *k2 = "";
      hf_check(hf_config_fusion(cfg, index, &file, &k1, &k2));
      summary.emplace_back(std::string(file) + (ok ? "" : "  (OUTPUTS DIFFER)"), speedup);
    }
    if (todo.size() > 1) {
      std::printf("\n%-40s %s\n", "pair", "fused over back to back");
      for (const auto &row : summary) std::printf("%-40s %+6.1f %%\n", row.first.c_str(), row.second);
    }
    hf_config_free(cfg);
    return all_ok ? 0 : 1;
  } catch (const std::exception &e) {
    std::fprintf(stderr, "hfuse-launch: %s\n", e.what());
    return 1;
  }
}
