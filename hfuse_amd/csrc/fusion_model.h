// Host-side model of a horizontal fusion: the kernel table, the fusion list and
// the thread partition of one fused variant.  Restates, for 64-lane wavefronts,
// the rules of the reference's Context (include/KernelFusion.h:35-92), its split
// enumeration (tools/llvm-smart-fuser/main.cpp:182-227) and the signature
// printer (lib/KernelFuser/KernelPrinter.cpp:42-70).
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace hfuse {

struct Dim3 {
  uint32_t x = 1, y = 1, z = 1;
  uint32_t size() const { return x * y * z; }
};

struct KernelRow {
  std::string key;   // map key (or KernelName in the list form)
  std::string name;  // KernelName
  bool has_barriers = false;
  Dim3 block_dim;
  uint32_t reg = 0;
  double exec_time = -1.0;
  uint32_t native_threads = 0;  // optional `NativeThreads:` key: block of the unfused launch when it is not BlockDim's product
  uint32_t native_block() const { return native_threads ? native_threads : block_dim.x * block_dim.y * block_dim.z; }
};

struct FusionRow {
  std::string file;
  std::vector<std::string> kernels;
  uint32_t split = 0;    // optional `Split:` key: threads of kernel 1 when the caller asks for the table split
  uint32_t threads = 0;  // optional `Threads:` key: threads of the whole fused block (needs Split)
  int lending = -1;      // optional `Lending:` key: 0 / 1 switch wave lending off / on, -1 = library default
  int launch_bound = -1; // optional `LaunchBound:` key: 0 / 1 pick the plain / register-bounded build, -1 = the preset's
  int barrier = -1;      // optional `Barrier:` key: an HF_BARRIER_* mode, -1 = library default
  std::vector<uint32_t> blocks;  // optional `Blocks:` key: threads of each kernel -- the block shape of a three-kernel entry,
                                 // or of a pair under a vertical preset (both bodies start at thread 0)
  std::string preset;            // optional `Preset:` key: the preset this entry ships with ("" = hfuse)
  uint32_t grids[2] = {0, 0};    // optional `Grids:` key of a pair: workgroups each kernel strides over under `Preset` (0 = the library's)
};

struct Config {
  std::vector<KernelRow> rows;  // table order
  std::vector<FusionRow> fusions;
  const KernelRow *find(const std::string &key) const;
};

// The four presets of main.cpp:182-193 as {BaseLine, BarSync, LaunchBound, ImBalancedThread}.
struct Preset {
  const char *name;
  bool base_line, bar_sync, launch_bound, imbalanced;
};
const Preset *find_preset(const std::string &name);

constexpr int kMaxFuse = 3;  // kernels in one fused kernel: pairs, and the three-kernel lists of the reference

struct Partition {
  int n = 2;  // kernels partitioned
  uint32_t lo[kMaxFuse] = {0, 0, 0}, hi[kMaxFuse] = {0, 0, 0};
  Dim3 block_dim[kMaxFuse];
  uint32_t launch_threads = 0, launch_blocks = 0;
  uint32_t bound_blocks = 0;  // the printer's min-blocks value whatever the preset (launch_blocks is 0 without LaunchBound)
  std::string name;  // <K1>_<K2>_fused_kernel_<preset>_idx_<n>
};

// gfx950 constants standing in for KernelPrinter.cpp:10-11 (64K registers, 2048 threads per SM):
// one CU holds 4 SIMDs x 512 VGPRs x 64 lanes and at most 2048 resident work-items.
constexpr uint32_t kRegFile = 4 * 512 * 64;
constexpr uint32_t kMaxResidentThreads = 2048;
constexpr uint32_t kWave = 64;
constexpr uint32_t kMaxBlock = 1024;

bool parse_config(const char *fusion_yaml, const char *kernels_yaml, Config &cfg, std::string &err);

// Number of variants the split loop prints for a horizontal preset (main.cpp:221-223).
int num_splits(const KernelRow &k1, const KernelRow &k2);

// split_threads > 0: explicit size of kernel 1's part; else split_idx >= 0: the reference's
// enumeration (Split = 128*(idx+1)); else (-1) the table's own BlockDim.
// Returns 0, or a negative HF_E* code with `err` set.
int make_partition(const KernelRow &k1, const KernelRow &k2, const Preset &preset, int split_idx,
                   int split_threads, Partition &out, std::string &err);

// The same for a fusion of `n` kernels (the Context partitions a block among any number,
// include/KernelFusion.h:45-80; the driver's split loop still varies only the first two,
// main.cpp:215-227, the others keep the table's ExecTime, -1 when the row has none).
//   split_idx >= 0: ExecTime_0 = 128*(idx+1), ExecTime_1 = (d_0 + d_1) - ExecTime_0, then the re-split
//   in proportion to all ExecTimes, each part rounded down to whole wavefronts, the last takes the rest;
//   HF_SPLIT_EXECTIME: the same with the table's ExecTimes; HF_SPLIT_TABLE: the table's BlockDims.
int make_partition_n(const KernelRow *const *rows, int n, const Preset &preset, int split_idx, Partition &out,
                     std::string &err);

// ThreadInfoRewriter.cpp:38-58
Dim3 local_index(uint32_t tid, uint32_t lo, const Dim3 &dim);

}  // namespace hfuse
