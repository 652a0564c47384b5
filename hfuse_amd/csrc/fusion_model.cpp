#include "fusion_model.h"

#include <algorithm>
#include <cstdlib>

#include "../../include/hfuse_gfx950.h"
#include "yaml_lite.h"

namespace hfuse {
namespace {

const Preset kPresets[] = {
    // name        BaseLine BarSync LaunchBound ImBalanced   (main.cpp:182-193)
    {"vfuse_lb", true, false, true, false},
    {"vfuse", true, false, false, false},
    {"hfuse", false, false, false, true},
    {"hfuse_lb", false, false, true, true},
};

bool to_uint(const YamlNode *n, uint32_t &out) {
  if (!n || n->kind != YamlNode::Scalar || n->scalar.empty()) return false;
  char *end = nullptr;
  unsigned long v = std::strtoul(n->scalar.c_str(), &end, 10);
  if (*end != 0 || n->scalar[0] == '-') return false;
  out = (uint32_t)v;
  return true;
}

bool to_bool(const YamlNode *n, bool &out) {
  if (!n || n->kind != YamlNode::Scalar) return false;
  std::string s = n->scalar;
  std::transform(s.begin(), s.end(), s.begin(), ::tolower);
  if (s == "true" || s == "yes" || s == "on") { out = true; return true; }
  if (s == "false" || s == "no" || s == "off") { out = false; return true; }
  return false;
}

std::string at(const YamlNode &n) { return "line " + std::to_string(n.line) + ": "; }

// One kernel row.  Map form: all of KernelName/HasBarriers/BlockDim/Reg are required
// (KernelFusion.h:131-137); the older list form was written without Reg.
bool parse_row(const YamlNode &n, bool reg_required, KernelRow &row, std::string &err) {
  if (n.kind != YamlNode::Map) { err = at(n) + "kernel row must be a mapping"; return false; }
  const YamlNode *name = n.get("KernelName");
  if (!name || name->kind != YamlNode::Scalar || name->scalar.empty()) {
    err = at(n) + "missing required key 'KernelName'";
    return false;
  }
  row.name = name->scalar;
  if (!to_bool(n.get("HasBarriers"), row.has_barriers)) {
    err = at(n) + "missing or invalid required key 'HasBarriers'";
    return false;
  }
  const YamlNode *bd = n.get("BlockDim");
  if (!bd || bd->kind != YamlNode::Map || !to_uint(bd->get("X"), row.block_dim.x) ||
      !to_uint(bd->get("Y"), row.block_dim.y) || !to_uint(bd->get("Z"), row.block_dim.z)) {
    err = at(n) + "missing or invalid required key 'BlockDim' {X, Y, Z}";
    return false;
  }
  // A block of zero threads divides by zero further on; more than 1024 cannot be launched.
  if (row.block_dim.x == 0 || row.block_dim.y == 0 || row.block_dim.z == 0 || row.block_dim.x > kMaxBlock ||
      row.block_dim.y > kMaxBlock || row.block_dim.z > kMaxBlock ||
      (uint64_t)row.block_dim.x * row.block_dim.y * row.block_dim.z > kMaxBlock) {
    err = at(*bd) + "'BlockDim' must be 1..1024 threads in total, no component 0";
    return false;
  }
  const YamlNode *reg = n.get("Reg");
  if (reg) {
    if (!to_uint(reg, row.reg)) { err = at(n) + "invalid 'Reg'"; return false; }
  } else if (reg_required) {
    err = at(n) + "missing required key 'Reg'";
    return false;
  }
  const YamlNode *et = n.get("ExecTime");
  row.exec_time = -1.0;
  if (et) {
    char *end = nullptr;
    row.exec_time = std::strtod(et->scalar.c_str(), &end);
    if (et->kind != YamlNode::Scalar || et->scalar.empty() || *end != 0) {
      err = at(n) + "invalid 'ExecTime'";
      return false;
    }
  }
  // Not in the reference's schema: the block the unfused kernel is launched with on this GPU, where that
  // is not BlockDim (which stays the basis of the split enumeration and must keep pair totals within 1024).
  if (const YamlNode *nt = n.get("NativeThreads")) {
    if (!to_uint(nt, row.native_threads) || row.native_threads == 0 || row.native_threads % kWave != 0 ||
        row.native_threads > kMaxBlock) {
      err = at(*nt) + "'NativeThreads' must be a multiple of 64 between 64 and 1024";
      return false;
    }
  }
  for (auto &kv : n.map) {
    const std::string &k = kv.first;
    if (k != "KernelName" && k != "HasBarriers" && k != "BlockDim" && k != "Reg" && k != "ExecTime" &&
        k != "NativeThreads") {
      err = at(kv.second) + "unknown key '" + k + "'";
      return false;
    }
  }
  return true;
}

}  // namespace

const KernelRow *Config::find(const std::string &key) const {
  for (auto &r : rows)
    if (r.key == key) return &r;
  return nullptr;
}

const Preset *find_preset(const std::string &name) {
  for (auto &p : kPresets)
    if (name == p.name) return &p;
  return nullptr;
}

bool parse_config(const char *fusion_yaml, const char *kernels_yaml, Config &cfg, std::string &err) {
  cfg = Config();
  if (!kernels_yaml) { err = "kernel table is null"; return false; }
  YamlNode kroot;
  if (!yaml_parse(kernels_yaml, kroot, err)) { err = "kernel table: " + err; return false; }
  if (kroot.kind == YamlNode::Map) {
    for (auto &kv : kroot.map) {
      KernelRow row;
      row.key = kv.first;
      if (!parse_row(kv.second, true, row, err)) { err = "kernel table: " + err; return false; }
      cfg.rows.push_back(row);
    }
  } else if (kroot.kind == YamlNode::Seq) {
    for (auto &n : kroot.seq) {
      KernelRow row;
      if (!parse_row(n, false, row, err)) { err = "kernel table: " + err; return false; }
      row.key = row.name;
      if (cfg.find(row.key)) { err = "kernel table: duplicate kernel '" + row.key + "'"; return false; }
      cfg.rows.push_back(row);
    }
  } else {
    err = "kernel table: expected a mapping of kernels or a list of kernel rows";
    return false;
  }
  if (cfg.rows.empty()) { err = "kernel table: no kernels"; return false; }

  if (!fusion_yaml) {
    if (kroot.kind != YamlNode::Seq) { err = "fusion list is null"; return false; }
    FusionRow f;
    for (auto &r : cfg.rows) f.kernels.push_back(r.key);
    cfg.fusions.push_back(f);
  } else {
    YamlNode froot;
    if (!yaml_parse(fusion_yaml, froot, err)) { err = "fusion list: " + err; return false; }
    if (froot.kind != YamlNode::Seq) { err = "fusion list: expected a sequence of {File, Kernels}"; return false; }
    for (auto &n : froot.seq) {
      FusionRow f;
      const YamlNode *file = n.kind == YamlNode::Map ? n.get("File") : nullptr;
      const YamlNode *ks = n.kind == YamlNode::Map ? n.get("Kernels") : nullptr;
      if (!file || file->kind != YamlNode::Scalar) { err = "fusion list: " + at(n) + "missing required key 'File'"; return false; }
      if (!ks || ks->kind != YamlNode::Seq) { err = "fusion list: " + at(n) + "missing required key 'Kernels'"; return false; }
      f.file = file->scalar;
      if (const YamlNode *sp = n.get("Split")) {
        // not in the reference's schema: a tuned default for the thread partition of this pair
        if (!to_uint(sp, f.split) || f.split == 0 || f.split % kWave != 0) {
          err = "fusion list: " + at(*sp) + "'Split' must be a positive multiple of 64 threads";
          return false;
        }
      }
      if (const YamlNode *th = n.get("Threads")) {
        if (!to_uint(th, f.threads) || f.threads % kWave != 0 || f.threads > kMaxBlock || f.split == 0 ||
            f.threads <= f.split) {
          err = "fusion list: " + at(*th) + "'Threads' must be a multiple of 64, at most 1024 and larger than 'Split'";
          return false;
        }
      }
      if (const YamlNode *ln = n.get("Lending")) {
        if (ln->kind == YamlNode::Scalar && (ln->scalar == "true" || ln->scalar == "1")) f.lending = 1;
        else if (ln->kind == YamlNode::Scalar && (ln->scalar == "false" || ln->scalar == "0")) f.lending = 0;
        else { err = "fusion list: " + at(*ln) + "'Lending' must be true or false"; return false; }
      }
      if (const YamlNode *lb = n.get("LaunchBound")) {
        if (lb->kind == YamlNode::Scalar && (lb->scalar == "true" || lb->scalar == "1")) f.launch_bound = 1;
        else if (lb->kind == YamlNode::Scalar && (lb->scalar == "false" || lb->scalar == "0")) f.launch_bound = 0;
        else { err = "fusion list: " + at(*lb) + "'LaunchBound' must be true or false"; return false; }
      }
      if (const YamlNode *bn = n.get("Barrier")) {
        static const char *const kModes[] = {"none", "matched", "subset", "blockidx"};  // HF_BARRIER_* order
        for (int m = 0; m < 4; m++)
          if (bn->kind == YamlNode::Scalar && bn->scalar == kModes[m]) f.barrier = m;
        if (f.barrier < 0) {
          err = "fusion list: " + at(*bn) + "'Barrier' must be one of none, matched, subset, blockidx";
          return false;
        }
      }
      if (const YamlNode *bl = n.get("Blocks")) {
        // not in the reference's schema: one thread count per kernel -- the block shape of a three-kernel entry, or
        // of a pair under a vertical preset
        if (bl->kind != YamlNode::Seq || bl->seq.size() != ks->seq.size() || (ks->seq.size() != 3 && ks->seq.size() != 2)) {
          err = "fusion list: " + at(*bl) + "'Blocks' must list one thread count per kernel of a pair or a three-kernel entry";
          return false;
        }
        for (auto &b : bl->seq) {
          uint32_t t = 0;
          if (!to_uint(&b, t) || t == 0 || t % kWave != 0 || t > kMaxBlock) {
            err = "fusion list: " + at(b) + "'Blocks' entries must be multiples of 64 between 64 and 1024";
            return false;
          }
          f.blocks.push_back(t);
        }
      }
      if (const YamlNode *pr = n.get("Preset")) {
        // not in the reference's schema: which of the driver's four presets (main.cpp:182-193) this entry ships with
        if (pr->kind != YamlNode::Scalar || !find_preset(pr->scalar)) {
          err = "fusion list: " + at(*pr) + "'Preset' must be one of vfuse_lb, vfuse, hfuse, hfuse_lb";
          return false;
        }
        f.preset = pr->scalar;
      }
      if (const YamlNode *gr = n.get("Grids")) {
        uint32_t g0 = 0, g1 = 0;
        if (gr->kind != YamlNode::Seq || gr->seq.size() != 2 || ks->seq.size() != 2 || !to_uint(&gr->seq[0], g0) ||
            !to_uint(&gr->seq[1], g1) || g0 > (1u << 24) || g1 > (1u << 24)) {
          err = "fusion list: " + at(*gr) + "'Grids' must list two workgroup counts (0 = the library's) of a pair";
          return false;
        }
        f.grids[0] = g0;
        f.grids[1] = g1;
      }
      for (auto &kv : n.map)
        if (kv.first != "File" && kv.first != "Kernels" && kv.first != "Split" && kv.first != "Threads" &&
            kv.first != "Lending" && kv.first != "Barrier" && kv.first != "LaunchBound" && kv.first != "Blocks" &&
            kv.first != "Preset" && kv.first != "Grids") {
          err = "fusion list: " + at(kv.second) + "unknown key '" + kv.first + "'";
          return false;
        }
      for (auto &k : ks->seq) {
        if (k.kind != YamlNode::Scalar) { err = "fusion list: " + at(k) + "kernel name must be a scalar"; return false; }
        f.kernels.push_back(k.scalar);
      }
      cfg.fusions.push_back(f);
    }
  }
  for (auto &f : cfg.fusions) {
    // (the schema allows any number of kernels, include/KernelFusion.h:140-146; plans are built for pairs)
    if (f.kernels.empty()) { err = "fusion '" + f.file + "': no kernels"; return false; }
    for (auto &k : f.kernels)
      if (!cfg.find(k)) { err = "fusion '" + f.file + "': kernel '" + k + "' is not in the kernel table"; return false; }
  }
  return true;
}

int num_splits(const KernelRow &k1, const KernelRow &k2) {
  uint32_t end = k1.block_dim.size() + k2.block_dim.size();
  int n = 0;
  for (uint32_t split = 128; split < end; split += 128) n++;
  return n;
}

int make_partition(const KernelRow &k1, const KernelRow &k2, const Preset &preset, int split_idx,
                   int split_threads, Partition &out, std::string &err) {
  const KernelRow *rows[2] = {&k1, &k2};
  Dim3 dims[2] = {k1.block_dim, k2.block_dim};
  const uint32_t total = dims[0].size() + dims[1].size();
  if (dims[0].size() == 0 || dims[1].size() == 0) { err = "empty BlockDim"; return HF_EINVAL; }
  std::string variant = preset.name;

  if (!preset.base_line) {
    uint32_t first = dims[0].size();
    bool resplit = false;
    if (split_threads > 0) {
      first = (uint32_t)split_threads;
      resplit = true;
      variant += "_split_" + std::to_string(first);
    } else if (split_idx >= 0 || split_idx == HF_SPLIT_EXECTIME) {
      // Context's imbalanced re-split (KernelFusion.h:63-72) with the wavefront as granule.
      double e0, e1;
      if (split_idx >= 0) {
        if (split_idx >= num_splits(k1, k2)) { err = "split index beyond the enumeration 128*(n+1) < d1+d2"; return HF_EINVAL; }
        e0 = 128.0 * (split_idx + 1);  // main.cpp:224-225
        e1 = (double)total - e0;
        variant += "_idx_" + std::to_string(split_idx);
      } else {
        e0 = k1.exec_time;
        e1 = k2.exec_time;
        if (!(e0 > 0) || !(e1 > 0)) { err = "ExecTime split requested but the table has no ExecTime"; return HF_EINVAL; }
        variant += "_exectime";
      }
      first = (uint32_t)((int)(e0 / (e0 + e1) * total / kWave)) * kWave;
      resplit = true;
    } else {
      variant += "_table";
    }
    if (resplit) {
      if (first == 0 || first >= total) { err = "split leaves one kernel without threads"; return HF_EINVAL; }
      uint32_t parts[2] = {first, total - first};
      for (int i = 0; i < 2; i++) {
        if (dims[i].y == 0 || dims[i].z != 1 || parts[i] % dims[i].y != 0) {
          err = "split of " + std::to_string(parts[i]) + " threads does not divide by BlockDim.Y of '" + rows[i]->name + "'";
          return HF_EINVAL;
        }
        dims[i].x = parts[i] / dims[i].y;  // KernelFusion.h:72
      }
    }
    for (int i = 0; i < 2; i++) {
      if (dims[i].size() % kWave != 0) {
        err = "part of '" + rows[i]->name + "' is " + std::to_string(dims[i].size()) + " threads: not a multiple of the 64-lane wavefront";
        return HF_EINVAL;
      }
    }
    if (dims[0].size() + dims[1].size() > kMaxBlock) {
      err = "fused block of " + std::to_string(dims[0].size() + dims[1].size()) + " threads exceeds 1024";
      return HF_EINVAL;
    }
  } else {
    variant += "_idx_0";  // main.cpp:218-219,223: the vertical presets print one variant
    if (std::max(dims[0].size(), dims[1].size()) > kMaxBlock) { err = "block exceeds 1024 threads"; return HF_EINVAL; }
    // the vertical kernel hands each body whole wavefronts too: a ragged BlockDim would leave its last lanes' items undone
    for (int i = 0; i < 2; i++) {
      if (dims[i].size() % kWave != 0) {
        err = "BlockDim of '" + rows[i]->name + "' is " + std::to_string(dims[i].size()) + " threads: not a multiple of the 64-lane wavefront";
        return HF_EINVAL;
      }
    }
  }

  uint32_t b = 0;
  for (int i = 0; i < 2; i++) {
    out.lo[i] = b;
    out.hi[i] = b + dims[i].size();
    out.block_dim[i] = dims[i];
    if (!preset.base_line) b += dims[i].size();  // KernelFusion.h:76-78
  }
  // KernelPrinter.cpp:46-66
  uint32_t max_thread = 0, max_block = 9999999u, sum = 0;
  for (int i = 0; i < 2; i++) {
    uint32_t size = dims[i].size();
    if (rows[i]->reg) max_block = std::min(kRegFile / rows[i]->reg / size, max_block);
    sum += size;
    max_thread = std::max(max_thread, size);
  }
  max_block = std::min(max_block, kMaxResidentThreads / sum);
  out.launch_threads = preset.base_line ? max_thread : sum;
  out.launch_blocks = preset.launch_bound ? max_block : 0;
  out.bound_blocks = max_block;
  out.name = k1.name + "_" + k2.name + "_fused_kernel_" + variant;  // KernelPrinter.cpp:67-70
  return HF_OK;
}

int make_partition_n(const KernelRow *const *rows, int n, const Preset &preset, int split_idx, Partition &out,
                     std::string &err) {
  if (n < 2 || n > kMaxFuse) { err = "a fused kernel holds two or three kernels"; return HF_EUNSUPPORTED; }
  Dim3 dims[kMaxFuse];
  uint32_t total = 0;
  for (int i = 0; i < n; i++) {
    dims[i] = rows[i]->block_dim;
    if (dims[i].size() == 0) { err = "empty BlockDim"; return HF_EINVAL; }
    total += dims[i].size();
  }
  std::string variant = preset.name;
  if (!preset.base_line && (split_idx >= 0 || split_idx == HF_SPLIT_EXECTIME)) {
    // Context's imbalanced re-split (KernelFusion.h:53-72) with the wavefront as granule.
    double e[kMaxFuse], total_time = 0.0;
    for (int i = 0; i < n; i++) e[i] = rows[i]->exec_time;
    if (split_idx >= 0) {
      const uint32_t end = dims[0].size() + dims[1].size();  // main.cpp:219-225: only the first two vary
      uint32_t count = 0;
      for (uint32_t split = 128; split < end; split += 128) count++;
      if ((uint32_t)split_idx >= count) { err = "split index beyond the enumeration 128*(n+1) < d1+d2"; return HF_EINVAL; }
      e[0] = 128.0 * (split_idx + 1);
      e[1] = (double)end - e[0];
      variant += "_idx_" + std::to_string(split_idx);
    } else {
      for (int i = 0; i < n; i++)
        if (!(e[i] > 0)) { err = "ExecTime split requested but the table has no ExecTime"; return HF_EINVAL; }
      variant += "_exectime";
    }
    for (int i = 0; i < n; i++) total_time += e[i];
    if (!(total_time > 0)) { err = "ExecTimes do not sum to a positive time"; return HF_EINVAL; }
    uint32_t allocated = 0;
    for (int i = 0; i < n; i++) {
      uint32_t part;
      if (i == n - 1) {
        if (allocated >= total) { err = "split leaves one kernel without threads"; return HF_EINVAL; }
        part = total - allocated;
      } else {
        const double share = e[i] / total_time * total / kWave;
        if (!(share >= 1.0) || share > 1e6) { err = "split leaves one kernel without threads"; return HF_EINVAL; }
        part = (uint32_t)((int)share) * kWave;
        allocated += part;
      }
      if (dims[i].z != 1 || part % dims[i].y != 0) {
        err = "split of " + std::to_string(part) + " threads does not divide by BlockDim.Y of '" + rows[i]->name + "'";
        return HF_EINVAL;
      }
      dims[i].x = part / dims[i].y;  // KernelFusion.h:72
    }
  } else if (!preset.base_line) {
    variant += "_table";
  } else {
    variant += "_idx_0";
  }
  uint32_t sum = 0, max_thread = 0, max_block = 9999999u, b = 0;
  for (int i = 0; i < n; i++) {
    const uint32_t size = dims[i].size();
    if (size == 0 || size % kWave != 0) {
      err = "part of '" + rows[i]->name + "' is " + std::to_string(size) + " threads: not a multiple of the 64-lane wavefront";
      return HF_EINVAL;
    }
    out.lo[i] = b;
    out.hi[i] = b + size;
    out.block_dim[i] = dims[i];
    if (!preset.base_line) b += size;  // KernelFusion.h:76-78
    if (rows[i]->reg) max_block = std::min(kRegFile / rows[i]->reg / size, max_block);  // KernelPrinter.cpp:46-60
    sum += size;
    max_thread = std::max(max_thread, size);
  }
  if ((preset.base_line ? max_thread : sum) > kMaxBlock) {
    err = "fused block of " + std::to_string(preset.base_line ? max_thread : sum) + " threads exceeds 1024";
    return HF_EINVAL;
  }
  max_block = std::min(max_block, kMaxResidentThreads / sum);
  out.n = n;
  out.launch_threads = preset.base_line ? max_thread : sum;
  out.launch_blocks = preset.launch_bound ? max_block : 0;
  out.bound_blocks = max_block;
  out.name.clear();
  for (int i = 0; i < n; i++) out.name += rows[i]->name + "_";  // KernelPrinter.cpp:67-70
  out.name += "fused_kernel_" + variant;
  return HF_OK;
}

Dim3 local_index(uint32_t tid, uint32_t lo, const Dim3 &dim) {
  uint32_t t = tid - lo;
  Dim3 r;
  r.x = t % dim.x;
  r.y = t / dim.x % dim.y;
  r.z = t / (dim.x * dim.y);
  return r;
}

}  // namespace hfuse
