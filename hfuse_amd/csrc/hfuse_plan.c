/*
 * hfuse-plan: what the reference's command line printed, without the rewriting.
 *
 * `llvm-smart-fuser <fusion.yaml> <kernels.yaml> <dir>` walks every pair of the
 * fusion list, every preset (vfuse_lb, vfuse, hfuse, hfuse_lb: tools/llvm-smart-fuser/
 * main.cpp:182-193) and, for the horizontal presets, every split 128*(n+1) < d1+d2
 * (main.cpp:215-227), and emits one fused kernel per variant.  This program walks
 * the same enumeration through the C-ABI and prints one line per variant: the fused
 * kernel's name, each kernel's thread bounds and block shape, the launch block and
 * the launch-bounds hint -- the numbers a caller needs to launch the variant with
 * hf_plan_create + hf_launch_fused (hf_launch_fused_n for an entry of three kernels,
 * whose lines carry three bounds and three block shapes).
 *
 * Plain C99 against include/hfuse_gfx950.h only (it doubles as the check that the
 * header is a C header).  Needs no GPU.
 *
 *   hfuse-plan <fusion.yaml> <kernels.yaml>         all variants, tab separated
 *   hfuse-plan -                <kernels.yaml>         older per-pair table (no fusion list)
 */
#include <stdio.h>
#include <string.h>

#include "../../include/hfuse_gfx950.h"

static const char *const kPresets[] = {"vfuse_lb", "vfuse", "hfuse", "hfuse_lb"};
static const char *const kBarrier[] = {"none", "matched", "subset", "blockidx"};

static int print_variant(const hf_config *cfg, int fusion, const char *file, const char *preset, int split_idx) {
  hf_plan *plan = NULL;
  hf_partition_n p;
  int k;
  int rc = hf_plan_create(cfg, fusion, preset, split_idx, 0, &plan);
  if (rc != HF_OK) {
    /* the reference prints the problem and goes on to the next variant (main.cpp:69-71) */
    printf("# %s\t%s\tidx %d\t%s\n", file, preset, split_idx, hf_last_error());
    return rc;
  }
  rc = hf_plan_partition_n(plan, &p);
  if (rc == HF_OK) {
    /* one bounds column and one block-shape column per kernel: two of each for a pair, three for a three-kernel entry */
    printf("%s\t%s\t%s\t%d", file, p.name, preset, split_idx);
    for (k = 0; k < p.n; k++) printf("\t[%u,%u)", p.lo[k], p.hi[k]);
    for (k = 0; k < p.n; k++) printf("\t%ux%ux%u", p.block_dim[k].x, p.block_dim[k].y, p.block_dim[k].z);
    printf("\t%u\t%u\t%s\n", p.launch_threads, p.launch_blocks, kBarrier[p.barrier_mode & 3]);
  }
  hf_plan_free(plan);
  return rc;
}

int main(int argc, char **argv) {
  hf_config *cfg = NULL;
  int n, i, failures = 0;
  if (argc != 3) {
    fprintf(stderr, "usage: %s <fusion.yaml | -> <kernels.yaml>\n", argv[0]);
    return 2;
  }
  if (hf_config_load_files(strcmp(argv[1], "-") == 0 ? NULL : argv[1], argv[2], &cfg) != HF_OK) {
    fprintf(stderr, "%s\n", hf_last_error());
    return 1;
  }
  n = hf_config_num_fusions(cfg);
  printf("# file\tname\tpreset\tsplit_idx\tbounds1\tbounds2\tblockdim1\tblockdim2\tlaunch_threads\tlaunch_blocks\tbarrier\n");
  printf("# (entries of three kernels: bounds1..3, blockdim1..3)\n");
  for (i = 0; i < n; i++) {
    const char *file = "", *k1 = "", *k2 = "";
    size_t pi;
    if (hf_config_fusion(cfg, i, &file, &k1, &k2) != HF_OK) {
      fprintf(stderr, "%s\n", hf_last_error());
      failures++;
      continue;
    }
    for (pi = 0; pi < sizeof kPresets / sizeof kPresets[0]; pi++) {
      const int horizontal = strncmp(kPresets[pi], "hfuse", 5) == 0;
      const int splits = horizontal ? hf_plan_num_splits(cfg, i) : 0;
      int s;
      if (!horizontal || splits <= 0) {
        /* vertical presets have one variant (idx 0, main.cpp:232-235) */
        failures += print_variant(cfg, i, file, kPresets[pi], horizontal ? HF_SPLIT_TABLE : 0) != HF_OK;
        continue;
      }
      for (s = 0; s < splits; s++) failures += print_variant(cfg, i, file, kPresets[pi], s) != HF_OK;
    }
  }
  hf_config_free(cfg);
  return failures ? 1 : 0;
}
