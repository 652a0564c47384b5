/*
 * hfuse_gfx950.h -- C-ABI of the MI355X (gfx950) horizontally fused kernel library.
 *
 * The reference (aoli-al/HFuse) is a source rewriter: its interface for this
 * path is (1) two YAML files, (2) the name / thread partition / argument order
 * of the fused kernel it prints, and (3) the argument lists of the original
 * kernels.  This header is what an external host program binds instead of
 * including the generated `<K1>_<K2>_.inc` text:
 *
 *   - hf_config_*   : the fusion list and kernel table
 *                     (include/KernelFusion.h:129-159, configs/ml_fusion.yaml,
 *                      configs/ml_kernels.yaml, configs/crypto_*.yaml)
 *   - hf_plan_*     : one fused variant = pair x preset x split
 *                     (include/KernelFusion.h:45-80,
 *                      tools/llvm-smart-fuser/main.cpp:182-193,215-227,
 *                      lib/KernelFuser/KernelPrinter.cpp:42-70)
 *   - hf_*_args     : each original kernel's argument list, field for field
 *                     (scripts/data/ml-event.csv, scripts/data/ethminer_event.csv)
 *   - hf_launch_*   : native launch of one kernel, and the fused launch taking
 *                     kernel 1's arguments then kernel 2's
 *                     (lib/KernelFuser/KernelPrinter.cpp:107-115,
 *                      scripts/configs/hist_norm.json:5)
 *
 * All pointers inside argument structs are caller-owned device memory; the
 * library allocates no device memory.  Every call returns 0 or a negative
 * HF_E* code and never throws; hf_last_error() gives the text for the calling
 * thread.  Launches are asynchronous on the caller's hipStream_t (passed as
 * void*; NULL is the default stream).
 */
#ifndef HFUSE_GFX950_H
#define HFUSE_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HF_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ errors */
enum {
  HF_OK = 0,
  HF_EINVAL = -1,      /* bad argument (null pointer, bad shape, bad split ...) */
  HF_EPARSE = -2,      /* YAML does not follow the reference schema            */
  HF_ENOTFOUND = -3,   /* unknown kernel / pair / preset                       */
  HF_EUNSUPPORTED = -4,/* legal in the reference, not built here               */
  HF_EHIP = -5,        /* a HIP runtime call failed                            */
  HF_EIO = -6,         /* file could not be read                               */
  HF_ENOMEM = -7       /* host allocation failed (or another C++ exception)    */
};

HF_API const char *hf_last_error(void);
HF_API int hf_version(void);

/* ------------------------------------------------------------ configuration */
typedef struct hf_config hf_config;

typedef struct {
  uint32_t x, y, z;
} hf_dim3;

/* One row of the kernel table: include/KernelFusion.h:21-27,129-138. */
typedef struct {
  char kernel_name[96];
  int has_barriers;
  hf_dim3 block_dim;
  uint32_t reg;
  double exec_time; /* -1 when the YAML has no ExecTime */
  uint32_t native_threads; /* block of the unfused launch: BlockDim's product unless the row has NativeThreads */
} hf_kernel_info;

/*
 * Parse the two YAML documents of the reference's CLI
 * (tools/llvm-smart-fuser/main.cpp:263-270): a sequence of {File, Kernels}
 * and a string-keyed map of kernel rows.  `kernels_yaml` may also be the older
 * per-pair form, a bare sequence of rows (configs/im2col_maxpool.yaml); then
 * `fusion_yaml` may be NULL and the single fusion is that list in order.
 * Block and flow sequences are both read (`Kernels: [a, b]`).
 * Keys beyond the reference's schema are accepted in a fusion entry (the split
 * tuner writes them); all of them apply to plans created with HF_SPLIT_TABLE and
 * no explicit split_threads -- a plan of an explicit variant starts from the
 * library's defaults:
 *   `Split: <threads>`    kernel 1's share of the thread partition's block, and
 *   `Threads: <threads>`  the size of that block (kernel 2 gets Threads - Split);
 *   `Lending: true|false` the plan's default for hf_plan_set_lending;
 *   `Barrier: none|matched|subset|blockidx` the one for hf_plan_set_barrier_mode
 *                         (an illegal mode fails hf_plan_create);
 *   `LaunchBound: true|false` the one for hf_plan_set_launch_bound;
 *   `Preset: <preset>`    the preset the entry ships with, which a plan created
 *                         with the preset "shipped" gets (the reference prints
 *                         all four presets and the user keeps the fastest,
 *                         main.cpp:182-193; without the key: hfuse);
 *   `Blocks: [t1, t2]`    the threads that run each body under a vertical preset
 *                         (for a three-kernel entry: the block shape, one count
 *                         per kernel);
 *   `Grids: [g1, g2]`     the workgroups each kernel of a pair strides over under
 *                         the entry's own preset (hf_plan_set_grids; 0 = the
 *                         library's choice).
 * A kernel row may carry one extra key, `NativeThreads: <threads>` (a multiple of 64, at most 1024): the
 * block the unfused kernel is launched with by hf_time_pair when that differs from BlockDim, which stays
 * the basis of the split enumeration (the histogram runs fastest alone at 768 threads, and BlockDim 768
 * would push its pairs' totals d1 + d2 beyond 1024).
 */
HF_API int hf_config_load_text(const char *fusion_yaml, const char *kernels_yaml, hf_config **out);
HF_API int hf_config_load_files(const char *fusion_path, const char *kernels_path, hf_config **out);
HF_API void hf_config_free(hf_config *cfg);
HF_API int hf_config_num_fusions(const hf_config *cfg);
HF_API int hf_config_num_kernels(const hf_config *cfg);
/*
 * Names of the i-th fusion's kernels (NUL-terminated, valid while cfg lives).  The schema lets an
 * entry name any number of kernels (include/KernelFusion.h:140-146; configs/crypt_four.yaml names
 * three): such a list loads, hf_config_fusion gives its first two names (k2 = "" for a single one),
 * hf_config_fusion_size / hf_config_fusion_kernel give all of them.  Plans exist for entries of two
 * and of three kernels; hf_plan_create answers HF_EUNSUPPORTED for any other size.
 */
HF_API int hf_config_fusion(const hf_config *cfg, int i, const char **file, const char **k1,
                            const char **k2);
HF_API int hf_config_fusion_size(const hf_config *cfg, int i);
HF_API int hf_config_fusion_kernel(const hf_config *cfg, int i, int k, const char **name);
HF_API int hf_config_kernel(const hf_config *cfg, const char *name, hf_kernel_info *out);

/* ------------------------------------------------------------------- plans */
typedef struct hf_plan hf_plan;

/*
 * What the Context constructor and the printer decide for one variant
 * (include/KernelFusion.h:45-80, lib/KernelFuser/KernelPrinter.cpp:42-70).
 */
typedef struct {
  char name[256];          /* <K1>_<K2>_fused_kernel_<preset>_idx_<n>           */
  uint32_t lo[2], hi[2];   /* thread bounds of each kernel inside the block      */
  hf_dim3 block_dim[2];    /* per-kernel block shape after the re-split          */
  uint32_t launch_threads; /* d1+d2 (hfuse) or max(d1,d2) (vfuse)                */
  uint32_t launch_blocks;  /* min-blocks hint, 0 when the preset has none        */
  int barrier_mode;        /* HF_BARRIER_* chosen for this pair                  */
} hf_partition;

enum {
  HF_BARRIER_NONE = 0,     /* neither half synchronises                          */
  HF_BARRIER_MATCHED = 1,  /* both halves execute the same s_barrier sequence    */
  HF_BARRIER_SUBSET = 2,   /* LDS-counter barrier among one half's wavefronts    */
  HF_BARRIER_BLOCKIDX = 3  /* fallback: halves live in different workgroups      */
};

#define HF_SPLIT_TABLE (-1)
#define HF_SPLIT_EXECTIME (-2)
#define HF_WAVE 64         /* split granularity (reference: 32, KernelFusion.h:66) */
#define HF_MAX_BLOCK 1024

/*
 * Create a plan for fusion `fusion_index` of `cfg`.
 *   preset    : "hfuse" | "hfuse_lb" | "vfuse" | "vfuse_lb" (main.cpp:182-193), or
 *               "shipped": the one the entry's `Preset:` key names (hfuse without it).
 *               The hfuse presets partition the block's threads between the two
 *               kernels; the vfuse presets are the reference's baseline in which
 *               the same threads run kernel 1 and then kernel 2 (block =
 *               max(d1, d2)).  The _lb variants report the launch_blocks hint
 *               and run the register-bounded build (hf_plan_set_launch_bound).
 *   split_idx : the reference's enumeration index n (Split = 128*(n+1) threads
 *               for kernel 1, main.cpp:216-227); HF_SPLIT_TABLE keeps the
 *               YAML's BlockDim as the split; HF_SPLIT_EXECTIME re-splits in
 *               proportion to the table's ExecTime (KernelFusion.h:63-72).
 *   split_threads : when > 0 overrides split_idx with an explicit thread count
 *               for kernel 1 (must be a multiple of 64).
 * Both parts must be non-empty multiples of 64 and d1+d2 <= 1024.
 */
HF_API int hf_plan_create(const hf_config *cfg, int fusion_index, const char *preset, int split_idx,
                          int split_threads, hf_plan **out);
HF_API void hf_plan_free(hf_plan *plan);
/*
 * Override the barrier design of a plan (HF_BARRIER_*).  The default is
 * HF_BARRIER_NONE when neither body synchronises and HF_BARRIER_SUBSET when
 * one does.  HF_BARRIER_MATCHED is legal when both bodies synchronise (they
 * then share the hardware barrier); HF_BARRIER_BLOCKIDX is always legal.
 */
HF_API int hf_plan_set_barrier_mode(hf_plan *plan, int mode);
/*
 * Per-kernel grids of the fused launch when the caller leaves grid_blocks <= 0:
 * kernel k strides over blocks [0, grid_k) and the launch covers max(grid1, grid2)
 * blocks.  0 keeps the library's choice for that kernel.  (The reference's halves
 * share the launch grid; a half that wants fewer blocks simply ends early in
 * the surplus ones.)  Under a vertical preset this is how a few resident blocks
 * take both kernels' work in turn: with grid_k = the number of CUs every block
 * stays on its CU and its threads loop over kernel 1's work and then kernel 2's.
 */
HF_API int hf_plan_set_grids(hf_plan *plan, int grid1, int grid2);
/*
 * Give the fused block an explicit shape: threads1 for kernel 1 and threads2 for
 * kernel 2 (multiples of 64, sum <= 1024), independent of the kernel table's
 * BlockDim, which stays the native launch shape.  The reference reaches the same
 * freedom through per-pair kernel tables (configs/im2col_maxpool.yaml ...).
 * Under a vertical preset both bodies start at thread 0 (KernelFusion.h:76-78):
 * the two counts are the threads that run each body (each <= 1024) and the block
 * is the larger of them.
 */
HF_API int hf_plan_set_block(hf_plan *plan, int threads1, int threads2);
/*
 * Wave lending (on by default).  When the two halves stride over different numbers
 * of blocks, the blocks beyond the smaller grid have one half without work.  With
 * lending on, that half's wavefronts run the partner's body there (the partner must
 * walk a flat 1-D index range: im2col, max-pool, upsample, SHA-256d, Blake2b), so
 * such a block is d1+d2 threads of the partner.  Off: the idle half's waves end at
 * once, which is what the reference's generated kernel does.  Results are identical.
 */
HF_API int hf_plan_set_lending(hf_plan *plan, int on);
/*
 * Which build of the fused (or vertical) kernel a launch runs.  The reference's *_lb presets
 * print `__launch_bounds__(T, B)` with B = min_k(regfile / Reg_k / size_k), capped by the
 * resident-thread limit (lib/KernelFuser/KernelPrinter.cpp:44-66), so that the compiler keeps
 * the fused kernel's registers within the occupancy the natives had.  On gfx950 that request
 * is a waves-per-SIMD bound, fixed at compile time: w = ceil(B * T / 256) with this part's 128 K
 * registers and 2048 resident threads per CU (B blocks of T threads are B * T / 64 waves on four
 * SIMDs, and all of them have to fit).  Every pair is built plain (bounded only by its launch
 * bound of 1024 or 512 threads, which holds four waves per SIMD) and register-bounded for 8 waves
 * per SIMD (at most 64 vector registers, spilling to a private stack if it must).  The five
 * benchmarked pairs (im2col + max-pool, batch-norm + upsample, histogram + max-pool, SHA-256d +
 * Sia-Blake2b, Ethash + Sia-Blake2b) are built for each of 5, 6, 7 and 8 waves, so whatever block
 * shape a plan of theirs has, a launch-bound preset runs the build bounded at exactly the
 * formula's value; three more pairs of the shipped list have a second build at the value of
 * their shipped shape (im2col + histogram 7, im2col + nearest / bilinear upsampling 6).  A
 * request for w waves runs the smallest built bound that is not below w.  A three-kernel plan
 * has the plain build and, for the launch-bound presets, one bounded for 8 waves.
 *   hf_plan_set_launch_bound: on = 1 / 0 run the bounded / the plain build whatever the preset;
 *                on < 0 by the preset (default): hfuse_lb and vfuse_lb run the bounded build when
 *                the formula asks for more than 4 waves per SIMD.
 *   hf_plan_set_launch_waves: waves = 1..8 asks for a bounded build at that many waves per SIMD
 *                (and switches the bounded build on); 0 goes back to the formula's value.
 *   hf_plan_launch_waves: *formula = what the formula gives for this plan's block shape,
 *                *built = the bound of the build a launch would run now (0: the plain build).
 * The blockIdx fallback has no bounded build and the vertical baseline only the 8-wave one.
 * Results are identical; only the time differs.
 */
HF_API int hf_plan_set_launch_bound(hf_plan *plan, int on);
HF_API int hf_plan_set_launch_waves(hf_plan *plan, int waves);
HF_API int hf_plan_launch_waves(const hf_plan *plan, int *formula, int *built);
HF_API int hf_plan_partition(const hf_plan *plan, hf_partition *out);
/*
 * Three-kernel fusions.  The reference's Context partitions one block among any number of kernels
 * (include/KernelFusion.h:45-80) and its lists name three in configs/crypt_four.yaml
 * (blake2b_gpu_hash, sha256d_gpu_hash_shared, ethash_search4), configs/im2col_maxpool_norm.yaml
 * and configs/maxpool_summary_norm.yaml; those three lists are built, and a list that names the
 * same three kernels in another order runs the same instantiation with the thread bounds of its
 * own order (any other three kernels: HF_EUNSUPPORTED from hf_plan_create).
 * hf_plan_create on such an entry gives a plan whose block is kernel 0's threads, then kernel
 * 1's, then kernel 2's, in the order the list names them (vfuse presets: all three start at thread
 * 0 of a block of max threads); argument lists follow the list's order as well.
 *   split_idx     : as the reference's driver does it (main.cpp:215-227): only the first two
 *                   kernels' ExecTimes are varied, ExecTime_0 = 128*(idx+1), ExecTime_1 =
 *                   (d0 + d1) - ExecTime_0, the third keeps the table's (-1 without the key); the
 *                   Context then re-splits d0 + d1 + d2 in proportion, whole wavefronts each,
 *                   the last kernel taking the rest.  HF_SPLIT_EXECTIME / HF_SPLIT_TABLE as for pairs.
 *   split_threads : must be 0; hf_plan_set_block_n shapes the block freely.
 * Each kernel strides over its own number of workgroups (the launch covers the largest); in a
 * block beyond a kernel's own number its wavefronts end at once.  A body that synchronises does
 * so on its own LDS arrival counter.  The calls that shape a pair (hf_plan_set_block / _grids /
 * _lending / _barrier_mode / _launch_bound / _launch_waves, hf_plan_partition, hf_launch_fused,
 * hf_time_pair) answer HF_EINVAL for a three-kernel plan; hf_plan_bind_constants and
 * hf_plan_local_index (half = 0..2) apply.
 */
#define HF_MAX_FUSE 4
typedef struct {
  char name[256];                /* <K0>_<K1>_<K2>_fused_kernel_<preset>_idx_<n>    */
  int n;                         /* kernels in the plan: 2 or 3                      */
  uint32_t lo[HF_MAX_FUSE], hi[HF_MAX_FUSE];
  hf_dim3 block_dim[HF_MAX_FUSE];
  uint32_t launch_threads, launch_blocks;
  int barrier_mode;
} hf_partition_n;
HF_API int hf_plan_num_kernels(const hf_plan *plan);
HF_API int hf_plan_partition_n(const hf_plan *plan, hf_partition_n *out);
/* threads[k] for kernel k (multiples of 64 that divide by its BlockDim.Y; sum <= 1024, 512 for the searches). */
HF_API int hf_plan_set_block_n(hf_plan *plan, const int *threads, int n);

/* Number of variants the reference's split loop would print (main.cpp:221-223). */
HF_API int hf_plan_num_splits(const hf_config *cfg, int fusion_index);
/* Local (x,y,z) of flat thread `tid` in half `half`: ThreadInfoRewriter.cpp:38-58. */
HF_API int hf_plan_local_index(const hf_plan *plan, int half, uint32_t tid, hf_dim3 *out);

/* ------------------------------------------------- original argument lists */

/* im2col_kernel<float> -- scripts/data/ml-event.csv:17 */
typedef struct {
  int64_t n;
  const float *data_im;
  int64_t height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
      dilation_w, height_col, width_col;
  float *data_col;
} hf_im2col_args;

/* MaxPoolForward<float,float> -- scripts/data/ml-event.csv:5 */
typedef struct {
  int nthreads;
  const float *bottom_data;
  int num, channels, height, width, pooled_height, pooled_width, kernel_h, kernel_w, stride_h,
      stride_w, pad_h, pad_w, dilation_h, dilation_w;
  float *top_data;
  int64_t *top_mask;
} hf_maxpool_args;

/* PackedTensorAccessor<float,N,...,int> flattened to {ptr, sizes, strides}. */
typedef struct {
  float *data;
  int sizes[3];
  int strides[3];
} hf_accessor3;
typedef struct {
  float *data;
  int sizes[1];
  int strides[1];
} hf_accessor1;

/*
 * batch_norm_collect_statistics_kernel<InvStd,float,float,float,int>
 * -- scripts/data/ml-event.csv:14, call text scripts/configs/hist_norm.json:5.
 * running_mean / running_var / momentum are accepted and ignored, as in the
 * reference's call (dummy tensors, momentum 0.0).
 */
typedef struct {
  hf_accessor3 input; /* [N, C, L] */
  float epsilon;
  float momentum;
  hf_accessor1 running_mean, running_var, save_mean, save_transformed_var;
} hf_bn_stats_args;

/*
 * upsample_nearest2d_out_frame<float> (PyTorch).  The reference's table lists
 * the bilinear kernel (configs/ml_kernels.yaml:1-9, declared further down); the
 * benchmarked pair uses nearest, whose argument list is the one below.
 */
typedef struct {
  const float *idata;
  float *odata;
  size_t nc, height1, width1, height2, width2;
  float height_scale, width_scale;
} hf_upsample_nearest_args;

/* PackedTensorAccessor<float,4,DefaultPtrTraits,long> flattened. */
typedef struct {
  float *data;
  int64_t sizes[4];
  int64_t strides[4];
} hf_accessor4;

/*
 * upsample_bilinear2d_out_frame<float,float> -- scripts/data/ml-event.csv:9,
 * configs/ml_kernels.yaml:1-9.  n = height2 * width2 (the original runs one
 * thread per output pixel and loops over batch and channels); rheight / rwidth
 * are PyTorch's area_pixel_compute_scale values; align_corners is the bool.
 */
typedef struct {
  int n;
  float rheight, rwidth;
  int align_corners;
  hf_accessor4 idata, odata; /* [N, C, H, W] */
} hf_upsample_bilinear_args;

/* cuda::detail::TensorInfo<float,long> flattened. */
#define HF_MAX_TENSORINFO_DIMS 8
typedef struct {
  float *data;
  int64_t sizes[HF_MAX_TENSORINFO_DIMS];
  int64_t strides[HF_MAX_TENSORINFO_DIMS];
  int dims;
} hf_tensorinfo;

/*
 * kernelHistogram1D<float,float,long,1,2,-1,SHARED,Op>
 * -- scripts/data/ml-event.csv:2, call text scripts/configs/hist_norm.json:5.
 * a = output counts (fp32, caller-zeroed, accumulated with atomics),
 * p = partial output (unused in SHARED mode), b = input.  getOp is the
 * constant-1 functor of histc; a NULL function pointer slot keeps the arity.
 * Only 1-D tensors and a contiguous `a` are built (HF_EUNSUPPORTED otherwise).
 * Up to 15360 bins are counted in LDS and flushed once per workgroup; more bins
 * are counted in global memory directly, as the original's GLOBAL memory type
 * (fp32 counts stay exact up to 2^24 per bin).
 */
typedef struct {
  hf_tensorinfo a, p, b;
  int nbins;
  float minvalue, maxvalue;
  int64_t total_elements;
  const void *get_op;
} hf_histc_args;

/* Search results shared by the three nonce searches (layout is this library's own). */
#define HF_MAX_SEARCH_RESULTS 64
typedef struct {
  uint64_t nonce;     /* sha256d: 32-bit nonce; sia: the 8-byte word at offset 32; ethash: nonce */
  uint32_t digest[8]; /* the 32 digest bytes as they lie in memory                               */
  uint32_t mix[8];    /* ethash mix digest, zero otherwise                                       */
} hf_search_hit;
typedef struct {
  uint32_t count;     /* total hits found (may exceed the recorded slots)                        */
  uint32_t pad;
  hf_search_hit hit[HF_MAX_SEARCH_RESULTS]; /* unordered; callers sort by nonce                  */
} hf_search_results;

/*
 * ethash_search(volatile Search_results*, uint64_t) -- scripts/data/ethminer_event.csv:9.
 * Like the original (gid = blockIdx * blockDim + threadIdx) it takes no count: a launch scans
 * grid_blocks * block threads nonces from start_nonce, where the block is the kernel's own in
 * a native launch and its share of the fused block (hf_plan_partition: hi[k] - lo[k]) in a
 * fused one.  grid_blocks <= 0 means 8192 blocks, the reference traces' launch.
 */
typedef struct {
  hf_search_results *g_output;
  uint64_t start_nonce;
} hf_ethash_args;

/* sha256d_gpu_hash_shared(uint32, uint32, uint32*) -- scripts/data/ethminer_event.csv:26 */
typedef struct {
  uint32_t threads;
  uint32_t start_nonce;
  uint32_t *res_nonces; /* points at an hf_search_results */
} hf_sha256d_args;

/* sia_blake2b_gpu_hash / blake2b_gpu_hash(uint32, uint32, uint32*, uint2)
 * -- scripts/data/ethminer_event.csv:2,22 */
typedef struct {
  uint32_t threads;
  uint32_t start_nonce;
  uint32_t *res_nonce; /* points at an hf_search_results */
  uint32_t target2[2]; /* uint2: {low, high} words of the 64-bit target */
} hf_blake2b_args;

/*
 * Constants the original kernels read from __constant__ symbols set by their
 * host program (DAG pointer and size, header, midstate, target).  The library
 * keeps them in host memory and passes them in the kernel-argument segment of
 * each launch, next to the original argument list; nothing is copied to the
 * device by these calls and `stream` is ignored (kept for source compatibility
 * with a cudaMemcpyToSymbolAsync-style caller).
 *
 * These four calls write ONE process-wide set, as the original symbols are one
 * per device: each call replaces its values atomically, and every launch reads
 * the set as it is when the launch call is made.  Two host threads that search
 * different headers must not share it -- they use hf_constants below.
 */
/* ethash: DAG of 128-byte items, 32-byte header hash, 64-bit target. */
HF_API int hf_ethash_set_constants(const void *dag, uint32_t dag_items, const uint8_t header[32],
                                   uint64_t target, void *stream);
/* sha256d: 80-byte header (nonce bytes 76..79 ignored) and the top 64 bits of
 * the little-endian 256-bit target. */
HF_API int hf_sha256d_set_block(const uint8_t header[80], uint64_t target64, void *stream);
/* sia blake2b / ccminer blake2b: 80-byte header. */
HF_API int hf_sia_blake2b_set_block(const uint8_t header[80], void *stream);
HF_API int hf_blake2b_set_block(const uint8_t header[80], void *stream);

/*
 * A caller-owned set of the same constants (no counterpart in the reference, whose host
 * programs are single-threaded).  One thread fills it; hf_plan_bind_constants copies it into
 * a plan, whose fused launches then use that copy instead of the process-wide set (NULL
 * unbinds), and hf_launch_native_with launches one original kernel with it.  Setting the
 * constants and launching is thereby one unit per plan / per call, whatever other threads do.
 */
typedef struct hf_constants hf_constants;
HF_API int hf_constants_create(hf_constants **out);
HF_API void hf_constants_free(hf_constants *c);
HF_API int hf_constants_set_ethash(hf_constants *c, const void *dag, uint32_t dag_items,
                                   const uint8_t header[32], uint64_t target);
HF_API int hf_constants_set_sha256d(hf_constants *c, const uint8_t header[80], uint64_t target64);
HF_API int hf_constants_set_sia_blake2b(hf_constants *c, const uint8_t header[80]);
HF_API int hf_constants_set_blake2b(hf_constants *c, const uint8_t header[80]);
HF_API int hf_plan_bind_constants(hf_plan *plan, const hf_constants *c);

/* ----------------------------------------------------------------- launches */
/*
 * Native launch of one original kernel by its YAML name; `args` points at the
 * matching hf_*_args.  grid_blocks <= 0 lets the library size the grid from the
 * work; block threads come from block_threads (<= 0: the kernel's default --
 * 128 for the searches, 256 for max-pooling, 768 for the histogram, 512 otherwise).
 */
HF_API int hf_launch_native(const char *kernel_name, const void *args, int grid_blocks,
                            int block_threads, void *stream);
/* The same with the search constants of `constants` instead of the process-wide set. */
HF_API int hf_launch_native_with(const char *kernel_name, const void *args,
                                 const hf_constants *constants, int grid_blocks, int block_threads,
                                 void *stream);
/*
 * Fused launch: one kernel whose workgroup is [0,d1) running kernel 1's body
 * and [d1,d1+d2) running kernel 2's, arguments in YAML order
 * (KernelPrinter.cpp:107-115).  grid_blocks <= 0: sized by the library.
 */
HF_API int hf_launch_fused(const hf_plan *plan, const void *args1, const void *args2,
                           int grid_blocks, void *stream);

/*
 * Fused launch of a plan of n kernels: args[k] points at kernel k's argument list, in YAML order
 * (n = 2 is hf_launch_fused).  grid_blocks > 0: every kernel strides over that many workgroups.
 */
HF_API int hf_launch_fused_n(const hf_plan *plan, const void *const *args, int n, int grid_blocks,
                             void *stream);
/*
 * hf_time_pair for a three-kernel plan: mode 2 = the three native kernels back to back on
 * `stream`, mode 3 = the fused kernel; args[s * n + k] is kernel k's argument list of set s.
 */
HF_API int hf_time_fused_n(const hf_plan *plan, int mode, const void *const *args, int n, int nsets,
                           int first_set, int warmup, int iters, int grid_blocks, void *stream,
                           float *elapsed_ms);

/*
 * Timing helper used by the benchmark: runs `iters` repetitions of
 *   mode 0: native kernel 1      mode 1: native kernel 2
 *   mode 2: kernel 1 then kernel 2 back to back on `stream`
 *   mode 3: the fused kernel
 *   mode 4: kernel 1 on `stream` and kernel 2 on a second stream of the
 *           library's own, forked and joined with events every repetition
 *           (the two-stream launch the reference's traces were taken with)
 * cycling through `nsets` argument sets (args1[i], args2[i]) so repeats do not
 * hit in the last-level cache, and returns the elapsed milliseconds measured
 * with HIP events recorded on `stream` around the timed launches.  Repetition r
 * (warm-ups included) uses set (first_set + r) % nsets: a caller that times in
 * several short calls passes the set after the last one used, so that the calls
 * together keep walking the whole rotation instead of re-reading the first sets.
 */
HF_API int hf_time_pair(const hf_plan *plan, int mode, const void *const *args1,
                        const void *const *args2, int nsets, int first_set, int warmup,
                        int iters, int grid_blocks, void *stream, float *elapsed_ms);

/* --------------------------------------------------------- support kernels */
/* dst[i] = SplitMix64 counter generator word i (seeded synthetic DAG / inputs). */
HF_API int hf_fill_splitmix64(uint64_t *dst, uint64_t nwords, uint64_t seed, void *stream);
/* Plain device copy, the unit the HBM counters are calibrated against. */
HF_API int hf_copy_f32(const float *src, float *dst, uint64_t n, void *stream);

/*
 * Bare stream kernels (no counterpart in the reference): what the memory system of this part delivers for the
 * access patterns of the kernels above, measured by the benchmark in the same run as the kernels that are judged
 * against them.  16-byte non-temporal accesses; `bytes` is what one launch reads (HF_STREAM_WRITE: writes).
 *   HF_STREAM_EMPTY       an empty kernel (the cost of a launch); the other arguments are ignored
 *   HF_STREAM_READ        every workgroup reads one contiguous share of `src`; `dst` = 4 bytes, never written
 *   HF_STREAM_WRITE       every workgroup writes one contiguous share of `dst` (`bytes`); `src` is ignored
 *   HF_STREAM_WRITE_STRIDED  the same bytes written by a grid-stride loop (the whole grid inside one window at a time)
 *   HF_STREAM_WRITE_XCD   HF_STREAM_WRITE with the workgroups renumbered so that each of the eight XCDs owns one
 *                         contiguous eighth of `dst` (the grid must be a multiple of eight)
 *   HF_STREAM_READ_LINES  uniformly random 128-byte lines out of `src` (`bytes` large), eight lanes a line, `bytes`
 *                         read in total: the DAG reads of ethash_search; `dst` = 4 bytes, never written
 *   HF_STREAM_COPY_1_4    reads `bytes` from `src`, writes them to four planes of `dst` (4 * `bytes`): the shape of
 *                         upsample_nearest2d_out_frame
 * `bytes` must divide into whole 16-byte vectors per workgroup (per thread and trip for the random lines).
 */
enum { HF_STREAM_EMPTY = 0, HF_STREAM_READ = 1, HF_STREAM_WRITE = 2, HF_STREAM_READ_LINES = 3, HF_STREAM_COPY_1_4 = 4,
       HF_STREAM_WRITE_STRIDED = 5, HF_STREAM_WRITE_XCD = 6 };
HF_API int hf_stream_probe(int pattern, const void *src, void *dst, uint64_t bytes, int grid_blocks, int block_threads,
                           void *stream);
/*
 * `warmup` untimed and `iters` timed launches of one pattern between two events on `stream`; launch r works on
 * src + (r % nbuf) * src_stride and dst + (r % nbuf) * dst_stride (bytes), so that a rotation through more than the
 * 256 MB memory-side cache holds reads from HBM.  *elapsed_ms = milliseconds of the `iters` launches.
 */
HF_API int hf_time_stream_probe(int pattern, const void *src, void *dst, uint64_t bytes, uint64_t src_stride,
                                uint64_t dst_stride, int nbuf, int grid_blocks, int block_threads, int warmup, int iters,
                                void *stream, float *elapsed_ms);

#ifdef __cplusplus
}
#endif
#endif /* HFUSE_GFX950_H */
