/*
 * tritonix_hip.h -- C ABI of libtritonix_hip.so, the gfx950 (MI355X) tiled-GEMM engine.
 *
 * Every entry point takes plain pointers and sizes; nothing here depends on
 * PyTorch.  The library never allocates or frees device memory, never
 * synchronises, and launches asynchronously on the stream the caller passes.
 *
 * Reference interfaces these entry points stand in for (paths are inside the
 * ayghri/tritonix tree):
 *   - the Triton launch `matmul_kernel[grid](a, b, c, m, n, k, 6 strides,
 *     block_m=, block_n=, block_k=, group_m=, num_stages=, num_warps=)`
 *     tritonix/ops/matmul.py:43-108, launched from :217-237;
 *   - `gemm_splitk_kernel[grid](..., split_k=)` tritonix/ops/matmul.py:147-202,
 *     launched from :240-264, with its `_zero_output` pre-run hook :205-210;
 *   - `glu_kernel[grid](x, w12, z, m, n, k, 6 strides, block_*=, group_m=,
 *     use_tf32=, activation=, num_stages=, num_warps=)`
 *     tritonix/ops/swiglu.py:24-110 (phase 1 of swiglu_kernel :155-205);
 *   - the int8 -> int32 kernel playground/test_int8_mma.py:7-42;
 *   - `triton.OutOfResources` as raised by the Triton launcher and caught at
 *     tritonix/autotune.py:134 (here: TNX_E_LDS + tnx_gemm_lds_bytes());
 *   - `conv2d_forward_kernel[grid](output, input, weight, bias, 9 sizes, 6 stride/pad/dilation values,
 *     GEMM_M, GEMM_N, GEMM_K, BLOCK_SIZE_M=, BLOCK_SIZE_N=, BLOCK_SIZE_K=, GROUP_SIZE_M=, OUT_DTYPE=,
 *     USE_TF32=)` tritonix/ops/conv2d/forward.py:19-165, launched from :202-311 (tnx_conv2d_forward).
 */
#ifndef TRITONIX_HIP_H
#define TRITONIX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TNX_VERSION 1

/* element types */
enum tnx_dtype {
  TNX_F16 = 0,  /* IEEE binary16 */
  TNX_BF16 = 1, /* bfloat16 */
  TNX_I8 = 2,   /* signed 8-bit */
  TNX_I32 = 3,  /* signed 32-bit (output of the int8 path) */
  TNX_F32 = 4   /* binary32: the type of split-K slices in the workspace, and an output type: a bf16 / f16 GEMM on
                   a tile of at most 128x128 may write its fp32 sums unrounded (out_dtype = TNX_F32).  No kernel
                   takes binary32 operands; tnx_split_f32 turns them into bf16 operands of a three-term product */
};

/* epilogues fused after the K loop (tritonix/ops/swiglu.py:98-104).
 * For the GLU epilogues `n` is the interleaved width of B (even columns are
 * the gate, odd columns the linear branch) and C has n/2 columns. */
enum tnx_epilogue {
  TNX_EPI_NONE = 0,
  TNX_EPI_GLU_SILU = 1,     /* silu(gate) * lin   (activation == "silu")        */
  TNX_EPI_GLU_SIGMOID = 2,  /* sigmoid(gate) * lin                               */
  TNX_EPI_GLU_IDENTITY = 3  /* gate * lin (the reference's fall-through branch)  */
};

/* how tiles are handed to workgroups (flags, may be combined) */
enum tnx_schedule {
  TNX_SCHED_DEFAULT = 0,    /* one workgroup per tile; launch order = XCD-aware remap + tl.swizzle2d(group_m),
                               the order of tritonix/ops/matmul.py:70                                           */
  TNX_SCHED_PERSISTENT = 1, /* one workgroup per CU walks its tiles; the next tile's first K slabs load while
                               the current tile's epilogue runs (the reference's draft of the same idea:
                               playground/persistent_mma.py:47-141).  Needs split_k == 1, the DMA layout,
                               k >= num_stages * block_k and a tile built with this variant, else
                               TNX_E_UNSUPPORTED                                                                */
  TNX_SCHED_SUPERBLOCK = 2, /* launch order = 16x16 super-blocks of tiles walked in serpentine order, an 8x4
                               sub-block per XCD: consecutive rounds of 256 workgroups share half of their
                               operand panels.  Ignored (default order) when split_k > 1                       */
  TNX_SCHED_ATOMIC_REDUCE = 4 /* split_k > 1: the K slices are added into ONE fp32 / int32 copy of each cut tile
                               with device-scope atomic adds (the reference adds with tl.atomic_add too,
                               tritonix/ops/matmul.py:202, but into C and after rounding to the output type;
                               here the sum stays fp32 and is rounded once) instead of being stored apart and
                               summed in slice order.  Float results then depend on arrival order in the
                               last bits.  The workspace bytes [TNX_WS_COUNTER_BYTES, TNX_WS_COUNTER_BYTES +
                               cut tiles * block_m * block_n * 4) must be zero when the launch starts; the
                               launch leaves them zero (an ordered-mode launch on the same workspace does not) */
};

/* status codes */
enum tnx_status {
  TNX_OK = 0,
  TNX_E_INVALID = 1,     /* null pointer, negative size, bad enum                     */
  TNX_E_UNSUPPORTED = 2, /* no kernel is built for this tile / dtype / layout combo   */
  TNX_E_LDS = 3,         /* the tile config needs more LDS than one CU has            */
  TNX_E_WORKSPACE = 4,   /* split_k > 1 and the workspace is missing or too small     */
  TNX_E_HIP = 5,         /* the HIP runtime reported an error (see tnx_last_hip_error) */
  TNX_E_STATIC_LIMIT = 6 /* tnx_gemm_static_workspace: the launch needs more scratch than the static buffer */
};

/* Per-CU LDS capacity on gfx950; the budget tile configs are pruned against. */
#define TNX_LDS_LIMIT_BYTES 163840

typedef struct tnx_gemm_args {
  const void* a;   /* [m, k], element strides stride_am / stride_ak             */
  const void* b;   /* [k, n], element strides stride_bk / stride_bn             */
  void* c;         /* [m, n] (or [m, n/2] with a GLU epilogue)                  */
  int64_t m, n, k;
  int64_t stride_am, stride_ak;
  int64_t stride_bk, stride_bn;
  int64_t stride_cm, stride_cn;
  int32_t in_dtype;   /* tnx_dtype of a and b                                    */
  int32_t out_dtype;  /* tnx_dtype of c                                          */
  int32_t block_m, block_n, block_k; /* workgroup tile                           */
  int32_t group_m;    /* rows of tiles per L2 super-group (tl.swizzle2d size_g)  */
  int32_t split_k;    /* 1 = no split; >1 = K is cut into split_k slices         */
  int32_t num_stages; /* LDS ring depth of the global->LDS pipeline              */
  int32_t num_warps;  /* wavefronts (64 lanes) per workgroup: 4 or 8             */
  int32_t epilogue;   /* tnx_epilogue                                            */
  int32_t tail_tiles; /* with split_k > 1: 0 = every tile is cut; t > 0 = see below    */
  int32_t schedule;   /* tnx_schedule flags, 0 = one workgroup per tile in tl.swizzle2d order */
  void* workspace;    /* device scratch for split_k > 1 (see tnx_gemm_workspace_bytes) */
  size_t workspace_bytes;
  void* stream;       /* hipStream_t; NULL = the null stream                     */
} tnx_gemm_args;

/* tail_tiles: with split_k > 1 and tail_tiles = t > 0 only the last t tiles in launch order
 * are cut along K, the tiles before them are computed whole by one workgroup each.  This
 * fills the last, partial wave of workgroups when the tile count is not a multiple of the
 * CU count (the reference's answer to the same problem is a persistent kernel,
 * playground/persistent_mma.py:47-141). */

/* Launch one GEMM.  Returns a tnx_status.  Asynchronous.
 * Which loader moves the operands follows from their layout, not from an argument:
 *   - A row-major (stride_ak == 1) and B row-major (stride_bn == 1): the direct-to-LDS loader of every built tile.
 *     With K a multiple of block_k, 16-byte aligned rows and base pointers and N a multiple of 16 bytes of elements
 *     every K slab goes through it; otherwise (rows and pointers at the element's own alignment, any K and N, row
 *     pitches at least the row length) the last K slab is loaded chunk by chunk with zero fill and the slabs
 *     before it through the direct loader.
 *     TNX_SCHED_PERSISTENT takes the first form only.
 *   - A row-major and B k-contiguous (stride_bk == 1, the view w.t() of a row-major weight): a direct-to-LDS loader
 *     of its own, in the tiles whose K slab is 128 bytes per row, under the same two sets of conditions (K a multiple
 *     of block_k and 16-byte aligned rows and pointers, or else the last K slab loaded chunk by chunk).
 *   - anything else (strided A, overlapping rows, ...): the element-wise loader, built for two tiles per type
 *     (128x128 and 64x128, four waves, two stages); other tiles return TNX_E_UNSUPPORTED. */
int tnx_gemm(const tnx_gemm_args* args);

/* tnx_gemm without any allocation on anyone's side.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory at the call site (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  Same arguments and results as tnx_gemm, except that
 * `workspace` / `workspace_bytes` are ignored: a split-K launch takes its scratch from a buffer of
 * TNX_STATIC_WORKSPACE_BYTES that is part of the library's device image (every GPU the library runs
 * on holds one copy until the process ends).  A launch that needs more returns TNX_E_STATIC_LIMIT and
 * launches nothing.  The call makes no hipMalloc / hipFree and calls no allocating routine; it enqueues
 * one extra tiny kernel that clears the arrival counters it is about to use.  All calls on one GPU share
 * that GPU's buffer: calls that may overlap on one GPU (different streams, or different threads) race
 * and must be ordered by the caller.  The first call on a device looks the buffer's address up
 * (hipGetSymbolAddress) and must therefore happen outside graph capture. */
#define TNX_STATIC_WORKSPACE_BYTES (65536 + (32 << 20))
int tnx_gemm_static_workspace(const tnx_gemm_args* args);

/* Bytes of device scratch tnx_gemm needs for these args (0 when split_k <= 1):
 * the counters plus split_k fp32/int32 copies of every tile that is cut.
 * The workspace must be 256-byte aligned.  Its first TNX_WS_COUNTER_BYTES hold
 * per-tile arrival counters: they must be zero before the first launch that
 * uses the workspace, and every launch leaves them zero again, so one
 * zero-fill at allocation is enough (calls sharing a workspace must be
 * ordered on one stream).  The rest needs no initialisation.  C itself is
 * never pre-zeroed: this replaces the reference's `_zero_output` hook
 * (tritonix/ops/matmul.py:205-210). */
#define TNX_WS_COUNTER_BYTES 65536
size_t tnx_gemm_workspace_bytes(const tnx_gemm_args* args);

/* LDS bytes per workgroup the tile config in `args` would use.  Pure host
 * arithmetic, no GPU needed: lets the tuner's trie prune a config without
 * launching it.  Returns -1 if the config is malformed. */
int64_t tnx_gemm_lds_bytes(const tnx_gemm_args* args);

/* TNX_OK if tnx_gemm would accept these args (pointers are not inspected),
 * otherwise the status it would return.  Pure host arithmetic. */
int tnx_gemm_supported(const tnx_gemm_args* args);

/* Fill block_m/n/k, group_m, split_k, tail_tiles, num_stages, num_warps of
 * `args` with a built-in choice for its shape and dtype (used when nothing
 * was tuned).  split_k > 1 comes back only for shapes whose tiles alone leave
 * CUs idle; a caller that cannot provide a workspace may reset split_k to 1
 * and tail_tiles to 0. */
int tnx_gemm_default_config(tnx_gemm_args* args);

/* Which tile the workgroup with launch-order id `id` computes (no split): the host-side copy of the device
 * functions, for tests and tooling.  Default schedule: XCD-aware remap followed by tl.swizzle2d with
 * size_g = group_m (tritonix/ops/matmul.py:70; triton/language/standard.py:80-116).  With
 * TNX_SCHED_SUPERBLOCK: the super-block order.  Either is a bijection of [0, tiles_m*tiles_n) onto the grid. */
int tnx_tile_coords(int schedule, int id, int tiles_m, int tiles_n, int group_m, int* tile_m, int* tile_n);

/* float32 operands.  The reference's kernels take whatever tl.dot takes (tritonix/ops/matmul.py:98), float32 included,
 * which Triton multiplies in TF32 (`use_tf32`, tritonix/ops/swiglu.py:89-93).  gfx950 has no TF32 matrix instruction;
 * a float32 product runs here on the bf16 instructions as three terms: with x = hi(x) + lo(x) + O(2^-17 |x|), hi and lo
 * both bf16 (round to nearest even), a @ b = hi(a) @ hi(b) + hi(a) @ lo(b) + lo(a) @ hi(b) + O(2^-16), accumulated
 * in fp32 -- tighter than TF32's 2^-11.  tnx_split_f32 writes the bf16 operand of that product for one float32
 * matrix src[rows, cols] (element strides stride_r, stride_c), contiguous and row-major in dst:
 *   side 0 (the A operand):  dst[rows, 3 * cols] = [ hi | hi | lo ]      side 1 (the B operand):  dst[3 * rows, cols] = [ hi ; lo ; hi ]
 *   side 2:  dst[rows, 3 * cols] = [ hi | lo | hi ]  (the partner of side 0 when both operands are cut along their
 *   columns: conv2d's NCHW input, side 0, and KCRS weight, side 2, both along c_in)
 * so that one tnx_gemm with k' = 3k, in_dtype = TNX_BF16 and out_dtype = TNX_F32 (or a GLU epilogue on top) is the
 * float32 product.  A non-finite element is carried by the first copy of its head alone: its tail and the second copy
 * of its head (the one multiplied with the other operand's tail) are zero, so inf * finite stays inf and does not
 * become inf + inf * 0 = NaN.  dst holds 3 * rows * cols bf16 values.
 * Asynchronous on `stream`; allocates nothing. */
int tnx_split_f32(const float* src, int64_t rows, int64_t cols, int64_t stride_r, int64_t stride_c, void* dst, int side,
                  void* stream);

/* Number of compiled tile kernels, and a description of the i-th one:
 * "dtype bm bn bk warps stages [generic] [persistent]" as a NUL-terminated string (static storage);
 * "generic": also built with the element-wise loader; "persistent": also built for TNX_SCHED_PERSISTENT. */
int tnx_kernel_count(void);
const char* tnx_kernel_name(int i);

/* ---- conv2d forward (implicit GEMM on the same LDS layout and MFMA fragments) ------------------------------
 * Stands in for conv2d_forward_kernel, tritonix/ops/conv2d/forward.py:19-165: contiguous NCHW input, KCRS
 * weight, NCHW output of the input's type, GEMM_M = batch * h_out * w_out, GEMM_N = c_out, GEMM_K = c_in *
 * filter_h * filter_w, zero padding, fp32 accumulation, optional bias added in fp32 before the one rounding.
 * block_pixels / block_cout / block_k / group_pixels are the reference's BLOCK_SIZE_M / BLOCK_SIZE_N /
 * BLOCK_SIZE_K / GROUP_SIZE_M.  dtype is TNX_F16 or TNX_BF16 (the reference's float32-with-TF32 mode has no
 * matrix instruction on gfx950 and is not built: TNX_E_UNSUPPORTED).  Limits: batch * h_out * w_out and the
 * element counts of input and weight below 2^31, h_in / w_in / pad / (filter - 1) * dilation at most 16384. */
typedef struct tnx_conv2d_args {
  const void* input;   /* [batch, c_in, h_in, w_in]                                 */
  const void* weight;  /* [c_out, c_in, filter_h, filter_w]                         */
  const void* bias;    /* [c_out] of bias_dtype, or NULL                            */
  void* output;        /* [batch, c_out, h_out, w_out], same type as the input (binary32 with out_f32) */
  int32_t batch, c_in, h_in, w_in;
  int32_t c_out, filter_h, filter_w;
  int32_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int32_t dtype;       /* tnx_dtype of input, weight and output                     */
  int32_t bias_dtype;  /* TNX_F16 / TNX_BF16 / TNX_F32                              */
  int32_t block_pixels, block_cout, block_k; /* workgroup tile; 0 0 0 = built-in choice */
  int32_t group_pixels; /* pixel tiles per L2 group (tl.swizzle2d size_g); 0 = 8    */
  int32_t loader;      /* tnx_conv_loader; 0 = the library chooses                   */
  void* stream;        /* hipStream_t; NULL = the null stream                       */
  int32_t out_f32;     /* non-zero: `output` is binary32, the fp32 sums (+ bias) unrounded -- what makes a float32
                          convolution a three-term bf16 one: split the input along its channels with
                          tnx_split_f32(side 0) and the weight with side 2, tripling c_in                    */
} tnx_conv2d_args;

/* How the slabs reach LDS.  Two kernels exist: one stages both operands through registers (any stride, padding,
 * dilation, any c_in * filter_h * filter_w; tiles up to 256 x 128), the other is the GEMM kernel with a
 * direct-to-LDS im2col loader (needs stride_w == 1, c_in * filter_h * filter_w a multiple of block_k = 64, a 16-byte
 * aligned weight; tiles of 128 or 256 channels x 128 or 256 pixels).  With TNX_CONV_LOADER_AUTO and no tile given
 * the library takes the direct-to-LDS kernel whenever the problem allows it and has enough tiles to fill the chip;
 * with a tile given it takes it when the tile exists only there, or exists in both and the problem allows it.
 * A third way serves 1x1 filters with unit stride and no padding: such a layer is, image by image, the plain GEMM
 * out[n] = weight[c_out, c_in] x input[n][c_in, h * w] (+ bias per row), and TNX_CONV_LOADER_GEMM runs it on the
 * GEMM tile kernels themselves, all images in one grid (tile = block_cout x block_pixels x block_k of any built GEMM
 * tile up to 128x128, or all three zero for a built-in choice; any c_in, any h * w).  TNX_CONV_LOADER_AUTO takes it with the
 * built-in tile on every such layer (a tile given by the caller names a conv2d kernel).
 * Asking for a loader the problem or tile does not allow returns TNX_E_UNSUPPORTED. */
enum tnx_conv_loader {
  TNX_CONV_LOADER_AUTO = 0,
  TNX_CONV_LOADER_REGISTERS = 1,
  TNX_CONV_LOADER_DMA = 2,
  TNX_CONV_LOADER_GEMM = 3
};

/* Launch one conv2d forward.  Returns a tnx_status.  Asynchronous, allocates nothing. */
int tnx_conv2d_forward(const tnx_conv2d_args* args);

/* TNX_OK if tnx_conv2d_forward would accept these args (pointers are not inspected, apart from their
 * alignment), otherwise the status it would return.  Pure host arithmetic. */
int tnx_conv2d_supported(const tnx_conv2d_args* args);

/* h_out / w_out as the reference computes them (tritonix/ops/conv2d/forward.py:226-227); either may come
 * back <= 0 for a filter larger than the padded image, which tnx_conv2d_forward rejects. */
void tnx_conv2d_output_size(const tnx_conv2d_args* args, int32_t* h_out, int32_t* w_out);

/* Fill block_pixels / block_cout / block_k / group_pixels / loader with the built-in choice for this problem (a
 * non-NULL weight pointer is checked for the 16-byte alignment the direct-to-LDS kernel needs). */
int tnx_conv2d_default_config(tnx_conv2d_args* args);

/* Compiled conv2d tiles: count, and "dtype block_cout block_pixels block_k loader" of the i-th (static storage;
 * loader is "registers" or "dma"). */
int tnx_conv2d_kernel_count(void);
const char* tnx_conv2d_kernel_name(int i);

const char* tnx_strerror(int status);
int tnx_last_hip_error(void); /* hipError_t of the last TNX_E_HIP on this thread */
int tnx_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TRITONIX_HIP_H */
