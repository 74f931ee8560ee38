// C ABI of libtritonix_hip.so: argument checking, tile-kernel lookup, launch.
// Declarations and the reference interfaces they replace: include/tritonix_hip.h
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "../../include/tritonix_hip.h"
#include "registry.h"

using namespace tnx;

extern "C" const KernelGroup* tnx_kernel_groups(int* ngroups);  // generated

static thread_local int g_last_hip_error = 0;
namespace tnx {
void note_hip_error(int err) { g_last_hip_error = err; }
}

static int elem_size(int dt) { return dt == TNX_I8 ? 1 : (dt == TNX_F16 || dt == TNX_BF16) ? 2 : 4; }

static const KernelEntry* find_entry(const tnx_gemm_args* a) {
  int ng = 0;
  const KernelGroup* g = tnx_kernel_groups(&ng);
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < g[i].count; ++j) {
      const KernelEntry& e = g[i].entries[j];
      if (e.dtype == a->in_dtype && e.bm == a->block_m && e.bn == a->block_n && e.bk == a->block_k &&
          e.nw == a->num_warps && e.stages == a->num_stages)
        return &e;
    }
  return nullptr;
}

static bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

// LDS bytes of a tile config, whether or not a kernel is built for it
static bool is_skinny_cfg(const tnx_gemm_args* a) {
  return a->block_m == SKINNY_BM && a->block_n == SKINNY_BN && a->block_k == SKINNY_BK && a->num_warps == SKINNY_NW;
}

static int64_t lds_bytes_of(const tnx_gemm_args* a) {
  if (a->block_m <= 0 || a->block_n <= 0 || a->block_k <= 0 || a->num_stages <= 0) return -1;
  if (is_skinny_cfg(a)) return (int64_t)a->num_stages * SKINNY_NW * SKINNY_STEP_BYTES;
  int es = elem_size(a->in_dtype);
  const int64_t ring = (int64_t)a->num_stages * ((int64_t)a->block_m * a->block_k + (int64_t)a->block_k * a->block_n) * es;
  // the epilogue passes the accumulators through per-wave LDS strips laid over the ring (EpiStage in
  // gemm_tile.h): waves x MFMA rows x (wave-tile width x 4 bytes + 16).  Same wave grid as TileCfg.
  const int nw = a->num_warps > 0 ? a->num_warps : 4;
  const int wgm = nw == 4 ? 2 : (a->block_m > a->block_n ? 4 : 2), wgn = nw / wgm > 0 ? nw / wgm : 1;
  const int wtm = a->block_m / wgm, wtn = a->block_n / wgn;
  const int mi = 16;   // TileCfg::MI
  const int rows = mi;   // EpiStage::ROWS
  (void)wtm;
  const int64_t strips = (int64_t)nw * rows * (wtn * 4 + 16);
  // the persistent kernel keeps its (smaller) strips beside the ring: MI rows of 256 bytes per wave
  if (a->schedule & TNX_SCHED_PERSISTENT) return ring + (int64_t)nw * mi * 256;
  return ring > strips ? ring : strips;
}

static int check_common(const tnx_gemm_args* a) {
  if (!a) return TNX_E_INVALID;
  if (a->m < 0 || a->n < 0 || a->k < 0) return TNX_E_INVALID;
  if (a->in_dtype != TNX_F16 && a->in_dtype != TNX_BF16 && a->in_dtype != TNX_I8) return TNX_E_INVALID;
  if (a->epilogue < TNX_EPI_NONE || a->epilogue > TNX_EPI_GLU_IDENTITY) return TNX_E_INVALID;
  if (a->block_m <= 0 || a->block_n <= 0 || a->block_k <= 0 || a->group_m <= 0 || a->split_k <= 0 ||
      a->num_stages <= 0 || a->num_warps <= 0 || a->tail_tiles < 0 || a->schedule < 0 ||
      a->schedule > (TNX_SCHED_PERSISTENT | TNX_SCHED_SUPERBLOCK | TNX_SCHED_ATOMIC_REDUCE))
    return TNX_E_INVALID;
  // output type is tied to the input type: f16->f16, bf16->bf16, i8->i32
  // ... or binary32 for the 16-bit float types, on the tiles that carry that epilogue (f32_out_tile in gemm_tile.h)
  int want_out = a->in_dtype == TNX_I8 ? TNX_I32 : a->in_dtype;
  if (a->out_dtype != want_out) {
    const bool f32_out = a->out_dtype == TNX_F32 && a->in_dtype != TNX_I8 && (int64_t)a->block_m * a->block_n <= 128 * 128 &&
                         !(a->schedule & TNX_SCHED_PERSISTENT) && !is_skinny_cfg(a);
    if (!f32_out) return TNX_E_UNSUPPORTED;
  }
  if (a->epilogue != TNX_EPI_NONE && (a->in_dtype == TNX_I8 || (a->n & 1))) return TNX_E_UNSUPPORTED;
  if (a->m > 0x7fffffff || a->n > 0x7fffffff || a->k > 0x7fffffff) return TNX_E_UNSUPPORTED;
  return TNX_OK;
}

// Which DMA loader the operands can take: 0 = none (element-wise loader only), 1 = row-major B
// (stride_bn == 1), 2 = k-contiguous B (stride_bk == 1, the layout of x @ w.t()).  Both need row-major A,
// 16-byte aligned rows and base pointers and k % block_k == 0.
// 0: element-wise loader; 1: DMA loader, A and B row-major; 2: DMA loader, B k-contiguous.
// *tail (layout 1 only): the operands are row-major but not as the DMA loader likes them best -- K no multiple of
// block_k, rows or base pointers not 16-byte aligned (the loads take any byte address: probed on the hardware),
// N ending inside a 16-byte chunk -- so the last K slab, the only one whose chunks can cross the end of a row of A
// or of the last row of B, is loaded element by element instead (GemmParams::tail_slab).
static int dma_layout(const tnx_gemm_args* a, bool* tail = nullptr) {
  const int es = elem_size(a->in_dtype);
  const int vec = 16 / es;
  if (tail) *tail = false;
  if (a->stride_ak != 1 || a->k == 0 || a->stride_am < 0) return 0;
  // per-lane DMA offsets are 32-bit
  if ((int64_t)a->block_m * a->stride_am * es >= (1ll << 32)) return 0;
  const bool a_aligned = (a->stride_am * es) % 16 == 0 && !((uintptr_t)a->a & 15) && !((uintptr_t)a->b & 15);
  if (a->stride_bn == 1 && a->stride_bk >= 0 &&
      (int64_t)a->block_k * a->stride_bk * es + (int64_t)a->block_n * es < (1ll << 32)) {
    const bool strict = a_aligned && a->k % a->block_k == 0 && (a->stride_bk * es) % 16 == 0 && a->n % vec == 0 && a->n >= vec;
    if (strict) return 1;
    const bool loose_ok = tail && a->stride_am >= a->k && a->stride_bk >= a->n;
    if (loose_ok) {
      *tail = true;
      return 1;
    }
  }
  if (a->stride_bk == 1 && a->stride_bn >= 0 && (int64_t)a->block_n * a->stride_bn * es + (int64_t)a->block_k * es < (1ll << 32)) {
    if (a_aligned && a->k % a->block_k == 0 && (a->stride_bn * es) % 16 == 0) return 2;
    // the same relaxation for a k-contiguous B: rows of B^T at any alignment, any K
    if (tail && a->stride_am >= a->k && a->stride_bn >= a->k) {
      *tail = true;
      return 2;
    }
  }
  return 0;
}
extern "C" int64_t tnx_gemm_lds_bytes(const tnx_gemm_args* a) {
  if (!a) return -1;
  return lds_bytes_of(a);
}

// tiles that are cut along K: all of them, or the last tail_tiles in launch order
static int64_t cut_tiles(const tnx_gemm_args* a) {
  if (a->block_m <= 0 || a->block_n <= 0) return 0;
  int64_t tiles = ((a->m + a->block_m - 1) / a->block_m) * ((a->n + a->block_n - 1) / a->block_n);
  if (a->split_k <= 1) return 0;
  return a->tail_tiles > 0 && a->tail_tiles < tiles ? a->tail_tiles : tiles;
}

extern "C" size_t tnx_gemm_workspace_bytes(const tnx_gemm_args* a) {
  if (!a || a->split_k <= 1 || a->m <= 0 || a->n <= 0) return 0;
  if (is_skinny_cfg(a)) return 0;   // the eight K slices meet in LDS
  // every slice of a cut tile is kept whole (block_m x block_n accumulators of 4 bytes)
  return (size_t)WS_COUNTER_BYTES + (size_t)a->split_k * (size_t)cut_tiles(a) * (size_t)a->block_m * (size_t)a->block_n * 4;
}

static int supported_impl(const tnx_gemm_args* a, const KernelEntry** out, bool* fast, bool inspect_ptrs, bool* bt = nullptr,
                          bool* tail = nullptr) {
  if (bt) *bt = false;
  if (tail) *tail = false;
  int st = check_common(a);
  if (st != TNX_OK) return st;
  int64_t lds = lds_bytes_of(a);
  if (lds > TNX_LDS_LIMIT_BYTES) return TNX_E_LDS;
  if (is_skinny_cfg(a)) {
    // m <= 16 rows, K cut eight ways inside the workgroup, DMA loader only
    if (a->split_k != SKINNY_SPLIT || a->epilogue != TNX_EPI_NONE || a->in_dtype == TNX_I8) return TNX_E_UNSUPPORTED;
    if (!skinny_lookup(a->in_dtype, a->num_stages)) return TNX_E_UNSUPPORTED;
    if (a->m > SKINNY_BM || a->m < 1 || a->n % SKINNY_BN != 0 || a->k % (SKINNY_SPLIT * SKINNY_BK) != 0 || a->k == 0)
      return TNX_E_UNSUPPORTED;
    if (a->stride_ak != 1 || a->stride_bn != 1 || (a->stride_am * 2) % 16 != 0 || (a->stride_bk * 2) % 16 != 0 ||
        a->stride_am < 0 || a->stride_bk < 0)
      return TNX_E_UNSUPPORTED;
    if (inspect_ptrs && ((((uintptr_t)a->a) & 15) || (((uintptr_t)a->b) & 15))) return TNX_E_UNSUPPORTED;
    if ((int64_t)SKINNY_BK * a->stride_bk * 2 >= (1ll << 32) || (int64_t)SKINNY_BM * a->stride_am * 2 >= (1ll << 32))
      return TNX_E_UNSUPPORTED;
    if (out) *out = nullptr;
    if (fast) *fast = true;
    return TNX_OK;
  }
  const KernelEntry* e = find_entry(a);
  if (!e) return TNX_E_UNSUPPORTED;
  tnx_gemm_args tmp = *a;
  if (!inspect_ptrs) { tmp.a = nullptr; tmp.b = nullptr; }
  bool tail_slab = false;
  // the persistent kernel keeps the strict layout
  const int layout = dma_layout(&tmp, (a->schedule & TNX_SCHED_PERSISTENT) ? nullptr : &tail_slab);
  if (tail) *tail = tail_slab;
  bool f = layout == 1 || (layout == 2 && e->fast_bt);
  if (!f && !e->generic) return TNX_E_UNSUPPORTED;
  if (a->schedule & TNX_SCHED_PERSISTENT) {
    if (!e->persist || layout != 1 || a->split_k != 1 || a->k < (int64_t)a->num_stages * a->block_k) return TNX_E_UNSUPPORTED;
  }
  if (bt) *bt = f && layout == 2;
  int64_t tiles = ((a->m + a->block_m - 1) / a->block_m) * ((a->n + a->block_n - 1) / a->block_n);
  if (tiles * a->split_k > 0x7fffffffll) return TNX_E_UNSUPPORTED;
  if (cut_tiles(a) > WS_MAX_TILES) return TNX_E_UNSUPPORTED;  // one arrival counter per cut tile
  if (tnx_gemm_workspace_bytes(a) >= (1ull << 32)) return TNX_E_UNSUPPORTED;  // slices are addressed with 32-bit offsets
  if (out) *out = e;
  if (fast) *fast = f;
  return TNX_OK;
}

// CUs of the current device (the persistent kernel launches one workgroup per CU); looked up once per device
static int compute_units(int* out) {
  static int cached[64];
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) { g_last_hip_error = (int)err; return TNX_E_HIP; }
  if (dev < 0 || dev >= 64) return TNX_E_UNSUPPORTED;
  if (!cached[dev]) {
    int n = 0;
    err = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess || n <= 0) { g_last_hip_error = (int)err; return TNX_E_HIP; }
    cached[dev] = n;
  }
  *out = cached[dev];
  return TNX_OK;
}

extern "C" int tnx_gemm_supported(const tnx_gemm_args* a) { return supported_impl(a, nullptr, nullptr, false); }

extern "C" int tnx_gemm(const tnx_gemm_args* a) { return tnx::gemm_launch(a, nullptr); }

bool tnx::gemm_tile_for(int dtype, int bm, int bn, int bk, int* num_warps, int* num_stages) {
  int ng = 0;
  const KernelGroup* g = tnx_kernel_groups(&ng);
  const KernelEntry* best = nullptr;
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < g[i].count; ++j) {
      const KernelEntry& e = g[i].entries[j];
      if (e.dtype != dtype || e.bm != bm || e.bn != bn || e.bk != bk || !e.fast || e.bm * e.bn > 128 * 128) continue;
      // Eight waves and two ring slots first, then the shallowest ring: these problems stream their operands once
      // through a short K loop, and what hides the latency of a tile's first slab and of its stores is more waves and a
      // second workgroup on the CU, not a deeper ring (measured on GEMMs shaped like the 1x1 layers of a ResNet-50:
      // 128x128x64 with 8 waves / 2 slots 39 us, 4 / 2 43 us, 4 / 3 75 us on [512 x 256] x [256 x 100352])
      // A 64x64 tile is too little work for eight waves: four waves and three slots there (measured on the small
      // layers, 2048 -> 512 channels at 7x7: 16.3 against 21.9 us).
      auto score = [](const KernelEntry& k) {
        const bool small = k.bm * k.bn <= 64 * 64;
        return (k.nw == (small ? 4 : 8) ? 100 : 0) + (k.stages == (small ? 3 : 2) ? 50 : 0) - k.stages;
      };
      if (!best || score(e) > score(*best)) best = &e;
    }
  if (!best) return false;
  *num_warps = best->nw;
  *num_stages = best->stages;
  return true;
}

int tnx::gemm_launch(const tnx_gemm_args* a, const GemmBatch* extra) {
  const KernelEntry* e = nullptr;
  bool fast = false, bt = false, tail_slab = false;
  int st = supported_impl(a, &e, &fast, true, &bt, &tail_slab);
  if (st != TNX_OK) return st;
  if (extra && (e->bm * e->bn > 128 * 128 || a->split_k != 1 || (a->schedule & TNX_SCHED_PERSISTENT) || is_skinny_cfg(a) || extra->batch < 1 ||
                a->epilogue != TNX_EPI_NONE || (extra->bias && a->in_dtype == TNX_I8)))
    return TNX_E_UNSUPPORTED;
  if (!a->a || !a->b || !a->c) {
    if (a->m == 0 || a->n == 0) return TNX_OK;
    if (!a->c || (a->k > 0 && (!a->a || !a->b))) return TNX_E_INVALID;
  }
  if (a->m == 0 || a->n == 0) return TNX_OK;
  if (tnx_gemm_workspace_bytes(a) > 0 &&
      (!a->workspace || a->workspace_bytes < tnx_gemm_workspace_bytes(a) || ((uintptr_t)a->workspace & 255)))
    return TNX_E_WORKSPACE;

  const int es_out = elem_size(a->out_dtype);
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t*)a->a;
  p.b = (const uint8_t*)a->b;
  p.c = (uint8_t*)a->c;
  p.ws = (uint8_t*)a->workspace;
  p.m = a->m; p.n = a->n; p.k = a->k;
  p.sam = a->stride_am; p.sak = a->stride_ak;
  p.sbk = a->stride_bk; p.sbn = a->stride_bn;
  p.scm = a->stride_cm; p.scn = a->stride_cn;
  p.tiles_m = (int)((a->m + a->block_m - 1) / a->block_m);
  p.tiles_n = (int)((a->n + a->block_n - 1) / a->block_n);
  p.group_m = a->group_m;
  p.split_k = a->split_k;
  const int64_t ncut = cut_tiles(a);
  p.split_tile0 = a->split_k > 1 ? (int)((int64_t)p.tiles_m * p.tiles_n - ncut) : 0;
  int kt_total = (int)((a->k + a->block_k - 1) / a->block_k);
  p.ktiles_per_split = (kt_total + a->split_k - 1) / a->split_k;
  p.epilogue = a->epilogue;
  p.out_dtype = a->out_dtype;
  p.b_once = p.tiles_m == 1;
  p.tile_order = (a->schedule & TNX_SCHED_SUPERBLOCK) && a->split_k == 1 ? 1 : 0;
  p.atomic_reduce = (a->schedule & TNX_SCHED_ATOMIC_REDUCE) && a->split_k > 1 ? 1 : 0;
  p.c_vec_ok = a->stride_cn == 1 && ((a->stride_cm * es_out) % 16) == 0 && (((uintptr_t)a->c) % 16) == 0;
  p.c_row_ok = a->stride_cn == 1;
  p.tail_slab = tail_slab ? 1 : 0;
  int64_t problems = 1;
  if (extra) {
    p.batch = extra->batch;
    p.b_batch_bytes = extra->b_batch_bytes;
    p.c_batch_bytes = extra->c_batch_bytes;
    p.cv.bias = (const uint8_t*)extra->bias;
    p.cv.bias_dtype = extra->bias_dtype;
    problems = extra->batch;
    if ((int64_t)p.tiles_m * p.tiles_n * problems > 0x7fffffffll) return TNX_E_UNSUPPORTED;
  }

  hipStream_t stream = (hipStream_t)a->stream;
  hipError_t err;
  if (is_skinny_cfg(a)) {
    err = skinny_lookup(a->in_dtype, a->num_stages)(p, (unsigned)(a->n / SKINNY_BN), stream);
  } else if (a->schedule & TNX_SCHED_PERSISTENT) {
    int cus = 0;
    const int st2 = compute_units(&cus);
    if (st2 != TNX_OK) return st2;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    err = e->persist(p, (unsigned)(tiles < cus ? tiles : cus), stream);
  } else {
    unsigned grid = a->split_k > 1 ? (unsigned)(p.split_tile0 + ncut * a->split_k) : (unsigned)((int64_t)p.tiles_m * p.tiles_n * problems);
    err = (bt ? e->fast_bt : fast ? e->fast : e->generic)(p, grid, stream);
  }
  if (err != hipSuccess) { g_last_hip_error = (int)err; return TNX_E_HIP; }

  return TNX_OK;
}

// ---------------------------------------------------------------------------
// tnx_gemm_static_workspace: the split-K scratch lives in a file-scope device array instead of a
// caller-provided workspace, so the call allocates nothing.  `scratch` is a host-side handle here:
// the device address is looked up once per device with hipGetSymbolAddress and only that pointer
// is ever handed to kernels.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[TNX_STATIC_WORKSPACE_BYTES];

static constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mutex;

__global__ void zero_words_kernel(int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// device address of this device's copy of `scratch` (each GPU holds its own copy at its own address)
static int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) { g_last_hip_error = (int)err; return TNX_E_HIP; }
  if (dev < 0 || dev >= MAX_DEVICES) return TNX_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr) { g_last_hip_error = (int)err; return TNX_E_HIP; }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return TNX_OK;
}

extern "C" int tnx_gemm_static_workspace(const tnx_gemm_args* a) {
  if (!a) return TNX_E_INVALID;
  tnx_gemm_args t = *a;
  t.workspace = nullptr;
  t.workspace_bytes = 0;
  const size_t need = tnx_gemm_workspace_bytes(&t);
  if (need > 0) {
    if (need > (size_t)TNX_STATIC_WORKSPACE_BYTES) return TNX_E_STATIC_LIMIT;
    int st = supported_impl(&t, nullptr, nullptr, true);
    if (st != TNX_OK) return st;
    void* ptr = nullptr;
    st = scratch_of_current_device(&ptr);
    if (st != TNX_OK) return st;
    // The array keeps what the last call left.  The arrival counters of the tiles this launch cuts must
    // start at zero; a launch leaves them zero, but one that was aborted does not, so they are cleared
    // here with a small fill kernel (legal under graph capture, unlike a memset node).
    const int words = (int)cut_tiles(&t);
    hipLaunchKernelGGL(zero_words_kernel, dim3((words + 255) / 256), dim3(256), 0, (hipStream_t)t.stream, (int*)ptr, words);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) { g_last_hip_error = (int)err; return TNX_E_HIP; }
    if (t.schedule & TNX_SCHED_ATOMIC_REDUCE) {
      // The atomic reduction adds every slice into one copy behind the counters and needs that copy zero at
      // launch.  A launch of this kind leaves it zero, but the array may hold the slices of an earlier ordered
      // launch (or of another tile shape), so the copy this launch adds into is cleared first, same fill kernel.
      const int64_t sum_words = cut_tiles(&t) * (int64_t)t.block_m * t.block_n;   // < 2^23: need <= TNX_STATIC_WORKSPACE_BYTES
      hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((sum_words + 255) / 256)), dim3(256), 0, (hipStream_t)t.stream,
                         (int*)((unsigned char*)ptr + WS_COUNTER_BYTES), (int)sum_words);
      err = hipGetLastError();
      if (err != hipSuccess) { g_last_hip_error = (int)err; return TNX_E_HIP; }
    }
    t.workspace = ptr;
    t.workspace_bytes = TNX_STATIC_WORKSPACE_BYTES;
  }
  return tnx_gemm(&t);
}

extern "C" int tnx_gemm_default_config(tnx_gemm_args* a) {
  if (!a) return TNX_E_INVALID;
  const int es = elem_size(a->in_dtype);
  const int bk = es == 1 ? 128 : 64;   // 128 bytes of K per LDS row for either element size
  // Workgroups that run together: the CU count of the current device, or MI355X's 256 when no device can be asked
  // (host-side planning).  The cost constants below are measured on MI355X.
  int64_t cus = 256;
  {
    int n = 0;
    if (compute_units(&n) == TNX_OK && n > 0) cus = n;
  }
  a->group_m = 8;
  a->split_k = 1;
  a->tail_tiles = 0;
  a->schedule = TNX_SCHED_DEFAULT;
  a->block_k = bk;
  bool dma_ok;
  {
    tnx_gemm_args t = *a;   // a and b, when given, count with their base alignment (null = aligned)
    if (t.stride_ak == 0 && t.stride_bn == 0) { t.stride_am = t.k; t.stride_ak = 1; t.stride_bk = t.n; t.stride_bn = 1; }
    t.block_m = 128; t.block_n = 128; t.block_k = bk;
    bool tail_slab = false;
    dma_ok = dma_layout(&t, &tail_slab) != 0;     // every tile the choice below proposes is built for both DMA layouts
  }
  if (a->m <= 64 && dma_ok) {
    // skinny: B is streamed once; K is split until every CU owns one workgroup (measured on the
    // M=16, N=4096, K=14336 shape: 8 waves, 3 stages, 256 workgroups stream at the HBM read limit)
    a->block_m = 64; a->block_n = 128; a->num_stages = 3; a->num_warps = 8;
    int64_t tiles = (a->n + a->block_n - 1) / a->block_n;
    int64_t kt = (a->k + a->block_k - 1) / a->block_k;
    int s = 1;
    while (tiles * s < cus && s * 2 <= 16 && kt / (s * 2) >= 4) s *= 2;
    a->split_k = s;
    return TNX_OK;
  }
  // operands the DMA loader cannot take (not row-major with unit inner strides, int8 rows that are not 16-byte
  // aligned) go to one of the two tiles that are also built with the element-wise loader
  if (!dma_ok) {
    a->block_m = a->m <= 64 ? 64 : 128; a->block_n = 128; a->num_stages = 2; a->num_warps = 4;
    return TNX_OK;
  }
  // Pick the tile and the K cut with the smallest modelled time.  A wave is 256 workgroups (one per CU); a tile
  // costs its multiply-adds over the rate a CU sustains with that tile (relative rates measured on 8192^3 and
  // 2048^2 x 8192: 256x256 1.0, 256x128 0.9, 128x128 0.75); a last, partial wave costs 0.75 of a full one (the
  // part is power-limited: fewer busy CUs clock higher; measured 0.70-0.80 on 6144^3, 5120^2 x 8192,
  // 4096 x 5120 x 4096).  Cutting K costs a hand-over: a fixed 9 us plus the slices the finishing workgroup
  // reads back at about 60 GB/s.  Three shapes of launch are priced per tile: uncut; every tile cut (only when
  // the tiles alone leave CUs idle); only the tiles of the partial wave cut (tail_tiles).  Slices never get
  // shorter than eight K slabs.
  // (the sixth, 192x192, exists for the 16-bit types: it is what divides sides like 1536, 3072 or 4608 into whole
  // rounds -- 3072^3 is 144 tiles of 256x256 on 256 CUs, and 256 of these: measured 62 -> 47 us)
  // (192x256 and 256x192 likewise: 4096 x 2560 x 8192 is 160 tiles of 256x256, 0.63 of a round, and 220 of 192x256:
  // measured 141 -> 128 us; their rate lies between what they reach against 256x256 on 8192^3, 0.86, and on
  // launches of a round or two at K = 4096, where they run at the full 0.75 of its tile time)
  static const int cand[][4] = {{256, 256, 2, 4}, {256, 128, 3, 4}, {128, 128, 3, 4}, {64, 128, 3, 4}, {64, 64, 4, 4}, {192, 192, 3, 8},
                                {192, 256, 2, 8}, {256, 192, 2, 8}};
  static const double rate[] = {1.0, 0.9, 0.75, 0.5, 0.35, 0.92, 0.9, 0.9};
  const int ncand = 8;
  // int8: rows of a 64-wide B tile are too short for the transposing read; the 192-wide tiles exist for it too
  // (3072 x 4096 x 4096: 53.6 -> 45.7 us with 192x256, 4096 x 3072 x 4096: 52.8 -> 47.3 us with 256x192)
  // (a binary32 result exists on the tiles up to 128x128 only)
  auto usable = [&](int i) { return (es == 2 || i != 4) && (a->out_dtype != TNX_F32 || (i >= 2 && i <= 4)); };
  const double cu_flops = 5.5e12 * (es == 1 ? 1.7 : 1.0);          // per CU with the largest tile
  const double launch = 3e-6, handover = 9e-6, readback = 60e9;
  const int64_t kt = (a->k + bk - 1) / bk;
  double best = 1e300;
  int bi = es == 1 ? 3 : 4, bs = 1, btail = 0;
  auto offer = [&](double t, int i, int s, int tail) {
    if (t < best * 0.97) { best = t; bi = i; bs = s; btail = tail; }   // ties go to the earlier (larger, less cut) choice
  };
  // (The 0.75 holds for nearly full last waves of the large tiles too: 220 tiles of 192x256 on 256 CUs took 0.80 of a
  // full wave's time; a cost that rises with the fill, 0.7 + 0.3 * rem / 256, was tried on 382 shapes and moved a
  // third of 75 choices for the worse by up to 20 %.  The tiles up to 128x128 do not load the power limit, so their
  // partial wave runs no faster than a full one: 128 tiles of 64x128 took 0.91 of the modelled full wave where 256
  // tiles of 64x64 took 1.0 of theirs; they are priced at 0.9.)
  for (int i = 0; i < ncand; ++i) {
    if (!usable(i)) continue;
    const int64_t tiles = ((a->m + cand[i][0] - 1) / cand[i][0]) * ((a->n + cand[i][1] - 1) / cand[i][1]);
    const double tile_t = 2.0 * cand[i][0] * cand[i][1] * (double)a->k / (cu_flops * rate[i]);
    const double slice_bytes = (double)cand[i][0] * cand[i][1] * 4;
    const double part = (i >= 2 && i <= 4) ? 0.9 : 0.75;            // cost of a last, partial wave (see above)
    const int64_t full = tiles / cus, rem = tiles % cus;
    offer((double)full * tile_t + (rem ? part * tile_t : 0.0) + launch, i, 1, 0);
    for (int s = 2; s <= 16; s *= 2) {
      if (kt / s < 8) break;
      if (full == 0 && tiles * s <= cus)                             // every tile cut (one wave at most)
        offer(tile_t / s + handover + s * slice_bytes / readback + launch, i, s, 0);
      if (full > 0 && rem > 0 && rem * s <= cus)                     // only the partial wave cut
        offer((double)full * tile_t + tile_t / s + handover + s * slice_bytes / readback + launch, i, s, (int)rem);
    }
  }
  a->block_m = cand[bi][0]; a->block_n = cand[bi][1]; a->num_stages = cand[bi][2]; a->num_warps = cand[bi][3];
  // The 128x128 tile, and the 64x128 tile of the 16-bit types, run with eight waves: problems that end up on them are
  // a few rounds of short tiles, and two waves per SIMD hide more of a tile's start and end than one (measured on
  // fifteen bf16 shapes from 768x3072x768 to 1024x4096x4096, three ring slots both: 1-14 % faster on every one, e.g.
  // 2048^3 21.2 -> 19.6 us, 2048^2 x 512 9.4 -> 8.1 us, 1024^3 9.1 -> 7.9 us; int8 128x128 5-13 % on seven shapes,
  // int8 64x128 mixed).
  if (bi == 2 || (es == 2 && bi == 3)) a->num_warps = 8;
  // 16-bit problems with a short K loop (at most 64 slabs per tile) spend a visible share of every tile outside
  // it; two waves per SIMD cover that better than one (measured on 4096 x 28672 x 4096, gated: +2.4 %), at the
  // price of half again as many LDS reads, which is what loses on the long, power-limited 8192^3 loops.
  // (cut tiles too: 4096 x 5120 x 4096 with its last 64 tiles cut, 155 -> 140 us)
  if (es == 2 && bi == 0 && kt <= 64) a->num_warps = 8;
  a->split_k = bs;
  a->tail_tiles = btail;
  // Grids of several rounds of 256 tiles in both directions: the super-block order keeps what one round reads
  // to 16 + 16 operand panels and lets consecutive rounds share half of them (measured on 8192^3: int8 +4 %,
  // bf16 unchanged on random operands -- that launch is limited by board power -- and +12 % on operands that
  // draw less power; never slower).  The persistent schedule is not chosen: measured 1-3 % slower on the
  // benchmark shapes (it gives up the dynamic hand-out of tiles to whichever CU is free).
  {
    const int64_t tm = (a->m + a->block_m - 1) / a->block_m, tn = (a->n + a->block_n - 1) / a->block_n;
    if (bs == 1 && tm >= 16 && tn >= 16) a->schedule = TNX_SCHED_SUPERBLOCK;
  }
  return TNX_OK;
}

// ---------------------------------------------------------------------------
// float32 operands as bf16 head and tail (see tnx_split_f32 in the header)
// ---------------------------------------------------------------------------
__global__ void split_f32_kernel(const float* src, int64_t rows, int64_t cols, int64_t sr, int64_t sc, uint16_t* dst, int side) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= rows * cols) return;
  const int64_t i = idx / cols, j = idx - i * cols;
  const float v = src[i * sr + j * sc];
  const __bf16 hi = (__bf16)v;                                        // round to nearest even
  const float rest = v - (float)hi;
  // An infinity or NaN lives in the head alone: its tail is zero, and so is the second copy of its head -- the one
  // that meets the other operand's tail -- or inf * (a tail that happens to be 0) would turn an infinite sum into NaN.
  const bool fin = __builtin_isfinite(rest) && __builtin_isfinite((float)hi);
  const __bf16 lo = fin ? (__bf16)rest : (__bf16)0.0f;
  const uint16_t h = __builtin_bit_cast(uint16_t, hi), l = __builtin_bit_cast(uint16_t, lo);
  const uint16_t h2 = fin ? h : (uint16_t)0;
  if (side == 0 || side == 2) {
    uint16_t* row = dst + i * 3 * cols;
    row[j] = h;
    row[cols + j] = side == 0 ? h2 : l;
    row[2 * cols + j] = side == 0 ? l : h2;
  } else {
    dst[i * cols + j] = h;
    dst[(rows + i) * cols + j] = l;
    dst[(2 * rows + i) * cols + j] = h2;
  }
}

extern "C" int tnx_split_f32(const float* src, int64_t rows, int64_t cols, int64_t stride_r, int64_t stride_c, void* dst, int side,
                             void* stream) {
  if (rows < 0 || cols < 0 || side < 0 || side > 2) return TNX_E_INVALID;
  if (rows == 0 || cols == 0) return TNX_OK;
  if (!src || !dst) return TNX_E_INVALID;
  const int64_t total = rows * cols;
  if (rows > 0x7fffffff || cols > 0x7fffffff || (total + 255) / 256 > 0x7fffffffll) return TNX_E_UNSUPPORTED;
  hipLaunchKernelGGL(split_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, src, rows, cols,
                     stride_r, stride_c, (uint16_t*)dst, side);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) { g_last_hip_error = (int)err; return TNX_E_HIP; }
  return TNX_OK;
}

extern "C" int tnx_tile_coords(int schedule, int id, int tiles_m, int tiles_n, int group_m, int* tile_m, int* tile_n) {
  if (!tile_m || !tile_n || tiles_m <= 0 || tiles_n <= 0 || group_m <= 0 || id < 0 ||
      (int64_t)id >= (int64_t)tiles_m * tiles_n || (int64_t)tiles_m * tiles_n > 0x7fffffffll)
    return TNX_E_INVALID;
  // the same functions the kernels call (gemm_tile.h), compiled for the host
  if (schedule & TNX_SCHED_SUPERBLOCK) {
    superblock_order(id, tiles_m, tiles_n, tile_m, tile_n);
  } else {
    const int logical = xcd_remap(id, tiles_m * tiles_n, 8);
    swizzle2d(logical / tiles_n, logical % tiles_n, tiles_m, tiles_n, group_m, tile_m, tile_n);
  }
  return TNX_OK;
}

extern "C" int tnx_kernel_count(void) {
  int ng = 0, n = 0;
  const KernelGroup* g = tnx_kernel_groups(&ng);
  for (int i = 0; i < ng; ++i) n += g[i].count;
  return n;
}

extern "C" const char* tnx_kernel_name(int idx) {
  static thread_local char buf[96];
  int ng = 0;
  const KernelGroup* g = tnx_kernel_groups(&ng);
  for (int i = 0; i < ng; ++i) {
    if (idx < g[i].count) {
      const KernelEntry& e = g[i].entries[idx];
      const char* dn = e.dtype == TNX_F16 ? "f16" : e.dtype == TNX_BF16 ? "bf16" : "i8";
      snprintf(buf, sizeof(buf), "%s %d %d %d %d %d%s%s", dn, e.bm, e.bn, e.bk, e.nw, e.stages, e.generic ? " generic" : "",
               e.persist ? " persistent" : "");
      if (e.fast_bt) strncat(buf, " bt", sizeof(buf) - strlen(buf) - 1);
      return buf;
    }
    idx -= g[i].count;
  }
  return nullptr;
}

extern "C" const char* tnx_strerror(int status) {
  switch (status) {
    case TNX_OK: return "ok";
    case TNX_E_INVALID: return "invalid argument";
    case TNX_E_UNSUPPORTED: return "no kernel is built for this tile / dtype / layout";
    case TNX_E_LDS: return "tile configuration exceeds the per-CU LDS budget";
    case TNX_E_WORKSPACE: return "split-K workspace missing or too small";
    case TNX_E_HIP: return "HIP runtime error";
    case TNX_E_STATIC_LIMIT: return "split-K scratch of this launch exceeds TNX_STATIC_WORKSPACE_BYTES (use tnx_gemm with a workspace)";
    default: return "unknown status";
  }
}

extern "C" int tnx_last_hip_error(void) { return g_last_hip_error; }
extern "C" int tnx_version(void) { return TNX_VERSION; }
