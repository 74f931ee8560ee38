// Tiled GEMM for gfx950 (MI355X): C[m,n] = A[m,k] @ B[k,n], optional split-K
// partials and a fused GLU epilogue.
//
// What it computes follows tritonix/ops/matmul.py:43-108 (matmul_kernel),
// :147-202 (gemm_splitk_kernel) and tritonix/ops/swiglu.py:24-110 (glu_kernel):
// a block_m x block_n output tile per workgroup, a K loop of block_k slabs with
// fp32 (int32 for int8) accumulation, an M/N-masked store.  How it computes it
// is specific to CDNA4:
//   * global -> LDS with the 16-byte direct-to-LDS load (no VGPR staging), a
//     ring of STAGES LDS slabs, one workgroup barrier per K slab;
//   * A fragments with ds_read_b128, B fragments (B is row-major [k,n], MFMA
//     wants k-contiguous lanes) with the transposing ds_read_b64_tr_b16/_b8;
//   * XOR-swizzled 16-byte chunks so neither the DMA writes nor the fragment
//     reads collide on LDS banks;
//   * v_mfma_f32_16x16x32 (bf16/f16) and v_mfma_i32_16x16x64_i8 (the 32x32 shapes
//     stay selectable through TileCfg::MI);
//   * a 1-D grid whose block index is remapped XCD-first, then by the
//     group-M order of tl.swizzle2d (tritonix/ops/matmul.py:70).
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

// Attribution builds (never the shipped library): -D TNX_LADDER=n strips the K loop of the DMA kernels down to a rung
// of the ladder  1: MFMAs only (both fragment sets filled once from the first slab)  2: + the fragment reads from
// LDS and the per-slab barrier, no refill of the ring  3: + the refill, but always of the tile's first slabs, so every
// load is served by the L2  4: the full loop without its waits for the loads  (0: the kernel as shipped).  Results
// of rungs 1-4 are wrong on purpose; they are timed with power and clock sampling beside the full kernel to say
// what each part of the loop costs on a power-limited board.
#ifndef TNX_LADDER
#define TNX_LADDER 0
#endif
// Development schedule (never the shipped library): -D TNX_PINGPONG=1 runs the K loop of the eight-wave two-slot
// tiles with two k steps per slab as a ping-pong: the two waves of every SIMD alternate, a barrier apart, between
// reading a whole slab's fragments from LDS and multiplying them at raised priority (see pingpong_loop).  Values
// above 1 are its attribution forms: 2 priority not raised; 3 without the fragment reads, 4 without the DMA refill,
// 5 without the MFMAs (3-5: wrong results on purpose).  Measured, it loses to the interleaved loop on every operand.
#ifndef TNX_PINGPONG
#define TNX_PINGPONG 0
#endif

namespace tnx {

typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

#define TNX_LDS(T, addr) ((T __attribute__((address_space(3)))*)(uintptr_t)(addr))

enum { DT_F16 = 0, DT_BF16 = 1, DT_I8 = 2, DT_I32 = 3, DT_F32 = 4 };
enum { EPI_NONE = 0, EPI_GLU_SILU = 1, EPI_GLU_SIGMOID = 2, EPI_GLU_IDENTITY = 3 };

// n / d for 0 <= n < 2^31 by multiply-high and shift (d >= 1); built on the host.
struct FastDiv {
  uint32_t mul, shift;
};
inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f = {0u, 0u};
  if (d <= 1) return f;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.shift = s;
  f.mul = (uint32_t)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
  return f;
}
__host__ __device__ __forceinline__ uint32_t fd_div(uint32_t n, FastDiv f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (__umulhi(n, f.mul) + n) >> f.shift;
#else
  return (uint32_t)((((uint64_t)n * f.mul) >> 32) + n) >> f.shift;
#endif
}

// Geometry of a conv2d forward run on the GEMM kernel (gemm_tile_kernel<..., CONV>): A is the KCRS weight as
// [c_out, c_in*R*S], the B operand is generated from the NCHW input by the DMA loader, column n of the product is
// pixel (image, h_out, w) of a pixel index space whose rows are `wp` wide (w_out rounded up to 8, so that a 16-byte
// chunk of 8 pixels never leaves its output row; the pixels w >= w_out of a row are computed and dropped).
struct ConvGeom {
  int h_in, w_in, c_out, h_out, w_out, wp;
  int stride_h, pad_h, pad_w;
  int hw_in, chw_in;               // h_in*w_in, c_in*h_in*w_in
  int n_total;                     // batch * h_out * wp
  uint32_t x_bytes;                // size of the input tensor
  FastDiv div_hwp, div_wp;         // by h_out*wp, by wp
  FastDiv div_rs, div_s;           // by R*S, by S
  int rs, fw, dil_h, dil_w;
  // one K slab (block_k rows) further along k: what is added to a tap's (dw, dh, element offset), the limits at which
  // dw and dh wrap, and what a wrap adds to the element offset
  int step_dw, step_dh, step_koff, lim_w, lim_h, adj_w, adj_h;
  const uint8_t* bias;             // [c_out] or null
  int bias_dtype;
};

struct GemmParams {
  const uint8_t* a;
  const uint8_t* b;
  uint8_t* c;
  uint8_t* ws;            // split-K workspace: tile counters, then the slices [slice][cut tile][wave][group][lane]
  int64_t m, n, k;
  int64_t sam, sak;       // element strides of A
  int64_t sbk, sbn;       // element strides of B
  int64_t scm, scn;       // element strides of C
  int tiles_m, tiles_n;
  int group_m;
  int split_k;
  int split_tile0;        // tiles [0, split_tile0) in launch order are computed whole; the rest are cut split_k ways
  int ktiles_per_split;   // K slabs handled by one split
  int epilogue;
  int out_dtype;
  bool c_vec_ok;          // C takes 16-byte stores along n (stride_cn == 1, 16-byte aligned rows)
  bool c_row_ok;          // stride_cn == 1: rows of C take 16-byte stores at the element's own alignment
  int tail_slab;          // DMA kernels: the last K slab (whole or partial) goes through the element-wise loader
  bool b_once;            // every element of B is read by exactly one workgroup (one tile row): stream it non-temporally
  int tile_order;         // 0: XCD remap + tl.swizzle2d(group_m); 1: 16x16 super-blocks in serpentine order (superblock_order)
  int atomic_reduce;      // split-K: slices are added into one fp32/int32 copy with device-scope atomics instead of being kept apart
  int batch;              // uncut, non-persistent launches of tiles up to 128x128: the grid holds `batch` problems that share A (0 or 1: one problem);
  int64_t b_batch_bytes, c_batch_bytes;   // problem i reads B + i * b_batch_bytes and writes C + i * c_batch_bytes
  ConvGeom cv;            // read by the CONV kernels; cv.bias / cv.bias_dtype also by the plain epilogue (a bias per row of C)
};

// ---------------------------------------------------------------------------
// element tags
// ---------------------------------------------------------------------------
struct TagF16 { static constexpr int ES = 2; static constexpr int ID = DT_F16; typedef float acc_s; };
struct TagBF16 { static constexpr int ES = 2; static constexpr int ID = DT_BF16; typedef float acc_s; };
struct TagI8 { static constexpr int ES = 1; static constexpr int ID = DT_I8; typedef int acc_s; };

template <class T, int MI> struct Mma;
template <> struct Mma<TagBF16, 32> {
  typedef f32x16 acc_t;
  static __device__ __forceinline__ acc_t run(i32x4 a, i32x4 b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<TagBF16, 16> {
  typedef f32x4 acc_t;
  static __device__ __forceinline__ acc_t run(i32x4 a, i32x4 b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<TagF16, 32> {
  typedef f32x16 acc_t;
  static __device__ __forceinline__ acc_t run(i32x4 a, i32x4 b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<TagF16, 16> {
  typedef f32x4 acc_t;
  static __device__ __forceinline__ acc_t run(i32x4 a, i32x4 b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<TagI8, 32> {
  typedef i32x16 acc_t;
  static __device__ __forceinline__ acc_t run(i32x4 a, i32x4 b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
template <> struct Mma<TagI8, 16> {
  typedef i32x4 acc_t;
  static __device__ __forceinline__ acc_t run(i32x4 a, i32x4 b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
};

// ---------------------------------------------------------------------------
// tile-id remap.  Workgroups are dealt round-robin to the 8 XCDs (each has its
// own L2), so consecutive *logical* tile ids are first gathered per XCD, then
// ordered group-M-first exactly like tl.swizzle2d on the row-major tile index
// (triton/language/standard.py:80-116, called at tritonix/ops/matmul.py:70).
// ---------------------------------------------------------------------------
__host__ __device__ inline int xcd_remap(int pid, int total, int nxcd) {
  int q = total / nxcd, r = total % nxcd;
  int x = pid % nxcd, idx = pid / nxcd;
  int start = x * q + (x < r ? x : r);
  return start + idx;
}

__host__ __device__ inline void swizzle2d(int i, int j, int size_i, int size_j, int size_g, int* oi, int* oj) {
  int ij = i * size_j + j;
  int size_gj = size_g * size_j;
  int group_id = ij / size_gj;
  int off_i = group_id * size_g;
  int g = size_i - off_i < size_g ? size_i - off_i : size_g;
  int r = ij % size_gj;
  *oi = off_i + r % g;
  *oj = r / g;
}

// Chip-level tile order for grids much larger than the CU count.  The 256 workgroups that run
// together (one per CU) take one 16x16 super-block of tiles, so one "round" touches 16 row panels
// of A and 16 column panels of B; super-blocks are walked in serpentine order, so consecutive
// rounds share half of their operands (which then come from the 256 MiB memory-side cache instead
// of HBM); inside a super-block each XCD owns an 8x4 sub-block (12 panels through its L2).
// A bijection from [0, tiles_m*tiles_n) onto the tile grid for every grid size.
__host__ __device__ inline void superblock_order(int pid, int tiles_m, int tiles_n, int* pm, int* pn) {
  constexpr int SB = 16, CHUNK = SB * SB;
  const int total = tiles_m * tiles_n;
  // ids congruent mod 8 (one XCD) become one run inside each aligned chunk of 256 ids
  const int chunk0 = pid - pid % CHUNK;
  const int csize = total - chunk0 < CHUNK ? total - chunk0 : CHUNK;
  const int s = chunk0 + xcd_remap(pid - chunk0, csize, 8);
  // s-th tile of the walk: rows of super-blocks top to bottom, alternating direction
  const int row_tiles = SB * tiles_n;
  const int i = s / row_tiles;
  int rem = s - i * row_tiles;
  const int h = tiles_m - i * SB < SB ? tiles_m - i * SB : SB;
  const int nsb = (tiles_n + SB - 1) / SB;
  const int wlast = tiles_n - (nsb - 1) * SB;
  const bool rev = i & 1;
  int jw, w;
  if (!rev) {
    jw = rem / (h * SB);
    if (jw > nsb - 1) jw = nsb - 1;
    w = jw == nsb - 1 ? wlast : SB;
    rem -= jw * h * SB;
  } else if (rem < h * wlast) {
    jw = 0;
    w = wlast;
  } else {
    rem -= h * wlast;
    jw = 1 + rem / (h * SB);
    w = SB;
    rem -= (jw - 1) * h * SB;
  }
  const int j = rev ? nsb - 1 - jw : jw;
  int r, c;
  if (h == SB && w == SB) {
    const int sub = rem / 32, idx = rem % 32;     // XCD sub-block: 2 x 4 of them, each 8 rows x 4 columns, walked down the rows
    r = 8 * (sub / 4) + idx % 8;
    c = 4 * (sub % 4) + idx / 8;
  } else {
    r = rem % h;
    c = rem / h;
  }
  *pm = i * SB + r;
  *pn = j * SB + c;
}

// vmcnt-only wait (lgkmcnt and expcnt left at "no wait") in the gfx9 encoding
#define TNX_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | ((((n) >> 4) & 0x3) << 14) | 0x0F70)

// 16 bytes per lane, global -> LDS without touching VGPRs.  LDS destination is
// lds_base + lane*16 (lds_base wave-uniform, carried in M0).  M0 is written inside the asm and
// cannot be named as clobbered (the compiler reserves it and rejects it in a clobber list); that
// is sound only while no compiler-generated instruction of these kernels reads M0 -- none does
// (no register-indexed arrays, no LDS-direct or GWS operations: every array is fully unrolled).
// The builtin form of this load is not used because the compiler then waits for vmcnt(0) before
// every later LDS read, which serialises the ring.
__device__ __forceinline__ void dma16(const uint8_t* sbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base), "v"(voff), "s"(sbase)
               : "memory");
}

// The same load in two parts, so that a useful instruction (an LDS read) can take the place of the wait
// state the hardware needs between the write of M0 and the load that uses it.  Nothing that reads or
// writes M0 may be placed between the two.
__device__ __forceinline__ void dma16_set_m0(uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0" : : "s"(lds_base) : "memory");
}
template <bool NT> __device__ __forceinline__ void dma16_go(const uint8_t* sbase, uint32_t voff) {
  if (NT) asm volatile("global_load_lds_dwordx4 %0, %1 nt" : : "v"(voff), "s"(sbase) : "memory");
  else asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(sbase) : "memory");
}

// same, with the non-temporal hint: for an operand that is streamed from HBM once and never reused
__device__ __forceinline__ void dma16_nt(const uint8_t* sbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :
               : "s"(lds_base), "v"(voff), "s"(sbase)
               : "memory");
}

__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
  uint64_t v = (uint64_t)(uintptr_t)p;
  uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// Device-scope (all XCDs) 16-byte accesses for data that workgroups hand to each other inside one kernel,
// as raw buffer operations with the sc1 bit: on gfx942/gfx950 that is the encoding of a monotonic atomic
// access at agent scope (the store writes through the XCD's L2, the load does not hit a stale line of it),
// so no whole-cache write-back or invalidate is needed around them.  They are compiler builtins, so the
// compiler itself places the s_waitcnt before the first use of a loaded value.
constexpr int CPOL_SC1 = 16;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t agent_window(const void* base) {
  // raw buffer (stride 0) of 4 GiB - 1 bytes starting at base; offsets are unsigned 32-bit
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
}
__device__ __forceinline__ void store16_agent(__amdgpu_buffer_rsrc_t w, uint32_t off, i32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, w, off, 0, CPOL_SC1);
}
__device__ __forceinline__ i32x4 load16_agent(__amdgpu_buffer_rsrc_t w, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b128(w, off, 0, CPOL_SC1);
}

// 16 bytes of C, stored with the non-temporal hint.  C is written once and never read by the kernel; without the
// hint its lines are kept in the L2 and the memory-side cache and push out operand panels that the other tiles of the
// round still need.  Measured on the 8192^3 bf16 problem: 1531 -> 1595 TFLOP/s on data-like operands (power-limited),
// 1712 -> 2026 on all-zero operands (clock at its maximum: the memory side decides); the gated GEMM 1414 -> 1475,
// int8 2798 -> 2845 TOP/s.  (The same hint on the B *loads* costs 4-20 %: operands are re-read.)
// A launch whose output the next launch reads at once (the feed-forward block's up-projection) loses that read's
// cache hits: the block's down-projection runs ~22 us slower, less than the ~30 us its up-projection gains.
// (A run-time switch `if (keep) plain store else hinted store` is no way to have both: the compiler sinks the two
// stores into one and drops the hint, measured as the full loss of the gain.)
typedef i32x4 __attribute__((aligned(2))) i32x4_loose;
typedef i32x4 __attribute__((aligned(1))) i32x4_bytes;
__device__ __forceinline__ void store16_stream(void* dst, i32x4 v) { __builtin_nontemporal_store(v, (i32x4*)dst); }
__device__ __forceinline__ void store16_stream_loose(void* dst, i32x4 v) { __builtin_nontemporal_store(v, (i32x4_loose*)dst); }

template <int ES> __device__ __forceinline__ i32x2 lds_read_tr(uint32_t addr);
template <> __device__ __forceinline__ i32x2 lds_read_tr<2>(uint32_t addr) {
  return __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(TNX_LDS(i16x4, addr)));
}
template <> __device__ __forceinline__ i32x2 lds_read_tr<1>(uint32_t addr) {
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32(TNX_LDS(i32x2, addr));
}

__device__ __forceinline__ float quad_swap1(float v) {
  // lanes (0,1,2,3) <- (1,0,3,2)
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}

__device__ __forceinline__ float glu_gate(float g, int epi) {
  if (epi == EPI_GLU_IDENTITY) return g;
  float s = 1.0f / (1.0f + __expf(-g));
  return epi == EPI_GLU_SILU ? g * s : s;
}

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                             // round to nearest even
  return (uint16_t)(u >> 16);
}

template <class ACC> __device__ __forceinline__ void store_out(uint8_t* c, int64_t off, ACC v, int out_dtype);
template <> __device__ __forceinline__ void store_out<float>(uint8_t* c, int64_t off, float v, int out_dtype) {
  if (out_dtype == DT_BF16) ((uint16_t*)c)[off] = f32_to_bf16(v);
  else if (out_dtype == DT_F16) ((_Float16*)c)[off] = (_Float16)v;
  else ((float*)c)[off] = v;
}
template <> __device__ __forceinline__ void store_out<int>(uint8_t* c, int64_t off, int v, int out_dtype) {
  ((int*)c)[off] = v;
}

// ---------------------------------------------------------------------------
// static description of one tile configuration
// ---------------------------------------------------------------------------
template <class T, int BM_, int BN_, int BK_, int NW_, int STAGES_>
struct TileCfg {
  static constexpr int ES = T::ES;
  static constexpr int BM = BM_, BN = BN_, BK = BK_, NW = NW_, STAGES = STAGES_;
  static constexpr int THREADS = NW * 64;
  static constexpr int WGM = (NW == 4) ? 2 : (BM > BN ? 4 : 2);  // wave grid
  static constexpr int WGN = NW / WGM;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;            // wave tile
  // MFMA shape: 16x16 (x32 for 16-bit, x64 for int8).  With operands that toggle like real data the part runs
  // against its board-power limit, and per multiply-add the 16x16 instructions draw measurably less than the
  // 32x32 ones (an MFMA-only loop on random registers sustains 11-15 % more with them, for all three types),
  // which outweighs their four points of extra issue overhead.  The 32x32 code paths below stay usable
  // (MI = 32 needs WTM % 32 == 0 && WTN % 32 == 0).
  static constexpr int MI = 16;
  static constexpr int TM = WTM / MI, TN = WTN / MI;
  static constexpr int KB = (MI == 32) ? 32 : 64;                 // k bytes one MFMA consumes
  static constexpr int MMA_K = KB / ES;
  static constexpr int KSTEPS = (BK * ES) / KB;
  static constexpr int KGROUPS = 64 / MI;                         // lane groups along k
  static constexpr int ROWB_A = BK * ES, CPR_A = ROWB_A / 16;
  static constexpr int ROWB_B = BN * ES, CPR_B = ROWB_B / 16;
  static constexpr int A_BYTES = BM * ROWB_A, B_BYTES = BK * ROWB_B;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  static constexpr int A_LOADS = A_BYTES / 1024, B_LOADS = B_BYTES / 1024;  // wave-wide 1 KiB DMA ops
  static constexpr int A_LPW = (A_LOADS + NW - 1) / NW, B_LPW = (B_LOADS + NW - 1) / NW;
  static constexpr int LPW = A_LPW + B_LPW;                       // DMA ops one wave issues per slab
  static constexpr int ACC_N = (MI == 32) ? 16 : 4;
  static constexpr bool VALID =
      (WTM % 16 == 0) && (WTN % 16 == 0) && (BK * ES) % KB == 0 && KSTEPS >= 1 && CPR_A >= 4 &&
      CPR_B >= 8 && CPR_B % (ES == 1 ? 4 : 8) == 0 && A_BYTES % 1024 == 0 && B_BYTES % 1024 == 0 &&
      A_LOADS % NW == 0 && B_LOADS % NW == 0 && LDS_BYTES <= 163840 && TM * TN * ACC_N <= 256 && (STAGES - 2) * LPW <= 63 && STAGES >= 2;

  // chunk-index XOR applied to row `row` of the A slab.  A fragment read is one ds_read_b128 with lane = 16 * kg +
  // row: the LDS serves it in four cycles of 16 lanes, and the 16 are not consecutive lanes -- measured with a
  // one-wave probe and SQ_LDS_BANK_CONFLICT, lanes {0-3, 12-15, 20-27} share a cycle and {4-11, 16-19, 28-31} the
  // next (the same again from lane 32), i.e. all 16 rows of the fragment, but rows 4-11 with the neighbouring k
  // chunk.  The XOR therefore has to place rows r, r + 4, r + 8, r + 12 (which share the banks of a 128- or 64-byte
  // row) so that chunk kg of two of them and chunk kg ^ 1 of the other two fall on four different slots; both
  // formulas below do, and the probe counts no conflict cycle for them (the previous pair, (row & 7) ^ (row >> 3 & 1)
  // and (row >> 1 & 3) ^ (row >> 3 & 1), assumed 16 consecutive lanes per cycle and took 8 cycles per read, not 4).
  static __host__ __device__ constexpr int swzA(int row) {
    return CPR_A >= 8 ? ((row & 7) ^ ((row >> 2) & 1)) : (((row >> 3) & 1) << 1);
  }
  // chunk-index XOR applied to row `row` (a k index) of the B slab
  // (A transposing read serves the four 16-lane groups of a wave in two passes; with 16x16 MFMA tiles the two
  // groups of a pass read the same columns 8 k rows apart (16 for int8), so one more row bit enters the XOR to
  // keep them on different banks: it moves the second group onto exactly the chunk slots the first leaves free.)
  static __host__ __device__ constexpr int swzB(int row) {
    if (ES == 2) {
      const int pass = MI == 16 ? (((row >> 3) ^ (row >> 4)) & 1) << 1 : 0;
      if (CPR_B % 16 == 0) { int k = row & 3; return ((2 * k + (k >> 1)) << 1) ^ pass; }
      return ((row & 3) << 1) ^ pass;       // stays inside a group of 8 chunks: also for rows of 24 chunks (BN = 192)
    } else {
      const int pass = MI == 16 ? ((row >> 4) ^ (row >> 5)) & 1 : 0;
      if (CPR_B % 16 == 0) { int k = row & 7; return (2 * k + (k >> 2)) ^ pass; }
      if (CPR_B % 8 == 0) return (row & 7) ^ pass;
      // Rows of 12 chunks (BN = 192), 192 bytes: consecutive rows already start 48 banks apart, so the 8 rows of a
      // 16-lane group only collide with the row 4 below, and the two groups of a pass (rows r and r + 16) with each
      // other: one XOR bit for each, inside a group of 4 chunks.
      return ((row >> 2) & 1) | (((row >> 4) & 1) << 1);
    }
  }
};

// ---------------------------------------------------------------------------
// output conversion and the store of a wave's accumulators
// ---------------------------------------------------------------------------
struct OutBF16 {
  typedef uint16_t raw;
  static __device__ __forceinline__ raw cvt(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }  // RNE
};
struct OutF16 {
  typedef uint16_t raw;
  static __device__ __forceinline__ raw cvt(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};
// binary32 output of a 16-bit-float GEMM: the accumulator as it is.  It is what lets a float32 product run on the
// bf16 matrix instructions as a three-term split (the host side cuts each operand into a bf16 head and a bf16 tail
// and lays the terms out along K); built for the tiles up to 128x128 (f32_out_tile).
struct OutF32 {
  typedef float raw;
  static __device__ __forceinline__ raw cvt(float v) { return v; }
};
template <class T> struct OutOf;
template <> struct OutOf<TagBF16> { typedef OutBF16 type; };
template <> struct OutOf<TagF16> { typedef OutF16 type; };
template <> struct OutOf<TagI8> { typedef int type; };


// LDS one wave needs to pass one row-block (MI rows) of its accumulators through LDS: raw
// 32-bit values, rows padded by 16 bytes to spread the banks.
template <class C> struct EpiStage {
  static constexpr int PITCH = C::WTN * 4 + 16;
  // row-blocks per pass.  Two (32 rows per pass, half as many passes) was measured on the gated 4096x28672x4096
  // problem and lost 2-3 %: the longer read-back of a pass delays the first stores.
  static constexpr int RB = 1;
  static constexpr int ROWS = RB * C::MI;
  static constexpr int WAVE_BYTES = ROWS * PITCH;
  static constexpr int BYTES = C::NW * WAVE_BYTES;
};

// 16 bytes of output from NF accumulator values that sit row-major in LDS.
// GLU: values come in (gate, linear) pairs, one output per pair.
template <class O, class S, bool GLU> struct Pack16;
template <class O, bool GLU> struct Pack16<O, float, GLU> {   // 16-bit float outputs: 8 per lane
  typedef typename O::raw raw;
  static constexpr int OUTV = 8, NF = GLU ? 16 : 8;
  static __device__ __forceinline__ void run(const float* f, int epi, raw* out) {
#pragma unroll
    for (int x = 0; x < OUTV; ++x) out[x] = O::cvt(GLU ? glu_gate(f[2 * x], epi) * f[2 * x + 1] : f[x]);
  }
};
template <bool GLU> struct Pack16<OutF32, float, GLU> {       // binary32 outputs: 4 per lane
  typedef float raw;
  static constexpr int OUTV = 4, NF = GLU ? 8 : 4;
  static __device__ __forceinline__ void run(const float* f, int epi, raw* out) {
#pragma unroll
    for (int x = 0; x < OUTV; ++x) out[x] = GLU ? glu_gate(f[2 * x], epi) * f[2 * x + 1] : f[x];
  }
};
template <bool GLU> struct Pack16<int, int, GLU> {            // int32 outputs: 4 per lane
  typedef int raw;
  static constexpr int OUTV = 4, NF = 4;
  static __device__ __forceinline__ void run(const int* f, int, raw* out) {
#pragma unroll
    for (int x = 0; x < 4; ++x) out[x] = f[x];
  }
};

// Where the split-K slices of one wave's part of a tile sit in the workspace.  A slice is
// stored exactly as the wave holds it: group q = (i*TN + j)*NGRP + g of four accumulator
// registers is one 16-byte element per lane at q*1024 + lane*16, so every store and load
// instruction moves one contiguous KiB.
struct SliceSrc {
  const uint8_t* base;     // this wave's part of slice 0
  uint32_t slice_stride;   // bytes from one slice to the next (the host keeps nslices * slice_stride under 4 GiB)
  int nslices;
  bool rezero;             // atomic reduction: the one slice holds the finished sums; it is cleared again after the read
};

// Sum of the split-K slices of one row-block of a wave, group by group, into the wave's LDS
// strip (same places the accumulators of an uncut tile go).  ZB slices of G = 32 / ZB groups
// are fetched together; slices are added in slice order whatever ZB is.
// largest batch of groups <= cap that divides the nq groups of a row-block (nq is 6 for the 192-wide tiles)
constexpr int slice_batch(int nq, int cap) {
  int g = cap < nq ? cap : nq;
  while (nq % g) --g;
  return g;
}
template <class ACC4, int ZB, int NQ, int MI, int NGRP>
__device__ __forceinline__ void sum_slices(__amdgpu_buffer_rsrc_t win, uint32_t q0, const SliceSrc& src, uint32_t wbase,
                                           bool row_ok) {
  constexpr int G = slice_batch(NQ, 32 / ZB);
  static_assert(NQ % G == 0, "groups per row-block must be a multiple of the batch");
#pragma unroll 1
  for (int jg0 = 0; jg0 < NQ; jg0 += G) {
    ACC4 v[G];
#pragma unroll
    for (int x = 0; x < G; ++x) v[x] = ACC4{0, 0, 0, 0};
    // lanes whose row lies past the last row of the problem were not stored and are not read
#pragma unroll 1
    for (int z0 = 0; row_ok && z0 < src.nslices; z0 += ZB) {
      i32x4 w[G * ZB];
#pragma unroll
      for (int x = 0; x < G; ++x)
#pragma unroll
        for (int u = 0; u < ZB; ++u) {
          const int z = z0 + u < src.nslices ? z0 + u : src.nslices - 1;
          w[x * ZB + u] = load16_agent(win, q0 + (uint32_t)(jg0 + x) * 1024u + (uint32_t)z * src.slice_stride);
        }
      if (src.rezero) {
        // atomic reduction: what was just read is the sum; leave zeros behind for the next launch
#pragma unroll
        for (int x = 0; x < G; ++x) store16_agent(win, q0 + (uint32_t)(jg0 + x) * 1024u, i32x4{0, 0, 0, 0});
      }
#pragma unroll
      for (int x = 0; x < G; ++x)
#pragma unroll
        for (int u = 0; u < ZB; ++u)
          if (z0 + u < src.nslices) {
            ACC4 t;
            __builtin_memcpy(&t, &w[x * ZB + u], 16);
            v[x] += t;
          }
    }
#pragma unroll
    for (int x = 0; x < G; ++x) {
      const int j = (jg0 + x) / NGRP, g = (jg0 + x) % NGRP;
      *TNX_LDS(ACC4, wbase + (j * MI + g * 8) * 4) = v[x];
    }
  }
}

template <class C> constexpr bool multi_problem_tile() { return C::BM * C::BN <= 128 * 128; }
// tiles whose kernels carry a second copy of the epilogue that writes binary32 (16-bit float inputs only)
template <class T, class C> constexpr bool f32_out_tile() { return T::ES == 2 && C::BM * C::BN <= 128 * 128; }

__device__ __forceinline__ float bias_value(const uint8_t* bias, int row, int dtype) {
  if (dtype == DT_F32) return ((const float*)bias)[row];
  if (dtype == DT_F16) return (float)((const _Float16*)bias)[row];
  return __builtin_bit_cast(float, (uint32_t)((const uint16_t*)bias)[row] << 16);
}

// The MFMA result is C^T: lane l owns output row m = l % MI and, per group of four accumulator
// registers, four consecutive columns n.  Each wave passes one row-block at a time through its
// private LDS strip: raw accumulators in (one ds_write_b128 per group), then a plain loop reads
// the strip row-major, converts / gates, and stores 16 bytes per lane, so every row of C
// receives full contiguous runs.  Keeping the conversion out of the unrolled part keeps the
// epilogue variants of a 256x256 tile inside the instruction cache.
// FROM_WS: the values do not come from this wave's registers but from the split-K slices in
// the workspace, added in slice order (the result does not depend on which workgroup does it).
template <class T, class C, class O, bool GLU, bool FROM_WS, bool BIAS = false, class ACC>
__device__ __forceinline__ void epilogue_store(ACC (&acc)[C::TM][C::TN], const SliceSrc& src, uint8_t* cbase,
                                               uint32_t lds_strip, int lane, int64_t gm0, int64_t gc0, int64_t m,
                                               int64_t ncols, int64_t scm, int64_t scn, bool vec_ok, int epi,
                                               const uint8_t* bias = nullptr, int bias_dtype = 0) {
  typedef typename T::acc_s acc_s;
  typedef Pack16<O, acc_s, GLU> PK;
  typedef typename PK::raw raw;
  typedef acc_s acc4 __attribute__((ext_vector_type(4)));
  constexpr int MI = C::MI;
  constexpr int NGRP = C::ACC_N / 4;                    // groups of four consecutive columns per accumulator tile
  constexpr int PITCH = EpiStage<C>::PITCH;
  constexpr int RB = EpiStage<C>::RB, ROWS = EpiStage<C>::ROWS;   // a pass moves RB row-blocks = ROWS rows
  constexpr int WCOLS = GLU ? C::WTN / 2 : C::WTN;      // output columns of the wave tile
  constexpr int CPRW = WCOLS / PK::OUTV;                // 16-byte output chunks per strip row
  constexpr int ITERS = (ROWS * CPRW + 63) / 64;
  constexpr int UNR = ITERS % 4 == 0 ? 4 : (ITERS % 2 == 0 ? 2 : 1);   // read-back rows in flight together
  static_assert(WCOLS % PK::OUTV == 0, "wave tile too narrow for 16-byte stores");
  raw* cp = (raw*)cbase;
  const uint32_t wbase0 = lds_strip + (lane % MI) * PITCH + (lane / MI) * 16;
  // A bias per row of C (conv2d's 1x1 layers): lane l fetches the values of rows l, l + 64, .. of the wave tile now,
  // so that the loads fly under the first pass through the strip; the row loop below picks its value from the lane that holds it.
  constexpr bool WITH_BIAS = BIAS && std::is_same<acc_s, float>::value && !GLU;
  constexpr int NBR = (C::WTM + 63) / 64;
  float bias_rows[NBR] = {};
  if constexpr (WITH_BIAS) {
    if (bias) {
#pragma unroll
      for (int r = 0; r < NBR; ++r) {
        const int64_t g = gm0 + r * 64 + lane;
        if (r * 64 + lane < C::WTM && g < m) bias_rows[r] = bias_value(bias, (int)g, bias_dtype);
      }
    }
  }
#pragma unroll
  for (int i0 = 0; i0 < C::TM; i0 += RB) {
    if (gm0 + i0 * MI >= m) break;                      // row-blocks past the last row hold nothing
#pragma unroll
    for (int ii = 0; ii < RB; ++ii) {
      const int i = i0 + ii;
      const uint32_t wbase = wbase0 + ii * MI * PITCH;
      if constexpr (!FROM_WS) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
          for (int g = 0; g < NGRP; ++g)
            // (typed vector store: __builtin_bit_cast on an ext-vector element reads element 0)
            *TNX_LDS(acc4, wbase + (j * MI + g * 8) * 4) =
                acc4{acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
      } else {
        // 32 loads per lane in flight (G groups x ZB slices): the hand-over is latency-bound otherwise
        const __amdgpu_buffer_rsrc_t win = agent_window(src.base);
        const uint32_t q0 = (uint32_t)i * (C::TN * NGRP) * 1024u + lane * 16u;
        const bool row_ok = gm0 + i * MI + lane % MI < m;
        if (src.nslices <= 2)
          sum_slices<acc4, 2, C::TN * NGRP, MI, NGRP>(win, q0, src, wbase, row_ok);
        else if (src.nslices <= 4)
          sum_slices<acc4, 4, C::TN * NGRP, MI, NGRP>(win, q0, src, wbase, row_ok);
        else
          sum_slices<acc4, 8, C::TN * NGRP, MI, NGRP>(win, q0, src, wbase, row_ok);
      }
    }
    // the strip is private to this wave: its own LDS writes are ordered before its reads
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll 1
    for (int it0 = 0; it0 < ITERS; it0 += UNR) {
      // UNR rows of LDS reads are issued together, then converted and stored one after the other
      acc_s f[UNR][PK::NF];
      float bv[UNR] = {};
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int q = (it0 + u) * 64 + lane;
        int row = q / CPRW;
        const int cc = q % CPRW;
        if (ROWS * CPRW % 64 != 0 && row >= ROWS) row = ROWS - 1;
        if constexpr (WITH_BIAS) {
          const int rt = i0 * MI + row;                 // row of the wave tile: held by lane rt % 64 in bias_rows[rt / 64]
          if (bias)
#pragma unroll
          for (int r = 0; r < NBR; ++r) {
            const float t = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((rt & 63) * 4, __builtin_bit_cast(int, bias_rows[r])));
            if ((rt >> 6) == r) bv[u] = t;
          }
        }
#pragma unroll
        for (int x = 0; x < PK::NF / 4; ++x) {
          const i32x4 v = *TNX_LDS(i32x4, lds_strip + row * PITCH + (cc * PK::NF + 4 * x) * 4);
          __builtin_memcpy(&f[u][4 * x], &v, 16);
        }
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int q = (it0 + u) * 64 + lane;
        const int row = q / CPRW, cc = q % CPRW;
        const int64_t gm = gm0 + i0 * MI + row;
        const int64_t gc = gc0 + cc * PK::OUTV;
        if ((ROWS * CPRW % 64 != 0 && row >= ROWS) || gm >= m) continue;
        if constexpr (WITH_BIAS) {
          // added to the finished fp32 sum before the one rounding
          if (bias)
#pragma unroll
            for (int x = 0; x < PK::NF; ++x) f[u][x] += bv[u];
        }
        raw out[PK::OUTV];
        PK::run(f[u], epi, out);
        raw* dst = cp + gm * scm + gc * scn;
        if (vec_ok && gc + PK::OUTV <= ncols) {
          i32x4 v;
          __builtin_memcpy(&v, out, 16);
          store16_stream_loose(dst, v);                 // rows of C need not be 16-byte aligned
        } else {
#pragma unroll 1
          for (int x = 0; x < PK::OUTV; ++x)
            if (gc + x < ncols) dst[x * scn] = out[x];
        }
      }
    }
    // the next pass overwrites the strip: wait for the reads above
    __builtin_amdgcn_s_waitcnt(0xC07F);
  }
}

// Epilogue of the persistent kernel.  The ring is already being refilled with the next tile's
// first slabs while this runs, so the accumulators pass through a small strip of their own: per wave
// MI rows x 64 accumulator columns (64 / MI MFMA tiles side by side), rows 256 bytes apart with the
// 16-byte chunk index XOR-ed with the row, so neither the column-wise writes nor
// the row-wise read-back collide on banks.  FULL: the tile lies inside C and C takes 16-byte
// stores, so the number of store instructions per wave is the compile-time STORES (the caller's
// vmcnt arithmetic relies on it).
template <class C> struct PairStrip {
  static constexpr int WAVE_BYTES = C::MI * 256;              // MI rows of 64 accumulator columns
  static constexpr int BYTES = C::NW * WAVE_BYTES;
  static constexpr int TPP = 64 / C::MI;                      // MFMA tiles side by side in one pass
};
template <class T, class C, class O, bool GLU> struct PairEpilogue {
  typedef typename T::acc_s acc_s;
  typedef Pack16<O, acc_s, GLU> PK;
  static constexpr int OCOLS = GLU ? 32 : 64;                 // output columns per pass
  static constexpr int CPRW = OCOLS / PK::OUTV;               // lanes per output row
  static constexpr int ITERS = C::MI * CPRW / 64;
  static constexpr int CH = PK::NF / 4;                       // 16-byte chunks one lane reads back
  static constexpr int STORES = C::TM * (C::TN / PairStrip<C>::TPP) * ITERS;  // store instructions per wave on a FULL tile
};
template <class T, class C, class O, bool GLU, bool FULL, class ACC>
__device__ __forceinline__ void epilogue_store_pairs(ACC (&acc)[C::TM][C::TN], uint8_t* cbase, uint32_t strip, int lane,
                                                     int64_t gm0, int64_t gc0, int64_t m, int64_t ncols, int64_t scm,
                                                     int64_t scn, bool vec_ok, int epi) {
  constexpr int MI = C::MI, TPP = PairStrip<C>::TPP, NGRP = C::ACC_N / 4;
  static_assert(C::TN % TPP == 0 && MI * PairEpilogue<T, C, O, GLU>::CPRW >= 64, "a pass is 64 accumulator columns wide");
  typedef PairEpilogue<T, C, O, GLU> E;
  typedef typename E::acc_s acc_s;
  typedef typename E::PK PK;
  typedef typename PK::raw raw;
  typedef acc_s acc4 __attribute__((ext_vector_type(4)));
  raw* cp = (raw*)cbase;
  const int wrow = lane % MI, wk = lane / MI;
  const uint32_t wbase = strip + wrow * 256;
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    if (!FULL && gm0 + i * MI >= m) break;
#pragma unroll
    for (int jp = 0; jp < C::TN / TPP; ++jp) {
#pragma unroll
      for (int jj = 0; jj < TPP; ++jj)
#pragma unroll
        for (int g = 0; g < NGRP; ++g) {
          // chunk of four columns inside the 64-column pass: tile jj, then the lane's column group
          const int c = jj * (MI / 4) + g * (64 / MI) + wk;
          *TNX_LDS(acc4, wbase + ((c ^ (wrow & 15)) << 4)) =
              acc4{acc[i][TPP * jp + jj][4 * g + 0], acc[i][TPP * jp + jj][4 * g + 1], acc[i][TPP * jp + jj][4 * g + 2],
                   acc[i][TPP * jp + jj][4 * g + 3]};
        }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the strip is private to the wave
      acc_s f[E::ITERS][PK::NF];
#pragma unroll
      for (int it = 0; it < E::ITERS; ++it) {
        const int q = it * 64 + lane;
        const int row = q / E::CPRW, cc = q % E::CPRW;
#pragma unroll
        for (int x = 0; x < E::CH; ++x) {
          const i32x4 v = *TNX_LDS(i32x4, strip + row * 256 + (((cc * E::CH + x) ^ (row & 15)) << 4));
          __builtin_memcpy(&f[it][4 * x], &v, 16);
        }
      }
#pragma unroll
      for (int it = 0; it < E::ITERS; ++it) {
        const int q = it * 64 + lane;
        const int row = q / E::CPRW, cc = q % E::CPRW;
        const int64_t gm = gm0 + i * MI + row;
        const int64_t gc = gc0 + jp * E::OCOLS + cc * PK::OUTV;
        raw out[PK::OUTV];
        PK::run(f[it], epi, out);
        raw* dst = cp + gm * scm + gc * scn;
        if (FULL) {
          i32x4 v;
          __builtin_memcpy(&v, out, 16);
          store16_stream(dst, v);
        } else if (gm < m) {
          if (vec_ok && gc + PK::OUTV <= ncols) {
            i32x4 v;
            __builtin_memcpy(&v, out, 16);
            store16_stream(dst, v);
          } else {
#pragma unroll 1
            for (int x = 0; x < PK::OUTV; ++x)
              if (gc + x < ncols) dst[x * scn] = out[x];
          }
        }
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // the next pass overwrites the strip
    }
  }
}

// The first WS_COUNTER_BYTES of the split-K workspace hold one arrival counter per cut tile.
// They must be zero when a launch starts; every launch leaves them zero.
constexpr int WS_COUNTER_BYTES = 65536;
constexpr int WS_MAX_TILES = WS_COUNTER_BYTES / 4;

// One K slice of a cut tile leaves the workgroup: every wave writes its accumulators to its
// part of the slice with device-scope (sc1) stores, one lane bumps the tile's arrival counter,
// and the function returns true in the workgroup that arrived last.  That workgroup then reads
// all slices back with device-scope loads and runs the ordinary epilogue on their sum.
// Whole-L2 write-backs and invalidates (what a device-scope fence costs on a part with eight
// L2s) are avoided on purpose: they cost more than the GEMM.
template <class T, class C, class ACC>
__device__ __forceinline__ bool splitk_arrive(ACC (&acc)[C::TM][C::TN], uint8_t* wave_slice, uint32_t lds_strip, int lane,
                                              int64_t gm0, int64_t m, int* counter, int* flag, int nslices, bool atomic) {
  typedef typename T::acc_s acc_s;
  typedef acc_s acc4 __attribute__((ext_vector_type(4)));
  constexpr int NGRP = C::ACC_N / 4;
  constexpr int NQ = C::TN * NGRP;                      // 16-byte groups per lane and row-block
  const __amdgpu_buffer_rsrc_t win = agent_window(wave_slice);
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    if (gm0 + i * C::MI >= m) break;
    if (atomic) {
      // every slice adds into the same copy (wave_slice is slice 0 for all of them); same element order as a stored slice
      if (gm0 + i * C::MI + lane % C::MI < m) {
        acc_s* dst = (acc_s*)(wave_slice + (int64_t)i * NQ * 1024 + lane * 16);
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
          for (int g = 0; g < NGRP; ++g)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              __hip_atomic_fetch_add(dst + (j * NGRP + g) * 256 + e, acc[i][j][4 * g + e], __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
      }
      continue;
    }
    // registers -> LDS -> registers keeps the copy loop rolled (the accumulators may sit in AGPRs,
    // which a 16-byte device-scope store cannot name directly)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int g = 0; g < NGRP; ++g)
        *TNX_LDS(acc4, lds_strip + (j * NGRP + g) * 1024 + lane * 16) =
            acc4{acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    const uint32_t dst = (uint32_t)i * NQ * 1024u + lane * 16u;
    if (gm0 + i * C::MI + lane % C::MI < m) {            // a lane is one row: rows past the problem are not stored
#pragma unroll 4
      for (int q = 0; q < NQ; ++q)
        store16_agent(win, dst + q * 1024u, *TNX_LDS(i32x4, lds_strip + q * 1024 + lane * 16));
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
  }
  // device-scope stores: once they are acknowledged they are visible to every XCD, so the
  // arrival count may follow
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the last arrival re-arms the counter for the next launch
    if (prev == nslices - 1) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = prev;
  }
  __syncthreads();
  const bool last = *flag == nslices - 1;
  __syncthreads();                                      // the flag's LDS word is reused by the epilogue strips
  return last;
}

// 16 bytes from an address that is only 2-byte aligned
struct __attribute__((packed, aligned(2))) Loose16 {
  i32x4 v;
};


// Epilogue of the CONV kernels: rows are output channels, columns are pixels of the padded pixel index space.  Same
// pass through the wave's LDS strip as epilogue_store; a 16-byte chunk is 8 pixels of one output row, so it is one
// run of the NCHW output (cut at w_out: the pixels past it exist only in the index space).  Bias is added in fp32.
template <class T, class C, class O, class ACC>
__device__ __forceinline__ void epilogue_store_conv(ACC (&acc)[C::TM][C::TN], uint8_t* ybase, uint32_t lds_strip, int lane,
                                                    int gm0, int gn0, const ConvGeom& g) {
  typedef typename O::raw raw;                          // 16-bit outputs, or binary32 (the fp32 sums + bias as they are)
  typedef float acc4 __attribute__((ext_vector_type(4)));
  constexpr int MI = C::MI;
  constexpr int NGRP = C::ACC_N / 4;
  constexpr int PITCH = EpiStage<C>::PITCH;
  constexpr int ROWS = EpiStage<C>::ROWS;
  constexpr int CPRW = C::WTN / 8;                       // a lane handles 8 pixels: one 16-byte chunk of the im2col slab
  constexpr int ITERS = (ROWS * CPRW + 63) / 64;
  constexpr int UNR = ITERS % 4 == 0 ? 4 : (ITERS % 2 == 0 ? 2 : 1);
  static_assert(EpiStage<C>::RB == 1 && C::WTN % 8 == 0, "one row-block per pass, 8 outputs per chunk");
  raw* yp = (raw*)ybase;
  const uint32_t wbase = lds_strip + (lane % MI) * PITCH + (lane / MI) * 16;
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    if (gm0 + i * MI >= g.c_out) break;
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int q = 0; q < NGRP; ++q)
        *TNX_LDS(acc4, wbase + (j * MI + q * 8) * 4) =
            acc4{acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll 1
    for (int it0 = 0; it0 < ITERS; it0 += UNR) {
      float f[UNR][8];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int q = (it0 + u) * 64 + lane;
        int row = q / CPRW;
        const int cc = q % CPRW;
        if (ROWS * CPRW % 64 != 0 && row >= ROWS) row = ROWS - 1;
#pragma unroll
        for (int x = 0; x < 2; ++x) {
          const i32x4 v = *TNX_LDS(i32x4, lds_strip + row * PITCH + (cc * 8 + 4 * x) * 4);
          __builtin_memcpy(&f[u][4 * x], &v, 16);
        }
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int q = (it0 + u) * 64 + lane;
        const int row = q / CPRW, cc = q % CPRW;
        const int gm = gm0 + i * MI + row;
        const int gc = gn0 + cc * 8;
        if ((ROWS * CPRW % 64 != 0 && row >= ROWS) || gm >= g.c_out || gc >= g.n_total) continue;
        const int img = (int)fd_div((uint32_t)gc, g.div_hwp);
        const int r = gc - img * (g.h_out * g.wp);
        const int ho = (int)fd_div((uint32_t)r, g.div_wp);
        const int wq = r - ho * g.wp;
        const int valid = g.w_out - wq;              // pixels of this chunk that exist
        if (valid <= 0) continue;
        const float bv = g.bias ? bias_value(g.bias, gm, g.bias_dtype) : 0.0f;
        raw out[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) out[x] = O::cvt(f[u][x] + bv);
        raw* dst = yp + (((int64_t)img * g.c_out + gm) * g.h_out + ho) * g.w_out + wq;
        if (valid >= 8) {
          i32x4 v[sizeof(raw) / 2];
          __builtin_memcpy(v, out, 8 * sizeof(raw));
#pragma unroll
          for (int h = 0; h < (int)sizeof(raw) / 2; ++h)
            store16_stream_loose((uint8_t*)dst + 16 * h, v[h]);    // element-aligned: w_out need not be a multiple of 8
        } else {
#pragma unroll 1
          for (int x = 0; x < valid; ++x) dst[x] = out[x];
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
  }
}

template <class X> struct TypeTag { typedef X type; };
template <bool B> struct BoolTag { static constexpr bool value = B; };
template <int V> struct IntTag { static constexpr int value = V; };

// ---------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------
// BT: B is k-contiguous (element (k, n) at b + n * stride_bn + k, the layout of `x @ w.t()` with a
// row-major weight): its slab sits in LDS as BN rows of BK elements exactly like the A slab, and its
// fragments are read with plain ds_read_b128 -- no transposing read is needed.
// CONV: conv2d forward (ConvGeom): A is the weight, the B slab is gathered from the NCHW input by the DMA loader --
// one 16-byte raw-buffer load per chunk of 8 pixels from an address that is only 2-byte aligned, with an
// out-of-range offset (the buffer bound answers zero) for chunks whose input row lies in the padding.  The elements
// of a chunk that fall into the left / right padding have to be zeroed in LDS afterwards, by the wave that loaded
// them.  Done between the wait for the loads and the barrier that publishes the slab, that fix-up sits on the
// critical path of every K slab (measured: 340 instead of 630 TFLOP/s on a 3x3 layer), so the ring has three slots
// and a slab is fixed well before it is read: slab t+3 is issued during the first half of period t, waited for in
// the middle of period t+1 (by then only that period's own loads may still be outstanding), fixed in the second
// half of period t+1 -- one read-modify-write of the chunk per op, slotted behind MFMAs -- and published by barrier
// t+2, before whose period nothing reads it.  16-bit types, stride_w == 1, k % BK == 0.
template <class T, class C, bool FAST, bool PERSIST = false, bool BT = false, bool CONV = false>
__global__ __launch_bounds__(C::THREADS) void gemm_tile_kernel(GemmParams p) {
  constexpr int ES = C::ES, BM = C::BM, BN = C::BN, BK = C::BK, NW = C::NW, STAGES = C::STAGES;
  constexpr int MI = C::MI, TM = C::TM, TN = C::TN;
  static_assert(C::VALID, "tile configuration not supported by this kernel");
  static_assert(!PERSIST || FAST, "the persistent kernel is built with the DMA loader only");
  static_assert(!BT || (FAST && C::B_LOADS % NW == 0), "the k-contiguous B variant is built with the DMA loader only");
  static_assert(!CONV || (FAST && !PERSIST && !BT && ES == 2 && STAGES == 3 && MI == 16 && (NW * 64) % C::CPR_B == 0),
                "the conv2d variant: DMA loader, 16-bit types, three ring slots");
  typedef Mma<T, MI> MMA;
  typedef typename MMA::acc_t acc_t;
  typedef typename T::acc_s acc_s;
  // Several problems in one grid and a bias per row (GemmParams::batch, cv.bias) exist in the tiles up to 128x128:
  // the 256-wide tiles have no register to spare for the extra state (measured: 20 more spilled registers, -0.4 %).
  constexpr bool MULTI = !PERSIST && !CONV && multi_problem_tile<C>();

  // one workgroup per tile: the epilogue strips are laid over the ring once the K loop is done.
  // persistent: the ring is refilled for the next tile during the epilogue, so the strips follow it.
  constexpr int RING_OR_STRIPS = C::LDS_BYTES > EpiStage<C>::BYTES ? C::LDS_BYTES : EpiStage<C>::BYTES;
  // CONV: behind the ring, a table of the 81 16-byte masks that keep elements [lo, hi) of a chunk (0 <= lo, hi <= 8),
  // and two tables of the filter taps of one K slab (BK entries of 8 bytes: element offset, dh | dw << 16)
  constexpr int CV_TABLE_BYTES = CONV ? 81 * 16 + 2 * BK * 8 : 0;
  constexpr int SMEM_BYTES = (PERSIST ? C::LDS_BYTES + PairStrip<C>::BYTES : RING_OR_STRIPS) + CV_TABLE_BYTES;
  static_assert(SMEM_BYTES <= 163840, "LDS budget of one CU exceeded");
  __shared__ __attribute__((aligned(1024))) uint8_t smem[SMEM_BYTES];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(uint8_t __attribute__((address_space(3)))*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- which tile / split ------------------------------------------------
  // Tiles [0, split_tile0) in launch order are computed whole by one workgroup each; the
  // tiles after them are cut split_k ways along K (all tiles when split_tile0 == 0: plain
  // split-K; only the last partial wave of tiles when the tile count does not fill the CUs).
  // The persistent kernel never cuts: workgroup b computes tiles b, b + gridDim.x, ... whole.
  const int ntiles = p.tiles_m * p.tiles_n;
  int split = 0, logical = 0;
  bool cut = false;
  // launch-order id -> tile coordinates
  auto locate = [&](int id, int* pid_m, int* pid_n) __attribute__((always_inline)) {
    if (p.tile_order == 1) {
      superblock_order(id, p.tiles_m, p.tiles_n, pid_m, pid_n);
    } else {
      const int lg = xcd_remap(id, ntiles, 8);
      swizzle2d(lg / p.tiles_n, lg % p.tiles_n, p.tiles_m, p.tiles_n, p.group_m, pid_m, pid_n);
    }
  };
  int pid_m, pid_n;
  if (PERSIST || p.split_k <= 1) {
    int bid = blockIdx.x;
    if constexpr (MULTI) {
      // several problems with one A in one grid (conv2d's 1x1 layers: one per image): problem after problem
      if (p.batch > 1) {
        const int img = bid / ntiles;
        bid -= img * ntiles;
        p.b += (int64_t)img * p.b_batch_bytes;
        p.c += (int64_t)img * p.c_batch_bytes;
      }
    }
    locate(bid, &pid_m, &pid_n);
  } else {
    if ((int)blockIdx.x < p.split_tile0) {
      logical = xcd_remap(blockIdx.x, p.split_tile0, 8);
    } else {
      const int ncut = ntiles - p.split_tile0;
      int t = blockIdx.x - p.split_tile0;
      split = t / ncut;
      t -= split * ncut;
      logical = p.split_tile0 + xcd_remap(t, ncut, 8);
      cut = true;
    }
    swizzle2d(logical / p.tiles_n, logical % p.tiles_n, p.tiles_m, p.tiles_n, p.group_m, &pid_m, &pid_n);
  }

  const int kt_total = (int)((p.k + BK - 1) / BK);
  const int kt0 = cut ? split * p.ktiles_per_split : 0;
  int kt1 = cut ? kt0 + p.ktiles_per_split : kt_total;
  if (kt1 > kt_total) kt1 = kt_total;
  // FAST kernels move their slabs with the DMA loader.  It wants chunks that lie inside their row: with a K that is
  // no multiple of BK, rows that are not 16-byte aligned or an N that ends inside a chunk, the host sets tail_slab
  // and the last slab of the K range (the only one whose chunks can cross the end of a row of A, or the end of the
  // last row of B) is left out of the ring and loaded element by element, zero-filled, after the K loop.
  const bool tail_here = FAST && !PERSIST && !CONV && p.tail_slab != 0 && kt1 == kt_total && kt1 > kt0;
  const int KT = kt1 > kt0 ? kt1 - kt0 - (tail_here ? 1 : 0) : 0;          // slabs of this workgroup in the ring (per tile)

  // ---- the tile the loader works on: origin, DMA bases and per-lane byte offsets.
  // (In the persistent kernel the loader moves on to the next tile before the epilogue of the
  // current one has run, so the epilogue keeps its own copy of the origin.)
  int64_t m0 = 0, n0 = 0;
  uint32_t a_voff[C::A_LPW], b_voff[C::B_LPW];
  constexpr bool PINGPONG_TILE = TNX_PINGPONG && FAST && !PERSIST && !BT && !CONV && NW == 8 && STAGES == 2 && C::KSTEPS == 2;
  // CONV: a lane's B ops all fetch the same 16-byte LDS column slot; the pixel chunk that lands there is one of
  // two (the LDS swizzle moves it by two chunks depending on the k row): element offset of (image, channel 0,
  // h0, w0) and the packed (h0, w0) for both, (h0, w0) being the input position of filter tap (0, 0).  Pixels past
  // the end get h0 = -32768, which no tap brings back into the image.  The filter taps (dh, dw, element offset) of
  // the k rows of a slab come from a 64-entry table in LDS that the first 64 threads write one period ahead, each
  // keeping the running tap of one k row and moving it one slab on per period (additions and wrap-arounds only):
  // per op a lane reads one entry instead of doing that arithmetic itself.
  constexpr int CONV_STEP = (NW * 64) / C::CPR_B;          // k rows covered by one B op of the workgroup
  const int cv_r0 = tid / C::CPR_B;                          // k row of this lane in the first op of a slab
  int pix_off0 = 0, pix_off1 = 0, pix_hw0 = 0, pix_hw1 = 0;   // (scalars, not arrays: an array indexed by a run-time bit is moved to LDS by the compiler)
  int tap_dh = 0, tap_dw = 0;                                // (wave 0 only) tap of k row `tid` of the next slab to tabulate
  uint32_t tap_off = 0;
  int cv_wr = 0, cv_rd = 0;                                  // next slab to tabulate / to issue (their parities pick the table)
  i32x2 cv_ent[CONV ? C::B_LPW : 1];                         // the table entries of this lane's ops of the slab being issued
  uint32_t cv_fix[CONV ? C::B_LPW : 1];                      // per op of the slab in flight: what its fix-up has to do
  int cv_o[CONV ? C::B_LPW : 1];                             // ... and the element offset its chunk starts at
  bool cv_pending = false;
  uint32_t cv_dst = 0;
  constexpr uint32_t CV_OUTSIDE = 0xffffffffu, CV_NOFIX = 8u * 16u;   // a note is the byte offset of mask (lo, hi) in the table: (lo * 9 + hi) * 16
  const uint32_t cv_table = lds0 + RING_OR_STRIPS;
  const uint32_t cv_ktab = cv_table + 81 * 16;
  i32x4 cv_rsrc = {0, 0, 0, 0};
  if constexpr (CONV) {
    if (tid < 81) {
      const int lo = tid / 9, hi = tid % 9;
      i32x4 m;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        m[d] = (int)((2 * d >= lo && 2 * d < hi ? 0xffffu : 0u) | (2 * d + 1 >= lo && 2 * d + 1 < hi ? 0xffff0000u : 0u));
      *TNX_LDS(i32x4, cv_table + tid * 16) = m;
    }
    __syncthreads();
    const uint64_t xa = (uint64_t)(uintptr_t)p.b;
    cv_rsrc = i32x4{(int)__builtin_amdgcn_readfirstlane((uint32_t)xa), (int)(__builtin_amdgcn_readfirstlane((uint32_t)(xa >> 32)) & 0xffff),
                    (int)__builtin_amdgcn_readfirstlane(p.cv.x_bytes), 0x00020000};
  }
  const uint8_t* a_sbase = p.a;
  const uint8_t* b_sbase = p.b;
  auto place_tile = [&](int tile_m, int tile_n) __attribute__((always_inline)) {
    m0 = (int64_t)tile_m * BM;
    n0 = (int64_t)tile_n * BN;
    if (FAST) {
      const int64_t lda = p.sam, ldb = BT ? p.sbn : p.sbk;
      // wave-uniform by construction; say so, so both stay in SGPRs for the DMA's scalar base operand
      a_sbase = uniform_ptr(p.a + (m0 * lda + (int64_t)kt0 * BK) * ES);
      b_sbase = uniform_ptr(BT ? p.b + (n0 * ldb + (int64_t)kt0 * BK) * ES : p.b + ((int64_t)kt0 * BK * ldb + n0) * ES);
      const int64_t mrem = p.m - 1 - m0;  // last valid row inside this tile
#pragma unroll
      for (int q = 0; q < C::A_LPW; ++q) {
        int P = (q * NW + wave) * 64 + lane;
        int row = P / C::CPR_A, cs = P % C::CPR_A;
        int c = cs ^ C::swzA(row);
        int64_t r = row < mrem ? row : mrem;
        a_voff[q] = (uint32_t)(r * lda * ES + c * 16);
      }
      if constexpr (CONV) {
        const ConvGeom& g = p.cv;
        const int cs = tid % C::CPR_B;
        const int c0 = cs ^ C::swzB(cv_r0 & 7);              // rows 0-7: the swizzle without its pass term
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const int n = (int)n0 + ((c0 ^ (v << 1)) << 3);
          int off = 0, h0 = -32768, w0 = 0;
          if (n < g.n_total) {
            const int img = (int)fd_div((uint32_t)n, g.div_hwp);
            const int r = n - img * (g.h_out * g.wp);
            const int ho = (int)fd_div((uint32_t)r, g.div_wp);
            h0 = ho * g.stride_h - g.pad_h;
            w0 = (r - ho * g.wp) - g.pad_w;
            off = img * g.chw_in + h0 * g.w_in + w0;
          }
          const int hw = (int)(((uint32_t)h0 << 16) | ((uint32_t)w0 & 0xffffu));
          if (v == 0) { pix_off0 = off; pix_hw0 = hw; } else { pix_off1 = off; pix_hw1 = hw; }
        }
        // the tap of k row tid (< BK) of slab 0 (the K loop starts at k = 0: these kernels are never cut along K)
        const int krow = tid & (BK - 1);
        const int cin = (int)fd_div((uint32_t)krow, g.div_rs);
        const int r = krow - cin * g.rs;
        const int th = (int)fd_div((uint32_t)r, g.div_s);
        tap_dh = th * g.dil_h;
        tap_dw = (r - th * g.fw) * g.dil_w;
        tap_off = (uint32_t)(cin * g.hw_in + tap_dh * g.w_in + tap_dw);
        cv_wr = 0;
        cv_rd = 0;
      }
      const int64_t nrem = p.n - 1 - n0;  // last valid column inside this tile
#pragma unroll
      for (int q = 0; q < (CONV ? 0 : C::B_LPW); ++q) {
        int P = (q * NW + wave) * 64 + lane;
        if (BT) {
          // rows of the slab are columns of B: same chunk layout and swizzle as the A slab
          int row = P / C::CPR_A, cs = P % C::CPR_A;
          int c = cs ^ C::swzA(row);
          int64_t r = row < nrem ? row : nrem;
          b_voff[q] = (uint32_t)(r * ldb * ES + c * 16);
        } else {
          int row = P / C::CPR_B, cs = P % C::CPR_B;
          int c = cs ^ C::swzB(row);
          // column chunk past N: any valid address.  (A chunk that starts below N and ends above it -- tail_slab
          // launches only -- is loaded as it is: its upper elements come from the next k row, which exists because
          // the last slab is not loaded here, and belong to columns that are never stored.)
          if (n0 + (int64_t)c * (16 / ES) >= p.n || (!p.tail_slab && n0 + (int64_t)(c + 1) * (16 / ES) > p.n)) c = 0;
          b_voff[q] = (uint32_t)((int64_t)row * ldb * ES + c * 16);
        }
      }
    }
  };
  place_tile(pid_m, pid_n);

  // Loader for what the DMA path does not take: any strides, any ragged edge, zero fill.  One 16-byte chunk of the
  // slab per thread and trip: a chunk that lies inside the matrix along a unit-stride dimension is one vector load
  // at the element's own alignment, any other chunk is put together element by element.  Used for every slab of the
  // kernels built without the DMA loader and for the left-out last slab of a tail_slab launch.
  // (t0: the thread's index in the workgroup, handed in so that the DMA kernels need not keep threadIdx.x alive
  // across their K loop for the one call after it)
  // The loader in two halves, so that the kernels built without the DMA loader can fetch slab t + STAGES into
  // registers before the MFMAs of a period and put it into LDS after them (gen_fetch, gen_store).
  constexpr int GEN_B_ROWS = BT ? BN : BK, GEN_B_CPR = BT ? C::CPR_A : C::CPR_B;
  constexpr int GEN_NA = (BM * C::CPR_A + C::THREADS - 1) / C::THREADS;
  constexpr int GEN_NB = (GEN_B_ROWS * GEN_B_CPR + C::THREADS - 1) / C::THREADS;
  typedef typename std::conditional<ES == 2, uint16_t, uint8_t>::type gen_elem_t;
  typedef typename std::conditional<ES == 2, i32x4_loose, i32x4_bytes>::type gen_chunk_t;
  constexpr int EPC = 16 / ES;                           // elements per chunk
  // chunk idx of the A part of slab kt_global: row idx / CPR_A, k chunk idx % CPR_A
  auto gen_fetch_a = [&](int kt_global, int idx) __attribute__((always_inline)) -> i32x4 {
    const gen_elem_t* ap = (const gen_elem_t*)p.a;
    const int row = idx / C::CPR_A, cs = idx % C::CPR_A;
    const int64_t gm = m0 + row, gk = (int64_t)kt_global * BK + cs * EPC;
    i32x4 v = {0, 0, 0, 0};
    if (idx < BM * C::CPR_A && gm < p.m && gk < p.k) {
      if (p.sak == 1 && gk + EPC <= p.k) {
        v = *(const gen_chunk_t*)(ap + gm * p.sam + gk);
      } else {
        gen_elem_t e[EPC];
#pragma unroll
        for (int x = 0; x < EPC; ++x) e[x] = gk + x < p.k ? ap[gm * p.sam + (gk + x) * p.sak] : (gen_elem_t)0;
        __builtin_memcpy(&v, e, 16);
      }
    }
    return v;
  };
  // chunk idx of the B part: k row idx / CPR_B, column chunk idx % CPR_B -- or, for the k-contiguous-B kernels, whose
  // slab holds BN rows of B^T chunked and swizzled like the A slab, column idx / CPR_A, k chunk idx % CPR_A
  auto gen_fetch_b = [&](int kt_global, int idx) __attribute__((always_inline)) -> i32x4 {
    const gen_elem_t* bp = (const gen_elem_t*)p.b;
    const int row = idx / GEN_B_CPR, cs = idx % GEN_B_CPR;
    const int64_t k0 = (int64_t)kt_global * BK;
    i32x4 v = {0, 0, 0, 0};
    if constexpr (BT) {
      const int64_t gn = n0 + row, gk = k0 + cs * EPC;
      if (idx < GEN_B_ROWS * GEN_B_CPR && gn < p.n && gk < p.k) {
        if (p.sbk == 1 && gk + EPC <= p.k) {
          v = *(const gen_chunk_t*)(bp + gn * p.sbn + gk);
        } else {
          gen_elem_t e[EPC];
#pragma unroll
          for (int x = 0; x < EPC; ++x) e[x] = gk + x < p.k ? bp[gn * p.sbn + (gk + x) * p.sbk] : (gen_elem_t)0;
          __builtin_memcpy(&v, e, 16);
        }
      }
    } else {
      const int64_t gk = k0 + row, gn = n0 + cs * EPC;
      if (idx < GEN_B_ROWS * GEN_B_CPR && gk < p.k && gn < p.n) {
        if (p.sbn == 1 && gn + EPC <= p.n) {
          v = *(const gen_chunk_t*)(bp + gk * p.sbk + gn);
        } else {
          gen_elem_t e[EPC];
#pragma unroll
          for (int x = 0; x < EPC; ++x) e[x] = gn + x < p.n ? bp[gk * p.sbk + (gn + x) * p.sbn] : (gen_elem_t)0;
          __builtin_memcpy(&v, e, 16);
        }
      }
    }
    return v;
  };
  auto gen_store_a = [&](uint32_t stage_base, int idx, i32x4 v) __attribute__((always_inline)) {
    const int row = idx / C::CPR_A, cs = idx % C::CPR_A;
    if (idx < BM * C::CPR_A) *TNX_LDS(i32x4, stage_base + row * C::ROWB_A + ((cs ^ C::swzA(row)) << 4)) = v;
  };
  auto gen_store_b = [&](uint32_t stage_base, int idx, i32x4 v) __attribute__((always_inline)) {
    const int row = idx / GEN_B_CPR, cs = idx % GEN_B_CPR;
    if (idx < GEN_B_ROWS * GEN_B_CPR) {
      if constexpr (BT) *TNX_LDS(i32x4, stage_base + C::A_BYTES + row * C::ROWB_A + ((cs ^ C::swzA(row)) << 4)) = v;
      else *TNX_LDS(i32x4, stage_base + C::A_BYTES + row * C::ROWB_B + ((cs ^ C::swzB(row)) << 4)) = v;
    }
  };
  auto gen_fetch = [&](int kt_global, int t0, i32x4 (&ra)[GEN_NA], i32x4 (&rb)[GEN_NB]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < GEN_NA; ++u) ra[u] = gen_fetch_a(kt_global, t0 + u * C::THREADS);
#pragma unroll
    for (int u = 0; u < GEN_NB; ++u) rb[u] = gen_fetch_b(kt_global, t0 + u * C::THREADS);
  };
  auto gen_store = [&](uint32_t stage_base, int t0, const i32x4 (&ra)[GEN_NA], const i32x4 (&rb)[GEN_NB]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < GEN_NA; ++u) gen_store_a(stage_base, t0 + u * C::THREADS, ra[u]);
#pragma unroll
    for (int u = 0; u < GEN_NB; ++u) gen_store_b(stage_base, t0 + u * C::THREADS, rb[u]);
  };
  // one chunk at a time: for the prologue of the kernels without the DMA loader and the one call after the K loop
  // of a tail_slab launch, where nothing is there to overlap with and registers are better left alone
  auto load_slab_generic = [&](int kt_global, uint32_t stage_base, int t0) __attribute__((always_inline)) {
#pragma unroll 1
    for (int idx = t0; idx < BM * C::CPR_A; idx += C::THREADS) gen_store_a(stage_base, idx, gen_fetch_a(kt_global, idx));
#pragma unroll 1
    for (int idx = t0; idx < GEN_B_ROWS * GEN_B_CPR; idx += C::THREADS) gen_store_b(stage_base, idx, gen_fetch_b(kt_global, idx));
  };

  // CONV: the first 64 threads write the taps of the next slab to tabulate into the table of its parity and move
  // their tap one slab on; every lane reads the entries of its ops of the slab that is about to be issued.
  auto conv_tab_write = [&]() __attribute__((always_inline)) {
    if constexpr (CONV) {
      const ConvGeom& g = p.cv;
      if (wave == 0) {
        *TNX_LDS(i32x2, cv_ktab + (uint32_t)(cv_wr & 1) * (BK * 8) + (uint32_t)lane * 8u) =
            i32x2{(int)tap_off, (int)((uint32_t)tap_dh | ((uint32_t)tap_dw << 16))};
        int ndw = tap_dw + g.step_dw;
        const bool wrap_w = ndw >= g.lim_w;
        ndw -= wrap_w ? g.lim_w : 0;
        int ndh = tap_dh + g.step_dh + (wrap_w ? g.dil_h : 0);
        const bool wrap_h = ndh >= g.lim_h;
        ndh -= wrap_h ? g.lim_h : 0;
        tap_off += (uint32_t)(g.step_koff + (wrap_w ? g.adj_w : 0) + (wrap_h ? g.adj_h : 0));
        tap_dw = ndw;
        tap_dh = ndh;
      }
      ++cv_wr;
    }
  };
  auto conv_tab_read = [&]() __attribute__((always_inline)) {
    if constexpr (CONV) {
#pragma unroll
      for (int qb = 0; qb < C::B_LPW; ++qb)
        cv_ent[qb] = *TNX_LDS(i32x2, cv_ktab + (uint32_t)(cv_rd & 1) * (BK * 8) + (uint32_t)(qb * CONV_STEP + cv_r0) * 8u);
      ++cv_rd;
    }
  };
  // CONV: byte offset of B op qb's chunk inside the input (or CV_OUTSIDE) and its fix-up note
  uint32_t cv_voff = 0;
  auto conv_prepare = [&](int qb, uint32_t stage_base) __attribute__((always_inline)) {
    const ConvGeom& g = p.cv;
    const int row = qb * CONV_STEP + cv_r0;
    const bool second = ((row >> 3) ^ (row >> 4)) & 1;      // the pass term of swzB
    const int off = second ? pix_off1 : pix_off0, hw = second ? pix_hw1 : pix_hw0;
    const int h0 = hw >> 16, w0 = (int)(int16_t)(hw & 0xffff);
    const int dh = cv_ent[qb].y & 0xffff, dw = (int)((uint32_t)cv_ent[qb].y >> 16);
    const int o = off + cv_ent[qb].x;
    int lo = -(w0 + dw), hi = g.w_in - (w0 + dw);            // elements [lo, hi) of the chunk lie inside the input row
    lo = lo < 0 ? 0 : lo;
    hi = hi > 8 ? 8 : hi;
    const bool ok = (uint32_t)(h0 + dh) < (uint32_t)g.h_in && lo < hi;
    // A chunk that starts before the tensor (first row of the first image, left padding) or ends after it (last
    // row of the last image, right padding) cannot be fetched whole: the buffer bound drops every dword that is not
    // entirely inside, valid elements included (a negative offset wraps to one past every bound).  Its inside
    // elements are written by the fix-up, which recognises the case from the offset kept here.
    cv_voff = ok ? (uint32_t)o * 2u : CV_OUTSIDE;
    cv_fix[qb] = ok ? (uint32_t)(lo * 9 + hi) * 16u : CV_NOFIX;
    cv_o[qb] = o;
    cv_dst = stage_base;
    cv_pending = true;
  };
  auto conv_go = [&]() __attribute__((always_inline)) {
    asm volatile("buffer_load_dwordx4 %0, %1, 0 offen lds" : : "v"(cv_voff), "s"(cv_rsrc) : "memory");
  };
  // Fix-up of one op's chunk: zero the elements outside [lo, hi): chunk & mask(lo, hi), the mask read from the
  // table.  In two parts so that the two LDS reads have returned when the second part runs: fix_read, a few MFMA
  // slots, fix_write.  Every lane does it for every op, needed or not (its mask is all ones when it has nothing to
  // zero): straight-line code lets the compiler wait for exactly these reads, where a branch around them made it
  // wait for every LDS read in flight (measured: 433 with the branch, 618 TFLOP/s with no fix-up at all).
  // A chunk that could not be fetched whole at either end of the tensor (conv_prepare) was loaded as zeros and
  // has its inside elements filled in one by one afterwards (fix_special); that happens in a handful of
  // workgroups at most and costs the others one uniform branch per period.
  i32x4 cv_rmw[CONV ? C::B_LPW : 1], cv_msk[CONV ? C::B_LPW : 1];
  auto conv_fix_at = [&](int qb, uint32_t dst) __attribute__((always_inline)) {
    return dst + C::A_BYTES + (uint32_t)(qb * NW + wave) * 1024u + (uint32_t)lane * 16u;
  };
  auto conv_fix_read = [&](int qb, uint32_t note, uint32_t dst) __attribute__((always_inline)) {
    cv_msk[qb] = *TNX_LDS(i32x4, cv_table + (note & 0xffffu));
    cv_rmw[qb] = *TNX_LDS(i32x4, conv_fix_at(qb, dst));
  };
  auto conv_fix_write = [&](int qb, uint32_t note, uint32_t dst) __attribute__((always_inline)) {
    *TNX_LDS(i32x4, conv_fix_at(qb, dst)) = cv_rmw[qb] & cv_msk[qb];
  };
  auto conv_fix_special = [&](const uint32_t (&notes)[CONV ? C::B_LPW : 1], const int (&os)[CONV ? C::B_LPW : 1],
                              uint32_t dst) __attribute__((always_inline)) {
    const int x_elems = (int)(p.cv.x_bytes >> 1);
    bool any = false;
#pragma unroll
    for (int qb = 0; qb < (CONV ? C::B_LPW : 0); ++qb) any |= notes[qb] != CV_NOFIX && (os[qb] < 0 || os[qb] > x_elems - 8);
    if (__builtin_amdgcn_ballot_w64(any) != 0) {
#pragma unroll 1
      for (int qb = 0; qb < (CONV ? C::B_LPW : 0); ++qb) {
        uint32_t note = CV_NOFIX;
        int o = 0;
#pragma unroll
        for (int x = 0; x < (CONV ? C::B_LPW : 0); ++x) {   // no register-indexed array
          note = x == qb ? notes[x] : note;
          o = x == qb ? os[x] : o;
        }
        if (note != CV_NOFIX && (o < 0 || o > x_elems - 8)) {
          const uint32_t at = conv_fix_at(qb, dst);
          const int idx = (int)(note >> 4), lo = idx / 9, hi = idx % 9;
          const uint16_t* src = (const uint16_t*)p.b + o;
#pragma unroll 1
          for (int e = lo; e < hi; ++e) *TNX_LDS(uint16_t, at + 2 * e) = src[e];
        }
      }
    }
  };
  // the whole fix-up of the slab whose notes are in `notes`, in one go (prologue and the first draining period)
  auto conv_fixup_all = [&](const uint32_t (&notes)[CONV ? C::B_LPW : 1], const int (&os)[CONV ? C::B_LPW : 1],
                            uint32_t dst) __attribute__((always_inline)) {
    if constexpr (CONV) {
#pragma unroll
      for (int qb = 0; qb < C::B_LPW; ++qb) conv_fix_read(qb, notes[qb], dst);
#pragma unroll
      for (int qb = 0; qb < C::B_LPW; ++qb) conv_fix_write(qb, notes[qb], dst);
      conv_fix_special(notes, os, dst);
    }
  };
  auto conv_fixup = [&]() __attribute__((always_inline)) {
    if constexpr (CONV) {
      if (cv_pending) {
        conv_fixup_all(cv_fix, cv_o, cv_dst);
        cv_pending = false;
      }
    }
  };
  // Inside a period the fix-up works on a copy of the notes taken when the period starts (the period's own B ops
  // write new notes): part one of op qb behind MFMA slot CV_FS * qb, part two CV_FD slots later.
  uint32_t cv_old[CONV ? C::B_LPW : 1];
  int cv_old_o[CONV ? C::B_LPW : 1];
  uint32_t cv_old_dst = 0;
  // ... and the lanes fetch the table entries of the slab this period issues, and the first 64 threads tabulate the
  // slab after it (into the table that was last read one period ago, before the barrier that has just been passed)
  auto conv_period_begin = [&]() __attribute__((always_inline)) {
    if constexpr (CONV) {
#pragma unroll
      for (int qb = 0; qb < C::B_LPW; ++qb) { cv_old[qb] = cv_fix[qb]; cv_old_o[qb] = cv_o[qb]; }
      cv_old_dst = cv_dst;
      conv_tab_read();
      conv_tab_write();
    }
  };
  // The period's own loads are all issued in its first half; in the middle of the period the wave waits until only
  // those are outstanding, i.e. until the slab issued one period earlier has landed (loads retire in issue order),
  // and fixes that slab in the second half.  A slab so has a period and a half to arrive.
  constexpr int CV_PERIOD = C::KSTEPS * TM * TN;
  constexpr int CV_WAIT_SLOT = CV_PERIOD / 2;
  constexpr int CV_FD = CV_PERIOD >= 32 ? 6 : 3;                                        // slots between read and write
  constexpr int CV_FS = !CONV ? 1 : ((CV_PERIOD / 2 - CV_FD - 3) / C::B_LPW >= 4 ? 4 : ((CV_PERIOD / 2 - CV_FD - 3) / C::B_LPW >= 2 ? 2 : 1));
  static_assert(!CONV || CV_WAIT_SLOT + 1 + CV_FS * (C::B_LPW - 1) + CV_FD + 1 < CV_PERIOD, "no room for the fix-up in half a period");
  auto conv_fix_slot = [&](int slot) __attribute__((always_inline)) {
    if constexpr (CONV) {
      if (slot == CV_WAIT_SLOT) { TNX_WAIT_VM(C::LPW); }
#pragma unroll
      for (int qb = 0; qb < C::B_LPW; ++qb) {
        if (slot == CV_WAIT_SLOT + 1 + CV_FS * qb) conv_fix_read(qb, cv_old[qb], cv_old_dst);
        if (slot == CV_WAIT_SLOT + 1 + CV_FS * qb + CV_FD) conv_fix_write(qb, cv_old[qb], cv_old_dst);
      }
      if (slot == CV_WAIT_SLOT + 1 + CV_FS * (C::B_LPW - 1) + CV_FD + 1) conv_fix_special(cv_old, cv_old_o, cv_old_dst);
    }
  };

  // one DMA op (q-th of this wave) of local slab t, into ring slot t % STAGES
  auto dma_op = [&](int q, uint32_t stage_base) __attribute__((always_inline)) {
    if (CONV && q >= C::A_LPW) {
      conv_prepare(q - C::A_LPW, stage_base);
      dma16_set_m0(stage_base + C::A_BYTES + ((q - C::A_LPW) * NW + wave) * 1024);
      asm volatile("s_nop 0" ::: "memory");
      conv_go();
    } else if (q < C::A_LPW) {
      dma16(a_sbase, a_voff[q], stage_base + (q * NW + wave) * 1024);
    } else {
      // short tiles are the ones used on skinny problems, where B is the HBM stream
      if (BM <= 64 && p.b_once)
        dma16_nt(b_sbase, b_voff[q - C::A_LPW], stage_base + C::A_BYTES + ((q - C::A_LPW) * NW + wave) * 1024);
      else
        dma16(b_sbase, b_voff[q - C::A_LPW], stage_base + C::A_BYTES + ((q - C::A_LPW) * NW + wave) * 1024);
    }
  };
  // the same op in two parts (see dma16_set_m0): LDS target first, the load after one other instruction
  auto dma_target = [&](int q, uint32_t stage_base) __attribute__((always_inline)) {
    if (CONV && q >= C::A_LPW) conv_prepare(q - C::A_LPW, stage_base);
    if (q < C::A_LPW) dma16_set_m0(stage_base + (q * NW + wave) * 1024);
    else dma16_set_m0(stage_base + C::A_BYTES + ((q - C::A_LPW) * NW + wave) * 1024);
  };
  auto dma_go = [&](int q) __attribute__((always_inline)) {
    if (CONV && q >= C::A_LPW) conv_go();
    else if (q < C::A_LPW) dma16_go<false>(a_sbase, a_voff[q]);
    else if (BM <= 64 && p.b_once) dma16_go<true>(b_sbase, b_voff[q - C::A_LPW]);
    else dma16_go<false>(b_sbase, b_voff[q - C::A_LPW]);
  };
  auto dma_advance = [&]() __attribute__((always_inline)) {
    if (TNX_LADDER == 3) return;        // + DMA ops, always of the tile's first slabs (served by the L2)
    a_sbase += BK * ES;
    if (!CONV) b_sbase += BT ? (int64_t)BK * ES : (int64_t)BK * p.sbk * ES;
  };
  auto stage_of = [&](int t) __attribute__((always_inline)) { return lds0 + (uint32_t)(t % STAGES) * C::STAGE_BYTES; };

  // ---- fragment addressing ----------------------------------------------
  const int wy = wave / C::WGN, wx = wave % C::WGN;
  const int a_row = wy * C::WTM + (lane % MI);
  const int a_kg = lane / MI;
  const int a_sw = C::swzA(a_row);
  uint32_t a_koff[C::KSTEPS];   // byte offset inside the A slab, per k step
#pragma unroll
  for (int ks = 0; ks < C::KSTEPS; ++ks)
    a_koff[ks] = a_row * C::ROWB_A + (((ks * (C::KB / 16) + a_kg) ^ a_sw) << 4);

  const int blk = lane >> 4, li = lane & 15;
  const int b_kg = (MI == 32) ? (blk >> 1) : blk;
  const int b_sub = (ES == 2) ? (li >> 2) : (li >> 1);               // k row inside the transposed block
  const int b_colb0 = (wx * C::WTN + ((MI == 32) ? 16 * (blk & 1) : 0)) * ES + ((ES == 2) ? 8 * (li & 3) : 8 * (li & 1));
  constexpr int RPR = 8 / ES;                                       // k rows one transposing read covers
  const int b_sw = C::swzB((16 / ES) * b_kg + b_sub);     // the same for every k step and both halves of a fragment
  uint32_t b_joff[TN];          // byte offset inside the B slab, per column block
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int colb = b_colb0 + j * MI * ES;
    b_joff[j] = (uint32_t)(((16 / ES) * b_kg + b_sub) * C::ROWB_B) + (((colb >> 4) ^ b_sw) << 4) + (colb & 15);
  }

  // k-contiguous B: fragment j of k step ks sits at bt_koff[ks] + j * MI rows, read like an A fragment
  const int bt_row = wx * C::WTN + (lane % MI);
  uint32_t bt_koff[C::KSTEPS];
#pragma unroll
  for (int ks = 0; ks < C::KSTEPS; ++ks)
    bt_koff[ks] = bt_row * C::ROWB_A + (((ks * (C::KB / 16) + a_kg) ^ C::swzA(bt_row)) << 4);

  acc_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{};

  // two register sets of fragments: one being multiplied, one being filled
  i32x4 fa[2][TM];
  i32x2 fb[2][TN][2];
  i32x4 fbq[2][TN];             // k-contiguous B: one 16-byte read per fragment
  constexpr int NBREAD = BT ? TN : 2 * TN;
  constexpr int NREAD = NBREAD + TM, NMMA = TM * TN;
  constexpr int RPM = (NREAD + NMMA - 1) / NMMA;        // LDS reads slotted behind each MFMA
  constexpr int DPM = (C::LPW + NMMA - 1) / NMMA;       // DMA ops slotted behind each MFMA

  auto read_one = [&](int set, int idx, uint32_t sa, uint32_t sb, int ks) __attribute__((always_inline)) {
    if (BT && idx < NBREAD) {
      fbq[set][idx] = *TNX_LDS(i32x4, sb + bt_koff[ks] + idx * MI * C::ROWB_A);
    } else if (idx < NBREAD) {
      int j = idx >> 1, h = idx & 1;
      fb[set][j][h] = lds_read_tr<ES>(sb + b_joff[j] + ks * C::MMA_K * C::ROWB_B + h * RPR * C::ROWB_B);
    } else {
      int i = idx - NBREAD;
      fa[set][i] = *TNX_LDS(i32x4, sa + a_koff[ks] + i * MI * C::ROWB_A);
    }
  };
  auto mma_one = [&](int set, int idx) __attribute__((always_inline)) {
    int i = idx / TN, j = idx % TN;
    if (i & 1) j = TN - 1 - j;   // serpentine walk of the wave's MFMA tiles: one operand changes per instruction, never both
    i32x4 b4 = BT ? fbq[set][j] : i32x4{fb[set][j][0].x, fb[set][j][0].y, fb[set][j][1].x, fb[set][j][1].y};
    acc[i][j] = MMA::run(b4, fa[set][i], acc[i][j]);   // rows = n, cols = m: the tile comes out transposed
  };

  // ---- pipeline ----------------------------------------------------------
  // Ring of STAGES slabs, one workgroup barrier per slab.  barrier(t) sits
  // before the last k step of slab t: every wave has then issued and received
  // all its LDS reads of slab t, so the slot of slab t is handed to the DMA of
  // slab t+STAGES, and slab t+1 is known to have landed, so its first
  // fragments are fetched under the last k step's MFMAs.  A "period" is the
  // code between barrier(t) and barrier(t+1): the last k step of slab t, then
  // k steps 0..KSTEPS-2 of slab t+1.  The DMA ops of one refill are slotted
  // behind the period's MFMAs at an even rate (a burst of them backs up the
  // texture-address queue and stalls the wave); with only two slabs in the
  // ring the refill is due at the very next barrier, so it is issued in the
  // first k step of the period instead.  The K loop is cut in three (refills
  // to issue / ring draining / final step) so the accumulators flow through
  // straight-line code.
  constexpr int PERIOD = C::KSTEPS * NMMA;                       // MFMA slots per period
  // slots the refill is spread over.  Two-slab rings: the refill is due at the next barrier, so it
  // is front-loaded: over the first half of the period with one wave per SIMD (measured on 8192^3,
  // bf16 256x256x64: a quarter of the period 477, three eighths 853, half 1430, three quarters
  // 1380 TFLOP/s -- a faster burst backs up the texture address path and stalls the wave for far
  // longer than it saves; spread further, the last loads are waited for as soon as they are
  // issued), over the first quarter with two waves per SIMD (the other wave covers the stall).
  constexpr int SPAN2 = (NW == 4 ? PERIOD / 2 : PERIOD / 4) > 0 ? (NW == 4 ? PERIOD / 2 : PERIOD / 4) : 1;
  // (CONV: three slots, but every load is waited for at the next barrier as with two)
  constexpr int SPAN = (STAGES == 2 || !FAST || CONV) ? SPAN2 : PERIOD;
  // loads of this wave that may still be in flight when a period starts (CONV: the slab issued in the period
  // before, which is waited for in the middle of this one)
  constexpr int PWAIT = CONV ? C::LPW : (STAGES - 2) * C::LPW;
  constexpr int LAST = (C::KSTEPS - 1) & 1;                      // register set holding the last k step
  constexpr int NEXT0 = C::KSTEPS & 1;                           // set that receives step 0 of the next slab

  // One MFMA slot: the MFMA, then the LDS reads and DMA ops slotted behind it.  When exactly one DMA op and at
  // least one read are due, the read sits between the op's M0 write and its load (it fills the wait state).
  auto slot_body = [&](int mset, int x, int rset, int& rd, uint32_t sa, uint32_t sb, int ks_next, bool with_dma, int slot,
                       uint32_t dst) __attribute__((always_inline)) {
    mma_one(mset, x);
    if (TNX_LADDER == 1) {              // MFMAs only
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    if (TNX_LADDER == 2) with_dma = false;   // + fragment reads: the ring keeps the slabs of the prologue
    if (with_dma) conv_fix_slot(slot);
    int lo = 0, hi = 0;
    if (with_dma && slot < SPAN) { lo = slot * C::LPW / SPAN; hi = (slot + 1) * C::LPW / SPAN; }
    const bool paired = hi - lo == 1 && rd < NREAD;
    if (paired) dma_target(lo, dst);
#pragma unroll
    for (int q = 0; q < RPM; ++q)
      if (rd < NREAD) { read_one(rset, rd, sa, sb, ks_next); ++rd; }
    if (paired) dma_go(lo);
    else
#pragma unroll
      for (int q = lo; q < hi; ++q) dma_op(q, dst);
    __builtin_amdgcn_sched_barrier(0);
  };
  // `par` (0 or 1, compile-time) is added to every register-set index: with an odd number of k steps per slab
  // the two sets trade roles from one slab to the next, and the unrolled bulk of the K loop follows that by
  // alternating par; where the slab index is a run-time value (par = 0) the sets are swapped by copying.
  auto inner_steps = [&](uint32_t sa, uint32_t sb, auto with_dma, uint32_t dst, auto par) __attribute__((always_inline)) {
    constexpr bool WITH_DMA = decltype(with_dma)::value;
    constexpr int P = decltype(par)::value;
#pragma unroll
    for (int ks = 0; ks + 1 < C::KSTEPS; ++ks) {
      int rd = 0;
#pragma unroll
      for (int x = 0; x < NMMA; ++x)
        slot_body((ks + P) & 1, x, (ks + 1 + P) & 1, rd, sa, sb, ks + 1, WITH_DMA, NMMA + ks * NMMA + x, dst);
    }
  };
  // last k step of the slab whose fragments sit in set LAST; prefetches step 0 of the slab at (sa1, sb1)
  // (`par` is the parity of the slab that is ending; `swap`: bring the sets back to par = 0 by copying)
  auto last_step = [&](uint32_t sa1, uint32_t sb1, auto with_dma, uint32_t dst, auto par, auto swap) __attribute__((always_inline)) {
    constexpr bool WITH_DMA = decltype(with_dma)::value;
    constexpr int P = decltype(par)::value;
    int rd = 0;
#pragma unroll
    for (int x = 0; x < NMMA; ++x) slot_body((LAST + P) & 1, x, (NEXT0 + P) & 1, rd, sa1, sb1, 0, WITH_DMA, x, dst);
    if ((C::KSTEPS & 1) && decltype(swap)::value) {   // odd KSTEPS: the two register sets trade roles every slab
#pragma unroll
      for (int i = 0; i < TM; ++i) { i32x4 tmp = fa[0][i]; fa[0][i] = fa[1][i]; fa[1][i] = tmp; }
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) { i32x2 tmp = fb[0][j][h]; fb[0][j][h] = fb[1][j][h]; fb[1][j][h] = tmp; }
#pragma unroll
      for (int j = 0; j < TN; ++j) { i32x4 tmp = fbq[0][j]; fbq[0][j] = fbq[1][j]; fbq[1][j] = tmp; }
    }
  };
  typedef BoolTag<true> Yes;
  typedef BoolTag<false> No;
  typedef IntTag<0> Par0;

  // first STAGES slabs of the tile the loader stands on
  auto issue_prologue = [&]() __attribute__((always_inline)) {
    if constexpr (CONV) {
      // slabs 0 and 1 are read before any period could fix them: both are issued, waited for and fixed here;
      // slab 2 is issued afterwards and takes the regular route.  The tap tables of slabs 0..3 are written on the
      // way, each behind a barrier that separates it from the reads of the table it replaces; the table of slab 3
      // is published by the first period's barrier.
      uint32_t first[C::B_LPW];
      int first_o[C::B_LPW];
      const uint32_t dst0 = stage_of(0);
      conv_tab_write();                       // slab 0 -> table 0
      __syncthreads();
      conv_tab_read();
      if (KT > 0) {
#pragma unroll
        for (int q = 0; q < C::LPW; ++q) dma_op(q, dst0);
        dma_advance();
#pragma unroll
        for (int qb = 0; qb < C::B_LPW; ++qb) { first[qb] = cv_fix[qb]; first_o[qb] = cv_o[qb]; }
      }
      conv_tab_write();                       // slab 1 -> table 1
      __syncthreads();
      conv_tab_read();
      if (KT > 1) {
#pragma unroll
        for (int q = 0; q < C::LPW; ++q) dma_op(q, stage_of(1));
        dma_advance();
      }
      TNX_WAIT_VM(0);
      if (KT > 0) conv_fixup_all(first, first_o, dst0);
      if (KT > 1) conv_fixup_all(cv_fix, cv_o, stage_of(1));
      cv_pending = false;
      conv_tab_write();                       // slab 2 -> table 0 (its readers passed the barrier above)
      __syncthreads();
      conv_tab_read();
      if (KT > 2) {
#pragma unroll
        for (int q = 0; q < C::LPW; ++q) dma_op(q, stage_of(2));
        dma_advance();
      }
      conv_tab_write();                       // slab 3 -> table 1
      __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the fix-up writes are done before the barrier that follows
      return;
    }
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
      if (s < KT) {
        if constexpr (FAST) {
#pragma unroll
          for (int q = 0; q < C::LPW; ++q) dma_op(q, stage_of(s));
          dma_advance();
        } else {
          load_slab_generic(kt0 + s, stage_of(s), tid);
        }
      }
    }
  };
  // the K loop of one tile, from "slab 0 has landed" to the last MFMA; the prologue has been issued
  auto k_loop = [&]() __attribute__((always_inline)) {
  if (KT > 0) {
    __syncthreads();
    const uint32_t sa = stage_of(0), sb = sa + C::A_BYTES;
#pragma unroll
    for (int r = 0; r < NREAD; ++r) read_one(0, r, sa, sb, 0);
    if (TNX_LADDER == 1) {
#pragma unroll
      for (int r = 0; r < NREAD; ++r) read_one(1, r, sa, sb, C::KSTEPS > 1 ? 1 : 0);
    }
    inner_steps(sa, sb, No{}, 0u, Par0{});
  }

  int t = 0;
  // (1) periods that issue the refill of slab t+STAGES into the slot of slab t.  The bulk runs
  // STAGES periods per trip so every ring slot is a compile-time constant there (LDS addresses
  // become instruction immediates, DMA targets become scalar constants); what is left over runs
  // with run-time slots.
  // With an odd number of k steps per slab the trip covers an even number of periods, so that the register
  // sets are back in their starting roles at the end of every trip without a copy.
  if constexpr (FAST) {
    constexpr int U = ((C::KSTEPS & 1) && (STAGES & 1)) ? 2 * STAGES : STAGES;
    for (; t + U + STAGES - 1 < KT; t += U) {
      auto period = [&](auto jtag) __attribute__((always_inline)) {
        constexpr int j = decltype(jtag)::value;
        constexpr int P = (C::KSTEPS & 1) ? (j & 1) : 0;          // parity of the slab whose last k step runs now
        if (TNX_LADDER != 1) {
          if (TNX_LADDER != 4) __builtin_amdgcn_s_waitcnt((PWAIT & 0xF) | (((PWAIT >> 4) & 0x3) << 14) | 0x0070);
          __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_sched_barrier(0);
        conv_period_begin();
        const uint32_t dst = lds0 + (uint32_t)(j % STAGES) * C::STAGE_BYTES;
        const uint32_t sa1 = lds0 + (uint32_t)((j + 1) % STAGES) * C::STAGE_BYTES, sb1 = sa1 + C::A_BYTES;
        last_step(sa1, sb1, Yes{}, dst, IntTag<P>{}, No{});
        inner_steps(sa1, sb1, Yes{}, dst, IntTag<(C::KSTEPS & 1) ? (P ^ 1) : 0>{});
        dma_advance();
      };
      static_assert(U <= 12, "unroll table below covers twelve periods");
      period(IntTag<0>{});
      if constexpr (U > 1) period(IntTag<1>{});
      if constexpr (U > 2) period(IntTag<2>{});
      if constexpr (U > 3) period(IntTag<3>{});
      if constexpr (U > 4) period(IntTag<4>{});
      if constexpr (U > 5) period(IntTag<5>{});
      if constexpr (U > 6) period(IntTag<6>{});
      if constexpr (U > 7) period(IntTag<7>{});
      if constexpr (U > 8) period(IntTag<8>{});
      if constexpr (U > 9) period(IntTag<9>{});
      if constexpr (U > 10) period(IntTag<10>{});
      if constexpr (U > 11) period(IntTag<11>{});
    }
  }
  for (; t + STAGES < KT; ++t) {
    __builtin_amdgcn_s_waitcnt((PWAIT & 0xF) | (((PWAIT >> 4) & 0x3) << 14) | 0x0070);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    conv_period_begin();
    const uint32_t dst = stage_of(t);
    const uint32_t sa1 = stage_of(t + 1), sb1 = sa1 + C::A_BYTES;
    if constexpr (FAST) {
      last_step(sa1, sb1, Yes{}, dst, Par0{}, Yes{});
      inner_steps(sa1, sb1, Yes{}, dst, Par0{});
      dma_advance();
    } else {
      // slab t + STAGES: fetched into registers now, written to the freed slot after this period's MFMAs; the
      // writes have to be in LDS before the next barrier lets anyone read them
      i32x4 ra[GEN_NA], rb[GEN_NB];
      gen_fetch(kt0 + t + STAGES, tid, ra, rb);
      last_step(sa1, sb1, No{}, 0u, Par0{}, Yes{});
      inner_steps(sa1, sb1, No{}, 0u, Par0{});
      gen_store(dst, tid, ra, rb);
      __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
    }
  }
  // (2) ring draining: nothing left to issue
  for (; t + 1 < KT; ++t) {
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    conv_fixup();      // CONV: the last slab that was issued has landed; nothing reads it before the next barrier
    const uint32_t sa1 = stage_of(t + 1), sb1 = sa1 + C::A_BYTES;
    last_step(sa1, sb1, No{}, 0u, Par0{}, Yes{});
    inner_steps(sa1, sb1, No{}, 0u, Par0{});
  }
  // (3) last k step of the final slab
  if (KT > 0) {
#pragma unroll
    for (int x = 0; x < NMMA; ++x) mma_one(LAST, x);
  }
  };

  // Ping-pong form of the K loop (TNX_PINGPONG builds).  The waves 0..NW/2-1 ("lead") and NW/2..NW-1 share the SIMDs
  // pairwise.  Time runs in phases 0..2*KT, a workgroup barrier before each; slab v takes two of them:
  //   phase 2v     lead: reads both k steps' fragments of slab v from LDS      other: the MFMAs of slab v-1
  //                both: issue their DMA ops of slab v+1 into the slot slab v-1 has left (read last in phase 2v-1)
  //   phase 2v+1   lead: the MFMAs of slab v, priority raised                   other: reads slab v; all wait for the DMA
  // and phase 2*KT for the second group's last slab.  Each group runs its own straight loop; both execute 2*KT+1
  // barriers.  Needs an even KT >= 2 (the prologue has issued slabs 0 and 1); the caller falls back to k_loop().
  auto pingpong_loop = [&]() __attribute__((always_inline)) {
    constexpr int NRD = C::KSTEPS * NREAD, NMM = C::KSTEPS * NMMA;
    auto load_phase = [&](uint32_t sa, auto with_dma, uint32_t dst) __attribute__((always_inline)) {
      constexpr bool WITH_DMA = decltype(with_dma)::value;
      // opaque slot base: the lane addresses of the phase are formed here and die with it, instead of one set per
      // slot living in registers through every phase
      asm volatile("" : "+s"(sa));
      const uint32_t sb = sa + C::A_BYTES;
#pragma unroll
      for (int i = 0; i < NRD; ++i) {
        if (TNX_PINGPONG != 3) read_one(i / NREAD, i % NREAD, sa, sb, i / NREAD);
        if constexpr (WITH_DMA) {
#pragma unroll
          for (int q = i * C::LPW / NRD; q < (i + 1) * C::LPW / NRD; ++q) if (TNX_PINGPONG != 4) dma_op(q, dst);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (WITH_DMA) dma_advance();
      __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the slot may be refilled after the next barrier
    };
    auto mma_phase = [&](auto with_dma, uint32_t dst) __attribute__((always_inline)) {
      constexpr bool WITH_DMA = decltype(with_dma)::value;
      constexpr int HALF = NMM / 2;         // the refill goes out under the first half of the MFMAs
      if (TNX_PINGPONG != 2) __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int i = 0; i < NMM; ++i) {
        if (TNX_PINGPONG != 5) mma_one(i / NMMA, i % NMMA);
        if constexpr (WITH_DMA) {
          if (i < HALF) {
#pragma unroll
            for (int q = i * C::LPW / HALF; q < (i + 1) * C::LPW / HALF; ++q) if (TNX_PINGPONG != 4) dma_op(q, dst);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_setprio(0);
      if constexpr (WITH_DMA) dma_advance();
    };
    auto phase_barrier = [&]() __attribute__((always_inline)) {
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    const uint32_t s0 = lds0, s1 = lds0 + C::STAGE_BYTES;
    if (wave < NW / 2) {
      for (int v = 0; v < KT; v += 2) {
        phase_barrier();                                             // phase 2v
        if (v > 0) load_phase(s0, Yes{}, s1); else load_phase(s0, No{}, 0u);
        phase_barrier();                                             // 2v+1
        mma_phase(No{}, 0u);
        TNX_WAIT_VM(0);
        phase_barrier();                                             // 2v+2
        if (v + 2 < KT) load_phase(s1, Yes{}, s0); else load_phase(s1, No{}, 0u);
        phase_barrier();                                             // 2v+3
        mma_phase(No{}, 0u);
        TNX_WAIT_VM(0);
      }
      phase_barrier();                                               // phase 2*KT: the other group's last MFMAs
    } else {
      phase_barrier();                                               // phase 0: nothing to multiply yet
      for (int v = 0; v + 2 < KT; v += 2) {
        phase_barrier();                                             // 2v+1
        load_phase(s0, No{}, 0u);
        TNX_WAIT_VM(0);
        phase_barrier();                                             // 2v+2: slab v, and the DMA of slab v+2
        mma_phase(Yes{}, s0);
        phase_barrier();                                             // 2v+3
        load_phase(s1, No{}, 0u);
        TNX_WAIT_VM(0);
        phase_barrier();                                             // 2v+4: slab v+1, and the DMA of slab v+3
        mma_phase(Yes{}, s1);
      }
      phase_barrier();                                               // the last two slabs: nothing left to fetch
      load_phase(s0, No{}, 0u);
      TNX_WAIT_VM(0);
      phase_barrier();
      mma_phase(No{}, 0u);
      phase_barrier();
      load_phase(s1, No{}, 0u);
      phase_barrier();                                               // phase 2*KT
      mma_phase(No{}, 0u);
    }
  };
  typedef typename OutOf<T>::type O;
  if constexpr (!PERSIST) {
    if (KT > 0) {
      issue_prologue();
      if (KT >= STAGES) { TNX_WAIT_VM((STAGES - 1) * C::LPW); } else { TNX_WAIT_VM(0); }
    }
    if (PINGPONG_TILE && KT >= 2 && (KT & 1) == 0) pingpong_loop();
    else k_loop();
    if constexpr (FAST && !CONV) {
      if (tail_here) {
        // the left-out slab: every wave is done with the ring, slot 0 takes it, one slab of MFMAs follows
        __syncthreads();
        load_slab_generic(kt1 - 1, stage_of(0), wave * 64 + lane);
        __syncthreads();
        const uint32_t sa = stage_of(0), sb = sa + C::A_BYTES;
#pragma unroll
        for (int ks = 0; ks < C::KSTEPS; ++ks) {
#pragma unroll
          for (int idx = 0; idx < NREAD; ++idx) read_one(0, idx, sa, sb, ks);
#pragma unroll
          for (int x = 0; x < NMMA; ++x) mma_one(0, x);
        }
      }
    }

    // ---- epilogue ------------------------------------------------------------
    // every wave is done with the slabs before the LDS is reused for the output strips
    __syncthreads();
    const int64_t gm0 = m0 + wy * C::WTM;
    const int64_t gn0 = n0 + wx * C::WTN;
    const uint32_t strip = lds0 + wave * EpiStage<C>::WAVE_BYTES;
    if constexpr (CONV) {
      if (p.out_dtype == DT_F32) epilogue_store_conv<T, C, OutF32>(acc, p.c, strip, lane, (int)gm0, (int)gn0, p.cv);
      else epilogue_store_conv<T, C, O>(acc, p.c, strip, lane, (int)gm0, (int)gn0, p.cv);
      return;
    }
    // the output type: the input's own 16-bit type (int32 for int8), or binary32 where that epilogue is built
    auto finish = [&](auto otag) __attribute__((always_inline)) {
      typedef typename decltype(otag)::type OT;
      if (cut) {
        // workspace after the counters: [slice][cut tile][wave][group][lane] 16-byte elements
        const int ncut = ntiles - p.split_tile0, ctile = logical - p.split_tile0;
        const int64_t slice_stride = (int64_t)ncut * BM * BN * 4;
        uint8_t* wave0 = p.ws + WS_COUNTER_BYTES + ((int64_t)ctile * NW + wave) * (C::WTM * C::WTN * 4);
        const bool atomic = p.atomic_reduce != 0;
        if (!splitk_arrive<T, C>(acc, wave0 + (atomic ? 0 : split * slice_stride), strip, lane, gm0, p.m, (int*)p.ws + ctile,
                                 (int*)smem, p.split_k, atomic))
          return;
        const SliceSrc src = {wave0, (uint32_t)slice_stride, atomic ? 1 : p.split_k, atomic};
        if (p.epilogue == EPI_NONE)
          epilogue_store<T, C, OT, false, true>(acc, src, p.c, strip, lane, gm0, gn0, p.m, p.n, p.scm, p.scn, p.c_row_ok, 0);
        else
          epilogue_store<T, C, OT, true, true>(acc, src, p.c, strip, lane, gm0, gn0 >> 1, p.m, p.n >> 1, p.scm, p.scn,
                                               p.c_row_ok, p.epilogue);
      } else {
        const SliceSrc none = {nullptr, 0, 0, false};
        if (p.epilogue == EPI_NONE)
          epilogue_store<T, C, OT, false, false, MULTI>(acc, none, p.c, strip, lane, gm0, gn0, p.m, p.n, p.scm, p.scn, p.c_row_ok, 0,
                                                        p.cv.bias, p.cv.bias_dtype);
        else
          epilogue_store<T, C, OT, true, false>(acc, none, p.c, strip, lane, gm0, gn0 >> 1, p.m, p.n >> 1, p.scm, p.scn,
                                                p.c_row_ok, p.epilogue);
      }
    };
    if constexpr (f32_out_tile<T, C>()) {
      if (p.out_dtype == DT_F32) {
        finish(TypeTag<OutF32>{});
        return;
      }
    }
    finish(TypeTag<O>{});
  } else {
    // ---- persistent: this workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ... ------------
    // The host launches it only with KT >= STAGES.  While the epilogue of a tile runs, the first
    // STAGES slabs of the next tile are already on their way into the ring, and the epilogue's
    // stores drain under the next tile's first K slabs.  vmcnt retires in issue order, so
    // "at most X operations outstanding" means the X youngest: after an epilogue these are its
    // stores, and everything older -- the next tile's prologue -- has landed.  X may therefore
    // include the stores only when their number is known exactly (a tile fully inside C with
    // 16-byte stores); otherwise it is the (STAGES - 1) slabs of the prologue that may stay in
    // flight, as for the first tile.
    const uint32_t strip = lds0 + C::LDS_BYTES + wave * PairStrip<C>::WAVE_BYTES;
    constexpr int X_FIRST = (STAGES - 1) * C::LPW;
    constexpr int NST_PLAIN = PairEpilogue<T, C, O, false>::STORES, NST_GLU = PairEpilogue<T, C, O, true>::STORES;
    constexpr int X_PLAIN = X_FIRST + NST_PLAIN > 63 ? 63 : X_FIRST + NST_PLAIN;
    constexpr int X_GLU = X_FIRST + NST_GLU > 63 ? 63 : X_FIRST + NST_GLU;
    const bool glu = p.epilogue != EPI_NONE;
    issue_prologue();
    TNX_WAIT_VM(X_FIRST);
    for (int id = blockIdx.x; id < ntiles; id += gridDim.x) {
      k_loop();
      // every wave is done with the ring: it can take the next tile's first slabs
      __syncthreads();
      const int64_t gm0 = m0 + wy * C::WTM;
      const int64_t gn0 = n0 + wx * C::WTN;
      const bool full = p.c_vec_ok && m0 + BM <= p.m && n0 + BN <= p.n;
      const int next = id + gridDim.x;
      if (next < ntiles) {
        int nm, nn;
        locate(next, &nm, &nn);
        place_tile(nm, nn);
        issue_prologue();
      }
      // The epilogue's per-lane offsets depend only on the lane: left alone, the compiler computes them once
      // before the tile loop and keeps them in registers across every K loop, which spills.  An opaque copy of
      // the lane index ties them to this iteration.
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      if (!glu) {
        if (full) epilogue_store_pairs<T, C, O, false, true>(acc, p.c, strip, lane_e, gm0, gn0, p.m, p.n, p.scm, p.scn, true, 0);
        else epilogue_store_pairs<T, C, O, false, false>(acc, p.c, strip, lane_e, gm0, gn0, p.m, p.n, p.scm, p.scn, p.c_vec_ok, 0);
      } else {
        if (full) epilogue_store_pairs<T, C, O, true, true>(acc, p.c, strip, lane_e, gm0, gn0 >> 1, p.m, p.n >> 1, p.scm, p.scn, true, p.epilogue);
        else epilogue_store_pairs<T, C, O, true, false>(acc, p.c, strip, lane_e, gm0, gn0 >> 1, p.m, p.n >> 1, p.scm, p.scn, p.c_vec_ok, p.epilogue);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{};
      if (next < ntiles) {
        if (!full) { TNX_WAIT_VM(X_FIRST); }
        else if (glu) { TNX_WAIT_VM(X_GLU); }
        else { TNX_WAIT_VM(X_PLAIN); }
      }
    }
  }
}

}  // namespace tnx
