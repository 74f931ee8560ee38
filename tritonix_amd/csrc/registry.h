// Table of compiled tile kernels.  Each generated instance file contributes
// one array of KernelEntry; capi.hip looks a tile config up in the union.
#pragma once
#include <hip/hip_runtime.h>

#include "gemm_tile.h"

struct tnx_gemm_args;

namespace tnx {

typedef hipError_t (*launch_fn)(const GemmParams& p, unsigned grid, hipStream_t stream);

struct KernelEntry {
  int dtype, bm, bn, bk, nw, stages;
  int lds_bytes;
  launch_fn fast;     // DMA loader: row-major, 16-byte aligned, k % bk == 0
  launch_fn generic;  // element-wise loader: any strides / ragged k; may be null
  launch_fn persist;  // DMA loader, one workgroup per CU walking its tiles; may be null
  launch_fn fast_bt;  // DMA loader for k-contiguous B (stride_bk == 1, the `x @ w.t()` layout); may be null
  launch_fn conv;     // conv2d forward on the DMA loader (GemmParams::cv); may be null
};

// records the hipError_t behind a TNX_E_HIP for tnx_last_hip_error() (per thread)
void note_hip_error(int err);
// tnx_gemm with `batch` problems in one grid -- same A, problem i reads b + i * b_batch_bytes and writes
// c + i * c_batch_bytes -- and an optional bias per row of C, added to the fp32 sum before the rounding (float types).
// Uncut, non-persistent launches of tiles up to 128x128 only (multi_problem_tile).  conv2d's 1x1 layers are this GEMM,
// one problem per image.
struct GemmBatch {
  int batch;
  int64_t b_batch_bytes, c_batch_bytes;
  const void* bias;
  int bias_dtype;
};
int gemm_launch(const tnx_gemm_args* a, const GemmBatch* extra);
// waves and stages of a built tile with these dimensions that gemm_launch takes with a GemmBatch (eight waves and
// two ring slots first); false: none built
bool gemm_tile_for(int dtype, int bm, int bn, int bk, int* num_warps, int* num_stages);

struct KernelGroup {
  KernelEntry* entries;
  int count;
};

template <class T, class C, bool FAST, bool PERSIST = false, bool BT = false, bool CONV = false>
hipError_t launch_tile(const GemmParams& p, unsigned grid, hipStream_t stream) {
  static_assert(C::VALID, "tile configuration is not buildable");
  hipLaunchKernelGGL((gemm_tile_kernel<T, C, FAST, PERSIST, BT, CONV>), dim3(grid), dim3(C::THREADS), 0, stream, p);
  return hipGetLastError();
}

// The persistent variant exists for the four-wave tiles from 128x128 to 256x128 / 128x256: their ring leaves
// room for the epilogue's own strips (MI rows of 256 bytes per wave) inside the 160 KiB of one CU, and a wave's
// accumulators take at most 128 registers, so the state the tile loop carries still fits the register file
// (with the 256 accumulator registers of a 256x256 tile it does not: the compiler spills inside the K loop).
template <class C> constexpr bool persist_ok() {
  return C::NW == 4 && C::BM >= 128 && C::BN >= 128 && C::TN % PairStrip<C>::TPP == 0 &&
         C::TM * C::TN * C::ACC_N <= 128 && C::LDS_BYTES + PairStrip<C>::BYTES <= 163840;
}
template <class T, class C, bool OK = persist_ok<C>()> struct PersistLaunch {
  static constexpr launch_fn fn = nullptr;
};
template <class T, class C> struct PersistLaunch<T, C, true> {
  static constexpr launch_fn fn = &launch_tile<T, C, true, true>;
};

// skinny kernel (gemm_skinny.h): tile 16 x 32 x 32, eight waves, split_k == 8 inside the workgroup,
// num_stages = ring depth per wave.  Null when that depth / dtype is not built.
launch_fn skinny_lookup(int dtype, int ring);
constexpr int SKINNY_BM = 16, SKINNY_BN = 32, SKINNY_BK = 32, SKINNY_NW = 8, SKINNY_SPLIT = 8;
constexpr int SKINNY_STEP_BYTES = 3072;

// The k-contiguous-B variant exists for the tiles whose K slab is one 128-byte line per row (the tiles the
// built-in choice uses).
template <class C> constexpr bool bt_ok() { return C::BK * C::ES == 128; }
template <class T, class C, bool OK = bt_ok<C>()> struct BtLaunch {
  static constexpr launch_fn fn = nullptr;
};
template <class T, class C> struct BtLaunch<T, C, true> {
  static constexpr launch_fn fn = &launch_tile<T, C, true, false, true>;
};

// The conv2d variant exists for the three-slot, eight-wave 16-bit tiles 128x128, 256x128 and 128x256 with a 128-byte K
// slab (with four waves it was measured 15-20 % slower, and 256x256 then has no registers left for the loader's state;
// three slots of 256x256 do not fit the LDS; a 64-channel tile was measured and loses to the
// register-staged kernel).  The second half of a period must have room for the slotted fix-up of all B ops.
template <class C> constexpr bool conv_ok() {
  return C::ES == 2 && C::NW == 8 && C::KSTEPS * C::TM * C::TN >= 16 &&
         C::KSTEPS * C::TM * C::TN / 2 > C::B_LPW + (C::KSTEPS * C::TM * C::TN >= 32 ? 6 : 3) + 1 && C::STAGES == 3 && C::BK == 64 &&
         C::BM >= 128 && C::BN >= 128 && C::TM * C::TN * C::ACC_N <= 128 && (C::NW * 64) % C::CPR_B == 0;
}
template <class T, class C, bool OK = conv_ok<C>()> struct ConvLaunch {
  static constexpr launch_fn fn = nullptr;
};
template <class T, class C> struct ConvLaunch<T, C, true> {
  static constexpr launch_fn fn = &launch_tile<T, C, true, false, false, true>;
};

// The element-wise loader is built only for the tiles that ask for it (a conditional expression would instantiate
// the kernel for every tile and merely not point at it).
template <class T, class C, bool WANTED> struct GenericLaunch {
  static constexpr launch_fn fn = nullptr;
};
template <class T, class C> struct GenericLaunch<T, C, true> {
  static constexpr launch_fn fn = &launch_tile<T, C, false>;
};

#define TNX_ENTRY(TAG, BM, BN, BK, NW, ST, GENERIC)                                                          \
  {TAG::ID, BM, BN, BK, NW, ST, TileCfg<TAG, BM, BN, BK, NW, ST>::LDS_BYTES,                                 \
   &launch_tile<TAG, TileCfg<TAG, BM, BN, BK, NW, ST>, true>,                                                \
   GenericLaunch<TAG, TileCfg<TAG, BM, BN, BK, NW, ST>, GENERIC>::fn,                                        \
   PersistLaunch<TAG, TileCfg<TAG, BM, BN, BK, NW, ST>>::fn, BtLaunch<TAG, TileCfg<TAG, BM, BN, BK, NW, ST>>::fn,     \
   ConvLaunch<TAG, TileCfg<TAG, BM, BN, BK, NW, ST>>::fn}

}  // namespace tnx
