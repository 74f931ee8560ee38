// Skinny GEMM for decode shapes (m <= 16): C[m,n] = A[m,k] @ B[k,n] with B streamed once from HBM.
//
// Same contract as the split-K kernel of the reference (tritonix/ops/matmul.py:147-202): K is
// cut into slices, slices are accumulated in fp32 and rounded once.  Here the split is
// wavefront-level: the eight waves of a workgroup own one 32-column strip of C and one eighth
// of K each, stream their slice through a private LDS ring with 16-byte direct-to-LDS loads
// (no workgroup barrier in the loop, no global partials, no second pass) and meet once, in
// LDS, at the end.  One k step is 32 rows: two 1 KiB DMA ops for B[32 x 32], one for A[16 x 32],
// one ds_read_b128 + four transposing ds_read_b64_tr_b16 and two v_mfma_f32_16x16x32.
#pragma once
#include "gemm_tile.h"

namespace tnx {

constexpr int SK_WAVES = 8;    // = the split factor
constexpr int SK_BN = 32;      // columns per workgroup
constexpr int SK_KSTEP = 32;   // k rows per step
constexpr int SK_STEP_BYTES = 3072;  // B 32x32 (2 KiB) + A 16x32 (1 KiB), 16-bit elements

template <class T, int RING>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(GemmParams p) {
  static_assert(T::ES == 2, "16-bit element types only");
  static_assert(RING >= 2 && (RING - 1) * 3 <= 63, "ring depth out of range for vmcnt");
  typedef Mma<T, 16> MMA;
  constexpr int LDS_BYTES = SK_WAVES * RING * SK_STEP_BYTES;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BYTES];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(uint8_t __attribute__((address_space(3)))*)smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ntiles = (int)(p.n / SK_BN);
  const int64_t n0 = (int64_t)xcd_remap(blockIdx.x, ntiles, 8) * SK_BN;   // neighbouring strips share an L2
  const int64_t kw = p.k / SK_WAVES;                                       // k rows of this wave
  const int steps = (int)(kw / SK_KSTEP);
  const int64_t k0 = (int64_t)wave * kw;
  const uint32_t ring = lds0 + (uint32_t)wave * RING * SK_STEP_BYTES;

  // ---- DMA source offsets (bytes, constant over the loop); the chunk XORs spread LDS banks
  const int drow = lane >> 2, dchunk = lane & 3;
  const int64_t ldb = p.sbk, lda = p.sam;
  uint32_t b_voff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = drow + 16 * h;
    const int c = dchunk ^ (((row >> 1) & 1) << 1);
    b_voff[h] = (uint32_t)(row * ldb * 2 + c * 16);
  }
  const int arow = drow < p.m ? drow : (int)p.m - 1;                       // rows past m: any valid row
  const uint32_t a_voff = (uint32_t)(arow * lda * 2 + ((dchunk ^ ((drow ^ (drow >> 2)) & 3)) * 16));
  const uint8_t* b_base = uniform_ptr(p.b + (k0 * ldb + n0) * 2);
  const uint8_t* a_base = uniform_ptr(p.a + k0 * 2);
  const int64_t b_step = (int64_t)SK_KSTEP * ldb * 2;

  auto issue = [&](int s) {
    const uint32_t slot = ring + (uint32_t)(s % RING) * SK_STEP_BYTES;
    dma16(b_base, b_voff[0], slot);
    dma16(b_base, b_voff[1], slot + 1024);
    dma16(a_base, a_voff, slot + 2048);
    b_base += b_step;
    a_base += SK_KSTEP * 2;
  };

  // ---- fragment read offsets inside a ring slot
  const int blk = lane >> 4, li = lane & 15;
  // A: row li, k chunk blk
  const uint32_t a_off = 2048 + li * 64 + ((blk ^ ((li ^ (li >> 2)) & 3)) << 4);
  // B (transposing read): k rows 8*blk + 4*h + (li >> 2), columns 16*j + 4*(li & 3) .. +3
  uint32_t b_off[2][2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = 8 * blk + 4 * h + (li >> 2);
      const int colb = j * 32 + 8 * (li & 3);
      b_off[j][h] = row * 64 + ((((colb >> 4) ^ (((row >> 1) & 1) << 1))) << 4) + (colb & 15);
    }

  f32x4 acc[2] = {f32x4{}, f32x4{}};
  auto compute = [&](int s) {
    const uint32_t slot = ring + (uint32_t)(s % RING) * SK_STEP_BYTES;
    const i32x4 af = *TNX_LDS(i32x4, slot + a_off);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const i32x2 lo = lds_read_tr<2>(slot + b_off[j][0]);
      const i32x2 hi = lds_read_tr<2>(slot + b_off[j][1]);
      acc[j] = MMA::run(i32x4{lo.x, lo.y, hi.x, hi.y}, af, acc[j]);   // rows = n, cols = m
    }
  };

  // ---- stream: RING-1 steps in flight, no workgroup barrier
  for (int s = 0; s < RING - 1 && s < steps; ++s) issue(s);
  int s = 0;
  for (; s + RING - 1 < steps; ++s) {
    issue(s + RING - 1);                       // refills the slot step s-1 was read from
    TNX_WAIT_VM((RING - 1) * 3);               // step s has landed
    compute(s);
  }
  TNX_WAIT_VM(0);
  for (; s < steps; ++s) compute(s);

  // ---- meet in LDS: red[wave][m][n] fp32, then 512 threads own one output each
  __syncthreads();
  float* red = (float*)smem;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    // lane: column m = lane % 16 of C^T, rows n = 16*j + 4*(lane / 16) + 0..3
    float* dst = red + (wave * 16 + li) * SK_BN + j * 16 + 4 * blk;
    *(f32x4*)dst = acc[j];
  }
  __syncthreads();
  const int om = tid / SK_BN, on = tid % SK_BN;
  float sum = 0.f;
#pragma unroll
  for (int w = 0; w < SK_WAVES; ++w) sum += red[(w * 16 + om) * SK_BN + on];
  if (om < p.m) {
    const int64_t off = (int64_t)om * p.scm + (n0 + on) * p.scn;
    if (T::ID == DT_BF16) ((uint16_t*)p.c)[off] = f32_to_bf16(sum);
    else ((_Float16*)p.c)[off] = (_Float16)sum;
  }
}

template <class T, int RING>
hipError_t launch_skinny(const GemmParams& p, unsigned grid, hipStream_t stream) {
  hipLaunchKernelGGL((gemm_skinny_kernel<T, RING>), dim3(grid), dim3(SK_WAVES * 64), 0, stream, p);
  return hipGetLastError();
}

}  // namespace tnx
