// Measurement aid: what the MFMA pipes of this board sustain with no data movement at all.
//
// One workgroup of four waves per CU; every wave keeps a 128x128 accumulator tile and 16 operand
// fragments in registers and issues nothing but MFMAs on them (plus one bit-flip per 8 MFMAs so the
// operands are not loop-invariant).  With operands that toggle like real data the board runs into
// its power limit and lowers the shader clock, so the rate this loop reaches is an upper bound for
// any GEMM kernel on such operands -- the kernels in gemm_tile.h add LDS, L2 and HBM traffic on top.
// With all-zero operands the same loop runs at the full clock.
//
// Second aid: one wave issuing one kind of LDS instruction on a caller-given table of per-lane addresses, for the
// bank-conflict counters (which lanes an instruction serves in one cycle is not documented; the A-slab swizzle in
// gemm_tile.h is built on what this probe shows).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tritonix_hip.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
#define TNX_LDS(T, addr) ((T __attribute__((address_space(3)))*)(uintptr_t)(addr))

__device__ __forceinline__ unsigned mix(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}
// two 16-bit floats with random sign and mantissa and an exponent in a band of eight binades (the spread of
// N(0,1) samples); for int8 all 32 bits are random
__device__ __forceinline__ int operand_word(unsigned seed, int dtype, int zero) {
  if (zero) return 0;
  const unsigned h = mix(seed), g = mix(seed ^ 0x9e3779b9U);
  if (dtype == TNX_I8) return (int)h;
  if (dtype == TNX_BF16) {
    const unsigned lo = (h & 0x807fU) | ((115U + ((h >> 8) & 7U)) << 7), hi = (g & 0x807fU) | ((115U + ((g >> 8) & 7U)) << 7);
    return (int)(lo | (hi << 16));
  }
  const unsigned lo = (h & 0x83ffU) | ((8U + ((h >> 10) & 7U)) << 10), hi = (g & 0x83ffU) | ((8U + ((g >> 10) & 7U)) << 10);
  return (int)(lo | (hi << 16));
}

#define TNX_MFMA(NAME, ACC, A, B) asm volatile(NAME " %0, %1, %2, %0" : "+a"(ACC) : "v"(A), "v"(B))

template <int DT, int SHAPE>
__global__ __launch_bounds__(256) void mfma_only_kernel(float* out, int iters, int zero) {
  const unsigned tid = blockIdx.x * 256 + threadIdx.x;
  i32x4 fa[8], fb[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      fa[i][e] = operand_word(tid * 64 + i * 4 + e, DT, zero);
      fb[i][e] = operand_word(tid * 64 + 32 + i * 4 + e, DT, zero);
    }
  float res = 0;
  if (SHAPE == 32) {
    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x16{};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const int j = (i & 1) ? 3 - jj : jj;
            if (DT == TNX_BF16) TNX_MFMA("v_mfma_f32_32x32x16_bf16", acc[i][j], fb[j + 4 * ks], fa[i + 4 * ks]);
            if (DT == TNX_F16) TNX_MFMA("v_mfma_f32_32x32x16_f16", acc[i][j], fb[j + 4 * ks], fa[i + 4 * ks]);
            if (DT == TNX_I8) TNX_MFMA("v_mfma_i32_32x32x32_i8", acc[i][j], fb[j + 4 * ks], fa[i + 4 * ks]);
          }
#pragma unroll
      for (int i = 0; i < 8; ++i) fa[i].x ^= (it & 1) << 3;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) res += acc[i][j][0] + acc[i][j][7];
  } else {
    f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          const int j = (i & 1) ? 7 - jj : jj;
          if (DT == TNX_BF16) TNX_MFMA("v_mfma_f32_16x16x32_bf16", acc[i][j], fb[j], fa[i]);
          if (DT == TNX_F16) TNX_MFMA("v_mfma_f32_16x16x32_f16", acc[i][j], fb[j], fa[i]);
          if (DT == TNX_I8) TNX_MFMA("v_mfma_i32_16x16x64_i8", acc[i][j], fb[j], fa[i]);
        }
#pragma unroll
      for (int i = 0; i < 8; ++i) fa[i].x ^= (it & 1) << 3;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) res += acc[i][j][0] + acc[i][j][3];
  }
  out[tid] = res;
}

template <int DT> hipError_t launch(int shape, float* out, unsigned grid, int iters, int zero, hipStream_t s) {
  if (shape == 32) hipLaunchKernelGGL((mfma_only_kernel<DT, 32>), dim3(grid), dim3(256), 0, s, out, iters, zero);
  else hipLaunchKernelGGL((mfma_only_kernel<DT, 16>), dim3(grid), dim3(256), 0, s, out, iters, zero);
  return hipGetLastError();
}

// One wave, one LDS instruction kind, per-lane byte addresses from a table: eight instructions per iteration at
// table[lane] + u * 4096 (the multiple of the bank period keeps the pattern).  Read under
// `rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_LDS`: conflict cycles per instruction.
template <int OP> __global__ __launch_bounds__(64) void lds_pattern_kernel(const uint32_t* table, int iters, int* out) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[65536];
  const uint32_t base = (uint32_t)(uintptr_t)(uint8_t __attribute__((address_space(3)))*)smem;
  for (int i = threadIdx.x; i < 16384; i += 64) ((int*)smem)[i] = i;
  __syncthreads();
  const uint32_t a = base + table[threadIdx.x];
  i32x4 acc = {0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t addr = a + u * 4096;
      if (OP == TNX_LDS_READ_B128) acc ^= *TNX_LDS(i32x4, addr);
      if (OP == TNX_LDS_WRITE_B128) *TNX_LDS(i32x4, addr) = i32x4{it, u, it, u};
      if (OP == TNX_LDS_READ_TR16_B64) {
        const i32x2 v = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(TNX_LDS(i16x4, addr)));
        acc.x ^= v.x, acc.y ^= v.y;
      }
      if (OP == TNX_LDS_READ_TR8_B64) {
        const i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(TNX_LDS(i32x2, addr));
        acc.x ^= v.x, acc.y ^= v.y;
      }
    }
    asm volatile("" ::: "memory");
  }
  out[threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

}  // namespace

extern "C" int tnx_probe_lds(int op, const uint32_t* lane_offsets, int iterations, void* scratch, size_t scratch_bytes,
                             void* stream) {
  if (op < TNX_LDS_READ_B128 || op > TNX_LDS_READ_TR8_B64 || !lane_offsets || iterations <= 0 || !scratch) return TNX_E_INVALID;
  if (scratch_bytes < 512) return TNX_E_WORKSPACE;
  for (int l = 0; l < 64; ++l)
    if (lane_offsets[l] > 32768u || (lane_offsets[l] & (op <= TNX_LDS_WRITE_B128 ? 15u : 7u))) return TNX_E_INVALID;
  hipStream_t s = (hipStream_t)stream;
  uint32_t* table = (uint32_t*)scratch;
  int* out = (int*)scratch + 64;
  if (hipMemcpyAsync(table, lane_offsets, 256, hipMemcpyHostToDevice, s) != hipSuccess) return TNX_E_HIP;
  if (op == TNX_LDS_READ_B128) hipLaunchKernelGGL((lds_pattern_kernel<TNX_LDS_READ_B128>), dim3(1), dim3(64), 0, s, table, iterations, out);
  else if (op == TNX_LDS_WRITE_B128) hipLaunchKernelGGL((lds_pattern_kernel<TNX_LDS_WRITE_B128>), dim3(1), dim3(64), 0, s, table, iterations, out);
  else if (op == TNX_LDS_READ_TR16_B64) hipLaunchKernelGGL((lds_pattern_kernel<TNX_LDS_READ_TR16_B64>), dim3(1), dim3(64), 0, s, table, iterations, out);
  else hipLaunchKernelGGL((lds_pattern_kernel<TNX_LDS_READ_TR8_B64>), dim3(1), dim3(64), 0, s, table, iterations, out);
  return hipGetLastError() == hipSuccess ? TNX_OK : TNX_E_HIP;
}

extern "C" int tnx_probe_mfma(int dtype, int mfma_rows, int zero_operands, int workgroups, int iterations, void* scratch,
                              size_t scratch_bytes, void* stream, double* ops_per_launch) {
  if ((dtype != TNX_F16 && dtype != TNX_BF16 && dtype != TNX_I8) || (mfma_rows != 16 && mfma_rows != 32) || workgroups <= 0 ||
      workgroups > 65536 || iterations <= 0 || !scratch)
    return TNX_E_INVALID;
  if (scratch_bytes < (size_t)workgroups * 256 * sizeof(float)) return TNX_E_WORKSPACE;
  // one iteration of one wave: 128 x 128 x 32 multiply-adds (x64 for int8) whatever the MFMA shape
  if (ops_per_launch) *ops_per_launch = (double)workgroups * 4 * iterations * 2.0 * 128 * 128 * (dtype == TNX_I8 ? 64 : 32);
  hipError_t err;
  if (dtype == TNX_BF16) err = launch<TNX_BF16>(mfma_rows, (float*)scratch, workgroups, iterations, zero_operands, (hipStream_t)stream);
  else if (dtype == TNX_F16) err = launch<TNX_F16>(mfma_rows, (float*)scratch, workgroups, iterations, zero_operands, (hipStream_t)stream);
  else err = launch<TNX_I8>(mfma_rows, (float*)scratch, workgroups, iterations, zero_operands, (hipStream_t)stream);
  return err == hipSuccess ? TNX_OK : TNX_E_HIP;
}
