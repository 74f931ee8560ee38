// Conv2d forward as an implicit GEMM on the tile engine's LDS layout and MFMA fragments (gfx950).
//
// What it computes follows tritonix/ops/conv2d/forward.py:19-165 (conv2d_forward_kernel): NCHW input,
// KCRS weight, NCHW output, GEMM_M = batch * h_out * w_out pixels, GEMM_N = c_out, GEMM_K = c_in * R * S with
// k -> (c_in, filter row, filter column), zero fill outside the image, fp32 accumulation, optional bias added
// in fp32, one rounding to the output type.
//
// How it maps here: the product is formed transposed, out[c_out, pixel] = W[c_out, k] x im2col[k, pixel].
// W is row-major with k contiguous, which is exactly the A slab of the GEMM kernel; im2col rows (one per k) are
// runs of consecutive pixels, which is the B slab (rows of k, n contiguous, read with the transposing LDS
// reads); and a row of the result is a run of consecutive pixels of one output plane, so NCHW output needs no
// transpose.  Nothing in the image is 16-byte aligned once a filter tap shifts it, so the slabs are staged
// through registers instead of the direct-to-LDS loads: the loads of slab t+1 are issued before the MFMAs of
// slab t and written to the other LDS slot after them.
#pragma once
#include "gemm_tile.h"

namespace tnx {

struct ConvParams {
  const uint8_t* x;       // [batch, c_in, h_in, w_in]
  const uint8_t* w;       // [c_out, c_in, fh, fw]  ==  [c_out, gemm_k] row-major
  const uint8_t* bias;    // [c_out] or null
  uint8_t* y;             // [batch, c_out, h_out, w_out]
  int batch, c_in, h_in, w_in, c_out, h_out, w_out, fh, fw;
  int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int gemm_k;             // c_in * fh * fw
  int pixels;             // batch * h_out * w_out
  int hw_in, hw_out;
  uint32_t x_bytes, w_bytes;   // sizes of the input and weight tensors
  int x_last_vec;         // batch * c_in * h_in * w_in - 8: last element offset a 16-byte load may start at (negative: none)
  FastDiv div_hw_out, div_w_out, div_rs, div_s;
  // one K slab further (block_k taps along (c_in, fh, fw)): what is added to a tap's (dw, dh, element offset), the limits
  // at which dw and dh wrap, and what a wrap adds to the element offset
  int step_dw, step_dh, step_koff, lim_w, lim_h, adj_w, adj_h;
  int tiles_cout, tiles_pix, group;
  int bias_dtype;
  bool w_vec_ok;          // weight rows take 16-byte loads: gemm_k % 8 == 0 and a 16-byte aligned base
  bool y_vec_ok;          // four consecutive pixels lie in one plane and take one 8-byte store: hw_out % 4 == 0, aligned base
  bool flat;              // 1x1 filter, unit strides, no padding: all pixels of one image plane are contiguous in the input
  bool out_f32;           // y is binary32: the fp32 sums (+ bias) as they are (y_vec_ok then means one 16-byte store)
};

typedef hipError_t (*conv_launch_fn)(const ConvParams& p, unsigned grid, hipStream_t stream);

struct ConvEntry {
  int dtype, block_cout, block_pix, block_k;
  int lds_bytes;
  conv_launch_fn launch;
};
struct ConvGroup {
  ConvEntry* entries;
  int count;
};

// C = TileCfg<T, block_cout, block_pix, block_k, 4 waves, 2 slots>
#ifndef TNX_CONV_OCC
#define TNX_CONV_OCC 1
#endif
template <class T, class C>
__global__ __launch_bounds__(C::THREADS, TNX_CONV_OCC) void conv2d_tile_kernel(ConvParams p) {
  constexpr int ES = C::ES, BM = C::BM, BN = C::BN, BK = C::BK;
  constexpr int MI = C::MI, TM = C::TM, TN = C::TN, THREADS = C::THREADS;
  static_assert(C::VALID && ES == 2 && C::STAGES == 2 && MI == 16, "conv2d is built for 16-bit floats, two LDS slots");
  static_assert(THREADS % C::CPR_B == 0 && (BM * C::CPR_A) % THREADS == 0 && (BK * C::CPR_B) % THREADS == 0,
                "slab chunks must divide evenly over the threads");
  typedef Mma<T, MI> MMA;
  typedef typename MMA::acc_t acc_t;
  typedef typename OutOf<T>::type O;
  constexpr int A_CH = BM * C::CPR_A / THREADS;       // 16-byte chunks of the weight slab per thread
  constexpr int B_CH = BK * C::CPR_B / THREADS;       // 16-byte chunks of the im2col slab per thread
  constexpr int B_ROWS = THREADS / C::CPR_B;          // k rows the threads cover in one sweep

  __shared__ __attribute__((aligned(1024))) uint8_t smem[C::LDS_BYTES];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(uint8_t __attribute__((address_space(3)))*)smem;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // launch order: XCD-first, then groups of `group` pixel tiles walked channel tile by channel tile
  // (tl.swizzle2d over (pixel tile, channel tile), tritonix/ops/conv2d/forward.py:50-56)
  const int ntiles = p.tiles_cout * p.tiles_pix;
  const int lg = xcd_remap(blockIdx.x, ntiles, 8);
  int pt, ct;
  swizzle2d(lg / p.tiles_cout, lg % p.tiles_cout, p.tiles_pix, p.tiles_cout, p.group, &pt, &ct);
  const int m0 = ct * BM;          // first output channel of the tile
  const int n0 = pt * BN;          // first pixel of the tile
  const int KT = (p.gemm_k + BK - 1) / BK;

  const uint16_t* x16 = (const uint16_t*)p.x;
  const uint16_t* w16 = (const uint16_t*)p.w;

  // ---- im2col columns of this thread: one 16-byte chunk column = 8 consecutive pixels -------------------
  // per pixel: element offset of (image, channel 0, h0, w0) and the packed (h0, w0), where (h0, w0) is the
  // input position of filter tap (0, 0) -- negative inside the padding.  Pixels past the end get h0 = -32768,
  // which no tap brings back into the image.
  const int b_cs = tid % C::CPR_B;
  const int b_row0 = tid / C::CPR_B;
  int col_off[8], col_hw[8];
  bool run = true;                 // the 8 pixels are consecutive in one input row (or plane, when flat): one vector load
  {
    int img0 = 0, ho0 = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int n = n0 + b_cs * 8 + e;
      int off = 0, h0 = -32768, w0 = 0;
      if (n < p.pixels) {
        const int img = (int)fd_div((uint32_t)n, p.div_hw_out);
        const int r = n - img * p.hw_out;
        const int ho = (int)fd_div((uint32_t)r, p.div_w_out);
        const int wo = r - ho * p.w_out;
        h0 = ho * p.stride_h - p.pad_h;
        w0 = wo * p.stride_w - p.pad_w;
        off = img * (p.c_in * p.hw_in) + h0 * p.w_in + w0;
        if (e == 0) { img0 = img; ho0 = ho; }
        else if (img != img0 || (!p.flat && ho != ho0)) run = false;
      } else {
        run = false;
      }
      col_off[e] = off;
      col_hw[e] = (int)(((uint32_t)h0 << 16) | ((uint32_t)w0 & 0xffffu));
    }
    if (p.stride_w != 1) run = false;
  }

  // Staging registers.  Nothing here may consume a loaded value before the MFMAs of the current slab have
  // been issued (the wave would wait for the loads first), so masks and packing are left to store_lds:
  // st_b holds either 16 raw bytes (words 0-3) with the element range [lo, hi) to keep, or eight
  // zero-extended elements that are already zero where the image ends.
  constexpr uint32_t GATHERED = 0x10000u;
  i32x4 st_a[A_CH];
  uint32_t st_b[B_CH][8], st_m[B_CH];

  // Raw-buffer windows over the input and the weights: a load whose offset lies outside the window returns
  // zero, which is how padding, ragged edges and masked-off elements are filled without a branch per element.
  constexpr uint32_t OUTSIDE = 0xffffffffu;
  const __amdgpu_buffer_rsrc_t xwin = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.x), 0, p.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wwin = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.w), 0, p.w_bytes, 0x00020000);

  // Per chunk of this thread, set up once: the weight chunk's byte offset at slab 0, and the im2col chunk's filter
  // tap (dh, dw) = (tap row * dil_h, tap column * dil_w) with its element offset c_in * plane + dh * w_in + dw.
  // load_regs is called for slabs 0, 1, 2, ... in order and moves every tap one slab (block_k taps) on after use,
  // with additions and wrap-arounds only: the integer divisions and multiplications of the k -> (c_in, fh, fw)
  // decomposition run once per thread, not once per chunk and slab (32-bit multiplies are quarter rate).
  uint32_t a_off[A_CH];
  int a_k[A_CH];
  bool a_ok[A_CH];
#pragma unroll
  for (int q = 0; q < A_CH; ++q) {
    const int P = q * THREADS + tid;
    const int row = P / C::CPR_A, cs = P % C::CPR_A;
    a_k[q] = cs * 8;
    a_ok[q] = m0 + row < p.c_out;
    a_off[q] = (uint32_t)((m0 + row) * p.gemm_k + cs * 8) * 2u;
  }
  int tap_dh[B_CH], tap_dw[B_CH];
  uint32_t tap_off[B_CH];      // unsigned: past the last k it keeps growing unused and may wrap
#pragma unroll
  for (int q = 0; q < B_CH; ++q) {
    const int gk = q * B_ROWS + b_row0;
    const int cin = (int)fd_div((uint32_t)gk, p.div_rs);
    const int r = gk - cin * (p.fh * p.fw);
    const int tap_h = (int)fd_div((uint32_t)r, p.div_s);
    const int tap_w = r - tap_h * p.fw;
    tap_dh[q] = tap_h * p.dil_h;
    tap_dw[q] = tap_w * p.dil_w;
    tap_off[q] = (uint32_t)(cin * p.hw_in + tap_dh[q] * p.w_in + tap_dw[q]);
  }

  auto load_regs = [&](int kt) __attribute__((always_inline)) {
    const int k0 = kt * BK;
    // weights
#pragma unroll
    for (int q = 0; q < A_CH; ++q) {
      const int gk = k0 + a_k[q];
      const uint32_t off = a_off[q] + (uint32_t)k0 * 2u;
      if (p.w_vec_ok) {
        st_a[q] = __builtin_amdgcn_raw_buffer_load_b128(wwin, a_ok[q] && gk < p.gemm_k ? off : OUTSIDE, 0, 0);
      } else {
        // ragged or unaligned rows (c_in * R * S not a multiple of 8): element loads; rare, and allowed to wait
        uint32_t e[8];
#pragma unroll
        for (int x = 0; x < 8; ++x)
          e[x] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(wwin, a_ok[q] && gk + x < p.gemm_k ? off + 2u * x : OUTSIDE, 0, 0);
        st_a[q] = i32x4{(int)(e[0] | (e[1] << 16)), (int)(e[2] | (e[3] << 16)), (int)(e[4] | (e[5] << 16)), (int)(e[6] | (e[7] << 16))};
      }
    }
    // im2col
#pragma unroll
    for (int q = 0; q < B_CH; ++q) {
      // this chunk's tap, then one slab further for the next call (no multiply, no divide: see the set-up below)
      const bool k_ok = k0 + q * B_ROWS + b_row0 < p.gemm_k;
      const int dh = k_ok ? tap_dh[q] : 1 << 20;      // k past the end: a tap far outside every image
      const int dw = tap_dw[q], koff = k_ok ? (int)tap_off[q] : 0;
      {
        int ndw = tap_dw[q] + p.step_dw;
        const bool wrap_w = ndw >= p.lim_w;
        ndw -= wrap_w ? p.lim_w : 0;
        int ndh = tap_dh[q] + p.step_dh + (wrap_w ? p.dil_h : 0);
        const bool wrap_h = ndh >= p.lim_h;
        ndh -= wrap_h ? p.lim_h : 0;
        tap_off[q] += (uint32_t)(p.step_koff + (wrap_w ? p.adj_w : 0) + (wrap_h ? p.adj_h : 0));
        tap_dw[q] = ndw;
        tap_dh[q] = ndh;
      }
      const int h0 = col_hw[0] >> 16, w0 = (int)(int16_t)(col_hw[0] & 0xffff);
      const int o = col_off[0] + koff;
      if (run && o >= 0 && o <= p.x_last_vec) {
        // the 8 pixels read 8 consecutive input elements, all inside the tensor; those outside the image row
        // are masked at store time (flat: every element is inside the plane)
        int lo = -(w0 + dw), hi = p.flat ? 8 : p.w_in - (w0 + dw);   // elements [lo, hi) are inside the row
        lo = lo < 0 ? 0 : lo;
        hi = hi > 8 ? 8 : hi;
        const i32x4 v = ((const Loose16*)(x16 + o))->v;
        st_b[q][0] = v.x; st_b[q][1] = v.y; st_b[q][2] = v.z; st_b[q][3] = v.w;
        st_m[q] = ((uint32_t)(h0 + dh) < (uint32_t)p.h_in && lo < hi) ? (uint32_t)lo | ((uint32_t)hi << 8) : 0u;
      } else {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          const int hin = (col_hw[x] >> 16) + dh, win = (int)(int16_t)(col_hw[x] & 0xffff) + dw;
          const bool ok = (uint32_t)hin < (uint32_t)p.h_in && (uint32_t)win < (uint32_t)p.w_in;
          st_b[q][x] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(xwin, ok ? (uint32_t)(col_off[x] + koff) * 2u : OUTSIDE, 0, 0);
        }
        st_m[q] = GATHERED;
      }
    }
  };

  auto store_lds = [&](uint32_t stage) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < A_CH; ++q) {
      const int P = q * THREADS + tid;
      const int row = P / C::CPR_A, cs = P % C::CPR_A;
      *TNX_LDS(i32x4, stage + row * C::ROWB_A + ((cs ^ C::swzA(row)) << 4)) = st_a[q];
    }
#pragma unroll
    for (int q = 0; q < B_CH; ++q) {
      const int row = q * B_ROWS + b_row0;
      i32x4 v;
      if (st_m[q] & GATHERED) {
        v = i32x4{(int)(st_b[q][0] | (st_b[q][1] << 16)), (int)(st_b[q][2] | (st_b[q][3] << 16)),
                  (int)(st_b[q][4] | (st_b[q][5] << 16)), (int)(st_b[q][6] | (st_b[q][7] << 16))};
      } else {
        const int lo = (int)(st_m[q] & 0xff), hi = (int)(st_m[q] >> 8);
        v = i32x4{(int)st_b[q][0], (int)st_b[q][1], (int)st_b[q][2], (int)st_b[q][3]};
        if (hi - lo < 8) {
          // element e stays when lo <= e < hi: two packed 16-bit subtractions whose sign bits, spread by an arithmetic
          // shift, are the two halves of the test
          typedef short s16x2 __attribute__((ext_vector_type(2)));
          const s16x2 lo2 = {(short)lo, (short)lo}, hi2 = {(short)hi, (short)hi};
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const s16x2 e = {(short)(2 * d), (short)(2 * d + 1)};
            const s16x2 below_lo = (e - lo2) >> 15, below_hi = (e - hi2) >> 15;
            v[d] &= __builtin_bit_cast(int, below_hi & ~below_lo);
          }
        }
      }
      *TNX_LDS(i32x4, stage + C::A_BYTES + row * C::ROWB_B + ((b_cs ^ C::swzB(row)) << 4)) = v;
    }
  };

  // ---- fragment addressing: the same slab layout as the GEMM kernel ----------------------------------------
  const int wy = wave / C::WGN, wx = wave % C::WGN;
  const int a_row = wy * C::WTM + (lane % MI);
  const int a_kg = lane / MI;
  const int a_sw = C::swzA(a_row);
  const int blk = lane >> 4, li = lane & 15;
  const int b_sub = li >> 2;
  const int b_colb0 = (wx * C::WTN) * ES + 8 * (li & 3);
  const int b_krow = 8 * blk + b_sub;
  const int b_sw = C::swzB(b_krow);

  acc_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{};

  auto compute = [&](uint32_t stage) __attribute__((always_inline)) {
    const uint32_t sa = stage, sb = stage + C::A_BYTES;
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ++ks) {
      i32x4 fa[TM];
      i32x2 fb[TN][2];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[i] = *TNX_LDS(i32x4, sa + (a_row + i * MI) * C::ROWB_A + (((ks * (C::KB / 16) + a_kg) ^ a_sw) << 4));
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int colb = b_colb0 + j * MI * ES;
#pragma unroll
        for (int h = 0; h < 2; ++h)
          fb[j][h] = lds_read_tr<ES>(sb + (b_krow + ks * C::MMA_K + h * 4) * C::ROWB_B + (((colb >> 4) ^ b_sw) << 4) + (colb & 15));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const i32x4 b4 = {fb[j][0].x, fb[j][0].y, fb[j][1].x, fb[j][1].y};
          acc[i][j] = MMA::run(b4, fa[i], acc[i][j]);
        }
    }
  };

  // ---- K loop: registers take slab t+1 while the MFMAs of slab t run ---------------------------------------
  load_regs(0);
  store_lds(lds0);
  __syncthreads();
  for (int t = 0; t < KT; ++t) {
    const uint32_t cur = lds0 + (uint32_t)(t & 1) * C::STAGE_BYTES, nxt = lds0 + (uint32_t)((t + 1) & 1) * C::STAGE_BYTES;
    if (t + 1 < KT) load_regs(t + 1);
    __builtin_amdgcn_sched_barrier(0);
    compute(cur);
    __builtin_amdgcn_sched_barrier(0);
    // the other slot was last read one trip ago, before that trip's barrier
    if (t + 1 < KT) store_lds(nxt);
    __syncthreads();
  }

  // ---- epilogue: lane l holds, per MFMA tile, row l % 16 (an output channel) and four consecutive pixels ----
  uint16_t* y16 = (uint16_t*)p.y;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = m0 + wy * C::WTM + i * MI + (lane % MI);
    if (row >= p.c_out) continue;
    const float bv = p.bias ? bias_value(p.bias, row, p.bias_dtype) : 0.0f;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wx * C::WTN + j * MI + (lane / MI) * 4;
      if (n >= p.pixels) continue;
      if (p.out_f32) {
        float* y32 = (float*)p.y;
        if (p.y_vec_ok) {
          const int img = (int)fd_div((uint32_t)n, p.div_hw_out);
          const int r0 = n - img * p.hw_out;
          const f32x4 v = {acc[i][j][0] + bv, acc[i][j][1] + bv, acc[i][j][2] + bv, acc[i][j][3] + bv};
          __builtin_nontemporal_store(v, (f32x4*)(y32 + ((int64_t)img * p.c_out + row) * p.hw_out + r0));
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if (n + r >= p.pixels) break;
            const int img = (int)fd_div((uint32_t)(n + r), p.div_hw_out);
            const int r0 = n + r - img * p.hw_out;
            y32[((int64_t)img * p.c_out + row) * p.hw_out + r0] = acc[i][j][r] + bv;
          }
        }
        continue;
      }
      typename O::raw out[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) out[r] = O::cvt(acc[i][j][r] + bv);
      if (p.y_vec_ok) {
        // pixels n..n+3 exist together and share a plane
        const int img = (int)fd_div((uint32_t)n, p.div_hw_out);
        const int r0 = n - img * p.hw_out;
        i32x2 v = {(int)(out[0] | ((uint32_t)out[1] << 16)), (int)(out[2] | ((uint32_t)out[3] << 16))};
        __builtin_nontemporal_store(v, (i32x2*)(y16 + ((int64_t)img * p.c_out + row) * p.hw_out + r0));   // written once, never read here
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (n + r >= p.pixels) break;
          const int img = (int)fd_div((uint32_t)(n + r), p.div_hw_out);
          const int r0 = n + r - img * p.hw_out;
          y16[((int64_t)img * p.c_out + row) * p.hw_out + r0] = out[r];
        }
      }
    }
  }
}

template <class T, class C>
hipError_t launch_conv(const ConvParams& p, unsigned grid, hipStream_t stream) {
  hipLaunchKernelGGL((conv2d_tile_kernel<T, C>), dim3(grid), dim3(C::THREADS), 0, stream, p);
  return hipGetLastError();
}

#define TNX_CONV_ENTRY(TAG, BCOUT, BPIX, BK) \
  {TAG::ID, BCOUT, BPIX, BK, TileCfg<TAG, BCOUT, BPIX, BK, 4, 2>::LDS_BYTES, &launch_conv<TAG, TileCfg<TAG, BCOUT, BPIX, BK, 4, 2>>}

}  // namespace tnx
