// C ABI of the conv2d forward path: argument checking, tile lookup, launch.
// Declarations and the reference interface they replace: include/tritonix_hip.h
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include "../../include/tritonix_hip.h"
#include "conv_tile.h"
#include "registry.h"

using namespace tnx;

extern "C" const ConvGroup* tnx_conv_groups(int* ngroups);      // generated
extern "C" const KernelGroup* tnx_kernel_groups(int* ngroups);  // generated

// The GEMM kernel's conv2d variant for this tile (three ring slots), or null.  Eight waves are preferred (and the
// only ones built): the loader's address arithmetic and the fix-up are vector instructions in the MFMA stream, and
// with two waves per SIMD one wave's arithmetic runs under the other's MFMAs (measured on 3x3 layers, batch 32,
// against four-wave builds: 256x128 524 -> 620 TFLOP/s at 56x56 / 256 channels, 128x128 248 -> 292 at 28x28 / 128
// and 351 -> 420 at 14x14 / 512).
static const KernelEntry* find_dma(int dtype, int bcout, int bpix, int bk) {
  int ng = 0;
  const KernelGroup* g = tnx_kernel_groups(&ng);
  const KernelEntry* four = nullptr;
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < g[i].count; ++j) {
      const KernelEntry& e = g[i].entries[j];
      if (e.dtype != dtype || e.bm != bcout || e.bn != bpix || e.bk != bk || e.stages != 3 || !e.conv) continue;
      if (e.nw == 8) return &e;
      if (e.nw == 4) four = &e;
    }
  return four;
}

static const ConvEntry* find_conv(int dtype, int bcout, int bpix, int bk) {
  int ng = 0;
  const ConvGroup* g = tnx_conv_groups(&ng);
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < g[i].count; ++j) {
      const ConvEntry& e = g[i].entries[j];
      if (e.dtype == dtype && e.block_cout == bcout && e.block_pix == bpix && e.block_k == bk) return &e;
    }
  return nullptr;
}

extern "C" void tnx_conv2d_output_size(const tnx_conv2d_args* a, int32_t* h_out, int32_t* w_out) {
  // floor division as Python's // does it (tritonix/ops/conv2d/forward.py:226-227)
  auto fdiv = [](int64_t x, int64_t d) { return x >= 0 ? x / d : -((-x + d - 1) / d); };
  int64_t h = 0, w = 0;
  if (a && a->stride_h > 0 && a->stride_w > 0) {
    h = fdiv((int64_t)a->h_in + 2 * (int64_t)a->pad_h - (int64_t)a->dil_h * (a->filter_h - 1) - 1, a->stride_h) + 1;
    w = fdiv((int64_t)a->w_in + 2 * (int64_t)a->pad_w - (int64_t)a->dil_w * (a->filter_w - 1) - 1, a->stride_w) + 1;
  }
  if (h_out) *h_out = (int32_t)h;
  if (w_out) *w_out = (int32_t)w;
}

// Measured on ResNet-style layers (3x3 / 1x1 / strided, 64-512 channels, batch 32): 64 pixels per tile is the
// fastest width everywhere -- the im2col loader's address arithmetic grows with the pixel width of the tile, the
// weight slab it shares the LDS with is reused from L2 -- and a 128-channel tile beats 64 whenever the layer has
// that many channels.
static void builtin_tile(const tnx_conv2d_args* a, int64_t pixels, int* bcout, int* bpix, int* bk) {
  (void)pixels;
  const int64_t gemm_k = (int64_t)a->c_in * a->filter_h * a->filter_w;
  *bcout = a->c_out > 64 ? 128 : 64;
  *bpix = 64;
  *bk = gemm_k > 32 ? 64 : 32;
}

// The image the direct-to-LDS kernel is given.  A 1x1 filter with unit strides and no padding reads whole planes
// in order, so the plane is handed over as one row of h*w pixels: the pixel index space then pads h*w, not every
// row, to a multiple of 8 (14x14: 200 columns per image instead of 224).  Only while h*w fits the kernel's 16-bit
// pixel coordinates.
struct DmaImage {
  int h_in, w_in, h_out, w_out, wp;
};
static DmaImage dma_image(const tnx_conv2d_args* a, int h_out, int w_out) {
  DmaImage g = {a->h_in, a->w_in, h_out, w_out, 0};
  if (a->filter_h == 1 && a->filter_w == 1 && a->stride_h == 1 && a->stride_w == 1 && a->pad_h == 0 && a->pad_w == 0 &&
      (int64_t)a->h_in * a->w_in <= 16384) {
    g.h_in = g.h_out = 1;
    g.w_in = g.w_out = a->h_in * a->w_in;
  }
  g.wp = (g.w_out + 7) / 8 * 8;
  return g;
}
static int64_t dma_cols(const tnx_conv2d_args* a, int h_out, int w_out) {
  const DmaImage g = dma_image(a, h_out, w_out);
  return (int64_t)a->batch * g.h_out * g.wp;
}

// Direct-to-LDS kernel: 256 channels x 128 pixels when that still leaves every CU two tiles, else 128 x 128.
// Measured on 3x3 layers (batch 32, eight-wave builds): 256x128 620 against 476 TFLOP/s for 128x128 at 56x56 / 256
// channels, 128x128 ahead of it at 28x28 / 128 channels (292 : 228) and 14x14 / 512 channels (420 : 337), and both
// well ahead of the register-staged kernel (392, 162, 165) down to a few dozen tiles.
static bool builtin_dma_tile(const tnx_conv2d_args* a, int h_out, int w_out, int* bcout, int* bpix, int* bk) {
  const int64_t cols = dma_cols(a, h_out, w_out);
  const int64_t t256 = ((cols + 127) / 128) * (((int64_t)a->c_out + 255) / 256);
  const int64_t t128 = ((cols + 127) / 128) * (((int64_t)a->c_out + 127) / 128);
  *bpix = 128;
  *bk = 64;
  if (a->c_out > 128 && t256 >= 512 && find_dma(a->dtype, 256, 128, 64)) {
    *bcout = 256;
    return true;
  }
  if (a->c_out > 64 && t128 >= 32 && find_dma(a->dtype, 128, 128, 64)) {
    *bcout = 128;
    return true;
  }
  return false;
}

// `rows` taps further along k = (c_in, fh, fw): rows = sc * (R*S) + sh * S + sw
static void tap_step(const tnx_conv2d_args* a, int rows, int hw_in, int* step_dw, int* step_dh, int* step_koff, int* lim_w,
                     int* lim_h, int* adj_w, int* adj_h) {
  const int rs = a->filter_h * a->filter_w;
  const int sc = rows / rs, sh = (rows % rs) / a->filter_w, sw = rows % a->filter_w;
  *step_dw = sw * a->dil_w;
  *step_dh = sh * a->dil_h;
  // (unsigned: for planes so large that `rows` channels further leaves the tensor the sum may wrap; such taps are
  // past the last k and never used)
  *step_koff = (int)((uint32_t)sc * (uint32_t)hw_in + (uint32_t)(*step_dh * a->w_in + *step_dw));
  *lim_w = a->filter_w * a->dil_w;
  *lim_h = a->filter_h * a->dil_h;
  *adj_w = a->dil_h * a->w_in - *lim_w;          // dw wraps: one filter row down
  *adj_h = hw_in - *lim_h * a->w_in;             // dh wraps: next input channel
}

// everything about the problem except the tile
static int check_problem(const tnx_conv2d_args* a, int32_t* h_out, int32_t* w_out) {
  if (!a) return TNX_E_INVALID;
  if (a->batch <= 0 || a->c_in <= 0 || a->h_in <= 0 || a->w_in <= 0 || a->c_out <= 0 || a->filter_h <= 0 ||
      a->filter_w <= 0 || a->stride_h <= 0 || a->stride_w <= 0 || a->pad_h < 0 || a->pad_w < 0 || a->dil_h <= 0 ||
      a->dil_w <= 0 || a->block_pixels < 0 || a->block_cout < 0 || a->block_k < 0 || a->group_pixels < 0)
    return TNX_E_INVALID;
  if (a->dtype == TNX_F32) return TNX_E_UNSUPPORTED;
  if (a->dtype != TNX_F16 && a->dtype != TNX_BF16) return TNX_E_INVALID;
  if (a->bias && a->bias_dtype != TNX_F16 && a->bias_dtype != TNX_BF16 && a->bias_dtype != TNX_F32) return TNX_E_INVALID;
  tnx_conv2d_output_size(a, h_out, w_out);
  if (*h_out <= 0 || *w_out <= 0) return TNX_E_INVALID;
  const int64_t lim = (1ll << 31) - 4096;
  const int64_t pixels = (int64_t)a->batch * *h_out * *w_out;
  const int64_t x_elems = (int64_t)a->batch * a->c_in * a->h_in * a->w_in;
  const int64_t w_elems = (int64_t)a->c_out * a->c_in * a->filter_h * a->filter_w;
  if (pixels >= lim || x_elems >= lim || w_elems >= lim) return TNX_E_UNSUPPORTED;
  if (a->h_in > 16384 || a->w_in > 16384 || a->pad_h > 16384 || a->pad_w > 16384 ||
      (int64_t)(a->filter_h - 1) * a->dil_h > 16384 || (int64_t)(a->filter_w - 1) * a->dil_w > 16384)
    return TNX_E_UNSUPPORTED;
  return TNX_OK;
}

// what the direct-to-LDS kernel needs of the problem (not of the tile)
static bool dma_problem_ok(const tnx_conv2d_args* a, int h_out, int w_out, bool inspect_ptrs) {
  const int64_t gemm_k = (int64_t)a->c_in * a->filter_h * a->filter_w;
  if (a->stride_w != 1 || gemm_k % 64 != 0) return false;
  if (dma_cols(a, h_out, w_out) >= (1ll << 31) - 4096) return false;
  if (inspect_ptrs && ((uintptr_t)a->weight & 15)) return false;
  // per-lane DMA offsets of the weight slab are 32-bit
  if (256 * gemm_k * 2 >= (1ll << 32)) return false;
  return true;
}

struct Resolved {
  const ConvEntry* reg;      // register-staged kernel, or
  const KernelEntry* dma;    // the GEMM kernel's conv2d variant, or
  bool gemm;                 // the plain GEMM kernel, one problem per image (1x1 filters, unit stride, no padding)
  int gemm_warps, gemm_stages;
  int bcout, bpix, bk;
  int h_out, w_out;
};

// A 1x1 filter with unit stride and no padding: out[n] = W[c_out, c_in] x X[n][c_in, h*w] + bias, image by image.
static bool gemm_problem_ok(const tnx_conv2d_args* a) {
  return a->filter_h == 1 && a->filter_w == 1 && a->stride_h == 1 && a->stride_w == 1 && a->pad_h == 0 && a->pad_w == 0;
}

// Built-in tile for that GEMM: 128 x 128, narrowed to 64 channels or 64 pixels where the layer is that small or the
// grid would leave CUs idle (measured on the 1x1 layers of a ResNet-50 at batch 8, 32 and 128).
static bool builtin_gemm_tile(const tnx_conv2d_args* a, int* bcout, int* bpix, int* bk, int* nw, int* st) {
  const int64_t hw = (int64_t)a->h_in * a->w_in;
  int bm = a->c_out <= 64 ? 64 : 128, bn = hw <= 64 ? 64 : 128;
  auto tiles = [&](int m, int n) { return (((int64_t)a->c_out + m - 1) / m) * ((hw + n - 1) / n) * a->batch; };
  if (tiles(bm, bn) < 256 && bm > 64) bm = 64;
  if (tiles(bm, bn) < 256 && bn > 64) bn = 64;
  *bcout = bm; *bpix = bn; *bk = 64;
  return gemm_tile_for(a->dtype, bm, bn, 64, nw, st);
}

static void fill_gemm(const tnx_conv2d_args* a, const Resolved& r, tnx_gemm_args* g, GemmBatch* x) {
  const int64_t hw = (int64_t)a->h_in * a->w_in;
  *g = tnx_gemm_args{};
  g->a = a->weight; g->b = a->input; g->c = a->output;
  g->m = a->c_out; g->n = hw; g->k = a->c_in;
  g->stride_am = a->c_in; g->stride_ak = 1;
  g->stride_bk = hw; g->stride_bn = 1;
  g->stride_cm = hw; g->stride_cn = 1;
  g->in_dtype = a->dtype; g->out_dtype = a->out_f32 ? TNX_F32 : a->dtype;
  g->block_m = r.bcout; g->block_n = r.bpix; g->block_k = r.bk;
  g->group_m = 8; g->split_k = 1;
  g->num_stages = r.gemm_stages; g->num_warps = r.gemm_warps;
  g->epilogue = TNX_EPI_NONE;
  g->stream = a->stream;
  x->batch = a->batch;
  x->b_batch_bytes = (int64_t)a->c_in * hw * 2;
  x->c_batch_bytes = (int64_t)a->c_out * hw * (a->out_f32 ? 4 : 2);
  x->bias = a->bias;
  x->bias_dtype = a->bias_dtype;
}

static int resolve(const tnx_conv2d_args* a, Resolved* r, bool inspect_ptrs) {
  int32_t h_out = 0, w_out = 0;
  const int st = check_problem(a, &h_out, &w_out);
  if (st != TNX_OK) return st;
  if (a->loader < TNX_CONV_LOADER_AUTO || a->loader > TNX_CONV_LOADER_GEMM) return TNX_E_INVALID;
  const int64_t pixels = (int64_t)a->batch * h_out * w_out;
  const bool dma_ok = dma_problem_ok(a, h_out, w_out, inspect_ptrs);
  int bcout = a->block_cout, bpix = a->block_pixels, bk = a->block_k;
  const bool builtin = bcout == 0 && bpix == 0 && bk == 0;
  *r = Resolved{};
  r->h_out = h_out; r->w_out = w_out;
  if (a->loader == TNX_CONV_LOADER_GEMM && !gemm_problem_ok(a)) return TNX_E_UNSUPPORTED;
  // "auto" takes the GEMM route with the built-in tile (a caller's tile names a conv2d kernel) on every layer that is
  // such a GEMM: measured on the 1x1 layers of a ResNet-50 at batch 8, 32 and 128 it is level with or ahead of the
  // conv2d kernels on 34 of 36 (1.0x to 5.4x; 0.90x and 0.93x on 14x14 planes at batch 128, where it pads every image
  // to whole pixel tiles and the conv2d kernel packs the pixels of all images).
  const bool try_gemm = a->loader == TNX_CONV_LOADER_GEMM || (a->loader == TNX_CONV_LOADER_AUTO && builtin && gemm_problem_ok(a));
  if (try_gemm) {
    int nw = 0, st2 = 0;
    bool found = false;
    if (builtin) found = builtin_gemm_tile(a, &bcout, &bpix, &bk, &nw, &st2);
    else if (bcout > 0 && bpix > 0 && bk > 0) found = gemm_tile_for(a->dtype, bcout, bpix, bk, &nw, &st2);
    if (found) {
      r->gemm = true; r->gemm_warps = nw; r->gemm_stages = st2;
      r->bcout = bcout; r->bpix = bpix; r->bk = bk;
      tnx_gemm_args g;
      GemmBatch x;
      fill_gemm(a, *r, &g, &x);
      if (!inspect_ptrs) { g.a = nullptr; g.b = nullptr; g.c = nullptr; }
      const int sg = tnx_gemm_supported(&g);
      if (sg == TNX_OK && ((int64_t)((a->c_out + bcout - 1) / bcout) * (((int64_t)a->h_in * a->w_in + bpix - 1) / bpix) * a->batch < (1ll << 31)))
        return TNX_OK;
      if (a->loader == TNX_CONV_LOADER_GEMM) return sg == TNX_OK ? TNX_E_UNSUPPORTED : sg;
      r->gemm = false;
    } else if (a->loader == TNX_CONV_LOADER_GEMM) {
      return TNX_E_UNSUPPORTED;
    }
    bcout = a->block_cout; bpix = a->block_pixels; bk = a->block_k;
  }
  bool want_dma = a->loader == TNX_CONV_LOADER_DMA;
  if (builtin) {
    if (a->loader != TNX_CONV_LOADER_REGISTERS && dma_ok && builtin_dma_tile(a, h_out, w_out, &bcout, &bpix, &bk)) want_dma = true;
    else if (want_dma) return TNX_E_UNSUPPORTED;
    else builtin_tile(a, pixels, &bcout, &bpix, &bk);
  }
  if (bcout <= 0 || bpix <= 0 || bk <= 0) return TNX_E_INVALID;
  if (2ll * ((int64_t)bcout * bk + (int64_t)bk * bpix) * 2 > TNX_LDS_LIMIT_BYTES) return TNX_E_LDS;   // two slots: the smaller of the two kernels
  const ConvEntry* reg = find_conv(a->dtype, bcout, bpix, bk);
  const KernelEntry* dma = find_dma(a->dtype, bcout, bpix, bk);
  if (!builtin && a->loader == TNX_CONV_LOADER_AUTO) want_dma = dma && dma_ok;
  if (want_dma && !(dma && dma_ok)) {
    if (a->loader == TNX_CONV_LOADER_DMA) return TNX_E_UNSUPPORTED;
    want_dma = false;
  }
  if (!want_dma && !reg) return TNX_E_UNSUPPORTED;
  const int64_t cols = want_dma ? dma_cols(a, h_out, w_out) : pixels;
  if (((cols + bpix - 1) / bpix) * (((int64_t)a->c_out + bcout - 1) / bcout) >= (1ll << 31)) return TNX_E_UNSUPPORTED;
  r->reg = want_dma ? nullptr : reg;
  r->dma = want_dma ? dma : nullptr;
  r->bcout = bcout; r->bpix = bpix; r->bk = bk;
  r->h_out = h_out; r->w_out = w_out;
  return TNX_OK;
}

static void fill_registers(const tnx_conv2d_args* a, const Resolved& r, ConvParams* p, unsigned* grid) {
  const int h_out = r.h_out, w_out = r.w_out, bk = r.bk;
  const int64_t pixels = (int64_t)a->batch * h_out * w_out;
  const int64_t tiles_pix = (pixels + r.bpix - 1) / r.bpix, tiles_cout = ((int64_t)a->c_out + r.bcout - 1) / r.bcout;
  const int64_t gemm_k = (int64_t)a->c_in * a->filter_h * a->filter_w;
  const int64_t x_elems = (int64_t)a->batch * a->c_in * a->h_in * a->w_in;
  p->x = (const uint8_t*)a->input;
  p->w = (const uint8_t*)a->weight;
  p->bias = (const uint8_t*)a->bias;
  p->y = (uint8_t*)a->output;
  p->batch = a->batch; p->c_in = a->c_in; p->h_in = a->h_in; p->w_in = a->w_in;
  p->c_out = a->c_out; p->h_out = h_out; p->w_out = w_out; p->fh = a->filter_h; p->fw = a->filter_w;
  p->stride_h = a->stride_h; p->stride_w = a->stride_w; p->pad_h = a->pad_h; p->pad_w = a->pad_w;
  p->dil_h = a->dil_h; p->dil_w = a->dil_w;
  p->gemm_k = (int)gemm_k;
  p->pixels = (int)pixels;
  p->hw_in = a->h_in * a->w_in;
  p->hw_out = h_out * w_out;
  p->x_last_vec = (int)(x_elems - 8);
  p->x_bytes = (uint32_t)(x_elems * 2);
  p->w_bytes = (uint32_t)((int64_t)a->c_out * gemm_k * 2);
  p->div_hw_out = make_fastdiv((uint32_t)p->hw_out);
  p->div_w_out = make_fastdiv((uint32_t)w_out);
  p->div_rs = make_fastdiv((uint32_t)(a->filter_h * a->filter_w));
  p->div_s = make_fastdiv((uint32_t)a->filter_w);
  tap_step(a, bk, p->hw_in, &p->step_dw, &p->step_dh, &p->step_koff, &p->lim_w, &p->lim_h, &p->adj_w, &p->adj_h);
  p->tiles_cout = (int)tiles_cout;
  p->tiles_pix = (int)tiles_pix;
  p->group = a->group_pixels > 0 ? a->group_pixels : 8;
  p->bias_dtype = a->bias_dtype;
  p->w_vec_ok = gemm_k % 8 == 0 && ((uintptr_t)a->weight & 15) == 0;
  p->out_f32 = a->out_f32 != 0;
  p->y_vec_ok = p->hw_out % 4 == 0 && ((uintptr_t)a->output & (p->out_f32 ? 15 : 7)) == 0;
  p->flat = a->filter_h == 1 && a->filter_w == 1 && a->stride_h == 1 && a->stride_w == 1 && a->pad_h == 0 && a->pad_w == 0;
  *grid = (unsigned)(tiles_pix * tiles_cout);
}

// GemmParams of the GEMM kernel's conv2d variant: m = c_out, n = padded pixel index, k = c_in * R * S
static void fill_dma(const tnx_conv2d_args* a, const Resolved& r, GemmParams* p, unsigned* grid) {
  const DmaImage im = dma_image(a, r.h_out, r.w_out);
  const int h_out = im.h_out, w_out = im.w_out, wp = im.wp;
  const int64_t gemm_k = (int64_t)a->c_in * a->filter_h * a->filter_w;
  const int64_t n_total = (int64_t)a->batch * h_out * wp;
  memset(p, 0, sizeof *p);
  p->a = (const uint8_t*)a->weight;
  p->b = (const uint8_t*)a->input;
  p->c = (uint8_t*)a->output;
  p->m = a->c_out; p->n = n_total; p->k = gemm_k;
  p->sam = gemm_k; p->sak = 1;
  p->tiles_m = (int)(((int64_t)a->c_out + r.bcout - 1) / r.bcout);
  p->tiles_n = (int)((n_total + r.bpix - 1) / r.bpix);
  p->group_m = 8;            // with one or two channel tiles: the channel tiles of one pixel tile run side by side
  p->split_k = 1;
  p->ktiles_per_split = (int)(gemm_k / r.bk);
  p->out_dtype = a->out_f32 ? TNX_F32 : a->dtype;
  ConvGeom& g = p->cv;
  g.h_in = im.h_in; g.w_in = im.w_in; g.c_out = a->c_out; g.h_out = h_out; g.w_out = w_out; g.wp = wp;
  g.stride_h = a->stride_h; g.pad_h = a->pad_h; g.pad_w = a->pad_w;
  g.hw_in = a->h_in * a->w_in;
  g.chw_in = a->c_in * g.hw_in;
  g.n_total = (int)n_total;
  g.x_bytes = (uint32_t)((int64_t)a->batch * g.chw_in * 2);
  g.div_hwp = make_fastdiv((uint32_t)(h_out * wp));
  g.div_wp = make_fastdiv((uint32_t)wp);
  g.rs = a->filter_h * a->filter_w;
  g.fw = a->filter_w;
  g.div_rs = make_fastdiv((uint32_t)g.rs);
  g.div_s = make_fastdiv((uint32_t)g.fw);
  g.dil_h = a->dil_h; g.dil_w = a->dil_w;
  // the taps are tabulated slab by slab: one step is block_k rows
  tap_step(a, r.bk, g.hw_in, &g.step_dw, &g.step_dh, &g.step_koff, &g.lim_w, &g.lim_h, &g.adj_w, &g.adj_h);
  g.bias = (const uint8_t*)a->bias;
  g.bias_dtype = a->bias_dtype;
  *grid = (unsigned)((int64_t)p->tiles_m * p->tiles_n);
}

extern "C" int tnx_conv2d_supported(const tnx_conv2d_args* a) {
  Resolved r;
  return resolve(a, &r, false);
}

extern "C" int tnx_conv2d_default_config(tnx_conv2d_args* a) {
  if (!a) return TNX_E_INVALID;
  tnx_conv2d_args tmp = *a;
  tmp.block_cout = tmp.block_pixels = tmp.block_k = 0;
  Resolved r;
  const int st = resolve(&tmp, &r, a->weight != nullptr);     // a weight pointer, when given, is checked for alignment
  if (st != TNX_OK) return st;
  a->block_cout = r.bcout;
  a->block_pixels = r.bpix;
  a->block_k = r.bk;
  a->group_pixels = 8;
  a->loader = r.gemm ? TNX_CONV_LOADER_GEMM : r.dma ? TNX_CONV_LOADER_DMA : TNX_CONV_LOADER_REGISTERS;
  return TNX_OK;
}

extern "C" int tnx_conv2d_forward(const tnx_conv2d_args* a) {
  Resolved r;
  const int st = resolve(a, &r, true);
  if (st != TNX_OK) return st;
  if (!a->input || !a->weight || !a->output) return TNX_E_INVALID;
  // 16-bit elements are read and written as such
  if (((uintptr_t)a->input & 1) || ((uintptr_t)a->weight & 1) || ((uintptr_t)a->output & (a->out_f32 ? 3 : 1))) return TNX_E_INVALID;
  if (a->bias && ((uintptr_t)a->bias & (a->bias_dtype == TNX_F32 ? 3 : 1))) return TNX_E_INVALID;
  unsigned grid = 0;
  hipError_t err;
  if (r.gemm) {
    tnx_gemm_args g;
    GemmBatch x;
    fill_gemm(a, r, &g, &x);
    return gemm_launch(&g, &x);
  }
  if (r.dma) {
    GemmParams p;
    fill_dma(a, r, &p, &grid);
    err = r.dma->conv(p, grid, (hipStream_t)a->stream);
  } else {
    ConvParams p;
    fill_registers(a, r, &p, &grid);
    err = r.reg->launch(p, grid, (hipStream_t)a->stream);
  }
  if (err != hipSuccess) {
    note_hip_error((int)err);
    return TNX_E_HIP;
  }
  return TNX_OK;
}

// register-staged tiles first, then the GEMM kernel's conv2d variants
template <class F> static void each_conv_kernel(F f) {
  int ng = 0;
  const ConvGroup* g = tnx_conv_groups(&ng);
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < g[i].count; ++j) f(g[i].entries[j].dtype, g[i].entries[j].block_cout, g[i].entries[j].block_pix, g[i].entries[j].block_k, false);
  const KernelGroup* k = tnx_kernel_groups(&ng);
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < k[i].count; ++j)
      if (k[i].entries[j].conv && find_dma(k[i].entries[j].dtype, k[i].entries[j].bm, k[i].entries[j].bn, k[i].entries[j].bk) == &k[i].entries[j])
        f(k[i].entries[j].dtype, k[i].entries[j].bm, k[i].entries[j].bn, k[i].entries[j].bk, true);
}

extern "C" int tnx_conv2d_kernel_count(void) {
  int n = 0;
  each_conv_kernel([&](int, int, int, int, bool) { ++n; });
  return n;
}

extern "C" const char* tnx_conv2d_kernel_name(int idx) {
  static thread_local char buf[64];
  int n = 0;
  buf[0] = 0;
  each_conv_kernel([&](int dtype, int bc, int bp, int bk, bool dma) {
    if (n++ == idx) snprintf(buf, sizeof buf, "%s %d %d %d %s", dtype == TNX_F16 ? "f16" : "bf16", bc, bp, bk, dma ? "dma" : "registers");
  });
  return buf;
}
