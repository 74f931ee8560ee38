// C ABI of the conv2d forward path: argument checking, tile lookup, launch.
// Declarations and the reference interface they replace: include/tritonix_hip.h
#include <hip/hip_runtime.h>
#include <stdio.h>

#include "../../include/tritonix_hip.h"
#include "conv_tile.h"
#include "registry.h"

using namespace tnx;

extern "C" const ConvGroup* tnx_conv_groups(int* ngroups);  // generated

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

static int resolve(const tnx_conv2d_args* a, const ConvEntry** entry, ConvParams* p, unsigned* grid) {
  int32_t h_out = 0, w_out = 0;
  const int st = check_problem(a, &h_out, &w_out);
  if (st != TNX_OK) return st;
  const int64_t pixels = (int64_t)a->batch * h_out * w_out;
  int bcout = a->block_cout, bpix = a->block_pixels, bk = a->block_k;
  if (bcout == 0 && bpix == 0 && bk == 0) builtin_tile(a, pixels, &bcout, &bpix, &bk);
  if (bcout <= 0 || bpix <= 0 || bk <= 0) return TNX_E_INVALID;
  if (2ll * ((int64_t)bcout * bk + (int64_t)bk * bpix) * 2 > TNX_LDS_LIMIT_BYTES) return TNX_E_LDS;
  const ConvEntry* e = find_conv(a->dtype, bcout, bpix, bk);
  if (!e) return TNX_E_UNSUPPORTED;
  const int64_t tiles_pix = (pixels + bpix - 1) / bpix, tiles_cout = ((int64_t)a->c_out + bcout - 1) / bcout;
  if (tiles_pix * tiles_cout >= (1ll << 31)) return TNX_E_UNSUPPORTED;
  *entry = e;
  if (!p) return TNX_OK;

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
  {
    // block_k = sc * (R*S) + sh * S + sw
    const int rs = a->filter_h * a->filter_w;
    const int sc = bk / rs, sh = (bk % rs) / a->filter_w, sw = bk % a->filter_w;
    p->step_dw = sw * a->dil_w;
    p->step_dh = sh * a->dil_h;
    p->step_koff = sc * p->hw_in + p->step_dh * a->w_in + p->step_dw;
    p->lim_w = a->filter_w * a->dil_w;
    p->lim_h = a->filter_h * a->dil_h;
    p->adj_w = a->dil_h * a->w_in - p->lim_w;          // dw wraps: one filter row down
    p->adj_h = p->hw_in - p->lim_h * a->w_in;          // dh wraps: next input channel
  }
  p->tiles_cout = (int)tiles_cout;
  p->tiles_pix = (int)tiles_pix;
  p->group = a->group_pixels > 0 ? a->group_pixels : 8;
  p->bias_dtype = a->bias_dtype;
  p->w_vec_ok = gemm_k % 8 == 0 && ((uintptr_t)a->weight & 15) == 0;
  p->y_vec_ok = p->hw_out % 4 == 0 && ((uintptr_t)a->output & 7) == 0;
  p->flat = a->filter_h == 1 && a->filter_w == 1 && a->stride_h == 1 && a->stride_w == 1 && a->pad_h == 0 && a->pad_w == 0;
  *grid = (unsigned)(tiles_pix * tiles_cout);
  return TNX_OK;
}

extern "C" int tnx_conv2d_supported(const tnx_conv2d_args* a) {
  const ConvEntry* e = nullptr;
  return resolve(a, &e, nullptr, nullptr);
}

extern "C" int tnx_conv2d_default_config(tnx_conv2d_args* a) {
  int32_t h_out = 0, w_out = 0;
  const int st = check_problem(a, &h_out, &w_out);
  if (st != TNX_OK) return st;
  int bcout, bpix, bk;
  builtin_tile(a, (int64_t)a->batch * h_out * w_out, &bcout, &bpix, &bk);
  a->block_cout = bcout;
  a->block_pixels = bpix;
  a->block_k = bk;
  a->group_pixels = 8;
  return TNX_OK;
}

extern "C" int tnx_conv2d_forward(const tnx_conv2d_args* a) {
  const ConvEntry* e = nullptr;
  ConvParams p;
  unsigned grid = 0;
  const int st = resolve(a, &e, &p, &grid);
  if (st != TNX_OK) return st;
  if (!a->input || !a->weight || !a->output) return TNX_E_INVALID;
  // 16-bit elements are read and written as such
  if (((uintptr_t)a->input & 1) || ((uintptr_t)a->weight & 1) || ((uintptr_t)a->output & 1)) return TNX_E_INVALID;
  if (a->bias && ((uintptr_t)a->bias & (a->bias_dtype == TNX_F32 ? 3 : 1))) return TNX_E_INVALID;
  const hipError_t err = e->launch(p, grid, (hipStream_t)a->stream);
  if (err != hipSuccess) {
    note_hip_error((int)err);
    return TNX_E_HIP;
  }
  return TNX_OK;
}

extern "C" int tnx_conv2d_kernel_count(void) {
  int ng = 0, n = 0;
  const ConvGroup* g = tnx_conv_groups(&ng);
  for (int i = 0; i < ng; ++i) n += g[i].count;
  return n;
}

extern "C" const char* tnx_conv2d_kernel_name(int idx) {
  static thread_local char buf[64];
  int ng = 0, n = 0;
  const ConvGroup* g = tnx_conv_groups(&ng);
  for (int i = 0; i < ng; ++i)
    for (int j = 0; j < g[i].count; ++j, ++n)
      if (n == idx) {
        const ConvEntry& e = g[i].entries[j];
        snprintf(buf, sizeof buf, "%s %d %d %d", e.dtype == TNX_F16 ? "f16" : "bf16", e.block_cout, e.block_pix, e.block_k);
        return buf;
      }
  return "";
}
