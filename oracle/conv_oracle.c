/*
 * CPU restatement of the reference's conv2d forward (implicit GEMM).  TEST
 * INFRASTRUCTURE ONLY: tests/, __graft_entry__.smoke() and the cpu_baseline leg
 * of bench.py may link or call this; the product (tritonix_amd/) never does.
 *
 *   oracle_conv2d_output_size  H_OUT / W_OUT, tritonix/ops/conv2d/forward.py:226-227
 *   oracle_conv2d_f32          conv2d_forward_kernel, tritonix/ops/conv2d/forward.py:19-165,
 *                              program by program: tile (pid_m over GEMM_M = N*H_OUT*W_OUT,
 *                              pid_n over GEMM_N = C_OUT), K loop over GEMM_K = C_IN*R*S in
 *                              BLOCK_SIZE_K slabs; gemm_m -> (batch, h_out, w_out) :87-90,
 *                              gemm_k -> (c_in, fh, fw) :105-108, input position and its mask
 *                              :110-127, weight offset :131-136, fp32 accumulation :147, bias in
 *                              fp32 :150-155, NCHW store :157-165
 *
 * Inputs are fp32 arrays that already hold the bf16/fp16-rounded values, so
 * the only rounding the caller adds is the final one to the output dtype.
 * Pinned in tests/test_conv2d_oracle.py against torch.nn.functional.conv2d in
 * float64 (a library routine) over asymmetric strides / paddings / dilations,
 * and against closed forms (1x1 = a matrix product, a one-hot filter = a
 * shifted copy, an all-ones filter = box sums from a summed-area table).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int64_t floordiv(int64_t a, int64_t b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

void oracle_conv2d_output_size(int h_in, int w_in, int fh, int fw, int stride_h, int stride_w, int pad_h, int pad_w,
                               int dil_h, int dil_w, int* h_out, int* w_out) {
  *h_out = (int)(floordiv((int64_t)h_in + 2 * pad_h - (int64_t)dil_h * (fh - 1) - 1, stride_h) + 1);
  *w_out = (int)(floordiv((int64_t)w_in + 2 * pad_w - (int64_t)dil_w * (fw - 1) - 1, stride_w) + 1);
}

/* y[batch, c_out, h_out, w_out] (fp32, before the final rounding).  bias may be NULL.  Returns 0, or -1 when the
 * output would be empty. */
int oracle_conv2d_f32(const float* x, const float* w, const float* bias, float* y, int batch, int c_in, int h_in,
                      int w_in, int c_out, int fh, int fw, int stride_h, int stride_w, int pad_h, int pad_w, int dil_h,
                      int dil_w, int block_m, int block_n, int block_k) {
  int h_out, w_out;
  oracle_conv2d_output_size(h_in, w_in, fh, fw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &h_out, &w_out);
  if (h_out <= 0 || w_out <= 0) return -1;
  const int64_t gemm_m = (int64_t)batch * h_out * w_out, gemm_n = c_out, gemm_k = (int64_t)c_in * fh * fw;
  const int64_t grid_m = (gemm_m + block_m - 1) / block_m, grid_n = (gemm_n + block_n - 1) / block_n;
  float* acc = (float*)malloc(sizeof(float) * block_m * block_n);
  if (!acc) return -2;
  for (int64_t pid_m = 0; pid_m < grid_m; ++pid_m)
    for (int64_t pid_n = 0; pid_n < grid_n; ++pid_n) {
      memset(acc, 0, sizeof(float) * block_m * block_n);
      for (int64_t k0 = 0; k0 < gemm_k; k0 += block_k)
        for (int im = 0; im < block_m; ++im) {
          const int64_t gm = pid_m * block_m + im;
          if (gm >= gemm_m) break;
          const int64_t batch_idx = gm / ((int64_t)h_out * w_out);
          const int64_t offs_out = gm % ((int64_t)h_out * w_out);
          const int64_t ho = offs_out / w_out, wo = offs_out % w_out;
          const int64_t base_h0 = ho * stride_h - pad_h, base_w0 = wo * stride_w - pad_w;
          for (int in = 0; in < block_n; ++in) {
            const int64_t cout = pid_n * block_n + in;
            if (cout >= gemm_n) break;
            float s = acc[im * block_n + in];
            for (int kk = 0; kk < block_k; ++kk) {
              const int64_t gk = k0 + kk;
              if (gk >= gemm_k) break;               /* offs_cin < C_IN mask */
              const int64_t cin = gk / ((int64_t)fh * fw);
              const int64_t resid = gk % ((int64_t)fh * fw);
              const int64_t tap_h = resid / fw, tap_w = resid % fw;
              const int64_t hin = base_h0 + tap_h * dil_h, win = base_w0 + tap_w * dil_w;
              if (hin < 0 || hin >= h_in || win < 0 || win >= w_in) continue;   /* other = 0 */
              const float xv = x[((batch_idx * c_in + cin) * h_in + hin) * w_in + win];
              const float wv = w[cout * gemm_k + cin * ((int64_t)fh * fw) + tap_h * fw + tap_w];
              s += xv * wv;
            }
            acc[im * block_n + in] = s;
          }
        }
      for (int im = 0; im < block_m; ++im) {
        const int64_t gm = pid_m * block_m + im;
        if (gm >= gemm_m) break;
        const int64_t batch_idx = gm / ((int64_t)h_out * w_out);
        const int64_t offs_out = gm % ((int64_t)h_out * w_out);
        for (int in = 0; in < block_n; ++in) {
          const int64_t cout = pid_n * block_n + in;
          if (cout >= gemm_n) break;
          float v = acc[im * block_n + in];
          if (bias) v = v + bias[cout];
          y[(batch_idx * c_out + cout) * ((int64_t)h_out * w_out) + offs_out] = v;
        }
      }
    }
  free(acc);
  return 0;
}
