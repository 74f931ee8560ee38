/*
 * CPU restatement of the reference's tiled-GEMM path.  TEST INFRASTRUCTURE
 * ONLY: tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py
 * may link or call this; the product (tritonix_amd/) never does.
 *
 * Every function restates one piece of the reference's algorithm, tile by
 * tile and K block by K block, the way the Triton programs walk it -- not a
 * call into a BLAS:
 *   oracle_swizzle2d      tl.swizzle2d as called at tritonix/ops/matmul.py:70,172
 *                         (triton/language/standard.py:80-116; restated in
 *                         playground/swizzle.py:7-41)
 *   oracle_grouped_launch tritonix/ops/matmul.py:111-130
 *   oracle_matmul_f32     matmul_kernel, tritonix/ops/matmul.py:43-108: 2-D grid
 *                         of (block_m x block_n) programs, swizzled, K loop of
 *                         block_k slabs masked at the K tail, fp32 accumulate,
 *                         M/N-masked store
 *   oracle_matmul_i8      same walk, int8 x int8 -> int32
 *                         (playground/test_int8_mma.py:7-42)
 *   oracle_splitk_f32     gemm_splitk_kernel, tritonix/ops/matmul.py:147-202:
 *                         program pid_k takes K blocks pid_k, pid_k+split_k, ...
 *                         (:176,:185-193); partials are summed in fp32 and
 *                         rounded once by the caller (the reference rounds each
 *                         partial to the output dtype before its atomic add,
 *                         :195-202; the build deliberately does not)
 *   oracle_splitk_cover   how many programs touch each k (must be exactly 1)
 *   oracle_glu_f32        glu_kernel, tritonix/ops/swiglu.py:24-110: same main
 *                         loop on the interleaved weight, epilogue :98-104
 *                         (even column = gate, odd = linear; silu only when
 *                         activation == "silu"; sigmoid added; else identity)
 *   oracle_xcd_remap      block id -> logical tile id used by the HIP kernels
 *                         (no counterpart in the reference; must be a bijection)
 *
 * Inputs are fp32 arrays that already hold the bf16/fp16-rounded values, so
 * the only rounding the caller adds is the final one to the output dtype.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int64_t imin(int64_t a, int64_t b) { return a < b ? a : b; }
static int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

void oracle_swizzle2d(int i, int j, int size_i, int size_j, int size_g, int* out_i, int* out_j) {
  int ij = i * size_j + j;
  int size_gj = size_g * size_j;
  int group_id = ij / size_gj;
  int off_i = group_id * size_g;
  int g = (int)imin(size_i - off_i, size_g);
  ij = ij % size_gj;
  *out_i = off_i + ij % g;
  *out_j = ij / g;
}

void oracle_grouped_launch(int pid, int m, int n, int block_m, int block_n, int group_m, int* pid_m, int* pid_n) {
  int grid_m = (int)cdiv(m, block_m), grid_n = (int)cdiv(n, block_n);
  int width = group_m * grid_n;
  int group_id = pid / width;
  int group_size = (int)imin(grid_m - group_id * group_m, group_m);
  *pid_m = group_id * group_m + (pid % group_size);
  *pid_n = (pid % width) / group_size;
}

int oracle_xcd_remap(int pid, int total, int nxcd) {
  int q = total / nxcd, r = total % nxcd;
  int x = pid % nxcd, idx = pid / nxcd;
  return x * q + (x < r ? x : r) + idx;
}

/* one (pid_m, pid_n[, pid_k]) program of the reference kernels: accumulate the tile into acc[block_m*block_n] */
static void tile_program_f32(const float* a, const float* b, float* acc, int64_t m, int64_t n, int64_t k, int64_t sam,
                             int64_t sak, int64_t sbk, int64_t sbn, int pid_m, int pid_n, int pid_k, int split_k,
                             int block_m, int block_n, int block_k) {
  int64_t grid_k = cdiv(k, (int64_t)block_k * split_k);
  memset(acc, 0, sizeof(float) * block_m * block_n);
  for (int64_t k_loop = 0; k_loop < grid_k; ++k_loop) {
    int64_t kbase = (k_loop * split_k + pid_k) * block_k; /* offs_k = pid_k*block_k + arange, stepped by block_k*split_k */
    for (int kk = 0; kk < block_k; ++kk) {
      int64_t gk = kbase + kk;
      if (gk >= k) break; /* K-tail mask: other = 0 */
      for (int r = 0; r < block_m; ++r) {
        int64_t gm = (int64_t)pid_m * block_m + r;
        if (gm >= m) continue; /* rows past M are never stored */
        float av = a[gm * sam + gk * sak];
        for (int c = 0; c < block_n; ++c) {
          int64_t gn = (int64_t)pid_n * block_n + c;
          if (gn >= n) continue;
          acc[r * block_n + c] += av * b[gk * sbk + gn * sbn];
        }
      }
    }
  }
}

static void walk_f32(const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int64_t sam, int64_t sak,
                     int64_t sbk, int64_t sbn, int64_t scm, int64_t scn, int block_m, int block_n, int block_k,
                     int group_m, int split_k) {
  int num_pid_m = (int)cdiv(m, block_m), num_pid_n = (int)cdiv(n, block_n);
  float* acc = (float*)malloc(sizeof(float) * block_m * block_n);
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) c[i * scm + j * scn] = 0.0f; /* _zero_output / torch.zeros */
  for (int gi = 0; gi < num_pid_m; ++gi)
    for (int gj = 0; gj < num_pid_n; ++gj) {
      int pid_m, pid_n;
      oracle_swizzle2d(gi, gj, num_pid_m, num_pid_n, group_m, &pid_m, &pid_n);
      for (int pid_k = 0; pid_k < split_k; ++pid_k) {
        tile_program_f32(a, b, acc, m, n, k, sam, sak, sbk, sbn, pid_m, pid_n, pid_k, split_k, block_m, block_n,
                         block_k);
        for (int r = 0; r < block_m; ++r)
          for (int cc = 0; cc < block_n; ++cc) {
            int64_t gm = (int64_t)pid_m * block_m + r, gn = (int64_t)pid_n * block_n + cc;
            if (gm < m && gn < n) c[gm * scm + gn * scn] += acc[r * block_n + cc];
          }
      }
    }
  free(acc);
}

void oracle_matmul_f32(const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int64_t sam,
                       int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn, int block_m, int block_n,
                       int block_k, int group_m) {
  walk_f32(a, b, c, m, n, k, sam, sak, sbk, sbn, scm, scn, block_m, block_n, block_k, group_m, 1);
}

void oracle_splitk_f32(const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int64_t sam,
                       int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn, int block_m, int block_n,
                       int block_k, int group_m, int split_k) {
  walk_f32(a, b, c, m, n, k, sam, sak, sbk, sbn, scm, scn, block_m, block_n, block_k, group_m, split_k);
}

/* cover[kk] = number of (pid_k, k_loop, lane) triples of the split-K walk that load index kk */
void oracle_splitk_cover(int64_t k, int block_k, int split_k, int32_t* cover) {
  int64_t grid_k = cdiv(k, (int64_t)block_k * split_k);
  for (int64_t i = 0; i < k; ++i) cover[i] = 0;
  for (int pid_k = 0; pid_k < split_k; ++pid_k)
    for (int64_t k_loop = 0; k_loop < grid_k; ++k_loop) {
      int64_t k_remaining = k - k_loop * ((int64_t)block_k * split_k);
      for (int lane = 0; lane < block_k; ++lane) {
        int64_t offs_k = (int64_t)pid_k * block_k + lane; /* tritonix/ops/matmul.py:176 */
        if (offs_k < k_remaining) cover[k_loop * (int64_t)block_k * split_k + offs_k] += 1;
      }
    }
}

void oracle_matmul_i8(const int8_t* a, const int8_t* b, int32_t* c, int64_t m, int64_t n, int64_t k, int64_t sam,
                      int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn, int block_m, int block_n,
                      int block_k) {
  int num_pid_m = (int)cdiv(m, block_m), num_pid_n = (int)cdiv(n, block_n);
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * block_m * block_n);
  for (int pid_m = 0; pid_m < num_pid_m; ++pid_m)
    for (int pid_n = 0; pid_n < num_pid_n; ++pid_n) {
      memset(acc, 0, sizeof(int32_t) * block_m * block_n);
      for (int64_t k0 = 0; k0 < k; k0 += block_k)
        for (int kk = 0; kk < block_k && k0 + kk < k; ++kk)
          for (int r = 0; r < block_m; ++r) {
            int64_t gm = (int64_t)pid_m * block_m + r;
            if (gm >= m) continue;
            int32_t av = a[gm * sam + (k0 + kk) * sak];
            for (int cc = 0; cc < block_n; ++cc) {
              int64_t gn = (int64_t)pid_n * block_n + cc;
              if (gn < n) acc[r * block_n + cc] += av * (int32_t)b[(k0 + kk) * sbk + gn * sbn];
            }
          }
      for (int r = 0; r < block_m; ++r)
        for (int cc = 0; cc < block_n; ++cc) {
          int64_t gm = (int64_t)pid_m * block_m + r, gn = (int64_t)pid_n * block_n + cc;
          if (gm < m && gn < n) c[gm * scm + gn * scn] = acc[r * block_n + cc];
        }
    }
  free(acc);
}

/* activation: 1 = silu, 2 = sigmoid, anything else = identity gate */
void oracle_glu_f32(const float* x, const float* w12, float* z, int64_t m, int64_t n, int64_t k, int64_t sxm,
                    int64_t sxk, int64_t swk, int64_t swn, int64_t szm, int64_t szn, int block_m, int block_n,
                    int block_k, int group_m, int activation) {
  int num_pid_m = (int)cdiv(m, block_m), num_pid_n = (int)cdiv(n, block_n);
  float* acc = (float*)malloc(sizeof(float) * block_m * block_n);
  for (int gi = 0; gi < num_pid_m; ++gi)
    for (int gj = 0; gj < num_pid_n; ++gj) {
      int pid_m, pid_n;
      oracle_swizzle2d(gi, gj, num_pid_m, num_pid_n, group_m, &pid_m, &pid_n);
      tile_program_f32(x, w12, acc, m, n, k, sxm, sxk, swk, swn, pid_m, pid_n, 0, 1, block_m, block_n, block_k);
      /* reshape(block_m, block_n/2, 2); z, raw = split */
      for (int r = 0; r < block_m; ++r)
        for (int h = 0; h < block_n / 2; ++h) {
          float g = acc[r * block_n + 2 * h], raw = acc[r * block_n + 2 * h + 1];
          if (activation == 1) g = (1.0f / (1.0f + expf(-g))) * g;
          else if (activation == 2) g = 1.0f / (1.0f + expf(-g));
          int64_t gm = (int64_t)pid_m * block_m + r, gc = (int64_t)pid_n * (block_n / 2) + h;
          if (gm < m && gc < n / 2) z[gm * szm + gc * szn] = g * raw;
        }
    }
  free(acc);
}
