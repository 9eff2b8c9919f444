/*
 * CPU oracle for the fused Winograd F(2x2,3x3) forward convolution.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT.  It is a plain-C restatement of
 * the arithmetic of UDC-GAC/openCNN's hot path, used only by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker.
 * Nothing in opencnn_amd/ links, loads or calls it.
 *
 * The reference (CUDA, needs nvcc + cuDNN + cuRAND + an NVIDIA device) cannot be
 * compiled here, and it ships no tests, fixtures or golden vectors; every function
 * below is therefore pinned by closed forms and brute force in tests/test_oracle.py:
 *
 *   oracle_direct_conv_f64   textbook cross-correlation, pad 1, stride 1 (the semantics
 *                            of the cuDNN descriptor the reference checks itself
 *                            against, src/openCNN_winograd.cu:369-372, and of its
 *                            checker's KHWN<->NCHW index map, :185-186).
 *                            Pinned against an independent numpy einsum on padded
 *                            inputs and against single-impulse known answers.
 *   oracle_fx                src/FX_m2.cu:23-47,68-86 (U = G g G^T, CRSK in,
 *                            [C][16][K] out).  Pinned against the closed form with
 *                            the textbook G in fp64, delta filters and the all-ones
 *                            filter.
 *   oracle_input_transform   src/convolutionForward_32x64x8.cu:59-80 (V = B^T d B,
 *                            columns first, then rows).  Pinned against B^T d B in
 *                            fp64 on integer patches (adds only: exact).
 *   oracle_output_transform  src/store_and_transform_output_optSTS64.cuh:29-51
 *                            (Y = A^T M A).  Pinned against A^T M A in fp64 on
 *                            integer inputs.
 *   oracle_winograd_f32      the whole path in the reference's order: masks
 *                            src/convolutionForward_32x64x8.cu:179-183 and
 *                            src/store_and_transform_output_optSTS64.cuh:65-67,
 *                            tiling src/openCNN_winograd.cu:286-288, reduction as one
 *                            fp32 FMA per input channel, ascending c
 *                            (src/convolutionForward_32x64x8.cu:210-257,
 *                            src/outer_product_suffle.cuh).  Pinned against
 *                            oracle_direct_conv_f64 on odd and even H (mask errors
 *                            are O(1) there) and, bit-exactly, on small-integer
 *                            tensors where every summation order agrees.
 *                            One thing stays "parity unpinned" by construction:
 *                            that nvcc contracted each `acc += a*b` into an FFMA
 *                            (assumed from nvcc's default -fmad=true; the effect is
 *                            at the 1e-7 level, two orders below the 1e-5 bar).
 *   quantised variant        V and U rounded (RNE) to fp16 / bf16 before the GEMM,
 *                            fp32 accumulate; no counterpart in the reference
 *                            (it is fp32 only), checked against the fp64 direct
 *                            convolution with the looser bound stated in the tests.
 *   oracle_round_operand     the RNE roundings of that variant.  Pinned against numpy's
 *                            float16 cast, torch's CPU bfloat16 / float16 casts and
 *                            round-to-nearest-even written from its definition in exact
 *                            rationals (ties of both parities, carries, subnormals,
 *                            overflow, signed zeros).
 *   oracle_compare_*         the error metric (relative L2, max |diff|, max |want|).
 *                            Pinned against numpy norms; NaN / Inf poison both figures.
 *
 * Layouts (all row-major, last index fastest):
 *   x   CHWN  [C][H][W][N]   src/openCNN_winograd.cu:149-150,230
 *   w   CRSK  [C][3][3][K]   src/openCNN_winograd.cu:235, src/FX_m2.cu:56-57,69
 *   Ww  [C][16][K]           src/FX_m2.cu:58-59,84
 *   y   KHWN  [K][H][W][N]   src/store_and_transform_output_optSTS64.cuh:85-87
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* tiles per image side: ceil(ceil((W+2)/2) - 1), src/openCNN_winograd.cu:286-288 */
int oracle_tiles_dim(int in_w) {
  return (int)ceil(ceil((double)(in_w + 2) / 2.0) - 1.0);
}

/* ------------------------------------------------------------------ direct conv */

/* y[k][h][w][n] = sum_{c,r,s} x[c][h+r-1][w+s-1][n] * g[c][r][s][k]; fp64 accumulate.
 * Filters in CRSK; output in fp64 KHWN.  H and W may differ. */
void oracle_direct_conv_f64(const float *x, const float *w_crsk, double *y,
                            int N, int C, int H, int W, int K) {
  const long HWN = (long)H * W * N;
#pragma omp parallel
  {
    double *acc = (double *)malloc(sizeof(double) * (size_t)W * N);
#pragma omp for collapse(2) schedule(static)
    for (int k = 0; k < K; k++) {
      for (int h = 0; h < H; h++) {
        for (long i = 0; i < (long)W * N; i++) acc[i] = 0.0;
        for (int c = 0; c < C; c++) {
          for (int r = 0; r < 3; r++) {
            int hh = h + r - 1;
            if (hh < 0 || hh >= H) continue;
            const float *row = x + (long)c * HWN + (long)hh * W * N;
            for (int s = 0; s < 3; s++) {
              const double g = (double)w_crsk[(((long)c * 3 + r) * 3 + s) * K + k];
              int w0 = (s == 0) ? 1 : 0;          /* first valid output column   */
              int w1 = (s == 2) ? W - 1 : W;      /* one past last valid column  */
              const float *src = row + (long)(w0 + s - 1) * N;
              double *dst = acc + (long)w0 * N;
              long cnt = (long)(w1 - w0) * N;
              for (long i = 0; i < cnt; i++) dst[i] += g * (double)src[i];
            }
          }
        }
        double *out = y + ((long)k * H + h) * W * N;
        memcpy(out, acc, sizeof(double) * (size_t)W * N);
      }
    }
    free(acc);
  }
}

/* ------------------------------------------------------------------ transforms */

/* One filter: g[9] (r*3+s) -> U[16] (i*4+j).  src/FX_m2.cu:23-47,68-86. */
void oracle_fx_one(const float *g, float *U) {
  float t[12]; /* t[i*3+s] = (G g)[i][s] */
  for (int s = 0; s < 3; s++) {
    t[0 * 3 + s] = g[s];
    t[1 * 3 + s] = (float)(0.5 * (double)((g[s] + g[6 + s]) + g[3 + s]));
    t[2 * 3 + s] = (float)(0.5 * (double)((g[s] + g[6 + s]) - g[3 + s]));
    t[3 * 3 + s] = g[6 + s];
  }
  for (int i = 0; i < 4; i++) {
    const float *ti = t + i * 3;
    U[i * 4 + 0] = ti[0];
    U[i * 4 + 1] = (float)(0.5 * (double)((ti[0] + ti[2]) + ti[1]));
    U[i * 4 + 2] = (float)(0.5 * (double)((ti[0] + ti[2]) - ti[1]));
    U[i * 4 + 3] = ti[2];
  }
}

/* CRSK [C][3][3][K] -> Ww [C][16][K].  src/FX_m2.cu:51-91. */
void oracle_fx(const float *w_crsk, float *Ww, int C, int K) {
#pragma omp parallel for schedule(static)
  for (int c = 0; c < C; c++) {
    for (int k = 0; k < K; k++) {
      float g[9], U[16];
      for (int i = 0; i < 9; i++) g[i] = w_crsk[((long)c * 9 + i) * K + k];
      oracle_fx_one(g, U);
      for (int p = 0; p < 16; p++) Ww[((long)c * 16 + p) * K + k] = U[p];
    }
  }
}

/* d[16] (i*4+j) -> V[16] = B^T d B, columns first then rows.
 * src/convolutionForward_32x64x8.cu:59-80. */
void oracle_input_transform(const float *d, float *V) {
  float t[16];
  for (int j = 0; j < 4; j++) {
    t[0 + j] = d[0 + j] - d[8 + j];
    t[4 + j] = d[4 + j] + d[8 + j];
    t[8 + j] = d[8 + j] - d[4 + j];
    t[12 + j] = d[4 + j] - d[12 + j];
  }
  for (int i = 0; i < 4; i++) {
    V[i * 4 + 0] = t[i * 4 + 0] - t[i * 4 + 2];
    V[i * 4 + 1] = t[i * 4 + 1] + t[i * 4 + 2];
    V[i * 4 + 2] = t[i * 4 + 2] - t[i * 4 + 1];
    V[i * 4 + 3] = t[i * 4 + 1] - t[i * 4 + 3];
  }
}

/* m[16] (i*4+j) -> y[4] (a*2+b) = A^T m A.
 * src/store_and_transform_output_optSTS64.cuh:29-51. */
void oracle_output_transform(const float *m, float *y) {
  float a[8];
  for (int j = 0; j < 4; j++) {
    a[j] = (m[j] + m[4 + j]) + m[8 + j];
    a[4 + j] = (m[4 + j] - m[8 + j]) - m[12 + j];
  }
  for (int i = 0; i < 2; i++) {
    y[i * 2 + 0] = (a[i * 4 + 0] + a[i * 4 + 1]) + a[i * 4 + 2];
    y[i * 2 + 1] = (a[i * 4 + 1] - a[i * 4 + 2]) - a[i * 4 + 3];
  }
}

/* ------------------------------------------------------------------ rounding */

static float round_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7f800000u) == 0x7f800000u) return f; /* inf / nan unchanged */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  u &= 0xffff0000u;
  memcpy(&f, &u, 4);
  return f;
}

/* Round-to-nearest-even to IEEE binary16 and back (handles subnormals, overflow->inf). */
static float round_fp16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = u & 0x80000000u;
  uint32_t au = u & 0x7fffffffu;
  float af;
  memcpy(&af, &au, 4);
  if (au >= 0x7f800000u) return f;
  float r;
  if (af >= 65520.0f) {
    r = INFINITY;
  } else if (af < 6.103515625e-05f) { /* below 2^-14: fixed quantum 2^-24 */
    r = (float)(nearbyint((double)af * 16777216.0) / 16777216.0);
  } else {
    uint32_t lsb = (au >> 13) & 1u;
    uint32_t v = au + 0xfffu + lsb;
    v &= 0xffffe000u;
    memcpy(&r, &v, 4);
  }
  uint32_t ru;
  memcpy(&ru, &r, 4);
  ru |= sign;
  memcpy(&r, &ru, 4);
  return r;
}

float oracle_round_operand(float f, int quant) {
  if (quant == 1) return round_fp16(f);
  if (quant == 2) return round_bf16(f);
  return f;
}

/* ------------------------------------------------------------------ full path */

/* Whole Winograd path in the reference's arithmetic order.
 *   quant: 0 = fp32 operands (the reference), 1 = fp16, 2 = bf16 GEMM operands.
 * Square images only (H == W), like the reference's masks.  Returns 0, or -1 on a
 * shape it does not model. */
int oracle_winograd_f32(const float *x, const float *w_crsk, float *y,
                        int N, int C, int H, int W, int K, int quant) {
  if (H != W || N <= 0 || C <= 0 || K <= 0 || H <= 0) return -1;
  const int td = oracle_tiles_dim(W);
  const long HWN = (long)H * W * N;

  float *U = (float *)malloc(sizeof(float) * (size_t)C * 16 * K);
  if (!U) return -1;
  oracle_fx(w_crsk, U, C, K);
  if (quant) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)C * 16 * K; i++) U[i] = oracle_round_operand(U[i], quant);
  }

#pragma omp parallel
  {
    float *M = (float *)malloc(sizeof(float) * (size_t)16 * K * N); /* [p][k][n] */
    float *V = (float *)malloc(sizeof(float) * (size_t)16 * N);     /* [p][n]    */
#pragma omp for schedule(dynamic, 1)
    for (int tile = 0; tile < td * td; tile++) {
      const int ty = tile / td, tx = tile % td;
      memset(M, 0, sizeof(float) * (size_t)16 * K * N);
      for (int c = 0; c < C; c++) {
        /* gather the 4x4 patch at (2ty-1, 2tx-1), zero outside the image
         * (src/convolutionForward_32x64x8.cu:118-147,179-183), and transform */
        for (int n = 0; n < N; n++) {
          float d[16], v[16];
          for (int i = 0; i < 4; i++) {
            for (int j = 0; j < 4; j++) {
              int hh = 2 * ty - 1 + i, ww = 2 * tx - 1 + j;
              d[i * 4 + j] = (hh >= 0 && hh < H && ww >= 0 && ww < W)
                                 ? x[(long)c * HWN + ((long)hh * W + ww) * N + n]
                                 : 0.0f;
            }
          }
          oracle_input_transform(d, v);
          for (int p = 0; p < 16; p++) V[(long)p * N + n] = oracle_round_operand(v[p], quant);
        }
        /* one FMA per (p,k,n) per channel, ascending c */
        for (int p = 0; p < 16; p++) {
          const float *Vp = V + (long)p * N;
          const float *Up = U + ((long)c * 16 + p) * K;
          for (int k = 0; k < K; k++) {
            const float u = Up[k];
            float *Mk = M + ((long)p * K + k) * N;
            for (int n = 0; n < N; n++) Mk[n] = fmaf(Vp[n], u, Mk[n]);
          }
        }
      }
      /* output transform + masked store (odd sizes drop the last row/column) */
      for (int k = 0; k < K; k++) {
        for (int n = 0; n < N; n++) {
          float m[16], o[4];
          for (int p = 0; p < 16; p++) m[p] = M[((long)p * K + k) * N + n];
          oracle_output_transform(m, o);
          for (int a = 0; a < 2; a++) {
            for (int b = 0; b < 2; b++) {
              int hh = 2 * ty + a, ww = 2 * tx + b;
              if (hh < H && ww < W) y[(long)k * HWN + ((long)hh * W + ww) * N + n] = o[a * 2 + b];
            }
          }
        }
      }
    }
    free(M);
    free(V);
  }
  free(U);
  return 0;
}

/* ------------------------------------------------------------------ metrics */

/* rel_l2 = ||got-want||_2 / ||want||_2, max_abs = max|got-want|, max_ref = max|want|.
 * `want` is fp64. */
void oracle_compare_f32_f64(const float *got, const double *want, long n, double *rel_l2,
                            double *max_abs, double *max_ref) {
  double num = 0.0, den = 0.0, ma = 0.0, mr = 0.0;
  long bad = 0;
#pragma omp parallel for reduction(+ : num, den, bad) reduction(max : ma, mr) schedule(static)
  for (long i = 0; i < n; i++) {
    double d = (double)got[i] - want[i];
    num += d * d;
    den += want[i] * want[i];
    double ad = fabs(d), ar = fabs(want[i]);
    if (!isfinite(d)) bad++;
    if (ad > ma) ma = ad;
    if (ar > mr) mr = ar;
  }
  *rel_l2 = (den > 0.0) ? sqrt(num / den) : sqrt(num);
  *max_abs = ma;
  if (bad) { *rel_l2 = NAN; *max_abs = NAN; } /* any NaN/inf in got poisons the verdict */
  *max_ref = mr;
}

void oracle_compare_f32_f32(const float *got, const float *want, long n, double *rel_l2,
                            double *max_abs, double *max_ref) {
  double num = 0.0, den = 0.0, ma = 0.0, mr = 0.0;
  long bad = 0;
#pragma omp parallel for reduction(+ : num, den, bad) reduction(max : ma, mr) schedule(static)
  for (long i = 0; i < n; i++) {
    double d = (double)got[i] - (double)want[i];
    num += d * d;
    den += (double)want[i] * (double)want[i];
    double ad = fabs(d), ar = fabs((double)want[i]);
    if (!isfinite(d)) bad++;
    if (ad > ma) ma = ad;
    if (ar > mr) mr = ar;
  }
  *rel_l2 = (den > 0.0) ? sqrt(num / den) : sqrt(num);
  *max_abs = ma;
  if (bad) { *rel_l2 = NAN; *max_abs = NAN; } /* any NaN/inf in got poisons the verdict */
  *max_ref = mr;
}
