// wgrad: bench CLI with the reference's shape arguments, on top of the C ABI.
//
// Host-side counterpart of the reference's bench driver (src/openCNN_winograd.cu:241-495):
//   wgrad N C H W K [C R S]        (the reference's positional list, :246-255)
//   wgrad N C H W K pad stride     (pad and stride surfaced; both must be 1, as the
//                                   reference's PAD_H/STR_H macros, src/config.hpp:43-46)
// Prints the reference's CSV prefix `in_n,in_c,in_h,filt_k,filt_w,ms,tflops` (:257,445; the
// tflops column keeps the reference's formula 2*N*C*(H+2)*(W+2)*K*9/2.25, :118-125) and
// appends effective TFLOP/s on direct-convolution FLOPs, the fused kernel's share of the
// MFMA peak and the HBM rate at the compulsory bytes.
//
// Where the reference runs cuDNN's Winograd and compares element-wise (:449-476), this CLI
// runs a naive fp64-accumulating direct convolution ON THE GPU and reports max error and
// relative L2; its exit status is non-zero when relative L2 exceeds 1e-3.
//
// Environment: WGRAD_ITERS (timed calls, default 100), WGRAD_OPERANDS = f16 | bf16 (GEMM
// operand precision; the peak share is then of the fp16 / bf16 matrix peak and the bound on
// relative L2 is 2e-3 / 1.5e-2).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/opencnn_amd.h"
#include "../../include/opencnn_amd_bench.h"

#define HIP_CALL(x)                                                                     \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      fprintf(stderr, "Error occurred: %s %s %d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      exit((int)e_);                                                                    \
    }                                                                                   \
  } while (0)

#define OPENCNN_CALL(x)                                                                 \
  do {                                                                                  \
    int e_ = (x);                                                                       \
    if (e_ != 0) {                                                                      \
      fprintf(stderr, "Error occurred: hipError_t %d (%s) %s %d\n", e_, opencnn_last_error(), \
              __FILE__, __LINE__);                                                      \
      exit(e_);                                                                         \
    }                                                                                   \
  } while (0)

// y[k][h][w][n] = sum_{c,r,s} x[c][h+r-1][w+s-1][n] * g[c][r][s][k], fp64 accumulate.
// One thread per output element; n fastest so loads of x are coalesced.
__global__ void direct_conv_check(const float* __restrict__ x, const float* __restrict__ g,
                                  double* __restrict__ y, int N, int C, int H, int W, int K) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)K * H * W * N;
  if (idx >= total) return;
  const int n = (int)(idx % N);
  const int w = (int)((idx / N) % W);
  const int h = (int)((idx / ((size_t)N * W)) % H);
  const int k = (int)(idx / ((size_t)N * W * H));
  double acc = 0.0;
  for (int c = 0; c < C; ++c)
    for (int r = 0; r < 3; ++r) {
      const int hh = h + r - 1;
      if (hh < 0 || hh >= H) continue;
      for (int s = 0; s < 3; ++s) {
        const int ww = w + s - 1;
        if (ww < 0 || ww >= W) continue;
        acc += (double)x[(((size_t)c * H + hh) * W + ww) * N + n] *
               (double)g[(((size_t)c * 3 + r) * 3 + s) * K + k];
      }
    }
  y[idx] = acc;
}

int main(int argc, char** argv) {
  // defaults: the reference's compiled-in shape (src/config.hpp:36-41)
  const int in_n = argc > 1 ? atoi(argv[1]) : 128;
  const int in_c = argc > 2 ? atoi(argv[2]) : 256;
  const int in_h = argc > 3 ? atoi(argv[3]) : 14;
  const int in_w = argc > 4 ? atoi(argv[4]) : 14;
  const int filt_k = argc > 5 ? atoi(argv[5]) : 256;
  int filt_c = in_c, filt_h = 3, filt_w = 3;
  if (argc == 8) {  // N C H W K pad stride
    if (atoi(argv[6]) != 1 || atoi(argv[7]) != 1) {
      fprintf(stderr, "wgrad: only pad 1, stride 1 is implemented\n");
      return 2;
    }
  } else if (argc > 6) {  // the reference's N C H W K C R S
    filt_c = atoi(argv[6]);
    if (argc > 7) filt_h = atoi(argv[7]);
    if (argc > 8) filt_w = atoi(argv[8]);
  }
  const int iterations = getenv("WGRAD_ITERS") ? atoi(getenv("WGRAD_ITERS")) : 100;

  const char* operands = getenv("WGRAD_OPERANDS");
  int precision = OPENCNN_F32;
  double peak_tflops = 157.3, rel_bound = 1e-3;
  if (operands && !strcmp(operands, "f16")) {
    precision = OPENCNN_F16, peak_tflops = 2500.0, rel_bound = 2e-3;
  } else if (operands && !strcmp(operands, "bf16")) {
    precision = OPENCNN_BF16, peak_tflops = 2500.0, rel_bound = 1.5e-2;
  } else if (operands && strcmp(operands, "f32")) {
    fprintf(stderr, "wgrad: WGRAD_OPERANDS must be f32, f16 or bf16\n");
    return 2;
  }

  OPENCNN_CALL(opencnn_init());
  OPENCNN_CALL(opencnn_set_operand_precision(precision));
  const int m = 2, tile_size = m + filt_h - 1;
  const int tiles_dim = opencnn_tiles_dim(in_w), elems_dim = tiles_dim * 4;
  const int out_n = in_n, out_c = filt_k, out_h = in_h, out_w = in_w;
  const size_t n_in = (size_t)in_n * in_c * in_h * in_w, n_filt = (size_t)filt_k * filt_c * 9;
  const size_t n_out = (size_t)out_n * out_c * out_h * out_w;

  std::vector<float> h_in(n_in), h_filt(n_filt);
  if (opencnn_synth_input(h_in.data(), in_n, in_c, in_h, in_w, OPENCNN_INPUT_CHWN, 0x0C99,
                          OPENCNN_DIST_UNIFORM, -1.0, 1.0) ||
      opencnn_synth_filter(h_filt.data(), filt_k, filt_c > 0 ? filt_c : 1, OPENCNN_FILTER_CRSK,
                           0xF117, OPENCNN_DIST_NORMAL, 0.0, std::sqrt(2.0 / (9.0 * in_c)))) {
    fprintf(stderr, "wgrad: bad shape\n");
    return 2;
  }

  float *in_data, *filt_data, *workspace, *out_data;
  HIP_CALL(hipMalloc(&in_data, n_in * sizeof(float)));
  HIP_CALL(hipMalloc(&filt_data, n_filt * sizeof(float)));
  HIP_CALL(hipMalloc(&workspace, opencnn_workspace_bytes(filt_c, filt_k)));
  HIP_CALL(hipMalloc(&out_data, n_out * sizeof(float)));
  HIP_CALL(hipMemcpy(in_data, h_in.data(), n_in * sizeof(float), hipMemcpyHostToDevice));
  HIP_CALL(hipMemcpy(filt_data, h_filt.data(), n_filt * sizeof(float), hipMemcpyHostToDevice));

  printf("%d,%d,%d,%d,%d,", in_n, in_c, in_h, filt_k, filt_h);

  // warm-up call, then `iterations` timed calls (src/openCNN_winograd.cu:426-444)
  OPENCNN_CALL(convolutionForward(in_data, in_h, in_w, filt_data, out_h, out_w, out_n, out_c,
                                  out_data, workspace, (unsigned)n_out, tiles_dim, in_n,
                                  tile_size, elems_dim, in_c, filt_k, filt_c, filt_h, filt_w,
                                  tile_size, m));
  float ms_total = 0.f, ms_main = 0.f, ms_fx = 0.f;
  OPENCNN_CALL(opencnn_time_forward(in_data, filt_data, out_data, workspace, in_n, in_c, in_h,
                                    in_w, filt_k, 1, iterations, &ms_total, &ms_main, &ms_fx));

  const double ref_flops = 2.0 * in_n * in_c * (in_h + 2.0) * (in_w + 2.0) * filt_k * 9.0 / 2.25;
  const double direct_flops = 2.0 * in_n * (double)filt_k * in_c * in_h * in_w * 9.0;
  const double tiles = (double)((in_h + 1) / 2) * ((in_w + 1) / 2);
  const double mfma_flops = 32.0 * in_n * tiles * in_c * filt_k;
  const double bytes_min = 4.0 * ((double)n_in + 9.0 * filt_k * in_c + 32.0 * filt_k * in_c + (double)n_out);
  printf("%.3f,%.2f", ms_total, ref_flops / (ms_total * 1e9));
  printf(",%.2f,%.1f,%.1f,%.4f,%.4f\n", direct_flops / (ms_total * 1e9),
         100.0 * mfma_flops / (ms_main * 1e9) / peak_tflops, bytes_min / (ms_total * 1e6), ms_main, ms_fx);

  // comparison run: fp64 direct convolution on the GPU
  printf("********************************************\n");
  double* ref_data;
  HIP_CALL(hipMalloc(&ref_data, n_out * sizeof(double)));
  direct_conv_check<<<(unsigned)((n_out + 255) / 256), 256>>>(in_data, filt_data, ref_data, in_n,
                                                             in_c, in_h, in_w, filt_k);
  HIP_CALL(hipGetLastError());
  std::vector<float> got(n_out);
  std::vector<double> want(n_out);
  HIP_CALL(hipMemcpy(got.data(), out_data, n_out * sizeof(float), hipMemcpyDeviceToHost));
  HIP_CALL(hipMemcpy(want.data(), ref_data, n_out * sizeof(double), hipMemcpyDeviceToHost));
  OPENCNN_CALL(opencnn_check_status());  // every launch handed its partial tiles over
  double max_error = 0.0, num = 0.0, den = 0.0;
  long bad = 0;
  for (size_t i = 0; i < n_out; ++i) {
    const double d = (double)got[i] - want[i];
    if (!std::isfinite(d)) ++bad;
    if (std::fabs(d) > max_error) max_error = std::fabs(d);
    num += d * d;
    den += want[i] * want[i];
  }
  const double rel = den > 0 ? std::sqrt(num / den) : std::sqrt(num);
  printf("[max_error: %g][rel_l2: %g][non_finite: %ld] of %zu\n", max_error, rel, bad, n_out);

  HIP_CALL(hipFree(ref_data));
  HIP_CALL(hipFree(out_data));
  HIP_CALL(hipFree(workspace));
  HIP_CALL(hipFree(filt_data));
  HIP_CALL(hipFree(in_data));
  return (bad == 0 && rel <= rel_bound) ? 0 : 1;
}
