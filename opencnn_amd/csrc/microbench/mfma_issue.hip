// Issue-model micro-benchmarks for v_mfma_f32_32x32x2_f32 on gfx950, one wave per SIMD.
//
// The MI355X counterpart of the reference's shared-memory micro-benchmarks
// (bench/smem/LDS, bench/smem/STS: Turing SASS loops that motivated its STS.64/LDS.64
// store variants).  The questions asked here are the ones that shaped the fused kernel:
//   1. what one MFMA costs back to back (expected 64 cycles = 16 passes x 4);
//   2. what fp32 VALU instructions cost when they sit between MFMAs of the same wave,
//      interleaved one by one or issued as one burst;
//   3. the shader clock actually sustained by an MFMA loop on zero / random operands
//      (s_memtime against the constant 100 MHz wall clock).
// Output: one line per experiment, cycles per MFMA at the nominal 2.4 GHz.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef float v16f __attribute__((ext_vector_type(16)));

// NV fp32 adds per MFMA; INTERLEAVE: behind every MFMA, else all 16*NV after the 16 MFMAs.
template <int NV, bool INTERLEAVE>
__global__ void __launch_bounds__(256) mfma_valu(float* out, int iters, float a, float b) {
  v16f acc[16];
  for (int p = 0; p < 16; ++p)
    for (int r = 0; r < 16; ++r) acc[p][r] = 0.f;
  const float av = a + threadIdx.x;
  float bv[16], w[16];
  for (int p = 0; p < 16; ++p) {
    bv[p] = b + p;
    w[p] = 0.001f * p;
  }
  for (int i = 0; i < iters; ++i) {
    float nb[16];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      acc[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv[p], acc[p], 0, 0, 0);
      float t = w[p];
#pragma unroll
      for (int q = 0; q < NV; ++q) t = t + w[(p + q + 1) & 15];
      nb[p] = t;
    }
#pragma unroll
    for (int p = 0; p < 16; ++p) asm volatile("" : "+v"(nb[p]));
    if (INTERLEAVE && NV > 0) {
#pragma unroll
      for (int p = 0; p < 16; ++p) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);
      }
    } else {
      __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 16 * (NV > 0 ? NV : 1), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < 16; ++p) w[p] = nb[p];
  }
  float s = 0;
  for (int p = 0; p < 16; ++p) {
    for (int r = 0; r < 16; ++r) s += acc[p][r];
    s += w[p];
  }
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Pure MFMA loop on per-lane operands from memory; reports shader cycles and wall ticks.
__global__ void __launch_bounds__(256) mfma_clock(float* out, const float* in, int iters,
                                                  long long* clk) {
  v16f acc[16];
  for (int p = 0; p < 16; ++p)
    for (int r = 0; r < 16; ++r) acc[p][r] = 0.f;
  float av[16], bv[16];
  for (int p = 0; p < 16; ++p) {
    av[p] = in[(blockIdx.x * 256 + threadIdx.x) * 32 + p];
    bv[p] = in[(blockIdx.x * 256 + threadIdx.x) * 32 + 16 + p];
  }
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int p = 0; p < 16; ++p)
      acc[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[p], bv[p], acc[p], 0, 0, 0);
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = 0;
  for (int p = 0; p < 16; ++p)
    for (int r = 0; r < 16; ++r) s += acc[p][r];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    clk[0] = c1 - c0;
    clk[1] = w1 - w0;
  }
}

#define CHECK(x)                                                        \
  do {                                                                  \
    hipError_t e_ = (x);                                                \
    if (e_ != hipSuccess) {                                             \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));           \
      exit(1);                                                          \
    }                                                                   \
  } while (0)

template <int NV, bool INTERLEAVE>
void run_valu(const char* what, int iters) {
  float* out;
  CHECK(hipMalloc(&out, 256 * 256 * sizeof(float)));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  mfma_valu<NV, INTERLEAVE><<<256, 256>>>(out, 10, 1.f, 2.f);
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(e0));
  mfma_valu<NV, INTERLEAVE><<<256, 256>>>(out, iters, 1.f, 2.f);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  float ms;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  printf("%-44s %6.1f cycles per MFMA at 2.4 GHz\n", what, ms * 1e-3 / ((double)iters * 16) * 2.4e9);
  CHECK(hipFree(out));
}

void run_clock(const char* what, int mode, int iters) {
  const size_t n = (size_t)256 * 256 * 32;
  float* h = (float*)malloc(n * sizeof(float));
  srand(1);
  for (size_t i = 0; i < n; ++i) h[i] = mode ? (float)((double)rand() / RAND_MAX * 2 - 1) : 0.0f;
  float *in, *out;
  long long* clk;
  CHECK(hipMalloc(&in, n * sizeof(float)));
  CHECK(hipMalloc(&out, 256 * 256 * sizeof(float)));
  CHECK(hipMalloc(&clk, 2 * sizeof(long long)));
  CHECK(hipMemcpy(in, h, n * sizeof(float), hipMemcpyHostToDevice));
  mfma_clock<<<256, 256>>>(out, in, 100, clk);
  CHECK(hipDeviceSynchronize());
  mfma_clock<<<256, 256>>>(out, in, iters, clk);
  CHECK(hipDeviceSynchronize());
  long long hc[2];
  CHECK(hipMemcpy(hc, clk, sizeof(hc), hipMemcpyDeviceToHost));
  printf("%-44s %6.2f shader cycles per MFMA, shader clock %.2f GHz over %.2f ms\n", what,
         (double)hc[0] / iters / 16, (double)hc[0] / hc[1] * 0.1, hc[1] * 1e-5);
  free(h);
  CHECK(hipFree(in));
  CHECK(hipFree(out));
  CHECK(hipFree(clk));
}

int main() {
  run_valu<0, false>("16 MFMA, no VALU", 20000);
  run_valu<1, true>("1 v_add behind every MFMA", 20000);
  run_valu<2, true>("2 v_add behind every MFMA", 20000);
  run_valu<4, true>("4 v_add behind every MFMA", 20000);
  run_valu<8, true>("8 v_add behind every MFMA", 20000);
  run_valu<2, false>("16 MFMA then a burst of 32 v_add", 20000);
  run_valu<4, false>("16 MFMA then a burst of 64 v_add", 20000);
  run_clock("pure MFMA, zero operands, 1 ms", 0, 2000);
  run_clock("pure MFMA, random operands, 1 ms", 1, 2000);
  run_clock("pure MFMA, random operands, 10 ms", 1, 20000);
  run_clock("pure MFMA, random operands, 90 ms", 1, 200000);
  return 0;
}
