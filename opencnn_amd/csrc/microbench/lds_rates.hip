// Probe: what an LDS instruction costs on gfx950 with four waves of a workgroup at work (one per
// SIMD, as in the fused kernels): clocks per wave instruction and bytes per clock and compute unit,
// for the read and write patterns that the layouts of the transformed input V were chosen among.
// Prints a table; no arguments.  Build: make -C opencnn_amd/csrc microbench.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                      \
  do {                                                                \
    hipError_t e_ = (x);                                              \
    if (e_ != hipSuccess) {                                           \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));         \
      exit(1);                                                        \
    }                                                                 \
  } while (0)

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));

enum Kind { kReadB128, kReadB64, kReadB32, kRead2St64, kWriteB128, kWriteB64, kWrite2St64, kWrite2St64Slots, kWriteB64Slots };

template <int KIND>
__global__ void __launch_bounds__(256) probe(float* out, int iters, long long* clk) {
  __shared__ float lds[16384];
  for (int i = threadIdx.x; i < 16384; i += 256) lds[i] = i;
  __syncthreads();
  const unsigned a16 = threadIdx.x * 16, a8 = threadIdx.x * 8, a4 = threadIdx.x * 4;
  const unsigned lane = threadIdx.x & 63, wv = threadIdx.x >> 6, n = lane & 31, j = lane >> 5;
  // a layout with 16 contiguous bytes per (half h, column n): wave wv owns the dwords 2 * (wv & 1) + j of half wv >> 1
  const unsigned slot_dword = (wv >> 1) * 512 + n * 16 + (2 * (wv & 1) + j) * 4;  // one dword per lane into its slot
  const unsigned slot_pair = (wv >> 1) * 512 + n * 16 + (wv & 1) * 8 + j * 1024;  // 8 bytes per lane, halves one position apart
  v4f r4[8];
  v2f r2[8];
  float r1[8];
  for (int q = 0; q < 8; ++q) {
    r4[q] = 0;
    r2[q] = 0;
    r1[q] = 0;
  }
  const long long c0 = clock64();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      if (KIND == kReadB128) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r4[q]) : "v"(a16), "n"(q * 4096));
      if (KIND == kReadB64) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r2[q]) : "v"(a8), "n"(q * 2048));
      if (KIND == kReadB32) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r1[q]) : "v"(a4), "n"(q * 1024));
      if (KIND == kRead2St64)
        asm volatile("ds_read2st64_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(r2[q]) : "v"(a4), "n"(q * 2), "n"(q * 2 + 1));
      if (KIND == kWriteB128) asm volatile("ds_write_b128 %1, %0 offset:%2" ::"v"(r4[q]), "v"(a16), "n"(q * 4096) : "memory");
      if (KIND == kWriteB64) asm volatile("ds_write_b64 %1, %0 offset:%2" ::"v"(r2[q]), "v"(a8), "n"(q * 2048) : "memory");
      if (KIND == kWrite2St64)
        asm volatile("ds_write2st64_b32 %0, %1, %2 offset0:%3 offset1:%4" ::"v"(a4), "v"(r1[q]), "v"(r1[(q + 1) & 7]), "n"(q * 8),
                     "n"(q * 8 + 4)
                     : "memory");
      if (KIND == kWrite2St64Slots)
        asm volatile("ds_write2st64_b32 %0, %1, %2 offset0:%3 offset1:%4" ::"v"(slot_dword), "v"(r1[q]), "v"(r1[(q + 1) & 7]),
                     "n"(q * 8), "n"(q * 8 + 4)
                     : "memory");
      if (KIND == kWriteB64Slots) asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(slot_pair), "v"(r2[q]), "n"(q * 2048) : "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  const long long c1 = clock64();
  float s = 0;
  for (int q = 0; q < 8; ++q) s += r4[q][0] + r4[q][3] + r2[q][0] + r2[q][1] + r1[q];
  out[blockIdx.x * 256 + threadIdx.x] = s + lds[threadIdx.x];
  if (threadIdx.x == 0 && blockIdx.x == 0) clk[0] = c1 - c0;
}

template <int KIND>
void run(const char* what, int bytes_per_lane) {
  float* out;
  long long* clk;
  CHECK(hipMalloc(&out, 256 * 256 * 4));
  CHECK(hipMalloc(&clk, 8));
  const int iters = 20000;
  probe<KIND><<<256, 256>>>(out, 100, clk);
  CHECK(hipDeviceSynchronize());
  probe<KIND><<<256, 256>>>(out, iters, clk);
  CHECK(hipDeviceSynchronize());
  long long c;
  CHECK(hipMemcpy(&c, clk, 8, hipMemcpyDeviceToHost));
  const double bytes = (double)iters * 8 * 256 * bytes_per_lane;
  printf("%-44s %6.1f clocks per wave instruction, %6.1f B per clock and CU\n", what, (double)c / iters / 8, bytes / c);
  fflush(stdout);
  CHECK(hipFree(out));
  CHECK(hipFree(clk));
}

int main() {
  run<kReadB128>("ds_read_b128, lane * 16", 16);
  run<kReadB64>("ds_read_b64, lane * 8", 8);
  run<kReadB32>("ds_read_b32, lane * 4", 4);
  run<kRead2St64>("ds_read2st64_b32, lane * 4", 8);
  run<kWriteB128>("ds_write_b128, lane * 16", 16);
  run<kWriteB64>("ds_write_b64, lane * 8", 8);
  run<kWrite2St64>("ds_write2st64_b32, lane * 4", 8);
  run<kWrite2St64Slots>("ds_write2st64_b32, a dword into 16-byte slots", 8);
  run<kWriteB64Slots>("ds_write_b64, 8 bytes into 16-byte slots", 8);
  return 0;
}
