// Plain copy kernel of known size (256 MiB read, 256 MiB written per launch): calibrates the
// FETCH_SIZE / WRITE_SIZE counters that price the fused kernel's HBM traffic.
#include <hip/hip_runtime.h>
#include <cstdio>
__global__ void copy_kernel(const float4* __restrict__ a, float4* __restrict__ b, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) b[i] = a[i];
}
int main() {
  size_t bytes = 256u << 20; size_t n = bytes / 16;
  float4 *a, *b; (void)hipMalloc(&a, bytes); (void)hipMalloc(&b, bytes);
  (void)hipMemset(a, 1, bytes); (void)hipMemset(b, 0, bytes); (void)hipDeviceSynchronize();
  for (int i = 0; i < 3; ++i) copy_kernel<<<(unsigned)((n + 255) / 256), 256>>>(a, b, n);
  (void)hipDeviceSynchronize();
  printf("copied %zu bytes per launch\n", bytes);
  return 0;
}
