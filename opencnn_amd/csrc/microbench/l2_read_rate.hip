// Probe: how fast the compute units of gfx950 can read data that sits in L2 but not in their L1 -
// the roof over the fused fp16 / bf16 kernels, whose workgroups stream 96 KB of operands per
// 16-channel unit (64 KB of transformed filters that every compute unit reads at the same time,
// 32 KB of patches of its own) and use each byte once.
// One workgroup per compute unit; every wave keeps 16 loads of 16 bytes per lane in flight and
// walks through a region that is larger than L1 (32 KB) and fits L2 (4 MB per XCD):
//   shared   all workgroups read the same 1 MB, at the same time (the filters' pattern)
//   private  every workgroup reads 96 KB of its own (32 compute units of an XCD: 3 MB)
//   mixed    two loads of three shared, one private (the kernels' mix)
// Prints a table: waves per compute unit, pattern, TB/s over all compute units, bytes per clock
// and compute unit at the clock the run sustained.  No arguments.
// Build: make -C opencnn_amd/csrc microbench.
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

typedef unsigned v4u __attribute__((ext_vector_type(4)));

enum Pattern { kShared, kPrivate, kMixed };
constexpr unsigned kSharedBytes = 1u << 20, kPrivateBytes = 96u << 10;

template <int PATTERN>
__global__ void __launch_bounds__(1024) stream(const v4u* shared_src, const v4u* private_src, v4u* sink, int rounds,
                                               long long* clocks) {
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const v4u* mine = private_src + (size_t)blockIdx.x * (kPrivateBytes / 16);
  v4u acc = 0;
  const long long c0 = clock64();
  for (int r = 0; r < rounds; ++r) {
    v4u v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      // 1 KB per wave instruction, the waves of a workgroup side by side, 16 KB per wave and round
      const unsigned step = (unsigned)r * waves * 16 + wave * 16 + k;
      const bool from_private = PATTERN == kPrivate || (PATTERN == kMixed && k % 3 == 2);
      if (from_private)
        v[k] = mine[(step * 64 + lane) % (kPrivateBytes / 16)];
      else
        v[k] = shared_src[(step * 64 + lane) % (kSharedBytes / 16)];
    }
#pragma unroll
    for (int k = 0; k < 16; ++k) acc ^= v[k];
  }
  const long long c1 = clock64();
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[threadIdx.x] = acc;  // keeps the loads alive
  if (threadIdx.x == 0 && blockIdx.x == 0) *clocks = c1 - c0;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  v4u *shared_src, *private_src, *sink;
  long long* clocks;
  CHECK(hipMalloc(&shared_src, kSharedBytes));
  CHECK(hipMalloc(&private_src, (size_t)kPrivateBytes * cus));
  CHECK(hipMalloc(&sink, 1024 * sizeof(v4u)));
  CHECK(hipHostMalloc(&clocks, sizeof(long long)));
  CHECK(hipMemset(shared_src, 1, kSharedBytes));
  CHECK(hipMemset(private_src, 2, (size_t)kPrivateBytes * cus));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  printf("%d compute units\n", cus);
  printf("%-6s %-8s %10s %14s %12s\n", "waves", "pattern", "TB/s", "B/clk/CU@2.2GHz", "us/launch");
  const char* names[] = {"shared", "private", "mixed"};
  for (int waves : {4, 8, 16}) {
    for (int pattern = 0; pattern < 3; ++pattern) {
      const int rounds = 4096 / waves;  // 64 MB per compute unit and launch
      auto launch = [&] {
        if (pattern == kShared) stream<kShared><<<cus, waves * 64>>>(shared_src, private_src, sink, rounds, clocks);
        if (pattern == kPrivate) stream<kPrivate><<<cus, waves * 64>>>(shared_src, private_src, sink, rounds, clocks);
        if (pattern == kMixed) stream<kMixed><<<cus, waves * 64>>>(shared_src, private_src, sink, rounds, clocks);
      };
      for (int i = 0; i < 3; ++i) launch();
      CHECK(hipDeviceSynchronize());
      const int reps = 10;
      CHECK(hipEventRecord(e0));
      for (int i = 0; i < reps; ++i) launch();
      CHECK(hipEventRecord(e1));
      CHECK(hipEventSynchronize(e1));
      CHECK(hipGetLastError());
      float ms = 0;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      const double us = ms * 1e3 / reps;
      const double bytes = (double)cus * rounds * waves * 16 * 1024;
      printf("%-6d %-8s %10.2f %14.1f %12.1f\n", waves, names[pattern], bytes / us * 1e-6, bytes / cus / (us * 2200.0), us);
    }
  }
  return 0;
}
