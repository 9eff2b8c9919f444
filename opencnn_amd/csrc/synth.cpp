// Seeded synthetic tensors for tests, the bench and the wgrad CLI (host code).
//
// The reference fills its tensors with curand_uniform seeded from clock64()
// (src/openCNN_winograd.cu:127-145), which cannot be reproduced.  Here every element is a
// pure function of (seed, LOGICAL coordinate), so the NCHW / CHWN views of an input and the
// KCRS / CRSK views of a filter hold the same numbers, the relation the reference builds
// with its data_cpy transposes (src/openCNN_winograd.cu:147-153,230,235).
#include "../../include/opencnn_amd.h"
#include "../../include/opencnn_amd_bench.h"

#include <cmath>
#include <cstdint>

namespace {

inline uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// 24 random bits -> [0,1)
inline double u01(uint64_t bits) { return (double)(bits >> 40) * (1.0 / 16777216.0); }

inline float draw(uint64_t seed, uint64_t idx, int dist, double p0, double p1) {
  const uint64_t a = splitmix64(seed ^ (idx * 0xD1342543DE82EF95ull));
  if (dist == OPENCNN_DIST_UNIFORM) return (float)(p0 + (p1 - p0) * u01(a));
  const uint64_t b = splitmix64(a);
  const double u1 = ((double)(a >> 40) + 1.0) * (1.0 / 16777216.0);  // (0,1]
  const double u2 = u01(b);
  const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
  return (float)(p0 + p1 * z);
}

}  // namespace

extern "C" {

int opencnn_synth_input(float* dst, int n, int c, int h, int w, int layout,
                        unsigned long long seed, int dist, double p0, double p1) {
  if (!dst || n <= 0 || c <= 0 || h <= 0 || w <= 0) return 1;
  if (layout != OPENCNN_INPUT_CHWN && layout != OPENCNN_INPUT_NCHW) return 1;
  if (dist != OPENCNN_DIST_UNIFORM && dist != OPENCNN_DIST_NORMAL) return 1;
#pragma omp parallel for collapse(2) schedule(static)
  for (int ic = 0; ic < c; ++ic)
    for (int ih = 0; ih < h; ++ih)
      for (int iw = 0; iw < w; ++iw)
        for (int in = 0; in < n; ++in) {
          const uint64_t logical = (((uint64_t)in * c + ic) * h + ih) * w + iw;  // NCHW
          const size_t at = layout == OPENCNN_INPUT_CHWN
                                ? (((size_t)ic * h + ih) * w + iw) * n + in
                                : (size_t)logical;
          dst[at] = draw(seed, logical, dist, p0, p1);
        }
  return 0;
}

int opencnn_synth_filter(float* dst, int k, int c, int layout, unsigned long long seed,
                         int dist, double p0, double p1) {
  if (!dst || k <= 0 || c <= 0) return 1;
  if (layout != OPENCNN_FILTER_CRSK && layout != OPENCNN_FILTER_KCRS) return 1;
  if (dist != OPENCNN_DIST_UNIFORM && dist != OPENCNN_DIST_NORMAL) return 1;
#pragma omp parallel for schedule(static)
  for (int ic = 0; ic < c; ++ic)
    for (int rs = 0; rs < 9; ++rs)
      for (int ik = 0; ik < k; ++ik) {
        const uint64_t logical = ((uint64_t)ik * c + ic) * 9 + rs;  // KCRS
        const size_t at = layout == OPENCNN_FILTER_CRSK ? ((size_t)ic * 9 + rs) * k + ik
                                                        : (size_t)logical;
        dst[at] = draw(seed, logical, dist, p0, p1);
      }
  return 0;
}

}  // extern "C"
