// Filter transform U = G g G^T for Winograd F(2x2,3x3), gfx950.
//
// Replaces the reference's FX kernel (src/FX_m2.cu:51-91).  Arithmetic order follows
// src/FX_m2.cu:23-47 exactly (rows: (g0+g2)+-g1 then x0.5; same along columns), so the
// OPENCNN_WW_REFERENCE output is bit-identical to the reference's.
//
// HBM-bound streaming kernel: 9 floats in, 16 floats out per (c,k).
#pragma once
#include <hip/hip_runtime.h>

namespace opencnn {

// One 3x3 filter g[r*3+s] -> U[i*4+j].
__device__ __forceinline__ void fx_one(const float (&g)[9], float (&U)[16]) {
  float t[12];
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    t[0 * 3 + s] = g[s];
    t[1 * 3 + s] = 0.5f * ((g[s] + g[6 + s]) + g[3 + s]);
    t[2 * 3 + s] = 0.5f * ((g[s] + g[6 + s]) - g[3 + s]);
    t[3 * 3 + s] = g[6 + s];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    U[i * 4 + 0] = t[i * 3 + 0];
    U[i * 4 + 1] = 0.5f * ((t[i * 3 + 0] + t[i * 3 + 2]) + t[i * 3 + 1]);
    U[i * 4 + 2] = 0.5f * ((t[i * 3 + 0] + t[i * 3 + 2]) - t[i * 3 + 1]);
    U[i * 4 + 3] = t[i * 3 + 2];
  }
}

// Read one filter.  CRSK: w[(c*9+i)*K + k] (k contiguous across lanes).
// KCRS: w[(k*C+c)*9 + i].
template <bool KCRS>
__device__ __forceinline__ void load_filter(const float* __restrict__ w, int c, int k, int C,
                                            int K, float (&g)[9]) {
  if (KCRS) {
    const float* p = w + ((size_t)k * C + c) * 9;
#pragma unroll
    for (int i = 0; i < 9; ++i) g[i] = p[i];
  } else {
    const float* p = w + (size_t)c * 9 * K + k;
#pragma unroll
    for (int i = 0; i < 9; ++i) g[i] = p[(size_t)i * K];
  }
}

// Reference layout Ww[c][p][k].  grid (ceil(K/256), C), block 256: thread = one (c,k).
template <bool KCRS>
__global__ void __launch_bounds__(256) fx_reference_layout(const float* __restrict__ w,
                                                           float* __restrict__ Ww, int K,
                                                           int C) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  const int c = blockIdx.y;
  if (k >= K) return;
  float g[9], U[16];
  load_filter<KCRS>(w, c, k, C, K, g);
  fx_one(g, U);
  float* o = Ww + (size_t)c * 16 * K + k;
#pragma unroll
  for (int p = 0; p < 16; ++p) o[(size_t)p * K] = U[p];
}

// MFMA-operand layout read by the fused kernel:
//   Usw[kg][q][p/2][h][k32][p%2][s],  k = kg*32 + k32,  c = 4*q + 2*s + h
// so that lane (h*32 + k32) of a wave fetches, with one 16-byte load per pair of positions
// (p, p+1), the A operands of two consecutive v_mfma_f32_32x32x2_f32 steps (channels 4q+h and
// 4q+2+h) of both positions.
// Thread = (k, q, h): transforms the two channels c = 4q+h and 4q+2+h and writes float4.
// grid (ceil(K/128), Cpad/4), block 256 = 2 h x 128 k.
//
// Shapes the reference does not take (K not a multiple of 32, C not a multiple of 8) are
// padded here: the layout covers Kpad = 32*ceil(K/32) filters and Cpad = 8*ceil(C/8) channels,
// and the filters / channels that do not exist are written as zeros, so the fused kernel needs
// no special case in its reduction.
template <bool KCRS>
__global__ void __launch_bounds__(256) fx_mfma_layout(const float* __restrict__ w,
                                                      float* __restrict__ Usw, int K, int C) {
  const int h = threadIdx.x >> 7;
  const int k = blockIdx.x * 128 + (threadIdx.x & 127);
  const int q = blockIdx.y;
  if (k >= ((K + 31) & ~31)) return;
  float U0[16], U1[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) U0[p] = U1[p] = 0.0f;
  if (k < K) {
    float g[9];
    if (4 * q + h < C) {
      load_filter<KCRS>(w, 4 * q + h, k, C, K, g);
      fx_one(g, U0);
    }
    if (4 * q + 2 + h < C) {
      load_filter<KCRS>(w, 4 * q + 2 + h, k, C, K, g);
      fx_one(g, U1);
    }
  }
  const int kg = k >> 5, k32 = k & 31;
  float4* o = reinterpret_cast<float4*>(Usw) +
              (((size_t)kg * gridDim.y + q) * 8) * 64 + h * 32 + k32;
#pragma unroll
  for (int p = 0; p < 16; p += 2) o[(size_t)(p >> 1) * 64] = make_float4(U0[p], U1[p], U0[p + 1], U1[p + 1]);
}

// Reduced-precision MFMA-operand layout read by the fp16 / bf16 fused kernel:
//   Uh[kg][chunk][p][h][k32][e] (2-byte elements),  k = kg*32 + k32,  c = 16*chunk + 8*h + e
// so that lane (h*32 + k32) of a wave fetches, with one 16-byte load per position p, the A
// operand of one v_mfma_f32_32x32x16_{f16,bf16} (16 input channels).  U is computed in fp32 in
// the reference's order and rounded to nearest-even once.
// grid (Kpad/64, ceil(C/16)), block 256 = 64 k x 2 h x 2 halves of 4 channels.  The layout covers
// Kpad = 64*ceil(K/64) filters (whole pairs of 32-wide groups, the smallest workgroup of the
// fused kernel) and 16*ceil(C/16) channels; filters / channels that do not exist are zeros.
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v2b __attribute__((ext_vector_type(2)));
typedef float v2fx __attribute__((ext_vector_type(2)));

template <bool BF16>
__device__ __forceinline__ unsigned pack_pair(float lo, float hi) {
  v2fx f = {lo, hi};
  if (BF16) return __builtin_bit_cast(unsigned, __builtin_convertvector(f, v2b));
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f, v2h));
}

// One thread: filter k, four consecutive channels (a quarter of a 16-channel chunk), all 16
// positions; 8 bytes per position of the lane's 16-byte MFMA operand.  A workgroup covers 64
// filters of one chunk.
template <bool KCRS, bool BF16>
__global__ void __launch_bounds__(256) fx_mfma_layout_h16(const float* __restrict__ w,
                                                          uint2* __restrict__ Uh, int K, int C) {
  const int k = blockIdx.x * 64 + (threadIdx.x & 63);
  const int h = (threadIdx.x >> 6) & 1;   // which 8 channels of the chunk: the operand's lane half
  const int half = threadIdx.x >> 7;      // which 4 of those 8
  const int chunk = blockIdx.y;
  float U[4][16];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int c = 16 * chunk + 8 * h + 4 * half + e;
    if (k < K && c < C) {
      float g[9];
      load_filter<KCRS>(w, c, k, C, K, g);
      fx_one(g, U[e]);
    } else {
#pragma unroll
      for (int p = 0; p < 16; ++p) U[e][p] = 0.0f;
    }
  }
  const int kg = k >> 5, k32 = k & 31;
  uint2* o = Uh + ((((size_t)kg * gridDim.y + chunk) * 16) * 64 + h * 32 + k32) * 2 + half;
#pragma unroll
  for (int p = 0; p < 16; ++p)
    o[(size_t)p * 128] = make_uint2(pack_pair<BF16>(U[0][p], U[1][p]), pack_pair<BF16>(U[2][p], U[3][p]));
}

}  // namespace opencnn
