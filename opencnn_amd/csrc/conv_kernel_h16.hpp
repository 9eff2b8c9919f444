// Fused Winograd F(2x2,3x3) forward convolution with fp16 / bf16 GEMM operands, gfx950.
//
// Same tiling as the fp32 LDS kernel (conv_kernel_f32.hpp: one wave = 32 filters x 32 batch
// elements of one spatial tile for all 16 positions, fp32 accumulators, workgroup = KW filter
// groups sharing a column tile), with the 16 batched GEMMs on
// v_mfma_f32_32x32x16_{f16,bf16}: one MFMA per position consumes 16 input channels.
// Transforms stay in fp32; the transformed input V and the transformed filter U are rounded
// to nearest-even once, on their way into LDS / into the workspace.  The reference has no
// such path (it is fp32 only); the oracle's quantised restatement is the parity target.
//
// Per 16-channel chunk and column tile there are 16 x 32 patches to transform; the KW waves
// split them.  A lane transforms two ADJACENT channels of one batch element and packs the two
// results of every position into one dword, written to
//     Vh[buf][p][h][q][n]      c = 16*chunk + 8*h + 2*q + {0,1}
// (32 consecutive dwords per (p,h,q): conflict-free).  As B operand, lane (h, n) needs the four
// dwords q = 0..3 of its (p, h, n): two ds_read2_b32 per position.
#pragma once
#include <hip/hip_runtime.h>

#include "conv_kernel_f32.hpp"

namespace opencnn {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));
typedef _Float16 v2hh __attribute__((ext_vector_type(2)));
typedef __bf16 v2bb __attribute__((ext_vector_type(2)));
typedef unsigned int v4u32 __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ unsigned pack_rne(float lo, float hi) {
  v2f f = {lo, hi};
  if (BF16) return __builtin_bit_cast(unsigned, __builtin_convertvector(f, v2bb));
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f, v2hh));
}

template <bool BF16>
__device__ __forceinline__ v16f mfma16(v4u32 a, v4u32 b, v16f c) {
  if (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b, a), __builtin_bit_cast(v8b, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

// KW waves share a column tile; CW = 4/KW column tiles per workgroup.  C % 16 == 0.
//
// Pipeline (chunk = 16 channels, one MFMA per position):
//   during chunk i   the wave transforms its share of chunk i+2 into LDS buffer (i+2)%3 and
//                    issues the patch loads of chunk i+3;
//   per position p   MFMA(acc[p], u[p], v[p]) of chunk i, then u[p] and v[p] are refilled in
//                    place with chunk i+1 (global load / LDS read): single operand buffers that
//                    roll one chunk ahead, which is what the 256 arch VGPRs allow next to the
//                    256 accumulators;
//   end of chunk i   workgroup barrier, publishing chunk i+2's V.
// Chunk i+1's V was published by the barrier that ended chunk i-1, so the rolling reads need
// no further synchronisation; three LDS buffers keep the writes of chunk i+2 away from them.
//
// RAGGED = shapes outside N % 32 == 0, C % 16 == 0, K % 64 == 0, handled as in the fp32 kernels:
// groups and chunks rounded up (a.kgroups counts whole pairs of filter groups), lanes whose
// batch element does not exist read zeros and store nothing, the four-channel window of the
// last chunk ends with the tensor, filters and channels past K / C are zeros in the
// transformed filter, rows past K are not stored.
template <int KW, bool BF16, bool RAGGED = false>
__global__ void __launch_bounds__(256) wino_h16_fused_lds(ConvArgs a) {
  constexpr int CW = 4 / KW;
  constexpr int SPW = 4 / KW;  // channel-quads (slots) of a chunk transformed by one wave
  constexpr int kBufDwords = 16 * 2 * 4 * 32;
  extern __shared__ unsigned ldsu[];  // [CW][3][16][2][4][32] dwords
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kw = wave % KW, cw = wave / KW;
  const int L = logical_block();
  if (L >= a.nblocks) return;  // whole workgroup
  const int cg_raw = (L % a.colblocks) * CW + cw;
  const bool live = cg_raw < a.colgroups;
  // A workgroup whose last column tile does not exist keeps those waves busy on a copy of
  // the last real one (they must take part in the barriers) and drops their stores.
  const int cg = live ? cg_raw : a.colgroups - 1;
  WaveTile w;
  decode_tile<RAGGED>(a, (L / a.colblocks) * KW + kw, cg, lane, w);
  const int nl = lane & 31, j = lane >> 5;
  const size_t HWN = (size_t)a.H * a.W * a.N;

  // The transform lane (j, n) owns the adjacent channels 4*slot + 2*j + {0,1} of a chunk.
  // voff = byte offsets of the 4x4 patch of the first of them inside a window of x that
  // starts at channel 16*chunk + 4*slot; the second channel is one channel stride further.
  int voff[16];
#pragma unroll
  for (int e = 0; e < 16; ++e)
    voff[e] = w.voff[e] == kOutOfRange
                  ? kOutOfRange
                  : w.voff[e] + (int)((2 * j - w.hsel) * (long long)HWN * 4);  // w.voff carries hsel channels
  const int chan_bytes = (int)(HWN * 4);

  unsigned* vl = ldsu + cw * (3 * kBufDwords);
  unsigned* wl = vl + nl;                              // writes: + ((p*2 + h)*4 + q)*32
  const unsigned* rl = vl + (lane >> 5) * (4 * 32) + nl;  // B operand of lane (h, n): + p*256 + q*32
  auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  v16f acc[16];
#pragma unroll
  for (int p = 0; p < 16; ++p)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[p][r] = 0.0f;

  v4u32 u[16];          // A operands, rolling one chunk ahead
  v4u32 v[16];          // B operands, rolling one chunk ahead
  float d[SPW][2][16];  // this lane's patches (a channel pair per slot), in flight

  const int chunks = RAGGED ? (a.C + 15) >> 4 : a.C >> 4;
  const unsigned u_bytes = (unsigned)((size_t)chunks * 16 * 16 * (a.kgroups * 32) * 2);
  auto load_u1 = [&](int p, int chunk) {
    // past the last chunk: an empty descriptor, the load returns zeros without touching memory
    const __amdgpu_buffer_rsrc_t ru = make_rsrc(a.usw, chunk < chunks ? u_bytes : 0u);
    const int soff = __builtin_amdgcn_readfirstlane((w.kg * chunks + chunk) * (16 * 64 * 16));
    u[p] = __builtin_amdgcn_raw_buffer_load_b128(ru, lane * 16 + p * 1024, soff, 0);
  };
  auto load_patches = [&](int chunk) {
    const int ch = chunk < chunks ? chunk : chunks - 1;  // past the end: reload, unused
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      const int c0 = __builtin_amdgcn_readfirstlane(16 * ch + 4 * (kw * SPW + s));
      int window = 4;  // channels behind the descriptor
      if (RAGGED) window = a.C - c0 < 0 ? 0 : (a.C - c0 < 4 ? a.C - c0 : 4);
      const __amdgpu_buffer_rsrc_t r = make_rsrc(a.x + (size_t)c0 * HWN, (unsigned)(window * HWN * sizeof(float)));
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        d[s][0][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff[e], 0, 0));
        d[s][1][e] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(r, voff[e] == kOutOfRange ? kOutOfRange : voff[e] + chan_bytes, 0, 0));
      }
    }
  };
  auto transform_to_lds = [&](int bufofs) {
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      float t0[16], t1[16];
      input_transform(d[s][0], t0);
      input_transform(d[s][1], t1);
      const int slot = kw * SPW + s;     // channels 4*slot .. 4*slot+3 of the chunk
      const int h = slot >> 1;           // which half of the 16 channels
      const int q = 2 * (slot & 1) + j;  // dword inside the lane's 8-channel operand
#pragma unroll
      for (int p = 0; p < 16; ++p) wl[bufofs + ((p * 2 + h) * 4 + q) * 32] = pack_rne<BF16>(t0[p], t1[p]);
    }
  };
  auto read_v1 = [&](int p, int bufofs) {
    const unsigned* r = rl + bufofs + p * (2 * 4 * 32);
    v[p] = v4u32{r[0], r[32], r[64], r[96]};
  };

  // prologue: chunks 0 and 1 -> buffers 0 and 1, chunk 2 patches in flight, chunk 0 operands
  load_patches(0);
  transform_to_lds(0);
  load_patches(1);
  transform_to_lds(kBufDwords);
  load_patches(2);
  lds_barrier();
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    load_u1(p, 0);
    read_v1(p, 0);
  }

  int b1 = kBufDwords, b2 = 2 * kBufDwords;  // buffers of chunk i+1 and i+2
  for (int i = 0; i < chunks; ++i) {
    __builtin_amdgcn_sched_barrier(0);
    transform_to_lds(b2);
    __builtin_amdgcn_sched_barrier(0);
    load_patches(i + 3);
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      acc[p] = mfma16<BF16>(u[p], v[p], acc[p]);
      load_u1(p, i + 1);
      read_v1(p, b1);
    }
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    const int b0 = b1 == 0 ? 2 * kBufDwords : b1 - kBufDwords;  // buffer of the finished chunk
    b1 = b2;
    b2 = b0;
  }
  if (live) store_tile<kStorePlain, RAGGED>(a, w, acc);
}

}  // namespace opencnn
