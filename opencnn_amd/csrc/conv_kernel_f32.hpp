// Fused Winograd F(2x2,3x3) forward convolution, fp32 operands on fp32 MFMA, gfx950.
//
// Replaces the reference's Winograd_kernel and its helpers
// (src/convolutionForward_32x64x8.cu:53-262, src/outer_product_suffle.cuh,
// src/store_and_transform_output_optSTS64.cuh).  Same mathematics, different machine
// mapping:
//
//  * GEMM view.  For each of the 16 Winograd positions p:
//        M[p][k][(tile,n)] = sum_c U[p][k][c] * V[p][c][(tile,n)]
//    k sits on the MFMA row side (A operand = transformed filter U), the batch index n
//    on the column side (B operand = transformed input V).  One wave owns a
//    32 k x 32 n tile of ONE spatial tile for ALL 16 positions: 16 accumulators of
//    v_mfma_f32_32x32x2_f32 = 256 accumulator registers, one wave per SIMD.
//  * Input path.  Lane (h, n) (h = lane/32, n = lane%32) loads the 4x4 patch of channel
//    c0+h for batch element n0+n straight from CHWN memory: every load instruction is two
//    fully used 128-byte rows.  The patch is transformed (B^T d B, 32 add/sub) in
//    registers and IS the B operand of the MFMA: the transformed input never visits LDS.
//    Zero padding is implicit: out-of-image patch elements use a buffer offset beyond
//    num_records, for which buffer loads return 0 without touching memory
//    (the reference's bit masks, src/convolutionForward_32x64x8.cu:179-183).
//  * Output path.  Because a lane holds all 16 positions of its (k, n) elements, the
//    output transform A^T M A is element-wise across accumulators; the reference's four
//    rounds of shared-memory transposition
//    (src/store_and_transform_output_optSTS64.cuh:97-127) have no counterpart.  In the
//    MFMA D layout lanes 0-31 of an accumulator register are 32 consecutive n of one k,
//    so each store instruction writes two complete 128-byte rows of KHWN.
//  * Reduction order: channels ascending, two per MFMA step, fp32 accumulate
//    (the reference: one FMA per channel, ascending, src/convolutionForward_32x64x8.cu:210-257).
#pragma once
#include <hip/hip_runtime.h>

namespace opencnn {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

struct ConvArgs {
  const float* x;    // CHWN
  const float* usw;  // transformed filter, MFMA operand order (see fx_mfma_layout)
  float* y;          // KHWN
  int N, C, H, W, K;
  int tiles_h, tiles_w;  // 2x2 output tiles per image column / row
  int ngroups;           // ceil(N / 32)
  int colgroups;         // tiles_h * tiles_w * ngroups   (wave-level column tiles)
  int kgroups;           // ceil(K / 32)
  int nblocks;           // workgroup tiles: filter blocks x column blocks
  unsigned* sync;        // split-merge flags of this launch's stream (one set of g_split_sync)
  int colblocks;         // column blocks; workgroup tile T = filter block T / colblocks,
                         // column block T % colblocks (LDS kernels): an XCD's contiguous
                         // range of tiles then needs one filter block's share of Ww, which
                         // fits its L2, instead of all of it
  unsigned* status;      // status word of the flag set (host memory the GPU can write): a wave
                         // that gives up waiting for a flag stores 1 there
  unsigned spin_limit;   // polls after which a wait for a flag gives up
};

// Bounded wait for a split-merge flag.  A wave that gives up reports it in the launch's status
// word and goes on with whatever the output tensor holds (the launch's result is wrong, but
// every wave ends); the host finds the word at its next call.
__device__ __forceinline__ void wait_for_flag(const ConvArgs& a, const unsigned* flag, int lane) {
  unsigned spin = 0;
  while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 0) {
    if (++spin >= a.spin_limit) {
      if (lane == 0) __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      break;
    }
    __builtin_amdgcn_s_sleep(8);
  }
  asm volatile("" ::: "memory");  // the partial result is read after the flag, not before
}

// V = B^T d B, columns first then rows (src/convolutionForward_32x64x8.cu:59-80).
__device__ __forceinline__ void input_transform(const float (&d)[16], float (&v)[16]) {
  float t[16];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    t[0 + j] = d[0 + j] - d[8 + j];
    t[4 + j] = d[4 + j] + d[8 + j];
    t[8 + j] = d[8 + j] - d[4 + j];
    t[12 + j] = d[4 + j] - d[12 + j];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i * 4 + 0] = t[i * 4 + 0] - t[i * 4 + 2];
    v[i * 4 + 1] = t[i * 4 + 1] + t[i * 4 + 2];
    v[i * 4 + 2] = t[i * 4 + 2] - t[i * 4 + 1];
    v[i * 4 + 3] = t[i * 4 + 1] - t[i * 4 + 3];
  }
}

// Y = A^T m A (src/store_and_transform_output_optSTS64.cuh:29-51), m[i*4+j] -> o[a*2+b].
__device__ __forceinline__ void output_transform(const float (&m)[16], float (&o)[4]) {
  float a[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    a[j] = (m[j] + m[4 + j]) + m[8 + j];
    a[4 + j] = (m[4 + j] - m[8 + j]) - m[12 + j];
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    o[i * 2 + 0] = (a[i * 4 + 0] + a[i * 4 + 1]) + a[i * 4 + 2];
    o[i * 2 + 1] = (a[i * 4 + 1] - a[i * 4 + 2]) - a[i * 4 + 3];
  }
}

constexpr int kBufferFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family)
constexpr int kOutOfRange = (int)0x80000000;  // voffset no num_records can reach

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, kBufferFlags);
}

// ------------------------------------------------------------------------------------------
// Pieces shared by the kernels below.

struct WaveTile {
  int kg;        // 32-wide filter group
  int ng;        // 32-wide batch group
  int ty, tx;    // 2x2 output tile
  int hsel, nl;  // lane = hsel*32 + nl: channel parity / batch element of this lane
  int voff[16];  // byte offset of patch element (i,j) in a two-channel slab, or kOutOfRange
};

// RAGGED (here and below) = shapes outside the reference's N % 32 == 0, K % 32 == 0,
// C % 8 == 0: the groups are rounded up, lanes whose batch element does not exist read zeros
// and store nothing, channels past C read zeros on both operands, filters past K are zero
// in the transformed filter and are not stored.
template <bool RAGGED = false>
__device__ __forceinline__ void decode_tile(const ConvArgs& a, int kg, int cg, int lane, WaveTile& w) {
  const int tile = cg / a.ngroups;
  w.kg = kg;
  w.ng = cg - tile * a.ngroups;
  w.ty = tile / a.tiles_w;
  w.tx = tile - w.ty * a.tiles_w;
  w.hsel = lane >> 5;
  w.nl = lane & 31;
  const int HW = a.H * a.W;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int hh = 2 * w.ty - 1 + i, ww = 2 * w.tx - 1 + j;
      const bool ok = hh >= 0 && hh < a.H && ww >= 0 && ww < a.W &&
                      (!RAGGED || w.ng * 32 + w.nl < a.N);
      w.voff[i * 4 + j] =
          ok ? (int)(((size_t)w.hsel * HW + (size_t)hh * a.W + ww) * a.N + w.ng * 32 + w.nl) * 4
             : kOutOfRange;
    }
  }
}

// 4x4 patch of MFMA step `step` (channels 2*step + hsel); steps past the end reload the last
// slab (the data is never used; this keeps the pipeline free of branches).
// RAGGED: the slab ends with the tensor (an odd C leaves one channel in the last slab) and
// steps past the end read zeros, because the padded steps of the last chunk ARE multiplied.
template <bool RAGGED = false>
__device__ __forceinline__ void load_patch(const ConvArgs& a, const WaveTile& w, float (&d)[16], int step) {
  const size_t HWN = (size_t)a.H * a.W * a.N;
  int st, channels;
  if (RAGGED) {
    const int S = (a.C + 1) >> 1;
    st = step < S ? step : S - 1;
    channels = step < S ? (a.C - 2 * st < 2 ? a.C - 2 * st : 2) : 0;
  } else {
    const int S = a.C >> 1;
    st = step < S ? step : S - 1;
    channels = 2;
  }
  __amdgpu_buffer_rsrc_t r = make_rsrc(a.x + (size_t)st * 2 * HWN, (unsigned)(channels * HWN * sizeof(float)));
#pragma unroll
  for (int e = 0; e < 16; ++e)
    d[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, w.voff[e], 0, 0));
}

// A operands of filter quad `quad` (channels 4*quad .. 4*quad+3) for all 16 positions.
template <bool RAGGED = false>
__device__ __forceinline__ void load_u(const ConvArgs& a, const WaveTile& w, int lane, v2f (&u)[16], int quad) {
  const int Q = RAGGED ? ((a.C + 7) >> 3) * 2 : a.C >> 2;
  const int Kp = RAGGED ? (a.K + 31) & ~31 : a.K;
  const __amdgpu_buffer_rsrc_t ru = make_rsrc(a.usw, (unsigned)((size_t)Q * 4 * 16 * Kp * sizeof(float)));
  const int qd = quad < Q ? quad : Q - 1;
  const int soff = (w.kg * Q + qd) * (16 * 64 * 8);
#pragma unroll
  for (int p = 0; p < 16; p += 2) {
    const v4f pair = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(ru, lane * 16 + p * 512, soff, 0));
    u[p] = v2f{pair[0], pair[1]};
    u[p + 1] = v2f{pair[2], pair[3]};
  }
}

// Output transform and store.  Accumulator register r of lane (hsel, nl) is row
// k = 8*(r/4) + 4*hsel + r%4, column n = nl of the wave's 32x32 tile.
//   kStorePlain    write the result
//   kStorePublish  write a PARTIAL result (first half of a tile whose channel range is split
//                  between two workgroups) straight through to memory, so that a wave on
//                  another XCD (another L2) can read it without any cache-wide flush
//   kStoreMerge    read the published partial result past the caches, add, write the result
enum StoreMode { kStorePlain = 0, kStorePublish = 1, kStoreMerge = 2 };

__device__ __forceinline__ float load_through(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void store_through(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

template <StoreMode MODE, bool RAGGED = false>
__device__ __forceinline__ void store_tile(const ConvArgs& a, const WaveTile& w, const v16f (&acc)[16]) {
  const size_t HWN = (size_t)a.H * a.W * a.N;
  const bool row1 = 2 * w.ty + 1 < a.H;  // odd H: last tile row keeps only a = 0
  const bool col1 = 2 * w.tx + 1 < a.W;  // odd W: last tile column keeps only b = 0
  float* ybase = a.y + ((size_t)(2 * w.ty) * a.W + 2 * w.tx) * a.N + w.ng * 32 + w.nl;
  const size_t o1 = a.N, o2 = (size_t)a.W * a.N, o3 = o2 + a.N;
  // kStoreMerge: fetch the whole partial tile first (64 independent loads in flight at once;
  // read one by one, each uncached load would cost a full trip to memory).
  float part[MODE == kStoreMerge ? 16 : 1][4];
  if (MODE == kStoreMerge) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int k = w.kg * 32 + 8 * (r >> 2) + 4 * w.hsel + (r & 3);
      const float* yk = ybase + (size_t)k * HWN;
      part[r][0] = load_through(yk);
      part[r][1] = col1 ? load_through(yk + o1) : 0.0f;
      part[r][2] = row1 ? load_through(yk + o2) : 0.0f;
      part[r][3] = (row1 && col1) ? load_through(yk + o3) : 0.0f;
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float m[16], o[4];
#pragma unroll
    for (int p = 0; p < 16; ++p) m[p] = acc[p][r];
    output_transform(m, o);
    const int k = w.kg * 32 + 8 * (r >> 2) + 4 * w.hsel + (r & 3);
    float* yk = ybase + (size_t)k * HWN;
    if (MODE == kStoreMerge) {
#pragma unroll
      for (int q = 0; q < 4; ++q) o[q] += part[r][q];
    }
    if (RAGGED && !(k < a.K && w.ng * 32 + w.nl < a.N)) continue;
    if (MODE == kStorePublish) {
      store_through(yk, o[0]);
      if (col1) store_through(yk + o1, o[1]);
      if (row1) {
        store_through(yk + o2, o[2]);
        if (col1) store_through(yk + o3, o[3]);
      }
    } else {
      yk[0] = o[0];
      if (col1) yk[o1] = o[1];
      if (row1) {
        yk[o2] = o[2];
        if (col1) yk[o3] = o[3];
      }
    }
  }
}

// Logical block of this workgroup.  Workgroups are dealt round-robin to the 8 XCDs (one L2
// each); every XCD gets a contiguous range of logical blocks so that blocks sharing input
// columns and filters meet in one L2.
__device__ __forceinline__ int logical_block() {
  const int per_xcd = gridDim.x >> 3;
  return (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
}

// ------------------------------------------------------------------------------------------
// Kernel A: every wave transforms its own patches (no LDS, no barriers).
// Used when K is not a multiple of 64, and (RAGGED) for every shape outside the reference's
// N % 32 == 0, K % 32 == 0, C % 8 == 0.
//
// One MFMA step = two input channels.  Software pipeline, per step t (all in registers):
//   first   the 32 add/sub that turn the patch of step t+1 (loaded one step ago) into the
//           next B operands, as one burst (fp32 MFMA and fp32 VALU share the SIMD's ALUs on
//           gfx950, and every MFMA->VALU->MFMA alternation costs extra cycles);
//   then    the 16 MFMAs of step t, each followed by one or two of the loads of step t+2
//           (16 patch loads and, every other step, the 16 filter loads of the next quad).
// The scheduling barriers pin that order; left alone hipcc sinks the loads down to their
// first use to save registers, which exposes the full memory latency once per step.
template <bool RAGGED>
__global__ void __launch_bounds__(256) wino_f32_fused(ConvArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int L = logical_block();
  if (L >= a.nblocks) return;
  const int cg = (L / a.kgroups) * 4 + wave;
  if (cg >= a.colgroups) return;  // wave-uniform; this kernel has no barriers
  WaveTile w;
  decode_tile<RAGGED>(a, L % a.kgroups, cg, lane, w);

  v16f acc[16];
#pragma unroll
  for (int p = 0; p < 16; ++p)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[p][r] = 0.0f;

  v2f u[2][16];    // filter operands of the current / next quad
  float d[2][16];  // patches in flight: d[t&1] holds the patch of step t
  float v[2][16];  // B operands: v[t&1] holds the transformed patch of step t

  // prologue: patch 0 -> v[0]; patch 1 in flight in d[1]; quad 0 in u[0]
  load_u<RAGGED>(a, w, lane, u[0], 0);
  load_patch<RAGGED>(a, w, d[0], 0);
  load_patch<RAGGED>(a, w, d[1], 1);
  input_transform(d[0], v[0]);

  const int octs = RAGGED ? (a.C + 7) >> 3 : a.C >> 3;
  for (int oct = 0; oct < octs; ++oct) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int t = oct * 4 + s;
      __builtin_amdgcn_sched_barrier(0);
      input_transform(d[(s + 1) & 1], v[(s + 1) & 1]);
      // Anchor: the next B operands must exist when this region ends, or LLVM sinks the
      // transform into the next step, in front of the MFMAs that need it.
#pragma unroll
      for (int p = 0; p < 16; ++p) asm volatile("" : "+v"(v[(s + 1) & 1][p]));
      __builtin_amdgcn_sched_barrier(0);
      // d[t&1] was consumed by the transform of the previous step: refill it with step t+2
      load_patch<RAGGED>(a, w, d[s & 1], t + 2);
      if (s == 0) load_u<RAGGED>(a, w, lane, u[1], 2 * oct + 1);
      if (s == 2) load_u<RAGGED>(a, w, lane, u[0], 2 * oct + 2);
#pragma unroll
      for (int p = 0; p < 16; ++p)
        acc[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(u[s >> 1][p][s & 1], v[s & 1][p], acc[p], 0, 0, 0);
      // Loads are spread behind the MFMAs (a burst of them stalls the wave on the vector
      // memory address FIFO while the matrix pipe idles).
#pragma unroll
      for (int p = 0; p < 16; ++p) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                        // one MFMA
        if (s & 1)
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one of the 16 patch loads
        else
          __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);  // patch load + filter load
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  store_tile<kStorePlain, RAGGED>(a, w, acc);
}

// ------------------------------------------------------------------------------------------
// Kernel B: the KW waves of a workgroup that share one column tile (same spatial tile and
// batch group, KW different filter groups) split the input transform between them and
// exchange the transformed patches through LDS.
//
// Why: on gfx950 the fp32 MFMA and the fp32 VALU share the SIMD's ALUs (no co-execution:
// every v_add/v_sub costs 4+ MFMA cycles), so the 32 add/sub per step of kernel A are paid in
// full.  Sharing them KW ways cuts that to 32/KW; the LDS traffic that replaces them runs on
// the LDS pipe in the shadow of the MFMAs.
//
// Workgroup = KW x CW waves (KW*CW = 4): wave = cw*KW + kw owns filter group kb*KW+kw and
// column tile cb*CW+cw.  A chunk = 8 channels = 4 MFMA steps.  Wave kw transforms the steps
// kw*SPW .. kw*SPW+SPW-1 (SPW = 4/KW) of every chunk for its column tile and writes them to
//     V[cw][buf][step][p][lane]          (64 floats = one B operand register per wave)
// in exactly the lane order in which all KW waves read them back as MFMA B operands, so
// every LDS access is 256 contiguous bytes per wave: free of bank conflicts by construction.
// Double buffered: chunk i reads buf i&1 while the transforms of chunk i+1 fill the other;
// one workgroup barrier per chunk.
//
// BALANCED = true turns the kernel into a persistent one: gridDim.x workgroups (one per CU)
// share nblocks*chunks chunk-units evenly; a workgroup walks a contiguous range of units, so
// its first and last tile may be covered only in part.  Without it 784 equal tiles on 256 CUs
// take 4 rounds for 3.06 rounds of work.  The host only selects it when nblocks >= gridDim.x,
// which bounds every tile to at most TWO contributing workgroups; their partial outputs are
// merged through the output tensor itself: the wave that arrives first (atomic ticket) stores
// its partial result and raises a flag, the second adds its own on top.  a+b == b+a in fp32,
// so the result does not depend on the arrival order.  The second wave only ever waits for a
// wave that is already running its epilogue, never for one that has yet to be scheduled.
constexpr int kMaxBalancedBlocks = 1024;
// [set][boundary between workgroups b and b+1][wave] -> {ticket, flag}; zero between launches
// (the second contributor clears its pair).  Launches that may overlap in time must not share a
// set: the host hands one to every stream that launches and to every stream capture (api.hip).
constexpr int kEagerSets = 32;  // streams that launch directly
constexpr int kGraphSets = 16;  // launches recorded into HIP graphs
constexpr int kSyncSets = kEagerSets + kGraphSets;
constexpr int kSyncWords = kMaxBalancedBlocks * 4 * 2;
// (one more set at the end for launches that cut no tile: they are given it and never touch it)
static __device__ unsigned g_split_sync[(kSyncSets + 1) * kSyncWords];

template <int KW, bool BALANCED, bool RAGGED = false>
__global__ void __launch_bounds__(256) wino_f32_fused_lds(ConvArgs a) {
  constexpr int CW = 4 / KW;
  constexpr int SPW = 4 / KW;
  extern __shared__ float lds[];  // [CW][2][4][16][64]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kw = wave % KW, cw = wave / KW;
  const int L = logical_block();
  static_assert(!(BALANCED && RAGGED), "the merge of a cut tile is not predicated");
  const int chunks = RAGGED ? (a.C + 7) >> 3 : a.C >> 3;

  // chunk-units [unit, end) of this workgroup; unit = tile * chunks + chunk
  long long unit, end;
  if (BALANCED) {
    const long long total = (long long)a.nblocks * chunks;
    unit = total * L / gridDim.x;
    end = total * (L + 1) / gridDim.x;
  } else {
    if (L >= a.nblocks) return;  // whole workgroup
    unit = (long long)L * chunks;
    end = unit + chunks;
  }

  float* vl = lds + cw * (2 * 4 * 16 * 64) + lane;
  auto vaddr = [&](int buf, int step, int p) { return vl + ((buf * 4 + step) * 16 + p) * 64; };
  // LDS writes of this wave done, then workgroup barrier.  Deliberately not __syncthreads():
  // that would also wait for the global loads in flight (vmcnt(0)) once per chunk.
  auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  while (unit < end) {
    const int T = (int)(unit / chunks);
    const int c0 = (int)(unit - (long long)T * chunks);
    const int c1 = (end - unit) < (long long)(chunks - c0) ? c0 + (int)(end - unit) : chunks;
    unit += c1 - c0;

    const int cg_raw = (T % a.colblocks) * CW + cw;
    const bool live = cg_raw < a.colgroups;
    // A workgroup whose last column tile does not exist keeps those waves busy on a copy of
    // the last real one (they must take part in the barriers) and drops their stores.
    const int cg = live ? cg_raw : a.colgroups - 1;
    WaveTile w;
    decode_tile<RAGGED>(a, (T / a.colblocks) * KW + kw, cg, lane, w);

    v16f acc[16];
#pragma unroll
    for (int p = 0; p < 16; ++p)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[p][r] = 0.0f;

    v2f u[2][16];      // filter operands of the current / next quad
    float d[SPW][16];  // this wave's share of the next chunk's patches, in flight
    float v[2][16];    // B operands of the current / next step

    auto transform_to_lds = [&](int buf) {
#pragma unroll
      for (int j = 0; j < SPW; ++j) {
        float t[16];
        input_transform(d[j], t);
#pragma unroll
        for (int p = 0; p < 16; ++p) *vaddr(buf, kw * SPW + j, p) = t[p];
      }
    };
    auto load_patches = [&](int chunk) {
#pragma unroll
      for (int j = 0; j < SPW; ++j) load_patch<RAGGED>(a, w, d[j], chunk * 4 + kw * SPW + j);
    };
    auto read_v = [&](float (&dst)[16], int buf, int step) {
#pragma unroll
      for (int p = 0; p < 16; ++p) dst[p] = *vaddr(buf, step, p);
    };

    // prologue: chunk c0 -> buf 0; chunk c0+1 patches in flight; first quad in u[0].
    // (All reads of the previous tile's LDS data precede its last barrier, so buf 0 is free.)
    load_u<RAGGED>(a, w, lane, u[0], 2 * c0);
    load_patches(c0);
    transform_to_lds(0);
    load_patches(c0 + 1);
    lds_barrier();
    read_v(v[0], 0, 0);

    for (int i = c0; i < c1; ++i) {
      const int buf = (i - c0) & 1;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        __builtin_amdgcn_sched_barrier(0);
        if (s == 0) transform_to_lds(buf ^ 1);  // chunk i+1: one VALU burst, then its LDS writes
        __builtin_amdgcn_sched_barrier(0);
        if (s == 0) load_u<RAGGED>(a, w, lane, u[1], 2 * i + 1);
        if (s == 2) load_u<RAGGED>(a, w, lane, u[0], 2 * i + 2);
        // patches of chunk i+2: 16 loads per owned step; with two owned steps (KW = 2) the second
        // batch goes behind the MFMAs of step 3, which has no other loads
        if (s == 1) load_patch<RAGGED>(a, w, d[0], (i + 2) * 4 + kw * SPW);
        if (s == 3 && SPW == 2) load_patch<RAGGED>(a, w, d[1], (i + 2) * 4 + kw * SPW + 1);
        if (s < 3) read_v(v[(s + 1) & 1], buf, s + 1);
#pragma unroll
        for (int p = 0; p < 16; ++p)
          acc[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(u[s >> 1][p][s & 1], v[s & 1][p], acc[p], 0, 0, 0);
        // One memory instruction behind every MFMA.  Issued as a burst, the loads fill the
        // vector-memory address FIFO and the wave (the only one on its SIMD) sits on a load
        // instead of feeding the matrix pipe; spread out, each is absorbed in an MFMA's shadow.
#pragma unroll
        for (int p = 0; p < 16; ++p) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
          if (s != 3 || SPW == 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
          if (s != 3 && (p & 1)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      lds_barrier();
      read_v(v[0], buf ^ 1, 0);
    }

    if (!live) continue;
    if (!BALANCED || (c0 == 0 && c1 == chunks)) {
      store_tile<kStorePlain, RAGGED>(a, w, acc);
      continue;
    }
    // Partial tile: the other part belongs to the previous (c0 > 0) or next workgroup.
    // All traffic of the hand-over (partial result, ticket, flag) goes straight to memory with
    // per-access system-scope policy; no fence is used, because a device-scope fence writes
    // back / invalidates the whole L2 of the XCD under the other 31 workgroups' feet.
    unsigned* sync = a.sync + ((c0 > 0 ? L - 1 : L) * 4 + wave) * 2;
    unsigned ticket = 0;
    if (lane == 0) ticket = __hip_atomic_fetch_add(sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    ticket = __builtin_amdgcn_readfirstlane(ticket);
    if (ticket == 0) {
      store_tile<kStorePublish>(a, w, acc);
      // every write-through store of this wave acknowledged, then raise the flag
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (lane == 0) __hip_atomic_store(sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    } else {
      // The first contributor holds ticket 0 and is in its epilogue; bounded wait all the same.
      wait_for_flag(a, sync + 1, lane);
      store_tile<kStoreMerge>(a, w, acc);
      if (lane == 0) {
        __hip_atomic_store(sync, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(sync + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Kernel C: kernel B as ONE continuous software pipeline over the workgroup's whole range of
// (tile, chunk) units.  In kernel B every tile (or part of a tile) starts with a prologue whose
// first loads nobody prefetched (about 2 us of idle matrix pipe per tile, 8-10 % of a tile of
// 8-16 chunks).  Here the loads run two units ahead of the MFMAs ACROSS tile boundaries: while
// the last chunk of a tile is being multiplied, the first chunks of the next tile are already
// being loaded, transformed and published, so a tile boundary costs the output transform and
// the zeroing of the accumulators, nothing else.
//
// Three cursors walk the unit range: P (patch loads, two units ahead of the MFMAs), Q (first
// filter quad, one unit ahead) and M (the MFMAs and the epilogue).  Q and M only need
// wave-uniform tile coordinates.  P addresses its 16 patch elements in one of two ways:
//   SCALAR_PATCH = false  16 per-lane byte offsets (WaveTile::voff), re-decoded on a tile switch;
//   SCALAR_PATCH = true   one per-lane base offset plus 16 wave-uniform scalar offsets, the zero
//                         padding being a per-element choice between the real buffer descriptor
//                         and an empty one (a load through it returns 0 without touching memory).
// Which one hipcc turns into the faster loop depends on the register pressure of the
// instantiation (measured: scalar for KW = 4, per-lane for KW = 2).
struct TileState {
  int kg, ng, ty, tx;  // wave-uniform
  int live;            // 0: this wave's column tile does not exist (stores dropped)
};

template <int KW>
__device__ __forceinline__ int column_tile_of(const ConvArgs& a, int T, int cw, int& live) {
  constexpr int CW = 4 / KW;
  const int cg_raw = (T % a.colblocks) * CW + cw;
  live = cg_raw < a.colgroups;
  // A workgroup whose last column tile does not exist keeps those waves busy on a copy of
  // the last real one (they must take part in the barriers) and drops their stores.
  return live ? cg_raw : a.colgroups - 1;
}

template <int KW>
__device__ __forceinline__ void decode_state(const ConvArgs& a, int T, int kw, int cw, TileState& t) {
  const int cg = column_tile_of<KW>(a, T, cw, t.live);
  const int tile = cg / a.ngroups;
  t.kg = (T / a.colblocks) * KW + kw;
  t.ng = cg - tile * a.ngroups;
  t.ty = tile / a.tiles_w;
  t.tx = tile - t.ty * a.tiles_w;
}

struct ScalarPatch {
  unsigned vmask;  // bit i*4+j: patch element (i,j) lies inside the image (wave-uniform)
  int vbase;       // per lane: byte offset of (channel hsel, row 2ty, col 2tx, n) in a slab
};

__device__ __forceinline__ void decode_scalar_patch(const ConvArgs& a, const TileState& t, int lane, ScalarPatch& sp) {
  unsigned m = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int hh = 2 * t.ty - 1 + i, ww = 2 * t.tx - 1 + j;
      if (hh >= 0 && hh < a.H && ww >= 0 && ww < a.W) m |= 1u << (i * 4 + j);
    }
  sp.vmask = m;
  sp.vbase = (((lane >> 5) * a.H * a.W + 2 * t.ty * a.W + 2 * t.tx) * a.N + t.ng * 32 + (lane & 31)) * 4;
}

// Patch of MFMA step `step` (channels 2*step + hsel) through scalar offsets.
__device__ __forceinline__ void load_patch_s(const ConvArgs& a, const ScalarPatch& sp, float (&d)[16], int step) {
  const size_t HWN = (size_t)a.H * a.W * a.N;
  const int st = __builtin_amdgcn_readfirstlane(step);
  const int rowb = a.W * a.N * 4, colb = a.N * 4;
  // The base is moved back by one row and one column so that the per-lane offset is never
  // negative (it is range-checked on its own); valid elements still address inside x.
  const char* base = reinterpret_cast<const char*>(a.x + (size_t)st * 2 * HWN) - rowb - colb;
  const unsigned span = (unsigned)(2 * HWN * sizeof(float)) + 4u * (unsigned)rowb;
  const __amdgpu_buffer_rsrc_t real = make_rsrc(base, span);
  const __amdgpu_buffer_rsrc_t none = make_rsrc(base, 0u);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = (sp.vmask >> (i * 4 + j)) & 1u;
      d[i * 4 + j] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(ok ? real : none, sp.vbase, i * rowb + j * colb, 0));
    }
}

__device__ __forceinline__ void load_u_s(const ConvArgs& a, int kg, int lane, v2f (&u)[16], int quad) {
  const int Q = a.C >> 2;
  const __amdgpu_buffer_rsrc_t ru = make_rsrc(a.usw, (unsigned)((size_t)a.C * 16 * a.K * sizeof(float)));
  const int soff = __builtin_amdgcn_readfirstlane((kg * Q + quad) * (16 * 64 * 8));
#pragma unroll
  for (int p = 0; p < 16; p += 2) {
    const v4f pair = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(ru, lane * 16 + p * 512, soff, 0));
    u[p] = v2f{pair[0], pair[1]};
    u[p + 1] = v2f{pair[2], pair[3]};
  }
}

template <int KW, bool BALANCED, bool SCALAR_PATCH>
__global__ void __launch_bounds__(256) wino_f32_stream(ConvArgs a) {
  constexpr int SPW = 4 / KW;
  extern __shared__ float lds[];  // [CW][2][4][16][64]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kw = wave % KW, cw = wave / KW;
  const int L = logical_block();
  const int chunks = a.C >> 3;

  // units [begin, begin + n) of this workgroup; unit = tile * chunks + chunk
  int begin, n;
  if (BALANCED) {
    const long long total = (long long)a.nblocks * chunks;
    begin = (int)(total * L / gridDim.x);
    n = (int)(total * (L + 1) / gridDim.x) - begin;
  } else {
    if (L >= a.nblocks) return;  // whole workgroup
    begin = L * chunks;
    n = chunks;
  }
  const int T_first = begin / chunks, c_first = begin - T_first * chunks;

  float* vl = lds + cw * (2 * 4 * 16 * 64) + lane;
  auto vaddr = [&](int buf, int step, int p) { return vl + ((buf * 4 + step) * 16 + p) * 64; };
  auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  v2f u[2][16];      // filter operands of the current / next quad
  float d[SPW][16];  // this wave's share of the patches of the unit after next, in flight
  float v[2][16];    // B operands of the current / next step

  auto transform_to_lds = [&](int buf) {
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
      float t[16];
      input_transform(d[j], t);
#pragma unroll
      for (int p = 0; p < 16; ++p) *vaddr(buf, kw * SPW + j, p) = t[p];
    }
  };
  auto read_v = [&](float (&dst)[16], int buf, int step) {
#pragma unroll
    for (int p = 0; p < 16; ++p) dst[p] = *vaddr(buf, step, p);
  };

  // Cursors.  M: the unit being multiplied.  P: the unit whose patches are loaded (M + 2).
  // Q: the unit whose first filter quad is loaded (M + 1).  Past the last unit they stay on it
  // (the loads are repeated and never used).
  TileState tm;
  WaveTile wp;     // used when !SCALAR_PATCH
  ScalarPatch sp;  // used when SCALAR_PATCH
  int Tp = T_first, cp = c_first;  // P
  int Tq = T_first, cq = c_first;  // Q
  int kgq;
  auto decode_p = [&]() {
    if (SCALAR_PATCH) {
      TileState t;
      decode_state<KW>(a, Tp, kw, cw, t);
      decode_scalar_patch(a, t, lane, sp);
    } else {
      int live;
      const int cg = column_tile_of<KW>(a, Tp, cw, live);
      decode_tile(a, (Tp / a.colblocks) * KW + kw, cg, lane, wp);
    }
  };
  decode_p();
  decode_state<KW>(a, T_first, kw, cw, tm);
  kgq = tm.kg;
  auto advance_p = [&](int unit_index) {  // move P to begin + unit_index (if it exists)
    if (unit_index < n) {
      if (++cp == chunks) {
        cp = 0;
        ++Tp;
        decode_p();
      }
    }
  };
  auto advance_q = [&](int unit_index) {
    if (unit_index < n) {
      if (++cq == chunks) {
        cq = 0;
        ++Tq;
        kgq = (Tq / a.colblocks) * KW + kw;
      }
    }
  };
  auto load_patches = [&](int j) {
    if (SCALAR_PATCH)
      load_patch_s(a, sp, d[j], cp * 4 + kw * SPW + j);
    else
      load_patch(a, wp, d[j], cp * 4 + kw * SPW + j);
  };

  // prologue (once per workgroup): unit 0 -> buf 0; unit 1 patches in flight; first quad in u[0]
  load_u_s(a, kgq, lane, u[0], 2 * cq);
#pragma unroll
  for (int j = 0; j < SPW; ++j) load_patches(j);
  transform_to_lds(0);
  advance_p(1);
#pragma unroll
  for (int j = 0; j < SPW; ++j) load_patches(j);
  lds_barrier();
  read_v(v[0], 0, 0);

  int Tm = T_first, cm = c_first, g = 0;
  for (;;) {
    // one tile, or the part of it that falls into this workgroup's range: chunks cm .. seg_end-1
    const int seg_first = cm;
    const int seg_end = (n - g) < (chunks - cm) ? cm + (n - g) : chunks;
    v16f acc[16];
#pragma unroll
    for (int p = 0; p < 16; ++p)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[p][r] = 0.0f;

    for (; cm < seg_end; ++cm, ++g) {
      const int buf = g & 1;
      advance_p(g + 2);
      advance_q(g + 1);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        __builtin_amdgcn_sched_barrier(0);
        if (s == 0) transform_to_lds(buf ^ 1);  // unit g+1: one VALU burst, then its LDS writes
        __builtin_amdgcn_sched_barrier(0);
        if (s == 0) load_u_s(a, tm.kg, lane, u[1], 2 * cm + 1);
        if (s == 2) load_u_s(a, kgq, lane, u[0], 2 * cq);
        if (s == 1) load_patches(0);
        if (s == 3 && SPW == 2) load_patches(1);
        if (s < 3) read_v(v[(s + 1) & 1], buf, s + 1);
#pragma unroll
        for (int p = 0; p < 16; ++p)
          acc[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(u[s >> 1][p][s & 1], v[s & 1][p], acc[p], 0, 0, 0);
#pragma unroll
        for (int p = 0; p < 16; ++p) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
          if (s != 3 || SPW == 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
          if (s != 3 && (p & 1)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      lds_barrier();
      read_v(v[0], buf ^ 1, 0);
    }

    // output transform of the finished (part of the) tile: store, or merge with the other part
    WaveTile w;  // position only; store_tile does not use the patch offsets
    w.kg = tm.kg;
    w.ng = tm.ng;
    w.ty = tm.ty;
    w.tx = tm.tx;
    w.hsel = lane >> 5;
    w.nl = lane & 31;
    if (tm.live) {
      if (!BALANCED || (seg_first == 0 && seg_end == chunks)) {
        store_tile<kStorePlain>(a, w, acc);
      } else {
        // The roles are fixed by position, no ticket needed: a segment that starts inside a
        // tile (seg_first > 0) is this workgroup's FIRST one, finishes early and publishes; the
        // other part of that tile is the LAST segment of the previous workgroup, finishes late
        // and merges.  (Ranges are at least one tile long, so a segment is never both.)
        if (seg_first > 0) {
          unsigned* flag = a.sync + ((L - 1) * 4 + wave) * 2 + 1;
          store_tile<kStorePublish>(a, w, acc);
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // write-through stores acknowledged
          if (lane == 0) __hip_atomic_store(flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        } else {
          unsigned* flag = a.sync + (L * 4 + wave) * 2 + 1;
          // normally set long ago; bounded wait all the same (never hang the GPU on a bug)
          wait_for_flag(a, flag, lane);
          store_tile<kStoreMerge>(a, w, acc);
          if (lane == 0) __hip_atomic_store(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
      }
    }
    if (g >= n) break;
    ++Tm;
    cm = 0;
    decode_state<KW>(a, Tm, kw, cw, tm);
  }
}

}  // namespace opencnn
