// Layout shims: the reference's data_cpy kernel (src/openCNN_winograd.cu:147-153), which turns
// the cuDNN-side NCHW input into CHWN and KCRS filters into CRSK (:230,:235), and the inverse
// needed to hand a KHWN result back as NCHW.  All three are the 2-D transpose
//     dst[c][r] = src[r][c]
// of a [rows][cols] matrix (NCHW->CHWN: rows = N, cols = C*H*W; KCRS->CRSK: rows = K, cols = C*9;
// KHWN->NKHW: rows = K*H*W, cols = N).  HBM-bound: 8 bytes per element, 64x64 tiles through
// LDS so that both the reads and the writes are 256-byte rows; the +1 column pads away the
// bank conflicts of the transposed access.  The reference's version runs one thread per
// element with an in_c-sized block (C <= 1024) and strided writes.
#pragma once
#include <hip/hip_runtime.h>

namespace opencnn {

// One-dimensional grid over the 64x64 tiles, a row of tiles after the other (gridDim.x takes
// 2^31 - 1 blocks, so neither side of the matrix is limited by the 65535 of the other dimensions).
__global__ void __launch_bounds__(256) transpose_2d(const float* __restrict__ src, float* __restrict__ dst,
                                                    int rows, int cols, int col_tiles) {
  __shared__ float tile[64][65];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4 threads
  const int row_tile = blockIdx.x / col_tiles;
  const int c0 = (blockIdx.x - row_tile * col_tiles) * 64, r0 = row_tile * 64;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = r0 + ty + 4 * i, c = c0 + tx;
    if (r < rows && c < cols) tile[ty + 4 * i][tx] = src[(size_t)r * cols + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = c0 + ty + 4 * i, r = r0 + tx;
    if (r < rows && c < cols) dst[(size_t)c * rows + r] = tile[tx][ty + 4 * i];
  }
}

}  // namespace opencnn
