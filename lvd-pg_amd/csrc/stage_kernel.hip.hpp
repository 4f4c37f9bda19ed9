// Batch staging shared by both engines.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace pcm {

// Batch rows -> xb[var][example] (example fastest), through a 64 x 64 LDS tile.
static __global__ __launch_bounds__(256) void pcm_stage_kernel(const uint8_t* __restrict__ data,
                                                         int64_t stride_ex, int64_t stride_var,
                                                         const int32_t* __restrict__ idx, int B, int Bp,
                                                         int V, int C, uint8_t* __restrict__ xb) {
  __shared__ uint8_t t[64][65];
  const int b0 = blockIdx.x * 64, v0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = 0; r < 16; ++r) {
    const int bb = b0 + ty + 4 * r, vv = v0 + tx;
    uint8_t val = 0;
    if (bb < B && vv < V) {
      const int64_t row = idx ? idx[bb] : bb;
      val = data[row * stride_ex + vv * stride_var];
      val = val < C ? val : (uint8_t)(C - 1);   // keep table reads in range whatever the caller sent
    }
    t[ty + 4 * r][tx] = val;
  }
  __syncthreads();
  for (int r = 0; r < 16; ++r) {
    const int vv = v0 + ty + 4 * r, bb = b0 + tx;
    if (vv < V && bb < Bp) xb[(size_t)vv * Bp + bb] = t[tx][ty + 4 * r];
  }
}

}  // namespace pcm
