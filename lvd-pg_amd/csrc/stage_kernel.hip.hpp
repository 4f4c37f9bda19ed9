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

// The same for rows of consecutive bytes (stride_var == 1) whose starts are multiples of four: four
// variables per request coming in, four examples per request going out.
static __global__ __launch_bounds__(256) void pcm_stage_rows_kernel(const uint8_t* __restrict__ data, int64_t stride_ex,
                                                              const int32_t* __restrict__ idx, int B, int Bp, int V, int C,
                                                              uint8_t* __restrict__ xb) {
  __shared__ uint32_t t[64][17];   // [example][4 variables per word]
  const int b0 = blockIdx.x * 64, v0 = blockIdx.y * 64;
  const int q = threadIdx.x & 15, r0 = threadIdx.x >> 4;
  const uint32_t top = (uint32_t)(C - 1);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int bb = b0 + r0 + 16 * r, vv = v0 + 4 * q;
    uint32_t w = 0;
    if (bb < B && vv < V) {
      const int64_t row = idx ? idx[bb] : bb;
      const uint8_t* src = data + row * stride_ex + vv;
      if (vv + 4 <= V) {
        w = *reinterpret_cast<const uint32_t*>(src);
      } else {
        for (int i = 0; vv + i < V; ++i) w |= (uint32_t)src[i] << (8 * i);
      }
      // keep table reads in range whatever the caller sent
      uint32_t c = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) c |= min((w >> (8 * i)) & 0xffu, top) << (8 * i);
      w = c;
    }
    t[r0 + 16 * r][q] = w;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int vl = r0 + 16 * r, vv = v0 + vl, bb = b0 + 4 * q;   // variable vl of the tile, examples 4q .. 4q+3
    if (vv >= V || bb >= Bp) continue;
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) w |= ((t[4 * q + i][vl >> 2] >> (8 * (vl & 3))) & 0xffu) << (8 * i);
    *reinterpret_cast<uint32_t*>(xb + (size_t)vv * Bp + bb) = w;
  }
}

// Either of the two, by what the rows allow (Bp is a multiple of 16, so the word stores are aligned).
static inline void pcm_stage(const uint8_t* data, int64_t stride_ex, int64_t stride_var, const int32_t* idx, int B, int Bp, int V,
                             int C, uint8_t* xb, hipStream_t stream) {
  const dim3 grid((Bp + 63) / 64, (V + 63) / 64);
  if (stride_var == 1 && stride_ex % 4 == 0 && reinterpret_cast<uintptr_t>(data) % 4 == 0 && Bp % 4 == 0)
    hipLaunchKernelGGL(pcm_stage_rows_kernel, grid, dim3(256), 0, stream, data, stride_ex, idx, B, Bp, V, C, xb);
  else
    hipLaunchKernelGGL(pcm_stage_kernel, grid, dim3(256), 0, stream, data, stride_ex, stride_var, idx, B, Bp, V, C, xb);
}

}  // namespace pcm
