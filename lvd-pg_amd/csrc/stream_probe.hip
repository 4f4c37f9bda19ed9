// A plain streaming kernel as a measuring instrument: what this device's memory gives a kernel that does nothing
// but read R streams and write W streams, 16 bytes per lane and access, non-temporal, as the tile traffic of the
// walk kernels is.  The walks' counter-measured bytes per second are read against the figure for their own mix of
// reads and writes (4 : 3 going down, 1 : 3 going up, 6 : 1 for the statistics), not against the 8 TB/s of the data
// sheet alone.
#include "common.hpp"

#include <hip/hip_runtime.h>

namespace pcm {

typedef float probe4 __attribute__((ext_vector_type(4)));

template <int RD, int WR>   // per lane and iteration: RD loads and WR stores of 16 bytes, each from / to a stream of its own
__global__ __launch_bounds__(256) void stream_probe_kernel(const probe4* __restrict__ src, probe4* __restrict__ dst, int64_t lanes) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, nth = (int64_t)gridDim.x * blockDim.x;
  for (int64_t it = tid; it < lanes; it += nth) {
    probe4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < RD; ++r) acc += __builtin_nontemporal_load(src + it + (int64_t)r * lanes);
#pragma unroll
    for (int w = 0; w < WR; ++w) __builtin_nontemporal_store(acc, dst + it + (int64_t)w * lanes);
    if (WR == 0 && acc.x == 12345.f) dst[0] = acc;   // keeps the loads of the read-only case
  }
}

void stream_probe(const void* d_src, void* d_dst, int64_t lanes, int reads, int writes, int grid, hipStream_t stream) {
  if (lanes <= 0 || grid <= 0 || grid > (1 << 20)) fail(PCM_ERR_ARG, "stream probe: lanes %lld, grid %d", (long long)lanes, grid);
  if ((reads > 0 && !d_src) || !d_dst) fail(PCM_ERR_ARG, "stream probe: null buffer");
  const probe4* s = static_cast<const probe4*>(d_src);
  probe4* d = static_cast<probe4*>(d_dst);
#define PCM_PROBE(R_, W_)                                                                              \
  if (reads == R_ && writes == W_) {                                                                   \
    hipLaunchKernelGGL((stream_probe_kernel<R_, W_>), dim3(grid), dim3(256), 0, stream, s, d, lanes);  \
    hipError_t e = hipGetLastError();                                                                  \
    if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of stream_probe failed: %s", hipGetErrorString(e)); \
    return;                                                                                            \
  }
  PCM_PROBE(1, 0) PCM_PROBE(0, 1) PCM_PROBE(1, 1) PCM_PROBE(4, 3) PCM_PROBE(1, 3) PCM_PROBE(6, 1)
#undef PCM_PROBE
  fail(PCM_ERR_ARG, "stream probe: no kernel for %d reads : %d writes (1:0, 0:1, 1:1, 4:3, 1:3, 6:1)", reads, writes);
}

}  // namespace pcm
