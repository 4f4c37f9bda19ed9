// Relaxed (Gumbel-softmax) top-down sampling of HCLTs on the block form.
//
// Reference: src/queries/sample.jl:37-51 (a sum node's edges get u = exp((logp + g) / T),
// normalised over the node), :105-140 (top-down probability handed to prime and sub), :262-284
// (an input node adds td * exp(logp_c) to out[variable][c]).  With the compact noise of an HCLT
// (one draw g_v[j] per tree node and hidden state, shared by the K sum nodes of v):
//   u_v[k,j] = A_v[k,j] * E_v[j] / S_v[k],  A = exp((theta - rowmax) / T),  E = exp((g - max g) / T),  S = A E
//   p_v[j]   = E_v[j] * sum_k (q_v[k] / S_v[k]) * A_v[k,j],   q_c = p_v for the tree children, q_root = e_0
//   out[b][u][c] = sum_j p_{v(u)}[b][j] * exp(leaf[u][c][j])      (v(u): u's own tree node, or its parent's for a leaf of the tree)
// i.e. per (tree node, 16 examples) the forward contraction followed by the backward one of the
// EM kernels, on the matrix cores, with the exponentials taken out of the K x K loops.  The
// row and vector maxima keep every factor <= 1; a row whose admissible states all underflow
// against the noise (temperatures far below the spread of the noise) would lose its mass, so
// the host sends temperatures below kSoftMinTemperature to the layered engine instead.
#pragma once

#include "hclt_kernels.hip.hpp"

namespace pcm {

constexpr float kSoftMinTemperature = 0.2f;
constexpr int kSoftWalkWaves = 4;

// A_v in the two operand layouts of the contractions (per call: it depends on T).
template <int K>
__global__ void hclt_soft_w_kernel(const float* __restrict__ logtheta, float inv_t, int n_inner, float* __restrict__ Af,
                                   float* __restrict__ Ab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_inner * K) return;
  const int n = i / K, k = i % K;
  const float* lt = logtheta + (size_t)i * K;
  float m = -INFINITY;
  for (int j = 0; j < K; ++j) m = fmaxf(m, lt[j]);
  for (int j = 0; j < K; ++j)
    put_w<K>(Af + (size_t)n * K * K, Ab + (size_t)n * K * K, k, j, m == -INFINITY ? 0.f : __expf((lt[j] - m) * inv_t));
}

// p_v for every tree node: one workgroup per 16-example slice, nodes level by level from the
// root, the nodes of a level dealt to the four waves, a barrier between levels (a node reads
// its parent's tile, stored one level earlier by some wave of this workgroup).
template <int K>
__global__ __launch_bounds__(kSoftWalkWaves * 64) void hclt_soft_walk_kernel(
    const float* __restrict__ Af, const float* __restrict__ Ab, const int32_t* __restrict__ parent_of,
    const int32_t* __restrict__ order, const int32_t* __restrict__ level_ptr, int n_levels, const float* __restrict__ noise,
    int n_inner, int batch, int nslices, float inv_t, float* P) {
  constexpr int KT = K / 16;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int s = blockIdx.x, b = lane & 15, g = lane >> 4;
  const LaneOffs lo = lane_offs<K>(s, lane);
  const uint32_t tile_stride = (uint32_t)nslices * kSlice * K * 4;
  const float* grow = noise ? noise + (size_t)min(lo.bcol, batch - 1) * n_inner * K + 4 * g : nullptr;
  for (int l = 0; l < n_levels; ++l) {
    for (int i = level_ptr[l] + wave; i < level_ptr[l + 1]; i += kSoftWalkWaves) {
      const int n = order[i], par = parent_of[n];
      WTile<K> af, ab;
      w_load<K>(Af, n, lane, af);
      w_load<K>(Ab, n, lane, ab);
      Tile<K> e, q, t;
      if (par >= 0) {
        tile_load<K>(P, par, tile_stride, lo.tile, q);
      } else {
        tile_zero<K>(q);
        if (g == 0) q.v[0][0] = 1.f;
      }
      if (grow) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) e.v[kt] = *reinterpret_cast<const v4f*>(grow + (size_t)n * K + kt * 16);
        const float m = tile_rowmax<K>(e);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int c = 0; c < 4; ++c) e.v[kt][c] = __expf((e.v[kt][c] - m) * inv_t);
      } else {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) e.v[kt] = v4f{1.f, 1.f, 1.f, 1.f};
      }
      contract<K>(af, e, t);   // S[b,k] = sum_j A[k,j] E[b,j]
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int c = 0; c < 4; ++c) q.v[kt][c] = (t.v[kt][c] > 0.f && q.v[kt][c] > 0.f) ? q.v[kt][c] / t.v[kt][c] : 0.f;
      contract<K>(ab, q, t);   // sum_k A[k,j] R[b,k]
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) t.v[kt] *= e.v[kt];
      // default cache policy: the tile is read back by the children's steps and by the leaf kernel
      v4f* dst = reinterpret_cast<v4f*>(reinterpret_cast<char*>(P) + (size_t)n * tile_stride + lo.tile);
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) dst[kt * 64] = t.v[kt];
    }
    __syncthreads();
  }
}

// out[b][u][:] = p_{v(u)}[b][:] * exp(leaf[u])  (a [1 x K] by [K x C] product per example and
// variable).  A wave keeps exp(leaf[u]) of four categories per lane in registers for a run of
// examples; an example's K probabilities are wave-uniform and come through scalar registers,
// so the inner product is one fused multiply-add per (state, category).  Write-bound: the
// output is batch x V x C floats.
constexpr int kSoftLeafRun = 64;   // examples per wave

template <int K>
__global__ __launch_bounds__(256) void hclt_soft_leaves_kernel(const float* __restrict__ leaf,
                                                               const int32_t* __restrict__ state_node,
                                                               const float* __restrict__ P, int V, int C, int batch,
                                                               int nslices, float* __restrict__ out) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int u = blockIdx.x;
  const int b_first = (blockIdx.y * 4 + wave) * kSoftLeafRun;
  if (b_first >= batch) return;
  const int n = state_node[u];
  const float* ptile = P + (size_t)n * nslices * kSlice * K;
  for (int c0 = 4 * lane; c0 < C; c0 += 256) {
    float sv[K][4];
#pragma unroll
    for (int j4 = 0; j4 < K / 4; ++j4)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const v4f x = c0 + c < C ? *reinterpret_cast<const v4f*>(leaf + ((size_t)u * C + c0 + c) * K + 4 * j4)
                                 : v4f{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
        for (int i = 0; i < 4; ++i) sv[4 * j4 + i][c] = __expf(x[i]);
      }
    const int b_end = min(b_first + kSoftLeafRun, batch);
    // example bq = slice * 16 + bb holds state kt*16 + 4*g + i at float ((kt*64 + 16*g + bb) * 4 + i) of its tile;
    // the next example's probabilities are requested before this one's are used
    auto fetch = [&](int bq, v4f (&dst)[K / 4]) {
      const float* pe = ptile + (size_t)(bq >> 4) * (kSlice * K) + (bq & 15) * 4;   // wave-uniform address
#pragma unroll
      for (int q = 0; q < K / 4; ++q) dst[q] = *reinterpret_cast<const v4f*>(pe + (size_t)q * 64);
    };
    v4f pc[K / 4], pn[K / 4];
    fetch(b_first, pc);
    for (int bq = b_first; bq < b_end; ++bq) {
      fetch(min(bq + 1, b_end - 1), pn);
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < K / 4; ++q)   // q = kt * 4 + g: states q * 4 + i
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[c] = fmaf(pc[q][i], sv[4 * q + i][c], acc[c]);
#pragma unroll
      for (int q = 0; q < K / 4; ++q) pc[q] = pn[q];
      float* o = out + ((size_t)bq * V + u) * C + c0;
      if (c0 + 3 < C && (C & 3) == 0) {
        __builtin_nontemporal_store(v4f{acc[0], acc[1], acc[2], acc[3]}, reinterpret_cast<v4f*>(o));
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (c0 + c < C) o[c] = acc[c];
      }
    }
  }
}

}  // namespace pcm
