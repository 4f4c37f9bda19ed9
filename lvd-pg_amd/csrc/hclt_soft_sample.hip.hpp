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
// Waves of a walk workgroup: a level's nodes are dealt to them, and each holds a node's two
// operand tiles in registers.
constexpr int soft_walk_waves(int K) { return K > 32 ? 8 : 16; }

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
// root, the nodes of a level dealt to the waves, a barrier between levels (a node reads
// its parent's tile, stored one level earlier by some wave of this workgroup).
template <int K>
__global__ __launch_bounds__(soft_walk_waves(K) * 64) void hclt_soft_walk_kernel(
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
    for (int i = level_ptr[l] + wave; i < level_ptr[l + 1]; i += soft_walk_waves(K)) {
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

// out[b][u][:] = p_{v(u)}[b][:] * exp(leaf[u]): a [B x K] by [K x C] product per variable, on
// the matrix cores with categories as rows and the 16 examples of a slice as columns.  A wave
// keeps exp(leaf[u]) of kSoftLeafCats categories as A operands in registers for a run of
// run_slices slices; a slice's probabilities arrive in the tile layout the walk wrote them
// in, which is the B operand layout: with k-step (kt, i) standing for the states
// kt*16 + 4g + i, g = 0..3, component i of a lane's 16-byte word at kt is its B value and
// component i of the word at leaf[u][c][kt*16 + 4g] its A value.  A lane of the result holds
// four consecutive categories of one example.  With rows of whole 16-byte words (use_rows) the
// tiles of a slice are turned in a wave-private LDS pad and leave as one contiguous,
// non-temporal run of C floats per example (a quarter faster than 16-byte stores four lanes
// side by side, which is what other category counts get).  The output is batch x V x C floats; with the stores taken
// out the kernel still takes two thirds of its time (the matrix instructions alone 2.0 ms of 3.5 at 4096 examples of a
// 3072-variable circuit, against 1.3 ms at the data sheet's rate), and issuing a slice's rows between the matrix
// instructions of the next slice instead of behind its own gained 1 %.
// Slices of 16 examples per work item: every item loads and exponentiates its 32 KB of table rows again, so long runs
// are cheaper (4096 examples of the 3072-variable circuit: 3.55 ms with runs of 8, 3.1 with runs of 64) as long as the
// items still fill the device several times over.
inline int soft_leaf_run_slices(int64_t items_per_slice_run, int nslices) {
  for (int run = 64; run > 8; run /= 2)
    if (items_per_slice_run * ((nslices + run - 1) / run) >= 12288) return run;
  return 8;
}
constexpr int kSoftLeafCats = 256;   // categories per work item

template <int K>
__global__ __launch_bounds__(256) void hclt_soft_leaves_kernel(const float* __restrict__ leaf,
                                                               const int32_t* __restrict__ state_node,
                                                               const float* __restrict__ P, int V, int C, int batch,
                                                               int nslices, int nchunks, int run_slices, int use_rows, float* __restrict__ out) {
  constexpr int KT = K / 16, CT = kSoftLeafCats / 16;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int u = blockIdx.x;
  const int item = blockIdx.y * 4 + wave;
  const int chunk = item % nchunks, run = item / nchunks;
  const int s_first = run * run_slices;
  if (s_first >= nslices) return;
  const int s_end = min(s_first + run_slices, nslices);
  const int g = lane >> 4, bb = lane & 15;
  const int cbase = chunk * kSoftLeafCats;
  v4f a[CT][KT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = cbase + 16 * ct + bb;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      if (c < C) {
        const v4f x = *reinterpret_cast<const v4f*>(leaf + ((size_t)u * C + c) * K + kt * 16 + 4 * g);
        a[ct][kt] = v4f{__expf(x[0]), __expf(x[1]), __expf(x[2]), __expf(x[3])};
      } else {
        a[ct][kt] = v4f{0.f, 0.f, 0.f, 0.f};
      }
    }
  }
  const float* ptile = P + (size_t)state_node[u] * nslices * kSlice * K;
  // the next slice's probabilities are requested before this one's are used
  auto fetch = [&](int s, v4f (&dst)[KT]) {
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
      dst[kt] = *reinterpret_cast<const v4f*>(ptile + (size_t)s * (kSlice * K) + (size_t)(kt * 64 + lane) * 4);
  };
  v4f pc[KT], pn[KT];
  fetch(s_first, pc);
  const bool words = (C & 3) == 0;
  extern __shared__ float soft_pad[];   // use_rows: [4 waves][16][kSoftLeafCats + 4]
  float* pad = soft_pad + (size_t)wave * kSlice * (kSoftLeafCats + 4);
  const bool rows = use_rows != 0;
  for (int s = s_first; s < s_end; ++s) {
    fetch(min(s + 1, s_end - 1), pn);
    const int b = s * kSlice + bb;
    if (rows) {
      // whole rows: the tiles go through this wave's LDS pad [16 examples][kSoftLeafCats + 4] and leave
      // as one contiguous run per example (a wave's LDS accesses execute in order: no barrier)
      constexpr int PS = kSoftLeafCats + 4;
      const int cw = min(kSoftLeafCats, C - cbase);   // categories of this chunk
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        if (16 * ct >= cw) break;   // the same for the whole wave
        v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ct][kt][i], pc[kt][i], acc, 0, 0, 0);
        if (16 * ct + 4 * g < cw) *reinterpret_cast<v4f*>(pad + bb * PS + 16 * ct + 4 * g) = acc;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      const int nrow = min(kSlice, batch - s * kSlice);
      for (int r = 0; r < nrow; ++r) {
        float* o = out + ((size_t)(s * kSlice + r) * V + u) * C + cbase;
        for (int c0 = 4 * lane; c0 < cw; c0 += 256)
          __builtin_nontemporal_store(*reinterpret_cast<const v4f*>(pad + r * PS + c0), reinterpret_cast<v4f*>(o + c0));
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    } else {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      if (cbase + 16 * ct >= C) break;   // the same for the whole wave
      v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ct][kt][i], pc[kt][i], acc, 0, 0, 0);
      const int c = cbase + 16 * ct + 4 * g;
      if (b < batch) {
        float* o = out + ((size_t)b * V + u) * C + c;
        if (words && c + 3 < C) {
          *reinterpret_cast<v4f*>(o) = acc;   // default policy: the other half of the 128-byte line follows with the next tile
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (c + i < C) o[i] = acc[i];
        }
      }
    }
    }
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) pc[kt] = pn[kt];
  }
}

}  // namespace pcm
