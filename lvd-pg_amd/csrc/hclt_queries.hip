// Sampling from HCLT circuits.  Gumbel-max sampling has its own kernels on the block form
// (below); the relaxed sampler runs on the layered engine over the circuit's general form, with
// parameters exchanged in parameter-vector order, which both forms share.
#include "hclt_engine.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>

namespace pcm {

static void check_launch_q(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

// Four consecutive noise values, read once: a non-temporal request, so the stream does not push
// the tables out of the caches.
__device__ __forceinline__ float4 noise_word(const float* p) {
  typedef float v4f_t __attribute__((ext_vector_type(4)));
  const v4f_t t = __builtin_nontemporal_load(reinterpret_cast<const v4f_t*>(p));
  return make_float4(t[0], t[1], t[2], t[3]);
}

// ---- Gumbel-max sampling on the block form -------------------------------------------------
// A sample is a top-down walk: the root's single sum node picks hidden state
// j* = argmax_j(theta_root[0][j] + g[b][root][j]); a tree node whose parent picked k picks
// j* = argmax_j(theta_v[k][j] + g[b][v][j]) (first maximum wins); every variable then emits
// argmax_c(leaf[v][j*][c] + g_leaf[b][v][c]) with j* the state of its own tree node (inner
// nodes) or of its parent (leaf tree nodes).  Same additions and comparisons, in the same
// order, as the layered engine's sampler on the circuit's general form.

// States of the inner tree nodes, a lane per tree node: a wave takes one example and walks the
// levels from the root, 64 nodes of a level at a time (`passes` records of 64 {node, parent}
// pairs, -1: no node).  A lane reads its node's K noise values and the parameter row its
// parent's state selects (two contiguous rows of 4K bytes) and scans them in order: first
// maximum wins, no exchange between lanes.  The noise does not depend on any state, so its
// requests leave a pass ahead (up to K = 32, where a row fits the registers twice), or at
// least before the parent's state is read.  The chosen states live in LDS (one byte
// per node) and leave through a coalesced copy at the end; no barriers, a wave only reads its
// own example's bytes.
template <int K>
__global__ __launch_bounds__(256) void hclt_sample_states_node_kernel(const float* __restrict__ logtheta,
                                                                      const int2* __restrict__ passes_tab, int passes,
                                                                      const float* __restrict__ node_noise,
                                                                      int n_inner, int stride, int batch,
                                                                      uint8_t* __restrict__ states) {
  static_assert(K % 4 == 0, "rows are read as 16-byte words");
  constexpr int CH = K < 32 ? K : 32;   // values scanned per round: 8 words of noise and 8 of parameters in registers
  extern __shared__ uint8_t st[];   // [4 waves][stride]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = blockIdx.x * 4 + wave;
  if (b >= batch) return;
  uint8_t* mine = st + (size_t)wave * stride;
  const float* g = node_noise + (size_t)b * n_inner * K;
  if constexpr (K <= 32) {
    // the noise of a pass is requested one pass ahead (the table ends with two empty records)
    int2 rec0 = passes_tab[lane], rec1 = passes_tab[64 + lane];
    float4 z[K / 4];
#pragma unroll
    for (int i = 0; i < K / 4; ++i) z[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (rec0.x >= 0) {
#pragma unroll
      for (int i = 0; i < K / 4; ++i) z[i] = reinterpret_cast<const float4*>(g + (size_t)rec0.x * K)[i];
    }
    for (int ps = 0; ps < passes; ++ps) {
      const int n = rec0.x, par = rec0.y;
      const int2 rec2 = passes_tab[(size_t)(ps + 2) * 64 + lane];
      const int k = (n >= 0 && par >= 0) ? mine[par] : 0;
      float4 a[K / 4], zn[K / 4];
      if (n >= 0) {
        const float4* row = reinterpret_cast<const float4*>(logtheta + ((size_t)n * K + k) * K);
#pragma unroll
        for (int i = 0; i < K / 4; ++i) a[i] = row[i];
      }
#pragma unroll
      for (int i = 0; i < K / 4; ++i) zn[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (rec1.x >= 0) {
#pragma unroll
        for (int i = 0; i < K / 4; ++i) zn[i] = reinterpret_cast<const float4*>(g + (size_t)rec1.x * K)[i];
      }
      if (n >= 0) {
        float best = 0.f;
        int idx = 0;
#pragma unroll
        for (int i = 0; i < K / 4; ++i) {
          const float x[4] = {a[i].x + z[i].x, a[i].y + z[i].y, a[i].z + z[i].z, a[i].w + z[i].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = 4 * i + e;
            if (j == 0 || x[e] > best) { best = x[e]; idx = j; }
          }
        }
        mine[n] = (uint8_t)idx;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
      for (int i = 0; i < K / 4; ++i) z[i] = zn[i];
      rec0 = rec1;
      rec1 = rec2;
    }
  } else {
    // K = 64, 128: a row is scanned in rounds of 32 values, its noise requested with it
  int2 rec = passes_tab[lane];
    for (int ps = 0; ps < passes; ++ps) {
      const int n = rec.x, par = rec.y;
      if (ps + 1 < passes) rec = passes_tab[(size_t)(ps + 1) * 64 + lane];
      if (n >= 0) {
        const float4* gz = reinterpret_cast<const float4*>(g + (size_t)n * K);
        float best = 0.f;
        int idx = 0;
  #pragma unroll
        for (int j0 = 0; j0 < K; j0 += CH) {
          float4 z[CH / 4], a[CH / 4];
  #pragma unroll
          for (int i = 0; i < CH / 4; ++i) z[i] = gz[j0 / 4 + i];   // default policy: a lane's row is one cache line read in pieces
          const int k = par < 0 ? 0 : mine[par];
          const float4* row = reinterpret_cast<const float4*>(logtheta + ((size_t)n * K + k) * K);
  #pragma unroll
          for (int i = 0; i < CH / 4; ++i) a[i] = row[j0 / 4 + i];
  #pragma unroll
          for (int i = 0; i < CH / 4; ++i) {
            const float x[4] = {a[i].x + z[i].x, a[i].y + z[i].y, a[i].z + z[i].z, a[i].w + z[i].w};
  #pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int j = j0 + 4 * i + e;
              if (j == 0 || x[e] > best) { best = x[e]; idx = j; }
            }
          }
        }
        mine[n] = (uint8_t)idx;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // the next level's lanes read these bytes
    }
  }
  for (int i = lane; i < n_inner; i += 64) states[(size_t)b * n_inner + i] = mine[i];
}

// (value, category) of one lane against another's: the larger value, the lower category among equal values; a lane
// that has seen nothing carries category 0x7fffffff
__device__ __forceinline__ void argmax_take(float& bv, int& bx, float ov, int oi) {
  if (oi != 0x7fffffff && (bx == 0x7fffffff || ov > bv || (ov == bv && oi < bx))) { bv = ov; bx = oi; }
}

// The maxima of N examples over a wave as one butterfly: at the first log2(N) steps the two halves of a group of lanes
// swap half of the examples they still carry, the remaining steps reduce the one example a group of 64 / N lanes is
// left with.  Afterwards bv[0], bx[0] of lane l belong to example l / (64 / N).  2 (N - 1) + 2 log2(64 / N) cross-lane
// moves instead of 12 N; the moves go through the LDS unit, which in these kernels also serves the table rows.
template <int N>
__device__ __forceinline__ void argmax_deal(float (&bv)[N], int (&bx)[N], int lane) {
  static_assert(N == 2 || N == 4 || N == 8, "N examples on 64 lanes");
  int o = 32;
#pragma unroll
  for (int n = N; n > 1; n >>= 1, o >>= 1) {
    const bool up = lane & o;
#pragma unroll
    for (int i = 0; i < n / 2; ++i) {
      float kv = up ? bv[n / 2 + i] : bv[i];
      int ki = up ? bx[n / 2 + i] : bx[i];
      const float sv = up ? bv[i] : bv[n / 2 + i];
      const int si = up ? bx[i] : bx[n / 2 + i];
      argmax_take(kv, ki, __shfl_xor(sv, o), __shfl_xor(si, o));
      bv[i] = kv;
      bx[i] = ki;
    }
  }
#pragma unroll
  for (int r = 64 / N / 2; r > 0; r >>= 1) argmax_take(bv[0], bx[0], __shfl_xor(bv[0], r), __shfl_xor(bx[0], r));
}

// N = 4 written out (the category kernel with the table in LDS): the same moves, but the kernel around it comes out 8 %
// faster than with the loops above (2.71 against 2.96 ms at 4096 samples of a 3072-variable circuit).
template <>
__device__ __forceinline__ void argmax_deal<4>(float (&best)[4], int (&bi)[4], int lane) {
  const bool hb = lane & 32, qb = lane & 16;
  float k0 = hb ? best[2] : best[0], k1 = hb ? best[3] : best[1];
  int i0 = hb ? bi[2] : bi[0], i1 = hb ? bi[3] : bi[1];
  argmax_take(k0, i0, __shfl_xor(hb ? best[0] : best[2], 32), __shfl_xor(hb ? bi[0] : bi[2], 32));
  argmax_take(k1, i1, __shfl_xor(hb ? best[1] : best[3], 32), __shfl_xor(hb ? bi[1] : bi[3], 32));
  float bv = qb ? k1 : k0;
  int bx = qb ? i1 : i0;
  argmax_take(bv, bx, __shfl_xor(qb ? k0 : k1, 16), __shfl_xor(qb ? i0 : i1, 16));
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) argmax_take(bv, bx, __shfl_xor(bv, o), __shfl_xor(bx, o));
  best[0] = bv;
  bi[0] = bx;
}

// Categories.  A wave takes kVarsPerWave consecutive variables of one example, 64 lanes x 4
// categories each (more categories: further rounds), requests all their rows first and then
// reduces them one by one: per variable the wave keeps the largest value and, among equal
// values, the lowest category.
constexpr int kVarsPerWave = 8;

__global__ __launch_bounds__(256) void hclt_sample_leaves_kernel(const float* __restrict__ leaf_kc,
                                                                 const int32_t* __restrict__ state_node,
                                                                 const uint8_t* __restrict__ states,
                                                                 const float* __restrict__ leaf_noise, int V, int K,
                                                                 int C, int n_inner, int batch,
                                                                 uint8_t* __restrict__ out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = blockIdx.x;
  const int v0 = (blockIdx.y * 4 + wave) * kVarsPerWave;
  if (v0 >= V) return;
  const uint8_t* sb = states + (size_t)b * n_inner;
  const bool vec = (C & 3) == 0;
  float best[kVarsPerWave];
  int bi[kVarsPerWave];
#pragma unroll
  for (int q = 0; q < kVarsPerWave; ++q) { best[q] = -INFINITY; bi[q] = 0x7fffffff; }
  // the states pick the leaf rows: requested once, ahead of everything that waits for them
  int row[kVarsPerWave];
#pragma unroll
  for (int q = 0; q < kVarsPerWave; ++q) {
    const int v = min(v0 + q, V - 1);
    row[q] = v * K + sb[state_node[v]];
  }
  for (int c0 = lane * 4; c0 < C; c0 += 256) {
    float x[kVarsPerWave][4];
    if (vec) {
      // the noise needs no state: its requests leave first
      float4 n4[kVarsPerWave];
#pragma unroll
      for (int q = 0; q < kVarsPerWave; ++q)
        n4[q] = *reinterpret_cast<const float4*>(leaf_noise + ((size_t)b * V + min(v0 + q, V - 1)) * C + c0);
#pragma unroll
      for (int q = 0; q < kVarsPerWave; ++q) {
        const float4 a = *reinterpret_cast<const float4*>(leaf_kc + (size_t)row[q] * C + c0);
        x[q][0] = a.x + n4[q].x; x[q][1] = a.y + n4[q].y; x[q][2] = a.z + n4[q].z; x[q][3] = a.w + n4[q].w;
      }
    } else {
#pragma unroll
      for (int q = 0; q < kVarsPerWave; ++q) {
        const float* lp = leaf_kc + (size_t)row[q] * C;
        const float* g = leaf_noise + ((size_t)b * V + min(v0 + q, V - 1)) * C;
#pragma unroll
        for (int i = 0; i < 4; ++i) x[q][i] = c0 + i < C ? lp[c0 + i] + g[c0 + i] : -INFINITY;
      }
    }
#pragma unroll
    for (int q = 0; q < kVarsPerWave; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (c0 + i < C && (x[q][i] > best[q] || bi[q] == 0x7fffffff)) { best[q] = x[q][i]; bi[q] = c0 + i; }
  }
  argmax_deal<kVarsPerWave>(best, bi, lane);
  const int q = lane / (64 / kVarsPerWave);   // the variable this group of lanes is left with
  if (lane % (64 / kVarsPerWave) == 0 && v0 + q < V) out[(size_t)b * V + v0 + q] = (uint8_t)bi[0];
}

// Categories with the leaf table in LDS.  A workgroup takes one variable and kLeafExamples
// examples: it turns the variable's [C][K] table into [K][C + 4] in LDS (rows stay 16-byte
// aligned, the turning stores spread over the banks) and gathers the examples' states of the
// node that picks the row; then every wave takes kLeafUnroll examples at a time, requests
// their noise rows (C contiguous floats) and adds the table rows from LDS, so the table
// crosses the L2 once per workgroup instead of a row per example.  Same rule as above: largest
// value, lowest category among equal values.
constexpr int kLeafExamples = 512, kLeafUnroll = 4, kLeafWaves = 8;

__global__ __launch_bounds__(kLeafWaves * 64) void hclt_sample_leaves_lds_kernel(
    const float* __restrict__ leaf, const int32_t* __restrict__ state_node, const uint8_t* __restrict__ states,
    const float* __restrict__ leaf_noise, int V, int K, int C, int n_inner, int batch, uint8_t* __restrict__ out) {
  extern __shared__ float tab[];   // [K][C + 4] floats, then kLeafExamples state bytes
  const int CS = C + 4;
  uint8_t* ks = reinterpret_cast<uint8_t*>(tab + (size_t)K * CS);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int v = blockIdx.x, b0 = blockIdx.y * kLeafExamples;
  const int nb = min(kLeafExamples, batch - b0);
  {
    const float4* src = reinterpret_cast<const float4*>(leaf + (size_t)v * C * K);   // K is a multiple of 4
    for (int i = threadIdx.x; i < C * K / 4; i += kLeafWaves * 64) {
      const float4 x = src[i];
      const int c = (i * 4) / K, k = (i * 4) % K;
      tab[(k + 0) * CS + c] = x.x;
      tab[(k + 1) * CS + c] = x.y;
      tab[(k + 2) * CS + c] = x.z;
      tab[(k + 3) * CS + c] = x.w;
    }
    const int node = state_node[v];
    for (int e = threadIdx.x; e < kLeafExamples; e += kLeafWaves * 64)
      ks[e] = e < nb ? states[(size_t)(b0 + e) * n_inner + node] : 0;
  }
  __syncthreads();
  for (int e0 = wave * kLeafUnroll; e0 < nb; e0 += kLeafWaves * kLeafUnroll) {
    float best[kLeafUnroll];
    int bi[kLeafUnroll];
#pragma unroll
    for (int u = 0; u < kLeafUnroll; ++u) { best[u] = -INFINITY; bi[u] = 0x7fffffff; }
    for (int c0 = lane * 4; c0 < C; c0 += 256) {
      float4 n4[kLeafUnroll];
#pragma unroll
      for (int u = 0; u < kLeafUnroll; ++u) {
        const int e = min(e0 + u, nb - 1);
        n4[u] = noise_word(leaf_noise + ((size_t)(b0 + e) * V + v) * C + c0);
      }
#pragma unroll
      for (int u = 0; u < kLeafUnroll; ++u) {
        const int e = min(e0 + u, nb - 1);
        const float4 a = *reinterpret_cast<const float4*>(tab + (size_t)ks[e] * CS + c0);
        const float x[4] = {a.x + n4[u].x, a.y + n4[u].y, a.z + n4[u].z, a.w + n4[u].w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (x[i] > best[u] || bi[u] == 0x7fffffff) { best[u] = x[i]; bi[u] = c0 + i; }
      }
    }
    argmax_deal<kLeafUnroll>(best, bi, lane);
    const int bx = bi[0];
    const int u = lane / (64 / kLeafUnroll);   // the example this group of lanes is left with
    if (lane % (64 / kLeafUnroll) == 0 && e0 + u < nb) out[(size_t)(b0 + e0 + u) * V + v] = (uint8_t)bx;
  }
}

// leaf tables [V][C][K] -> [V][K][C] (a variable's categories contiguous per hidden state)
__global__ void hclt_leaf_kc_kernel(const float* __restrict__ leaf, float* __restrict__ leaf_kc, int V, int K, int C) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)V * K * C) return;
  const int c = (int)(i % C), jj = (int)((i / C) % K), v = (int)(i / ((int64_t)C * K));
  leaf_kc[i] = leaf[((size_t)v * C + c) * K + jj];
}

SparseCircuit* HcltCircuit::general() {
  no_forest("this query");
  no_missing("this query");
  if (!general_) {
    general_.reset(new SparseCircuit(flat_));
    general_->stream = stream;
    general_stale_ = true;
  }
  general_->stream = stream;
  if (general_stale_) {
    std::vector<float> p((size_t)size(0));
    vectorize(p.data(), (int64_t)p.size());
    general_->update_parameters(p.data(), (int64_t)p.size());
    general_stale_ = false;
  }
  return general_.get();
}

SparseCircuit* HcltCircuit::general_structure() {
  no_forest("this query");
  no_missing("this query");
  if (!general_) {
    general_.reset(new SparseCircuit(flat_));
    general_stale_ = true;
  }
  general_->stream = stream;
  return general_.get();
}

void HcltCircuit::pull_from_general() {
  std::vector<float> p((size_t)size(0));
  general_->vectorize(p.data(), (int64_t)p.size());
  update_parameters(p.data(), (int64_t)p.size());
  general_stale_ = false;
}

void HcltCircuit::sample(const float* d_node_noise, const float* d_leaf_noise, int32_t batch, uint8_t* d_out) {
  no_forest("this query");
  no_missing("this query");
  if (H_ > 0) fail(PCM_ERR_UNSUPPORTED, "sampling from a multi-head circuit needs a head choice");
  if (!d_node_noise || !d_leaf_noise || !d_out) fail(PCM_ERR_ARG, "null noise or output pointer");
  if (batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", batch);
  if ((reinterpret_cast<uintptr_t>(d_node_noise) | reinterpret_cast<uintptr_t>(d_leaf_noise)) & 15)
    fail(PCM_ERR_ARG, "noise pointers must be 16-byte aligned (rows are read as 16-byte words)");
  const bool rows_fit = K_ >= 4 && K_ <= 128 && (K_ & (K_ - 1)) == 0;   // rows of whole 16-byte words, states in a byte
  const int stride = (n_inner_ + 15) & ~15;   // bytes of one example's states in LDS
  const size_t st_bytes = (size_t)4 * stride;
  if (!rows_fit || st_bytes > (size_t)64 * 1024) {   // other hidden sizes: the layered engine's sampler
    SparseCircuit* g = general();
    DevBuf<int32_t> slots;
    slots.upload(noise_slot_, stream);
    g->sample_with_slots(d_node_noise, slots.p, sample_noise_size(), d_leaf_noise, batch, d_out);
    return;
  }
  if (d_sample_tabs_.n == 0) {
    // per inner node: its parent | per variable: the node whose state picks its leaf row
    std::vector<int32_t> t((size_t)n_inner_ + V_);
    for (int n = 0; n < n_inner_; ++n) {
      const int v = var_of_inner_[n];
      t[n] = parent_[v] < 0 ? -1 : inner_of_var_[parent_[v]];
    }
    for (int v = 0; v < V_; ++v) t[(size_t)n_inner_ + v] = children_[v].empty() ? inner_of_var_[parent_[v]] : inner_of_var_[v];
    // inner nodes level by level from the root in records of 64 {node, parent} pairs (-1: padding)
    std::vector<std::vector<int32_t>> by_depth;
    for (int n = 0; n < n_inner_; ++n) {
      const size_t dep = (size_t)depth_[var_of_inner_[n]];
      if (by_depth.size() <= dep) by_depth.resize(dep + 1);
      by_depth[dep].push_back(n);
    }
    std::vector<int32_t> rec;
    for (const auto& lvl : by_depth) {
      for (int32_t n : lvl) {
        rec.push_back(n);
        rec.push_back(t[n]);
      }
      while (rec.size() % 128) rec.push_back(-1);
    }
    sample_passes_ = (int)(rec.size() / 128);
    rec.resize(rec.size() + 256, -1);   // two empty records: the walk requests records two passes ahead
    d_sample_passes_.upload(rec, stream);
    d_sample_tabs_.upload(t, stream);
  }
  d_state_.ensure((size_t)batch * n_inner_);
  auto node_states = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(ceil_div(batch, 4)), dim3(256), st_bytes, stream, d_logtheta_.p,
                       reinterpret_cast<const int2*>(d_sample_passes_.p), sample_passes_, kernel_noise(d_node_noise, batch),
                       n_inner_, stride, batch, d_state_.p);
  };
  switch (K_) {
    case 4: node_states(&hclt_sample_states_node_kernel<4>); break;
    case 8: node_states(&hclt_sample_states_node_kernel<8>); break;
    case 16: node_states(&hclt_sample_states_node_kernel<16>); break;
    case 32: node_states(&hclt_sample_states_node_kernel<32>); break;
    case 64: node_states(&hclt_sample_states_node_kernel<64>); break;
    default: node_states(&hclt_sample_states_node_kernel<128>); break;
  }
  // the variable's table in LDS when the 160 KB of a compute unit hold it and its rows are whole 16-byte words
  const size_t lds = (size_t)K_ * (C_ + 4) * sizeof(float) + kLeafExamples;
  if ((C_ & 3) == 0 && (K_ & 3) == 0 && lds <= (size_t)160 * 1024) {
    if (lds > (size_t)64 * 1024)
      PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hclt_sample_leaves_lds_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    // (leaves: the caller's variables, which come first; the auxiliary ones have nothing to draw)
    hipLaunchKernelGGL(hclt_sample_leaves_lds_kernel, dim3(Vu_, ceil_div(batch, kLeafExamples)), dim3(kLeafWaves * 64), lds,
                       stream, d_leaf_.p, d_sample_tabs_.p + n_inner_, d_state_.p, d_leaf_noise, Vu_, K_, C_, n_inner_, batch,
                       d_out);
  } else {
    d_leaf_kc_.ensure((size_t)V_ * K_ * C_);
    const int64_t tot = (int64_t)V_ * K_ * C_;
    hipLaunchKernelGGL(hclt_leaf_kc_kernel, dim3((unsigned)ceil_div(tot, 256)), dim3(256), 0, stream, d_leaf_.p, d_leaf_kc_.p,
                       V_, K_, C_);
    hipLaunchKernelGGL(hclt_sample_leaves_kernel, dim3(batch, ceil_div(Vu_, 4 * kVarsPerWave)), dim3(256), 0, stream, d_leaf_kc_.p,
                       d_sample_tabs_.p + n_inner_, d_state_.p, d_leaf_noise, Vu_, K_, C_, n_inner_, batch, d_out);
  }
  check_launch_q("hclt_sample");
  sync_checked();
}

void HcltCircuit::sample_soft(const float* d_node_noise, float temperature, int32_t batch, float* d_out) {
  no_forest("this query");
  no_missing("this query");
  if (H_ > 0) fail(PCM_ERR_UNSUPPORTED, "sampling from a multi-head circuit needs a head choice");
  if (sample_soft_block(d_node_noise, temperature, batch, d_out)) return;
  SparseCircuit* g = general();
  DevBuf<int32_t> slots;
  slots.upload(noise_slot_, stream);
  g->sample_soft_with_slots(d_node_noise, slots.p, sample_noise_size(), temperature, batch, d_out);
}

}  // namespace pcm
