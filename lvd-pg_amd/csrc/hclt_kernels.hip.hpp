// gfx950 kernels of the dense-block HCLT engine.
//
// Work decomposition.  Examples are independent, tree nodes are not: a node's value needs
// its children's values (forward) and its parent's flows (backward).  The forward and
// backward kernels therefore give each workgroup ONE slice of 16 examples and let it walk
// the whole tree, level by level, its waves taking the nodes of a level in turn and
// meeting at a workgroup barrier -- no grid-wide synchronisation exists anywhere.  The
// sufficient statistics (edge flows summed over the batch, leaf histograms) need the whole
// batch per node instead, so a third kernel gives each workgroup one tree node and all
// slices, recomputing the node's flows from the stored node values.
//
// Register tile.  A wave holds a [16 examples x K states] tile as K/16 float4 per lane:
// lane = 16*g + b owns example b and states kt*16 + 4*g + i (kt < K/16, i < 4).  This is
// both the B-operand layout and the accumulator layout of v_mfma_f32_16x16x4_f32 with the
// parameter block as A-operand (rows = output states), so the output tile of one
// contraction feeds the next one, and HBM, unchanged.  Tiles are stored as K/16 runs of
// 64 float4 (1 KiB, fully coalesced).
#pragma once

#include <hip/hip_runtime.h>

#include "hclt_engine.hpp"

namespace pcm {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kSlice = 16;       // examples per tile
constexpr int kWalkWaves = 16;   // waves per workgroup in the tree-walk kernels
constexpr int kStatWaves = 8;    // most waves per workgroup in the statistics kernel

template <int K>
struct Tile {
  v4f v[K / 16];
};

template <int K>
__device__ __forceinline__ void tile_load(const float* base, int node, int nslices, int slice,
                                          int lane, Tile<K>& t) {
  const v4f* p = reinterpret_cast<const v4f*>(base + ((size_t)node * nslices + slice) * (kSlice * K));
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) t.v[kt] = p[kt * 64 + lane];
}

template <int K>
__device__ __forceinline__ void tile_store(float* base, int node, int nslices, int slice, int lane,
                                           const Tile<K>& t) {
  v4f* p = reinterpret_cast<v4f*>(base + ((size_t)node * nslices + slice) * (kSlice * K));
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) p[kt * 64 + lane] = t.v[kt];
}

// Row of the leaf table for this lane's example: log p(x_b,var | hidden state).
template <int K, bool kFirst>
__device__ __forceinline__ void leaf_row(const HcltDev& d, int var, int bcol, int g, Tile<K>& z) {
  int x = d.xb[(size_t)var * d.Bp + bcol];
  const v4f* row = reinterpret_cast<const v4f*>(d.leaf + ((size_t)var * d.C + x) * K);
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) {
    v4f t = row[kt * 4 + g];
    if (kFirst) z.v[kt] = t; else z.v[kt] += t;
  }
}

// Z = own leaf row + leaf rows of leaf children + value tiles of inner children;
// returns E = exp(Z - m) and the per-example maximum m.
template <int K>
__device__ __forceinline__ float gather_exp(const HcltDev& d, const HcltNode& nd, int slice,
                                            int lane, Tile<K>& e) {
  const int b = lane & 15, g = lane >> 4;
  const int bcol = slice * kSlice + b;
  leaf_row<K, true>(d, nd.var, bcol, g, e);
  for (int c = 0; c < nd.lc_cnt; ++c) leaf_row<K, false>(d, d.child_leaf[nd.lc_off + c], bcol, g, e);
  for (int c = 0; c < nd.ic_cnt; ++c) {
    Tile<K> o;
    tile_load<K>(d.O, d.child_inner[nd.ic_off + c], d.nslices, slice, lane, o);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt) e.v[kt] += o.v[kt];
  }
  float m = -INFINITY;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
    for (int i = 0; i < 4; ++i) m = fmaxf(m, e.v[kt][i]);
  m = fmaxf(m, __shfl_xor(m, 16));
  m = fmaxf(m, __shfl_xor(m, 32));
  if (m == -INFINITY) m = 0.f;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
    for (int i = 0; i < 4; ++i) e.v[kt][i] = __expf(e.v[kt][i] - m);
  return m;
}

// out[b, r] = sum_c W[r, c] * in[b, c] on the matrix cores; Wop is the node's block already
// laid out as A-operands: float4 (row tile rt, column tile ct, lane) holds
// W[rt*16 + lane%16][ct*16 + 4*(lane/16) + 0..3].
template <int K>
__device__ __forceinline__ void contract(const float* Wop, int lane, const Tile<K>& in, Tile<K>& out) {
  constexpr int KT = K / 16;
  const v4f* w = reinterpret_cast<const v4f*>(Wop);
#pragma unroll
  for (int rt = 0; rt < KT; ++rt) {
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ct = 0; ct < KT; ++ct) {
      v4f a = w[(rt * KT + ct) * 64 + lane];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], in.v[ct][i], acc, 0, 0, 0);
    }
    out.v[rt] = acc;
  }
}

// ---- forward: O_v = m + log(E W^T) --------------------------------------------------
template <int K>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_forward_kernel(
    HcltDev d, const int32_t* __restrict__ level_ptr, const int32_t* __restrict__ items,
    int n_levels, float* __restrict__ ll_out) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  for (int L = 0; L < n_levels; ++L) {
    const int beg = level_ptr[L], end = level_ptr[L + 1];
    for (int it = beg + wave; it < end; it += kWalkWaves) {
      const int n = items[it];
      const HcltNode nd = d.nodes[n];
      Tile<K> e, s;
      const float m = gather_exp<K>(d, nd, slice, lane, e);
      contract<K>(d.Wf + (size_t)n * K * K, lane, e, s);
#pragma unroll
      for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) s.v[kt][i] = m + __logf(s.v[kt][i]);
      tile_store<K>(d.O, n, d.nslices, slice, lane, s);
      if (nd.is_root && lane < 16 && slice * kSlice + lane < d.B) ll_out[slice * kSlice + lane] = s.v[0][0];
    }
    __syncthreads();
  }
}

// Flows arriving at the node's K sum nodes divided by their values: R = F / S, S = exp(O - m).
template <int K>
__device__ __forceinline__ void flow_ratio(const HcltDev& d, const HcltNode& nd, int n, int slice,
                                           int lane, float m, Tile<K>& r) {
  Tile<K> o;
  tile_load<K>(d.O, n, d.nslices, slice, lane, o);
  if (nd.is_root) {
    const bool live = lane < 16 && slice * kSlice + lane < d.B;
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt) r.v[kt] = v4f{0.f, 0.f, 0.f, 0.f};
    r.v[0][0] = live ? __expf(m - o.v[0][0]) : 0.f;
  } else {
    tile_load<K>(d.G, nd.parent, d.nslices, slice, lane, r);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) r.v[kt][i] = r.v[kt][i] * __expf(m - o.v[kt][i]);
  }
}

// ---- backward: G_v = E .* (R W), the flow every child of v (and v's own leaf) receives ---
template <int K>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_backward_kernel(
    HcltDev d, const int32_t* __restrict__ level_ptr, const int32_t* __restrict__ items,
    int n_levels) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  for (int L = 0; L < n_levels; ++L) {
    const int beg = level_ptr[L], end = level_ptr[L + 1];
    for (int it = beg + wave; it < end; it += kWalkWaves) {
      const int n = items[it];
      const HcltNode nd = d.nodes[n];
      if (!nd.has_inner_child) continue;   // nobody reads this node's G
      Tile<K> e, r, t;
      const float m = gather_exp<K>(d, nd, slice, lane, e);
      flow_ratio<K>(d, nd, n, slice, lane, m, r);
      contract<K>(d.Wb + (size_t)n * K * K, lane, r, t);
#pragma unroll
      for (int kt = 0; kt < K / 16; ++kt) t.v[kt] *= e.v[kt];
      tile_store<K>(d.G, n, d.nslices, slice, lane, t);
    }
    __syncthreads();
  }
}

// ---- statistics: one workgroup per tree node, all slices ------------------------------
//   edge_aggr[v][k][j] = rate*old + W[k][j] * sum_b R[b,k] E[b,j]
//   leaf_flow[u][c][j] = rate*old + sum_b [x_b,u = c] G_v[b,j]   for u = v and v's leaf children
// LDS: hist_floats floats holding nh histograms of C x (K+1), then per wave two [16][K+16]
// transposition pads.
template <int K>
__global__ __launch_bounds__(kStatWaves * 64) void hclt_stats_kernel(
    HcltDev d, float* __restrict__ edge_aggr, float* __restrict__ leaf_flow, float rate, int nh,
    int hist_floats) {
  constexpr int KT = K / 16;
  constexpr int LD = K + 16;   // row stride of the transposition pads: conflict-free column reads
  extern __shared__ float smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = lane & 15, g = lane >> 4;
  const int nwaves = blockDim.x >> 6;
  const int n = blockIdx.x;
  const HcltNode nd = d.nodes[n];
  const int hist_sz = d.C * (K + 1);
  float* hist = smem;
  float* Rl = smem + hist_floats + (size_t)wave * (2 * kSlice * LD);
  float* El = Rl + kSlice * LD;
  const int nu = 1 + nd.lc_cnt;

  v4f accA[KT][KT];
#pragma unroll
  for (int a = 0; a < KT; ++a)
#pragma unroll
    for (int c = 0; c < KT; ++c) accA[a][c] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int u0 = 0; u0 < nu; u0 += nh) {
    const int nhere = min(nh, nu - u0);
    for (int i = threadIdx.x; i < nhere * hist_sz; i += blockDim.x) hist[i] = 0.f;
    __syncthreads();
    for (int slice = wave; slice < d.nslices; slice += nwaves) {
      Tile<K> e, r, t;
      const float m = gather_exp<K>(d, nd, slice, lane, e);
      flow_ratio<K>(d, nd, n, slice, lane, m, r);
      contract<K>(d.Wb + (size_t)n * K * K, lane, r, t);
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) t.v[kt] *= e.v[kt];
      const int bcol = slice * kSlice + b;
      if (u0 == 0) {
        // A += R^T E over the 16 examples of the tile (contraction over examples)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
          *reinterpret_cast<v4f*>(&Rl[b * LD + kt * 16 + 4 * g]) = r.v[kt];
          *reinterpret_cast<v4f*>(&El[b * LD + kt * 16 + 4 * g]) = e.v[kt];
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          float ra[KT], eb[KT];
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) {
            ra[kt] = Rl[(4 * s + g) * LD + kt * 16 + b];
            eb[kt] = El[(4 * s + g) * LD + kt * 16 + b];
          }
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int jt = 0; jt < KT; ++jt)
              accA[kt][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[kt], eb[jt], accA[kt][jt], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      if (bcol < d.B) {
        for (int h = 0; h < nhere; ++h) {
          const int u = (u0 + h == 0) ? nd.var : d.child_leaf[nd.lc_off + u0 + h - 1];
          const int x = d.xb[(size_t)u * d.Bp + bcol];
          float* hrow = hist + (size_t)h * hist_sz + x * (K + 1);
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              __hip_atomic_fetch_add(&hrow[kt * 16 + 4 * g + i], t.v[kt][i], __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
    __syncthreads();
    for (int h = 0; h < nhere; ++h) {
      const int u = (u0 + h == 0) ? nd.var : d.child_leaf[nd.lc_off + u0 + h - 1];
      float* dst = leaf_flow + (size_t)u * d.C * K;
      const float* src = hist + (size_t)h * hist_sz;
      for (int i = threadIdx.x; i < d.C * K; i += blockDim.x) {
        const int c = i / K, j = i % K;
        const float old = rate != 0.f ? rate * dst[i] : 0.f;
        dst[i] = old + src[c * (K + 1) + j];
      }
    }
    __syncthreads();
  }

  // combine the waves' partial A through LDS, scale by W, write the node's block once
  float* abuf = smem;
  for (int i = threadIdx.x; i < K * K; i += blockDim.x) abuf[i] = 0.f;
  __syncthreads();
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int jt = 0; jt < KT; ++jt)
#pragma unroll
      for (int v = 0; v < 4; ++v)
        __hip_atomic_fetch_add(&abuf[(kt * 16 + 4 * g + v) * K + jt * 16 + b], accA[kt][jt][v],
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  __syncthreads();
  float* dst = edge_aggr + (size_t)n * K * K;
  const float* lt = d.logtheta + (size_t)n * K * K;
  for (int i = threadIdx.x; i < K * K; i += blockDim.x) {
    const float old = rate != 0.f ? rate * dst[i] : 0.f;
    dst[i] = old + __expf(lt[i]) * abuf[i];
  }
}

// ---- parameter kernels ----------------------------------------------------------------
template <int K>
__device__ __forceinline__ void put_w(float* Wf, float* Wb, int k, int j, float w) {
  constexpr int KT = K / 16;
  Wf[(((k / 16) * KT + j / 16) * 64 + ((j % 16) / 4) * 16 + k % 16) * 4 + j % 4] = w;
  Wb[(((j / 16) * KT + k / 16) * 64 + ((k % 16) / 4) * 16 + j % 16) * 4 + k % 4] = w;
}

// Wf / Wb from the log-parameters (after parameters were set from outside).
template <int K>
__global__ void hclt_rebuild_w_kernel(const float* __restrict__ logtheta, float* __restrict__ Wf,
                                      float* __restrict__ Wb, int n_inner) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)n_inner * K * K) return;
  const int n = (int)(i / (K * K)), k = (int)(i / K) % K, j = (int)(i % K);
  put_w<K>(Wf + (size_t)n * K * K, Wb + (size_t)n * K * K, k, j, __expf(logtheta[i]));
}

// Sum-edge update, one thread per sum node (tree node n, state k):
// add_pseudocount, aggr_node_flows, update_params of the reference's EM step.
template <int K>
__global__ void hclt_theta_update_kernel(const HcltNode* __restrict__ nodes, float* __restrict__ logtheta,
                                         float* __restrict__ Wf, float* __restrict__ Wb,
                                         float* __restrict__ edge_aggr, int n_inner,
                                         float pseudocount, float inertia) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_inner * K) return;
  const int n = i / K, k = i % K;
  if (nodes[n].is_root && k > 0) return;
  float* a = edge_aggr + ((size_t)n * K + k) * K;
  float* lt = logtheta + ((size_t)n * K + k) * K;
  const float share = pseudocount / (float)K;
  float tot = 0.f;
  for (int j = 0; j < K; ++j) {
    a[j] += share;
    tot += a[j];
  }
  for (int j = 0; j < K; ++j) {
    const float oldv = inertia * expf(lt[j]);
    const float newv = (1.f - inertia) * a[j] / tot;
    const float l = logf(oldv + newv);
    lt[j] = l;
    put_w<K>(Wf + (size_t)n * K * K, Wb + (size_t)n * K * K, k, j, expf(l));
  }
}

// Leaf update, one thread per (variable, hidden state); categories are strided by K so
// consecutive threads touch consecutive addresses.
__global__ void hclt_leaf_update_kernel(float* __restrict__ leaf, const float* __restrict__ leaf_flow,
                                        int V, int C, int K, float pseudocount, float inertia) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= V * K) return;
  const int u = i / K, j = i % K;
  float* lp = leaf + (size_t)u * C * K + j;
  const float* fl = leaf_flow + (size_t)u * C * K + j;
  float node_flow = 0.f;
  for (int c = 0; c < C; ++c) node_flow += fl[(size_t)c * K];
  node_flow += pseudocount;
  const float cat_pc = pseudocount / (float)C;
  for (int c = 0; c < C; ++c) {
    const float oldv = inertia * expf(lp[(size_t)c * K]);
    const float newv = (1.f - inertia) * (fl[(size_t)c * K] + cat_pc) / node_flow;
    lp[(size_t)c * K] = logf(oldv + newv);
  }
}

// Batch rows -> xb[var][example] (example fastest), through a 64 x 64 LDS tile.
__global__ __launch_bounds__(256) void hclt_stage_kernel(const uint8_t* __restrict__ data,
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
