// KL divergence between two HCLTs of one structure, its gradient, and the Adam step, on the
// block form.
//
// With P_v = exp(theta1_v) (K x K, row k = state of the tree parent), D_v = theta1_v - theta2_v,
// l_v[j] = KL of the leaf distributions of v's own variable and of its leaf tree children at
// hidden state j, the recursion of the reference (src/queries/kld.jl:95-128: a sum edge gives
// p1 * (kld(children) + logp1 - logp2), a product adds its children) reads
//   Z_v[j]  = l_v[j] + sum over non-leaf tree children c of KL_c[j]
//   KL_v[k] = sum_j P_v[k,j] * (Z_v[j] + D_v[k,j])
// and its reverse pass (src/queries/kld.jl:262-300, root gradient 1)
//   h_v[j]  = sum_k g_v[k] * P_v[k,j],   g_c = h_v for every tree child c, g_root = e_0
//   d/dtheta1_v[k,j] = g_v[k] * (P_v[k,j] * (Z_v[j] + D_v[k,j]) + P_v[k,j]),  d/dtheta2 = -g_v[k] * P_v[k,j]
// with the leaf lines written as the reference has them (src/queries/kld.jl:528-535,
// src/nodes/fixable_categorical_dist.jl:219): g * (a - b + 1) and g * exp(a - b).
//
// Only the two K-vector chains (KL_v up the tree, h_v down the tree) are sequential; one
// workgroup walks each of them level by level (deepest level first / root first), sixteen tree
// nodes (one per wave) between barriers.  A step's vectors stay in an LDS ring indexed by chain
// slot (a node's tree neighbours sit at most two levels' widths away), and the parameters of
// the steps to come are requested several steps ahead, so a step costs an LDS round trip and
// the chain runs at the rate one compute unit pulls the parameters from L2.  Everything else is
// a data-parallel kernel.
#include "hclt_engine.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>

namespace pcm {

static void check_launch_k(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

// kl_leaf[v][j] = sum_c exp(a) * (a - b), a = leaf1[v][c][j], b = leaf2[v][c][j]
// (src/nodes/fixable_categorical_dist.jl:187-192 in log-parameter form).
__global__ __launch_bounds__(256) void hclt_kld_leaf_kernel(const float* __restrict__ leaf1,
                                                            const float* __restrict__ leaf2, int K, int C,
                                                            float* __restrict__ kl_leaf) {
  __shared__ float part[256];
  const int v = blockIdx.x, t = threadIdx.x;
  const int j = t % K, cc = t / K, P = 256 / K;
  float acc = 0.f;
  if (cc < P) {
    const float* a = leaf1 + (size_t)v * C * K + j;
    const float* b = leaf2 + (size_t)v * C * K + j;
    for (int c = cc; c < C; c += P) {
      const float x = a[(size_t)c * K], y = b[(size_t)c * K];
      acc += expf(x) * (x - y);
    }
  }
  part[t] = acc;
  __syncthreads();
  if (t < K) {
    float s = 0.f;
    for (int q = 0; q < P; ++q) s += part[q * K + t];
    kl_leaf[(size_t)v * K + t] = s;
  }
}

// One tree node of a chain step (16 bytes, one vector load).
struct KlItem {
  int32_t n;      // inner id, -1: this wave idles
  int32_t c[3];   // up: chain slots of the non-leaf tree children (-1 none); c[2] <= -2: the third and
                  // further children are listed at ext[-(c[2] + 2)]: their number, then their slots
                  // down: c[0] = the parent's slot (-1: the root)
};
static_assert(sizeof(KlItem) == 16, "KlItem is read as one 16-byte word");

// Waves (= nodes per step) of a chain workgroup and the steps of parameters a lane keeps
// requested ahead: as many as its registers hold.
constexpr int kl_waves(int K) { return K > 32 ? 8 : 16; }
constexpr int kl_ahead(int K) { return K > 32 ? 2 : 4; }

// Operand layout of the chains: lane (part, r) of a wave, part = lane / K, r = lane % K, owns
// rows part * JP .. + JP (JP = K * K / 64) of its node's K x K operand at column r; the JP values
// are consecutive, so a step's operand is JP / 4 loads of 16 bytes per lane, 1 KB per wave each:
// word ((i / 4) * 64 + lane) * 4 + i % 4 of the slot holds row part * JP + i.

// Per tree node, everything of the recursion that does not wait for other nodes, stored where
// the chains will look for it: slot su = pos[n] of the upward chain's steps, slot sd =
// pos[n_inner + n] of the downward chain's.
//   ell[su][j]  = l_v[j]
//   base[su][k] = sum_j P[k,j] * (D[k,j] + ell[j])
//   pu[su]: operand (row j, column k) = P[k,j]   (upward chain: a lane's column is k)
//   pd[sd]: operand (row k, column j) = P[k,j]   (downward chain: a lane's column is j)
template <int K>
__global__ __launch_bounds__(256) void hclt_kld_base_kernel(const HcltNode* __restrict__ nodes,
                                                            const int32_t* __restrict__ child_leaf,
                                                            const int32_t* __restrict__ pos, int n_inner,
                                                            const float* __restrict__ theta1,
                                                            const float* __restrict__ theta2,
                                                            const float* __restrict__ kl_leaf, float* __restrict__ ell,
                                                            float* __restrict__ base, float* __restrict__ pu,
                                                            float* __restrict__ pd) {
  __shared__ float tile[K][K + 1];
  __shared__ float l[K];
  const int n = blockIdx.x, t = threadIdx.x;
  const HcltNode nd = nodes[n];
  const size_t su = (size_t)pos[n], sd = (size_t)pos[n_inner + n];
  if (t < K) {
    float s = kl_leaf[(size_t)nd.var * K + t];
    for (int q = 0; q < nd.lc_cnt; ++q) s += kl_leaf[(size_t)child_leaf[nd.lc_off + q] * K + t];
    l[t] = s;
    ell[su * K + t] = s;
  }
  __syncthreads();
  const int j = t % K;
  for (int k = t / K; k < K; k += 256 / K) {
    const float x = theta1[((size_t)n * K + k) * K + j], y = theta2[((size_t)n * K + k) * K + j];
    const float p = expf(x);
    tile[k][j] = p;
    float term = p > 0.f ? p * (x - y + l[j]) : 0.f;   // absent edges (the root's rows past the first) carry -inf
#pragma unroll
    for (int o = K / 2; o > 0; o >>= 1) term += __shfl_xor(term, o, K);
    if (j == 0) base[su * K + k] = term;
  }
  __syncthreads();
  // consecutive threads write consecutive words of the operand: word w = ((i4 * 64) + lane) * 4 + e
  constexpr int JP = K * K / 64;
  for (int w = t; w < K * K; w += 256) {
    const int e = w & 3, lane = (w >> 2) & 63, i4 = w >> 8;
    const int row = (lane / K) * JP + i4 * 4 + e, col = lane % K;
    pu[su * K * K + w] = tile[col][row];
    pd[sd * K * K + w] = tile[row][col];
  }
}

// Distances in floats between the arrays of consecutive rows when the chains run on a matrix of parameter rows (one
// pair of chains per row, blockIdx.y); all zero for the circuit's own parameters.
struct KlRowStrides {
  size_t pu, pd, vec, out, ring_up, ring_down;
  int down_only;   // 1: the launch has one workgroup per row and it walks down (the relaxed sampler on rows)
};

// The two chains.  Workgroup 0 walks up (KL_v, Z_v), workgroup 1 walks down (h_v); launched
// with one workgroup when only the divergence is wanted.  A step is kl_waves(K) independent
// nodes (same level).  The vectors a step reads were left in the ring by earlier steps of the
// same workgroup (slot & ring_mask; the host sizes the ring beyond the largest distance between
// a node and its tree neighbours), so a barrier orders them.  kLds: the ring is in LDS;
// otherwise (levels too wide for that) it is the whole chain in device memory.  The item,
// operand and constants of a step are requested D = kl_ahead(K) steps before it; the chains are
// padded to a multiple of D steps and the tables by D idle steps more, so the requests need no
// bounds and every lane's requests complete in the order the steps use them.
template <int K, bool kLds>
__global__ __launch_bounds__(kl_waves(K) * 64) void hclt_kld_chain_kernel(
    const KlItem* __restrict__ up_items, int up_steps, const KlItem* __restrict__ down_items, int down_steps,
    const int32_t* __restrict__ ext, const float* __restrict__ pu, const float* __restrict__ base,
    const float* __restrict__ ell, const float* __restrict__ pd, int ring_mask, float* ring_up, float* ring_down,
    float* __restrict__ klv, float* __restrict__ z, float* __restrict__ h, KlRowStrides rs) {
  constexpr int PARTS = 64 / K, JP = K / PARTS, Q = JP / 4, W = kl_waves(K), D = kl_ahead(K);
  extern __shared__ float lds_ring[];   // kLds: [ring_mask + 1][K]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane % K, part = lane / K;
  const bool up = blockIdx.x == 0 && !rs.down_only;
  {   // a row of a parameter matrix per blockIdx.y: its operands, constants and results sit rs.* floats further on
    const size_t row = blockIdx.y;
    pu += row * rs.pu; pd += row * rs.pd; base += row * rs.vec; ell += row * rs.vec;
    klv += row * rs.out; z += row * rs.out; h += row * rs.out;
    if (ring_up) ring_up += row * rs.ring_up;
    if (ring_down) ring_down += row * rs.ring_down;
  }
  const int steps = up ? up_steps : down_steps;
  const int4* __restrict__ items = reinterpret_cast<const int4*>(up ? up_items : down_items);
  const float4* __restrict__ par = reinterpret_cast<const float4*>(up ? pu : pd);
  float* ring_dev = up ? ring_up : ring_down;
  auto ring_at = [&](int slot) -> float* {
    if constexpr (kLds) return lds_ring + (size_t)(slot & ring_mask) * K;
    else return ring_dev + (size_t)slot * K;
  };
  // The first round (q0 = -D) computes nothing and only places the requests of steps 0 .. D-1:
  // with every request issued from the same place in the loop, the waits the compiler counts
  // from the order of issue let D - 1 steps of requests stay in flight.
  int4 it[D];
  float4 p[D][Q];
  float bs[D], el[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    it[d] = make_int4(-1, -1, -1, -1);
#pragma unroll
    for (int e = 0; e < Q; ++e) p[d][e] = make_float4(0.f, 0.f, 0.f, 0.f);
    bs[d] = el[d] = 0.f;
  }
  for (int q0 = -D; q0 < steps; q0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int q = q0 + d;   // steps is a multiple of D (idle steps at the end): no way round a step
      const int64_t slot = (int64_t)q * W + wave;
      const int n = __builtin_amdgcn_readfirstlane(it[d].x);
      const int c0 = __builtin_amdgcn_readfirstlane(it[d].y), c1 = __builtin_amdgcn_readfirstlane(it[d].z),
                c2 = __builtin_amdgcn_readfirstlane(it[d].w);
      if (n >= 0) {
        float acc = 0.f, s = 0.f;
        auto take = [&](int cslot) {   // acc += sum_i operand[part * JP + i] * vector[part * JP + i]
          const float* cv = ring_at(cslot);
          if (up) s += cv[r];
#pragma unroll
          for (int e = 0; e < Q; ++e) {
            const float4 x = *reinterpret_cast<const float4*>(cv + part * JP + 4 * e);
            acc += p[d][e].x * x.x + p[d][e].y * x.y + p[d][e].z * x.z + p[d][e].w * x.w;
          }
        };
        if (up) {
          if (c0 >= 0) take(c0);
          if (c1 >= 0) take(c1);
          if (c2 >= 0) take(c2);
          if (c2 < -1) {
            const int32_t* more = ext + (-(c2 + 2));
            const int cnt = more[0];
            for (int i = 0; i < cnt; ++i) take(more[1 + i]);
          }
        } else if (c0 >= 0) {
          take(c0);
        } else {
          acc = part == 0 ? p[d][0].x : 0.f;   // the root's incoming vector is e_0: row 0 of its operand
        }
#pragma unroll
        for (int o = K; o < 64; o <<= 1) acc += __shfl_xor(acc, o);
        if (part == 0) {
          const float out = up ? bs[d] + acc : acc;
          ring_at((int)slot)[r] = out;
          if (up) {
            klv[(size_t)n * K + r] = out;
            z[(size_t)n * K + r] = el[d] + s;
          } else {
            h[(size_t)n * K + r] = out;
          }
        }
      }
      const size_t nx = (size_t)(slot + D * W);
      it[d] = items[nx];
#pragma unroll
      for (int e = 0; e < Q; ++e) p[d][e] = par[(nx * Q + e) * 64 + lane];
      bs[d] = base[nx * K + r];
      el[d] = ell[nx * K + r];
      __syncthreads();
    }
  }
}

// Gradients of the sum parameters, in parameter-vector order (src/queries/kld.jl:271-272).
__global__ void hclt_kld_edge_grad_kernel(int64_t ns, int K, const int64_t* __restrict__ src,
                                          const int32_t* __restrict__ parent_of, const float* __restrict__ theta1,
                                          const float* __restrict__ theta2, const float* __restrict__ z,
                                          const float* __restrict__ h, float* __restrict__ gp,
                                          float* __restrict__ gq) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= ns) return;
  const int64_t s = src[i];
  const int j = (int)(s % K), k = (int)((s / K) % K);
  const int n = (int)(s / ((int64_t)K * K));
  const int par = parent_of[n];
  const float g = par < 0 ? 1.f : h[(size_t)par * K + k];
  const float a = theta1[s], b = theta2[s], p1 = expf(a);
  const float ek = p1 * (z[(size_t)n * K + j] + a - b);
  gp[i] = g * (ek + p1);
  gq[i] = -g * p1;
}

// Gradients of the leaf parameters: [V][C][K] tables in, parameter-vector order out (the C
// categories of input node (v, j) contiguous at in_pos[v][j] * C), 64 categories of one
// variable per workgroup, turned around in LDS.
constexpr int kLeafGradCats = 64;

__global__ __launch_bounds__(256) void hclt_kld_leaf_grad_kernel(const float* __restrict__ leaf1,
                                                                 const float* __restrict__ leaf2,
                                                                 const int32_t* __restrict__ state_node,
                                                                 const int32_t* __restrict__ in_pos,
                                                                 const float* __restrict__ h, int K, int C,
                                                                 float* __restrict__ gp, float* __restrict__ gq) {
  extern __shared__ float lg[];   // two tiles [kLeafGradCats][K + 1]
  const int v = blockIdx.x, c0 = blockIdx.y * kLeafGradCats, t = threadIdx.x;
  const int nc = min(kLeafGradCats, C - c0);
  float* t1 = lg;
  float* t2 = lg + kLeafGradCats * (K + 1);
  {
    const int j = t % K;
    const float g = h[(size_t)state_node[v] * K + j];
    for (int cc = t / K; cc < nc; cc += 256 / K) {
      const size_t at = ((size_t)v * C + c0 + cc) * K + j;
      const float a = leaf1[at], b = leaf2[at];
      t1[cc * (K + 1) + j] = g * (a - b + 1.f);
      t2[cc * (K + 1) + j] = g * expf(a - b);
    }
  }
  __syncthreads();
  const int cc = t % kLeafGradCats;
  if (cc < nc)
    for (int j = t / kLeafGradCats; j < K; j += 256 / kLeafGradCats) {
      const size_t at = (size_t)in_pos[(size_t)v * K + j] * C + c0 + cc;
      gp[at] = t1[cc * (K + 1) + j];
      gq[at] = t2[cc * (K + 1) + j];
    }
}

// Adam on the sum parameters (src/sgd/adam.jl:318-319 moments, :63-76 ascent step) and the
// per-sum-node normalisation into the circuit (:88-127), in one pass: every normalisation
// group of an HCLT is K consecutive entries of the parameter vector.
template <int K>
__global__ __launch_bounds__(256) void hclt_adam_kernel(int64_t ns, const float* __restrict__ grad,
                                                        float* __restrict__ params, float* __restrict__ m,
                                                        float* __restrict__ v, float lr, float b1, float b2, float eps,
                                                        float c1, float c2, const int64_t* __restrict__ src,
                                                        float* __restrict__ logtheta) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool live = i < ns;
  float p = -INFINITY;
  if (live) {
    const float g = grad[i];
    const float mi = b1 * m[i] + (1.f - b1) * g;
    const float vi = b2 * v[i] + (1.f - b2) * g * g;
    m[i] = mi;
    v[i] = vi;
    p = params[i] + lr * ((mi / c1) / (sqrtf(vi / c2) + eps));
    params[i] = p;
  }
  float s = expf(p);
  if constexpr (K <= 64) {
#pragma unroll
    for (int o = K / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, K);
  } else {   // K = 128: a group is two neighbouring waves of the workgroup
    static_assert(K == 128, "a normalisation group is at most two waves");
    __shared__ float half[4];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) half[wave] = s;
    __syncthreads();
    s = half[wave & ~1] + half[wave | 1];
  }
  if (live) logtheta[src[i]] = p - logf(s);
}

// Adam from flows (src/sgd/adam.jl:305-311, :27-61): gradient of the mean log-likelihood with respect to the
// unnormalised log-parameters, edge flows / batch size minus exp(theta) times their sum over the sum node.  A sum
// node is a row of K entries of the block arrays: first the row sums (a wave per row), then one thread per parameter.
__global__ __launch_bounds__(256) void hclt_row_sum_kernel(const float* __restrict__ edge_aggr, int64_t rows, int K,
                                                           float* __restrict__ row_sum) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  float s = 0.f;
  for (int j = lane; j < K; j += 64) s += edge_aggr[r * K + j];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) row_sum[r] = s;
}

__global__ void hclt_flow_grad_kernel(int64_t ns, const int64_t* __restrict__ src, const float* __restrict__ edge_aggr,
                                      const float* __restrict__ logtheta, const float* __restrict__ row_sum, int K,
                                      float inv_batch, float* __restrict__ grad) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= ns) return;
  const int64_t at = src[i];
  grad[i] = (edge_aggr[at] - expf(logtheta[at]) * row_sum[at / K]) * inv_batch;
}

// Adam on the input nodes (src/sgd/adam.jl:218-242), one thread per leaf parameter in parameter order: node (v, j)
// at position q has its C values at q * C; the tables are [V][C][K].  g = flow + exp(logp) * node flow, as the
// source has it; the steps go to the auxiliary copy, the circuit's leaves are not written.
__global__ __launch_bounds__(256) void hclt_leaf_node_flow_kernel(const float* __restrict__ leaf_flow, int C, int K,
                                                                  float* __restrict__ node_flow) {
  const int v = blockIdx.x;
  for (int j = threadIdx.x; j < K; j += blockDim.x) {
    float s = 0.f;
    for (int c = 0; c < C; ++c) s += leaf_flow[((size_t)v * C + c) * K + j];
    node_flow[(size_t)v * K + j] = s;
  }
}

__global__ __launch_bounds__(256) void hclt_leaf_adam_kernel(int64_t n_leaf, const int32_t* __restrict__ input_order, int C,
                                                             int K, const float* __restrict__ leaf,
                                                             const float* __restrict__ leaf_flow,
                                                             const float* __restrict__ node_flow, float* __restrict__ aux_p,
                                                             float* __restrict__ aux_m, float* __restrict__ aux_v, float lr,
                                                             float b1, float b2, float eps, float c1, float c2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_leaf) return;
  const int vj = input_order[i / C], c = (int)(i % C);
  const int v = vj / K, j = vj % K;
  const size_t at = ((size_t)v * C + c) * K + j;
  const float g = leaf_flow[at] + expf(leaf[at]) * node_flow[vj];
  const float m = b1 * aux_m[i] + (1.f - b1) * g, vv = b2 * aux_v[i] + (1.f - b2) * g * g;
  aux_m[i] = m;
  aux_v[i] = vv;
  aux_p[i] += lr * ((m / c1) / (sqrtf(vv / c2) + eps));
}

// ---- host --------------------------------------------------------------------------------

void HcltCircuit::flow_gradients(int32_t batch_size, float* d_grad) {
  no_forest("this query");
  no_missing("this query");
  if (!have_flows_) fail(PCM_ERR_STATE, "no flows have been computed on this circuit yet");
  if (flows_in_general_ || (!block_ && !wide_)) return general_->flow_gradients(batch_size, d_grad);
  if (!d_grad) fail(PCM_ERR_ARG, "gradient pointer is null");
  if (batch_size < 1) fail(PCM_ERR_ARG, "batch size must be positive, got %d", batch_size);
  const int64_t ns = (int64_t)sum_param_src_.size();
  const int64_t rows = (int64_t)n_inner_ * K_ + H_;
  d_row_sum_.ensure((size_t)rows);
  hipLaunchKernelGGL(hclt_row_sum_kernel, dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, stream, d_edge_aggr_.p, rows, K_,
                     d_row_sum_.p);
  hipLaunchKernelGGL(hclt_flow_grad_kernel, dim3((unsigned)ceil_div(ns, 256)), dim3(256), 0, stream, ns, d_sum_param_src_.p,
                     d_edge_aggr_.p, d_logtheta_.p, d_row_sum_.p, K_, 1.f / (float)batch_size, d_grad);
  check_launch_k("hclt_flow_grad");
}

void HcltCircuit::leaf_adam(float* d_aux_p, float* d_aux_m, float* d_aux_v, float lr, float b1, float b2, float eps, int t) {
  no_forest("Adam");
  no_missing("Adam");
  if (!have_flows_) fail(PCM_ERR_STATE, "no flows have been computed on this circuit yet");
  if (flows_in_general_ || (!block_ && !wide_)) return general_->leaf_adam(d_aux_p, d_aux_m, d_aux_v, lr, b1, b2, eps, t);
  if (!d_aux_p || !d_aux_m || !d_aux_v) fail(PCM_ERR_ARG, "null optimiser array");
  if (t < 1) fail(PCM_ERR_ARG, "step count must start at 1, got %d", t);
  if (d_input_order_.n == 0) d_input_order_.upload(input_order_, stream);
  d_row_sum_.ensure((size_t)V_ * K_);
  hipLaunchKernelGGL(hclt_leaf_node_flow_kernel, dim3(V_), dim3(std::min(256, ceil_div(K_, 64) * 64)), 0, stream,
                     d_leaf_flow_.p, C_, K_, d_row_sum_.p);
  const int64_t n_leaf = (int64_t)Vu_ * K_ * C_;   // (the caller's variables: auxiliary ones have no parameters)
  const float c1 = 1.f - std::pow(b1, (float)t), c2 = 1.f - std::pow(b2, (float)t);
  hipLaunchKernelGGL(hclt_leaf_adam_kernel, dim3((unsigned)ceil_div(n_leaf, 256)), dim3(256), 0, stream, n_leaf,
                     d_input_order_.p, C_, K_, d_leaf_.p, d_leaf_flow_.p, d_row_sum_.p, d_aux_p, d_aux_m, d_aux_v, lr, b1, b2,
                     eps, c1, c2);
  check_launch_k("hclt_leaf_adam");
}

HcltCircuit* HcltCircuit::same_tree(pcm_circuit* q) {
  no_forest("this query");
  no_missing("this query");
  if (H_ > 0) fail(PCM_ERR_UNSUPPORTED, "KL of multi-head circuits is not defined");
  auto* o = dynamic_cast<HcltCircuit*>(q);
  if (!o) fail(PCM_ERR_ARG, "the two circuits of a KL query must be of the same kind");
  o->no_forest("this query");
  o->no_missing("this query");
  if (o->K_ != K_ || o->C_ != C_ || o->H_ != H_ || o->parent_ != parent_)
    fail(PCM_ERR_SHAPE, "the two circuits of a KL query must share one structure");
  return o;
}

void HcltCircuit::build_kld_tables() {
  no_forest("this query");
  no_missing("this query");
  if (d_kl_up_.n) return;
  const int W = kl_waves(K_), D = kl_ahead(K_);
  std::vector<int32_t> pos((size_t)2 * n_inner_, 0);
  std::vector<int32_t> ext;
  int reach = 0;   // largest distance in chain slots between a node and a tree neighbour it reads
  auto chain = [&](bool up) {
    // nodes level by level (up: deepest level first, down: from the root), each level padded to
    // whole steps; D idle steps at the end for the requests that run ahead
    std::vector<std::vector<int32_t>> lv;
    for (int n = 0; n < n_inner_; ++n) {
      const size_t at = (size_t)depth_[var_of_inner_[n]];
      if (lv.size() <= at) lv.resize(at + 1);
      lv[at].push_back(n);
    }
    if (up) std::reverse(lv.begin(), lv.end());
    const KlItem idle{-1, {-1, -1, -1}};
    std::vector<KlItem> items;
    for (const auto& level : lv) {
      for (int32_t n : level) {
        KlItem it = idle;
        it.n = n;
        const int v = var_of_inner_[n];
        const int32_t me = (int32_t)items.size();
        if (up) {
          std::vector<int32_t> cs;
          for (int c : children_[v])
            if (!children_[c].empty()) cs.push_back(pos[inner_of_var_[c]]);
          for (int32_t c : cs) reach = std::max(reach, me - c);
          for (size_t i = 0; i < cs.size() && i < 3; ++i) it.c[i] = cs[i];
          if (cs.size() > 3) {
            it.c[2] = -((int32_t)ext.size() + 2);
            ext.push_back((int32_t)cs.size() - 2);
            ext.insert(ext.end(), cs.begin() + 2, cs.end());
          }
        } else if (parent_[v] >= 0) {
          it.c[0] = pos[n_inner_ + inner_of_var_[parent_[v]]];
          reach = std::max(reach, me - it.c[0]);
        }
        pos[(up ? 0 : n_inner_) + n] = me;
        items.push_back(it);
      }
      while (items.size() % W) items.push_back(idle);
    }
    while (items.size() % ((size_t)D * W)) items.push_back(idle);   // whole rounds of D steps
    items.resize(items.size() + (size_t)D * W, idle);
    return items;
  };
  std::vector<KlItem> up = chain(true), down = chain(false);
  kl_up_steps_ = (int)(up.size() / W) - D;
  kl_down_steps_ = (int)(down.size() / W) - D;
  // the ring: a power of two of slots beyond the reach, in LDS when 64 KB hold it
  int ring = 1;
  while (ring < reach + W) ring <<= 1;
  kl_ring_slots_ = (size_t)ring * K_ * sizeof(float) <= (size_t)64 * 1024 ? ring : 0;
  std::vector<int32_t> raw(up.size() * 4), rawd(down.size() * 4);
  std::memcpy(raw.data(), up.data(), up.size() * sizeof(KlItem));
  std::memcpy(rawd.data(), down.data(), down.size() * sizeof(KlItem));
  d_kl_down_.upload(rawd, stream);
  d_kl_pos_.upload(pos, stream);
  if (ext.empty()) ext.push_back(0);
  d_kl_ext_.upload(ext, stream);
  // per inner node: its parent | per variable: the inner node whose h reaches its leaf |
  // per input node (v, j): its position among the input nodes of the parameter vector
  std::vector<int32_t> t((size_t)n_inner_ + V_ + (size_t)V_ * K_, 0);
  for (int n = 0; n < n_inner_; ++n) {
    const int v = var_of_inner_[n];
    t[n] = parent_[v] < 0 ? -1 : inner_of_var_[parent_[v]];
  }
  for (int v = 0; v < V_; ++v)
    t[(size_t)n_inner_ + v] = children_[v].empty() ? inner_of_var_[parent_[v]] : inner_of_var_[v];
  for (size_t q = 0; q < input_order_.size(); ++q) t[(size_t)n_inner_ + V_ + input_order_[q]] = (int32_t)q;
  d_kl_tabs_.upload(t, stream);
  d_kl_up_.upload(raw, stream);   // last: marks the tables as built
}

// Runs the recursion of this circuit (p) against q; with_down also leaves h.
void HcltCircuit::kld_device(HcltCircuit* q, bool with_down) {
  build_kld_tables();
  const int W = kl_waves(K_), D = kl_ahead(K_);
  const size_t nk = (size_t)n_inner_ * K_;
  // chain slots, idle ones and the idle steps at the end included
  const size_t su = (size_t)(kl_up_steps_ + D) * W, sd = (size_t)(kl_down_steps_ + D) * W;
  const size_t sm = std::max(su, sd);   // ell and base have a row per slot of the longer chain: both chains request them
  d_kl_leaf_.ensure((size_t)V_ * K_);
  if (!d_kl_vec_.n) {
    d_kl_vec_.alloc(3 * nk + 2 * sm * K_ + (kl_ring_slots_ ? 0 : (su + sd) * K_));   // klv | z | h | ell | base | rings
    d_kl_par_.alloc((su + sd) * K_ * K_);    // pu | pd; idle slots are read (and ignored) by idle waves
    d_kl_vec_.zero(stream);
    d_kl_par_.zero(stream);
  }
  float* klv = d_kl_vec_.p;
  float* z = klv + nk;
  float* h = z + nk;
  float* ell = h + nk;
  float* base = ell + sm * K_;
  float* ring_up = kl_ring_slots_ ? nullptr : base + sm * K_;
  float* ring_down = kl_ring_slots_ ? nullptr : ring_up + su * K_;
  float* pu = d_kl_par_.p;
  float* pd = pu + su * K_ * K_;
  hipLaunchKernelGGL(hclt_kld_leaf_kernel, dim3(V_), dim3(256), 0, stream, d_leaf_.p, q->d_leaf_.p, K_, C_, d_kl_leaf_.p);
  PCM_DISPATCH_K(K_, {
    hipLaunchKernelGGL(hclt_kld_base_kernel<KK>, dim3(n_inner_), dim3(256), 0, stream, d_nodes_.p, d_child_leaf_.p,
                       d_kl_pos_.p, n_inner_, d_logtheta_.p, q->d_logtheta_.p, d_kl_leaf_.p, ell, base, pu, pd);
    auto chain = [&](auto kernel, size_t lds) {
      hipLaunchKernelGGL(kernel, dim3(with_down ? 2 : 1), dim3(kl_waves(KK) * 64), lds, stream,
                         reinterpret_cast<const KlItem*>(d_kl_up_.p), kl_up_steps_,
                         reinterpret_cast<const KlItem*>(d_kl_down_.p), kl_down_steps_, d_kl_ext_.p, pu, base, ell, pd,
                         kl_ring_slots_ - 1, ring_up, ring_down, klv, z, h, KlRowStrides{0, 0, 0, 0, 0, 0, 0});
    };
    if (kl_ring_slots_) chain(&hclt_kld_chain_kernel<KK, true>, (size_t)kl_ring_slots_ * KK * sizeof(float));
    else chain(&hclt_kld_chain_kernel<KK, false>, 0);
  });
  check_launch_k("hclt_kld");
}

void HcltCircuit::kld(pcm_circuit* q, float* out) {
  HcltCircuit* o = same_tree(q);
  check_walks();
  o->check_walks();
  if (!block_) {
    general()->kld(o->general(), out);
    return;
  }
  kld_device(o, false);
  const float* klv = d_kl_vec_.p;
  PCM_HIP(hipMemcpyAsync(out, klv + (size_t)inner_of_var_[root_] * K_, sizeof(float), hipMemcpyDeviceToHost, stream));
  PCM_HIP(hipStreamSynchronize(stream));
}

void HcltCircuit::kld_backward_dev(pcm_circuit* q, float* d_gp, float* d_gq, int64_t n) {
  HcltCircuit* o = same_tree(q);
  if (!block_) {
    general()->kld_backward_dev(o->general(), d_gp, d_gq, n);
    return;
  }
  if (n != size(0)) fail(PCM_ERR_ARG, "gradient vectors have %lld entries, circuit has %lld parameters", (long long)n, (long long)size(0));
  if (!d_gp || !d_gq) fail(PCM_ERR_ARG, "gradient pointer is null");
  kld_device(o, true);
  const size_t nk = (size_t)n_inner_ * K_;
  const float* z = d_kl_vec_.p + nk;
  const float* h = d_kl_vec_.p + 2 * nk;
  const int64_t ns = (int64_t)sum_param_src_.size();
  hipLaunchKernelGGL(hclt_kld_edge_grad_kernel, dim3((unsigned)ceil_div(ns, 256)), dim3(256), 0, stream, ns, K_,
                     d_sum_param_src_.p, d_kl_tabs_.p, d_logtheta_.p, o->d_logtheta_.p, z, h, d_gp, d_gq);
  // (the caller's variables: an auxiliary one has no parameters to differentiate)
  hipLaunchKernelGGL(hclt_kld_leaf_grad_kernel, dim3(Vu_, ceil_div(C_, kLeafGradCats)), dim3(256),
                     2 * kLeafGradCats * (K_ + 1) * sizeof(float), stream, d_leaf_.p, o->d_leaf_.p, d_kl_tabs_.p + n_inner_,
                     d_kl_tabs_.p + n_inner_ + V_, h, K_, C_, d_gp + ns, d_gq + ns);
  check_launch_k("hclt_kld_backward");
}

void HcltCircuit::kld_backward(pcm_circuit* q, float* gp, float* gq, int64_t n) {
  HcltCircuit* o = same_tree(q);
  if (!block_) {
    general()->kld_backward(o->general(), gp, gq, n);
    return;
  }
  if (!gp || !gq) fail(PCM_ERR_ARG, "gradient pointer is null");
  DevBuf<float> d1, d2;
  d1.alloc((size_t)std::max<int64_t>(n, 1));
  d2.alloc((size_t)std::max<int64_t>(n, 1));
  kld_backward_dev(q, d1.p, d2.p, n);
  PCM_HIP(hipMemcpyAsync(gp, d1.p, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, stream));
  PCM_HIP(hipMemcpyAsync(gq, d2.p, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, stream));
  PCM_HIP(hipStreamSynchronize(stream));
}

void HcltCircuit::adam_step(const float* d_grad, float* d_params, float* d_m, float* d_v, float lr, float b1,
                            float b2, float eps, int t) {
  no_forest("Adam");
  no_missing("Adam");
  if (!block_ && !wide_) {
    general()->adam_step(d_grad, d_params, d_m, d_v, lr, b1, b2, eps, t);
    PCM_HIP(hipStreamSynchronize(stream));
    pull_from_general();
    return;
  }
  if (!d_grad || !d_params || !d_m || !d_v) fail(PCM_ERR_ARG, "null optimiser array");
  if (t < 1) fail(PCM_ERR_ARG, "step count must start at 1, got %d", t);
  const int64_t ns = (int64_t)sum_param_src_.size();
  const float c1 = 1.f - std::pow(b1, (float)t), c2 = 1.f - std::pow(b2, (float)t);
  if (wide_)
    hipLaunchKernelGGL(hclt_adam_kernel<128>, dim3((unsigned)ceil_div(ns, 256)), dim3(256), 0, stream, ns, d_grad, d_params, d_m,
                       d_v, lr, b1, b2, eps, c1, c2, d_sum_param_src_.p, d_logtheta_.p);
  else
    PCM_DISPATCH_K(K_, hipLaunchKernelGGL(hclt_adam_kernel<KK>, dim3((unsigned)ceil_div(ns, 256)), dim3(256), 0, stream, ns,
                                          d_grad, d_params, d_m, d_v, lr, b1, b2, eps, c1, c2, d_sum_param_src_.p,
                                          d_logtheta_.p));
  check_launch_k("hclt_adam");
  rebuild_w();
  general_stale_ = true;
  PCM_HIP(hipStreamSynchronize(stream));
}

// ---------------------------------------------------------------------------------------------------------
// The same recursion on a MATRIX of parameter rows (`kld(mbpc, params1[R, n], params2[R, n])` src/queries/kld.jl:164-206,
// `kld_backward` :593-649, reached from src/utils/cuda_preallocation.jl:47-78 with one row per example): every row is a
// pair of circuits of this structure, and nothing couples two rows, so the block-form pipeline above runs with the row
// as a second grid dimension -- the leaf terms straight from the rows (a wave per (input node, row), 16-byte loads: nine
// tenths of the bytes of a query), the per-node operands gathered from the rows through a block-entry -> parameter
// table, one pair of chains per row, and the gradients written in parameter order where they belong.  Against the
// per-layer kernels of the general form (one launch per layer and a lane group per (node, row)) this is six launches.
// ---------------------------------------------------------------------------------------------------------

constexpr float kRowsNormEps = 1e-8f;   // leaf parameters that are probabilities: fixable_categorical_dist.jl:182-186

template <bool kNorm>
__device__ __forceinline__ float rows_leaf_term(float x, float y) {
  return kNorm ? x * (logf(x + kRowsNormEps) - logf(y + kRowsNormEps)) : expf(x) * (x - y);
}

// kl_leaf[row][v * K + j] of input node i = (v, j): a wave takes four input nodes of one row
template <bool kNorm, bool kVec>
__global__ __launch_bounds__(256) void hclt_rows_leaf_kl_kernel(const float* __restrict__ P1, const float* __restrict__ P2,
                                                                size_t n_par, size_t ns, int C, int n_inputs,
                                                                const int32_t* __restrict__ input_order, size_t vk,
                                                                float* __restrict__ kl_leaf) {
  const int lane = threadIdx.x & 63;
  const int i0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4;
  const size_t row = blockIdx.y;
  if (i0 >= n_inputs) return;
  const float* a = P1 + row * n_par + ns + (size_t)i0 * C;
  const float* b = P2 + row * n_par + ns + (size_t)i0 * C;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (kVec) {
    for (int c4 = lane; c4 < C / 4; c4 += 64) {
      float4 x[4], y[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int iu = min(i0 + u, n_inputs - 1) - i0;   // (past the last node: the last node again, not added)
        x[u] = reinterpret_cast<const float4*>(a + (size_t)iu * C)[c4];
        y[u] = reinterpret_cast<const float4*>(b + (size_t)iu * C)[c4];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        acc[u] += (rows_leaf_term<kNorm>(x[u].x, y[u].x) + rows_leaf_term<kNorm>(x[u].y, y[u].y)) +
                  (rows_leaf_term<kNorm>(x[u].z, y[u].z) + rows_leaf_term<kNorm>(x[u].w, y[u].w));
    }
  } else {
    for (int c = lane; c < C; c += 64)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int iu = min(i0 + u, n_inputs - 1) - i0;
        acc[u] += rows_leaf_term<kNorm>(a[(size_t)iu * C + c], b[(size_t)iu * C + c]);
      }
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc[u] += __shfl_xor(acc[u], o);
    if (lane == 0 && i0 + u < n_inputs) kl_leaf[row * vk + input_order[i0 + u]] = acc[u];
  }
}

// hclt_kld_base_kernel for (tree node, row): theta through blk2par (entry of the [n_inner][K][K] blocks -> parameter,
// -1: an edge that is not there, the root's rows past the first)
template <int K>
__global__ __launch_bounds__(256) void hclt_rows_base_kernel(const HcltNode* __restrict__ nodes,
                                                             const int32_t* __restrict__ child_leaf,
                                                             const int32_t* __restrict__ pos, int n_inner,
                                                             const int32_t* __restrict__ blk2par,
                                                             const float* __restrict__ P1, const float* __restrict__ P2,
                                                             size_t n_par, const float* __restrict__ kl_leaf, size_t vk,
                                                             float* __restrict__ ell, float* __restrict__ base,
                                                             float* __restrict__ pu, float* __restrict__ pd, KlRowStrides rs) {
  // (kl_leaf null: the leaf terms are not known yet -- the gradient's downward chain runs before the one pass over the
  // leaf parameters -- and base gets the node's own part sum_j p (x - y) only; hclt_rows_soft_base2_kernel adds
  // sum_j p * ell[j] from the operand afterwards)
  __shared__ float tile[K][K + 1];
  __shared__ float l[K];
  const int n = blockIdx.x, t = threadIdx.x;
  const size_t row = blockIdx.y;
  const HcltNode nd = nodes[n];
  const size_t su = (size_t)pos[n], sd = (size_t)pos[n_inner + n];
  const float* p1 = P1 + row * n_par;
  const float* p2 = P2 + row * n_par;
  ell += row * rs.vec;
  base += row * rs.vec;
  if (t < K) {
    float s = 0.f;
    if (kl_leaf) {
      kl_leaf += row * vk;
      s = kl_leaf[(size_t)nd.var * K + t];
      for (int q = 0; q < nd.lc_cnt; ++q) s += kl_leaf[(size_t)child_leaf[nd.lc_off + q] * K + t];
      ell[su * K + t] = s;
    }
    l[t] = s;
  }
  __syncthreads();
  const int j = t % K;
  for (int k = t / K; k < K; k += 256 / K) {
    const int idx = blk2par[((size_t)n * K + k) * K + j];
    const float x = idx >= 0 ? p1[idx] : -INFINITY, y = idx >= 0 ? p2[idx] : 0.f;
    const float p = expf(x);
    tile[k][j] = p;
    float term = p > 0.f ? p * (x - y + l[j]) : 0.f;
#pragma unroll
    for (int o = K / 2; o > 0; o >>= 1) term += __shfl_xor(term, o, K);
    if (j == 0) base[su * K + k] = term;
  }
  __syncthreads();
  constexpr int JP = K * K / 64;
  float* pur = pu + row * rs.pu + su * K * K;
  float* pdr = pd ? pd + row * rs.pd + sd * K * K : nullptr;
  for (int w = t; w < K * K; w += 256) {
    const int e = w & 3, lane = (w >> 2) & 63, i4 = w >> 8;
    const int rw = (lane / K) * JP + i4 * 4 + e, col = lane % K;
    pur[w] = tile[col][rw];
    if (pdr) pdr[w] = tile[rw][col];
  }
}

__global__ void hclt_rows_take_kernel(const float* __restrict__ klv, size_t nk, size_t at, int rows, float* __restrict__ out) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < rows) out[r] = klv[(size_t)r * nk + at];
}

// hclt_kld_edge_grad_kernel on rows: the parameters are the rows' own entries.  A thread takes one parameter through
// kEdgeGradRows rows, so its place in the blocks is looked up once.
constexpr int kEdgeGradRows = 8;

__global__ void hclt_rows_edge_grad_kernel(int64_t ns, int K, const int64_t* __restrict__ src,
                                           const int32_t* __restrict__ parent_of, const float* __restrict__ P1,
                                           const float* __restrict__ P2, size_t n_par, const float* __restrict__ z,
                                           const float* __restrict__ h, size_t nk, int rows, float* __restrict__ G1,
                                           float* __restrict__ G2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= ns) return;
  const int64_t s = src[i];
  const int j = (int)(s % K), k = (int)((s / K) % K);
  const int n = (int)(s / ((int64_t)K * K));
  const int par = parent_of[n];
  const size_t zat = (size_t)n * K + j, hat = par < 0 ? 0 : (size_t)par * K + k;
  const int r0 = blockIdx.y * kEdgeGradRows;
  float a[kEdgeGradRows], b[kEdgeGradRows], zz[kEdgeGradRows], g[kEdgeGradRows];
#pragma unroll
  for (int q = 0; q < kEdgeGradRows; ++q) {
    const size_t row = (size_t)min(r0 + q, rows - 1);
    a[q] = P1[row * n_par + i];
    b[q] = P2[row * n_par + i];
    zz[q] = z[row * nk + zat];
    g[q] = h[row * nk + hat];
  }
#pragma unroll
  for (int q = 0; q < kEdgeGradRows; ++q) {
    if (r0 + q >= rows) break;
    const size_t row = (size_t)(r0 + q);
    const float gg = par < 0 ? 1.f : g[q], p1 = expf(a[q]);
    G1[row * n_par + i] = gg * (p1 * (zz[q] + a[q] - b[q]) + p1);
    G2[row * n_par + i] = -gg * p1;
  }
}

// The two leaf passes of the gradient in one: the leaf terms of the divergence (hclt_rows_leaf_kl_kernel) and the
// gradients of the leaf parameters (src/queries/kld.jl:528-535, src/nodes/fixable_categorical_dist.jl:216-219) read
// the same two runs of C values per input node, and
// the gradient's weight h comes from the DOWNWARD chain, which needs only the parameters -- so it can run first and
// the leaf parameters, nine tenths of a row, cross the memory bus once.  L lanes (a power of two, at most 64) per
// (input node, row): 64 where C >= 256, fewer for short category lists so that no lane idles.
template <bool kNorm>
__global__ __launch_bounds__(256) void hclt_rows_leaf_kl_grad_kernel(const float* __restrict__ P1, const float* __restrict__ P2,
                                                                     size_t n_par, size_t ns, int C, int K, int n_inputs, int L,
                                                                     const int32_t* __restrict__ input_order,
                                                                     const int32_t* __restrict__ state_node,
                                                                     const float* __restrict__ h, size_t nk, size_t vk,
                                                                     float* __restrict__ kl_leaf, float* __restrict__ G1,
                                                                     float* __restrict__ G2) {
  const int lane = threadIdx.x % L;
  const int i = (blockIdx.x * 256 + threadIdx.x) / L;
  const size_t row = blockIdx.y;
  if (i >= n_inputs) return;
  const int vj = input_order[i];
  const float g = h[row * nk + (size_t)state_node[vj / K] * K + vj % K];
  const size_t at = row * n_par + ns + (size_t)i * C;
  const float4* a4 = reinterpret_cast<const float4*>(P1 + at);
  const float4* b4 = reinterpret_cast<const float4*>(P2 + at);
  float4* g1 = reinterpret_cast<float4*>(G1 + at);
  float4* g2 = reinterpret_cast<float4*>(G2 + at);
  auto d1 = [&](float x, float y) { return kNorm ? g * (logf(x + kRowsNormEps) - logf(y + kRowsNormEps) + 1.f) : g * (x - y + 1.f); };
  auto d2 = [&](float x, float y) { return kNorm ? g * x / (y + kRowsNormEps) : g * expf(x - y); };
  float acc = 0.f;
  for (int c4 = lane; c4 < C / 4; c4 += L) {
    const float4 a = a4[c4], b = b4[c4];
    g1[c4] = make_float4(d1(a.x, b.x), d1(a.y, b.y), d1(a.z, b.z), d1(a.w, b.w));
    g2[c4] = make_float4(d2(a.x, b.x), d2(a.y, b.y), d2(a.z, b.z), d2(a.w, b.w));
    acc += (rows_leaf_term<kNorm>(a.x, b.x) + rows_leaf_term<kNorm>(a.y, b.y)) +
           (rows_leaf_term<kNorm>(a.z, b.z) + rows_leaf_term<kNorm>(a.w, b.w));
  }
  for (int o = L / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);   // (the L lanes of a node leave or stay together)
  if (lane == 0) kl_leaf[row * vk + vj] = acc;
}

template <int K>
__global__ void hclt_rows_soft_base2_kernel(const HcltNode* __restrict__ nodes, const int32_t* __restrict__ child_leaf,
                                            const int32_t* __restrict__ pos, int n_inner, const float* __restrict__ leaf_grad,
                                            size_t vk, const float* __restrict__ pd, float* __restrict__ ell,
                                            float* __restrict__ base, KlRowStrides rs, int add);

// KL of every row (d_klds, may be null with gradients) and, with d_g1 / d_g2, its gradients in the layout of the inputs
void HcltCircuit::kld_rows_block(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm,
                                 float* d_klds, float* d_g1, float* d_g2) {
  const bool with_down = d_g1 != nullptr;
  build_kld_tables();
  const int64_t ns = (int64_t)sum_param_src_.size();
  const int64_t n = size(0);
  if (d_blk2par_.n == 0) {
    std::vector<int32_t> b2p((size_t)n_inner_ * K_ * K_, -1);
    for (int64_t i = 0; i < ns; ++i) b2p[(size_t)sum_param_src_[i]] = (int32_t)i;
    d_blk2par_.upload(b2p, stream);
  }
  if (d_input_order_.n == 0) d_input_order_.upload(input_order_, stream);
  const float* p1 = rows_packed_in(d_p1, sr, sp, rows, n, d_rows_pk1_, stream);
  const float* p2 = rows_packed_in(d_p2, sr, sp, rows, n, d_rows_pk2_, stream);
  const bool direct = sp == 1 && sr == n;
  float* g1 = d_g1;
  float* g2 = d_g2;
  if (with_down && !direct) {
    d_rows_pg1_.ensure((size_t)rows * n);
    d_rows_pg2_.ensure((size_t)rows * n);
    g1 = d_rows_pg1_.p;
    g2 = d_rows_pg2_.p;
  }
  const int W = kl_waves(K_), D = kl_ahead(K_);
  const size_t nk = (size_t)n_inner_ * K_, vk = (size_t)V_ * K_;
  const size_t su = (size_t)(kl_up_steps_ + D) * W, sd = (size_t)(kl_down_steps_ + D) * W, sm = std::max(su, sd);
  KlRowStrides rs;
  rs.pu = su * K_ * K_;
  rs.pd = with_down ? sd * K_ * K_ : 0;
  rs.vec = sm * K_;
  rs.out = nk;
  rs.ring_up = kl_ring_slots_ ? 0 : su * K_;
  rs.ring_down = kl_ring_slots_ ? 0 : sd * K_;
  rs.down_only = 0;
  const size_t per_row = vk + 2 * rs.vec + rs.pu + rs.pd + 3 * nk + rs.ring_up + rs.ring_down;
  // rows at a time: what keeps the scratch arrays within 8 GB
  const int chunk = (int)std::max<size_t>(1, std::min<size_t>((size_t)rows, ((size_t)2 << 30) / per_row));
  d_rows_scratch_.ensure((size_t)chunk * per_row);
  float* kl_leaf = d_rows_scratch_.p;
  float* ell = kl_leaf + (size_t)chunk * vk;
  float* base = ell + (size_t)chunk * rs.vec;
  float* pu = base + (size_t)chunk * rs.vec;
  float* pd = with_down ? pu + (size_t)chunk * rs.pu : nullptr;
  float* klv = pu + (size_t)chunk * (rs.pu + rs.pd);
  float* z = klv + (size_t)chunk * nk;
  float* h = z + (size_t)chunk * nk;
  float* ring_up = kl_ring_slots_ ? nullptr : h + (size_t)chunk * nk;
  float* ring_down = kl_ring_slots_ ? nullptr : ring_up + (size_t)chunk * rs.ring_up;
  // (klv, z and h of a row sit nk apart per row, not behind one another: rs.out strides each of them)
  const int n_inputs = (int)input_order_.size();
  const bool vec = C_ % 4 == 0 && n % 4 == 0 && ns % 4 == 0 && ((reinterpret_cast<uintptr_t>(p1) | reinterpret_cast<uintptr_t>(p2)) & 15) == 0;
  const bool vec_g = vec && (!with_down || ((reinterpret_cast<uintptr_t>(g1) | reinterpret_cast<uintptr_t>(g2)) & 15) == 0);
  if (with_down && !vec_g) fail(PCM_ERR_UNSUPPORTED, "row gradients on the block kernels need 16-byte aligned matrices and a category count divisible by 4");
  const size_t root_at = (size_t)inner_of_var_[root_] * K_;
  for (int r0 = 0; r0 < rows; r0 += chunk) {
    const int rc = std::min(chunk, rows - r0);
    const float* q1 = p1 + (size_t)r0 * n;
    const float* q2 = p2 + (size_t)r0 * n;
    auto chain = [&](int down_only) {   // one workgroup per row, up the tree or down it
      KlRowStrides r2 = rs;
      r2.down_only = down_only;
      PCM_DISPATCH_K(K_, {
        auto launch = [&](auto kernel, size_t lds) {
          hipLaunchKernelGGL(kernel, dim3(1, rc), dim3(kl_waves(KK) * 64), lds, stream,
                             reinterpret_cast<const KlItem*>(d_kl_up_.p), kl_up_steps_,
                             reinterpret_cast<const KlItem*>(d_kl_down_.p), kl_down_steps_, d_kl_ext_.p, pu, base, ell, pd,
                             kl_ring_slots_ - 1, ring_up, ring_down, klv, z, h, r2);
        };
        if (kl_ring_slots_) launch(&hclt_kld_chain_kernel<KK, true>, (size_t)kl_ring_slots_ * KK * sizeof(float));
        else launch(&hclt_kld_chain_kernel<KK, false>, 0);
      });
    };
    auto base_pass = [&](const float* leaf_terms, float* up, float* down) {
      PCM_DISPATCH_K(K_, hipLaunchKernelGGL(hclt_rows_base_kernel<KK>, dim3(n_inner_, rc), dim3(256), 0, stream, d_nodes_.p,
                                            d_child_leaf_.p, d_kl_pos_.p, n_inner_, d_blk2par_.p, q1, q2, (size_t)n, leaf_terms,
                                            vk, ell, base, up, down, rs));
    };
    if (!with_down) {
      const dim3 lgrid(ceil_div(n_inputs, 16), rc);
      auto leaf = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, lgrid, dim3(256), 0, stream, q1, q2, (size_t)n, (size_t)ns, C_, n_inputs, d_input_order_.p, vk, kl_leaf);
      };
      if (norm) { if (vec) leaf(&hclt_rows_leaf_kl_kernel<true, true>); else leaf(&hclt_rows_leaf_kl_kernel<true, false>); }
      else { if (vec) leaf(&hclt_rows_leaf_kl_kernel<false, true>); else leaf(&hclt_rows_leaf_kl_kernel<false, false>); }
      base_pass(kl_leaf, pu, nullptr);
      chain(0);
    } else {
      // the operands, the downward chain (it needs nothing but the parameters), ONE pass over the leaf parameters for the
      // leaf terms and the leaf gradients, then the constants of the upward chain, that chain, the sum parameters
      float* o1 = g1 + (size_t)r0 * n;
      float* o2 = g2 + (size_t)r0 * n;
      base_pass(nullptr, pu, pd);
      chain(1);
      int L = 1;
      while (L < 64 && L * 4 < C_) L *= 2;
      const dim3 ggrid((unsigned)ceil_div((int64_t)n_inputs * L, 256), rc);
      if (norm)
        hipLaunchKernelGGL(hclt_rows_leaf_kl_grad_kernel<true>, ggrid, dim3(256), 0, stream, q1, q2, (size_t)n, (size_t)ns, C_, K_,
                           n_inputs, L, d_input_order_.p, d_kl_tabs_.p + n_inner_, h, nk, vk, kl_leaf, o1, o2);
      else
        hipLaunchKernelGGL(hclt_rows_leaf_kl_grad_kernel<false>, ggrid, dim3(256), 0, stream, q1, q2, (size_t)n, (size_t)ns, C_, K_,
                           n_inputs, L, d_input_order_.p, d_kl_tabs_.p + n_inner_, h, nk, vk, kl_leaf, o1, o2);
      PCM_DISPATCH_K(K_, hipLaunchKernelGGL(hclt_rows_soft_base2_kernel<KK>, dim3(n_inner_, rc), dim3(256), 0, stream, d_nodes_.p,
                                            d_child_leaf_.p, d_kl_pos_.p, n_inner_, kl_leaf, vk, pd, ell, base, rs, 1));
      chain(0);
      hipLaunchKernelGGL(hclt_rows_edge_grad_kernel, dim3((unsigned)ceil_div(ns, 256), ceil_div(rc, kEdgeGradRows)), dim3(256), 0,
                         stream, ns, K_, d_sum_param_src_.p, d_kl_tabs_.p, q1, q2, (size_t)n, z, h, nk, rc, o1, o2);
    }
    if (d_klds)
      hipLaunchKernelGGL(hclt_rows_take_kernel, dim3(ceil_div(rc, 256)), dim3(256), 0, stream, klv, nk, root_at, rc, d_klds + r0);
  }
  if (with_down && !direct) {
    rows_unpack_out(g1, d_g1, sr, sp, rows, n, stream);
    rows_unpack_out(g2, d_g2, sr, sp, rows, n, stream);
  }
  check_launch_k("hclt_kld_rows");
}

// ---- the relaxed sampler on parameter rows (`gumbel_sample(mbpc, params[R, n], ...)`, src/queries/sample.jl:338-383) ----
// A sum node hands its top-down probability to its edges in shares softmax((logp + g) / T) over the node (sample.jl:37-51,
// :105-140), a product passes it on, an input node adds td * its distribution to out[variable] (:262-284).  On the block
// form that is the downward chain above with the softmax weights as operand: per (tree node, row) the K x K weights,
// one chain per row, then per (variable, row) the mixture of the variable's K leaf distributions.

// pd[sd]: operand (row k, column j) = softmax_j((theta[k,j] + g[k,j]) / T); noise in parameter order like the rows (null: none)
template <int K>
__global__ __launch_bounds__(256) void hclt_rows_soft_base_kernel(const int32_t* __restrict__ pos, int n_inner,
                                                                  const int32_t* __restrict__ blk2par,
                                                                  const float* __restrict__ P, size_t n_par,
                                                                  const float* __restrict__ noise, size_t ns, float inv_t,
                                                                  float* __restrict__ pd, float* __restrict__ pu, KlRowStrides rs) {
  __shared__ float tile[K][K + 1];
  const int n = blockIdx.x, t = threadIdx.x;
  const size_t row = blockIdx.y;
  const size_t sd = (size_t)pos[n_inner + n], su = (size_t)pos[n];
  const float* p = P + row * n_par;
  const float* g = noise ? noise + row * ns : nullptr;
  const int j = t % K;
  for (int k = t / K; k < K; k += 256 / K) {
    const int idx = blk2par[((size_t)n * K + k) * K + j];
    float x = -INFINITY;
    if (idx >= 0) x = (p[idx] + (g ? g[idx] : 0.f)) * inv_t;
    float m = x;
#pragma unroll
    for (int o = K / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, K));
    const float e = x > -INFINITY ? expf(x - m) : 0.f;
    float sum = e;
#pragma unroll
    for (int o = K / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o, K);
    tile[k][j] = sum > 0.f ? e / sum : 0.f;
  }
  __syncthreads();
  constexpr int JP = K * K / 64;
  float* pdr = pd + row * rs.pd + sd * K * K;
  float* pur = pu ? pu + row * rs.pu + su * K * K : nullptr;   // (the reverse pass walks up with the same weights)
  for (int w = t; w < K * K; w += 256) {
    const int e = w & 3, lane = (w >> 2) & 63, i4 = w >> 8;
    const int rw = (lane / K) * JP + i4 * 4 + e, col = lane % K;
    pdr[w] = tile[rw][col];
    if (pur) pur[w] = tile[col][rw];
  }
}

// where entry (row rw, column col) of a K x K operand sits in its slot (the layout the chains read, see above)
template <int K>
__device__ __forceinline__ int kl_operand_word(int rw, int col) {
  constexpr int JP = K * K / 64;
  const int part = rw / JP, i = rw % JP;
  return (((i >> 2) * 64) + part * K + col) * 4 + (i & 3);
}

// Reverse pass, input nodes (gumbel_input_sample_up_kernel, sample.jl:531-598): the gradient of a leaf parameter is
// og[v][c] * td(v, j) -- per PROBABILITY of the category, with probability-valued parameters or not, as the source writes
// it (:560-570) -- and the node's own gradient sum_c p(c) * og[v][c] goes to leaf_grad[row][v * K + j].  A wave per
// two input nodes and row, 16-byte accesses.
template <bool kNorm>
__global__ __launch_bounds__(256) void hclt_rows_soft_back_leaf_kernel(const float* __restrict__ P, size_t n_par, size_t ns, int C,
                                                                       int K, int V, int n_inputs,
                                                                       const int32_t* __restrict__ input_order,
                                                                       const int32_t* __restrict__ state_node,
                                                                       const float* __restrict__ h, size_t nk,
                                                                       const float* __restrict__ og, size_t vk,
                                                                       float* __restrict__ leaf_grad, float* __restrict__ G) {
  const int lane = threadIdx.x & 63;
  const int i0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 2;   // two nodes per wave: both nodes' loads leave before either is used
  const size_t row = blockIdx.y;
  if (i0 >= n_inputs) return;
  const bool two = i0 + 1 < n_inputs;
  const int vj0 = input_order[i0], vj1 = input_order[two ? i0 + 1 : i0];
  const int v0 = vj0 / K, v1 = vj1 / K;
  const float t0 = h[row * nk + (size_t)state_node[v0] * K + vj0 % K];
  const float t1 = h[row * nk + (size_t)state_node[v1] * K + vj1 % K];
  const size_t at = row * n_par + ns + (size_t)i0 * C;
  const float4* p0 = reinterpret_cast<const float4*>(P + at);
  const float4* p1 = reinterpret_cast<const float4*>(P + at + (two ? C : 0));
  const float4* o0 = reinterpret_cast<const float4*>(og + (row * V + v0) * C);
  const float4* o1 = reinterpret_cast<const float4*>(og + (row * V + v1) * C);
  float4* g0 = reinterpret_cast<float4*>(G + at);
  float4* g1 = reinterpret_cast<float4*>(G + at + C);
  auto dot = [&](const float4& x, const float4& oc) {
    return kNorm ? (x.x * oc.x + x.y * oc.y) + (x.z * oc.z + x.w * oc.w)
                 : (expf(x.x) * oc.x + expf(x.y) * oc.y) + (expf(x.z) * oc.z + expf(x.w) * oc.w);
  };
  float acc0 = 0.f, acc1 = 0.f;
  for (int c4 = lane; c4 < C / 4; c4 += 64) {
    const float4 x0 = p0[c4], x1 = p1[c4], oc0 = o0[c4], oc1 = o1[c4];
    g0[c4] = make_float4(oc0.x * t0, oc0.y * t0, oc0.z * t0, oc0.w * t0);
    if (two) g1[c4] = make_float4(oc1.x * t1, oc1.y * t1, oc1.z * t1, oc1.w * t1);
    acc0 += dot(x0, oc0);
    acc1 += dot(x1, oc1);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    acc0 += __shfl_xor(acc0, off);
    acc1 += __shfl_xor(acc1, off);
  }
  if (lane == 0) {
    leaf_grad[row * vk + vj0] = acc0;
    if (two) leaf_grad[row * vk + vj1] = acc1;
  }
}

// Reverse pass, what the upward chain starts from, per (tree node, row): ell[su][j] = the gradients of the leaves that
// are factors of product j, base[su][k] = sum_j w[k,j] * ell[j] with the weights read back from the downward operand
// (add: on top of what base holds -- the KL gradient on rows, whose base starts as the node's own part)
template <int K>
__global__ __launch_bounds__(256) void hclt_rows_soft_base2_kernel(const HcltNode* __restrict__ nodes,
                                                                   const int32_t* __restrict__ child_leaf,
                                                                   const int32_t* __restrict__ pos, int n_inner,
                                                                   const float* __restrict__ leaf_grad, size_t vk,
                                                                   const float* __restrict__ pd, float* __restrict__ ell,
                                                                   float* __restrict__ base, KlRowStrides rs, int add) {
  __shared__ float l[K];
  const int n = blockIdx.x, t = threadIdx.x;
  const size_t row = blockIdx.y;
  const HcltNode nd = nodes[n];
  const size_t su = (size_t)pos[n], sd = (size_t)pos[n_inner + n];
  leaf_grad += row * vk;
  ell += row * rs.vec;
  base += row * rs.vec;
  if (t < K) {
    float s = leaf_grad[(size_t)nd.var * K + t];
    for (int q = 0; q < nd.lc_cnt; ++q) s += leaf_grad[(size_t)child_leaf[nd.lc_off + q] * K + t];
    l[t] = s;
    ell[su * K + t] = s;
  }
  __syncthreads();
  const float* w = pd + row * rs.pd + sd * K * K;
  const int j = t % K;
  for (int k = t / K; k < K; k += 256 / K) {
    float term = w[kl_operand_word<K>(k, j)] * l[j];
#pragma unroll
    for (int o = K / 2; o > 0; o >>= 1) term += __shfl_xor(term, o, K);
    if (j == 0) base[su * K + k] = add ? base[su * K + k] + term : term;
  }
}

// Reverse pass, sum parameters (gumbel_params_up_layer_kernel, sample.jl:391-480): edge (k, j) of tree node n gets
// td(S_n[k]) * (Z_n[j] - grad(S_n[k])) * w[k,j] / T, without the w when the gradient is wanted per probability (:466-469).
template <int K>
__global__ void hclt_rows_soft_edge_grad_kernel(int64_t ns, const int64_t* __restrict__ src, const int32_t* __restrict__ parent_of,
                                                const int32_t* __restrict__ pos, int n_inner, const float* __restrict__ pd,
                                                const float* __restrict__ z, const float* __restrict__ klv,
                                                const float* __restrict__ h, size_t nk, KlRowStrides rs, float inv_t, int wrt_log,
                                                int rows, size_t n_par, float* __restrict__ G) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= ns) return;
  const int64_t s = src[i];
  const int j = (int)(s % K), k = (int)((s / K) % K);
  const int n = (int)(s / ((int64_t)K * K));
  const int par = parent_of[n];
  const size_t wat = (size_t)pos[n_inner + n] * K * K + kl_operand_word<K>(k, j);
  const size_t zat = (size_t)n * K + j, kat = (size_t)n * K + k, hat = par < 0 ? 0 : (size_t)par * K + k;
  const int r0 = blockIdx.y * kEdgeGradRows;
#pragma unroll
  for (int q = 0; q < kEdgeGradRows; ++q) {
    if (r0 + q >= rows) break;
    const size_t row = (size_t)(r0 + q);
    const float t = par < 0 ? 1.f : h[row * nk + hat];
    const float w = wrt_log ? pd[row * rs.pd + wat] : 1.f;
    G[row * n_par + i] = t * (z[row * nk + zat] - klv[row * nk + kat]) * w * inv_t;
  }
}

// out[row][v][c] = sum_j h[state node of v][j] * distribution of input node (v, j) at c
template <bool kNorm>
__global__ __launch_bounds__(256) void hclt_rows_soft_leaf_kernel(const float* __restrict__ P, size_t n_par, size_t ns, int C, int K,
                                                                  int V, const int32_t* __restrict__ state_node,
                                                                  const int32_t* __restrict__ in_pos, const float* __restrict__ h,
                                                                  size_t nk, float* __restrict__ out) {
  __shared__ float td[64];
  __shared__ int at[64];
  const int v = blockIdx.x;
  const size_t row = blockIdx.y;
  if ((int)threadIdx.x < K) {
    td[threadIdx.x] = h[row * nk + (size_t)state_node[v] * K + threadIdx.x];
    at[threadIdx.x] = in_pos[(size_t)v * K + threadIdx.x];
  }
  __syncthreads();
  const float* p = P + row * n_par + ns;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f;
    for (int j0 = 0; j0 < K; j0 += 8) {   // eight rows requested before the first is used
      float x[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) x[q] = p[(size_t)at[j0 + q] * C + c];
#pragma unroll
      for (int q = 0; q < 8; ++q) acc += td[j0 + q] * (kNorm ? x[q] : expf(x[q]));
    }
    out[(row * V + v) * C + c] = acc;
  }
}

void HcltCircuit::gumbel_sample_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                     float temperature, bool norm_params, float* d_out) {
  if (!block_queries() || H_ > 0 || missing_)
    return general_structure()->gumbel_sample_rows(d_params, sr, sp, rows, d_noise, temperature, norm_params, d_out);
  if (!d_params) fail(PCM_ERR_ARG, "parameter matrix is null");
  if (rows < 1) fail(PCM_ERR_ARG, "need at least one parameter row, got %d", rows);
  if (rows > 65535) fail(PCM_ERR_UNSUPPORTED, "at most 65535 parameter rows per call, got %d", rows);
  if (sr == 0 || sp == 0) fail(PCM_ERR_ARG, "parameter matrix strides must not be zero");
  if (!d_out) fail(PCM_ERR_ARG, "output pointer is null");
  if (!(temperature > 0.f)) fail(PCM_ERR_ARG, "temperature must be positive");
  build_kld_tables();
  const int64_t ns = (int64_t)sum_param_src_.size();
  const int64_t n = size(0);
  if (d_blk2par_.n == 0) {
    std::vector<int32_t> b2p((size_t)n_inner_ * K_ * K_, -1);
    for (int64_t i = 0; i < ns; ++i) b2p[(size_t)sum_param_src_[i]] = (int32_t)i;
    d_blk2par_.upload(b2p, stream);
  }
  const float* p = rows_packed_in(d_params, sr, sp, rows, n, d_rows_pk1_, stream);
  const int W = kl_waves(K_), D = kl_ahead(K_);
  const size_t nk = (size_t)n_inner_ * K_;
  const size_t su = (size_t)(kl_up_steps_ + D) * W, sd = (size_t)(kl_down_steps_ + D) * W, sm = std::max(su, sd);
  KlRowStrides rs;
  rs.pu = 0;               // (a chain that walks down reads no upward operand; the constants it requests are not used)
  rs.pd = sd * K_ * K_;
  rs.vec = sm * K_;
  rs.out = nk;
  rs.ring_up = 0;
  rs.ring_down = kl_ring_slots_ ? 0 : sd * K_;
  rs.down_only = 1;
  const size_t per_row = rs.pd + rs.vec + nk + rs.ring_down;
  const int chunk = (int)std::max<size_t>(1, std::min<size_t>((size_t)rows, ((size_t)2 << 30) / per_row));
  d_rows_scratch_.ensure((size_t)chunk * per_row + su * K_ * K_);
  float* pd = d_rows_scratch_.p;
  float* vec = pd + (size_t)chunk * rs.pd;
  float* h = vec + (size_t)chunk * rs.vec;
  float* ring_down = kl_ring_slots_ ? nullptr : h + (size_t)chunk * nk;
  float* pu = d_rows_scratch_.p + (size_t)chunk * per_row;   // never used, but named by the kernel's requests
  const float inv_t = 1.f / temperature;
  for (int r0 = 0; r0 < rows; r0 += chunk) {
    const int rc = std::min(chunk, rows - r0);
    const float* q = p + (size_t)r0 * n;
    const float* g = d_noise ? d_noise + (size_t)r0 * ns : nullptr;
    PCM_DISPATCH_K(K_, {
      hipLaunchKernelGGL(hclt_rows_soft_base_kernel<KK>, dim3(n_inner_, rc), dim3(256), 0, stream, d_kl_pos_.p, n_inner_,
                         d_blk2par_.p, q, (size_t)n, g, (size_t)ns, inv_t, pd, (float*)nullptr, rs);
      auto chain = [&](auto kernel, size_t lds) {
        hipLaunchKernelGGL(kernel, dim3(1, rc), dim3(kl_waves(KK) * 64), lds, stream,
                           reinterpret_cast<const KlItem*>(d_kl_up_.p), kl_up_steps_,
                           reinterpret_cast<const KlItem*>(d_kl_down_.p), kl_down_steps_, d_kl_ext_.p, pu, vec, vec, pd,
                           kl_ring_slots_ - 1, (float*)nullptr, ring_down, h, h, h, rs);
      };
      if (kl_ring_slots_) chain(&hclt_kld_chain_kernel<KK, true>, (size_t)kl_ring_slots_ * KK * sizeof(float));
      else chain(&hclt_kld_chain_kernel<KK, false>, 0);
    });
    float* out = d_out + (size_t)r0 * Vu_ * C_;
    const dim3 lgrid(Vu_, rc);
    if (norm_params)
      hipLaunchKernelGGL(hclt_rows_soft_leaf_kernel<true>, lgrid, dim3(256), 0, stream, q, (size_t)n, (size_t)ns, C_, K_, Vu_,
                         d_kl_tabs_.p + n_inner_, d_kl_tabs_.p + n_inner_ + V_, h, nk, out);
    else
      hipLaunchKernelGGL(hclt_rows_soft_leaf_kernel<false>, lgrid, dim3(256), 0, stream, q, (size_t)n, (size_t)ns, C_, K_, Vu_,
                         d_kl_tabs_.p + n_inner_, d_kl_tabs_.p + n_inner_ + V_, h, nk, out);
  }
  check_launch_k("hclt_gumbel_sample_rows");
}

void HcltCircuit::gumbel_sample_backward_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                              float temperature, bool norm_params, bool grad_wrt_logparams,
                                              const float* d_out_grad, float* d_grads) {
  const int64_t ns = (int64_t)sum_param_src_.size();
  const int64_t n = size(0);
  const bool direct = sp == 1 && sr == n;
  // 16-byte rows on every side: the leaf kernel moves four categories at a time
  const bool aligned = C_ % 4 == 0 && n % 4 == 0 && ns % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out_grad) & 15) == 0 &&
                       (!direct || ((reinterpret_cast<uintptr_t>(d_params) | reinterpret_cast<uintptr_t>(d_grads)) & 15) == 0);
  if (!block_queries() || H_ > 0 || missing_ || !aligned)
    return general_structure()->gumbel_sample_backward_rows(d_params, sr, sp, rows, d_noise, temperature, norm_params,
                                                            grad_wrt_logparams, d_out_grad, d_grads);
  if (!d_params) fail(PCM_ERR_ARG, "parameter matrix is null");
  if (rows < 1) fail(PCM_ERR_ARG, "need at least one parameter row, got %d", rows);
  if (rows > 65535) fail(PCM_ERR_UNSUPPORTED, "at most 65535 parameter rows per call, got %d", rows);
  if (sr == 0 || sp == 0) fail(PCM_ERR_ARG, "parameter matrix strides must not be zero");
  if (!d_out_grad || !d_grads) fail(PCM_ERR_ARG, "gradient pointer is null");
  if (!(temperature > 0.f)) fail(PCM_ERR_ARG, "temperature must be positive");
  build_kld_tables();
  if (d_blk2par_.n == 0) {
    std::vector<int32_t> b2p((size_t)n_inner_ * K_ * K_, -1);
    for (int64_t i = 0; i < ns; ++i) b2p[(size_t)sum_param_src_[i]] = (int32_t)i;
    d_blk2par_.upload(b2p, stream);
  }
  if (d_input_order_.n == 0) d_input_order_.upload(input_order_, stream);
  const float* p = rows_packed_in(d_params, sr, sp, rows, n, d_rows_pk1_, stream);
  float* gout = d_grads;
  if (!direct) {
    d_rows_pg1_.ensure((size_t)rows * n);
    gout = d_rows_pg1_.p;
  }
  const int W = kl_waves(K_), D = kl_ahead(K_);
  const size_t nk = (size_t)n_inner_ * K_, vk = (size_t)V_ * K_;
  const size_t su = (size_t)(kl_up_steps_ + D) * W, sd = (size_t)(kl_down_steps_ + D) * W, sm = std::max(su, sd);
  KlRowStrides rs;
  rs.pu = su * K_ * K_;
  rs.pd = sd * K_ * K_;
  rs.vec = sm * K_;
  rs.out = nk;
  rs.ring_up = kl_ring_slots_ ? 0 : su * K_;
  rs.ring_down = kl_ring_slots_ ? 0 : sd * K_;
  rs.down_only = 0;
  const size_t per_row = rs.pu + rs.pd + 2 * rs.vec + 3 * nk + vk + rs.ring_up + rs.ring_down;
  const int chunk = (int)std::max<size_t>(1, std::min<size_t>((size_t)rows, ((size_t)2 << 30) / per_row));
  d_rows_scratch_.ensure((size_t)chunk * per_row);
  float* pd = d_rows_scratch_.p;
  float* pu = pd + (size_t)chunk * rs.pd;
  float* ell = pu + (size_t)chunk * rs.pu;
  float* base = ell + (size_t)chunk * rs.vec;
  float* h = base + (size_t)chunk * rs.vec;
  float* klv = h + (size_t)chunk * nk;
  float* z = klv + (size_t)chunk * nk;
  float* leaf_grad = z + (size_t)chunk * nk;
  float* ring_up = kl_ring_slots_ ? nullptr : leaf_grad + (size_t)chunk * vk;
  float* ring_down = kl_ring_slots_ ? nullptr : ring_up + (size_t)chunk * rs.ring_up;
  const float inv_t = 1.f / temperature;
  const int n_inputs = (int)input_order_.size();
  for (int r0 = 0; r0 < rows; r0 += chunk) {
    const int rc = std::min(chunk, rows - r0);
    const float* q = p + (size_t)r0 * n;
    const float* g = d_noise ? d_noise + (size_t)r0 * ns : nullptr;
    const float* og = d_out_grad + (size_t)r0 * Vu_ * C_;
    float* out = gout + (size_t)r0 * n;
    PCM_DISPATCH_K(K_, {
      auto chain = [&](int down_only) {
        KlRowStrides r2 = rs;
        r2.down_only = down_only;
        auto launch = [&](auto kernel, size_t lds) {
          hipLaunchKernelGGL(kernel, dim3(1, rc), dim3(kl_waves(KK) * 64), lds, stream,
                             reinterpret_cast<const KlItem*>(d_kl_up_.p), kl_up_steps_,
                             reinterpret_cast<const KlItem*>(d_kl_down_.p), kl_down_steps_, d_kl_ext_.p, pu, base, ell, pd,
                             kl_ring_slots_ - 1, ring_up, ring_down, klv, z, h, r2);
        };
        if (kl_ring_slots_) launch(&hclt_kld_chain_kernel<KK, true>, (size_t)kl_ring_slots_ * KK * sizeof(float));
        else launch(&hclt_kld_chain_kernel<KK, false>, 0);
      };
      hipLaunchKernelGGL(hclt_rows_soft_base_kernel<KK>, dim3(n_inner_, rc), dim3(256), 0, stream, d_kl_pos_.p, n_inner_,
                         d_blk2par_.p, q, (size_t)n, g, (size_t)ns, inv_t, pd, pu, rs);
      chain(1);   // the top-down probabilities
      const dim3 lgrid(ceil_div(n_inputs, 8), rc);
      if (norm_params)
        hipLaunchKernelGGL(hclt_rows_soft_back_leaf_kernel<true>, lgrid, dim3(256), 0, stream, q, (size_t)n, (size_t)ns, C_, K_, Vu_,
                           n_inputs, d_input_order_.p, d_kl_tabs_.p + n_inner_, h, nk, og, vk, leaf_grad, out);
      else
        hipLaunchKernelGGL(hclt_rows_soft_back_leaf_kernel<false>, lgrid, dim3(256), 0, stream, q, (size_t)n, (size_t)ns, C_, K_, Vu_,
                           n_inputs, d_input_order_.p, d_kl_tabs_.p + n_inner_, h, nk, og, vk, leaf_grad, out);
      hipLaunchKernelGGL(hclt_rows_soft_base2_kernel<KK>, dim3(n_inner_, rc), dim3(256), 0, stream, d_nodes_.p, d_child_leaf_.p,
                         d_kl_pos_.p, n_inner_, leaf_grad, vk, pd, ell, base, rs, 0);
      chain(0);   // the gradients of the sum nodes, bottom-up
      hipLaunchKernelGGL(hclt_rows_soft_edge_grad_kernel<KK>, dim3((unsigned)ceil_div(ns, 256), ceil_div(rc, kEdgeGradRows)),
                         dim3(256), 0, stream, ns, d_sum_param_src_.p, d_kl_tabs_.p, d_kl_pos_.p, n_inner_, pd, z, klv, h, nk, rs,
                         inv_t, grad_wrt_logparams ? 1 : 0, rc, (size_t)n, out);
    });
  }
  if (!direct) rows_unpack_out(gout, d_grads, sr, sp, rows, n, stream);
  check_launch_k("hclt_gumbel_sample_backward_rows");
}

static void check_rows_block_args(const void* p1, const void* p2, int64_t sr, int64_t sp, int rows) {
  if (!p1 || !p2) fail(PCM_ERR_ARG, "parameter matrix is null");
  if (rows < 1) fail(PCM_ERR_ARG, "need at least one parameter row, got %d", rows);
  if (rows > 65535) fail(PCM_ERR_UNSUPPORTED, "at most 65535 parameter rows per call, got %d", rows);
  if (sr == 0 || sp == 0) fail(PCM_ERR_ARG, "parameter matrix strides must not be zero");
}

void HcltCircuit::kld_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                           float* d_out) {
  if (!block_queries() || H_ > 0 || missing_) return general_structure()->kld_rows(d_p1, d_p2, sr, sp, rows, norm_params, d_out);
  check_rows_block_args(d_p1, d_p2, sr, sp, rows);
  if (!d_out) fail(PCM_ERR_ARG, "output pointer is null");
  kld_rows_block(d_p1, d_p2, sr, sp, rows, norm_params, d_out, nullptr, nullptr);
}

void HcltCircuit::kld_backward_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                                    float* d_g1, float* d_g2, float* d_klds) {
  const bool aligned = C_ % 4 == 0 && size(0) % 4 == 0 && (int64_t)sum_param_src_.size() % 4 == 0 &&
                       ((reinterpret_cast<uintptr_t>(d_p1) | reinterpret_cast<uintptr_t>(d_p2) | reinterpret_cast<uintptr_t>(d_g1) |
                         reinterpret_cast<uintptr_t>(d_g2)) & 15) == 0;
  if (!block_queries() || H_ > 0 || missing_ || !aligned)
    return general_structure()->kld_backward_rows(d_p1, d_p2, sr, sp, rows, norm_params, d_g1, d_g2, d_klds);
  check_rows_block_args(d_p1, d_p2, sr, sp, rows);
  if (!d_g1 || !d_g2) fail(PCM_ERR_ARG, "parameter or gradient matrix is null");
  kld_rows_block(d_p1, d_p2, sr, sp, rows, norm_params, d_klds, d_g1, d_g2);
}

}  // namespace pcm
