// Multi-head HCLTs on the block engine: H head sum nodes over the K products of the root
// tree node (reference: src-jl/multi_head_pc/bit_circuit.jl:4-56 builds such circuits from
// `pcs` sharing one body; likelihood.jl:3-18, flow.jl:141-176).
//
// The body runs through the ordinary walk kernels with the root's parameter block set to the
// identity, which makes the root tile O_root[b,k] the root's Z[b,k] (less the row maxima of the tree's
// nodes, which the walk keeps apart: `base` below is their sum) and turns the root step of
// the backward walk into G_root = E .* R_root for whatever R_root it is handed.  Two small
// kernels per pass do the heads, one workgroup per 16-example slice:
//   forward   ll[h][b] = base + m + log sum_j Wh[h,j] E[b,j],  E = exp(Z - m)   (+ the mask-weighted mixture)
//   backward  R[b,h] = mask[h][b] / S[b,h],  T[b,j] = sum_h Wh[h,j] R[b,h]  -> stored as R_root;
//             head_aggr[h,j] += Wh[h,j] * sum_b R[b,h] E[b,j]
// The statistics kernel then finds R_root = T like any other node's ratio tile and histograms
// the root variable from G_root = E .* T without knowing about heads.  Its fixed-point
// histograms need a bound on the flow of one example: the backward kernel leaves
// ceil(log2(max_b sum_h mask[h][b])) in a device word.
//
// Head blocks are [Hp][K] (Hp = H rounded up to 16, padding rows zero) in the two MFMA
// A-operand layouts: hwf: rows = heads, contraction over states; hwb: rows = states,
// contraction over heads.
//
// A forest (several trees over one batch, H heads each) runs the same kernels with the tree in
// blockIdx.y: every per-tree array is [tree][...], the root tiles are found through `root_node`
// (each tree's root node, whose tiles start `tile_floats` floats per node into the value / ratio arrays).
#pragma once

#include "hclt_kernels.hip.hpp"

namespace pcm {

constexpr int kHeadWaves = 4;

__device__ __forceinline__ size_t head_wf_at(int h, int j, int K) {
  return ((((size_t)(h / 16) * (K / 16) + j / 16) * 64) + ((j % 16) / 4) * 16 + h % 16) * 4 + j % 4;
}
__device__ __forceinline__ size_t head_wb_at(int h, int j, int Hp) {
  return ((((size_t)(j / 16) * (Hp / 16) + h / 16) * 64) + ((h % 16) / 4) * 16 + j % 16) * 4 + h % 4;
}

// operand layouts from the head log-parameters [H][K]
__global__ void hclt_heads_rebuild_kernel(const float* __restrict__ head_logp, int H, int Hp, int K, float* __restrict__ hwf,
                                          float* __restrict__ hwb) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= Hp * K) return;
  head_logp += (size_t)blockIdx.y * H * K;
  hwf += (size_t)blockIdx.y * Hp * K;
  hwb += (size_t)blockIdx.y * Hp * K;
  const int h = i / K, j = i % K;
  const float w = h < H ? __expf(head_logp[(size_t)h * K + j]) : 0.f;
  hwf[head_wf_at(h, j, K)] = w;
  hwb[head_wb_at(h, j, Hp)] = w;
}

// E tile and row maxima of the root's Z (= its value tile under the identity block)
template <int K>
__device__ __forceinline__ float heads_load_e(const float* __restrict__ O_root, int slice, int lane, Tile<K>& e) {
  const v4f* src = reinterpret_cast<const v4f*>(O_root + (size_t)slice * kSlice * K);
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) e.v[kt] = src[kt * 64 + lane];
  const float m = tile_rowmax<K>(e);
  tile_exp_sub<K>(e, m);
  return m;
}

// S[b, heads of tile ht] = sum_j Wh[h,j] E[b,j]
template <int K>
__device__ __forceinline__ v4f heads_contract_f(const float* __restrict__ hwf, int ht, int lane, const Tile<K>& e) {
  const v4f* w = reinterpret_cast<const v4f*>(hwf) + (size_t)ht * (K / 16) * 64 + lane;
  v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int jt = 0; jt < K / 16; ++jt) {
    const v4f a = w[jt * 64];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], e.v[jt][i], acc, 0, 0, 0);
  }
  return acc;
}

// Per-head log-likelihoods [H][B] and/or the mask-weighted mixture
//   logsumexp_h(ll_h + log mask_h) - log sum_h mask_h   (src-jl/multi_head_pc/likelihood.jl:3-12).
template <int K>
__global__ __launch_bounds__(kHeadWaves * 64) void hclt_heads_forward_kernel(const float* __restrict__ O,
                                                                             const float* __restrict__ M, int Bp,
                                                                             const int32_t* __restrict__ root_node,
                                                                             int64_t tile_floats,
                                                                             const float* __restrict__ hwf, int H, int Hp,
                                                                             int B, const float* __restrict__ mask,
                                                                             float* __restrict__ ll_heads,
                                                                             float* __restrict__ ll_mix,
                                                                             float* __restrict__ head_aggr, float rate,
                                                                             int* __restrict__ flow_shift) {
  __shared__ float pm[kHeadWaves * 4][16], ps[kHeadWaves * 4][16], pt[kHeadWaves * 4][16];
  __shared__ double pb[kHeadWaves * 4][16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, slice = blockIdx.x, tree = blockIdx.y;
  const float* __restrict__ O_root = O + (size_t)root_node[tree] * tile_floats;
  hwf += (size_t)tree * Hp * K;
  if (mask) mask += (size_t)tree * H * B;
  if (ll_heads) ll_heads += (size_t)tree * H * B;
  if (ll_mix) ll_mix += (size_t)tree * B;
  if (head_aggr) head_aggr += (size_t)tree * H * K;
  if (head_aggr) {   // ahead of a flow pass: previous head statistics times the flow memory rate, flow bound cleared
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < H * K; i += gridDim.x * blockDim.x)
      head_aggr[i] = rate != 0.f ? head_aggr[i] * rate : 0.f;
    if (blockIdx.x == 0 && threadIdx.x == 0) *flow_shift = 0;
  }
  const int b = lane & 15, g = lane >> 4, col = slice * kSlice + b;
  // base: the row maxima of the tree's nodes (post-order goes tree after tree: the nodes after the root before
  // up to this tree's root), every sixteenth node per group of lanes, the groups' sums added in order
  double base;
  {
    const int n_lo = tree > 0 ? root_node[tree - 1] + 1 : 0, n_hi = root_node[tree];
    double acc = 0.0;
    for (int n = n_lo + wave * 4 + g; n <= n_hi; n += kHeadWaves * 4) acc += (double)M[(size_t)n * Bp + col];
    pb[wave * 4 + g][b] = acc;
    __syncthreads();
    base = 0.0;
#pragma unroll
    for (int q = 0; q < kHeadWaves * 4; ++q) base += pb[q][b];
  }
  Tile<K> e;
  const float m = heads_load_e<K>(O_root, slice, lane, e);
  float mx = -INFINITY, sm = 0.f, tot = 0.f;   // running mixture over this lane's heads
  for (int ht = wave; ht < Hp / 16; ht += kHeadWaves) {
    const v4f s = heads_contract_f<K>(hwf, ht, lane, e);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = ht * 16 + 4 * g + i;
      if (h >= H || col >= B) continue;
      const float val = (float)(base + (double)(m + __logf(s[i])));
      if (ll_heads) ll_heads[(size_t)h * B + col] = val;
      if (mask) {
        const float mk = mask[(size_t)h * B + col];
        tot += mk;
        const float t = val + __logf(mk);
        if (t > mx) { sm = sm * __expf(mx - t) + 1.f; mx = t; }
        else if (t != -INFINITY) sm += __expf(t - mx);
      }
    }
  }
  if (!ll_mix) return;
  pm[wave * 4 + g][b] = mx; ps[wave * 4 + g][b] = sm; pt[wave * 4 + g][b] = tot;
  __syncthreads();
  if (threadIdx.x < 16 && col < B) {
    float M = -INFINITY, T = 0.f;
    for (int q = 0; q < kHeadWaves * 4; ++q) { M = fmaxf(M, pm[q][b]); T += pt[q][b]; }
    float S = 0.f;
    for (int q = 0; q < kHeadWaves * 4; ++q)
      if (pm[q][b] != -INFINITY) S += ps[q][b] * __expf(pm[q][b] - M);
    ll_mix[col] = M + __logf(S) - __logf(T);
  }
}

// Head flows (src-jl/multi_head_pc/flow.jl:141-176: head h of example b starts with flow mask[h][b]).
template <int K>
__global__ __launch_bounds__(kHeadWaves * 64) void hclt_heads_backward_kernel(
    const float* __restrict__ O, float* __restrict__ R, const int32_t* __restrict__ root_node, int64_t tile_floats,
    const float* __restrict__ hwf, const float* __restrict__ hwb, int H, int Hp, int B, const float* __restrict__ mask,
    float* __restrict__ head_part, int* __restrict__ flow_shift) {
  extern __shared__ float lds[];   // R [16][Hp] | E [16][K] | partial T tiles [waves][16*K] | mask totals [waves][16]
  float* Rl = lds;
  float* El = Rl + 16 * Hp;
  float* Tl = El + 16 * K;
  float* Fl = Tl + kHeadWaves * 16 * K;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, slice = blockIdx.x, tree = blockIdx.y;
  const float* __restrict__ O_root = O + (size_t)root_node[tree] * tile_floats;
  float* __restrict__ R_root = R + (size_t)root_node[tree] * tile_floats;
  hwf += (size_t)tree * Hp * K;
  hwb += (size_t)tree * Hp * K;
  mask += (size_t)tree * H * B;
  const int b = lane & 15, g = lane >> 4, col = slice * kSlice + b;
  Tile<K> e;
  heads_load_e<K>(O_root, slice, lane, e);
  if (wave == 0)
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) El[b * K + kt * 16 + 4 * g + i] = e.v[kt][i];
  Tile<K> t;
  tile_zero<K>(t);
  float ftot = 0.f;   // this lane's share of its example's total mask
  for (int ht = wave; ht < Hp / 16; ht += kHeadWaves) {
    const v4f s = heads_contract_f<K>(hwf, ht, lane, e);
    v4f r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = ht * 16 + 4 * g + i;
      const float f = (h < H && col < B) ? mask[(size_t)h * B + col] : 0.f;
      ftot += fmaxf(f, 0.f);
      r[i] = (f > 0.f && s[i] > 0.f) ? f / s[i] : 0.f;
      Rl[b * Hp + h] = r[i];
    }
    // T[b, j] += sum over the heads of this tile of Wh[h,j] R[b,h]
    const v4f* w = reinterpret_cast<const v4f*>(hwb) + (size_t)ht * 64 + lane;
#pragma unroll
    for (int jt = 0; jt < K / 16; ++jt) {
      const v4f a = w[(size_t)jt * (Hp / 16) * 64];
#pragma unroll
      for (int i = 0; i < 4; ++i) t.v[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], r[i], t.v[jt], 0, 0, 0);
    }
  }
  v4f* tl = reinterpret_cast<v4f*>(Tl) + (size_t)wave * (K / 16) * 64;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) tl[kt * 64 + lane] = t.v[kt];
  ftot += __shfl_xor(ftot, 16);
  ftot += __shfl_xor(ftot, 32);
  if (lane < 16) Fl[wave * 16 + lane] = ftot;
  __syncthreads();
  if (wave == 0) {
    v4f* dst = reinterpret_cast<v4f*>(R_root + (size_t)slice * kSlice * K);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt) {
      v4f sum = reinterpret_cast<const v4f*>(Tl)[kt * 64 + lane];
#pragma unroll
      for (int w2 = 1; w2 < kHeadWaves; ++w2) sum += reinterpret_cast<const v4f*>(Tl)[((size_t)w2 * (K / 16) + kt) * 64 + lane];
      dst[kt * 64 + lane] = sum;
    }
  }
  // bound on the flow of one example, as a power of two: total mask <= 2^shift
  if (threadIdx.x < 16 && col < B) {
    float tot = 0.f;
    for (int w2 = 0; w2 < kHeadWaves; ++w2) tot += Fl[w2 * 16 + b];
    int ex = 0;
    frexpf(tot, &ex);
    if (ex > 0) atomicMax(flow_shift, ex);
  }
  // head statistics of this slice, without the head weight: row `slice` of head_part [slices][H * K], which
  // sum_parts_kernel adds up in slice order and weights
  float* part = head_part + ((size_t)tree * gridDim.x + slice) * H * K;
  for (int o = threadIdx.x; o < H * K; o += blockDim.x) {
    const int h = o / K, j = o % K;
    float a = 0.f;
#pragma unroll
    for (int bb = 0; bb < 16; ++bb) a += Rl[bb * Hp + h] * El[bb * K + j];
    part[o] = a;
  }
}

// add_pseudocount / aggr_node_flows / update_params for the head sum nodes (one wave per head; blockIdx.y: tree);
// also refreshes the two operand layouts (their padding rows stay zero)
__global__ __launch_bounds__(256) void hclt_heads_update_kernel(float* __restrict__ head_logp, float* __restrict__ head_aggr,
                                                                int H, int Hp, int K, float pseudocount, float inertia,
                                                                float* __restrict__ hwf, float* __restrict__ hwb,
                                                                const int32_t* __restrict__ void_pass) {
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (h >= H) return;
  if (void_pass && *void_pass) return;
  head_logp += (size_t)blockIdx.y * H * K;
  head_aggr += (size_t)blockIdx.y * H * K;
  hwf += (size_t)blockIdx.y * Hp * K;
  hwb += (size_t)blockIdx.y * Hp * K;
  float* a = head_aggr + (size_t)h * K;
  float* lt = head_logp + (size_t)h * K;
  const float share = pseudocount / (float)K;
  float tot = 0.f;
  for (int j = lane; j < K; j += 64) { a[j] += share; tot += a[j]; }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) tot += __shfl_xor(tot, o);
  for (int j = lane; j < K; j += 64) {
    const float w = inertia * expf(lt[j]) + (1.f - inertia) * a[j] / tot;
    lt[j] = logf(w);
    hwf[head_wf_at(h, j, K)] = w;
    hwb[head_wb_at(h, j, Hp)] = w;
  }
}

}  // namespace pcm
