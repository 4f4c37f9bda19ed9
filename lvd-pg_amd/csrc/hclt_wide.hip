// Block kernels for wide hidden sizes (K = 128): a K x K parameter block no longer fits a
// wave's registers, so a 16-example tile is shared by the four waves of a workgroup, each
// producing a quarter of the output states and streaming its quarter of the block (64 KB per
// node at K = 128, shared by all workgroups through L2) as MFMA A-operands.  Trees with wide
// blocks are small (tens of nodes), so a workgroup simply walks the nodes in post-order
// (forward) or reverse post-order (backward) with a barrier between nodes; tiles travel
// through memory.
//
// Tile layout (same as the walk kernels'): lane = 16*g + b owns example b and states
// kt*16 + 4*g + i (kt < K/16, i < 4); a tile is K/16 runs of 64 float4.  This is both the
// B-operand and the accumulator layout of v_mfma_f32_16x16x4_f32 with the parameter block
// (Wf / Wb, pre-swizzled) as A-operand.
//
// Algebra per tree node (reference: src/queries/likelihood.jl:4-68, src/queries/flow.jl:8-106,
// :165-195 on the K^2 sum edges of src/structures/hclts.jl:133):
//   Z = leaf rows + children's tiles, m = max_j Z, E = exp(Z - m)
//   O[k] = log(sum_j W[k,j] E[j])                                  forward: the tiles hold log S, numbers of order one;
//                                                                  a node's full value is O[k] plus the maxima m of its
//                                                                  whole subtree, which only the log-likelihood needs
//   R[k] = F[k] / exp(O[k]),  G[j] = E[j] * sum_k W[k,j] R[k]       backward (F = parent's G, root: e_0)
//   edge_aggr[k,j] += W[k,j] * sum_b R[b,k] E[b,j];  leaf_flow[u][x_b,u][j] += G[b,j]
#include <hip/hip_ext.h>

#include "hclt_engine.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

namespace pcm {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWideWaves = 4;   // waves of the edge and leaf statistics kernels

// waves of a walk workgroup: one 16-state row tile of the output per wave (8 at K = 128, 4 at K = 64)
template <int K>
constexpr int wide_walk_waves() { return K / 16 > 8 ? 8 : K / 16; }

static void check_launch_w(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

template <int K>
struct WideLds {
  v4f e[K / 16][64];   // E tile of the node
  v4f r[K / 16][64];   // R tile (backward)
  float mx[wide_walk_waves<K>()][16];
};

// Operands of a node's Z that can be requested a node ahead (they do not depend on the node
// before): its own leaf row and the rows of its first three leaf children (their categories come
// packed in one word per example, xn), and up to two value tiles of non-leaf children.  The
// forward walk leaves out the child that was computed just before the node (in post-order the
// last non-leaf child is always the node before): each wave still has its 16 states of that tile
// in registers.  Operands beyond these are fetched at the point of use.
constexpr int kWidePre = 6;
constexpr uint32_t kWideLeaf = 0x80000000u, kWideTile = 0x40000000u;

typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wide_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// What a walk keeps in scalar registers for its requests: one descriptor over the whole leaf (or
// value) table and one over the value tiles, and the strides.  Slots 0..3 of a node's operand list
// are always leaf rows, slots 4..5 always value tiles, so a request is one multiply for the
// offset and a raw buffer load; an absent operand is pushed out of the descriptor's range (the
// load returns zeros and never reaches memory), so there is no control flow for the compiler to
// place waits at and the values stay in flight until the next node consumes them.
struct WideRsrc {
  __amdgpu_buffer_rsrc_t leaf, tile;
  uint32_t leaf_stride, tile_stride, leaf_lane, tile_lane;   // *_lane: this lane's byte offset inside a row / a node's tiles
};

template <int K>
__device__ __forceinline__ WideRsrc wide_rsrcs(const HcltDev& d, int s, int lane) {
  WideRsrc r;
  r.leaf = wide_rsrc(d.leaf, (uint32_t)d.V * d.leaf_stride);
  r.tile = wide_rsrc(d.O, (uint32_t)d.n_inner * d.tile_stride);
  r.leaf_stride = d.leaf_stride;
  r.tile_stride = d.tile_stride;
  r.leaf_lane = (uint32_t)s * d.leaf_slice + (uint32_t)(lane >> 4) * 16;
  r.tile_lane = (uint32_t)s * (kSlice * K * 4) + (uint32_t)lane * 16;
  return r;
}

constexpr uint32_t kWideAbsent = 0x80000000u;   // beyond any table (the host keeps them under 2 GB), and the row-tile steps cannot wrap

template <int K>
__device__ __forceinline__ void wide_request_leaf(const WideRsrc& r, uint32_t op_, uint32_t xpack, int wave,
                                                  v4f (&out)[(K / 16) / wide_walk_waves<K>()]) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  const uint32_t op = (uint32_t)__builtin_amdgcn_readfirstlane((int)op_);
  const uint32_t x = (xpack >> (8u * ((op >> 24) & 3u))) & 0xffu;
  const uint32_t voff = op ? x * (K * 4) + r.leaf_lane : kWideAbsent;
  const uint32_t soff = (op & 0xffffffu) * r.leaf_stride;
#pragma unroll
  for (int q = 0; q < Q; ++q)
    out[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r.leaf, (int)(voff + (wave * Q + q) * 64), (int)soff, 0));
}

template <int K>
__device__ __forceinline__ void wide_request_tile(const WideRsrc& r, uint32_t op_, int wave,
                                                  v4f (&out)[(K / 16) / wide_walk_waves<K>()]) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  const uint32_t op = (uint32_t)__builtin_amdgcn_readfirstlane((int)op_);
  const uint32_t voff = op ? r.tile_lane : kWideAbsent;
  const uint32_t soff = (op & 0xffffffu) * r.tile_stride;
#pragma unroll
  for (int q = 0; q < Q; ++q)
    out[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r.tile, (int)(voff + (wave * Q + q) * 1024), (int)soff, 0));
}

// point-of-use form for the rare operands beyond the prefetched ones
template <int K>
__device__ __forceinline__ void wide_request(const HcltDev& d, uint32_t op, uint32_t xpack, int s, int lane, int wave,
                                             v4f (&out)[(K / 16) / wide_walk_waves<K>()]) {
  const WideRsrc r = wide_rsrcs<K>(d, s, lane);
  if (op & kWideLeaf) wide_request_leaf<K>(r, op, xpack, wave, out);
  else wide_request_tile<K>(r, op, wave, out);
}

// operands beyond the prefetched ones: (variable | kWideLeaf) or (node | kWideTile), categories from xb
template <int K>
__device__ __forceinline__ void wide_extras(const HcltDev& d, const uint32_t* __restrict__ extra, int off, int cnt, int s,
                                            int lane, int wave, v4f (&z)[(K / 16) / wide_walk_waves<K>()]) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  const int col = s * kSlice + (lane & 15);
  for (int i = 0; i < cnt; ++i) {
    const uint32_t op = extra[off + i];
    v4f t[Q];
    if (op & kWideLeaf) {
      const int var = (int)(op & 0xffffffu);
      const uint32_t x = d.xb[(size_t)var * d.Bp + col];
      wide_request<K>(d, kWideLeaf | (uint32_t)var, x, s, lane, wave, t);
    } else {
      wide_request<K>(d, op, 0u, s, lane, wave, t);
    }
#pragma unroll
    for (int q = 0; q < Q; ++q) z[q] += t[q];
  }
}

// The operand table of small trees is copied to LDS once: read from memory it costs every node a
// scalar-cache round trip ahead of its requests.
__device__ __forceinline__ void wide_stage_ops(const WideOps* __restrict__ ops_g, int n_inner, int in_lds, uint32_t* sops_mem) {
  if (!in_lds) return;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(ops_g);
  const int words = n_inner * (int)(sizeof(WideOps) / 4);
  for (int i = threadIdx.x; i < words; i += blockDim.x) sops_mem[i] = src[i];
  __syncthreads();
}

// a node's entry, from LDS (explicitly: a generic pointer would turn every read into a flat load) or memory
__device__ __forceinline__ WideOps wide_ops_at(const WideOps* __restrict__ ops_g, int in_lds, const uint32_t* sops_mem, int n) {
  if (!in_lds) return ops_g[n];
  WideOps o;
  uint32_t* dst = reinterpret_cast<uint32_t*>(&o);
  const uint32_t* src = sops_mem + (size_t)n * (sizeof(WideOps) / 4);
#pragma unroll
  for (int i = 0; i < (int)(sizeof(WideOps) / 4); ++i) dst[i] = src[i];
  return o;
}

// E tile of the node from the waves' slices of Z: the row maxima are combined through LDS, E
// goes to LDS and comes back whole to every wave.  Returns m of the lane's example.  Two
// workgroup barriers.
template <int K>
__device__ __forceinline__ float wide_e_from_z(const v4f (&z)[(K / 16) / wide_walk_waves<K>()], int lane, int wave,
                                               WideLds<K>& L, v4f (&e)[K / 16]) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  const int b = lane & 15, g = lane >> 4;
  float m = -INFINITY;
#pragma unroll
  for (int q = 0; q < Q; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) m = fmaxf(m, z[q][i]);
  {   // lanes ^ 16 and ^ 32 with the row- and half-swap instructions, not through the LDS crossbar
    const int mi = __builtin_bit_cast(int, m);
    const auto r16 = __builtin_amdgcn_permlane16_swap(mi, mi, false, false);
    m = fmaxf(__builtin_bit_cast(float, (int)r16[0]), __builtin_bit_cast(float, (int)r16[1]));
    const int mj = __builtin_bit_cast(int, m);
    const auto r32 = __builtin_amdgcn_permlane32_swap(mj, mj, false, false);
    m = fmaxf(__builtin_bit_cast(float, (int)r32[0]), __builtin_bit_cast(float, (int)r32[1]));
  }
  if (g == 0) L.mx[wave][b] = m;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < WV; ++w) m = fmaxf(m, L.mx[w][b]);
  if (!(m > -INFINITY)) m = 0.f;   // an example of probability zero: E = 0 and a value of -inf, not NaN
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    v4f x;
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = __expf(z[q][i] - m);
    L.e[wave * Q + q][lane] = x;
  }
  __syncthreads();
#pragma unroll
  for (int kt = 0; kt < KT; ++kt) e[kt] = L.e[kt][lane];
  return m;
}

// Forward: one workgroup per 16-example slice walks the nodes children-first.  While a node is
// computed, the rows of the next node's parameter block, its prefetchable operands and the
// categories of the node after it are already on their way.
template <int K>
__global__ __launch_bounds__(wide_walk_waves<K>() * 64) void hclt_wide_forward_kernel(HcltDev d,
                                                                                      const WideOps* __restrict__ ops_g,
                                                                                      int ops_in_lds,
                                                                                      const uint32_t* __restrict__ extra,
                                                                                      float* __restrict__ ll) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  __shared__ WideLds<K> L;
  extern __shared__ uint32_t sops_mem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, s = blockIdx.x;
  const int b = lane & 15, g = lane >> 4, col = s * kSlice + b;
  wide_stage_ops(ops_g, d.n_inner, ops_in_lds, sops_mem);
  const WideRsrc rs = wide_rsrcs<K>(d, s, lane);
  v4f wn[Q][KT], pre[kWidePre][Q], prev_o[Q];
  uint32_t xnext = 0;
  WideOps on_next;
  auto request = [&](int n, uint32_t xpack) {
    const v4f* wf = reinterpret_cast<const v4f*>(d.Wf + (size_t)n * K * K);
#pragma unroll
    for (int q = 0; q < Q; ++q)
#pragma unroll
      for (int jt = 0; jt < KT; ++jt) wn[q][jt] = wf[((wave * Q + q) * KT + jt) * 64 + lane];
    xnext = d.xn[(size_t)min(n + 1, d.n_inner - 1) * d.Bp + col];
    on_next = wide_ops_at(ops_g, ops_in_lds, sops_mem, n);
#pragma unroll
    for (int i = 0; i < 4; ++i) wide_request_leaf<K>(rs, on_next.fwd[i], xpack, wave, pre[i]);
#pragma unroll
    for (int i = 4; i < kWidePre; ++i) wide_request_tile<K>(rs, on_next.fwd[i], wave, pre[i]);
  };
  request(0, d.xn[col]);
#pragma unroll
  for (int q = 0; q < Q; ++q) prev_o[q] = v4f{0.f, 0.f, 0.f, 0.f};
  double msum = 0.0;   // row maxima of all nodes so far: what the tiles leave out of the root's value
  for (int n = 0; n < d.n_inner; ++n) {
    const WideOps on = on_next;
    v4f z[Q], w[Q][KT];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      z[q] = pre[0][q];
#pragma unroll
      for (int i = 1; i < kWidePre; ++i) z[q] += pre[i][q];
#pragma unroll
      for (int jt = 0; jt < KT; ++jt) w[q][jt] = wn[q][jt];
    }
    const uint32_t xcur = xnext;
    request(min(n + 1, d.n_inner - 1), xcur);   // past the last node: a repeat of its requests, never used
    if (on.prev_child)
#pragma unroll
      for (int q = 0; q < Q; ++q) z[q] += prev_o[q];
    if (on.fwd_extra_cnt) wide_extras<K>(d, extra, on.fwd_extra_off, on.fwd_extra_cnt, s, lane, wave, z);
    v4f e[KT];
    const float m = wide_e_from_z<K>(z, lane, wave, L, e);
    msum += (double)m;
    v4f* out = reinterpret_cast<v4f*>(d.O + ((size_t)n * d.nslices + s) * kSlice * K);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      v4f part[4];   // four independent accumulation chains: a chain of KT*4 dependent MFMAs is half a microsecond
#pragma unroll
      for (int i = 0; i < 4; ++i) part[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jt = 0; jt < KT; ++jt)
#pragma unroll
        for (int i = 0; i < 4; ++i) part[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[q][jt][i], e[jt][i], part[i], 0, 0, 0);
      const v4f acc = (part[0] + part[1]) + (part[2] + part[3]);
      v4f o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = __logf(acc[i]);
      out[(wave * Q + q) * 64 + lane] = o;
      prev_o[q] = o;
      if (on.is_root && wave == 0 && q == 0 && g == 0 && col < d.B) ll[col] = (float)(msum + (double)o[0]);
    }
    // no barrier here: a wave reads from memory only what it wrote itself, and the next node's LDS
    // writes sit behind its own barriers
  }
}

// Backward: the same workgroups walk the nodes parents-first.  Besides the flow tile G handed
// to the children, every node leaves R and E in the operand layout of the statistics
// contraction: lane 16*g' + r holds, for t < 4, the value of example 4*t + g' at state
// kt*16 + r (the contraction runs over examples).  A node's own value tile, its operands and its
// parent's flow tile are requested a node ahead; when the parent is the node just computed (the
// last non-leaf child comes right after its parent in this order) its flows are still in registers.
template <int K>
__global__ __launch_bounds__(wide_walk_waves<K>() * 64) void hclt_wide_backward_kernel(HcltDev d,
                                                                                       const WideOps* __restrict__ ops_g,
                                                                                       int ops_in_lds,
                                                                                       const uint32_t* __restrict__ extra,
                                                                                       float* G, float* __restrict__ RS,
                                                                                       float* __restrict__ ES) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  __shared__ WideLds<K> L;
  extern __shared__ uint32_t sops_mem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, s = blockIdx.x;
  const int b = lane & 15, g = lane >> 4, col = s * kSlice + b;
  wide_stage_ops(ops_g, d.n_inner, ops_in_lds, sops_mem);
  const WideRsrc rs = wide_rsrcs<K>(d, s, lane);
  const bool live = col < d.B;
  v4f wn[Q][KT], pre[kWidePre][Q], o_next[Q], f_next[Q], prev_g[Q];
  uint32_t xnext = 0;
  WideOps on_next;
  auto request = [&](int n, uint32_t xpack) {
    const v4f* wb = reinterpret_cast<const v4f*>(d.Wb + (size_t)n * K * K);
#pragma unroll
    for (int q = 0; q < Q; ++q)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) wn[q][kt] = wb[((wave * Q + q) * KT + kt) * 64 + lane];
    xnext = d.xn[(size_t)max(n - 1, 0) * d.Bp + col];
    on_next = wide_ops_at(ops_g, ops_in_lds, sops_mem, n);
#pragma unroll
    for (int i = 0; i < 4; ++i) wide_request_leaf<K>(rs, on_next.bwd[i], xpack, wave, pre[i]);
#pragma unroll
    for (int i = 4; i < kWidePre; ++i) wide_request_tile<K>(rs, on_next.bwd[i], wave, pre[i]);
    const int par = __builtin_amdgcn_readfirstlane(on_next.parent);
    const bool from_mem = par >= 0 && par != n + 1;   // otherwise: the root, or the flows are still in registers
    const __amdgpu_buffer_rsrc_t ro = wide_rsrc(reinterpret_cast<const char*>(d.O) + (size_t)n * d.tile_stride, d.tile_stride);
    const __amdgpu_buffer_rsrc_t rg = wide_rsrc(reinterpret_cast<const char*>(G) + (size_t)max(par, 0) * d.tile_stride,
                                                from_mem ? d.tile_stride : 0u);
    const uint32_t voff = (uint32_t)s * (kSlice * K * 4) + (uint32_t)lane * 16;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      o_next[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(ro, (int)(voff + (wave * Q + q) * 1024), 0, 0));
      f_next[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rg, (int)(voff + (wave * Q + q) * 1024), 0, 0));
    }
  };
  request(d.n_inner - 1, d.xn[(size_t)(d.n_inner - 1) * d.Bp + col]);
#pragma unroll
  for (int q = 0; q < Q; ++q) prev_g[q] = v4f{0.f, 0.f, 0.f, 0.f};
  for (int n = d.n_inner - 1; n >= 0; --n) {
    const WideOps on = on_next;
    v4f z[Q], w[Q][KT], o[Q], f[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      z[q] = pre[0][q];
#pragma unroll
      for (int i = 1; i < kWidePre; ++i) z[q] += pre[i][q];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) w[q][kt] = wn[q][kt];
      o[q] = o_next[q];
      f[q] = f_next[q];
    }
    const uint32_t xcur = xnext;
    request(max(n - 1, 0), xcur);   // past the last node: a repeat of its requests, never used
    if (on.bwd_extra_cnt) wide_extras<K>(d, extra, on.bwd_extra_off, on.bwd_extra_cnt, s, lane, wave, z);
    v4f e[KT];
    wide_e_from_z<K>(z, lane, wave, L, e);
    const size_t tile = ((size_t)n * d.nslices + s) * kSlice * K;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      const int kt = wave * Q + q;
      v4f fq;
      if (on.parent < 0)   // the root: the flow the example starts with (1, or its weight) in state 0
        fq = v4f{kt == 0 && g == 0 && live ? (d.w ? d.w[col] : 1.f) : 0.f, 0.f, 0.f, 0.f};
      else if (on.parent == n + 1) fq = prev_g[q];
      else fq = f[q];
      v4f r;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float sc = __expf(o[q][i]);
        r[i] = (sc > 0.f && fq[i] > 0.f) ? fq[i] / sc : 0.f;
      }
      L.r[kt][lane] = r;
    }
    __syncthreads();
    v4f r[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) r[kt] = L.r[kt][lane];
    v4f* gout = reinterpret_cast<v4f*>(G + tile);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      const int jt = wave * Q + q;
      v4f part[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) part[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) part[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[q][kt][i], r[kt][i], part[i], 0, 0, 0);
      const v4f acc = (part[0] + part[1]) + (part[2] + part[3]);
      prev_g[q] = e[jt] * acc;
      gout[jt * 64 + lane] = prev_g[q];
    }
    // statistics operands: lane = 16*g' + row reads example 4*t + g', state kt*16 + row
    {
      const int row = lane & 15, gp = lane >> 4;
      const int src = 16 * (row >> 2) + gp, comp = row & 3;
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const int kt = wave * Q + q;
        v4f rs, es;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          rs[t] = reinterpret_cast<const float*>(&L.r[kt][src + 4 * t])[comp];
          es[t] = reinterpret_cast<const float*>(&L.e[kt][src + 4 * t])[comp];
        }
        reinterpret_cast<v4f*>(RS + tile)[kt * 64 + lane] = rs;
        reinterpret_cast<v4f*>(ES + tile)[kt * 64 + lane] = es;
      }
    }
    // no barrier here: see the forward walk (L.r and L.e are rewritten only behind the next node's barriers)
  }
}

// Edge statistics: R^T E over all examples.  Workgroup (node n, split p of the slices); its four waves share the
// rows of the block out (K / 64 row tiles each, all columns), so every wave keeps its accumulators to itself, the
// E tile of a slice is read from memory once per workgroup (the four waves' requests meet in L1) and serves
// K / 16 x K / 16 matrix instructions per wave.  (With a workgroup per row tile, as before, every row tile read
// all of E again: 0.5 GB of L2 traffic on C2, which bound the kernel at 77 us.)  The splits' shares go to rows
// of `part` [splits][n_inner * K * K]; sum_parts_kernel adds them in order and weights them.
constexpr int kWideEdgeSplits = 8;
template <int K>
__device__ __forceinline__ void wide_edge_block(const HcltDev& d, const float* __restrict__ RS, const float* __restrict__ ES,
                                                float* __restrict__ part, int n, int split, int n_splits) {
  constexpr int KT = K / 16, RT = KT / kWideWaves;
  static_assert(RT >= 1, "a wave takes at least one row tile");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int per = (d.nslices + n_splits - 1) / n_splits;
  const int s_begin = split * per, s_end = min(s_begin + per, d.nslices);
  v4f acc[RT][KT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int jt = 0; jt < KT; ++jt) acc[rt][jt] = v4f{0.f, 0.f, 0.f, 0.f};
  const v4f* rs = reinterpret_cast<const v4f*>(RS + (size_t)n * d.nslices * kSlice * K);
  const v4f* es = reinterpret_cast<const v4f*>(ES + (size_t)n * d.nslices * kSlice * K);
  v4f a[RT], e[KT];
  auto request = [&](int s) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a[rt] = rs[((size_t)s * KT + wave * RT + rt) * 64 + lane];
#pragma unroll
    for (int jt = 0; jt < KT; ++jt) e[jt] = es[((size_t)s * KT + jt) * 64 + lane];
  };
  if (s_begin < s_end) request(s_begin);
  for (int s = s_begin; s < s_end; ++s) {
    v4f a0[RT], e0[KT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a0[rt] = a[rt];
#pragma unroll
    for (int jt = 0; jt < KT; ++jt) e0[jt] = e[jt];
    if (s + 1 < s_end) request(s + 1);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int jt = 0; jt < KT; ++jt)
          acc[rt][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[rt][t], e0[jt][t], acc[rt][jt], 0, 0, 0);
  }
  float* out = part + ((size_t)split * d.n_inner + n) * K * K;
  const int g = lane >> 4, j0 = lane & 15;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int jt = 0; jt < KT; ++jt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        out[(size_t)((wave * RT + rt) * 16 + 4 * g + i) * K + jt * 16 + j0] = acc[rt][jt][i];
}

// Leaf histograms: workgroup (variable u, state tile kt) adds, for every example, the 16 flows
// of the tile to row x_b of a [C][16] table in LDS, as two-limb fixed-point integers (integer
// LDS atomics are more than ten times cheaper than floating-point ones here and make the sum
// independent of the order of arrival); flows are in [0, 1], or in [0, 2^shift] under per-example weights.
__device__ __forceinline__ void wide_leaf_block(const HcltDev& d, const float* __restrict__ G,
                                                const int32_t* __restrict__ state_node, int K,
                                                float* __restrict__ leaf_flow, float rate, int limb,
                                                const int* __restrict__ flow_shift, int u, int kt) {
  extern __shared__ unsigned hist[];   // [2][C][17]
  constexpr int HS = 17;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = lane & 15, g = lane >> 4;
  const int KT = K / 16;
  const int n = state_node[u];
  const int hw = d.C * HS;
  for (int i = threadIdx.x; i < 2 * hw; i += blockDim.x) hist[i] = 0u;
  __syncthreads();
  // (with per-example weights a flow is at most 2^shift, the bound the host left: counted in units of that)
  const int shift = flow_shift ? __builtin_amdgcn_readfirstlane(*flow_shift) : 0;
  const float scale = __builtin_ldexpf(1.f, limb), unit_inv = __builtin_ldexpf(1.f, -shift);
  const v4f* gt = reinterpret_cast<const v4f*>(G + (size_t)n * d.nslices * kSlice * K);
  for (int s = wave; s < d.nslices; s += kWideWaves) {
    const int col = s * kSlice + b;
    const int x = d.xb[(size_t)u * d.Bp + col];
    const v4f f = gt[((size_t)s * KT + kt) * 64 + lane];
    if (col < d.B) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = fminf(fmaxf(f[i] * unit_inv, 0.f), 1.f) * scale;
        const float fl = floorf(v);
        __hip_atomic_fetch_add(&hist[x * HS + 4 * g + i], (unsigned)fl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_fetch_add(&hist[hw + x * HS + 4 * g + i], (unsigned)((v - fl) * scale), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
  }
  __syncthreads();
  const float hi_inv = __builtin_ldexpf(1.f, shift - limb), lo_inv = __builtin_ldexpf(1.f, shift - 2 * limb);
  for (int i = threadIdx.x; i < d.C * 16; i += blockDim.x) {
    const int c = i >> 4, jj = i & 15;
    const float val = (float)hist[c * HS + jj] * hi_inv + (float)hist[hw + c * HS + jj] * lo_inv;
    const size_t at = ((size_t)u * d.C + c) * K + kt * 16 + jj;
    const float old = rate != 0.f ? rate * leaf_flow[at] : 0.f;
    leaf_flow[at] = old + val;
  }
}

template <int K>
__global__ __launch_bounds__(kWideWaves * 64) void hclt_wide_edge_kernel(HcltDev d, const float* __restrict__ RS,
                                                                         const float* __restrict__ ES,
                                                                         float* __restrict__ part) {
  wide_edge_block<K>(d, RS, ES, part, blockIdx.x, blockIdx.y, gridDim.y);
}

__global__ __launch_bounds__(kWideWaves * 64) void hclt_wide_leaf_kernel(HcltDev d, const float* __restrict__ G,
                                                                         const int32_t* __restrict__ state_node, int K,
                                                                         float* __restrict__ leaf_flow, float rate,
                                                                         int limb, const int* __restrict__ flow_shift) {
  wide_leaf_block(d, G, state_node, K, leaf_flow, rate, limb, flow_shift, blockIdx.x, blockIdx.y);
}

// ---- host --------------------------------------------------------------------------------

#define PCM_DISPATCH_WIDE_K(K_, ...)                                                         \
  switch (K_) {                                                                              \
    case 64: { constexpr int KK = 64; __VA_ARGS__; break; }                                  \
    case 128: { constexpr int KK = 128; __VA_ARGS__; break; }                                \
    default: fail(PCM_ERR_STATE, "no wide block kernel for hidden size %d", K_);             \
  }

// operand tables of the wide walks
void HcltCircuit::build_wide_tables() {
  std::vector<WideOps> t(n_inner_);
  std::vector<uint32_t> extra;
  std::vector<std::vector<int32_t>> ic(n_inner_), lc(n_inner_);
  for (int n = 0; n < n_inner_; ++n)
    for (int c : children_[var_of_inner_[n]]) {
      if (children_[c].empty()) lc[n].push_back(c); else ic[n].push_back(inner_of_var_[c]);
    }
  for (int n = 0; n < n_inner_; ++n) {
    WideOps& o = t[n];
    std::memset(&o, 0, sizeof(o));
    const int v = var_of_inner_[n];
    o.parent = parent_[v] < 0 ? -1 : inner_of_var_[parent_[v]];
    o.is_root = v == root_;
    o.fwd[0] = o.bwd[0] = kWideLeaf | (uint32_t)v;
    for (size_t i = 0; i < lc[n].size() && i < 3; ++i) o.fwd[1 + i] = o.bwd[1 + i] = kWideLeaf | ((uint32_t)(i + 1) << 24) | (uint32_t)lc[n][i];
    std::vector<uint32_t> fx, bx;
    for (size_t i = 3; i < lc[n].size(); ++i) { fx.push_back(kWideLeaf | (uint32_t)lc[n][i]); bx.push_back(fx.back()); }
    int nf = 0, nb = 0;
    for (int c : ic[n]) {
      const uint32_t op = kWideTile | (uint32_t)c;
      if (c == n - 1) o.prev_child = 1;
      else if (nf < 2) o.fwd[4 + nf++] = op;
      else fx.push_back(op);
      if (nb < 2) o.bwd[4 + nb++] = op; else bx.push_back(op);
    }
    o.fwd_extra_off = (int32_t)extra.size(); o.fwd_extra_cnt = (int32_t)fx.size();
    extra.insert(extra.end(), fx.begin(), fx.end());
    o.bwd_extra_off = (int32_t)extra.size(); o.bwd_extra_cnt = (int32_t)bx.size();
    extra.insert(extra.end(), bx.begin(), bx.end());
  }
  if (extra.empty()) extra.push_back(0);
  d_wide_ops_.upload(t);
  d_wide_extra_.upload(extra);
}

void HcltCircuit::wide_forward(const HcltDev& d, float* d_ll) {
  if (d_wide_ops_.n == 0) build_wide_tables();
  if ((size_t)V_ * d.leaf_stride >= ((size_t)1 << 31) || (size_t)n_inner_ * d.tile_stride >= ((size_t)1 << 31))
    fail(PCM_ERR_UNSUPPORTED, "batch of %d examples is too large for one call of the wide kernels", d.B);
  const size_t ops_bytes = (size_t)n_inner_ * sizeof(WideOps);
  const int ops_in_lds = ops_bytes <= 32768;
  // with timing on, a phase's start / stop events ride on its kernels' own dispatches
  hipEvent_t* ev = (timing & 1) ? ev_set() : nullptr;
  PCM_DISPATCH_WIDE_K(K_, hipExtLaunchKernelGGL(hclt_wide_forward_kernel<KK>, dim3(d.nslices), dim3(wide_walk_waves<KK>() * 64),
                                                (uint32_t)(ops_in_lds ? ops_bytes : 0), stream, ev ? ev[0] : nullptr,
                                                ev ? ev[1] : nullptr, 0, d, d_wide_ops_.p, ops_in_lds, d_wide_extra_.p, d_ll));
  check_launch_w("hclt_wide_forward");
}

// soft: the evidence is soft, the caller shares out the leaf flows from the G tiles itself
void HcltCircuit::wide_backward_stats(const HcltDev& d, float rate, bool soft) {
  if (d_wide_state_node_.n == 0) {
    std::vector<int32_t> t(V_);
    for (int v = 0; v < V_; ++v) t[v] = children_[v].empty() ? inner_of_var_[parent_[v]] : inner_of_var_[v];
    d_wide_state_node_.upload(t, stream);
  }
  int bits = 0;
  while ((1 << bits) < d.Bp) ++bits;
  const int limb = std::min(24, 32 - bits);
  if (limb < 12) fail(PCM_ERR_UNSUPPORTED, "batch of %d examples is too large for one call", d.B);
  hipEvent_t* ev = timing ? ev_set() : nullptr;
  const bool t_bwd = timing & 2, t_stat = timing & 4;
  PCM_DISPATCH_WIDE_K(K_, {
    const size_t ops_bytes = (size_t)n_inner_ * sizeof(WideOps);
    const int ops_in_lds = ops_bytes <= 32768;
    hipExtLaunchKernelGGL(hclt_wide_backward_kernel<KK>, dim3(d.nslices), dim3(wide_walk_waves<KK>() * 64),
                          (uint32_t)(ops_in_lds ? ops_bytes : 0), stream, t_bwd ? ev[2] : nullptr, t_bwd ? ev[3] : nullptr, 0, d,
                          d_wide_ops_.p, ops_in_lds, d_wide_extra_.p, d_G_.p, d_wide_rs_.p, d_wide_es_.p);
    check_launch_w("hclt_wide_backward");
    // statistics: the edge blocks by splits of the slices, the splits' sum, and (unless the evidence is soft) the leaf
    // histograms.  (Edge blocks and histograms as two halves of one launch ran slower than one after the other: 357
    // against 320 us per step on C2.)
    const int splits = std::min(kWideEdgeSplits, d.nslices);
    const int64_t n_edge = (int64_t)n_inner_ * KK * KK;
    d_part_.ensure((size_t)splits * n_edge);
    hipExtLaunchKernelGGL(hclt_wide_edge_kernel<KK>, dim3(n_inner_, splits), dim3(kWideWaves * 64), 0, stream,
                          t_stat ? ev[4] : nullptr, nullptr, 0, d, d_wide_rs_.p, d_wide_es_.p, d_part_.p);
    hipExtLaunchKernelGGL(sum_parts_kernel<true>, dim3(ceil_div(n_edge, 64)), dim3(256), 0, stream, nullptr,
                          t_stat && soft ? ev[5] : nullptr, 0, (const float*)d_part_.p, splits, n_edge,
                          (const float*)d_logtheta_.p, d_edge_aggr_.p, rate);
  });
  const size_t lds = 2 * (size_t)C_ * 17 * sizeof(unsigned);
  if (!soft)
    hipExtLaunchKernelGGL(hclt_wide_leaf_kernel, dim3(V_, K_ / 16), dim3(kWideWaves * 64), (uint32_t)lds, stream, nullptr,
                          t_stat ? ev[5] : nullptr, 0, d, d_G_.p, d_wide_state_node_.p, K_, d_leaf_flow_.p, rate, limb,
                          d.w ? (const int*)d_flow_shift_.p : (const int*)nullptr);
  check_launch_w("hclt_wide_stats");
}

}  // namespace pcm
