// Block kernels for wide hidden sizes (K = 128, and K = 64 on trees that do not fill the 16-wave walks): a
// K x K parameter block no longer fits a wave's registers, so a 16-example tile is shared by the waves of a
// workgroup, each producing 16 of the output states and streaming its rows of the block (64 KB per node at
// K = 128, shared by all workgroups through L2) as MFMA A-operands.  Trees with wide blocks are small (tens
// of nodes), so a workgroup walks the nodes of its slice itself, in an order the host lays out (two groups
// of waves, half a step apart: wide_schedule.hpp); tiles travel through memory.
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
#include "wide_schedule.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

namespace pcm {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWideWaves = 4;   // waves of the edge statistics kernel
constexpr int kWideLeafWaves = 16, kWideLeafAhead = 4;   // of the leaf histograms; slices a wave requests before it adds them

// waves of a walk workgroup: one 16-state row tile of the output per wave (8 at K = 128, 4 at K = 64)
template <int K>
constexpr int wide_walk_waves() { return K / 16 > 8 ? 8 : K / 16; }

static void check_launch_w(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

// LDS of one group of waves
template <int K>
struct WideLds {
  v4f e[K / 16][64];   // E tile of the node, each wave's row tile relative to that wave's own maximum (forward)
  float mx[wide_walk_waves<K>()][16];   // the waves' maxima
};
template <int K>
struct WideLdsB {
  v4f r[K / 16][64];   // R tile (backward)
  v4f e[K / 16][64];   // E tile, only for the statistics operands
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

// Barrier that orders LDS only: requests and stores of the wave stay in flight behind it.
__device__ __forceinline__ void wide_lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The schedule of small trees is copied to LDS once: read from memory it costs every slot a
// scalar-cache round trip ahead of its requests.
__device__ __forceinline__ void wide_stage_slots(const WideSlot* __restrict__ tbl, int n_slots, int in_lds, uint32_t* smem) {
  if (!in_lds) return;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(tbl);
  const int words = n_slots * (int)(sizeof(WideSlot) / 4);
  for (int i = threadIdx.x; i < words; i += blockDim.x) smem[i] = src[i];
  __syncthreads();
}

// a slot's entry, from LDS (explicitly: a generic pointer would turn every read into a flat load) or memory
__device__ __forceinline__ WideSlot wide_slot_at(const WideSlot* __restrict__ tbl, int in_lds, const uint32_t* smem, int i) {
  if (!in_lds) return tbl[i];
  WideSlot o;
  uint32_t* dst = reinterpret_cast<uint32_t*>(&o);
  const uint32_t* src = smem + (size_t)i * (sizeof(WideSlot) / 4);
#pragma unroll
  for (int k = 0; k < (int)(sizeof(WideSlot) / 4); ++k) dst[k] = src[k];
  return o;
}

// Forward: one workgroup per 16-example slice walks the nodes children-first.  What a node costs is not only
// its matrix instructions (32 per wave; with two waves of a group on a SIMD, 2048 cycles of its matrix core) but
// also what goes through the compute unit's vector memory path -- the 64 KB parameter block and the operand rows,
// about 1800 cycles at 64 B per cycle -- and the exchange of E between the waves, and with one set of waves
// these add up (5800 cycles per node, measured).  So the workgroup has TWO groups of waves, each with its own
// sequence of nodes (independent subtrees; the host's schedule says which), half a step apart: between two
// barriers one group sums its operands, takes the exponentials and requests its parameter block while the other
// runs its matrix instructions, then they swap.  A group's slot:
//   first half:  Z from the operands requested a slot ahead; the parameter block and the next slot's leaf rows are
//                requested; every wave takes the exponentials of its 16 states against its OWN maximum and leaves
//                tile and maximum in LDS (a maximum agreed on first would cost a barrier and an LDS round trip more);
//   second half: the next slot's value tiles are requested; every wave reads all tiles and maxima, rescales tile w
//                by exp(m_w - m), m the largest of them, and contracts; logarithms; the tile goes to memory.
// The barrier after the first half waits for the wave's memory traffic (the group is ahead of the other there
// anyway), the one after the second half only for LDS: a tile is in memory for the other group three half-steps
// after its slot began.
// The maxima m go to d.M: the backward walk takes them from there.
template <int K>
__global__ __launch_bounds__(2 * wide_walk_waves<K>() * 64) void hclt_wide_forward_kernel(HcltDev d,
                                                                                          const WideSlot* __restrict__ tbl,
                                                                                          int n_steps, int tbl_in_lds,
                                                                                          const uint32_t* __restrict__ extra,
                                                                                          float* __restrict__ ll) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  constexpr int NW = Q * KT;   // parameter row tiles a wave holds
  __shared__ WideLds<K> Lg[2];
  __shared__ double msum_of[2][16];
  extern __shared__ uint32_t slots_mem[];
  const int lane = threadIdx.x & 63, wave_all = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wave_all / WV, wave = wave_all % WV, s = blockIdx.x;
  const int b = lane & 15, g = lane >> 4, col = s * kSlice + b;
  WideLds<K>& L = Lg[grp];
  wide_stage_slots(tbl, 2 * n_steps, tbl_in_lds, slots_mem);
  const WideRsrc rs = wide_rsrcs<K>(d, s, lane);
  v4f w[NW], pre[kWidePre][Q], prev_o[Q];
  auto request_leaves = [&](const WideSlot& sl, uint32_t xpack) {
#pragma unroll
    for (int i = 0; i < 4; ++i) wide_request_leaf<K>(rs, sl.op[i], xpack, wave, pre[i]);
  };
  auto request_tiles = [&](const WideSlot& sl) {
#pragma unroll
    for (int i = 4; i < kWidePre; ++i) wide_request_tile<K>(rs, sl.op[i], wave, pre[i]);
  };
  auto slot_or_idle = [&](int t) {
    if (t < n_steps) return wide_slot_at(tbl, tbl_in_lds, slots_mem, t * 2 + grp);
    WideSlot idle = {};
    idle.node = -1;
    return idle;
  };
  auto cats_of = [&](const WideSlot& sl) { return sl.node >= 0 ? d.xn[(size_t)sl.node * d.Bp + col] : 0u; };
  WideSlot nxt = slot_or_idle(0);
  uint32_t xnext = cats_of(nxt);   // packed categories of the slot after the current one
  if (nxt.node >= 0) { request_leaves(nxt, xnext); request_tiles(nxt); }
  xnext = cats_of(slot_or_idle(1));
#pragma unroll
  for (int q = 0; q < Q; ++q) prev_o[q] = v4f{0.f, 0.f, 0.f, 0.f};
  double msum = 0.0;   // row maxima of this group's nodes: what the tiles leave out of the root's value
  float root_o = 0.f;
  bool has_root = false;
  if (grp == 1) __syncthreads();   // half a step behind
  for (int t = 0; t < n_steps; ++t) {
    const WideSlot cur = nxt;
    const int n = __builtin_amdgcn_readfirstlane(cur.node);
    nxt = slot_or_idle(t + 1);
    const int nn = __builtin_amdgcn_readfirstlane(nxt.node);
    // ---- first half
    if (n >= 0) {
      v4f z[Q];
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        z[q] = pre[0][q];
#pragma unroll
        for (int i = 1; i < kWidePre; ++i) z[q] += pre[i][q];
      }
      if (cur.flags & kWidePrev)
#pragma unroll
        for (int q = 0; q < Q; ++q) z[q] += prev_o[q];
      {
        const v4f* wf = reinterpret_cast<const v4f*>(d.Wf + (size_t)n * K * K);
#pragma unroll
        for (int i = 0; i < NW; ++i) w[i] = wf[((wave * Q + i / KT) * KT + i % KT) * 64 + lane];
      }
      if (cur.extra_cnt) wide_extras<K>(d, extra, cur.extra_off, cur.extra_cnt, s, lane, wave, z);
      if (nn >= 0) request_leaves(nxt, xnext);   // (they depend on no other node; the tiles wait for the second half)
      float mw = -INFINITY;
#pragma unroll
      for (int q = 0; q < Q; ++q)
#pragma unroll
        for (int i = 0; i < 4; ++i) mw = fmaxf(mw, z[q][i]);
      {   // lanes ^ 16 and ^ 32 with the row- and half-swap instructions, not through the LDS crossbar
        const int mi = __builtin_bit_cast(int, mw);
        const auto r16 = __builtin_amdgcn_permlane16_swap(mi, mi, false, false);
        mw = fmaxf(__builtin_bit_cast(float, (int)r16[0]), __builtin_bit_cast(float, (int)r16[1]));
        const int mj = __builtin_bit_cast(int, mw);
        const auto r32 = __builtin_amdgcn_permlane32_swap(mj, mj, false, false);
        mw = fmaxf(__builtin_bit_cast(float, (int)r32[0]), __builtin_bit_cast(float, (int)r32[1]));
      }
      const bool some = mw > -INFINITY;   // otherwise: all 16 states impossible, E = 0 (and not exp(-inf + inf))
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        v4f x;
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = some ? __expf(z[q][i] - mw) : 0.f;
        L.e[wave * Q + q][lane] = x;
      }
      if (g == 0) L.mx[wave][b] = mw;
    } else if (nn >= 0) {
      request_leaves(nxt, xnext);
    }
    __syncthreads();   // (with everything of this wave in memory: the tile of its slot before, which the other group may ask for from here on)
    // ---- second half
    if (nn >= 0) request_tiles(nxt);
    xnext = cats_of(slot_or_idle(t + 2));
    if (n >= 0) {
      float mall[WV], m = -INFINITY;
#pragma unroll
      for (int w2 = 0; w2 < WV; ++w2) {
        mall[w2] = L.mx[w2][b];
        m = fmaxf(m, mall[w2]);
      }
      if (!(m > -INFINITY)) m = 0.f;   // an example of probability zero: E = 0 and a value of -inf, not NaN
      msum += (double)m;
      if (wave == 0 && g == 0) d.M[(size_t)n * d.Bp + col] = m;
      v4f* out = reinterpret_cast<v4f*>(d.O + ((size_t)n * d.nslices + s) * kSlice * K);
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        v4f part[4];   // four independent accumulation chains: a chain of KT*4 dependent MFMAs is half a microsecond
#pragma unroll
        for (int i = 0; i < 4; ++i) part[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jt = 0; jt < KT; ++jt) {
          const v4f e = L.e[jt][lane] * __expf(mall[jt / Q] - m);
#pragma unroll
          for (int i = 0; i < 4; ++i) part[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[q * KT + jt][i], e[i], part[i], 0, 0, 0);
        }
        const v4f acc = (part[0] + part[1]) + (part[2] + part[3]);
        v4f o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = __logf(acc[i]);
        out[(wave * Q + q) * 64 + lane] = o;
        prev_o[q] = o;
        if ((cur.flags & kWideRoot) && wave == 0 && q == 0) { root_o = o[0]; has_root = true; }
      }
    }
    wide_lds_barrier();   // (the tile's store and the next slot's requests stay in flight)
  }
  if (grp == 0) __syncthreads();
  if (wave == 0 && g == 0) msum_of[grp][b] = msum;
  __syncthreads();
  if (has_root && g == 0 && col < d.B) ll[col] = (float)((msum_of[0][b] + msum_of[1][b]) + (double)root_o);
}

// Backward: the same workgroups walk the nodes parents-first, again as two groups of waves half a step apart.
// Besides the flow tile G handed to the children, every node leaves R and E in the operand layout of the
// statistics contraction: lane 16*g' + r holds, for t < 4, the value of example 4*t + g' at state
// kt*16 + r (the contraction runs over examples).  A node's own value tile, its operands, its row maxima
// (left by the forward walk) and its parent's flow tile are requested a slot ahead; when the parent was the
// group's slot before, its flows are still in registers.  So a wave has E and R of its own 16 states without
// asking the others: they go to LDS in the first half of the slot, and in the second every wave reads the whole
// R tile and contracts.
template <int K>
__global__ __launch_bounds__(2 * wide_walk_waves<K>() * 64) void hclt_wide_backward_kernel(HcltDev d,
                                                                                           const WideSlot* __restrict__ tbl,
                                                                                           int n_steps, int tbl_in_lds,
                                                                                           const uint32_t* __restrict__ extra,
                                                                                           float* G, float* __restrict__ RS,
                                                                                           float* __restrict__ ES) {
  constexpr int KT = K / 16, WV = wide_walk_waves<K>(), Q = KT / WV;
  constexpr int NW = Q * KT;
  __shared__ WideLdsB<K> Lg[2];
  extern __shared__ uint32_t slots_mem[];
  const int lane = threadIdx.x & 63, wave_all = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wave_all / WV, wave = wave_all % WV, s = blockIdx.x;
  const int b = lane & 15, g = lane >> 4, col = s * kSlice + b;
  WideLdsB<K>& L = Lg[grp];
  wide_stage_slots(tbl, 2 * n_steps, tbl_in_lds, slots_mem);
  const WideRsrc rs = wide_rsrcs<K>(d, s, lane);
  const bool live = col < d.B;
  v4f w[NW], pre[kWidePre][Q], o_next[Q], f_next[Q], prev_g[Q];
  float m_next = 0.f;
  const uint32_t voff = (uint32_t)s * (kSlice * K * 4) + (uint32_t)lane * 16;
  // what depends on no other node of this walk: the operands of Z, the node's own value tile and its row maxima
  auto request_own = [&](const WideSlot& sl, uint32_t xpack) {
    const int n = __builtin_amdgcn_readfirstlane(sl.node);
    m_next = d.M[(size_t)n * d.Bp + col];
#pragma unroll
    for (int i = 0; i < 4; ++i) wide_request_leaf<K>(rs, sl.op[i], xpack, wave, pre[i]);
#pragma unroll
    for (int i = 4; i < kWidePre; ++i) wide_request_tile<K>(rs, sl.op[i], wave, pre[i]);
    const __amdgpu_buffer_rsrc_t ro = wide_rsrc(reinterpret_cast<const char*>(d.O) + (size_t)n * d.tile_stride, d.tile_stride);
#pragma unroll
    for (int q = 0; q < Q; ++q)
      o_next[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(ro, (int)(voff + (wave * Q + q) * 1024), 0, 0));
  };
  // the parent's flow tile
  auto request_flow = [&](const WideSlot& sl) {
    const int par = __builtin_amdgcn_readfirstlane(sl.parent);
    const bool from_mem = par >= 0 && !(sl.flags & kWidePrev);   // otherwise: the root, or the flows are still in registers
    const __amdgpu_buffer_rsrc_t rg = wide_rsrc(reinterpret_cast<const char*>(G) + (size_t)max(par, 0) * d.tile_stride,
                                                from_mem ? d.tile_stride : 0u);
#pragma unroll
    for (int q = 0; q < Q; ++q)
      f_next[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rg, (int)(voff + (wave * Q + q) * 1024), 0, 0));
  };
  auto slot_or_idle = [&](int t) {
    if (t < n_steps) return wide_slot_at(tbl, tbl_in_lds, slots_mem, t * 2 + grp);
    WideSlot idle = {};
    idle.node = -1;
    return idle;
  };
  auto cats_of = [&](const WideSlot& sl) { return sl.node >= 0 ? d.xn[(size_t)sl.node * d.Bp + col] : 0u; };
  WideSlot nxt = slot_or_idle(0);
  uint32_t xnext = cats_of(nxt);   // packed categories of the slot after the current one
  if (nxt.node >= 0) { request_own(nxt, xnext); request_flow(nxt); }
  xnext = cats_of(slot_or_idle(1));
#pragma unroll
  for (int q = 0; q < Q; ++q) prev_g[q] = v4f{0.f, 0.f, 0.f, 0.f};
  if (grp == 1) __syncthreads();   // half a step behind
  for (int t = 0; t < n_steps; ++t) {
    const WideSlot cur = nxt;
    const int n = __builtin_amdgcn_readfirstlane(cur.node);
    nxt = slot_or_idle(t + 1);
    const int nn = __builtin_amdgcn_readfirstlane(nxt.node);
    const size_t tile = ((size_t)max(n, 0) * d.nslices + s) * kSlice * K;
    v4f e[Q];
    // ---- first half
    if (n >= 0) {
      v4f z[Q];
      const float m = m_next;
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        z[q] = pre[0][q];
#pragma unroll
        for (int i = 1; i < kWidePre; ++i) z[q] += pre[i][q];
      }
      {
        const v4f* wb = reinterpret_cast<const v4f*>(d.Wb + (size_t)n * K * K);
#pragma unroll
        for (int i = 0; i < NW; ++i) w[i] = wb[((wave * Q + i / KT) * KT + i % KT) * 64 + lane];
      }
      if (cur.extra_cnt) wide_extras<K>(d, extra, cur.extra_off, cur.extra_cnt, s, lane, wave, z);
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const int kt = wave * Q + q;
#pragma unroll
        for (int i = 0; i < 4; ++i) e[q][i] = __expf(z[q][i] - m);
        L.e[kt][lane] = e[q];
        v4f fq;
        if (cur.parent < 0)   // the root: the flow the example starts with (1, or its weight) in state 0
          fq = v4f{kt == 0 && g == 0 && live ? (d.w ? d.w[col] : 1.f) : 0.f, 0.f, 0.f, 0.f};
        else if (cur.flags & kWidePrev) fq = prev_g[q];
        else fq = f_next[q];
        v4f r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float sc = __expf(o_next[q][i]);
          r[i] = (sc > 0.f && fq[i] > 0.f) ? fq[i] / sc : 0.f;
        }
        L.r[kt][lane] = r;
      }
    }
    if (nn >= 0) request_own(nxt, xnext);
    __syncthreads();   // (with everything of this wave in memory: the flow tile of its slot before, which the other group may ask for from here on)
    // ---- second half
    if (nn >= 0) request_flow(nxt);
    xnext = cats_of(slot_or_idle(t + 2));
    if (n >= 0) {
      v4f* gout = reinterpret_cast<v4f*>(G + tile);
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const int jt = wave * Q + q;
        v4f part[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) part[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
          const v4f r = L.r[kt][lane];
#pragma unroll
          for (int i = 0; i < 4; ++i) part[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[q * KT + kt][i], r[i], part[i], 0, 0, 0);
        }
        const v4f acc = (part[0] + part[1]) + (part[2] + part[3]);
        prev_g[q] = e[q] * acc;
        gout[jt * 64 + lane] = prev_g[q];
      }
      // statistics operands: lane = 16*g' + row reads example 4*t + g', state kt*16 + row
      const int row = lane & 15, gp = lane >> 4;
      const int src = 16 * (row >> 2) + gp, comp = row & 3;
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const int kt = wave * Q + q;
        v4f rst, est;
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
          rst[t4] = reinterpret_cast<const float*>(&L.r[kt][src + 4 * t4])[comp];
          est[t4] = reinterpret_cast<const float*>(&L.e[kt][src + 4 * t4])[comp];
        }
        reinterpret_cast<v4f*>(RS + tile)[kt * 64 + lane] = rst;
        reinterpret_cast<v4f*>(ES + tile)[kt * 64 + lane] = est;
      }
    }
    wide_lds_barrier();   // (the stores and the next slot's request stay in flight)
  }
  if (grp == 0) __syncthreads();
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
  // (a wave's slices a few at a time, all requests first: one slice after the other, every slice cost a round trip)
  for (int s0 = wave; s0 < d.nslices; s0 += kWideLeafWaves * kWideLeafAhead) {
    int x[kWideLeafAhead];
    v4f f[kWideLeafAhead];
#pragma unroll
    for (int a = 0; a < kWideLeafAhead; ++a) {
      const int s = min(s0 + a * kWideLeafWaves, d.nslices - 1);
      x[a] = d.xb[(size_t)u * d.Bp + s * kSlice + b];
      f[a] = gt[((size_t)s * KT + kt) * 64 + lane];
    }
#pragma unroll
    for (int a = 0; a < kWideLeafAhead; ++a) {
      const int s = s0 + a * kWideLeafWaves;
      if (s >= d.nslices || s * kSlice + b >= d.B) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = fminf(fmaxf(f[a][i] * unit_inv, 0.f), 1.f) * scale;
        const float fl = floorf(v);
        __hip_atomic_fetch_add(&hist[x[a] * HS + 4 * g + i], (unsigned)fl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_fetch_add(&hist[hw + x[a] * HS + 4 * g + i], (unsigned)((v - fl) * scale), __ATOMIC_RELAXED,
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

__global__ __launch_bounds__(kWideLeafWaves * 64) void hclt_wide_leaf_kernel(HcltDev d, const float* __restrict__ G,
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

// schedules and operand tables of the wide walks
void HcltCircuit::build_wide_tables() {
  std::vector<int> par(n_inner_);
  std::vector<std::vector<int32_t>> ic(n_inner_), lc(n_inner_);
  for (int n = 0; n < n_inner_; ++n) {
    const int v = var_of_inner_[n];
    par[n] = parent_[v] < 0 ? -1 : inner_of_var_[parent_[v]];
    for (int c : children_[v]) {
      if (children_[c].empty()) lc[n].push_back(c); else ic[n].push_back(inner_of_var_[c]);
    }
  }
  std::vector<uint32_t> extra;
  auto table = [&](bool forward, int& n_steps) {
    const WideSchedule sch = wide_two_group_schedule(par, forward);
    const int bad = wide_schedule_fault(par, forward, sch);
    if (bad >= 0) fail(PCM_ERR_STATE, "schedule of the wide %s walk: node %d would run ahead of its operands", forward ? "forward" : "backward", bad);
    n_steps = sch.n_steps;
    std::vector<WideSlot> t((size_t)sch.n_steps * 2);
    for (auto& o : t) { std::memset(&o, 0, sizeof(o)); o.node = -1; o.parent = -1; }
    for (int n = 0; n < n_inner_; ++n) {
      WideSlot& o = t[(size_t)sch.step[n] * 2 + sch.group[n]];
      const int v = var_of_inner_[n];
      o.node = n;
      o.parent = par[n];
      o.flags = v == root_ ? kWideRoot : 0;
      o.op[0] = kWideLeaf | (uint32_t)v;
      for (size_t i = 0; i < lc[n].size() && i < 3; ++i) o.op[1 + i] = kWideLeaf | ((uint32_t)(i + 1) << 24) | (uint32_t)lc[n][i];
      o.extra_off = (int32_t)extra.size();
      for (size_t i = 3; i < lc[n].size(); ++i) extra.push_back(kWideLeaf | (uint32_t)lc[n][i]);
      int tiles = 0;
      for (int c : ic[n]) {
        // going up, the child of the group's slot before is still in registers
        if (forward && sch.group[c] == sch.group[n] && sch.step[c] == sch.step[n] - 1) { o.flags |= kWidePrev; continue; }
        const uint32_t op = kWideTile | (uint32_t)c;
        if (tiles < 2) o.op[4 + tiles++] = op; else extra.push_back(op);
      }
      if (!forward && par[n] >= 0 && sch.group[par[n]] == sch.group[n] && sch.step[par[n]] == sch.step[n] - 1) o.flags |= kWidePrev;
      o.extra_cnt = (int32_t)extra.size() - o.extra_off;
    }
    return t;
  };
  d_wide_fwd_.upload(table(true, wide_steps_f_));
  d_wide_bwd_.upload(table(false, wide_steps_b_));
  if (extra.empty()) extra.push_back(0);
  d_wide_extra_.upload(extra);
}

void HcltCircuit::wide_forward(const HcltDev& d, float* d_ll) {
  if (d_wide_fwd_.n == 0) build_wide_tables();
  if ((size_t)V_ * d.leaf_stride >= ((size_t)1 << 31) || (size_t)n_inner_ * d.tile_stride >= ((size_t)1 << 31))
    fail(PCM_ERR_UNSUPPORTED, "batch of %d examples is too large for one call of the wide kernels", d.B);
  const size_t tbl_bytes = (size_t)wide_steps_f_ * 2 * sizeof(WideSlot);
  const int tbl_in_lds = tbl_bytes <= 16384;
  // with timing on, a phase's start / stop events ride on its kernels' own dispatches
  hipEvent_t* ev = (timing & 1) ? ev_set() : nullptr;
  PCM_DISPATCH_WIDE_K(K_, hipExtLaunchKernelGGL(hclt_wide_forward_kernel<KK>, dim3(d.nslices), dim3(2 * wide_walk_waves<KK>() * 64),
                                                (uint32_t)(tbl_in_lds ? tbl_bytes : 0), stream, ev ? ev[0] : nullptr,
                                                ev ? ev[1] : nullptr, 0, d, d_wide_fwd_.p, wide_steps_f_, tbl_in_lds,
                                                d_wide_extra_.p, d_ll));
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
    const size_t tbl_bytes = (size_t)wide_steps_b_ * 2 * sizeof(WideSlot);
    const int tbl_in_lds = tbl_bytes <= 16384;
    hipExtLaunchKernelGGL(hclt_wide_backward_kernel<KK>, dim3(d.nslices), dim3(2 * wide_walk_waves<KK>() * 64),
                          (uint32_t)(tbl_in_lds ? tbl_bytes : 0), stream, t_bwd ? ev[2] : nullptr, t_bwd ? ev[3] : nullptr, 0, d,
                          d_wide_bwd_.p, wide_steps_b_, tbl_in_lds, d_wide_extra_.p, d_G_.p, d_wide_rs_.p, d_wide_es_.p);
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
  if (!soft && soft_reg_ > 0.f) PCM_HIP(hipMemsetAsync(d_leaf_hist_.p, 0, d_leaf_hist_.n * sizeof(float), stream));   // (the kernel adds to rate x what is there)
  if (!soft)
    hipExtLaunchKernelGGL(hclt_wide_leaf_kernel, dim3(V_, K_ / 16), dim3(kWideLeafWaves * 64), (uint32_t)lds, stream, nullptr,
                          t_stat ? ev[5] : nullptr, 0, d, d_G_.p, d_wide_state_node_.p, K_, stats_leaf_out(), rate, limb,
                          d.w ? (const int*)d_flow_shift_.p : (const int*)nullptr);
  check_launch_w("hclt_wide_stats");
  if (!soft) soft_reg_counts(rate);
}

}  // namespace pcm
