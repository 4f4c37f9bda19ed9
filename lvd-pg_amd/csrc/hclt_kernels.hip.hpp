// gfx950 kernels of the dense-block HCLT engine.
//
// Work decomposition.  Examples are independent, tree nodes are not: a node's value needs
// its children's values (forward) and its parent's flows (backward).  The forward and
// backward kernels therefore give each workgroup ONE slice of 16 examples and let it walk
// the whole tree in host-scheduled steps: in every step each of the 16 waves takes at most
// one tree node whose dependencies were produced in earlier steps, and the waves meet at a
// workgroup barrier -- no grid-wide synchronisation exists anywhere.  The tile a step
// produces for later steps (a node's values going up, the flow handed to its children
// going down) stays in LDS in a slot the host allocated; everything else a step needs is
// static, so it is requested from HBM one step ahead.  The sufficient statistics (edge
// flows summed over the batch, leaf histograms) need the whole batch per node instead, so
// a third kernel gives each workgroup one tree node and all slices.
//
// Register tile.  A wave holds a [16 examples x K states] tile as K/16 float4 per lane:
// lane = 16*g + b owns example b and states kt*16 + 4*g + i (kt < K/16, i < 4).  This is
// both the B-operand layout and the accumulator layout of v_mfma_f32_16x16x4_f32 with the
// parameter block as A-operand (rows = output states), so the output tile of one
// contraction feeds the next one, LDS and HBM unchanged.  Tiles are stored as K/16 runs of
// 64 float4 (1 KiB, fully coalesced).
#pragma once

#include <hip/hip_runtime.h>

#include "hclt_engine.hpp"
#include "stage_kernel.hip.hpp"

namespace pcm {

typedef float v4f __attribute__((ext_vector_type(4)));

// Cache policy of the tile stores (gfx950 buffer "aux" bits: sc0 = 1, nt = 2, sc1 = 16).
// Value and flow tiles are written once and read next by another kernel, long after far
// more than the caches' capacity has gone by: written through, non-temporal.  On the
// 3072-variable benchmark this alone takes 20 % off the forward kernel (the default policy
// makes every store burst wait on L2 allocation).
constexpr int kStreamStore = 1 | 2 | 16;
constexpr int kStreamLoad = 2;   // value and ratio tiles are read once per kernel: non-temporal, so that they do not push the
                                 // parameter blocks and leaf tables (read by every workgroup) out of the caches

// ceil(log2) of the largest per-example weight, at least 0: the bound on one example's flow that the statistics
// kernels' fixed-point counters are scaled by (heads_backward leaves the same bound for a head mask).
__global__ __launch_bounds__(256) void hclt_weight_shift_kernel(const float* __restrict__ w, int B, int* __restrict__ shift) {
  __shared__ int best;
  if (threadIdx.x == 0) best = 0;
  __syncthreads();
  int mine = 0;
  for (int b = threadIdx.x; b < B; b += blockDim.x) {
    int ex = 0;
    // (weights must be finite and >= 0: a binding checks that; what is not counts as the largest float here,
    // so that the scale stays defined whatever arrives)
    const float wb = w[b] >= 0.f ? fminf(w[b], 3.0e38f) : (w[b] < 0.f ? 0.f : 3.0e38f);
    if (frexpf(wb, &ex) == 0.5f) --ex;   // w <= 2^ex (a power of two is its own bound)
    mine = max(mine, ex);
  }
  atomicMax(&best, mine);
  __syncthreads();
  if (threadIdx.x == 0) *shift = best;
}

constexpr int kStatWaves = 12;   // waves per workgroup in the statistics kernel (168 registers each)

template <int K>
struct Tile {
  v4f v[K / 16];
};

template <int K>
__device__ __forceinline__ void tile_zero(Tile<K>& t) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) t.v[kt] = v4f{0.f, 0.f, 0.f, 0.f};
}

template <int K>
__device__ __forceinline__ void tile_add(Tile<K>& a, const Tile<K>& b) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) a.v[kt] += b.v[kt];
}

// Per-thread constants of the address arithmetic.  Every global access is "uniform 64-bit
// base + 32-bit per-lane byte offset", so the per-lane cost is one or two integer adds.
struct LaneOffs {
  uint32_t tile;   // byte offset of this lane's first float4 inside a node's [nslices] tile row
  uint32_t leaf;   // byte offset of this lane's first float4 inside a leaf-table row
  int bcol;        // batch column of this lane's example
};

template <int K>
__device__ __forceinline__ LaneOffs lane_offs(int slice, int lane) {
  LaneOffs o;
  o.tile = (uint32_t)slice * (kSlice * K * 4) + (uint32_t)lane * 16;
  o.leaf = (uint32_t)(lane >> 4) * 16;
  o.bcol = slice * kSlice + (lane & 15);
  return o;
}

template <int K>
__device__ __forceinline__ LaneOffs lane_offs(const HcltDev& d, int slice, int lane) {
  LaneOffs o = lane_offs<K>(slice, lane);
  o.leaf += (uint32_t)slice * d.leaf_slice;
  return o;
}

// All HBM traffic of the hot kernels goes through raw buffer descriptors (uniform base +
// size in scalar registers, 32-bit per-lane byte offset).  A descriptor of size 0 makes the
// access a no-op that still counts as issued: loads return zeros, stores are dropped, and
// nothing reaches the memory system.  That is how absent operands and idle waves are handled
// without branches, which keeps the number of requests in flight the same on every path.
typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <int K>
__device__ __forceinline__ void tile_load(const float* base, int node, uint32_t node_stride_bytes,
                                          uint32_t voff, Tile<K>& t) {
  const __amdgpu_buffer_rsrc_t r = make_rsrc(reinterpret_cast<const char*>(base) + (size_t)max(node, 0) * node_stride_bytes,
                                             node >= 0 ? node_stride_bytes : 0u);
  const uint32_t v = node >= 0 ? voff : 0u, step = node >= 0 ? 1024u : 0u;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    t.v[kt] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(v + kt * step), 0, 0));
}

template <int K>
__device__ __forceinline__ void tile_store(float* base, int node, uint32_t node_stride_bytes, uint32_t voff,
                                           const Tile<K>& t) {
  const __amdgpu_buffer_rsrc_t r = make_rsrc(reinterpret_cast<char*>(base) + (size_t)max(node, 0) * node_stride_bytes,
                                             node >= 0 ? node_stride_bytes : 0u);
  const uint32_t v = node >= 0 ? voff : 0u, step = node >= 0 ? 1024u : 0u;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, t.v[kt]), r, (int)(v + kt * step), 0, kStreamStore);
}

template <int K>
__device__ __forceinline__ void lds_tile_load(const float* lds, int slot, int lane, Tile<K>& t) {
  const v4f* p = reinterpret_cast<const v4f*>(lds + (size_t)slot * (kSlice * K));
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) t.v[kt] = p[kt * 64 + lane];
}

template <int K>
__device__ __forceinline__ void lds_tile_store(float* lds, int slot, int lane, const Tile<K>& t) {
  v4f* p = reinterpret_cast<v4f*>(lds + (size_t)slot * (kSlice * K));
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt) p[kt * 64 + lane] = t.v[kt];
}

__device__ __forceinline__ int load_x(const HcltDev& d, int var, int bcol) {
  return d.xb[(size_t)var * d.Bp + bcol];
}

// One static operand of a step: a leaf-table row (needs the category x), a value tile, or
// nothing (kOpNone: zeros, no request).  Skipping a request is safe for the request-ahead
// pipeline because everything issued AFTER the operands of a step (parameter block,
// categories, stores) is issued unconditionally: waiting until only those remain in flight
// always covers the operands, however many of them there were.
template <int K>
__device__ __forceinline__ void operand_load(const HcltDev& d, uint32_t op, uint32_t xpack, const LaneOffs& lo,
                                             Tile<K>& t) {
  if (op == kOpNone) {
    tile_zero<K>(t);
    return;
  }
  const bool leaf = (op & kOpLeaf) != 0;
  const uint32_t id = op & kOpIdMask;
  const char* base = leaf ? reinterpret_cast<const char*>(d.leaf) + (size_t)id * d.leaf_stride
                          : reinterpret_cast<const char*>(d.O) + (size_t)id * d.tile_stride;
  const __amdgpu_buffer_rsrc_t r = make_rsrc(base, leaf ? d.leaf_stride : d.tile_stride);
  const uint32_t x = (xpack >> (((op >> kXSelShift) & 3u) * 8u)) & 0xffu;
  const uint32_t voff = leaf ? x * (K * 4) + lo.leaf : lo.tile;
  const uint32_t step = leaf ? 64u : 1024u;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    t.v[kt] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(voff + kt * step), 0, 0));
}

// Categories of this lane's example for the leaf-row operands of a node, four bytes packed
// into one word (byte i: the operand whose selector is i); one request per item.
__device__ __forceinline__ uint32_t xpack_load(const HcltDev& d, int node, int bcol) {
  const __amdgpu_buffer_rsrc_t r = make_rsrc(d.xn + (size_t)max(node, 0) * d.Bp, node >= 0 ? (uint32_t)d.Bp * 4u : 0u);
  return __builtin_amdgcn_raw_buffer_load_b32(r, node >= 0 ? bcol * 4 : 0, 0, 0);
}

constexpr float kFlowRatioCap = 3.0e38f;   // largest value of 1 / S a flow is multiplied by
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Per-example maximum over the K states (the lanes b, b+16, b+32, b+48 share an example).
template <int K>
__device__ __forceinline__ float tile_rowmax(const Tile<K>& z) {
  float m = -INFINITY;
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
    for (int i = 0; i < 4; ++i) m = fmaxf(m, z.v[kt][i]);
  // lanes ^ 16 and ^ 32 with the row- and half-swap instructions (both operands equal: the two
  // results hold the two partners), not through the LDS crossbar
  {
    const int mi = __builtin_bit_cast(int, m);
    const auto r = __builtin_amdgcn_permlane16_swap(mi, mi, false, false);
    m = fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
  }
  {
    const int mi = __builtin_bit_cast(int, m);
    const auto r = __builtin_amdgcn_permlane32_swap(mi, mi, false, false);
    m = fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
  }
  return m == -INFINITY ? 0.f : m;
}

template <int K>
__device__ __forceinline__ void tile_exp_sub(Tile<K>& z, float m) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
    for (int i = 0; i < 4; ++i) z.v[kt][i] = __builtin_amdgcn_exp2f(fmaf(z.v[kt][i], kLog2e, -m * kLog2e));
}

// A node's parameter block as MFMA A-operands: float4 (row tile rt, column tile ct, lane)
// holds W[rt*16 + lane%16][ct*16 + 4*(lane/16) + 0..3].
template <int K>
struct WTile {
  v4f a[(K / 16) * (K / 16)];
};

template <int K>
__device__ __forceinline__ void w_load(const float* Wops, int node, int lane, WTile<K>& w) {
  const __amdgpu_buffer_rsrc_t r = make_rsrc(Wops + (size_t)max(node, 0) * K * K, node >= 0 ? K * K * 4u : 0u);
  const int v = node >= 0 ? lane * 16 : 0, step = node >= 0 ? 1024 : 0;
#pragma unroll
  for (int i = 0; i < (K / 16) * (K / 16); ++i)
    w.a[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, v + i * step, 0, 0));
}

// out[b, r] = sum_c W[r, c] * in[b, c] on the matrix cores.
template <int K>
__device__ __forceinline__ void contract(const WTile<K>& w, const Tile<K>& in, Tile<K>& out) {
  constexpr int KT = K / 16;
#pragma unroll
  for (int rt = 0; rt < KT; ++rt) {
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ct = 0; ct < KT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.a[rt * KT + ct][i], in.v[ct][i], acc, 0, 0, 0);
    out.v[rt] = acc;
  }
}

// Barrier that orders LDS only: HBM stores of a step keep draining behind it.  kFull is
// used when some dependency tile had to go through HBM.
template <bool kFull>
__device__ __forceinline__ void step_barrier() {
  if (kFull) {
    __syncthreads();
  } else {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  }
}

// Static operands beyond the kPre requested ahead (nodes with many children): fetched at
// the point of use, with the stall that implies.
template <int K>
__device__ __forceinline__ void operands_extra(const HcltDev& d, const StepItem* __restrict__ it, int n_g,
                                               int ext_off, int ext_cnt, const LaneOffs& lo, Tile<K>& z) {
  const int bcol = lo.bcol;
  for (int i = kPre; i < n_g; ++i) {
    Tile<K> t;
    const uint32_t op = it->g[i];
    operand_load<K>(d, op & ~(3u << kXSelShift), (op & kOpLeaf) ? (uint32_t)load_x(d, (int)(op & kOpIdMask), bcol) : 0u, lo, t);
    tile_add<K>(z, t);
  }
  const uint32_t* ext = d.ext_ops + ext_off;
  for (int i = 0; i < ext_cnt; ++i) {
    Tile<K> t;
    const uint32_t op = ext[i];
    operand_load<K>(d, op & ~(3u << kXSelShift), (op & kOpLeaf) ? (uint32_t)load_x(d, (int)(op & kOpIdMask), bcol) : 0u, lo, t);
    tile_add<K>(z, t);
  }
}

// What the statistics kernel keeps of its node's item in scalar registers.
struct PreRegs {
  int node, wnode;
  uint32_t g0, g1, g2;
};
static_assert(kPre == 3, "PreRegs holds three operands");

template <int K>
__device__ __forceinline__ void pre_request_ops(const HcltDev& d, const PreRegs& q, uint32_t xpack,
                                                const LaneOffs& lo, Tile<K> (&P)[kPre]) {
  operand_load<K>(d, q.g0, xpack, lo, P[0]);
  operand_load<K>(d, q.g1, xpack, lo, P[1]);
  operand_load<K>(d, q.g2, xpack, lo, P[2]);
}

// The step schedule of a walk is stored field by field, one row of n_steps entries per wave
// (kSchedFields rows per wave).  A wave keeps 64 consecutive steps of every field in
// registers, one step per lane, and reads the entry of a step with v_readlane: the inner
// loop does no scalar memory loads (whose latency a step is too short to hide).
struct SchedChunk {
  int v[kSchedFields];
  int base;
};

__device__ __forceinline__ void sched_refill(const int32_t* __restrict__ fields, int stride, int wave, int lane,
                                             int base, SchedChunk& c) {
#pragma unroll
  for (int f = 0; f < kSchedFields; ++f) c.v[f] = fields[((size_t)f * kWalkWaves + wave) * stride + base + lane];
  c.base = base;
}

__device__ __forceinline__ int sched_get(const SchedChunk& c, int field, int step) {
  return __builtin_amdgcn_readlane(c.v[field], step - c.base);
}

__device__ __forceinline__ PreRegs sched_pre(const SchedChunk& c, int step) {
  PreRegs q;
  q.node = sched_get(c, kFNode, step);
  q.wnode = sched_get(c, kFWnode, step);
  q.g0 = (uint32_t)sched_get(c, kFG0, step);
  q.g1 = (uint32_t)sched_get(c, kFG1, step);
  q.g2 = (uint32_t)sched_get(c, kFG2, step);
  return q;
}

// The walk kernels run a three-stage software pipeline over the steps.  At the top of
// step s a wave (1) consumes what it requested during step s-1 -- the static operands and
// parameter block of its item of step s and the categories for step s+1 --, (2) requests
// the operands and parameters of step s+1 and the categories of step s+2, (3) computes
// step s.  Every wave issues the same loads and stores in every step (an idle wave through
// empty buffer descriptors), so the waits the compiler places count exactly the requests
// that must have landed and never the ones just issued.
//
// ---- forward: O'_v = log(E W^T), E = exp(Z' - m) ---------------------------------------
// Static operands: the node's own leaf row and its leaf children's rows.  Dependencies:
// the value tiles of its inner children, read from their LDS slots (kSpill: or from HBM).
// The tiles hold log S only; the row maxima m_v go to d.M (when it is there) and their sum over all
// nodes is added to the root's tile value for the log-likelihood: see hclt_forward_lean_kernel.
template <int K, bool kSpill>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_forward_kernel(
    HcltDev d, const int32_t* __restrict__ fields, int stride, const StepItem* __restrict__ sched,
    int n_steps, float* __restrict__ ll_out) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  const LaneOffs lo = lane_offs<K>(d, slice, lane);
  const int bcol = lo.bcol;

  // prologue: the rows carry 64 idle steps past n_steps, so no index needs a guard
  SchedChunk sc;
  sched_refill(fields, stride, wave, lane, 0, sc);
  Tile<K> P[kPre];
  WTile<K> wn;
  uint32_t xs;
  {
    const PreRegs q0 = sched_pre(sc, 0), q1 = sched_pre(sc, 1);
    const uint32_t x0 = xpack_load(d, q0.wnode, bcol);
    pre_request_ops<K>(d, q0, x0, lo, P);
    w_load<K>(d.Wf, q0.wnode, lane, wn);
    xs = xpack_load(d, q1.wnode, bcol);
  }
  float ll = 0.f;
  double msum = 0.0;

  for (int s = 0; s < n_steps; ++s) {
    if (s - sc.base >= 61) sched_refill(fields, stride, wave, lane, s, sc);
    // (1) consume
    Tile<K> z = P[0];
#pragma unroll
    for (int i = 1; i < kPre; ++i) tile_add<K>(z, P[i]);
    const WTile<K> w = wn;
    const uint32_t xc = xs;
    // (2) request
    const PreRegs qa = sched_pre(sc, s + 1);
    pre_request_ops<K>(d, qa, xc, lo, P);
    w_load<K>(d.Wf, qa.wnode, lane, wn);
    xs = xpack_load(d, sched_get(sc, kFWnode, s + 2), bcol);
    // (3) compute
    const int node = sched_get(sc, kFStore, s), out_slot = sched_get(sc, kFOutSlot, s);
    const int flags = sched_get(sc, kFFlags, s);
    const int n_l = flags >> 8;
    if (flags & kItemOverflow) {
      const StepItem* itp = sched + (size_t)s * kWalkWaves + wave;
      operands_extra<K>(d, itp, itp->n_g, itp->ext_off, itp->ext_cnt, lo, z);
    }
#pragma unroll
    for (int c = 0; c < kInlineLds; ++c) {
      if (c < n_l) {
        const uint32_t l = (uint32_t)sched_get(sc, kFL0 + c, s);
        const int slot = (int)(l >> kSlotShift) - 1;
        Tile<K> t;
        if (!kSpill || slot >= 0) lds_tile_load<K>(lds, slot, lane, t);
        else tile_load<K>(d.O, (int)(l & kOpIdMask), d.tile_stride, lo.tile, t);
        tile_add<K>(z, t);
      }
    }
    const float m = tile_rowmax<K>(z);
    tile_exp_sub<K>(z, m);
    Tile<K> o;
    contract<K>(w, z, o);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o.v[kt][i] = __builtin_amdgcn_logf(o.v[kt][i]) * kLn2;
    tile_store<K>(d.O, node, d.tile_stride, lo.tile, o);
    lds_tile_store<K>(lds, out_slot, lane, o);
    if (node >= 0) {   // (idle waves have no node)
      msum += (double)m;
      if (d.M && lane < 16) d.M[(size_t)node * d.Bp + bcol] = m;
    }
    if (flags & kItemRoot) ll = o.v[0][0];
    step_barrier<kSpill>();
  }
  if (!ll_out) return;
  // the waves' sums of row maxima, added in wave order (the last step's barrier has freed the slots)
  double* part = reinterpret_cast<double*>(lds);
  if (lane < 16) part[wave * 16 + lane] = msum;
  __syncthreads();
  if (wave == 0 && lane < 16 && bcol < d.B) {   // the root is item 0 of the last step
    double tot = 0.0;
#pragma unroll
    for (int w = 0; w < kWalkWaves; ++w) tot += part[w * 16 + lane];
    ll_out[bcol] = (float)(tot + (double)ll);
  }
}

// ---- backward: R_v = F_v / S_v, G_v = E_v .* (R_v W_v) ----------------------------------
// Static operands: own leaf row, children's value tiles, leaf children's rows (-> E_v), and
// the node's own value tile O'_v (-> S_v = exp(O'_v)).  Dependency: F_v = G_parent from
// its LDS slot.  R_v goes to HBM for the statistics kernel, G_v to an LDS slot for the
// children (kSpill: to HBM when no slot was free).
// kHeads: multi-head circuit; the head kernel has left the root's ratio tile in memory.
template <int K, bool kSpill, bool kHeads>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_backward_kernel(
    HcltDev d, const int32_t* __restrict__ fields, int stride, const StepItem* __restrict__ sched,
    int n_steps) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  const LaneOffs lo = lane_offs<K>(d, slice, lane);
  const int bcol = lo.bcol;

  SchedChunk sc;
  sched_refill(fields, stride, wave, lane, 0, sc);
  Tile<K> P[kPre], ovn;
  WTile<K> wn;
  uint32_t xs;
  {
    const PreRegs q0 = sched_pre(sc, 0), q1 = sched_pre(sc, 1);
    const uint32_t x0 = xpack_load(d, q0.wnode, bcol);
    pre_request_ops<K>(d, q0, x0, lo, P);
    tile_load<K>(d.O, q0.node, d.tile_stride, lo.tile, ovn);
    w_load<K>(d.Wb, q0.wnode, lane, wn);
    xs = xpack_load(d, q1.wnode, bcol);
  }

  for (int s = 0; s < n_steps; ++s) {
    if (s - sc.base >= 61) sched_refill(fields, stride, wave, lane, s, sc);
    Tile<K> e = P[0];
#pragma unroll
    for (int i = 1; i < kPre; ++i) tile_add<K>(e, P[i]);
    const Tile<K> ov = ovn;
    const WTile<K> w = wn;
    const uint32_t xc = xs;
    const PreRegs qa = sched_pre(sc, s + 1);
    pre_request_ops<K>(d, qa, xc, lo, P);
    tile_load<K>(d.O, qa.node, d.tile_stride, lo.tile, ovn);
    w_load<K>(d.Wb, qa.wnode, lane, wn);
    xs = xpack_load(d, sched_get(sc, kFWnode, s + 2), bcol);

    const int node = sched_get(sc, kFStore, s), out_slot = sched_get(sc, kFOutSlot, s);
    const int in_slot = sched_get(sc, kFL0, s), flags = sched_get(sc, kFFlags, s);
    if (flags & kItemOverflow) {
      const StepItem* itp = sched + (size_t)s * kWalkWaves + wave;
      operands_extra<K>(d, itp, itp->n_g, itp->ext_off, itp->ext_cnt, lo, e);
    }
    const float m = tile_rowmax<K>(e);
    tile_exp_sub<K>(e, m);
    Tile<K> r, t;
    if (!kSpill || in_slot >= 0) lds_tile_load<K>(lds, in_slot, lane, r);
    else tile_load<K>(d.G, sched_get(sc, kFL1, s), d.tile_stride, lo.tile, r);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i)   // capped: a state (or a whole example) of probability zero has flow 0, not 0 * inf
        r.v[kt][i] *= fminf(__builtin_amdgcn_exp2f(ov.v[kt][i] * -kLog2e), kFlowRatioCap);
    if (flags & kItemRoot) {
      if (kHeads) {   // the heads' flows, already divided by their sums
        tile_load<K>(d.R, node, d.tile_stride, lo.tile, r);
      } else {        // flow 1 into the single root sum node of every live example
        tile_zero<K>(r);
        const bool live = lane < 16 && bcol < d.B;
        const float wgt = (d.w && live) ? d.w[bcol] : 1.f;   // per-example weights: the flow the example starts with
        r.v[0][0] = live ? wgt * fminf(__builtin_amdgcn_exp2f(ov.v[0][0] * -kLog2e), kFlowRatioCap) : 0.f;
      }
    }
    tile_store<K>(d.R, node, d.tile_stride, lo.tile, r);
    contract<K>(w, r, t);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt) t.v[kt] *= e.v[kt];
    lds_tile_store<K>(lds, out_slot, lane, t);
    if (kSpill && (flags & kItemSpillOut)) tile_store<K>(d.G, node, d.tile_stride, lo.tile, t);
    step_barrier<kSpill>();
  }
}

// ---- statistics: one workgroup per tree node, all slices ------------------------------
//   edge_aggr[v][k][j] = rate*old + W[k][j] * sum_b R[b,k] E[b,j]
//   leaf_flow[u][c][j] = rate*old + sum_b [x_b,u = c] G_v[b,j]   for u = v and v's leaf children
// with G_v = E .* (R W) recomputed from R_v (stored by the backward kernel) and the node's
// static operands; same request-ahead pipeline as the walks, over the wave's slices.
//
// Leaf histograms.  The scatter-add of every example's K flows into row x_b of a C x K table
// is done with LDS atomics, but not floating-point ones: ds_add_f32 retires about one lane
// per three cycles on this hardware, integer LDS atomics a whole wave in under ten.  Flows
// are non-negative and at most 1, so each is added as a fixed-point number split into two
// integer limbs of `limb` bits (hi + lo, 2*limb fractional bits in total); with
// limb = 32 - ceil(log2(batch)) neither limb sum can overflow, and 2*limb >= 32 bits keep the
// quantisation below fp32 rounding of the result.  The sum is also independent of the order
// in which the waves arrive.
//
// LDS (32-bit words): [nh][2][C][K+1] limb histograms | [waves][16][K+16] transposition pads.
// kSoft (soft evidence): no histograms; the child-flow tiles G replace the ratio tiles for the
// leaf-flow kernel.  A build of its own: the same store behind a run-time flag, never taken, was
// enough to make the second histogram pass of the categorical build lose flow.
template <int K, bool kSoft>
__global__ __launch_bounds__(kStatWaves * 64) void hclt_stats_kernel(
    HcltDev d, const StepItem* __restrict__ items, float* __restrict__ edge_aggr,
    float* __restrict__ leaf_flow, float rate, int nh, int hist_words, int limb, const int* __restrict__ flow_shift) {
  constexpr int KT = K / 16;
  constexpr int LD = K + 16;   // row stride of the pad: conflict-free column reads
  constexpr int HS = K + 1;    // row stride of a histogram: spreads equal states over banks
  extern __shared__ float smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = lane & 15, g = lane >> 4;
  const int nwaves = blockDim.x >> 6;
  // flows lie in [0, 2^shift]: 1 per example in a single-head circuit, the largest total head mask of an
  // example (left on the device by the head kernel) in a multi-head one
  const int shift = flow_shift ? __builtin_amdgcn_readfirstlane(*flow_shift) : 0;
  const float cap = __builtin_ldexpf(1.f, shift);
  const int n = blockIdx.x;
  const StepItem* itp = items + n;
  PreRegs q;
  q.node = n; q.wnode = n; q.g0 = itp->g[0]; q.g1 = itp->g[1]; q.g2 = itp->g[2];
  const int it_flags = itp->flags, it_ng = itp->n_g, it_eo = itp->ext_off, it_ec = itp->ext_cnt;
  const HcltNode nd = d.nodes[n];
  const int hist_sz = d.C * HS;                     // words per limb table
  unsigned* hist = reinterpret_cast<unsigned*>(smem);
  float* pad = smem + hist_words + (size_t)wave * (kSlice * LD);
  const int nu = kSoft ? 1 : 1 + nd.lc_cnt;
  const int last = d.nslices - 1;
  const float hi_scale = __builtin_ldexpf(1.f, limb - shift), lo_scale = __builtin_ldexpf(1.f, limb);

  WTile<K> w;
  w_load<K>(d.Wb, n, lane, w);
  v4f accA[KT][KT];
#pragma unroll
  for (int a = 0; a < KT; ++a)
#pragma unroll
    for (int c = 0; c < KT; ++c) accA[a][c] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int u0 = 0; u0 < nu; u0 += nh) {
    const int nhere = min(nh, nu - u0);
    if (!kSoft)
      for (int i = threadIdx.x; i < nhere * 2 * hist_sz; i += blockDim.x) hist[i] = 0u;
    __syncthreads();

    // prologue (slices past the end are clamped: harmless repeated loads)
    Tile<K> P[kPre], rn;
    uint32_t xs, xc;   // packed categories of the next-but-one / next slice (after the top: next / current)
    {
      const int sa = min(wave, last), sb = min(wave + nwaves, last);
      const LaneOffs la = lane_offs<K>(d, sa, lane);
      xc = xpack_load(d, n, la.bcol);
      pre_request_ops<K>(d, q, xc, la, P);
      tile_load<K>(d.R, n, d.tile_stride, la.tile, rn);
      xs = xpack_load(d, n, sb * kSlice + b);
    }
    for (int s0 = wave; s0 < d.nslices; s0 += nwaves) {
      const int s1 = min(s0 + nwaves, last), s2 = min(s0 + 2 * nwaves, last);
      Tile<K> e = P[0];
#pragma unroll
      for (int i = 1; i < kPre; ++i) tile_add<K>(e, P[i]);
      const Tile<K> r0 = rn;
      const uint32_t xh = xc;   // packed categories of the slice computed now
      xc = xs;
      const LaneOffs l1 = lane_offs<K>(d, s1, lane);
      pre_request_ops<K>(d, q, xc, l1, P);
      tile_load<K>(d.R, n, d.tile_stride, l1.tile, rn);
      xs = xpack_load(d, n, s2 * kSlice + b);

      if (it_flags & kItemOverflow) operands_extra<K>(d, itp, it_ng, it_eo, it_ec, lane_offs<K>(d, s0, lane), e);
      const float m = tile_rowmax<K>(e);
      tile_exp_sub<K>(e, m);
      Tile<K> t;
      contract<K>(w, r0, t);
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) t.v[kt] *= e.v[kt];
      const int bcol = s0 * kSlice + b;
      if (u0 == 0) {
        // A += R^T E over the 16 examples of the tile (contraction over examples): both
        // operands go through the wave's pad to reach the [state][example] operand layout
        float ra[4][KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<v4f*>(&pad[b * LD + kt * 16 + 4 * g]) = r0.v[kt];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) ra[s][kt] = pad[(4 * s + g) * LD + kt * 16 + b];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<v4f*>(&pad[b * LD + kt * 16 + 4 * g]) = e.v[kt];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          float eb[KT];
#pragma unroll
          for (int jt = 0; jt < KT; ++jt) eb[jt] = pad[(4 * s + g) * LD + jt * 16 + b];
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int jt = 0; jt < KT; ++jt)
              accA[kt][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[s][kt], eb[jt], accA[kt][jt], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      if (kSoft) {
        tile_store<K>(d.R, n, d.tile_stride, lane_offs<K>(s0, lane).tile, t);   // r0 of this slice is in registers
      } else if (bcol < d.B) {
        // fixed-point limbs of this lane's K/4 flows (clamped to [0, 2^shift])
        unsigned hi[KT][4], lo[KT][4];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float v = fminf(fmaxf(t.v[kt][i], 0.f), cap) * hi_scale;
            const float fl = floorf(v);
            hi[kt][i] = (unsigned)fl;
            lo[kt][i] = (unsigned)((v - fl) * lo_scale);
          }
        for (int h = 0; h < nhere; ++h) {
          // histogram variable u0+h: 0 is the node's own variable, then its leaf children;
          // the categories of the first four are in the packed word
          const int sel = u0 + h;
          const int u = sel == 0 ? nd.var : d.child_leaf[nd.lc_off + sel - 1];
          const int x = sel < 4 ? (int)((xh >> (8 * sel)) & 0xffu) : load_x(d, u, bcol);
          unsigned* hrow = hist + (size_t)h * 2 * hist_sz + x * HS;
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              __hip_atomic_fetch_add(&hrow[kt * 16 + 4 * g + i], hi[kt][i], __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_WORKGROUP);
              __hip_atomic_fetch_add(&hrow[hist_sz + kt * 16 + 4 * g + i], lo[kt][i], __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
      }
    }
    __syncthreads();
    const float hi_inv = __builtin_ldexpf(1.f, shift - limb), lo_inv = __builtin_ldexpf(1.f, shift - 2 * limb);
    for (int h = 0; h < nhere && !kSoft; ++h) {
      const int u = (u0 + h == 0) ? nd.var : d.child_leaf[nd.lc_off + u0 + h - 1];
      float* dst = leaf_flow + (size_t)u * d.C * K;
      const unsigned* src = hist + (size_t)h * 2 * hist_sz;
      for (int i = threadIdx.x; i < d.C * K; i += blockDim.x) {
        const int c = i / K, j = i % K;
        const float val = (float)src[c * HS + j] * hi_inv + (float)src[hist_sz + c * HS + j] * lo_inv;
        const float old = rate != 0.f ? rate * dst[i] : 0.f;
        dst[i] = old + val;
      }
    }
    __syncthreads();
  }

  // combine the waves' partial A through LDS, scale by W, write the node's block once.  A wave's lanes hold
  // every cell of the block exactly once, so the waves add their blocks in turn, wave 0 first: plain
  // read-modify-writes in a fixed order, the same sum on every run
  float* abuf = smem;
  for (int i = threadIdx.x; i < K * K; i += blockDim.x) abuf[i] = 0.f;
  __syncthreads();
  for (int turn = 0; turn < (int)(blockDim.x >> 6); ++turn) {
    if (turn == (int)(threadIdx.x >> 6)) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int jt = 0; jt < KT; ++jt)
#pragma unroll
          for (int v = 0; v < 4; ++v) abuf[(kt * 16 + 4 * g + v) * K + jt * 16 + b] += accA[kt][jt][v];
    }
    __syncthreads();
  }
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

// Parameter vector <-> block form (src/misc.jl:5-135 on the block layout): sum parameters are
// gathered / scattered through their positions in logtheta; the leaf tables [V][C][K] turn into
// the input nodes' runs of C values (node (v, j) at in_pos[v*K + j] * C) through LDS, 64
// categories of one variable per workgroup, so both sides move whole rows.
__global__ void hclt_params_gather_kernel(int64_t ns, const int64_t* __restrict__ src, const float* __restrict__ logtheta,
                                          float* __restrict__ vec) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < ns) vec[i] = logtheta[src[i]];
}

__global__ void hclt_params_scatter_kernel(int64_t ns, const int64_t* __restrict__ src, const float* __restrict__ vec,
                                           float* __restrict__ logtheta) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < ns) logtheta[src[i]] = vec[i];
}

constexpr int kLeafVecCats = 64;

template <bool kToVector>
__global__ __launch_bounds__(256) void hclt_leaf_vector_kernel(float* __restrict__ leaf, const int32_t* __restrict__ in_pos,
                                                               int K, int C, float* __restrict__ vec) {
  extern __shared__ float turn[];   // [kLeafVecCats][K + 1]
  const int v = blockIdx.x, c0 = blockIdx.y * kLeafVecCats, nc = min(kLeafVecCats, C - c0);
  float* rows = leaf + ((size_t)v * C + c0) * K;
  if (kToVector) {
    for (int i = threadIdx.x; i < nc * K; i += 256) turn[(i / K) * (K + 1) + i % K] = rows[i];
    __syncthreads();
    for (int i = threadIdx.x; i < nc * K; i += 256) {
      const int j = i / nc, cc = i % nc;
      vec[(size_t)in_pos[v * K + j] * C + c0 + cc] = turn[cc * (K + 1) + j];
    }
  } else {
    for (int i = threadIdx.x; i < nc * K; i += 256) {
      const int j = i / nc, cc = i % nc;
      turn[cc * (K + 1) + j] = vec[(size_t)in_pos[v * K + j] * C + c0 + cc];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nc * K; i += 256) rows[i] = turn[(i / K) * (K + 1) + i % K];
  }
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

// Sum-edge update (add_pseudocount, aggr_node_flows, update_params of the reference's EM
// step): a group of min(K, 64) lanes per sum node (tree node n, state k), so that a row of K
// edges is read and written in whole cache lines.
template <int K>
__global__ __launch_bounds__(256) void hclt_theta_update_kernel(const HcltNode* __restrict__ nodes,
                                                                float* __restrict__ logtheta, float* __restrict__ Wf,
                                                                float* __restrict__ Wb, float* __restrict__ edge_aggr,
                                                                int n_inner, float pseudocount, float inertia,
                                                                int skip_root, const int32_t* __restrict__ void_pass) {
  constexpr int G = K < 64 ? K : 64, E = K / G, RPB = 256 / G;
  const int row = blockIdx.x * RPB + threadIdx.x / G, l = threadIdx.x % G;
  if (row >= n_inner * K) return;
  if (void_pass && *void_pass) return;   // a walk of this pass gave up: its statistics must not reach the parameters
  const int n = row / K, k = row % K;
  // a root keeps one sum node (row 0), or none under heads (identity block); an auxiliary node (is_root 2) is all identity
  if (nodes[n].is_root && (k > 0 || skip_root || nodes[n].is_root == 2)) return;
  float* a = edge_aggr + (size_t)row * K;
  float* lt = logtheta + (size_t)row * K;
  const float share = pseudocount / (float)K;
  float av[E], tot = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    av[e] = a[l + e * G] + share;
    a[l + e * G] = av[e];
    tot += av[e];
  }
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) tot += __shfl_xor(tot, o, G);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int j = l + e * G;
    const float oldv = inertia * expf(lt[j]);
    const float newv = (1.f - inertia) * av[e] / tot;
    const float lg = logf(oldv + newv);
    lt[j] = lg;
    put_w<K>(Wf + (size_t)n * K * K, Wb + (size_t)n * K * K, k, j, expf(lg));
  }
}

// ---- soft_reg: smoothing of categorical data (src/regularization/reg_likelihood.jl:4-14, reg_flow.jl:3-22) ----------
// The smoothed value of a leaf depends on the example only through its category x:
//   soft_loglikelihood = log((1 - s) p[x] + s * mean(p[c], c in the window of x)),
//   window: c_start = max(0, x - width / 2) .. c_end = min(c_start + width - 1, C - 1),
// so it is a table of the shape of the leaf table itself, and the walks and the statistics kernel run on it as they
// run on the leaf table, on the categories as they are.  The statistics then hold, per leaf and category x, the flow
// of the examples that SHOWED x; soft_flow shares such an example's flow out over x and its window, which is a
// banded linear map of that histogram, applied by hclt_soft_counts_kernel.
__device__ __forceinline__ void soft_window(int x, int width, int C, int& c0, int& c1) {
  c0 = max(0, x - width / 2);
  c1 = min(c0 + width - 1, C - 1);
}

// smooth[v][x][k] from leaf[v][c][k]; thread = (v, x, k), k fastest
__global__ __launch_bounds__(256) void hclt_leaf_smooth_kernel(const float* __restrict__ leaf, float* __restrict__ smooth,
                                                               int64_t total, int C, int K, float s, int width) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int k = (int)(i % K), x = (int)((i / K) % C);
  const float* row = leaf + (i / ((int64_t)C * K)) * (int64_t)C * K + k;
  int c0, c1;
  soft_window(x, width, C, c0, c1);
  float sp = 0.f;
  for (int c = c0; c <= c1; ++c) sp += __expf(row[(int64_t)c * K]);
  sp /= (float)(c1 - c0 + 1);
  // PCs.logsumexp(logp + log(1 - s), log(sp) + log(s)), written on the probabilities
  smooth[i] = __logf((1.f - s) * __expf(row[(int64_t)x * K]) + s * sp);
}

// The same smoothing as soft evidence, for the engine without a smoothed leaf table (tempered flows of a smoothed
// batch run on the layered form): ev[b][v][c] = log((c == x) (1 - s) + (c in window(x)) s / n(x)), x the category example
// b shows at variable v -- under it a leaf's value is soft_loglikelihood and the share of its flow that category c
// gets is that of the derivative form below.  Thread = (b, v, c), c fastest.
__global__ __launch_bounds__(256) void hclt_soft_reg_evidence_kernel(BatchRef b, int V, int C, float s, int width,
                                                                    float* __restrict__ ev) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)b.batch * V * C) return;
  const int c = (int)(i % C), v = (int)((i / C) % V);
  const int64_t e = i / ((int64_t)C * V);
  const int64_t ex = b.d_idx ? b.d_idx[e] : e;
  const int x = b.d_data[ex * b.stride_ex + (int64_t)v * b.stride_var];
  int c0, c1;
  soft_window(x, width, C, c0, c1);
  float w = c >= c0 && c <= c1 ? s / (float)(c1 - c0 + 1) : 0.f;
  if (c == x) w += 1.f - s;
  ev[i] = __logf(w);   // (-inf outside the window)
}

// leaf_flow[v][c][k] = rate * leaf_flow[v][c][k] + sum over the categories x whose window holds c (or x = c) of
//   hist[v][x][k] * ((x == c) (1 - s) q[x] + (c in window(x)) s / n(x) q[c]) / base(x),
// where hist is the statistics' histogram by shown category.  soft_flow as the source has it (reg_flow.jl:12-17) takes
// q = the heap entries, i.e. LOG-probabilities, and base = (1 - s) logp[x] + s mean(p[window]) (as_written != 0);
// the derivative of the smoothed value -- the form of soft_flow_params, src/nodes/fixable_categorical_dist.jl:141-160 --
// takes q = p and base = (1 - s) p[x] + s mean(p[window]) = exp(smooth[x]).
__global__ __launch_bounds__(256) void hclt_soft_counts_kernel(const float* __restrict__ leaf, const float* __restrict__ smooth,
                                                               const float* __restrict__ hist, float* __restrict__ leaf_flow,
                                                               int64_t total, int C, int K, float s, int width, float rate,
                                                               int as_written) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int k = (int)(i % K), c = (int)((i / K) % C);
  const int64_t base_v = (i / ((int64_t)C * K)) * (int64_t)C * K + k;
  const float lc = leaf[base_v + (int64_t)c * K];
  const float qc = as_written ? lc : __expf(lc);
  float acc = 0.f;
  // x - width / 2 <= c (or c_start = 0) and c <= c_start + width - 1: x within [c - width, c + width / 2]
  for (int x = max(0, c - width); x <= min(C - 1, c + width / 2); ++x) {
    int c0, c1;
    soft_window(x, width, C, c0, c1);
    const bool in_window = c >= c0 && c <= c1;
    if (!in_window && x != c) continue;
    const float h = hist[base_v + (int64_t)x * K];
    if (h == 0.f) continue;
    const float lx = leaf[base_v + (int64_t)x * K], bs = __expf(smooth[base_v + (int64_t)x * K]);
    const float base = as_written ? (1.f - s) * lx + (bs - (1.f - s) * __expf(lx)) : bs;
    float coef = 0.f;
    if (x == c) coef += (1.f - s) * qc;
    if (in_window) coef += s / (float)(c1 - c0 + 1) * qc;
    acc += h * coef / base;
  }
  leaf_flow[i] = (rate != 0.f ? rate * leaf_flow[i] : 0.f) + acc;
}

// Leaf update (the reference's per-input-node update with missing_flow = 0), one workgroup
// per (variable, run of 32 hidden states): thread (category group cg, hidden state j) holds the
// flows and parameters of its categories (every kCats-th one) in registers -- all of its requests
// are in flight at once, and nothing is read twice -- sums its flows, the groups are combined
// through LDS, then every thread rewrites its categories.  Consecutive threads touch consecutive
// addresses.  blockDim.x * kCats >= 32 * C.
// missing != 0: row C - 1 is not a category but the marker of a missing value: its flow is the reference's
// missing_flow (src/nodes/fixable_categorical_dist.jl:233-241: a missing value spreads over the categories as the
// leaf's own distribution), its log-probability stays 0, and the pseudocount is shared by the C - 1 real categories.
template <int kCats>
__global__ __launch_bounds__(1024) void hclt_leaf_update_kernel(float* __restrict__ leaf,
                                                               const float* __restrict__ leaf_flow, int C, int K,
                                                               float pseudocount, float inertia, int missing,
                                                               const int32_t* __restrict__ void_pass) {
  __shared__ float part[1024];
  __shared__ float miss[32];
  if (void_pass && *void_pass) return;   // (uniform: every thread reads the same word)
  const int u = blockIdx.x;
  const int jl = threadIdx.x & 31, cg = threadIdx.x >> 5, ncg = blockDim.x >> 5;
  const int j = blockIdx.y * 32 + jl;
  const bool valid = j < K;
  float* lp = leaf + (size_t)u * C * K;
  const float* fl = leaf_flow + (size_t)u * C * K;
  float f[kCats], p[kCats];
#pragma unroll
  for (int q = 0; q < kCats; ++q) {
    const int c = cg + q * ncg;
    const bool in = valid && c < C;
    f[q] = in ? __builtin_nontemporal_load(&fl[(size_t)c * K + j]) : 0.f;   // read once; the parameters are what should stay cached
    p[q] = in ? lp[(size_t)c * K + j] : 0.f;
  }
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < kCats; ++q) {
    s += f[q];
    if (missing && cg + q * ncg == C - 1) miss[jl] = f[q];
  }
  part[threadIdx.x] = s;
  __syncthreads();
  if (!valid) return;
  float node_flow = pseudocount;   // (the marker's flow is part of the sum, as the reference adds missing_flow)
  for (int q = 0; q < ncg; ++q) node_flow += part[q * 32 + jl];
  const int n_real = missing ? C - 1 : C;
  const float missing_flow = missing ? miss[jl] : 0.f;
  const float cat_pc = pseudocount / (float)n_real, scale = (1.f - inertia) / node_flow;
#pragma unroll
  for (int q = 0; q < kCats; ++q) {
    const int c = cg + q * ncg;
    const float oldp = __expf(p[q]);
    if (c < n_real) lp[(size_t)c * K + j] = __logf(inertia * oldp + (f[q] + cat_pc + missing_flow * oldp) * scale);
  }
}

// Sampling noise comes indexed by the caller's tree nodes; where nodes were split, the kernels' nodes include the
// auxiliary ones: dst[b][n][:] = src[b][user_index[n]][:], zero for an auxiliary node (whose identity block leaves no
// choice to the noise).
__global__ void hclt_expand_noise_kernel(const float4* __restrict__ src, const int32_t* __restrict__ user_index, int n_inner,
                                         int n_user, int K4, int64_t total, float4* __restrict__ dst) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int q = (int)(i % K4);
  const int64_t r = i / K4;
  const int n = (int)(r % n_inner);
  const int64_t b = r / n_inner;
  const int u = user_index[n];
  dst[i] = u >= 0 ? src[(b * n_user + u) * K4 + q] : make_float4(0.f, 0.f, 0.f, 0.f);
}

// xn[node][example] = categories of the node's own variable (byte 0) and of its first three
// leaf children (bytes 1..3), so that a wave fetches all of them with one request.  A thread makes
// the words of four examples (Bp is a multiple of 16): one word of four categories in per variable,
// one request of four words out.
__global__ void hclt_pack_x_kernel(const HcltNode* __restrict__ nodes, const int32_t* __restrict__ child_leaf,
                                   const uint8_t* __restrict__ xb, int n_inner, int Bp,
                                   uint32_t* __restrict__ xn) {
  const int b = 4 * (blockIdx.x * blockDim.x + threadIdx.x);
  const int n = blockIdx.y;
  if (b >= Bp) return;
  const HcltNode nd = nodes[n];
  uint32_t in[4] = {*reinterpret_cast<const uint32_t*>(xb + (size_t)nd.var * Bp + b), 0u, 0u, 0u};
  for (int i = 0; i < nd.lc_cnt && i < 3; ++i)
    in[i + 1] = *reinterpret_cast<const uint32_t*>(xb + (size_t)child_leaf[nd.lc_off + i] * Bp + b);
  uint4 out;
  uint32_t* o = &out.x;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    o[e] = ((in[0] >> (8 * e)) & 0xffu) | ((in[1] >> (8 * e)) & 0xffu) << 8 | ((in[2] >> (8 * e)) & 0xffu) << 16 |
           ((in[3] >> (8 * e)) & 0xffu) << 24;
  *reinterpret_cast<uint4*>(xn + (size_t)n * Bp + b) = out;
}

}  // namespace pcm
