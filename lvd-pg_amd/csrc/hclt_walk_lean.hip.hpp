// Lean tree-walk kernels: the same slice-persistent forward / backward walks as in
// hclt_kernels.hip.hpp, for the common case (no tile ever leaves LDS, at most three children
// per tree node, every array below 4 GiB), written for the fewest instructions per step.
//
// Why a second pair of kernels.  With one 16-example tile per wave and step, a step is only
// ~100 useful vector instructions (8 exp, 8 log, 16 MFMA, a few adds), and four waves share a
// SIMD: measured on gfx950 the general walk kernels are bound by instruction issue, not by
// memory -- their schedule decoding and 64-bit address arithmetic cost more instructions
// than the arithmetic.  Here
//   * every array is addressed through ONE buffer descriptor built before the loop; a node's
//     byte offset comes precomputed from the schedule and goes into the instruction's scalar
//     offset, the lane part is a per-thread constant, the tile row an immediate;
//   * operands are typed by position (own leaf row, own value tile, up to three children), so
//     an absent operand is a scalar branch around its loads and its adds -- nothing is
//     zero-filled, selected or copied;
//   * the parameter block is requested right after the contraction that used its
//     predecessor, into the same registers, so nothing rotates between steps.
// Idle waves work on a trash tile (row n_inner of the value arrays) and the trash LDS slot.
#pragma once

#include "hclt_kernels.hip.hpp"

namespace pcm {

// Field rows of a lean schedule, [field][wave][stride] like the general one.
//   kLW     byte offset of the node's parameter block
//   kLA0    byte offset of the node's own leaf rows (variable * leaf_stride)
//   kLA1..3 forward: leaf children's rows (-1: none; their categories are bytes 1..3 of the
//           packed word).  backward: children, -1: none, leaf child: row offset | 1 | category
//           byte << 1, inner child: node index << 3 (its value tile)
//   kLNode  node index (value / flow tile, packed-category row); idle waves: n_inner, the
//           trash tile (its category row is out of range and reads as zero)
//   kLSlots forward: out slot | child slots << 8, 16, 24 (0xff: none); backward: out slot |
//           slot of the parent's flow tile << 8
//   kLFlags bit 0: root
enum { kLW = 0, kLA0, kLA1, kLA2, kLA3, kLNode, kLSlots, kLFlags, kLeanFields };

constexpr int kLeanChunk = 62;   // steps per refill: 64 lanes minus two steps of look-ahead

struct LeanChunk {
  int v[kLeanFields];
  int base;
};

__device__ __forceinline__ void lean_refill(const int32_t* __restrict__ fields, int stride, int wave, int lane, int base,
                                            LeanChunk& c) {
#pragma unroll
  for (int f = 0; f < kLeanFields; ++f) c.v[f] = fields[((size_t)f * kWalkWaves + wave) * stride + base + lane];
  // the rows are used as landed from here on: no step waits for them (a step's own waits
  // then count only the requests of the steps)
#pragma unroll
  for (int f = 0; f < kLeanFields; ++f) asm volatile("" : "+v"(c.v[f]));
  c.base = base;
}

__device__ __forceinline__ int lean_get(const LeanChunk& c, int field, int step) {
  return __builtin_amdgcn_readlane(c.v[field], step - c.base);
}

template <int K>
__device__ __forceinline__ void lean_row_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, int soff, Tile<K>& t) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    t.v[kt] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(voff + kt * 64), soff, 0));
}

template <int K>
__device__ __forceinline__ void lean_tile_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, int soff, Tile<K>& t) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    t.v[kt] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(voff + kt * 1024), soff, 0));
}

template <int K>
__device__ __forceinline__ void lean_tile_store(__amdgpu_buffer_rsrc_t r, uint32_t voff, int soff, const Tile<K>& t) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, t.v[kt]), r, (int)(voff + kt * 1024), soff, kStreamStore);
}

template <int K>
__device__ __forceinline__ void lean_w_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, int soff, WTile<K>& w) {
#pragma unroll
  for (int i = 0; i < (K / 16) * (K / 16); ++i)
    w.a[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(voff + (i & 3) * 1024), soff + (i >> 2) * 4096, 0));
}

// byte offset of this lane's part of leaf row x (byte `sel` of the packed word)
template <int K>
__device__ __forceinline__ uint32_t lean_row_off(uint32_t xpack, int sel, uint32_t vleaf) {
  return ((xpack >> (8 * sel)) & 0xffu) * (K * 4) + vleaf;
}

__device__ __forceinline__ void lean_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- forward ------------------------------------------------------------------------------
template <int K>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_forward_lean_kernel(
    HcltDev d, const int32_t* __restrict__ fields, int stride, int n_steps, float* __restrict__ ll_out) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  const uint32_t vtile = (uint32_t)lane * 16, vleaf = (uint32_t)(lane >> 4) * 16, vx = (uint32_t)(lane & 15) * 4;
  const int bcol = slice * kSlice + (lane & 15);
  const uint32_t slice_bytes = (uint32_t)slice * (kSlice * K * 4);
  const __amdgpu_buffer_rsrc_t rO =
      make_rsrc(reinterpret_cast<const char*>(d.O) + slice_bytes, (uint32_t)(d.n_inner + 1) * d.tile_stride - slice_bytes);
  const __amdgpu_buffer_rsrc_t rW = make_rsrc(d.Wf, (uint32_t)d.n_inner * (K * K * 4));
  const __amdgpu_buffer_rsrc_t rL = make_rsrc(d.leaf, (uint32_t)d.V * d.leaf_stride);
  const __amdgpu_buffer_rsrc_t rX =
      make_rsrc(d.xn + (size_t)slice * kSlice, (uint32_t)d.n_inner * (uint32_t)d.Bp * 4u - (uint32_t)slice * (kSlice * 4));
  const int xrow = d.Bp * 4;

  LeanChunk sc;
  lean_refill(fields, stride, wave, lane, 0, sc);
  Tile<K> P0, P1, P2, P3;
  WTile<K> wA, wB;   // parameter blocks of the even / odd steps
  uint32_t xs;
  int a1, a2, a3;   // leaf children of the step whose operands are in flight
  {
    const uint32_t x0 = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, 0) * xrow, 0);
    xs = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, 1) * xrow, 0);
    lean_row_load<K>(rL, lean_row_off<K>(x0, 0, vleaf), lean_get(sc, kLA0, 0), P0);
    a1 = lean_get(sc, kLA1, 0); a2 = lean_get(sc, kLA2, 0); a3 = lean_get(sc, kLA3, 0);
    if (a1 >= 0) lean_row_load<K>(rL, lean_row_off<K>(x0, 1, vleaf), a1, P1);
    if (a2 >= 0) lean_row_load<K>(rL, lean_row_off<K>(x0, 2, vleaf), a2, P2);
    if (a3 >= 0) lean_row_load<K>(rL, lean_row_off<K>(x0, 3, vleaf), a3, P3);
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, 0), wA);
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, 1), wB);
  }
  float ll = 0.f;
  Tile<K> o_prev;   // the value tile of the previous step, stored at the top of the next one
  tile_zero<K>(o_prev);
  int store_prev = d.n_inner * (int)d.tile_stride;

  // the schedule is consumed in chunks of kLeanChunk steps (a chunk's registers also serve
  // the two steps of look-ahead past its end)
  auto step = [&](const int s, WTile<K>& w) {
    // (1) the static operands of this step have landed
    Tile<K> z = P0;
    if (a1 >= 0) tile_add<K>(z, P1);
    if (a2 >= 0) tile_add<K>(z, P2);
    if (a3 >= 0) tile_add<K>(z, P3);
    // the previous step's value tile goes out now
    lean_tile_store<K>(rO, vtile, store_prev, o_prev);
    // (2) request the leaf rows of step s+1 and the categories of step s+2
    {
      // (the categories first: everything that later waits for a leaf row then covers them)
      const uint32_t xc = xs;
      xs = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, s + 2) * xrow, 0);
      lean_row_load<K>(rL, lean_row_off<K>(xc, 0, vleaf), lean_get(sc, kLA0, s + 1), P0);
      a1 = lean_get(sc, kLA1, s + 1); a2 = lean_get(sc, kLA2, s + 1); a3 = lean_get(sc, kLA3, s + 1);
      if (a1 >= 0) lean_row_load<K>(rL, lean_row_off<K>(xc, 1, vleaf), a1, P1);
      if (a2 >= 0) lean_row_load<K>(rL, lean_row_off<K>(xc, 2, vleaf), a2, P2);
      if (a3 >= 0) lean_row_load<K>(rL, lean_row_off<K>(xc, 3, vleaf), a3, P3);
    }
    // (3) children from LDS, logsumexp through the matrix cores
    const uint32_t slots = (uint32_t)lean_get(sc, kLSlots, s);
#pragma unroll
    for (int c = 1; c <= 3; ++c) {
      const uint32_t sl = (slots >> (8 * c)) & 0xffu;
      if (sl != 0xffu) {
        Tile<K> t;
        lds_tile_load<K>(lds, (int)sl, lane, t);
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
      for (int i = 0; i < 4; ++i) o.v[kt][i] = fmaf(__builtin_amdgcn_logf(o.v[kt][i]), kLn2, m);
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, s + 2), w);   // the block of step s+2, same registers
    o_prev = o;
    store_prev = lean_get(sc, kLNode, s) * (int)d.tile_stride;
    lds_tile_store<K>(lds, (int)(slots & 0xffu), lane, o);
    if (lean_get(sc, kLFlags, s) & 1) ll = o.v[0][0];
    lean_barrier();
  };
  // The schedule is consumed in chunks of kLeanChunk steps (a chunk's registers also serve the
  // two steps of look-ahead past its end), two steps per trip: the parameter blocks alternate
  // between two register sets, each reloaded two steps ahead right after its use.  An odd
  // step count runs one idle step of the padding.
  for (int base = 0; base < n_steps; base += kLeanChunk) {
    if (base) lean_refill(fields, stride, wave, lane, base, sc);
    const int s_end = min(base + kLeanChunk, n_steps);
    for (int s = base; s < s_end; s += 2) {
      step(s, wA);
      step(s + 1, wB);
    }
  }
  lean_tile_store<K>(rO, vtile, store_prev, o_prev);
  if (ll_out && wave == 0 && lane < 16 && bcol < d.B) ll_out[bcol] = ll;   // the root is item 0 of the last step
}

// ---- backward -----------------------------------------------------------------------------
// kHeads: multi-head circuit, whose head kernel has left the root's ratio tile in memory (a
// build of its own: the extra load in the root branch costs the single-head walk 5%).
template <int K, bool kHeads>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_backward_lean_kernel(
    HcltDev d, const int32_t* __restrict__ fields, int stride, int n_steps) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  const uint32_t vtile = (uint32_t)lane * 16, vleaf = (uint32_t)(lane >> 4) * 16, vx = (uint32_t)(lane & 15) * 4;
  const int bcol = slice * kSlice + (lane & 15);
  const uint32_t slice_bytes = (uint32_t)slice * (kSlice * K * 4);
  const uint32_t arr_bytes = (uint32_t)(d.n_inner + 1) * d.tile_stride - slice_bytes;
  const __amdgpu_buffer_rsrc_t rO = make_rsrc(reinterpret_cast<const char*>(d.O) + slice_bytes, arr_bytes);
  const __amdgpu_buffer_rsrc_t rR = make_rsrc(reinterpret_cast<const char*>(d.R) + slice_bytes, arr_bytes);
  const __amdgpu_buffer_rsrc_t rW = make_rsrc(d.Wb, (uint32_t)d.n_inner * (K * K * 4));
  const __amdgpu_buffer_rsrc_t rL = make_rsrc(d.leaf, (uint32_t)d.V * d.leaf_stride);
  const __amdgpu_buffer_rsrc_t rX =
      make_rsrc(d.xn + (size_t)slice * kSlice, (uint32_t)d.n_inner * (uint32_t)d.Bp * 4u - (uint32_t)slice * (kSlice * 4));
  const int xrow = d.Bp * 4;

  // a child operand: value tile of an inner child, or leaf row of a leaf child
  auto child_load = [&](int c, uint32_t xpack, Tile<K>& t) {
    if (c & 1) lean_row_load<K>(rL, lean_row_off<K>(xpack, (c >> 1) & 3, vleaf), c & ~7, t);
    else lean_tile_load<K>(rO, vtile, (c >> 3) * (int)d.tile_stride, t);
  };

  LeanChunk sc;
  lean_refill(fields, stride, wave, lane, 0, sc);
  Tile<K> P0, OV, C1, C2, C3;
  WTile<K> wA, wB;
  uint32_t xs;
  int c1, c2, c3;
  {
    const uint32_t x0 = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, 0) * xrow, 0);
    xs = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, 1) * xrow, 0);
    lean_row_load<K>(rL, lean_row_off<K>(x0, 0, vleaf), lean_get(sc, kLA0, 0), P0);
    lean_tile_load<K>(rO, vtile, lean_get(sc, kLNode, 0) * (int)d.tile_stride, OV);
    c1 = lean_get(sc, kLA1, 0); c2 = lean_get(sc, kLA2, 0); c3 = lean_get(sc, kLA3, 0);
    if (c1 >= 0) child_load(c1, x0, C1);
    if (c2 >= 0) child_load(c2, x0, C2);
    if (c3 >= 0) child_load(c3, x0, C3);
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, 0), wA);
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, 1), wB);
  }

  auto step = [&](const int s, WTile<K>& w) {
    // (1) E_v (unnormalised) and the factor 1/S_v = exp(m - O_v) from the landed operands
    Tile<K> e = P0;
    if (c1 >= 0) tile_add<K>(e, C1);
    if (c2 >= 0) tile_add<K>(e, C2);
    if (c3 >= 0) tile_add<K>(e, C3);
    const float m = tile_rowmax<K>(e);
    Tile<K> sinv;
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i)   // capped: a state (or a whole example) of probability zero has flow 0, not 0 * inf
        sinv.v[kt][i] = fminf(__builtin_amdgcn_exp2f(fmaf(OV.v[kt][i], -kLog2e, m * kLog2e)), kFlowRatioCap);
    // (2) request the operands of step s+1 and the categories of step s+2
    {
      const uint32_t xc = xs;
      xs = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, s + 2) * xrow, 0);
      lean_row_load<K>(rL, lean_row_off<K>(xc, 0, vleaf), lean_get(sc, kLA0, s + 1), P0);
      lean_tile_load<K>(rO, vtile, lean_get(sc, kLNode, s + 1) * (int)d.tile_stride, OV);
      c1 = lean_get(sc, kLA1, s + 1); c2 = lean_get(sc, kLA2, s + 1); c3 = lean_get(sc, kLA3, s + 1);
      if (c1 >= 0) child_load(c1, xc, C1);
      if (c2 >= 0) child_load(c2, xc, C2);
      if (c3 >= 0) child_load(c3, xc, C3);
    }
    // (3) R_v = F_v / S_v, G_v = E_v .* (R_v W_v)
    tile_exp_sub<K>(e, m);
    const uint32_t slots = (uint32_t)lean_get(sc, kLSlots, s);
    Tile<K> r, t;
    lds_tile_load<K>(lds, (int)((slots >> 8) & 0xffu), lane, r);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt) r.v[kt] *= sinv.v[kt];
    const int fl = lean_get(sc, kLFlags, s);
    if (kHeads && (fl & 2)) {   // multi-head circuit: the head kernel has left the root's ratio tile in memory
      lean_tile_load<K>(rR, vtile, lean_get(sc, kLNode, s) * (int)d.tile_stride, r);
    } else if (fl & 1) {   // flow 1 into the single root sum node of every live example
      const float r00 = (lane < 16 && bcol < d.B) ? sinv.v[0][0] : 0.f;
      tile_zero<K>(r);
      r.v[0][0] = r00;
    }
    lean_tile_store<K>(rR, vtile, lean_get(sc, kLNode, s) * (int)d.tile_stride, r);
    contract<K>(w, r, t);
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, s + 2), w);
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt) t.v[kt] *= e.v[kt];
    lds_tile_store<K>(lds, (int)(slots & 0xffu), lane, t);
    lean_barrier();
  };
  for (int base = 0; base < n_steps; base += kLeanChunk) {
    if (base) lean_refill(fields, stride, wave, lane, base, sc);
    const int s_end = min(base + kLeanChunk, n_steps);
    for (int s = base; s < s_end; s += 2) {
      step(s, wA);
      step(s + 1, wB);
    }
  }
}

// ---- statistics -----------------------------------------------------------------------------
// Same job as hclt_stats_kernel (one workgroup per tree node, all slices; edge flows summed
// over the batch with the matrix cores, leaf histograms with integer LDS atomics), for nodes
// with at most three children, written like the lean walks: per-operand descriptors built once
// (the node is fixed, only the slice moves), typed operands behind scalar branches, every
// register reloaded right after its last use, the waves' partial edge-flow blocks combined by
// a plain LDS sum.  A node with leaf children runs one pass over the batch per variable it has
// to histogram (the LDS holds one histogram): pass 0 does all the arithmetic and leaves the
// child-flow tiles G where it read R from; the passes of the leaf children re-read G only.
constexpr int kStatLeanWaves = 16;

template <int K>
__global__ __launch_bounds__(kStatLeanWaves * 64) void hclt_stats_lean_kernel(
    HcltDev d, const StatNode* __restrict__ nodes, float* __restrict__ edge_aggr, float* __restrict__ leaf_flow,
    float rate, int hist_words, int limb, const int* __restrict__ flow_shift) {
  constexpr int KT = K / 16;
  constexpr int LD = K + 16;   // row stride of the pad: conflict-free column reads
  constexpr int HS = K + 1;    // row stride of a histogram: spreads equal states over banks
  extern __shared__ float smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = lane & 15, g = lane >> 4;
  const int n = blockIdx.x;
  const StatNode* __restrict__ np = nodes + n;   // fields are read where needed (a local copy indexed by the pass would live in scratch)
  const int own_var = np->var, n_hist = np->n_hist;
  const uint32_t vtile = (uint32_t)lane * 16, vleaf = (uint32_t)g * 16, vx = (uint32_t)b * 4;
  const int hist_sz = d.C * HS;
  unsigned* hist = reinterpret_cast<unsigned*>(smem);
  float* pad = smem + hist_words + (size_t)wave * (kSlice * LD);
  // flows lie in [0, 2^shift]: 1 per example in a single-head circuit, the largest total head
  // mask of an example (found on the device by the head kernel) in a multi-head one
  const int shift = flow_shift ? __builtin_amdgcn_readfirstlane(*flow_shift) : 0;
  const float scale = __builtin_ldexpf(1.f, limb), scale_in = __builtin_ldexpf(1.f, limb - shift);

  const __amdgpu_buffer_rsrc_t rR = make_rsrc(reinterpret_cast<const char*>(d.R) + (size_t)n * d.tile_stride, d.tile_stride);
  const __amdgpu_buffer_rsrc_t rX = make_rsrc(d.xn + (size_t)n * d.Bp, (uint32_t)d.Bp * 4u);
  const __amdgpu_buffer_rsrc_t rL0 = make_rsrc(reinterpret_cast<const char*>(d.leaf) + (size_t)own_var * d.leaf_stride, d.leaf_stride);
  auto child_rsrc = [&](int c) {
    return (c & 1) ? make_rsrc(reinterpret_cast<const char*>(d.leaf) + (size_t)(c >> 3) * d.leaf_stride, d.leaf_stride)
                   : make_rsrc(reinterpret_cast<const char*>(d.O) + (size_t)(max(c, 0) >> 3) * d.tile_stride, d.tile_stride);
  };
  const int c1 = np->c[0], c2 = np->c[1], c3 = np->c[2];
  const __amdgpu_buffer_rsrc_t rC1 = child_rsrc(c1), rC2 = child_rsrc(c2), rC3 = child_rsrc(c3);
  auto child_load = [&](__amdgpu_buffer_rsrc_t r, int c, uint32_t xpack, uint32_t slice_off, Tile<K>& t) {
    if (c & 1) lean_row_load<K>(r, lean_row_off<K>(xpack, (c >> 1) & 3, vleaf), 0, t);
    else lean_tile_load<K>(r, vtile, (int)slice_off, t);
  };

  WTile<K> w;
  lean_w_load<K>(make_rsrc(d.Wb + (size_t)n * K * K, K * K * 4u), vtile, 0, w);
  v4f accA[KT][KT];
#pragma unroll
  for (int a = 0; a < KT; ++a)
#pragma unroll
    for (int c = 0; c < KT; ++c) accA[a][c] = v4f{0.f, 0.f, 0.f, 0.f};

  // fixed-point limbs of this lane's K/4 flows (clamped to [0, 2^shift]) into row x of the histogram
  auto histogram = [&](const Tile<K>& t, uint32_t xpack, int sel) {
    const uint32_t x = (xpack >> (8 * sel)) & 0xffu;
    unsigned* hrow = hist + x * HS + 4 * g;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = __builtin_amdgcn_fmed3f(t.v[kt][i] * scale_in, 0.f, scale);
        const unsigned hi = (unsigned)v;
        const unsigned lo = (unsigned)(__builtin_amdgcn_fractf(v) * scale);
        __hip_atomic_fetch_add(&hrow[kt * 16 + i], hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_fetch_add(&hrow[hist_sz + kt * 16 + i], lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
  };

  const int last = d.nslices - 1;
  for (int pass = 0; pass < n_hist; ++pass) {
    for (int i = threadIdx.x; i < 2 * hist_sz; i += blockDim.x) hist[i] = 0u;
    __syncthreads();
    if (pass == 0) {
    // prologue: operands of the wave's first slice (slices past the end are clamped: harmless
    // repeated loads), categories of the second
    Tile<K> P0, R, C1, C2;   // (a third child is rare: it is fetched at the point of use)
    uint32_t xc, xn;
    {
      const int sa = min(wave, last), sb = min(wave + kStatLeanWaves, last);
      xc = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, sa * (kSlice * 4), 0);
      xn = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, sb * (kSlice * 4), 0);
      const uint32_t so = (uint32_t)sa * (kSlice * K * 4);
      lean_row_load<K>(rL0, lean_row_off<K>(xc, 0, vleaf), 0, P0);
      if (c1 >= 0) child_load(rC1, c1, xc, so, C1);
      if (c2 >= 0) child_load(rC2, c2, xc, so, C2);
      lean_tile_load<K>(rR, vtile, (int)so, R);
    }
    for (int s0 = wave; s0 < d.nslices; s0 += kStatLeanWaves) {
      const int s1 = min(s0 + kStatLeanWaves, last), s2 = min(s0 + 2 * kStatLeanWaves, last);
      const uint32_t so1 = (uint32_t)s1 * (kSlice * K * 4);
      // (1) E (unnormalised) from the landed operands; request the next slice's
      Tile<K> e = P0;
      if (c1 >= 0) tile_add<K>(e, C1);
      if (c2 >= 0) tile_add<K>(e, C2);
      const uint32_t xh = xc;   // categories of the slice computed now
      if (c3 >= 0) {
        Tile<K> t3;
        child_load(rC3, c3, xh, (uint32_t)s0 * (kSlice * K * 4), t3);
        tile_add<K>(e, t3);
      }
      xc = xn;
      xn = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, s2 * (kSlice * 4), 0);
      lean_row_load<K>(rL0, lean_row_off<K>(xc, 0, vleaf), 0, P0);
      if (c1 >= 0) child_load(rC1, c1, xc, so1, C1);
      if (c2 >= 0) child_load(rC2, c2, xc, so1, C2);
      // (2) E, the edge flows, then G = E .* (R W)
      const float m = tile_rowmax<K>(e);
      tile_exp_sub<K>(e, m);
      {
        // A += R^T E over the 16 examples of the tile (contraction over examples): both operands
        // go through the wave's pad to reach the [state][example] operand layout.  A wave's LDS
        // accesses execute in order, so the pad needs no barrier between its phases.
        float ra[4][KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<v4f*>(&pad[b * LD + kt * 16 + 4 * g]) = R.v[kt];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) ra[q][kt] = pad[(4 * q + g) * LD + kt * 16 + b];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<v4f*>(&pad[b * LD + kt * 16 + 4 * g]) = e.v[kt];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float eb[KT];
#pragma unroll
          for (int jt = 0; jt < KT; ++jt) eb[jt] = pad[(4 * q + g) * LD + jt * 16 + b];
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int jt = 0; jt < KT; ++jt)
              accA[kt][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[q][kt], eb[jt], accA[kt][jt], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      }
      Tile<K> t;
      contract<K>(w, R, t);
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) t.v[kt] *= e.v[kt];
      lean_tile_load<K>(rR, vtile, (int)so1, R);   // next slice's ratios, after the last use of these
      if (n_hist > 1) {
        // the later passes (one per leaf child) only need G: it replaces the tile of R just consumed
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, t.v[kt]), rR, (int)(vtile + kt * 1024),
                                                 (int)((uint32_t)s0 * (kSlice * K * 4)), 0);
      }
      // (3) histogram
      if (s0 * kSlice + b < d.B) histogram(t, xh, 0);
    }
    } else {
      // leaf child `pass`: G comes back from where pass 0 left it; only the categories differ
      Tile<K> T;
      uint32_t xc, xn;
      {
        const int sa = min(wave, last), sb = min(wave + kStatLeanWaves, last);
        xc = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, sa * (kSlice * 4), 0);
        xn = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, sb * (kSlice * 4), 0);
        lean_tile_load<K>(rR, vtile, (int)((uint32_t)sa * (kSlice * K * 4)), T);
      }
      for (int s0 = wave; s0 < d.nslices; s0 += kStatLeanWaves) {
        const int s1 = min(s0 + kStatLeanWaves, last), s2 = min(s0 + 2 * kStatLeanWaves, last);
        const uint32_t xh = xc;
        xc = xn;
        xn = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, s2 * (kSlice * 4), 0);
        if (s0 * kSlice + b < d.B) histogram(T, xh, pass);
        lean_tile_load<K>(rR, vtile, (int)((uint32_t)s1 * (kSlice * K * 4)), T);
      }
    }
    __syncthreads();
    {
      const float hi_inv = __builtin_ldexpf(1.f, shift - limb), lo_inv = __builtin_ldexpf(1.f, shift - 2 * limb);
      float* dst = leaf_flow + (size_t)np->hvar[pass] * d.C * K;
      for (int i = threadIdx.x; i < d.C * K; i += blockDim.x) {
        const int c = i / K, j = i % K;
        const float val = (float)hist[c * HS + j] * hi_inv + (float)hist[hist_sz + c * HS + j] * lo_inv;
        const float old = rate != 0.f ? rate * dst[i] : 0.f;
        dst[i] = old + val;
      }
    }
    __syncthreads();
  }

  // combine the waves' partial blocks: every wave parks its accumulators in LDS (the histogram
  // area is free now), then each thread adds up the waves' copies of its elements
  v4f* park = reinterpret_cast<v4f*>(smem);
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int jt = 0; jt < KT; ++jt) park[((size_t)wave * KT * KT + kt * KT + jt) * 64 + lane] = accA[kt][jt];
  __syncthreads();
  float* dst = edge_aggr + (size_t)n * K * K;
  const float* lt = d.logtheta + (size_t)n * K * K;
  for (int q = threadIdx.x; q < KT * KT * 64; q += blockDim.x) {
    v4f sum = park[q];
    for (int wv = 1; wv < kStatLeanWaves; ++wv) sum += park[(size_t)wv * KT * KT * 64 + q];
    const int kt = q / (KT * 64), jt = (q / 64) % KT, l = q % 64;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int idx = (kt * 16 + 4 * (l >> 4) + v) * K + jt * 16 + (l & 15);
      const float old = rate != 0.f ? rate * dst[idx] : 0.f;
      dst[idx] = old + __expf(lt[idx]) * sum[v];
    }
  }
}

}  // namespace pcm
