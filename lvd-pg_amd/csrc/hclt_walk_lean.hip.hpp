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
//           packed word).  backward: children, inner ones first, -1: none, leaf child: row
//           offset | 1 | category byte << 1, inner child: node index << 3 (its value tile)
//   kLNode  node index (value / flow tile, packed-category row, row of maxima); idle waves:
//           n_inner, the trash tile (its category row is out of range and reads as zero)
//   kLSlots forward: out slot | child slots << 8, 16, 24 (0xff: none); backward: slot holding
//           this node's ratio tile | slots of the inner children's ratio tiles << 8, 16, 24
//           (0xff: that child is a leaf or absent)
//   kLFlags bit 0: root; bit 1: root of a multi-head circuit
//   kLTurns which use of its slot a tile is, modulo 128, in the byte layout of kLSlots: a slot passes through
//           the states 2t (free for its t-th tile), 2t + 1 (that tile is there), 2t + 2 (read, free again)
enum { kLW = 0, kLA0, kLA1, kLA2, kLA3, kLNode, kLSlots, kLFlags, kLTurns, kLeanFields };
constexpr int kLeanFlagWords = 256;        // one state word per LDS slot, behind the slots
constexpr int kLeanSpinLimit = 1 << 22;    // polls before a wave gives up on a tile (never reached by a sound schedule)

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
    t.v[kt] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(voff + kt * 1024), soff, kStreamLoad));
}

#ifndef PCM_ST_O
#define PCM_ST_O kStreamStore
#endif
#ifndef PCM_ST_R
#define PCM_ST_R kStreamStore
#endif
template <int K, int kAux = kStreamStore>
__device__ __forceinline__ void lean_tile_store(__amdgpu_buffer_rsrc_t r, uint32_t voff, int soff, const Tile<K>& t) {
#pragma unroll
  for (int kt = 0; kt < K / 16; ++kt)
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, t.v[kt]), r, (int)(voff + kt * 1024), soff, kAux);
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

// Waits until the slot's state word reads `want`.  The walks have no barrier between steps: a wave goes on as
// soon as the tiles it needs are there, and hands its own tile on by advancing the slot's state.  Every wait is
// for a tile of an earlier step of the host's schedule, and every wave works through its steps in order, so the
// earliest unfinished step can always proceed.  The wait is bounded all the same: a wave that runs out of polls
// raises *err and carries on, so the kernel ends whatever the schedule holds.
__device__ __forceinline__ void lean_wait(const unsigned* state, unsigned want, const HcltDev& d) {
  int polls = 0;
  while (__builtin_amdgcn_readfirstlane(
             (int)__hip_atomic_load(state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) != (int)want) {
    if (++polls > kLeanSpinLimit) {
      if ((threadIdx.x & 63) == 0) {
        __hip_atomic_store(d.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(d.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Advances a slot's state once everything this wave did to the slot's tile before is in LDS order (a wave's
// LDS accesses execute in the order they were issued; the fence keeps the compiler to that order too).
__device__ __forceinline__ void lean_post(unsigned* state, unsigned value) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __hip_atomic_store(state, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// ---- forward ------------------------------------------------------------------------------
// A node's value is kept in two parts: the tile holds O'_v[k] = log S_v[k] = log sum_j W[k,j] exp(Z'_v[j] - m_v), numbers
// of order one, and the row of maxima holds m_v = max_j Z'_v[j], where Z'_v is the sum of the node's leaf rows and of its
// inner children's TILES (not of their full values).  The full value is O'_v[k] plus the maxima of all nodes of the
// subtree, a number that grows with the size of the subtree and is the same for all K states: nothing below needs it
// but the log-likelihood at the root.  Stored as one float32 it would cost every state of a 3000-variable circuit
// (values near -14000) an absolute error of 1e-3, which is a relative error of 1e-3 on every flow; in two parts the
// flows keep float32's relative accuracy at any depth.
template <int K>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_forward_lean_kernel(
    HcltDev d, const int32_t* __restrict__ fields, int stride, int n_steps, float* __restrict__ ll_out, int n_slots) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  unsigned* state = reinterpret_cast<unsigned*>(lds + (size_t)n_slots * (kSlice * K));
  for (int i = threadIdx.x; i < kLeanFlagWords; i += blockDim.x) state[i] = 0u;
  __syncthreads();
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
  // the row maxima M[node][example] go out beside the value tiles: the backward walk and the statistics
  // kernel scale by exactly these numbers (lanes 16..63 hold copies: their stores fall outside the buffer)
  const __amdgpu_buffer_rsrc_t rM =
      make_rsrc(d.M + (size_t)slice * kSlice, (uint32_t)(d.n_inner + 1) * (uint32_t)d.Bp * 4u - (uint32_t)slice * (kSlice * 4));
  const uint32_t vm = lane < 16 ? vx : 0x7ffffff0u;

  fields += (size_t)blockIdx.y * (kLeanFields * kWalkWaves) * stride;   // a forest's groups of trees: a schedule each
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
  double msum = 0.0;   // sum of the row maxima of this wave's nodes: the part of the log-likelihood the tiles leave out
  Tile<K> o_prev;   // the value tile of the previous step, stored at the top of the next one
  tile_zero<K>(o_prev);
  int store_prev = d.n_inner * (int)d.tile_stride;
  float m_prev = 0.f;
  int mrow_prev = d.n_inner * xrow;

  // the schedule is consumed in chunks of kLeanChunk steps (a chunk's registers also serve
  // the two steps of look-ahead past its end)
  auto step = [&](const int s, WTile<K>& w) {
    // (1) the static operands of this step have landed
    Tile<K> z = P0;
    if (a1 >= 0) tile_add<K>(z, P1);
    if (a2 >= 0) tile_add<K>(z, P2);
    if (a3 >= 0) tile_add<K>(z, P3);
    // the previous step's value tile goes out now
    lean_tile_store<K, PCM_ST_O>(rO, vtile, store_prev, o_prev);
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, m_prev), rM, (int)vm, mrow_prev, kStreamStore);
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
    const uint32_t slots = (uint32_t)lean_get(sc, kLSlots, s), turns = (uint32_t)lean_get(sc, kLTurns, s);
#pragma unroll
    for (int c = 1; c <= 3; ++c) {
      const uint32_t sl = (slots >> (8 * c)) & 0xffu, tn = (turns >> (8 * c)) & 0x7fu;
      if (sl != 0xffu) {
        lean_wait(state + sl, (2 * tn + 1) & 0xffu, d);
        Tile<K> t;
        lds_tile_load<K>(lds, (int)sl, lane, t);
        tile_add<K>(z, t);
        lean_post(state + sl, (2 * tn + 2) & 0xffu);   // read: the slot may take its next tile
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
    lean_w_load<K>(rW, vtile, lean_get(sc, kLW, s + 2), w);   // the block of step s+2, same registers
    o_prev = o;
    const int node = lean_get(sc, kLNode, s);
    store_prev = node * (int)d.tile_stride;
    m_prev = m;
    mrow_prev = node * xrow;
    if (node != d.n_inner) msum += (double)m;   // (idle steps work on the trash tile)
    {
      // idle steps and the root write the trash slot, which nobody reads: no hand-over there
      const uint32_t so = slots & 0xffu, tn = turns & 0x7fu;
      const bool handed = so != (uint32_t)(n_slots - 1);
      if (handed) lean_wait(state + so, (2 * tn) & 0xffu, d);
      lds_tile_store<K>(lds, (int)so, lane, o);
      if (handed) lean_post(state + so, (2 * tn + 1) & 0xffu);
    }
    if (lean_get(sc, kLFlags, s) & 1) ll = o.v[0][0];
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
  lean_tile_store<K, PCM_ST_O>(rO, vtile, store_prev, o_prev);
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, m_prev), rM, (int)vm, mrow_prev, kStreamStore);
  // log-likelihood of a single-root circuit: the root's (scaled) value plus the row maxima of all nodes, the
  // waves' sums added in wave order (a multi-head circuit's head kernel adds up the stored maxima per tree)
  if (!ll_out) return;
  __syncthreads();   // every wave is through its steps: the slots are free
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

// ---- backward -----------------------------------------------------------------------------
// What travels down the tree through LDS is not the flow of a child's sum nodes but already their
// ratio tile R_c = F_c / S_c, built by the parent: with t = W_v^T R_v, F_c = G_v = exp(Z'_v - m_v) .* t
// and S_c = exp(O'_c) (the tiles hold log S, see the forward walk),
//   R_c[j] = t[j] * exp((Z'_v[j] - O'_c[j]) - m_v),
// where Z'_v - O'_c is the sum of v's OTHER operands (own leaf row, leaf children, further inner
// children's tiles): the child's own values cancel, so a node never reads its own value tile, and the
// exponent is formed from small numbers.  m_v are the row maxima the forward walk stored.  A state the
// child gives probability zero (O'_c = -inf) has flow 0 and keeps ratio 0.  A node without inner children
// only stores its tile.
// kHeads: multi-head circuit, whose head kernel has left the root's ratio tile in memory.
template <int K, bool kHeads>
__global__ __launch_bounds__(kWalkWaves * 64) void hclt_backward_lean_kernel(
    HcltDev d, const int32_t* __restrict__ fields, int stride, int n_steps, int n_slots) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slice = blockIdx.x;
  unsigned* state = reinterpret_cast<unsigned*>(lds + (size_t)n_slots * (kSlice * K));
  for (int i = threadIdx.x; i < kLeanFlagWords; i += blockDim.x) state[i] = 0u;
  __syncthreads();
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
  const __amdgpu_buffer_rsrc_t rM =
      make_rsrc(d.M + (size_t)slice * kSlice, (uint32_t)(d.n_inner + 1) * (uint32_t)d.Bp * 4u - (uint32_t)slice * (kSlice * 4));
  const int xrow = d.Bp * 4;

  // a child operand: value tile of an inner child, or leaf row of a leaf child
  auto child_load = [&](int c, uint32_t xpack, Tile<K>& t) {
    if (c & 1) lean_row_load<K>(rL, lean_row_off<K>(xpack, (c >> 1) & 3, vleaf), c & ~7, t);
    else lean_tile_load<K>(rO, vtile, (c >> 3) * (int)d.tile_stride, t);
  };
  auto is_inner = [](int c) { return c >= 0 && !(c & 1); };

  fields += (size_t)blockIdx.y * (kLeanFields * kWalkWaves) * stride;   // a forest's groups of trees: a schedule each
  LeanChunk sc;
  lean_refill(fields, stride, wave, lane, 0, sc);
  Tile<K> P0, C1, C2, C3;
  WTile<K> wA, wB;
  uint32_t xs;
  int c1, c2, c3;
  float mv;
  {
    const uint32_t x0 = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, 0) * xrow, 0);
    xs = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, 1) * xrow, 0);
    mv = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rM, (int)vx, lean_get(sc, kLNode, 0) * xrow, 0));
    lean_row_load<K>(rL, lean_row_off<K>(x0, 0, vleaf), lean_get(sc, kLA0, 0), P0);
    c1 = lean_get(sc, kLA1, 0); c2 = lean_get(sc, kLA2, 0); c3 = lean_get(sc, kLA3, 0);
    if (c1 >= 0) child_load(c1, x0, C1);
    if (c2 >= 0) child_load(c2, x0, C2);
    if (c3 >= 0) child_load(c3, x0, C3);
    // (a node without inner children has no use for its parameter block)
    if (is_inner(c1)) lean_w_load<K>(rW, vtile, lean_get(sc, kLW, 0), wA);
    if (is_inner(lean_get(sc, kLA1, 1))) lean_w_load<K>(rW, vtile, lean_get(sc, kLW, 1), wB);
  }

  // exponent tile of inner child `own` among the landed operands: the other operands minus m_v,
  // in base-2 units; -inf where the child's own value is -inf
  auto exponent = [&](const Tile<K>& own, bool has_a, const Tile<K>& a, bool has_b, const Tile<K>& b, Tile<K>& x) {
    const float dm = -mv * kLog2e;
#pragma unroll
    for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float rest = P0.v[kt][i];
        if (has_a) rest += a.v[kt][i];
        if (has_b) rest += b.v[kt][i];
        x.v[kt][i] = own.v[kt][i] == -INFINITY ? -INFINITY : fmaf(rest, kLog2e, dm);
      }
  };

  auto step = [&](const int s, WTile<K>& w) {
    // (1) from the landed operands: the exponent tiles of the inner children (they come first).  The first
    // stays in registers; a second and third wait in the LDS slots their ratio tiles will take.
    const bool in1 = is_inner(c1), in2 = is_inner(c2), in3 = is_inner(c3);
    const uint32_t slots = (uint32_t)lean_get(sc, kLSlots, s), turns = (uint32_t)lean_get(sc, kLTurns, s);
    {   // the children's slots are this wave's from here (scratch first, their ratio tiles at the end)
      if (in1) lean_wait(state + ((slots >> 8) & 0xffu), (2 * ((turns >> 8) & 0x7fu)) & 0xffu, d);
      if (in2) lean_wait(state + ((slots >> 16) & 0xffu), (2 * ((turns >> 16) & 0x7fu)) & 0xffu, d);
      if (in3) lean_wait(state + ((slots >> 24) & 0xffu), (2 * ((turns >> 24) & 0x7fu)) & 0xffu, d);
    }
    Tile<K> X1;
    if (in1) exponent(C1, c2 >= 0, C2, c3 >= 0, C3, X1);
    if (in2) {
      Tile<K> x;
      exponent(C2, true, C1, c3 >= 0, C3, x);
      lds_tile_store<K>(lds, (int)((slots >> 16) & 0xffu), lane, x);
    }
    if (in3) {
      Tile<K> x;
      exponent(C3, true, C1, true, C2, x);
      lds_tile_store<K>(lds, (int)((slots >> 24) & 0xffu), lane, x);
    }
    // (2) request the operands of step s+1 and the categories of step s+2
    {
      const uint32_t xc = xs;
      xs = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, lean_get(sc, kLNode, s + 2) * xrow, 0);
      mv = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rM, (int)vx, lean_get(sc, kLNode, s + 1) * xrow, 0));
      lean_row_load<K>(rL, lean_row_off<K>(xc, 0, vleaf), lean_get(sc, kLA0, s + 1), P0);
      c1 = lean_get(sc, kLA1, s + 1); c2 = lean_get(sc, kLA2, s + 1); c3 = lean_get(sc, kLA3, s + 1);
      if (c1 >= 0) child_load(c1, xc, C1);
      if (c2 >= 0) child_load(c2, xc, C2);
      if (c3 >= 0) child_load(c3, xc, C3);
    }
    // (3) this node's ratio tile: left in LDS by the parent (the root and idle steps read the trash slot)
    Tile<K> r;
    const bool handed = (slots & 0xffu) != (uint32_t)(n_slots - 1);
    if (handed) lean_wait(state + (slots & 0xffu), (2 * (turns & 0x7fu) + 1) & 0xffu, d);
    lds_tile_load<K>(lds, (int)(slots & 0xffu), lane, r);
    if (handed) lean_post(state + (slots & 0xffu), (2 * (turns & 0x7fu) + 2) & 0xffu);
    const int fl = lean_get(sc, kLFlags, s);
    if (kHeads && (fl & 2)) {   // multi-head circuit: the head kernel has left the root's ratio tile in memory
      lean_tile_load<K>(rR, vtile, lean_get(sc, kLNode, s) * (int)d.tile_stride, r);
    } else if (fl & 1) {   // flow 1 into the single root sum node of every live example: R = 1 / S = exp(-O')
      const float o00 = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(rO, (int)vtile, lean_get(sc, kLNode, s) * (int)d.tile_stride, 0));
      const bool live = lane < 16 && bcol < d.B;
      const float wgt = (d.w && live) ? d.w[bcol] : 1.f;   // per-example weights: the flow the example starts with
      const float r00 = live ? wgt * fminf(__builtin_amdgcn_exp2f(o00 * -kLog2e), kFlowRatioCap) : 0.f;
      tile_zero<K>(r);
      r.v[0][0] = r00;
    }
    lean_tile_store<K, PCM_ST_R>(rR, vtile, lean_get(sc, kLNode, s) * (int)d.tile_stride, r);
    // (4) the inner children's ratio tiles
    if (in1) {
      Tile<K> t;
      contract<K>(w, r, t);
      auto emit = [&](const Tile<K>& x, uint32_t slot) {
        Tile<K> rc;
#pragma unroll
        for (int kt = 0; kt < K / 16; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) rc.v[kt][i] = t.v[kt][i] * fminf(__builtin_amdgcn_exp2f(x.v[kt][i]), kFlowRatioCap);
        lds_tile_store<K>(lds, (int)slot, lane, rc);
      };
      emit(X1, (slots >> 8) & 0xffu);
      if (in2) {
        Tile<K> x;
        lds_tile_load<K>(lds, (int)((slots >> 16) & 0xffu), lane, x);
        emit(x, (slots >> 16) & 0xffu);
      }
      if (in3) {
        Tile<K> x;
        lds_tile_load<K>(lds, (int)((slots >> 24) & 0xffu), lane, x);
        emit(x, (slots >> 24) & 0xffu);
      }
      {
        lean_post(state + ((slots >> 8) & 0xffu), (2 * ((turns >> 8) & 0x7fu) + 1) & 0xffu);
        if (in2) lean_post(state + ((slots >> 16) & 0xffu), (2 * ((turns >> 16) & 0x7fu) + 1) & 0xffu);
        if (in3) lean_post(state + ((slots >> 24) & 0xffu), (2 * ((turns >> 24) & 0x7fu) + 1) & 0xffu);
      }
    }
    if (is_inner(lean_get(sc, kLA1, s + 2))) lean_w_load<K>(rW, vtile, lean_get(sc, kLW, s + 2), w);
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
// Same job as hclt_stats_kernel (a workgroup takes a tree node over all slices; edge flows summed
// over the batch with the matrix cores, leaf histograms with integer LDS atomics), for nodes
// with at most three children, written like the lean walks: one descriptor per array, a node's
// byte offsets as scalars, typed operands behind scalar branches, every register reloaded right
// after its last use, the waves' partial edge-flow blocks combined by a plain LDS sum.  The LDS
// holds up to `nh_pass` histograms (two where they fit: a node's own variable and its first leaf
// child then need one pass over the batch).  Pass 0 does all the arithmetic; a node with more
// variables than that leaves the child-flow tiles G where it read R from, and further passes
// re-read G only.
//
// The workgroups are persistent: one per compute unit, each working through nodes it claims from a
// counter in memory (the first two by its index), and a wave's stream of slices runs on from one
// node into the next: in its last two slices of a node the requests it sends ahead are the first
// operands of the next node, so that they land while the histograms are written out and the
// partial blocks are combined.  A node that needs several passes, and a batch of fewer than
// 32 slices, ends the stream: the node after it starts with requests of its own.
//
// LDS layouts, both without padding so that two histograms of 256 x 32 cells and sixteen pads fill
// 160 KB exactly: histogram cell (category x, state j) sits in word x*K + (j ^ (x % K)) of its limb
// (equal states of different categories spread over the banks); a wave's 16 x K transposition pad
// rotates row r by 8*r floats (column reads of four rows then cover every bank twice).  The
// histogram area is all zero whenever a node begins: whoever reads a cell out clears it.
constexpr int kStatLeanWaves = 16;

// A node's scalars as the statistics kernel uses them.
struct StatRef {
  int node;          // the node's index
  int tile_off;      // byte offset of the node's tiles in the value and ratio arrays
  int x_off;         // ... of its row of packed categories (and of row maxima)
  int leaf_off;      // ... of its own variable's leaf table
  int w_off;         // ... of its parameter block
  int c1, c2, c3;    // children as in StatNode
  int n_hist;
};

__device__ __forceinline__ StatRef stat_ref(const HcltDev& d, const StatNode* __restrict__ nodes, int pos, int kk4) {
  const StatNode* __restrict__ np = nodes + pos;
  const int n = np->node;
  StatRef r;
  r.node = n;
  r.tile_off = n * (int)d.tile_stride;
  r.x_off = n * d.Bp * 4;
  r.leaf_off = np->var * (int)d.leaf_stride;
  r.w_off = n * kk4;
  r.c1 = np->c[0];
  r.c2 = np->c[1];
  r.c3 = np->c[2];
  r.n_hist = np->n_hist;
  return r;
}

// Next node of a workgroup (-1: none left).  Tickets count from the third node of every workgroup; each
// workgroup draws until its first miss, so a launch hands out n_nodes - gridDim.x tickets in all, and whoever
// draws the last one puts the counter back to zero for the next launch.
__device__ __forceinline__ int stat_claim(unsigned* counter, int n_nodes) {
  const unsigned t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (t + 1u == (unsigned)n_nodes - gridDim.x) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned n = 2u * gridDim.x + t;
  return n < (unsigned)n_nodes ? (int)n : -1;
}

template <int K>
__global__ __launch_bounds__(kStatLeanWaves * 64) void hclt_stats_lean_kernel(
    HcltDev d, const StatNode* __restrict__ nodes, float* __restrict__ edge_aggr, float* __restrict__ leaf_flow,
    float rate, int hist_words, int nh_pass, int limb, const int* __restrict__ flow_shift, unsigned* __restrict__ counter,
    int n_nodes) {
  constexpr int KT = K / 16;
  extern __shared__ float smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = lane & 15, g = lane >> 4;
  const uint32_t vtile = (uint32_t)lane * 16, vleaf = (uint32_t)g * 16, vx = (uint32_t)b * 4;
  const int hist_sz = d.C * K;           // words per limb; a histogram is two limbs
  unsigned* hist = reinterpret_cast<unsigned*>(smem);
  float* pad = smem + hist_words + (size_t)wave * (kSlice * K);
  int* claim_word = reinterpret_cast<int*>(smem + hist_words);   // wave 0's pad, which is idle between two nodes
  // flows lie in [0, 2^shift]: 1 per example in a single-head circuit, the largest total head
  // mask of an example (found on the device by the head kernel) in a multi-head one
  const int shift = flow_shift ? __builtin_amdgcn_readfirstlane(*flow_shift) : 0;
  const float scale = __builtin_ldexpf(1.f, limb), scale_in = __builtin_ldexpf(1.f, limb - shift);
  const float hi_inv = __builtin_ldexpf(1.f, shift - limb), lo_inv = __builtin_ldexpf(1.f, shift - 2 * limb);

  const uint32_t tiles_bytes = (uint32_t)(d.n_inner + 1) * d.tile_stride;
  const __amdgpu_buffer_rsrc_t rR = make_rsrc(d.R, tiles_bytes);
  const __amdgpu_buffer_rsrc_t rO = make_rsrc(d.O, tiles_bytes);
  const __amdgpu_buffer_rsrc_t rL = make_rsrc(d.leaf, (uint32_t)d.V * d.leaf_stride);
  const __amdgpu_buffer_rsrc_t rX = make_rsrc(d.xn, (uint32_t)d.n_inner * (uint32_t)d.Bp * 4u);
  const __amdgpu_buffer_rsrc_t rM = make_rsrc(d.M, (uint32_t)(d.n_inner + 1) * (uint32_t)d.Bp * 4u);   // row maxima of the forward walk
  const __amdgpu_buffer_rsrc_t rW = make_rsrc(d.Wb, (uint32_t)d.n_inner * (K * K * 4));
  auto child_load = [&](int c, uint32_t xpack, int slice_off, Tile<K>& t) {
    if (c & 1) lean_row_load<K>(rL, lean_row_off<K>(xpack, (c >> 1) & 3, vleaf), (c >> 3) * (int)d.leaf_stride, t);
    else lean_tile_load<K>(rO, vtile, (c >> 3) * (int)d.tile_stride + slice_off, t);
  };
  auto load_x = [&](const StatRef& r, int s) {
    return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, r.x_off + s * (kSlice * 4), 0);
  };
  auto load_m = [&](const StatRef& r, int s) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rM, (int)vx, r.x_off + s * (kSlice * 4), 0));
  };

  // fixed-point limbs of this lane's K/4 flows (clamped to [0, 2^shift]) into row x of histogram h
  auto histogram = [&](const Tile<K>& t, uint32_t xpack, int sel, int h) {
    const uint32_t x = (xpack >> (8 * sel)) & 0xffu;
    unsigned* hrow = hist + (size_t)h * 2 * hist_sz + x * K;
    const uint32_t sw = x & (K - 1);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = __builtin_amdgcn_fmed3f(t.v[kt][i] * scale_in, 0.f, scale);
        const unsigned hi = (unsigned)v;
        const unsigned lo = (unsigned)(__builtin_amdgcn_fractf(v) * scale);
        const uint32_t col = (uint32_t)(kt * 16 + 4 * g + i) ^ sw;
        __hip_atomic_fetch_add(&hrow[col], hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_fetch_add(&hrow[hist_sz + col], lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
  };
  // a pass's histograms out to memory; every cell read is cleared for whoever uses the area next
  auto flush = [&](const StatNode* __restrict__ np, int h0, int nh) {
    for (int h = 0; h < nh; ++h) {
      float* dst = leaf_flow + (size_t)np->hvar[h0 + h] * d.C * K;
      unsigned* hh = hist + (size_t)h * 2 * hist_sz;
      for (int i = threadIdx.x; i < d.C * K; i += blockDim.x) {
        const int c = i / K, j = i % K;
        const int cell = c * K + (j ^ (c & (K - 1)));
        const float val = (float)hh[cell] * hi_inv + (float)hh[hist_sz + cell] * lo_inv;
        hh[cell] = 0u;
        hh[hist_sz + cell] = 0u;
        const float old = rate != 0.f ? rate * dst[i] : 0.f;
        __builtin_nontemporal_store(old + val, &dst[i]);   // read once more, by the update
      }
    }
  };
  // pad positions: this lane's float4 of example row b (states kt*16 + 4g ..), and the element
  // (example 4q + g, state kt*16 + b) of the transposed read
  auto pad_w = [&](int kt) { return b * K + ((kt * 16 + 4 * g + 8 * b) & (K - 1)); };
  auto pad_r = [&](int q, int kt) { return (4 * q + g) * K + ((kt * 16 + b + 8 * g) & (K - 1)); };

  const int last = d.nslices - 1;
  const bool stream_on = d.nslices >= 2 * kStatLeanWaves;   // every wave then has two slices of a node at least
  const int n_it = (d.nslices - wave + kStatLeanWaves - 1) / kStatLeanWaves;   // this wave's slices of a node
  constexpr int kTileBytes = kSlice * K * 4;

  int cur = blockIdx.x;
  int nxt = cur + (int)gridDim.x < n_nodes ? cur + (int)gridDim.x : -1;
  StatRef A = stat_ref(d, nodes, cur, K * K * 4);
  // loop-carried requests: operands of the wave's next slice, categories and row maxima of the one after
  Tile<K> P0, R, C1, C2;   // (a third child is rare: it is fetched at the point of use)
  uint32_t xc, xn;
  float mc, mn;
  WTile<K> w;
  // categories and row maxima of the wave's first two slices: requested before the histograms are cleared, so
  // that the leaf rows that depend on them can go out right behind the barrier
  xc = load_x(A, min(wave, last));
  xn = load_x(A, min(wave + kStatLeanWaves, last));
  mc = load_m(A, min(wave, last));
  mn = load_m(A, min(wave + kStatLeanWaves, last));
  lean_w_load<K>(rW, vtile, A.w_off, w);
  for (int i = threadIdx.x; i < hist_words; i += blockDim.x) hist[i] = 0u;
  __syncthreads();
  bool warm = false;   // the first slice's operands of `cur` are on their way already

  while (true) {
    const StatNode* __restrict__ np = nodes + cur;
    const StatRef B = stat_ref(d, nodes, max(nxt, 0), K * K * 4);
    const int n_pass = (A.n_hist + nh_pass - 1) / nh_pass;
    const bool cross = stream_on && nxt >= 0 && n_pass == 1;   // this wave's stream runs on into `nxt`
    if (!warm) {
      // operands of the wave's first slice (slices past the end are clamped: harmless repeated loads)
      const int so = min(wave, last) * kTileBytes;
      lean_row_load<K>(rL, lean_row_off<K>(xc, 0, vleaf), A.leaf_off, P0);
      if (A.c1 >= 0) child_load(A.c1, xc, so, C1);
      if (A.c2 >= 0) child_load(A.c2, xc, so, C2);
      lean_tile_load<K>(rR, vtile, A.tile_off + so, R);
    }
    v4f accA[KT][KT];
#pragma unroll
    for (int a = 0; a < KT; ++a)
#pragma unroll
      for (int c = 0; c < KT; ++c) accA[a][c] = v4f{0.f, 0.f, 0.f, 0.f};

    {
      const int nh = min(nh_pass, A.n_hist);   // pass 0 fills the histograms of the first nh variables
      for (int it = 0; it < n_it; ++it) {
        const int s0 = wave + it * kStatLeanWaves;
        // where the requests of this turn go: the next slice of this node, or the first of the next node
        const bool over1 = it + 1 >= n_it, over2 = it + 2 >= n_it;
        const bool x1 = cross && over1, x2 = cross && over2;
        const int s1 = x1 ? wave : min(s0 + kStatLeanWaves, last);
        const int s2 = x2 ? wave + (it + 2 - n_it) * kStatLeanWaves : min(s0 + 2 * kStatLeanWaves, last);
        const int t_tile = x1 ? B.tile_off : A.tile_off, t_leaf = x1 ? B.leaf_off : A.leaf_off;
        const int t_c1 = x1 ? B.c1 : A.c1, t_c2 = x1 ? B.c2 : A.c2;
        const int t_x = x2 ? B.x_off : A.x_off;
        const int so1 = s1 * kTileBytes;
        // (1) E (unnormalised) from the landed operands; request the next slice's
        Tile<K> e = P0;
        if (A.c1 >= 0) tile_add<K>(e, C1);
        if (A.c2 >= 0) tile_add<K>(e, C2);
        const uint32_t xh = xc;   // categories of the slice computed now
        if (A.c3 >= 0) {
          Tile<K> t3;
          child_load(A.c3, xh, s0 * kTileBytes, t3);
          tile_add<K>(e, t3);
        }
        xc = xn;
        xn = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rX, (int)vx, t_x + s2 * (kSlice * 4), 0);
        const float m = mc;   // the scale the backward walk built R with
        mc = mn;
        mn = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rM, (int)vx, t_x + s2 * (kSlice * 4), 0));
        lean_row_load<K>(rL, lean_row_off<K>(xc, 0, vleaf), t_leaf, P0);
        if (t_c1 >= 0) child_load(t_c1, xc, so1, C1);
        if (t_c2 >= 0) child_load(t_c2, xc, so1, C2);
        // (2) E, the edge flows, then G = E .* (R W)
        tile_exp_sub<K>(e, m);
        {
          // A += R^T E over the 16 examples of the tile (contraction over examples): both operands
          // go through the wave's pad to reach the [state][example] operand layout.  A wave's LDS
          // accesses execute in order, so the pad needs no barrier between its phases.
          float ra[4][KT];
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<v4f*>(&pad[pad_w(kt)]) = R.v[kt];
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) ra[q][kt] = pad[pad_r(q, kt)];
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<v4f*>(&pad[pad_w(kt)]) = e.v[kt];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float eb[KT];
#pragma unroll
            for (int jt = 0; jt < KT; ++jt) eb[jt] = pad[pad_r(q, jt)];
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
        lean_tile_load<K>(rR, vtile, t_tile + so1, R);   // next slice's ratios, after the last use of these
        if (n_pass > 1) {
          // the later passes only need G: it replaces the tile of R just consumed
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, t.v[kt]), rR, (int)(vtile + kt * 1024),
                                                   A.tile_off + s0 * kTileBytes, 0);
        }
        // (3) histograms: the node's own variable, and its first leaf child if the LDS holds two
        if (s0 * kSlice + b < d.B) {
          histogram(t, xh, 0, 0);
          if (nh > 1) histogram(t, xh, 1, 1);
        }
      }
      __syncthreads();
      // the node after next is drawn while the histograms go out
      if (threadIdx.x == 0) *claim_word = nxt >= 0 ? stat_claim(counter, n_nodes) : -1;
      flush(np, 0, nh);
      __syncthreads();
    }
    const int nxt2 = __builtin_amdgcn_readfirstlane(*claim_word);
    for (int pass = 1; pass < n_pass; ++pass) {
      // further leaf children: G comes back from where pass 0 left it; only the categories differ
      const int h0 = pass * nh_pass, nh = min(nh_pass, A.n_hist - h0);
      Tile<K> T;
      uint32_t yc = load_x(A, min(wave, last)), yn = load_x(A, min(wave + kStatLeanWaves, last));
      lean_tile_load<K>(rR, vtile, A.tile_off + min(wave, last) * kTileBytes, T);
      for (int s0 = wave; s0 < d.nslices; s0 += kStatLeanWaves) {
        const int s1 = min(s0 + kStatLeanWaves, last), s2 = min(s0 + 2 * kStatLeanWaves, last);
        const uint32_t xh = yc;
        yc = yn;
        yn = load_x(A, s2);
        if (s0 * kSlice + b < d.B) {
          histogram(T, xh, h0, 0);
          if (nh > 1) histogram(T, xh, h0 + 1, 1);
        }
        lean_tile_load<K>(rR, vtile, A.tile_off + s1 * kTileBytes, T);
      }
      __syncthreads();
      flush(np, h0, nh);
      __syncthreads();
    }

    // combine the waves' partial blocks: every wave parks its accumulators in LDS (the histogram area is free
    // now), then each thread adds up the waves' copies of its elements in wave order.  The edge weight of an
    // element is already in the lane that holds it -- the block as the backward contraction's operand has
    // element (k, j) where the accumulator tile has it -- so the partial sums are parked weighted and the
    // parameters are not read again.
    v4f* park = reinterpret_cast<v4f*>(smem);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int jt = 0; jt < KT; ++jt)
        park[((size_t)wave * KT * KT + kt * KT + jt) * 64 + lane] = accA[kt][jt] * w.a[jt * KT + kt];
    if (nxt >= 0) lean_w_load<K>(rW, vtile, B.w_off, w);   // the next node's block, into the registers just freed
    __syncthreads();
    {
      float* dst = edge_aggr + (size_t)A.node * K * K;
      float* parkf = smem;
      for (int t = threadIdx.x; t < K * K; t += blockDim.x) {   // one element a thread: (tile q, component v)
        const int q = t >> 2, v = t & 3;
        float sum = parkf[t];
        parkf[t] = 0.f;
#pragma unroll
        for (int wv = 1; wv < kStatLeanWaves; ++wv) {
          sum += parkf[wv * (K * K) + t];
          parkf[wv * (K * K) + t] = 0.f;
        }
        const int kt = q / (KT * 64), jt = (q / 64) % KT, l = q % 64;
        const int idx = (kt * 16 + 4 * (l >> 4) + v) * K + jt * 16 + (l & 15);
        const float old = rate != 0.f ? rate * dst[idx] : 0.f;
        dst[idx] = old + sum;
      }
    }
    if (nxt < 0) break;
    if (!cross) {
      // the stream ended with this node: first categories and row maxima of the next one
      xc = load_x(B, min(wave, last));
      xn = load_x(B, min(wave + kStatLeanWaves, last));
      mc = load_m(B, min(wave, last));
      mn = load_m(B, min(wave + kStatLeanWaves, last));
    }
    __syncthreads();   // the area is clear again before anyone counts into it
    warm = cross;
    cur = nxt;
    nxt = nxt2;
    A = B;
  }
}

}  // namespace pcm
