// Dense groups of the layered engine: sum nodes of one layer over ONE set of (prime, sub) children.
//
// Every structure builder of the reference emits them -- the K sum nodes of an HCLT's tree node over its K
// products (src/structures/hclts.jl:133), the heads of a multi-head circuit over the root's products, the
// doubled sums of grow_heads_by_flows over the doubled products -- and per edge they cost the layer kernels an
// exponential and two row reads per example.  A group of G sums over C children is the block algebra of the HCLT
// kernels instead:
//   X[c] = sum of the values of child c's factors,  m = max_c X[c],  E[c] = exp(X[c] - m)
//   S[g] = sum_c W[g,c] E[c],  value of sum g = m + log S[g]                       (forward; W = exp(log-parameters))
//   R[g] = flow of sum g / S[g],  flow into child c = E[c] * sum_g W[g,c] R[g]      (backward)
//   edge flow (g, c) summed over the batch = W[g,c] * sum_b R[b,g] E[b,c]
// (tempered flows, fscale != 1: going down W, E and the shares of R to the power 1 / fscale, R over the tempered sum)
// with the three contractions on v_mfma_f32_16x16x4_f32: C exponentials per example instead of G * C.  The two that
// sit in the chain of layers are one wave per (group, 16 examples) with everything in registers; the edge flows, which
// nothing waits for, are one launch per shape of group after the pass.
//
// A child whose prime is a product node of up to three factors that only groups use (as a prime) is taken apart: the
// group reads the product's factors, writes the product's value next to its own, and the product leaves the forward
// layers (in an HCLT: the product of a tree node's children, which otherwise is a layer between any two levels).  Going down, a
// group's row for child c is the whole flow of every node that nothing else reaches -- the product, its factors, their
// only children -- and the kernel writes those rows itself (`copies`), so they leave the backward layers; where some
// other node still adds the row to flows from elsewhere it is kept behind the node rows of the flow array (row
// n_nodes + slot), which the layer kernels read like the flow of a product parent.  In an HCLT this leaves one group
// launch per tree level and direction and nothing else between the leaves and the root.
// The edge flows go to the same rows of partial sums as the layer kernels' (one row per 64 examples, added in order
// afterwards), so results do not depend on the order in which workgroups run.
#pragma once

namespace pcm {

typedef float g4f __attribute__((ext_vector_type(4)));

// The tables the kernels index are padded to the tile sizes, group after group in launch order: Gp = 16 GT entries of
// sums (node id -1 past G), Cp = 16 CT entries of children (own = -2 past C: a child that is not there, X = -inf) and
// Gp x Cp of W (0 outside G x C), so a kernel finds its group's entries from its block index and tests no bounds.
struct GroupRec {
  int32_t G, C;
  int32_t pnode0;   // the group's first entry in the per-sum tables
  int32_t pslot0;   // ... in the per-child tables
  int64_t pw0;      // ... in the W tables
  int32_t gt, ct;   // Gp / 16, Cp / 16
};

constexpr int kGroupCopies = 8;   // rows a group's kernel writes per child: two int4 of row numbers, -1: none

struct GroupDev {
  const GroupRec* rec;
  const int32_t* node;    // per sum entry: node id
  const int32_t* edge;    // per entry of the padded Gp x Cp, [g][c]: the up edge of sum g to child c (the sums list their
                          // children in orders of their own); -1 outside G x C
  const int4* rows;       // per child entry: the value rows whose sum is X: three for the prime, one for the sub (the row of zeros where there are fewer)
  const int32_t* own;     // per child entry: the product node that is the prime taken apart, whose value the forward kernel writes; -1: none
  const int4* copies;     // per child entry: kGroupCopies rows of the flow array that take the child's flow
  const int32_t* order;   // groups by shape, for the launches that are not per layer
  const float* wf;        // W in the order the forward kernel's lanes take it: [gt][q][lane] = W[16 gt + lo][4 q + hi]
  const float* wb;        // ... and the backward kernel's: [ct][k][lane] = W[4 k + hi][16 ct + lo]
  float* m;               // [groups][Bp]: the maximum the forward kernel took out, per example
  float* xm;              // [child entries][Bp]: X - m as the forward kernel formed it (-inf: an impossible child), for the way down
  const float* logp;
  float* mars;
  float* flows;           // [n_nodes + slots][Bp]
  float* edge_part;       // [Bp / 64][n_edges]
  int64_t n_nodes, n_edges;
  int32_t B, Bp;
  // tempered flows (fscale of mini_batch_em_beta): shares to the power inv_f = 1 / fscale, normalised again by the
  // sums' rows of `norm` (row norm_row for every sum if it is >= 0: the row of zeros of a pass that is not tempered)
  float inv_f;
  const float* norm;
  int64_t norm_row;
};

// where the kernels of one launch find their groups' entries: group = group0 + block, entries at base + block * stride
struct GroupBase {
  int32_t group0, pnode0, pslot0;
  int64_t pw0;
};

constexpr int kGroupPad = 65;   // row length of the [.][64 examples] tiles in LDS

// LDS of a statistics workgroup, in floats: E [Cp][65] | R [Gp][65]
__host__ __device__ inline size_t group_lds_floats(int Gp, int Cp) { return (size_t)(Cp + Gp) * kGroupPad; }

__host__ __device__ inline int64_t group_wf_index(int g, int c, int ct) {   // ct = Cp / 16
  return ((int64_t)(g >> 4) * (ct * 4) + (c >> 2)) * 64 + (c & 3) * 16 + (g & 15);
}
__host__ __device__ inline int64_t group_wb_index(int g, int c, int gt) {   // gt = Gp / 16
  return ((int64_t)(c >> 4) * (gt * 4) + (g >> 2)) * 64 + (g & 3) * 16 + (c & 15);
}

// exp of the groups' log-parameters in both orders, once per pass (the parameters may have moved): thread = (group,
// entry of its padded Gp x Cp)
__global__ __launch_bounds__(256) void sparse_group_w_kernel(GroupDev d, const int32_t* __restrict__ group_of_elem, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const GroupRec r = d.rec[group_of_elem[i]];
  const int64_t local = i - r.pw0;
  const int g = (int)(local / (16 * r.ct)), c = (int)(local % (16 * r.ct));
  const int e = d.edge[i];
  const float w = e >= 0 ? __expf(d.logp[e] * d.inv_f) : 0.f;
  const_cast<float*>(d.wf)[r.pw0 + group_wf_index(g, c, r.ct)] = w;
  const_cast<float*>(d.wb)[r.pw0 + group_wb_index(g, c, r.gt)] = w;
}

__device__ __forceinline__ int guni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// X of a child for the example in column `col`: the value of its prime (the first three rows: the prime itself and
// two rows of zeros, or the factors of a product the group computes) plus its sub's (the last row; zeros: none)
__device__ __forceinline__ float group_prime_value(const GroupDev& d, const int4 rw, int64_t col) {
  return (d.mars[(int64_t)rw.x * d.Bp + col] + d.mars[(int64_t)rw.y * d.Bp + col]) + d.mars[(int64_t)rw.z * d.Bp + col];
}
__device__ __forceinline__ float group_x(const GroupDev& d, const int4 rw, int64_t col) {
  return group_prime_value(d, rw, col) + d.mars[(int64_t)rw.w * d.Bp + col];
}

// maximum over the four lanes that hold one example (lane, lane ^ 16, lane ^ 32, lane ^ 48)
__device__ __forceinline__ float group_max4(float v) {
  const int a = __builtin_bit_cast(int, v);
  const auto r16 = __builtin_amdgcn_permlane16_swap(a, a, false, false);
  v = fmaxf(__builtin_bit_cast(float, (int)r16[0]), __builtin_bit_cast(float, (int)r16[1]));
  const int b = __builtin_bit_cast(int, v);
  const auto r32 = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return fmaxf(__builtin_bit_cast(float, (int)r32[0]), __builtin_bit_cast(float, (int)r32[1]));
}

// Forward: values of the group's sums.  One wave per (group, 16 examples), nothing shared: lane 16 * hi + lo takes
// example lo and the children c = 4 q + hi, which is the B-operand layout of the matrix instruction's k-step q, so
// X, the maximum (two lane swaps), E and the contraction stay in the wave's registers.  GT = Gp / 16, CT = Cp / 16.
// What the kernel reads is requested in two rounds (row numbers, W and node ids; then the rows), everything of a round
// before anything of it is used and no branch around a load: a layer's launch lasts as long as its longest chain of
// requests.  The maximum goes to d.m for the backward kernels.
template <int GT, int CT>
__device__ __forceinline__ void group_forward_body(const GroupDev& d, const GroupBase& base, int bx, int lane, int slice) {
  constexpr int NK = CT * 4, Gp = GT * 16, Cp = CT * 16;
  constexpr bool kPre = GT * NK <= 64;   // W in registers before the rows arrive
  const int group = base.group0 + bx;
  const int lo = lane & 15, hi = lane >> 4;
  const int64_t col = (int64_t)slice * 16 + lo;
  const int4* rows = d.rows + base.pslot0 + (int64_t)bx * Cp;
  const int32_t* owns = d.own + base.pslot0 + (int64_t)bx * Cp;
  const int32_t* node = d.node + base.pnode0 + (int64_t)bx * Gp;
  const float* wg = d.wf + base.pw0 + (int64_t)bx * Gp * Cp + lane;
  int4 rw[NK];
  int own[NK];
#pragma unroll
  for (int q = 0; q < NK; ++q) { rw[q] = rows[4 * q + hi]; own[q] = owns[4 * q + hi]; }
  float a[kPre ? GT : 1][kPre ? NK : 1];
  if constexpr (kPre) {
#pragma unroll
    for (int gt = 0; gt < GT; ++gt)
#pragma unroll
      for (int q = 0; q < NK; ++q) a[gt][q] = wg[(gt * NK + q) * 64];
  }
  int4 nd4[GT];   // (the four sums of a lane's output rows are neighbours in the table: one request per tile)
#pragma unroll
  for (int gt = 0; gt < GT; ++gt) nd4[gt] = *reinterpret_cast<const int4*>(node + gt * 16 + 4 * hi);
  float x[NK], pv[NK];
#pragma unroll
  for (int q = 0; q < NK; ++q) {
    pv[q] = group_prime_value(d, rw[q], col);
    x[q] = pv[q] + d.mars[(int64_t)rw[q].w * d.Bp + col];
  }
#pragma unroll
  for (int q = 0; q < NK; ++q) if (own[q] == -2) x[q] = -INFINITY;
  float mx = x[0];
#pragma unroll
  for (int q = 1; q < NK; ++q) mx = fmaxf(mx, x[q]);
  mx = group_max4(mx);
  if (!(mx > -INFINITY)) mx = 0.f;   // every child impossible: E = 0, the sums come out as -inf
  float* xm = d.xm + (base.pslot0 + (int64_t)bx * Cp) * d.Bp + col;
#pragma unroll
  for (int q = 0; q < NK; ++q) {
    if (own[q] >= 0) d.mars[(int64_t)own[q] * d.Bp + col] = pv[q];
    const float xs = x[q] - mx;   // (-inf stays -inf)
    xm[(int64_t)(4 * q + hi) * d.Bp] = xs;
    x[q] = x[q] > -INFINITY ? __expf(xs) : 0.f;
  }
  if (hi == 0) d.m[(int64_t)group * d.Bp + col] = mx;
#pragma unroll
  for (int gt = 0; gt < GT; ++gt) {
    g4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < NK; ++q) {
      float av;
      if constexpr (kPre) av = a[gt][q];
      else av = wg[(gt * NK + q) * 64];
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av, x[q], acc, 0, 0, 0);
    }
    const int nd[4] = {nd4[gt].x, nd4[gt].y, nd4[gt].z, nd4[gt].w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (nd[i] >= 0) d.mars[(int64_t)nd[i] * d.Bp + col] = mx + __logf(acc[i]);
  }
}

template <int GT, int CT>
__global__ __launch_bounds__(64) void sparse_group_forward_kernel(GroupDev d, GroupBase base) {
  group_forward_body<GT, CT>(d, base, blockIdx.x, threadIdx.x, blockIdx.y);
}

// Backward, per layer: the rows the group hands its children, E[c] * sum_g W[g,c] R[g].  One wave per (group, 16
// examples) as going up: R of the sums g = 4 k + hi is the B operand of k-step k as it is loaded.  The same two
// rounds of requests where the registers hold a group's W and row numbers (kPre); 16 children at a time otherwise.
template <int GT, int CT>
__device__ __forceinline__ void group_backward_body(const GroupDev& d, const GroupBase& base, int bx, int lane, int slice) {
  constexpr int NG = GT * 4, Gp = GT * 16, Cp = CT * 16;
  constexpr bool kPre = CT <= 2 && GT * CT <= 16;
  constexpr int CL = kPre ? CT : 1;
  const int group = base.group0 + bx;
  const int lo = lane & 15, hi = lane >> 4;
  const int64_t col = (int64_t)slice * 16 + lo;
  const float* xm = d.xm + (base.pslot0 + (int64_t)bx * Cp) * d.Bp + col;
  const int4* copies = d.copies + 2 * (base.pslot0 + (int64_t)bx * Cp);
  const int32_t* node = d.node + base.pnode0 + (int64_t)bx * Gp;
  const float* wg = d.wb + base.pw0 + (int64_t)bx * Gp * Cp + lane;
  const float mb = d.m[(int64_t)group * d.Bp + col];
  int nd[NG];
#pragma unroll
  for (int k = 0; k < NG; ++k) nd[k] = node[4 * k + hi];
  int4 cpa[CL][4], cpb[CL][4];
  float a[CL][NG], e[CL][4];
  auto numbers = [&](int ct, int s) {   // row numbers and W for the children 16 ct + 4 hi + i
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = ct * 16 + 4 * hi + i;
      cpa[s][i] = copies[2 * c];
      cpb[s][i] = copies[2 * c + 1];
    }
#pragma unroll
    for (int k = 0; k < NG; ++k) a[s][k] = wg[(ct * NG + k) * 64];
  };
  auto values = [&](int ct, int s) {   // X - m as the forward kernel left it (a child that is not there: -inf)
#pragma unroll
    for (int i = 0; i < 4; ++i) e[s][i] = xm[(int64_t)(ct * 16 + 4 * hi + i) * d.Bp];
  };
  if constexpr (kPre) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) numbers(ct, ct);
  }
  float rv[NG];
  {   // R = F / S = F * exp(m - value): no flow stays no flow where the value is -inf.  (All rows requested, then used:
      // written as one loop the compiler waits for every sum's rows in turn.)
    float f[NG], v[NG], nv[NG];
#pragma unroll
    for (int k = 0; k < NG; ++k) {
      const int64_t n = nd[k] < 0 ? 0 : nd[k];
      f[k] = d.flows[n * d.Bp + col];
      v[k] = d.mars[n * d.Bp + col];
      nv[k] = 0.f;
    }
    if (d.norm_row < 0) {   // tempered flows only (the same for every lane: a branch around requests, none around a wait)
#pragma unroll
      for (int k = 0; k < NG; ++k) nv[k] = d.norm[(nd[k] < 0 ? 0 : (int64_t)nd[k]) * d.Bp + col];
    }
#pragma unroll
    for (int k = 0; k < NG; ++k)
      rv[k] = (nd[k] >= 0 && f[k] > 0.f && v[k] > -INFINITY) ? f[k] * __expf((mb - v[k]) * d.inv_f - nv[k]) : 0.f;
  }
  if constexpr (kPre) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) values(ct, ct);
  }
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int s = kPre ? ct : 0;
    if constexpr (!kPre) { numbers(ct, 0); values(ct, 0); }
    g4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < NG; ++k) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s][k], rv[k], acc, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float f = (e[s][i] > -INFINITY ? __expf(e[s][i] * d.inv_f) : 0.f) * acc[i];
      const int4 p = cpa[s][i], q = cpb[s][i];
      if (p.x >= 0) d.flows[(int64_t)p.x * d.Bp + col] = f;
      if (p.y >= 0) d.flows[(int64_t)p.y * d.Bp + col] = f;
      if (p.z >= 0) d.flows[(int64_t)p.z * d.Bp + col] = f;
      if (p.w >= 0) d.flows[(int64_t)p.w * d.Bp + col] = f;
      if (q.x >= 0) d.flows[(int64_t)q.x * d.Bp + col] = f;
      if (q.y >= 0) d.flows[(int64_t)q.y * d.Bp + col] = f;
      if (q.z >= 0) d.flows[(int64_t)q.z * d.Bp + col] = f;
      if (q.w >= 0) d.flows[(int64_t)q.w * d.Bp + col] = f;
    }
  }
}

template <int GT, int CT>
__global__ __launch_bounds__(64) void sparse_group_backward_kernel(GroupDev d, GroupBase base) {
  group_backward_body<GT, CT>(d, base, blockIdx.x, threadIdx.x, blockIdx.y);
}

// Walks: several consecutive layers of groups in ONE launch.  A launch that depends on the one before costs 4 to 5 us
// however little it does, and a circuit over a tree has as many layers of groups as the tree has levels; but everything
// a group reads and writes for 16 examples is read and written for those 16 examples only.  So a workgroup takes one
// slice of 16 examples through all the layers of a run (layers that hold groups of one shape and nothing else): a layer's
// groups dealt to its waves, a barrier between layers.  What a layer stores the next one reads through the same compute
// unit's cache, which the waves of a workgroup share: the barrier's wait for the stores is all the ordering it needs.
// Used where a layer's groups would not fill the device anyway (the host decides).
struct GroupWalk {
  const int2* levels;   // per layer of the run, in the order of the walk: {its first group, counted from the run's first; groups}
  int n_levels;
  GroupBase base;       // of the run's first group (the tables are padded: group i's entries are i strides further on)
};

template <int GT, int CT, int WV, bool kForward>
__global__ __launch_bounds__(WV * 64) void sparse_group_walk_kernel(GroupDev d, GroupWalk w) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int l = 0; l < w.n_levels; ++l) {
    const int2 lv = w.levels[l];
    for (int i = wave; i < lv.y; i += WV) {
      if constexpr (kForward) group_forward_body<GT, CT>(d, w.base, lv.x + i, lane, blockIdx.x);
      else group_backward_body<GT, CT>(d, w.base, lv.x + i, lane, blockIdx.x);
    }
    __syncthreads();
  }
}

// Edge flows of the groups of one shape, after the backward pass: W[g,c] * sum_b R[b,g] E[b,c] over a block of 64
// examples, from the values and flows the pass has left.  A workgroup takes (group, 64 examples): E and R in LDS (a
// wave stages every fourth child, whose row numbers are the same for its 64 lanes: scalar loads, the rows of eight
// children requested before the first is used), the GT x CT tiles of the result dealt out over its four waves.
template <int GT, int CT>
__global__ __launch_bounds__(256) void sparse_group_stats_kernel(GroupDev d, int first) {
  extern __shared__ float glds[];
  const int group = d.order[first + blockIdx.x];
  const GroupRec r = d.rec[group];
  constexpr int Gp = GT * 16, Cp = CT * 16;
  const int b0 = blockIdx.y * 64;
  float* E = glds;
  float* R = E + (size_t)Cp * kGroupPad;
  const int t = threadIdx.x;
  const int b = t & 63, part = guni(t >> 6);
  const float mb = d.m[(int64_t)group * d.Bp + b0 + b];
  for (int cb = part; cb < Cp; cb += 32) {
    float x[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int c = cb + 4 * q;
      x[q] = c < Cp ? d.xm[(int64_t)(r.pslot0 + c) * d.Bp + b0 + b] : -INFINITY;
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int c = cb + 4 * q;
      if (c < Cp) E[c * kGroupPad + b] = x[q] > -INFINITY ? __expf(x[q] * d.inv_f) : 0.f;
    }
  }
  for (int gb = part; gb < Gp; gb += 32) {   // (eight sums' rows requested before the first is used, as above)
    float f[8], v[8], nv[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int g = gb + 4 * q;
      f[q] = 0.f;
      v[q] = 0.f;
      nv[q] = 0.f;
      if (g < r.G) {
        const int64_t n = guni(d.node[r.pnode0 + g]);
        f[q] = d.flows[n * d.Bp + b0 + b];
        v[q] = d.mars[n * d.Bp + b0 + b];
        nv[q] = d.norm[(d.norm_row >= 0 ? d.norm_row : n) * d.Bp + b0 + b];
      }
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int g = gb + 4 * q;
      if (g < Gp) R[g * kGroupPad + b] = (f[q] > 0.f && v[q] > -INFINITY) ? f[q] * __expf((mb - v[q]) * d.inv_f - nv[q]) : 0.f;
    }
  }
  __syncthreads();
  const int lane = t & 63, wave = t >> 6;
  const int lo = lane & 15, hi = lane >> 4;
  float* part_row = d.edge_part + (size_t)blockIdx.y * d.n_edges;
  for (int tile = wave; tile < GT * CT; tile += 4) {
    const int gt = tile / CT, ct = tile % CT;
    g4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 16; ++kk)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(R[(gt * 16 + lo) * kGroupPad + kk * 4 + hi], E[(ct * 16 + lo) * kGroupPad + kk * 4 + hi],
                                                 acc, 0, 0, 0);
    const int c = ct * 16 + lo;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = gt * 16 + 4 * hi + i;
      if (g < r.G && c < r.C) part_row[d.edge[r.pw0 + g * Cp + c]] = d.wf[r.pw0 + group_wf_index(g, c, CT)] * acc[i];
    }
  }
}

}  // namespace pcm
