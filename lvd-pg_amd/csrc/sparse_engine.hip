// General engine: flattening of circuit DAGs and layered kernels for any circuit.
#include "sparse_engine.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <numeric>
#include <tuple>
#include <type_traits>
#include <unordered_map>

#include "stage_kernel.hip.hpp"

namespace pcm {

static void check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

// ---------------------------------------------------------------------------------------
// flattening
// ---------------------------------------------------------------------------------------

// Restates ProbabilisticCircuits.jl `BitsProbCircuit(pc)` (un-vendored; behaviour pinned by
// the reference's test/bits_circuit_tests.jl:13-24, test/misc_tests.jl:39-62 and
// test/queries/likelihood_tests.jl:24-37 on the 3-variable fixture): nodes are created in
// depth-first post-order from the root, children in order; a node with a single child is
// passed through; a product of exactly two plain nodes that has a single parent becomes a
// (prime, sub) edge of that parent; other products pair their children up into edges;
// up edges are grouped by layer (height), then by parent id.
FlatCircuit flatten_dag(int32_t num_nodes, const uint8_t* node_type, const int32_t* child_ptr,
                        const int32_t* child_idx, const float* sum_logp, const int32_t* input_var,
                        const float* input_logp, int32_t num_vars, int32_t num_cats, int32_t num_heads) {
  if (num_nodes < 1) fail(PCM_ERR_SHAPE, "circuit has no nodes");
  if (!node_type || !child_ptr || !input_var || !input_logp) fail(PCM_ERR_ARG, "null description array");
  if (num_cats < 1 || num_cats > 256) fail(PCM_ERR_SHAPE, "num_cats must be in 1..256, got %d", num_cats);
  if (num_heads < 0 || num_heads > num_nodes) fail(PCM_ERR_SHAPE, "num_heads %d out of range", num_heads);
  const int n_edges_in = child_ptr[num_nodes];
  if (n_edges_in > 0 && (!child_idx || !sum_logp)) fail(PCM_ERR_ARG, "null child arrays");
  std::vector<int64_t> in_rank(num_nodes, -1);
  int64_t n_in = 0;
  for (int n = 0; n < num_nodes; ++n) {
    if (node_type[n] > kMul) fail(PCM_ERR_SHAPE, "node %d has unknown type %d", n, node_type[n]);
    const int c0 = child_ptr[n], c1 = child_ptr[n + 1];
    if (c1 < c0) fail(PCM_ERR_SHAPE, "child_ptr decreases at node %d", n);
    if (node_type[n] == kInput) {
      if (c1 != c0) fail(PCM_ERR_SHAPE, "input node %d has children", n);
      if (input_var[n] < 0 || input_var[n] >= num_vars) fail(PCM_ERR_SHAPE, "input node %d reads variable %d", n, input_var[n]);
      in_rank[n] = n_in++;
    } else {
      if (c1 == c0) fail(PCM_ERR_SHAPE, "inner node %d has no children", n);
      for (int c = c0; c < c1; ++c)
        if (child_idx[c] < 0 || child_idx[c] >= n) fail(PCM_ERR_SHAPE, "node %d: child %d is not an earlier node", n, child_idx[c]);
    }
  }
  std::vector<int32_t> roots;
  if (num_heads == 0) roots.push_back(num_nodes - 1);
  else for (int h = 0; h < num_heads; ++h) roots.push_back(num_nodes - num_heads + h);

  // parents of reachable nodes
  std::vector<int32_t> nparents(num_nodes, 0);
  {
    std::vector<char> seen(num_nodes, 0);
    std::vector<int32_t> st(roots.begin(), roots.end());
    while (!st.empty()) {
      int n = st.back(); st.pop_back();
      if (seen[n]) continue;
      seen[n] = 1;
      for (int c = child_ptr[n]; c < child_ptr[n + 1]; ++c) { nparents[child_idx[c]]++; st.push_back(child_idx[c]); }
    }
  }

  FlatCircuit fc;
  fc.num_vars = num_vars; fc.num_cats = num_cats; fc.num_heads = num_heads;
  struct Info { int kind = -1; int32_t a = -1, b = -1; };   // kind 0: node a; 1: element (a, b)
  std::vector<Info> memo(num_nodes);
  struct Edge { int32_t prime, sub; float logp; };
  std::vector<std::vector<Edge>> edges;
  auto new_node = [&](uint8_t t, int32_t var, int64_t off) {
    fc.type.push_back(t); fc.in_var.push_back(var); fc.in_off.push_back(off);
    edges.emplace_back();
    return (int32_t)fc.type.size() - 1;
  };
  auto materialize = [&](Info& i) {
    if (i.kind == 1) {
      const int32_t id = new_node(kMul, -1, -1);
      edges[id].push_back({i.a, i.b, 0.f});
      i = Info{0, id, -1};
    }
    return i.a;
  };
  struct Frame { int32_t n, c; };
  for (int32_t root : roots) {
    std::vector<Frame> st;
    st.push_back({root, child_ptr[root]});
    while (!st.empty()) {
      Frame& f = st.back();
      const int n = f.n;
      if (memo[n].kind >= 0) { st.pop_back(); continue; }
      if (f.c < child_ptr[n + 1]) {
        const int c = child_idx[f.c++];
        if (memo[c].kind < 0) st.push_back({c, child_ptr[c]});
        continue;
      }
      Info info;
      const int c0 = child_ptr[n], c1 = child_ptr[n + 1];
      if (node_type[n] == kInput) {
        const int64_t off = (int64_t)fc.input_nodes.size() * num_cats;
        const int32_t id = new_node(kInput, input_var[n], off);
        fc.input_nodes.push_back(id);
        fc.leaf_logp.insert(fc.leaf_logp.end(), input_logp + in_rank[n] * num_cats, input_logp + (in_rank[n] + 1) * num_cats);
        info = Info{0, id, -1};
      } else if (c1 - c0 == 1) {
        info = memo[child_idx[c0]];
      } else if (node_type[n] == kSum) {
        std::vector<Edge> es;
        for (int c = c0; c < c1; ++c) {
          const Info& ci = memo[child_idx[c]];
          es.push_back({ci.a, ci.kind == 1 ? ci.b : -1, sum_logp[c]});
        }
        const int32_t id = new_node(kSum, -1, -1);
        edges[id] = es;
        info = Info{0, id, -1};
      } else {
        std::vector<int32_t> ids;
        for (int c = c0; c < c1; ++c) ids.push_back(materialize(memo[child_idx[c]]));
        if (ids.size() == 2 && nparents[n] <= 1) {
          info = Info{1, ids[0], ids[1]};
        } else {
          const int32_t id = new_node(kMul, -1, -1);
          for (size_t q = 0; q < ids.size(); q += 2)
            edges[id].push_back({ids[q], q + 1 < ids.size() ? ids[q + 1] : -1, 0.f});
          info = Info{0, id, -1};
        }
      }
      memo[n] = info;
      st.pop_back();
    }
    fc.heads.push_back(materialize(memo[root]));
  }
  if (num_heads == 0) fc.heads.clear();
  fc.desc_node.assign(num_nodes, -1);
  for (int n = 0; n < num_nodes; ++n)
    if (memo[n].kind == 0) fc.desc_node[n] = memo[n].a;

  // layers and up-edge order
  const int64_t nn = fc.n_nodes();
  fc.layer.assign(nn, 0);
  for (int64_t n = 0; n < nn; ++n)
    for (const Edge& e : edges[n]) {
      fc.layer[n] = std::max(fc.layer[n], fc.layer[e.prime] + 1);
      if (e.sub >= 0) fc.layer[n] = std::max(fc.layer[n], fc.layer[e.sub] + 1);
    }
  std::vector<int32_t> parents;
  for (int64_t n = 0; n < nn; ++n) if (!edges[n].empty()) parents.push_back((int32_t)n);
  std::stable_sort(parents.begin(), parents.end(), [&](int32_t a, int32_t b) { return fc.layer[a] < fc.layer[b]; });
  for (int32_t p : parents)
    for (const Edge& e : edges[p]) {
      fc.e_parent.push_back(p); fc.e_prime.push_back(e.prime); fc.e_sub.push_back(e.sub); fc.e_logp.push_back(e.logp);
    }
  fc.finish();
  return fc;
}

void FlatCircuit::finish() {
  const int64_t nn = n_nodes(), ne = n_edges();
  node_e0.assign(nn, 0); node_e1.assign(nn, 0);
  layer_ends.clear();
  edge2param.assign(ne, 0); param2edge.clear(); param2group.clear(); pargroup_sizes.clear();
  int64_t group = 0;
  for (int64_t e = 0; e < ne; ++e) {
    const int32_t p = e_parent[e];
    const bool first = e == 0 || e_parent[e - 1] != p, last = e + 1 == ne || e_parent[e + 1] != p;
    if (first) node_e0[p] = (int32_t)e;
    if (last) node_e1[p] = (int32_t)e + 1;
    if (e > 0 && layer[e_parent[e - 1]] != layer[p]) layer_ends.push_back(e);
    if (type[p] == kSum) {
      if (first) { ++group; pargroup_sizes.push_back(0); }
      param2edge.push_back(e + 1);
      edge2param[e] = (int64_t)param2edge.size();
      param2group.push_back(group);
      pargroup_sizes.back()++;
    }
  }
  if (ne) layer_ends.push_back(ne);
}

// ---------------------------------------------------------------------------------------
// kernels
// ---------------------------------------------------------------------------------------

}  // namespace pcm
#include "sparse_groups.hip.hpp"
namespace pcm {

struct SparseDev {
  const uint8_t* type;
  const int32_t* order;      // node ids sorted by layer
  const int4* fwd_rec;       // per position of `order`: {node, type, first up edge, end of up edges}
  const int4* bwd_rec;       // per position of the backward order: {node, seed index or -1, first in-edge, end of in-edges}
  const int2* bwd_alias;     // ... and its range in the alias list
  const int32_t *node_e0, *node_e1, *e_parent, *e_prime, *e_sub, *in_var, *in_ptr, *in_edge;
  const int4* in_rec;        // per incoming edge: {edge << 1 | role, parent (~parent: product), prime, sub}
  const float* in_logp;      // ... and the edge's log-parameter, gathered before every backward pass
  const int64_t* in_off;
  const float* logp;
  const float* leaf;
  const uint8_t* xb;         // [V][Bp]
  const float* ev;           // soft evidence instead of xb (else null): log-evidence of (example, variable, category)
  int64_t ev_se, ev_sv, ev_sc;   // ... at ev[row * ev_se + var * ev_sv + cat * ev_sc], row = ev_idx ? ev_idx[b] : b
  const int32_t* ev_idx;
  float* mars;               // [n_nodes][Bp]
  float* flows;
  int32_t B, Bp, C;
  int64_t n_nodes;
  int64_t n_flow_rows;       // node rows of the flow array + the rows dense groups hand their children
  const float* norm;         // tempered flows: [n_nodes + 1][Bp], log of a sum node's sum over its edges of share^(1 / fscale); 0 elsewhere
  float inv_f;               // ... and 1 / fscale
};

// ProbabilisticCircuits.jl logsumexp(x, y) as used by src/queries/likelihood.jl:101-102.
__device__ __forceinline__ float lse2(float x, float y) {
  if (isfinite(x) && isfinite(y)) return fmaxf(x, y) + log1pf(expf(-fabsf(x - y)));
  return fmaxf(x, y);
}


// The layer kernels are chains of memory round trips (edge records, then the rows they
// name), not arithmetic: a wave therefore takes its node's edges in runs of 16, then 4, then
// single ones, and requests all operands of a run before it uses the first.

// x where keep is all ones, +0 where it is zero: a select the compiler cannot turn into a branch
// around the load that produced x (a branch per edge would serialise the run's requests)
__device__ __forceinline__ float keep_bits(float x, unsigned keep) {
  return __builtin_bit_cast(float, __builtin_bit_cast(unsigned, x) & keep);
}


// A value every lane of the wave holds alike, moved to a scalar register: what is computed from it (row
// addresses, edge ranges, branch conditions) is then scalar work, and a row access becomes scalar base + lane
// offset.  Without it the layer kernels keep a copy of every index and 64-bit address per lane and run out of
// registers: 2 waves per SIMD with 32 edges in flight.
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float uni(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// The rows of the value and flow arrays, addressed the way the layer kernels need them: one descriptor per
// array in scalar registers, the row as a scalar byte offset, the example as the lane's byte offset -- a row
// costs one scalar register instead of a 64-bit address.  kBuf = false (arrays of 2 GiB or more, beyond a
// signed 32-bit row offset) keeps plain pointers.
template <bool kBuf>
struct Rows {
  const float* base;
  __amdgpu_buffer_rsrc_t rsrc;
  int row_bytes;
  __device__ __forceinline__ Rows(const float* p, int64_t n_rows, int Bp) : base(p), row_bytes(Bp * 4) {
    if constexpr (kBuf)
      rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p), 0, (int)(uint32_t)(n_rows * Bp * 4), 0x00020000);
  }
  // value of example b (a lane's own) in row `row` (wave-uniform)
  __device__ __forceinline__ float at(int row, int b) const {
    if constexpr (kBuf)
      return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, b * 4, row * row_bytes, 0));
    else
      return base[(size_t)row * (row_bytes >> 2) + b];
  }
};

template <int U, int EX, bool kBuf>
__device__ __forceinline__ void forward_run(const SparseDev& d, const Rows<kBuf>& mars, bool issum, int c0,
                                            const int (&bb)[EX], float (&m)[EX], float (&sum)[EX]) {
  float child[U][EX];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int e = c0 + u;
    const int pr = uni(d.e_prime[e]);
    const int s = uni(d.e_sub[e]);
    const unsigned has_sub = s >= 0 ? ~0u : 0u;
    const float lp = uni(d.logp[e]);   // 0 on product edges
#pragma unroll
    for (int x = 0; x < EX; ++x) child[u][x] = mars.at(pr, bb[x]) + keep_bits(mars.at(max(s, 0), bb[x]), has_sub) + lp;
  }
  // a run is folded in two passes: its maximum first, then one exponential per edge relative to the larger of
  // that and the maximum so far (the sum so far is rescaled once per run)
#pragma unroll
  for (int x = 0; x < EX; ++x) {
    if (!issum) {
#pragma unroll
      for (int u = 0; u < U; ++u) m[x] += child[u][x];
    } else {
      float mr = child[0][x];
#pragma unroll
      for (int u = 1; u < U; ++u) mr = fmaxf(mr, child[u][x]);
      const float mn = fmaxf(m[x], mr);
      if (mn != -INFINITY) {
        float s = sum[x] * __expf(m[x] - mn);
#pragma unroll
        for (int u = 0; u < U; ++u) s += __expf(child[u][x] - mn);
        sum[x] = s;
        m[x] = mn;
      }
    }
  }
}

// Forward, one layer: a workgroup takes one node of the layer and 64 * EX examples (lane t:
// examples t, t + 64, ...).  Restates src/regularization/reg_likelihood.jl:16-49 (inputs) and
// src/queries/likelihood.jl:29-48: a product adds its children, a sum node is the logsumexp of
// its edges in up-edge order -- kept as a running maximum and a sum of exponentials relative to
// it (one exponential per edge; the reference folds pairwise, the two agree to rounding).
// kLayerWaves waves share a node's edges: the kernels are chains of dependent memory round
// trips, so a layer too small to fill the machine finishes sooner when a node's chain is cut in
// four; layers with plenty of (node, 64 examples) pairs give each pair one wave.
// Which build of the two layer kernels a layer takes (measured on a 192-variable, K = 32, 128-head circuit at
// 1024 examples, 1.31 -> 0.72 ms per EM step together with the scalar indices and buffer-addressed rows above):
//   * nodes with at most kNarrowDegree edges: runs of 4 only (a third of the registers, three times the waves in
//     flight), from kManyPairs (node, 64 examples) pairs on with four examples per lane, so that a wave's index
//     fetches (node, edge range, edge records) serve 256 examples;
//   * otherwise, below kSplitBelow pairs: kSplitWaves waves share a node's edges (the layer cannot fill the
//     device with one wave per pair, and a wave's chain of round trips gets shorter);
//   * otherwise one wave per pair, runs of up to kWideRun edges requested at once (16: seven waves per SIMD;
//     32 halves the waves and is slower, 8 leaves too few requests in flight); from kSaturated pairs on, where the
//     device is full whatever the shape of a wave, two examples per lane and runs of 8, which halves the index
//     work per example (16 circuits of that kind compiled as one: 5.47 -> 5.17 ms per step).
constexpr int kSplitWaves = 4;
constexpr int kSplitRun = 16;       // longest run in the kernels that split a node over kSplitWaves waves
constexpr int kSplitBelow = 8192;   // (node, 64 examples) pairs in a layer below which its nodes are split
constexpr int kNarrowDegree = 8;    // a layer whose nodes have at most this many edges takes the kMaxRun = 4 kernels
constexpr int kWideRun = 16;        // longest run of edges requested at once in the one-wave kernels
constexpr int kSaturated = 32768;   // pairs from which a many-edged layer takes two examples per lane and runs of 8
constexpr int kManyPairs = 16384;   // (node, 64 examples) pairs from which a narrow layer takes four examples per lane

template <int EX, int kLayerWaves, int kMaxRun, bool kBuf>
__global__ __launch_bounds__(kLayerWaves * 64) void sparse_forward_kernel(SparseDev d, int n0) {
  __shared__ float xm[kLayerWaves][EX][64], xs[kLayerWaves][EX][64];
  const int4 rec = d.fwd_rec[n0 + blockIdx.x];   // one fetch instead of order -> type, edge range
  const int n = uni(rec.x);
  const int lane = threadIdx.x & 63, wave = uni((int)(threadIdx.x >> 6));
  const int b0 = blockIdx.y * (64 * EX) + lane;
  int bb[EX];
#pragma unroll
  for (int x = 0; x < EX; ++x) bb[x] = min(b0 + 64 * x, d.Bp - 1);
  float m[EX], sum[EX];
  const int type = uni(rec.y);
  if (type == kInput) {
    if (wave) return;
    if (d.ev) return;   // soft evidence: sparse_soft_input_kernel has filled the input rows
    {
      const uint8_t* xr = d.xb + (size_t)uni(d.in_var[n]) * d.Bp;
      const int64_t off = d.in_off[n];
      const float* row = d.leaf + (((int64_t)uni((int)(off >> 32)) << 32) | (uint32_t)uni((int)off));
#pragma unroll
      for (int x = 0; x < EX; ++x) { m[x] = row[xr[bb[x]]]; sum[x] = 1.f; }
    }
  } else {
    // the node's edges in kLayerWaves contiguous shares, one per wave; a share is folded as a
    // running maximum and a sum of exponentials (products: a plain sum), the shares are then
    // combined through LDS by the first wave
    const bool issum = type == kSum;
    const int e0 = uni(rec.z), e1 = uni(rec.w);
    const int per = (e1 - e0 + kLayerWaves - 1) / kLayerWaves;
    const int my0 = min(e0 + wave * per, e1), my1 = min(my0 + per, e1);
#pragma unroll
    for (int x = 0; x < EX; ++x) { m[x] = issum ? -INFINITY : 0.f; sum[x] = issum ? 0.f : 1.f; }
    const Rows<kBuf> mars(d.mars, d.n_nodes, d.Bp);
    int c0 = my0;
    if constexpr (kMaxRun >= 32)
      for (; c0 + 32 <= my1; c0 += 32) forward_run<32, EX, kBuf>(d, mars, issum, c0, bb, m, sum);
    if constexpr (kMaxRun >= 16)
      for (; c0 + 16 <= my1; c0 += 16) forward_run<16, EX, kBuf>(d, mars, issum, c0, bb, m, sum);
    if constexpr (kMaxRun == 8)
      for (; c0 + 8 <= my1; c0 += 8) forward_run<8, EX, kBuf>(d, mars, issum, c0, bb, m, sum);
    for (; c0 + 4 <= my1; c0 += 4) forward_run<4, EX, kBuf>(d, mars, issum, c0, bb, m, sum);
    for (; c0 < my1; ++c0) forward_run<1, EX, kBuf>(d, mars, issum, c0, bb, m, sum);
    if (e1 - e0 > per) {   // more than one share is in use (uniform over the workgroup)
#pragma unroll
      for (int x = 0; x < EX; ++x) { xm[wave][x][lane] = m[x]; xs[wave][x][lane] = sum[x]; }
      __syncthreads();
      if (wave) return;
#pragma unroll
      for (int x = 0; x < EX; ++x) {
        if (issum) {
          float mm = m[x];
#pragma unroll
          for (int w = 1; w < kLayerWaves; ++w) mm = fmaxf(mm, xm[w][x][lane]);
          float ss = 0.f;
#pragma unroll
          for (int w = 0; w < kLayerWaves; ++w) {
            const float mw = xm[w][x][lane];
            if (mw != -INFINITY) ss += xs[w][x][lane] * __expf(mw - mm);
          }
          m[x] = mm;
          sum[x] = mm == -INFINITY ? 1.f : ss;
        } else {
#pragma unroll
          for (int w = 1; w < kLayerWaves; ++w) m[x] += xm[w][x][lane];
        }
      }
    } else if (wave) {
      return;
    }
  }
#pragma unroll
  for (int x = 0; x < EX; ++x)
    if (b0 + 64 * x < d.Bp) d.mars[(size_t)n * d.Bp + b0 + 64 * x] = sum[x] == 1.f ? m[x] : m[x] + __logf(sum[x]);
}

// The input layer on categorical data when it holds thousands of nodes: a wave takes one input node through the whole
// batch, four examples a lane and request (a packed word of categories, four table entries, one 16-byte store) and
// four requests in flight, instead of the layer kernel's one wave per (node, 256 examples) with its three dependent
// round trips each (sixteen 192-variable K = 32 circuits as one, 1024 examples: 196 -> 135 us).
__global__ __launch_bounds__(256) void sparse_input_kernel(SparseDev d, int n0, int cnt) {
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * 4 + (int)(threadIdx.x >> 6);
  if (i >= cnt) return;
  const int n = uni(d.fwd_rec[n0 + i].x);
  const uchar4* xr4 = reinterpret_cast<const uchar4*>(d.xb + (size_t)uni(d.in_var[n]) * d.Bp);
  const int64_t off = d.in_off[n];
  const float* row = d.leaf + (((int64_t)uni((int)(off >> 32)) << 32) | (uint32_t)uni((int)off));
  float4* out = reinterpret_cast<float4*>(d.mars + (size_t)n * d.Bp);
  const int n4 = d.Bp / 4;   // (rows are padded to 64 examples, the padding holds categories like any other)
  constexpr int U = 4;
  for (int q0 = lane; q0 < n4; q0 += 64 * U) {
    uchar4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = xr4[min(q0 + 64 * u, n4 - 1)];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (q0 + 64 * u < n4) out[q0 + 64 * u] = make_float4(row[x[u].x], row[x[u].y], row[x[u].z], row[x[u].w]);
  }
}

// Sum over the 64 lanes of a wave, valid in every lane: butterflies inside rows of 16 lanes
// with data-parallel-primitive moves (lane ^ 1, lane ^ 2, mirror of 8, mirror of 16), then the
// four row sums through scalar registers.
__device__ __forceinline__ float wave_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                 0xf, 0xf, true));
  };
  v += dpp(v, std::integral_constant<int, 0xB1>{});    // quad_perm [1,0,3,2]
  v += dpp(v, std::integral_constant<int, 0x4E>{});    // quad_perm [2,3,0,1]
  v += dpp(v, std::integral_constant<int, 0x141>{});   // row_half_mirror
  v += dpp(v, std::integral_constant<int, 0x140>{});   // row_mirror
  const int iv = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
}

// The sums over the wave of U values at once (a run's edge flows): each of the first log2(U) pairings of lanes
// (lane ^ 32, lane ^ 16, mirror of 16, mirror of 8) adds partners and halves the values a lane carries -- one
// partner keeps the lower half of the values, the other the upper half -- and the remaining pairings add without
// halving, as wave_sum does.  Afterwards lane l holds the total of value (l >> kShift) & (U - 1), kShift =
// 6 - log2(U): about 40 instructions for 16 sums where one wave_sum per edge takes 190.
template <int U>
struct EdgeTotals {
  static_assert(U == 16 || U == 8 || U == 4, "runs of 16, 8 or 4 edges");
  static constexpr int kShift = U == 16 ? 2 : U == 8 ? 3 : 4;
  template <int CTRL>
  static __device__ __forceinline__ float dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
  }
  // lanes with `upper` keep b's sum over the pair, the others a's; CTRL names the pairing inside a row of 16
  template <int CTRL>
  static __device__ __forceinline__ float halve(float a, float b, bool upper) {
    const float keep = upper ? b : a, send = upper ? a : b;
    return keep + dpp<CTRL>(send);
  }
  static __device__ __forceinline__ float run(float (&v)[U], int lane) {
    float w8[U / 2];
#pragma unroll
    for (int i = 0; i < U / 2; ++i) {   // lane ^ 32
      const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, v[i]), __builtin_bit_cast(int, v[i + U / 2]), false, false);
      w8[i] = __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
    }
    float w4[U / 4];
#pragma unroll
    for (int i = 0; i < U / 4; ++i) {   // lane ^ 16
      const auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(int, w8[i]), __builtin_bit_cast(int, w8[i + U / 4]), false, false);
      w4[i] = __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
    }
    float t;
    if constexpr (U == 16) {
      const float a = halve<0x140>(w4[0], w4[2], lane & 8), b = halve<0x140>(w4[1], w4[3], lane & 8);   // row_mirror
      t = halve<0x141>(a, b, lane & 4);                                                                  // row_half_mirror
    } else if constexpr (U == 8) {
      t = halve<0x140>(w4[0], w4[1], lane & 8);
      t += dpp<0x141>(t);
    } else {
      t = w4[0];
      t += dpp<0x140>(t);
      t += dpp<0x141>(t);
    }
    t += dpp<0x4E>(t);   // quad_perm [2,3,0,1]
    t += dpp<0xB1>(t);   // quad_perm [1,0,3,2]
    return t;
  }
};

template <int U, int EX, bool kBuf, bool kTempered = false>
__device__ __forceinline__ void backward_run(const SparseDev& d, const Rows<kBuf>& mars, const Rows<kBuf>& flows, int c0,
                                             const int (&bb)[EX], const unsigned (&alive)[EX], float (&acc)[EX],
                                             float* __restrict__ edge_part) {
  const int zrow = (int)d.n_nodes;
  float fl[U][EX], ex[U][EX];
  int ies[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int4 rec = d.in_rec[c0 + u];   // one record per edge instead of a chain of four index fetches
    ies[u] = uni(rec.x);
    const int ry = uni(rec.y);
    const bool issum = ry >= 0;
    const int p = issum ? ry : ~ry;
    const int s = uni(rec.w), pr = uni(rec.z);    // (the row of zeros where the edge has no such operand)
    const int mrow = issum ? p : zrow;
    const float lp = uni(d.in_logp[c0 + u]);      // 0 on product edges
#pragma unroll
    for (int x = 0; x < EX; ++x) {
      fl[u][x] = keep_bits(flows.at(p, bb[x]), alive[x]);   // a lane past the padded batch repeats its last example
      ex[u][x] = mars.at(pr, bb[x]) + lp + mars.at(s, bb[x]) - mars.at(mrow, bb[x]);
      // tempered (src-jl/learning/flow.jl:259-262): the share to the power 1 / fscale over the node's sum of those
      if constexpr (kTempered) ex[u][x] = ex[u][x] * d.inv_f - d.norm[(size_t)mrow * d.Bp + bb[x]];
    }
  }
  float part[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    part[u] = 0.f;
#pragma unroll
    for (int x = 0; x < EX; ++x) {
      // (product edges carry exponent 0 and exp2(0) is 1; lanes between the batch and its padding carry flow 0
      // from the seeds on)
      float ef = fl[u][x] * __expf(ex[u][x]);
      // no flow stays no flow where the parent's value is -inf (an example of probability zero: -inf - -inf)
      if (ex[u][x] != ex[u][x]) ef = 0.f;
      acc[x] += ef;
      part[u] += ef;
    }
  }
  if (!edge_part) return;
  if constexpr (U >= 4 && U <= 16) {
    // all the run's sums at once; lane l ends up with the total of edge (l >> kShift) % U, whose record it reads itself
    const int lane = threadIdx.x & 63;
    const int mine = d.in_rec[c0 + ((lane >> EdgeTotals<U>::kShift) & (U - 1))].x;
    const float tot = EdgeTotals<U>::run(part, lane);
    if (!(lane & ((1 << EdgeTotals<U>::kShift) - 1)) && !(mine & 1)) edge_part[mine >> 1] = tot;   // this wave is the only writer of the cell
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (!(ies[u] & 1)) {
        const float tot = wave_sum(part[u]);
        if ((threadIdx.x & 63) == 0) edge_part[ies[u] >> 1] = tot;
      }
  }
}

// Backward, one layer (top-down): a workgroup takes one node and 64 * EX examples and adds up the
// flows of the node's incoming edges, src/queries/flow.jl:49-60: edge_flow = flows[parent]
// (product edge) or flows[parent] * exp(mars[prime] + logp (+ mars[sub]) - mars[parent]) (sum
// edge).  Each edge's flow is summed over the batch where the node is the edge's prime
// (:73-81): over the thread's examples, then over the wave; the wave's sum goes to row blockIdx.y of
// edge_part ([gridDim.y][n_edges]), whose rows a later kernel adds up in order.
template <int EX, int kLayerWaves, int kMaxRun, bool kBuf, bool kTempered = false>
__global__ __launch_bounds__(kLayerWaves * 64) void sparse_backward_kernel(SparseDev d, int n0,
                                                                           const float* __restrict__ seed,
                                                                           float* __restrict__ edge_part_all, int64_t n_edges,
                                                                           const int32_t* __restrict__ alias_list) {
  __shared__ float xa[kLayerWaves][EX][64];
  const int4 rec = d.bwd_rec[n0 + blockIdx.x];   // one fetch instead of order -> seed, in-edge range
  const int2 arec = d.bwd_alias[n0 + blockIdx.x];
  const int n = uni(rec.x);
  const int lane = threadIdx.x & 63, wave = uni((int)(threadIdx.x >> 6));
  const int b0 = blockIdx.y * (64 * EX) + lane;
  float* edge_part = edge_part_all ? edge_part_all + (size_t)blockIdx.y * n_edges : nullptr;
  int bb[EX];
  bool live[EX];
  unsigned alive[EX];   // all ones for the lanes inside the padded batch
  float acc[EX];
  const int sd = uni(rec.y);
#pragma unroll
  for (int x = 0; x < EX; ++x) {
    const int b = b0 + 64 * x;
    live[x] = b < d.B;
    alive[x] = b < d.Bp ? ~0u : 0u;
    bb[x] = min(b, d.Bp - 1);
    acc[x] = 0.f;
    if (sd >= 0 && wave == 0 && live[x]) acc[x] = seed ? seed[(size_t)sd * d.B + b] : 1.f;   // no flow past the batch
  }
  // the node's incoming edges in kLayerWaves contiguous shares, one per wave
  const int i0 = uni(rec.z), i1 = uni(rec.w);
  const int per = (i1 - i0 + kLayerWaves - 1) / kLayerWaves;
  const int my0 = min(i0 + wave * per, i1), my1 = min(my0 + per, i1);
  const Rows<kBuf> mars(d.mars, d.n_nodes + 1, d.Bp), flows(d.flows, d.n_flow_rows, d.Bp);
  int c0 = my0;
  if constexpr (kMaxRun >= 32)
    for (; c0 + 32 <= my1; c0 += 32) backward_run<32, EX, kBuf, kTempered>(d, mars, flows, c0, bb, alive, acc, edge_part);
  if constexpr (kMaxRun >= 16)
    for (; c0 + 16 <= my1; c0 += 16) backward_run<16, EX, kBuf, kTempered>(d, mars, flows, c0, bb, alive, acc, edge_part);
  if constexpr (kMaxRun == 8)
    for (; c0 + 8 <= my1; c0 += 8) backward_run<8, EX, kBuf, kTempered>(d, mars, flows, c0, bb, alive, acc, edge_part);
  for (; c0 + 4 <= my1; c0 += 4) backward_run<4, EX, kBuf, kTempered>(d, mars, flows, c0, bb, alive, acc, edge_part);
  for (; c0 < my1; ++c0) backward_run<1, EX, kBuf, kTempered>(d, mars, flows, c0, bb, alive, acc, edge_part);
  if (i1 - i0 > per) {   // more than one share is in use (uniform over the workgroup)
#pragma unroll
    for (int x = 0; x < EX; ++x) xa[wave][x][lane] = acc[x];
    __syncthreads();
    if (wave) return;
#pragma unroll
    for (int x = 0; x < EX; ++x)
#pragma unroll
      for (int w = 1; w < kLayerWaves; ++w) acc[x] += xa[w][x][lane];
  } else if (wave) {
    return;
  }
#pragma unroll
  for (int x = 0; x < EX; ++x) {
    const int b = b0 + 64 * x;
    if (b < d.Bp) d.flows[(size_t)n * d.Bp + b] = live[x] ? acc[x] : 0.f;
  }
  // input nodes that receive exactly this node's edge flows (the other factor of the same
  // two-child products) are not computed again: their rows are copies
  for (int q = uni(arec.x), q1 = uni(arec.y); q < q1; ++q) {
    const int t = uni(alias_list[q]);
#pragma unroll
    for (int x = 0; x < EX; ++x) {
      const int b = b0 + 64 * x;
      if (b < d.Bp) d.flows[(size_t)t * d.Bp + b] = live[x] ? acc[x] : 0.f;
    }
  }
}

// Leaf counters, src/nodes/fixable_categorical_dist.jl:121-130: an input node's flow goes to the
// counter of the example's category.  NT threads per input node over the whole batch -- a workgroup (NT = 256) where
// there are few nodes, a wave (NT = 64, four nodes per workgroup and no workgroup barrier: a wave's LDS operations
// execute in order) where there are thousands and a node's 1024 examples are four per thread: the node owns its C
// counters.  They are summed in LDS as 64-bit fixed-point integers, scaled so that the node's largest flow times the
// batch size still fits: integer sums do not depend on the order the lanes arrive in, so the counters come out the
// same on every run and under either NT.
template <int NT>
__global__ __launch_bounds__(256) void sparse_leaf_flow_kernel(SparseDev d, const int32_t* __restrict__ input_nodes,
                                                               int n_input_nodes, float* __restrict__ leaf_flow) {
  constexpr int G = 256 / NT;   // nodes per workgroup
  __shared__ unsigned long long hist_all[G][256];
  __shared__ float wave_max[4];
  const int grp = threadIdx.x / NT, t = threadIdx.x % NT;
  const int at = blockIdx.x * G + grp;
  if (at >= n_input_nodes) return;   // (NT = 64: a whole wave; NT = 256: never)
  unsigned long long* hist = hist_all[grp];
  const int n = input_nodes[at];
  for (int c = t; c < d.C; c += NT) hist[c] = 0ull;
  const uint8_t* xr = d.xb + (size_t)d.in_var[n] * d.Bp;
  const float* fr = d.flows + (size_t)n * d.Bp;
  // (rows are padded to whole 16-byte words; four words requested before the first is used: a loop of single
  // dependent loads made this kernel wait out sixteen memory latencies per node and pass)
  constexpr int U = 4;
  const float4* fr4 = reinterpret_cast<const float4*>(fr);
  const uchar4* xr4 = reinterpret_cast<const uchar4*>(xr);
  const int n4 = d.Bp / 4;
  float mx = 0.f;
  for (int q0 = t; q0 < n4; q0 += NT * U) {
    float4 f[U];
#pragma unroll
    for (int u = 0; u < U; ++u) f[u] = fr4[min(q0 + u * NT, n4 - 1)];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int b0 = (q0 + u * NT) * 4;   // (past the batch: not counted)
      if (b0 < d.B) mx = fmaxf(mx, f[u].x);
      if (b0 + 1 < d.B) mx = fmaxf(mx, f[u].y);
      if (b0 + 2 < d.B) mx = fmaxf(mx, f[u].z);
      if (b0 + 3 < d.B) mx = fmaxf(mx, f[u].w);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  if constexpr (NT == 256) {
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
  }
  if (!(mx > 0.f)) return;                       // no flow reached this node (uniform over the node's threads)
  int ex = 0;
  frexpf(mx, &ex);                               // every flow < 2^ex
  const int shift = 62 - (32 - __clz(d.B)) - ex; // flow * 2^shift < 2^62 / batch
  for (int q0 = t; q0 < n4; q0 += NT * U) {
    float4 f[U];
    uchar4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      f[u] = fr4[min(q0 + u * NT, n4 - 1)];
      x[u] = xr4[min(q0 + u * NT, n4 - 1)];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int b0 = (q0 + u * NT) * 4;
      if (b0 < d.B && f[u].x > 0.f) atomicAdd(&hist[x[u].x], (unsigned long long)ldexpf(f[u].x, shift));
      if (b0 + 1 < d.B && f[u].y > 0.f) atomicAdd(&hist[x[u].y], (unsigned long long)ldexpf(f[u].y, shift));
      if (b0 + 2 < d.B && f[u].z > 0.f) atomicAdd(&hist[x[u].z], (unsigned long long)ldexpf(f[u].z, shift));
      if (b0 + 3 < d.B && f[u].w > 0.f) atomicAdd(&hist[x[u].w], (unsigned long long)ldexpf(f[u].w, shift));
    }
  }
  if constexpr (NT == 256) __syncthreads();
  else __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  float* dst = leaf_flow + d.in_off[n];
  for (int c = t; c < d.C; c += NT) dst[c] += ldexpf((float)hist[c], -shift);
}

// Soft evidence, per variable.  All input nodes of a variable read the same evidence, so a
// workgroup stages a [64 examples][64 categories] tile of it in LDS once and every thread folds it
// into several nodes; the nodes' log-parameters (going up) and values / flows (going down) are
// uniform over a wave and come through the scalar cache.
constexpr int kSoftTile = 64;    // examples and categories per staged tile
constexpr int kSoftNodes = 16;   // nodes a thread carries at a time (x 4 waves = 64 nodes per round)

// Leaf values, src/regularization/reg_likelihood.jl:51-91: logsumexp_c(evidence_c + logp_c) as a
// running maximum and a sum of exponentials.  Workgroup = (variable, 64 examples); thread =
// (example, wave w): nodes w, w + 4, ... of the variable.
__global__ __launch_bounds__(256) void sparse_soft_input_kernel(SparseDev d, const int32_t* __restrict__ var_ptr,
                                                                const int32_t* __restrict__ var_nodes) {
  __shared__ float tile[kSoftTile][kSoftTile + 1];
  const int v = blockIdx.x, b0 = blockIdx.y * kSoftTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = var_ptr[v], nv = var_ptr[v + 1] - n0;
  for (int q0 = 0; q0 < nv; q0 += 4 * kSoftNodes) {
    float m[kSoftNodes], sm[kSoftNodes];
#pragma unroll
    for (int q = 0; q < kSoftNodes; ++q) { m[q] = -INFINITY; sm[q] = 0.f; }
    for (int c0 = 0; c0 < d.C; c0 += kSoftTile) {
      __syncthreads();
      for (int i = threadIdx.x; i < kSoftTile * kSoftTile; i += 256) {
        // the faster of the two strides goes to consecutive threads
        const int bi = d.ev_se <= d.ev_sc ? i % kSoftTile : i / kSoftTile, ci = d.ev_se <= d.ev_sc ? i / kSoftTile : i % kSoftTile;
        const int b = min(b0 + bi, d.B - 1), c = c0 + ci;
        tile[bi][ci] = c < d.C ? d.ev[(int64_t)(d.ev_idx ? d.ev_idx[b] : b) * d.ev_se + (int64_t)v * d.ev_sv + (int64_t)c * d.ev_sc]
                               : -INFINITY;
      }
      __syncthreads();
      const int nc = min(kSoftTile, d.C - c0);
#pragma unroll
      for (int q = 0; q < kSoftNodes; ++q) {
        const int qi = q0 + wave + 4 * q;
        if (qi >= nv) break;
        const float* lp = d.leaf + d.in_off[var_nodes[n0 + qi]] + c0;
        float mm = m[q], ss = sm[q];
        for (int c = 0; c < nc; ++c) {
          const float t = tile[lane][c] + lp[c];
          if (t > mm) { ss = ss * __expf(mm - t) + 1.f; mm = t; }
          else if (t != -INFINITY) ss += __expf(t - mm);
        }
        m[q] = mm; sm[q] = ss;
      }
    }
    if (b0 + lane < d.Bp)
#pragma unroll
      for (int q = 0; q < kSoftNodes; ++q) {
        const int qi = q0 + wave + 4 * q;
        if (qi >= nv) break;
        d.mars[(size_t)var_nodes[n0 + qi] * d.Bp + b0 + lane] = m[q] == -INFINITY ? m[q] : m[q] + __logf(sm[q]);
      }
  }
}

// Leaf counters, src/regularization/reg_flow.jl:50-82: category c of input node n receives
// sum_b flow[b] * exp(evidence[b][c] + logp_c - value[b]).  Workgroup = (variable, 64 categories,
// 16 of the variable's nodes); thread = (category, wave w): nodes w, w + 4, w + 8, w + 12 of the
// group; the batch goes by in tiles of 64 examples, with the nodes' values and flows beside the
// evidence tile in LDS.
constexpr int kFlowNodes = 4;   // nodes per thread; x 4 waves = 16 nodes per workgroup

__global__ __launch_bounds__(256) void sparse_leaf_flow_soft_kernel(SparseDev d, const int32_t* __restrict__ var_ptr,
                                                                    const int32_t* __restrict__ var_nodes,
                                                                    float* __restrict__ leaf_flow) {
  __shared__ float tile[kSoftTile][kSoftTile + 1];   // [example][category]
  __shared__ float vt[4 * kFlowNodes][kSoftTile], ft[4 * kFlowNodes][kSoftTile];
  const int v = blockIdx.x, c0 = blockIdx.y * kSoftTile, q0 = blockIdx.z * (4 * kFlowNodes);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = var_ptr[v], nv = var_ptr[v + 1] - n0;
  if (q0 >= nv) return;
  const int c = c0 + lane;
  float acc[kFlowNodes], lpc[kFlowNodes];
#pragma unroll
  for (int q = 0; q < kFlowNodes; ++q) {
    acc[q] = 0.f;
    const int qi = q0 + wave + 4 * q;
    lpc[q] = (qi < nv && c < d.C) ? d.leaf[d.in_off[var_nodes[n0 + qi]] + c] : -INFINITY;
  }
  for (int b0 = 0; b0 < d.B; b0 += kSoftTile) {
    __syncthreads();
    for (int i = threadIdx.x; i < kSoftTile * kSoftTile; i += 256) {
      const int bi = d.ev_se <= d.ev_sc ? i % kSoftTile : i / kSoftTile, ci = d.ev_se <= d.ev_sc ? i / kSoftTile : i % kSoftTile;
      const int b = b0 + bi, cc = c0 + ci;
      tile[bi][ci] = (b < d.B && cc < d.C)
                         ? d.ev[(int64_t)(d.ev_idx ? d.ev_idx[b] : b) * d.ev_se + (int64_t)v * d.ev_sv + (int64_t)cc * d.ev_sc]
                         : -INFINITY;
    }
    for (int i = threadIdx.x; i < 4 * kFlowNodes * kSoftTile; i += 256) {
      const int qi = q0 + i / kSoftTile, bi = i % kSoftTile;
      const bool ok = qi < nv && b0 + bi < d.B;
      const size_t at = ok ? (size_t)var_nodes[n0 + qi] * d.Bp + b0 + bi : 0;
      vt[i / kSoftTile][bi] = ok ? d.mars[at] : 0.f;
      ft[i / kSoftTile][bi] = ok ? d.flows[at] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kFlowNodes; ++q) {
      const int r = wave + 4 * q;
      float a = acc[q];
#pragma unroll 8
      for (int b = 0; b < kSoftTile; ++b) {
        const float t = tile[b][lane] + lpc[q], f = ft[r][b];
        if (t != -INFINITY && f != 0.f) a += __expf(t - vt[r][b]) * f;
      }
      acc[q] = a;
    }
  }
  if (c < d.C)
#pragma unroll
    for (int q = 0; q < kFlowNodes; ++q) {
      const int qi = q0 + wave + 4 * q;
      if (qi < nv) leaf_flow[d.in_off[var_nodes[n0 + qi]] + c] += acc[q];
    }
}

// (a record that names a dense group's row behind the node rows is not an edge: its flow is taken as it is)
__global__ void sparse_gather_in_logp_kernel(const int4* __restrict__ in_rec, const float* __restrict__ logp, int64_t n,
                                             int64_t n_nodes, float* __restrict__ in_logp) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int4 r = in_rec[i];
  in_logp[i] = (r.y < 0 && (int64_t)~r.y >= n_nodes) ? 0.f : logp[r.x >> 1];
}

__global__ void sparse_scale_kernel(float* p, int64_t n, float rate) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = rate != 0.f ? p[i] * rate : 0.f;
}

// EM update, one wave per node (lanes over the node's edges / categories): add_pseudocount,
// aggr_node_flows, update_params (src/pretrain/mini_batch_warmup.jl:4-17, :54-70 without the 1e-8
// guards) and the leaf update (src/nodes/fixable_categorical_dist.jl:223-248, missing_flow = 0).
__global__ __launch_bounds__(256) void sparse_update_kernel(SparseDev d, int n_nodes, float* __restrict__ logp,
                                                            float* __restrict__ leaf, float* __restrict__ edge_aggr,
                                                            const float* __restrict__ leaf_flow, float pseudocount,
                                                            float inertia) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= n_nodes) return;
  const int type = d.type[n];
  if (type == kSum) {
    const int e0 = d.node_e0[n], e1 = d.node_e1[n];
    const float share = pseudocount / (float)(e1 - e0);
    float tot = 0.f;
    for (int e = e0 + lane; e < e1; e += 64) { edge_aggr[e] += share; tot += edge_aggr[e]; }
    tot = wave_sum(tot);
    if (e1 - e0 == 1) return;
    for (int e = e0 + lane; e < e1; e += 64)
      logp[e] = logf(inertia * expf(logp[e]) + (1.f - inertia) * edge_aggr[e] / tot);
  } else if (type == kInput) {
    float* lp = leaf + d.in_off[n];
    const float* fl = leaf_flow + d.in_off[n];
    const float cat_pc = pseudocount / (float)d.C;
    if ((d.C & 3) == 0 && d.C <= 256) {
      // a node's row as one 16-byte word per lane, the parameters requested together with the flows: the loops below
      // are a chain of a dozen dependent round trips per node, and a circuit has a hundred thousand of these nodes
      const int c = 4 * lane;
      float4 f = make_float4(0.f, 0.f, 0.f, 0.f), l = f;
      if (c < d.C) {
        f = *reinterpret_cast<const float4*>(fl + c);
        l = *reinterpret_cast<const float4*>(lp + c);
      }
      const float node_flow = wave_sum((f.x + f.y) + (f.z + f.w)) + pseudocount;
      if (c < d.C)
        *reinterpret_cast<float4*>(lp + c) = make_float4(logf(inertia * expf(l.x) + (1.f - inertia) * (f.x + cat_pc) / node_flow),
                                                         logf(inertia * expf(l.y) + (1.f - inertia) * (f.y + cat_pc) / node_flow),
                                                         logf(inertia * expf(l.z) + (1.f - inertia) * (f.z + cat_pc) / node_flow),
                                                         logf(inertia * expf(l.w) + (1.f - inertia) * (f.w + cat_pc) / node_flow));
      return;
    }
    float node_flow = 0.f;
    for (int c = lane; c < d.C; c += 64) node_flow += fl[c];
    node_flow = wave_sum(node_flow) + pseudocount;
    for (int c = lane; c < d.C; c += 64)
      lp[c] = logf(inertia * expf(lp[c]) + (1.f - inertia) * (fl[c] + cat_pc) / node_flow);
  }
}

// KL recursion, one layer, one thread per node: src/queries/kld.jl:95-128 and the leaf term
// of src/nodes/fixable_categorical_dist.jl:187-192 (log-parameter form).
__global__ void sparse_kld_up_kernel(SparseDev d, int n0, int n1, const float* __restrict__ logp2,
                                     const float* __restrict__ leaf2, float* __restrict__ klds,
                                     float* __restrict__ edge_klds) {
  const int i = n0 + blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n1) return;
  const int n = d.order[i];
  float acc = 0.f;
  if (d.type[n] == kInput) {
    for (int c = 0; c < d.C; ++c) {
      const float a = d.leaf[d.in_off[n] + c], q = leaf2[d.in_off[n] + c];
      acc += expf(a) * (a - q);
    }
  } else {
    for (int e = d.node_e0[n]; e < d.node_e1[n]; ++e) {
      float k = klds[d.e_prime[e]];
      if (d.e_sub[e] >= 0) k += klds[d.e_sub[e]];
      if (d.type[n] == kSum) k = expf(d.logp[e]) * (k + d.logp[e] - logp2[e]);
      edge_klds[e] = k;
      acc = e == d.node_e0[n] ? k : acc + k;
    }
  }
  klds[n] = acc;
}

// Reverse pass of the KL recursion, node gradients of one layer (top-down):
// src/queries/kld.jl:262-300: a child receives g_parent * exp(p1) over a sum edge,
// g_parent over a product edge.
__global__ void sparse_kld_down_kernel(SparseDev d, int n0, int n1, int root, float* __restrict__ grads) {
  const int i = n0 + blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n1) return;
  const int n = d.order[i];
  float acc = n == root ? 1.f : 0.f;
  for (int q = d.in_ptr[n]; q < d.in_ptr[n + 1]; ++q) {
    const int e = d.in_edge[q] >> 1;
    const int p = d.e_parent[e];
    acc += grads[p] * (d.type[p] == kSum ? expf(d.logp[e]) : 1.f);
  }
  grads[n] = acc;
}

// Edge and leaf gradients, src/queries/kld.jl:271-272 and, written as the source has them,
// src/nodes/fixable_categorical_dist.jl:219.
__global__ void sparse_kld_edge_grad_kernel(SparseDev d, int64_t n_edges, const float* __restrict__ grads,
                                            const float* __restrict__ edge_klds, float* __restrict__ g1,
                                            float* __restrict__ g2) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n_edges) return;
  const int p = d.e_parent[e];
  if (d.type[p] == kSum) {
    const float g = grads[p], p1 = expf(d.logp[e]);
    g1[e] = g * (edge_klds[e] + p1);
    g2[e] = -g * p1;
  } else {
    g1[e] = 0.f;
    g2[e] = 0.f;
  }
}

__global__ void sparse_kld_leaf_grad_kernel(SparseDev d, const int32_t* __restrict__ input_nodes, int n_inputs,
                                            const float* __restrict__ leaf2, const float* __restrict__ grads,
                                            float* __restrict__ g1, float* __restrict__ g2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)n_inputs * d.C) return;
  const int n = input_nodes[i / d.C];
  const float g = grads[n], a = d.leaf[i], q = leaf2[i];
  g1[i] = g * (a - q + 1.f);
  g2[i] = g * expf(a - q);
}

// Gumbel-max sampling, one layer (top-down), thread = (node, example): a visited sum node
// keeps the edge maximising logp + noise (first maximum wins), a visited product visits all
// its edges, a visited input emits argmax_c(logp_c + noise_c).
__global__ void sparse_sample_kernel(SparseDev d, int n0, const int32_t* __restrict__ noise_slot,
                                     const int64_t* __restrict__ edge2param, int64_t noise_stride,
                                     const float* __restrict__ node_noise, const float* __restrict__ leaf_noise,
                                     int V, uint8_t* __restrict__ visit, uint8_t* __restrict__ out) {
  const int n = d.order[n0 + blockIdx.x];
  const int b = blockIdx.y * blockDim.x + threadIdx.x;
  if (b >= d.B || !visit[(size_t)n * d.Bp + b]) return;
  if (d.type[n] == kInput) {
    const float* lp = d.leaf + d.in_off[n];
    const float* g = leaf_noise + ((size_t)b * V + d.in_var[n]) * d.C;
    int best = 0;
    float bv = lp[0] + g[0];
    for (int c = 1; c < d.C; ++c) {
      const float v = lp[c] + g[c];
      if (v > bv) { bv = v; best = c; }
    }
    out[(size_t)b * V + d.in_var[n]] = (uint8_t)best;
  } else if (d.type[n] == kSum) {
    const float* en = node_noise + (size_t)b * noise_stride;
    const int e0 = d.node_e0[n], e1 = d.node_e1[n];
    int best = e0;
    float bv = -INFINITY;
    for (int e = e0; e < e1; ++e) {
      const int64_t slot = noise_slot ? noise_slot[e] : edge2param[e] - 1;
      const float v = d.logp[e] + en[slot];
      if (e == e0 || v > bv) { bv = v; best = e; }
    }
    visit[(size_t)d.e_prime[best] * d.Bp + b] = 1;
    if (d.e_sub[best] >= 0) visit[(size_t)d.e_sub[best] * d.Bp + b] = 1;
  } else {
    for (int e = d.node_e0[n]; e < d.node_e1[n]; ++e) {
      visit[(size_t)d.e_prime[e] * d.Bp + b] = 1;
      if (d.e_sub[e] >= 0) visit[(size_t)d.e_sub[e] * d.Bp + b] = 1;
    }
  }
}

// Relaxed (Gumbel-softmax) sampling at temperature T, src/queries/sample.jl:8-148.  Pass 1,
// thread = (sum node, example): the normaliser of the node's edge weights exp((logp + g)/T)
// (sample.jl:37-51), kept as (max, sum of exp relative to the max) so that small temperatures
// cannot overflow -- after normalisation identical to the reference's plain sum.
__global__ void sparse_soft_norm_kernel(SparseDev d, int n_nodes, const int32_t* __restrict__ noise_slot,
                                        const int64_t* __restrict__ edge2param, int64_t noise_stride,
                                        const float* __restrict__ noise, float inv_t, float* __restrict__ emax,
                                        float* __restrict__ esum) {
  const int n = blockIdx.x;
  const int b = blockIdx.y * blockDim.x + threadIdx.x;
  if (n >= n_nodes || b >= d.B || d.type[n] != kSum) return;
  const float* g = noise ? noise + (size_t)b * noise_stride : nullptr;
  float m = -INFINITY;
  for (int e = d.node_e0[n]; e < d.node_e1[n]; ++e) {
    const float v = (d.logp[e] + (g ? g[noise_slot ? noise_slot[e] : edge2param[e] - 1] : 0.f)) * inv_t;
    m = fmaxf(m, v);
  }
  float s = 0.f;
  for (int e = d.node_e0[n]; e < d.node_e1[n]; ++e) {
    const float v = (d.logp[e] + (g ? g[noise_slot ? noise_slot[e] : edge2param[e] - 1] : 0.f)) * inv_t;
    s += expf(v - m);
  }
  emax[(size_t)n * d.Bp + b] = m;
  esum[(size_t)n * d.Bp + b] = s;
}

// Pass 2, one layer top-down, thread = (node, example): top-down probability gathered over
// the incoming edges (sample.jl:105-140): a sum edge hands on td[parent] * w / normaliser, a
// product edge td[parent], to prime and sub alike.
__global__ void sparse_soft_down_kernel(SparseDev d, int n0, int root, const int32_t* __restrict__ noise_slot,
                                        const int64_t* __restrict__ edge2param, int64_t noise_stride,
                                        const float* __restrict__ noise, float inv_t, const float* __restrict__ emax,
                                        const float* __restrict__ esum, float* __restrict__ td) {
  const int n = d.order[n0 + blockIdx.x];
  const int b = blockIdx.y * blockDim.x + threadIdx.x;
  if (b >= d.B) return;
  const float* g = noise ? noise + (size_t)b * noise_stride : nullptr;
  float acc = n == root ? 1.f : 0.f;
  for (int i = d.in_ptr[n]; i < d.in_ptr[n + 1]; ++i) {
    const int e = d.in_edge[i] >> 1;
    const int p = d.e_parent[e];
    float f = td[(size_t)p * d.Bp + b];
    if (d.type[p] == kSum) {
      const float v = (d.logp[e] + (g ? g[noise_slot ? noise_slot[e] : edge2param[e] - 1] : 0.f)) * inv_t;
      f *= expf(v - emax[(size_t)p * d.Bp + b]) / esum[(size_t)p * d.Bp + b];
    }
    acc += f;
  }
  td[(size_t)n * d.Bp + b] = acc;
}

// Pass 3, thread = (variable, example, category): out[b][v][c] = sum over the variable's input
// nodes of td * exp(leaf_logp[c]) (sample.jl:262-284).
__global__ void sparse_soft_leaf_kernel(SparseDev d, const int32_t* __restrict__ var_ptr,
                                        const int32_t* __restrict__ var_nodes, int V, const float* __restrict__ td,
                                        float* __restrict__ out) {
  const int v = blockIdx.x, b = blockIdx.y;
  for (int c = threadIdx.x; c < d.C; c += blockDim.x) {
    float acc = 0.f;
    for (int i = var_ptr[v]; i < var_ptr[v + 1]; ++i) {
      const int n = var_nodes[i];
      acc += td[(size_t)n * d.Bp + b] * expf(d.leaf[d.in_off[n] + c]);
    }
    out[((size_t)b * V + v) * d.C + c] = acc;
  }
}

// Adam on the sum parameters: src/sgd/adam.jl:318-319 (moments), :63-76 (ascent step).
__global__ void sparse_adam_kernel(int64_t n, const float* __restrict__ grad, float* __restrict__ params,
                                   float* __restrict__ m, float* __restrict__ v, float lr, float b1, float b2,
                                   float eps, float c1, float c2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float g = grad[i];
  m[i] = b1 * m[i] + (1.f - b1) * g;
  v[i] = b2 * v[i] + (1.f - b2) * g * g;
  params[i] += lr * ((m[i] / c1) / (sqrtf(v[i] / c2) + eps));
}

// Per-sum-node normalisation into the circuit: src/sgd/adam.jl:88-127.
__global__ void sparse_normalize_kernel(int n_groups, const int32_t* __restrict__ group_ptr,
                                        const int32_t* __restrict__ param2edge, const float* __restrict__ params,
                                        float* __restrict__ logp) {
  const int gi = blockIdx.x * blockDim.x + threadIdx.x;
  if (gi >= n_groups) return;
  const int p0 = group_ptr[gi], p1 = group_ptr[gi + 1];
  if (p1 - p0 == 1) return;
  float s = 0.f;
  for (int p = p0; p < p1; ++p) s += expf(params[p]);
  const float l = logf(s);
  for (int p = p0; p < p1; ++p) logp[param2edge[p]] = params[p] - l;
}

__global__ void sparse_fill_u8_kernel(uint8_t* p, int64_t n, uint8_t v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ void sparse_set_row_u8_kernel(uint8_t* p, int B, uint8_t v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < B) p[i] = v;
}

__global__ void sparse_copy_rows_kernel(const float* __restrict__ mars, int Bp, int B, const int32_t* __restrict__ nodes,
                                        int n_rows, float* __restrict__ out) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  const int r = blockIdx.y;
  if (b < B && r < n_rows) out[(size_t)r * B + b] = mars[(size_t)nodes[r] * Bp + b];
}

// Mask-weighted mixture over the heads, src-jl/multi_head_pc/likelihood.jl:3-12:
// ll = logsumexp_h(mars[head_h] + log mask[h]) - log sum_h mask[h], folded head by head
// from -inf with the pairwise logsumexp.
constexpr int kMixGroups = 16;   // head groups per example in the mixture kernel

// workgroup = 64 examples x kMixGroups head groups: running maximum and sum per thread, combined through LDS
__global__ __launch_bounds__(64 * kMixGroups) void sparse_head_mixture_kernel(const float* __restrict__ mars, int Bp, int B,
                                                                              const int32_t* __restrict__ heads, int n_heads,
                                                                              const float* __restrict__ mask,
                                                                              float* __restrict__ out) {
  __shared__ float pm[kMixGroups][64], ps[kMixGroups][64], pt[kMixGroups][64];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int b = blockIdx.x * 64 + lane;
  float mx = -INFINITY, sm = 0.f, tot = 0.f;
  if (b < B)
    for (int h0 = g; h0 < n_heads; h0 += kMixGroups * 4) {   // four heads' requests before the first is folded in
      float m4[4], v4[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int h = min(h0 + u * kMixGroups, n_heads - 1);
        m4[u] = mask[(size_t)h * B + b];
        v4[u] = mars[(size_t)heads[h] * Bp + b];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (h0 + u * kMixGroups >= n_heads) break;
        const float m = m4[u];
        const float t = v4[u] + logf(m);
        tot += m;
        if (t > mx) { sm = sm * expf(mx - t) + 1.f; mx = t; }
        else if (t > -INFINITY) sm += expf(t - mx);
      }
    }
  pm[g][lane] = mx; ps[g][lane] = sm; pt[g][lane] = tot;
  __syncthreads();
  if (g || b >= B) return;
  float M = -INFINITY, T = 0.f, S = 0.f;
  for (int q = 0; q < kMixGroups; ++q) { M = fmaxf(M, pm[q][lane]); T += pt[q][lane]; }
  for (int q = 0; q < kMixGroups; ++q)
    if (pm[q][lane] > -INFINITY) S += ps[q][lane] * expf(pm[q][lane] - M);
  out[b] = M + logf(S) - logf(T);
}

// Tempered flows, scale_flows_kernel of src-jl/learning/flow.jl:120-175: per sum node and example the logarithm of the
// sum over the node's edges of exp((value of the edge's children + log-parameter - value of the node) / fscale); 0 for
// every other node and for the row of zeros behind the last node.  thread = (node, example)
__global__ __launch_bounds__(256) void sparse_tempered_norm_kernel(SparseDev d, float* __restrict__ norm) {
  const int64_t n = blockIdx.x;
  const int b = blockIdx.y * 256 + threadIdx.x;
  if (b >= d.Bp) return;
  float out = 0.f;
  if (n < d.n_nodes && d.type[n] == kSum) {
    const float v = d.mars[n * d.Bp + b];
    float mx = -INFINITY, s = 0.f;
    for (int e = d.node_e0[n]; e < d.node_e1[n]; ++e) {
      float t = d.mars[(int64_t)d.e_prime[e] * d.Bp + b] + d.logp[e];
      if (d.e_sub[e] >= 0) t += d.mars[(int64_t)d.e_sub[e] * d.Bp + b];
      t = (t - v) * d.inv_f;
      if (!(t > -INFINITY)) continue;   // (also an example of probability zero: -inf - -inf)
      if (t > mx) { s = s * __expf(mx - t) + 1.f; mx = t; }
      else s += __expf(t - mx);
    }
    if (s > 0.f) out = mx + __logf(s);
  }
  norm[n * d.Bp + b] = out;
}

// Edge flows of product edges whose child takes its flow from a group's kernel instead of a layer's: the edge's flow
// is its parent's, summed over each block of 64 examples into the block's row of partial sums.  One wave per
// (edge, block).
__global__ __launch_bounds__(256) void sparse_product_edge_kernel(const int2* __restrict__ pairs, int n_pairs,
                                                                  const float* __restrict__ flows, int Bp,
                                                                  float* __restrict__ edge_part, int64_t n_edges) {
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (i >= n_pairs) return;
  const int2 pe = pairs[i];
  const float tot = wave_sum(flows[(size_t)pe.y * Bp + (size_t)blockIdx.y * 64 + lane]);
  if (lane == 0) edge_part[(size_t)blockIdx.y * n_edges + pe.x] = tot;
}

// ---------------------------------------------------------------------------------------
// host
// ---------------------------------------------------------------------------------------

// Dense groups: sum nodes of one layer over one and the same set of (prime, sub) children (each may list them in an
// order of its own), at least kGroupMinSide sums over at least kGroupMinSide children and at most kGroupMaxSide of
// either (more sums: several groups over the same children).  group_of[node] = group or -1; edge_slot[edge] = the
// child's number among all groups' children (its "slot") for the edges of a group's first sum, -1 for all others.
// PCMI355_DENSE_GROUPS=0 in the environment keeps every node on the layer kernels (for comparisons).
constexpr int kGroupMinSide = 4, kGroupMinEdges = 64, kGroupMaxSide = 128;
static_assert(sizeof(GroupRec) == 2 * sizeof(int4), "a group's record is uploaded as two int4");

void SparseCircuit::build_groups(std::vector<int32_t>& group_of, std::vector<int32_t>& edge_slot) {
  const int64_t nn = fc_.n_nodes();
  const char* env = std::getenv("PCMI355_DENSE_GROUPS");
  std::vector<int32_t> g_node, g_edge, g_prime;
  struct Found { int layer; std::vector<int32_t> nodes; };
  std::vector<Found> found;
  // a sum's edges ordered by (prime, sub): the order of a group's children
  auto sorted_edges = [&](int32_t n) {
    std::vector<int32_t> es(fc_.node_e1[n] - fc_.node_e0[n]);
    for (size_t i = 0; i < es.size(); ++i) es[i] = fc_.node_e0[n] + (int32_t)i;
    std::sort(es.begin(), es.end(), [&](int32_t a, int32_t b) {
      return std::make_tuple(fc_.e_prime[a], fc_.e_sub[a], a) < std::make_tuple(fc_.e_prime[b], fc_.e_sub[b], b);
    });
    return es;
  };
  if (!(env && env[0] == '0')) {
    // candidates by (layer, number of children, hash of the children), then compared child by child
    std::unordered_map<uint64_t, std::vector<int32_t>> buckets;
    for (int64_t n = 0; n < nn; ++n) {
      const int c = fc_.node_e1[n] - fc_.node_e0[n];
      if (fc_.type[n] != kSum || c < kGroupMinSide || c > kGroupMaxSide) continue;
      uint64_t h = 1469598103934665603ull ^ (uint64_t)fc_.layer[n];
      for (int32_t e : sorted_edges((int32_t)n)) {
        h = (h ^ (uint64_t)(uint32_t)fc_.e_prime[e]) * 1099511628211ull;
        h = (h ^ (uint64_t)(uint32_t)fc_.e_sub[e]) * 1099511628211ull;
      }
      buckets[h].push_back((int32_t)n);
    }
    auto same_children = [&](int32_t a, int32_t b) {
      if (fc_.layer[a] != fc_.layer[b] || fc_.node_e1[b] - fc_.node_e0[b] != fc_.node_e1[a] - fc_.node_e0[a]) return false;
      const std::vector<int32_t> ea = sorted_edges(a), eb = sorted_edges(b);
      for (size_t i = 0; i < ea.size(); ++i)
        if (fc_.e_prime[ea[i]] != fc_.e_prime[eb[i]] || fc_.e_sub[ea[i]] != fc_.e_sub[eb[i]]) return false;
      return true;
    };
    std::vector<uint64_t> keys;
    for (auto& kv : buckets) keys.push_back(kv.first);
    std::sort(keys.begin(), keys.end());   // (an order that does not depend on the hash table's)
    for (uint64_t k : keys) {
      std::vector<int32_t>& cand = buckets[k];   // ascending node ids
      std::vector<char> used(cand.size(), 0);
      for (size_t i = 0; i < cand.size(); ++i) {
        if (used[i]) continue;
        std::vector<int32_t> members{cand[i]};
        for (size_t j = i + 1; j < cand.size(); ++j)
          if (!used[j] && same_children(cand[i], cand[j])) { members.push_back(cand[j]); used[j] = 1; }
        const int c = fc_.node_e1[cand[i]] - fc_.node_e0[cand[i]];
        for (size_t m0 = 0; m0 < members.size(); m0 += kGroupMaxSide) {
          const size_t g = std::min<size_t>(kGroupMaxSide, members.size() - m0);
          if ((int)g < kGroupMinSide || (int64_t)g * c < kGroupMinEdges) continue;
          found.push_back(Found{fc_.layer[cand[i]], std::vector<int32_t>(members.begin() + m0, members.begin() + m0 + g)});
        }
      }
    }
  }
  auto tiles = [](int x) { int t = 1; while (t * 16 < x) t *= 2; return t; };   // 16-row tiles, a power of two of them
  std::sort(found.begin(), found.end(), [&](const Found& a, const Found& b) {
    const int ca = fc_.node_e1[a.nodes[0]] - fc_.node_e0[a.nodes[0]], cb = fc_.node_e1[b.nodes[0]] - fc_.node_e0[b.nodes[0]];
    const auto ka = std::make_tuple(a.layer, tiles((int)a.nodes.size()), tiles(ca), a.nodes[0]);
    const auto kb = std::make_tuple(b.layer, tiles((int)b.nodes.size()), tiles(cb), b.nodes[0]);
    return ka < kb;
  });
  for (size_t gi = 0; gi < found.size(); ++gi)
    for (int32_t n : found[gi].nodes) group_of[n] = (int32_t)gi;
  // A product of at most three factors that only groups use, as the prime of a child, is computed by those groups
  // (every one of them writes its value; the values are the same).
  grp_expanded_.assign(nn, 0);
  if (!found.empty()) {
    std::vector<char> used_by_group(nn, 0), used_otherwise(nn, 0);
    for (int64_t e = 0; e < fc_.n_edges(); ++e) {
      const int32_t p = fc_.e_parent[e], pr = fc_.e_prime[e], sb = fc_.e_sub[e];
      (group_of[p] >= 0 ? used_by_group : used_otherwise)[pr] = 1;
      if (sb >= 0) used_otherwise[sb] = 1;
    }
    for (int32_t hd : fc_.heads) used_otherwise[hd] = 1;
    used_otherwise[nn - 1] = 1;
    for (int64_t n = 0; n < nn; ++n) {
      if (fc_.type[n] != kMul || !used_by_group[n] || used_otherwise[n]) continue;
      int factors = 0;
      for (int e = fc_.node_e0[n]; e < fc_.node_e1[n]; ++e) factors += 1 + (fc_.e_sub[e] >= 0);
      grp_expanded_[n] = factors <= 3;
    }
  }
  // the device tables, padded to the tiles: Gp entries of sums and Cp of children per group, Gp x Cp of W
  std::vector<int4> g_rows, dev_recs;
  std::vector<int32_t> g_own, elem, shape_gt, shape_ct;
  group_launches_.clear();
  group_stat_launches_.clear();
  grp_pslot_h_.clear();
  const int32_t zrow = (int32_t)nn;
  int32_t n_slots = 0;
  for (size_t gi = 0; gi < found.size(); ++gi) {
    const Found& f = found[gi];
    const std::vector<int32_t> first = sorted_edges(f.nodes[0]);
    const int32_t c = (int32_t)first.size(), gn = (int32_t)f.nodes.size();
    const int gt = tiles(gn), ct = tiles(c);
    shape_gt.push_back(gt);
    shape_ct.push_back(ct);
    const int32_t pnode0 = (int32_t)g_node.size(), pslot0 = (int32_t)g_rows.size();
    const int64_t pw0 = (int64_t)elem.size();
    dev_recs.push_back(int4{gn, c, pnode0, pslot0});
    dev_recs.push_back(int4{(int32_t)(pw0 & 0xffffffff), (int32_t)(pw0 >> 32), gt, ct});
    elem.insert(elem.end(), (size_t)gt * 16 * ct * 16, (int32_t)gi);
    for (int i = 0; i < gt * 16; ++i) {
      g_node.push_back(i < gn ? f.nodes[i] : -1);
      std::vector<int32_t> es;
      if (i < gn) es = sorted_edges(f.nodes[i]);
      for (int k = 0; k < ct * 16; ++k) g_edge.push_back(i < gn && k < c ? es[k] : -1);
    }
    for (int i = 0; i < ct * 16; ++i) {
      if (i >= c) { g_rows.push_back(int4{zrow, zrow, zrow, zrow}); g_own.push_back(-2); continue; }
      const int32_t pr = fc_.e_prime[first[i]], sb = fc_.e_sub[first[i]];
      edge_slot[first[i]] = n_slots + i;
      g_prime.push_back(pr);
      grp_pslot_h_.push_back(pslot0 + i);
      int32_t r[3] = {pr, zrow, zrow};   // (the row of zeros)
      if (grp_expanded_[pr]) {
        int k = 0;
        for (int e = fc_.node_e0[pr]; e < fc_.node_e1[pr]; ++e) {
          r[k++] = fc_.e_prime[e];
          if (fc_.e_sub[e] >= 0) r[k++] = fc_.e_sub[e];
        }
      }
      g_rows.push_back(int4{r[0], r[1], r[2], sb >= 0 ? sb : zrow});
      g_own.push_back(grp_expanded_[pr] ? pr : -1);
    }
    n_slots += c;
    if (!group_launches_.empty() && group_launches_.back().layer == f.layer && group_launches_.back().gt == gt &&
        group_launches_.back().ct == ct)
      group_launches_.back().count++;
    else
      group_launches_.push_back(GroupLaunch{f.layer, (int)gi, 1, gt, ct, pnode0, pslot0, pw0});
  }
  n_group_slots_ = n_slots;
  n_groups_ = (int64_t)found.size();
  grp_prime_h_ = g_prime;
  if (found.empty()) return;
  {   // the groups by shape, for the launches that take all layers at once
    std::vector<int32_t> by_shape(found.size());
    for (size_t gi = 0; gi < found.size(); ++gi) by_shape[gi] = (int32_t)gi;
    auto shape = [&](int32_t gi) { return std::make_pair(shape_gt[gi], shape_ct[gi]); };
    std::stable_sort(by_shape.begin(), by_shape.end(), [&](int32_t a, int32_t b) { return shape(a) < shape(b); });
    for (size_t i = 0; i < by_shape.size(); ++i) {
      const auto s = shape(by_shape[i]);
      if (!group_stat_launches_.empty() && group_stat_launches_.back().gt == s.first && group_stat_launches_.back().ct == s.second)
        group_stat_launches_.back().count++;
      else
        group_stat_launches_.push_back(GroupLaunch{-1, (int)i, 1, s.first, s.second, 0, 0, 0});
    }
    d_grp_order_.upload(by_shape);
  }
  n_group_elems_ = (int64_t)elem.size();
  d_grp_elem_.upload(elem);
  d_grp_wf_.alloc(elem.size());
  d_grp_wb_.alloc(elem.size());
  d_grp_rec_.upload(dev_recs);
  d_grp_node_.upload(g_node);
  d_grp_edge_.upload(g_edge);
  d_grp_rows_.upload(g_rows);
  d_grp_own_.upload(g_own);
}

#define PCM_GROUP_DEV(g, batch_, bp_)                                                                                 \
  GroupDev g{};                                                                                                      \
  g.rec = reinterpret_cast<const GroupRec*>(d_grp_rec_.p);                                                           \
  g.node = d_grp_node_.p; g.edge = d_grp_edge_.p;   g.rows = d_grp_rows_.p; g.own = d_grp_own_.p;                    \
  g.copies = d_grp_copies_.p; g.order = d_grp_order_.p; g.wf = d_grp_wf_.p; g.wb = d_grp_wb_.p; g.m = d_grp_m_.p;       \
  g.xm = d_grp_xm_.p;                                                                                                \
  g.logp = d_logp_.p; g.mars = d_mars_.p; g.flows = d_flows_.p; g.edge_part = d_edge_part_.p;                        \
  g.n_nodes = fc_.n_nodes(); g.n_edges = fc_.n_edges(); g.B = batch_; g.Bp = bp_;                                   \
  g.inv_f = 1.f; g.norm = d_mars_.p; g.norm_row = fc_.n_nodes()   /* (not tempered: the row of zeros for every sum) */

// exp of the groups' log-parameters, before a forward pass
void SparseCircuit::refresh_group_w(float inv_f) {
  if (n_group_elems_ == 0) return;
  PCM_GROUP_DEV(g, 0, 0);
  g.inv_f = inv_f;
  hipLaunchKernelGGL(sparse_group_w_kernel, dim3((unsigned)ceil_div(n_group_elems_, 256)), dim3(256), 0, stream, g, d_grp_elem_.p,
                     n_group_elems_);
}

// Runs of consecutive layers that hold groups of one shape and no node of the layer kernels: one walk launch each
// (sparse_group_walk_kernel) instead of a launch per layer, where a layer's groups are few.  Going up and going down have
// runs of their own: a node the layer kernels compute going up may take its flow from a group's kernel going down.
// PCMI355_GROUP_WALK=0 in the environment when the circuit is created keeps the launch per layer (for comparisons).
void SparseCircuit::build_group_runs() {
  group_runs_fwd_.clear();
  group_runs_bwd_.clear();
  n_walk_levels_ = 0;
  const char* env = std::getenv("PCMI355_GROUP_WALK");
  if (group_launches_.empty() || (env && env[0] == '0')) return;
  std::vector<int2> levels;
  auto collect = [&](const std::vector<int>& layer0, std::vector<GroupRun>& runs) {
    // per layer: the one launch of its groups (-1: none, -2: several shapes)
    std::vector<int> of_layer(n_layers_, -1);
    for (size_t i = 0; i < group_launches_.size(); ++i) {
      int& slot = of_layer[group_launches_[i].layer];
      slot = slot == -1 ? (int)i : -2;
    }
    GroupRun cur{};
    bool open = false;
    auto close = [&]() {
      if (open && cur.n_levels >= 2) runs.push_back(cur);
      open = false;
    };
    for (int l = 0; l < n_layers_; ++l) {
      const bool plain_nodes = layer0[l + 1] - layer0[l] > 0;
      if (plain_nodes || of_layer[l] == -2) { close(); continue; }
      if (of_layer[l] == -1) continue;   // (an empty layer: nothing to launch, nothing to wait for)
      const GroupLaunch& L = group_launches_[of_layer[l]];
      const bool shape_walks = L.gt == L.ct && (L.gt == 1 || L.gt == 2 || L.gt == 4);   // the shapes the walk kernels are built for
      if (!shape_walks) { close(); continue; }
      if (open && (cur.gt != L.gt || cur.ct != L.ct || cur.group0 + cur.n_groups != L.group0)) close();
      if (!open) {
        cur = GroupRun{l, l, L.gt, L.ct, L.group0, 0, L.pnode0, L.pslot0, L.pw0, (int)levels.size(), 0, 0};
        open = true;
      }
      levels.push_back(int2{L.group0 - cur.group0, L.count});
      cur.layer_last = l;
      cur.n_groups += L.count;
      cur.n_levels++;
      cur.max_count = std::max(cur.max_count, L.count);
    }
    close();
  };
  collect(fwd_layer0_, group_runs_fwd_);
  collect(bwd_layer0_, group_runs_bwd_);
  // the walk going down takes a run's layers from the last to the first
  for (GroupRun& r : group_runs_bwd_) std::reverse(levels.begin() + r.level0, levels.begin() + r.level0 + r.n_levels);
  for (const GroupRun& r : group_runs_fwd_) n_walk_levels_ += r.n_levels;
  if (!levels.empty()) d_grp_levels_.upload(levels);
}

// a run goes as one walk launch if its layers' groups are few: each slice of 16 examples is one workgroup whose waves
// share a layer's groups, so a layer of many groups is better off spread over the device by a launch of its own
static bool run_walks(int max_count, int Bp) {
  return max_count <= 32 && (int64_t)max_count * (Bp / 16) <= 4096;
}

bool SparseCircuit::launch_group_walk(const GroupRun& r, bool forward, int Bp, int batch, bool tempered) {
  if (!run_walks(r.max_count, Bp)) return false;
  PCM_GROUP_DEV(g, batch, Bp);
  if (tempered) { g.inv_f = 1.f / flow_scale; g.norm = d_norm_.p; g.norm_row = -1; }
  GroupWalk w;
  w.levels = d_grp_levels_.p + r.level0;
  w.n_levels = r.n_levels;
  w.base = GroupBase{r.group0, r.pnode0, r.pslot0, r.pw0};
  const dim3 grid(Bp / 16);
  // waves per workgroup: as many as the kernel's registers allow (going down a 32 x 32 group takes 128 and more)
#define PCM_WALK(GT_, WVF_, WVB_)                                                                                              \
  do {                                                                                                                         \
    if (forward) hipLaunchKernelGGL((sparse_group_walk_kernel<GT_, GT_, WVF_, true>), grid, dim3(WVF_ * 64), 0, stream, g, w);  \
    else hipLaunchKernelGGL((sparse_group_walk_kernel<GT_, GT_, WVB_, false>), grid, dim3(WVB_ * 64), 0, stream, g, w);         \
  } while (0)
  switch (r.gt) {
    case 1: PCM_WALK(1, 16, 16); break;
    case 2: PCM_WALK(2, 16, 8); break;
    default: PCM_WALK(4, 4, 4); break;
  }
#undef PCM_WALK
  return true;
}

// the group kernels of one layer: what = 0 values going up, 1 the children's rows going down; what = 2: the edge
// flows of every group, after the backward pass
void SparseCircuit::launch_groups(int layer, int what, int Bp, int batch, bool tempered) {
  if (group_launches_.empty()) return;
  PCM_GROUP_DEV(g, batch, Bp);
  if (tempered) { g.inv_f = 1.f / flow_scale; g.norm = d_norm_.p; g.norm_row = -1; }
  for (const GroupLaunch& L : what == 2 ? group_stat_launches_ : group_launches_) {
    if (what != 2 && L.layer != layer) continue;
    const size_t lds = what == 2 ? group_lds_floats(L.gt * 16, L.ct * 16) * sizeof(float) : 0;
    const dim3 grid(L.count, what == 2 ? Bp / 64 : Bp / 16), block(what == 2 ? 256 : 64);
    const GroupBase base{L.group0, L.pnode0, L.pslot0, L.pw0};
    auto run = [&](auto kernel, auto arg) {
      if (lds > 48 * 1024)
        PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      hipLaunchKernelGGL(kernel, grid, block, lds, stream, g, arg);
    };
#define PCM_GROUP_CT(GT_, CT_)                                                     \
    if (what == 0) run(&sparse_group_forward_kernel<GT_, CT_>, base);              \
    else if (what == 1) run(&sparse_group_backward_kernel<GT_, CT_>, base);        \
    else run(&sparse_group_stats_kernel<GT_, CT_>, L.group0);
#define PCM_GROUP_GT(GT_)                                                          \
    switch (L.ct) {                                                                \
      case 1: PCM_GROUP_CT(GT_, 1) break;                                          \
      case 2: PCM_GROUP_CT(GT_, 2) break;                                          \
      case 4: PCM_GROUP_CT(GT_, 4) break;                                          \
      default: PCM_GROUP_CT(GT_, 8) break;                                         \
    }
    switch (L.gt) {
      case 1: PCM_GROUP_GT(1) break;
      case 2: PCM_GROUP_GT(2) break;
      case 4: PCM_GROUP_GT(4) break;
      default: PCM_GROUP_GT(8) break;
    }
#undef PCM_GROUP_GT
#undef PCM_GROUP_CT
  }
}

SparseCircuit::SparseCircuit(FlatCircuit fc) : fc_(std::move(fc)) {
  const int64_t nn = fc_.n_nodes(), ne = fc_.n_edges();
  if (nn == 0) fail(PCM_ERR_SHAPE, "empty circuit");
  // nodes by layer
  std::vector<int32_t> order(nn);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return fc_.layer[a] < fc_.layer[b]; });
  n_layers_ = fc_.layer[order.back()] + 1;
  layer_node0_.assign(n_layers_ + 1, 0);
  for (int64_t i = 0; i < nn; ++i) layer_node0_[fc_.layer[order[i]] + 1]++;
  for (int l = 0; l < n_layers_; ++l) layer_node0_[l + 1] += layer_node0_[l];
  // incoming edges per node: entry = edge << 1 | as_sub
  std::vector<int32_t> in_ptr(nn + 1, 0), in_edge;
  for (int64_t e = 0; e < ne; ++e) { in_ptr[fc_.e_prime[e] + 1]++; if (fc_.e_sub[e] >= 0) in_ptr[fc_.e_sub[e] + 1]++; }
  for (int64_t n = 0; n < nn; ++n) in_ptr[n + 1] += in_ptr[n];
  in_edge.resize(in_ptr[nn]);
  {
    std::vector<int32_t> fill(in_ptr.begin(), in_ptr.end() - 1);
    for (int64_t e = 0; e < ne; ++e) {
      in_edge[fill[fc_.e_prime[e]]++] = (int32_t)(e << 1);
      if (fc_.e_sub[e] >= 0) in_edge[fill[fc_.e_sub[e]]++] = (int32_t)(e << 1 | 1);
    }
  }
  if (in_edge.empty()) in_edge.push_back(0);
  // dense groups: their sums' edges leave the records of the backward pass, one record per (group, child) takes
  // their place in the child's list (at the place of the first of them)
  std::vector<int32_t> group_of(nn, -1), edge_slot(std::max<int64_t>(ne, 1), -1);
  build_groups(group_of, edge_slot);
  // the backward pass's records per node, in the order of the edges: {edge << 1 | role, parent (~parent: product),
  // prime, sub} or, for a group's row, {slot << 1 | 1, ~(n_nodes + slot), row of zeros, row of zeros}: read like the
  // flow of a product parent, never written to the edge sums (odd first word)
  struct Entry { int4 rec; int32_t key; uint8_t role; };   // key: edge, or -1 - slot; role 1: the node is the sub
  std::vector<std::vector<Entry>> in_list(nn);
  const int32_t zrow = (int32_t)nn;
  for (int64_t e = 0; e < ne; ++e) {
    const int32_t p = fc_.e_parent[e], pr = fc_.e_prime[e], sb = fc_.e_sub[e];
    if (group_of[p] >= 0) {
      const int32_t slot = edge_slot[e];
      if (slot < 0) continue;   // (one record per child: from the edges of the group's first sum)
      const int4 rec{(slot << 1) | 1, ~(int32_t)(nn + slot), zrow, zrow};
      in_list[pr].push_back(Entry{rec, -1 - slot, 0});
      if (sb >= 0) in_list[sb].push_back(Entry{rec, -1 - slot, 1});
      continue;
    }
    // operands an edge does not have name the row of zeros behind the last node's: the flow through a product
    // edge is its parent's (exponent 0 - 0 + 0 - 0), a sum edge without a second child adds 0
    const bool sum_edge = fc_.type[p] == kSum;
    const int4 rec{(int32_t)(e << 1), sum_edge ? p : ~p, sum_edge ? pr : zrow, sum_edge && sb >= 0 ? sb : zrow};
    in_list[pr].push_back(Entry{rec, (int32_t)e, 0});
    if (sb >= 0) in_list[sb].push_back(Entry{int4{rec.x | 1, rec.y, rec.z, rec.w}, (int32_t)e, 1});
  }
  // A node that a single group row reaches, and nothing else, has that row as its flow, and so has a node whose only
  // parent is such a product: the group's kernel writes their rows (up to kGroupCopies per child) and they leave the
  // backward layers (in an HCLT: every product, every sum below the root's and every leaf).  The row itself is kept
  // only where a node that stays in the layers reads it.
  std::vector<char> copied(nn, 0);
  if (n_group_slots_) {
    std::vector<char> is_seed(nn, 0);
    if (fc_.heads.empty()) is_seed[nn - 1] = 1;
    else for (int32_t hd : fc_.heads) is_seed[hd] = 1;
    std::vector<int32_t> slot_of(nn, -1);
    std::vector<std::vector<int32_t>> rows_of((size_t)n_group_slots_);
    for (int64_t i = nn - 1; i >= 0; --i) {   // parents before children
      const int32_t n = order[i];
      if (in_list[n].size() != 1 || is_seed[n]) continue;
      const Entry& en = in_list[n][0];
      int32_t slot = -1;
      if (en.key < 0) slot = -1 - en.key;
      else if (fc_.type[fc_.e_parent[en.key]] == kMul && copied[fc_.e_parent[en.key]]) slot = slot_of[fc_.e_parent[en.key]];
      if (slot < 0 || (int)rows_of[slot].size() >= kGroupCopies - 1) continue;
      slot_of[n] = slot;
      copied[n] = 1;
      rows_of[slot].push_back(n);
    }
    for (int64_t n = 0; n < nn; ++n) {
      if (copied[n]) continue;
      for (const Entry& en : in_list[n])
        if (en.key < 0 && (rows_of[-1 - en.key].empty() || rows_of[-1 - en.key][0] != (int32_t)(nn + (-1 - en.key))))
          rows_of[-1 - en.key].insert(rows_of[-1 - en.key].begin(), (int32_t)(nn + (-1 - en.key)));
    }
    std::vector<int4> copies(2 * d_grp_rows_.n, int4{-1, -1, -1, -1});   // (by entry of the padded per-child tables)
    for (int64_t s = 0; s < n_group_slots_; ++s) {
      int32_t r[kGroupCopies];
      for (int k = 0; k < kGroupCopies; ++k) r[k] = k < (int)rows_of[s].size() ? rows_of[s][k] : -1;
      copies[2 * (size_t)grp_pslot_h_[s]] = int4{r[0], r[1], r[2], r[3]};
      copies[2 * (size_t)grp_pslot_h_[s] + 1] = int4{r[4], r[5], r[6], r[7]};
    }
    d_grp_copies_.upload(copies);
    // the product edges that no layer kernel sums any more (it is the wave of an edge's prime that does)
    std::vector<int2> pe;
    for (int64_t n = 0; n < nn; ++n)
      if (copied[n] && in_list[n][0].key >= 0 && in_list[n][0].role == 0) pe.push_back(int2{in_list[n][0].key, fc_.e_parent[in_list[n][0].key]});
    n_group_product_edges_ = (int)pe.size();
    if (!pe.empty()) d_grp_product_edges_.upload(pe);
  }
  std::vector<int32_t> rec_ptr(nn + 1, 0);
  for (int64_t n = 0; n < nn; ++n) rec_ptr[n + 1] = rec_ptr[n] + (int32_t)in_list[n].size();
  std::vector<int4> in_rec(std::max<size_t>(rec_ptr[nn], 1), int4{0, 0, 0, 0});
  for (int64_t n = 0; n < nn; ++n)
    for (size_t q = 0; q < in_list[n].size(); ++q) in_rec[rec_ptr[n] + q] = in_list[n][q].rec;
  d_in_rec_.upload(in_rec);
  d_type_.upload(fc_.type);
  d_order_.upload(order);
  {   // the forward layers: the nodes that no group's kernel computes
    std::vector<int4> fr;
    fwd_layer0_.assign(n_layers_ + 1, 0);
    layer_max_children_.assign(n_layers_, 0);
    for (int l = 0; l < n_layers_; ++l) {
      for (int i = layer_node0_[l]; i < layer_node0_[l + 1]; ++i) {
        const int32_t n = order[i];
        if (group_of[n] >= 0 || grp_expanded_[n]) continue;
        fr.push_back(int4{n, (int)fc_.type[n], fc_.node_e0[n], fc_.node_e1[n]});
        if (l == 0 && fc_.type[n] != kInput) layer0_inputs_only_ = false;
        if (fc_.type[n] != kInput) layer_max_children_[l] = std::max(layer_max_children_[l], (int)(fc_.node_e1[n] - fc_.node_e0[n]));
      }
      fwd_layer0_[l + 1] = (int)fr.size();
    }
    n_layer_nodes_ = (int64_t)fr.size();
    if (fr.empty()) fr.push_back(int4{0, 0, 0, 0});
    d_fwd_rec_.upload(fr);
  }
  d_node_e0_.upload(fc_.node_e0); d_node_e1_.upload(fc_.node_e1);
  auto up = [&](DevBuf<int32_t>& dst, std::vector<int32_t> v) { if (v.empty()) v.push_back(0); dst.upload(v); };
  up(d_e_parent_, fc_.e_parent); up(d_e_prime_, fc_.e_prime); up(d_e_sub_, fc_.e_sub);
  d_in_var_.upload(fc_.in_var);
  d_in_off_.upload(fc_.in_off);
  { std::vector<float> lp = fc_.e_logp; if (lp.empty()) lp.push_back(0.f); d_logp_.upload(lp); }
  d_leaf_.upload(fc_.leaf_logp);
  d_in_ptr_.upload(in_ptr); d_in_edge_.upload(in_edge);
  d_edge_aggr_.alloc(std::max<int64_t>(ne, 1)); d_edge_aggr_.zero();
  d_leaf_flow_.alloc(fc_.leaf_logp.size()); d_leaf_flow_.zero();
  // seed table: which root / head a node is (-1: none)
  std::vector<int32_t> seed_of(nn, -1);
  if (fc_.heads.empty()) seed_of[nn - 1] = 0;
  else for (size_t h = 0; h < fc_.heads.size(); ++h) seed_of[fc_.heads[h]] = (int32_t)h;
  if (!fc_.heads.empty()) d_head_nodes_.upload(fc_.heads);
  // An input node that is the second factor of two-child products and sees exactly the edges its
  // first factor (the prime) sees gets the same flow as the prime: it is dropped from the backward
  // layers and the prime's wave writes its row too (in an HCLT: every leaf).
  std::vector<int32_t> alias_of(nn, -1);
  for (int64_t b = 0; b < nn && ne; ++b) {
    const auto& lb = in_list[b];
    if (fc_.type[b] != kInput || seed_of[b] >= 0 || lb.empty() || !lb[0].role || copied[b]) continue;
    // the prime beside which b stands in its first record
    const int32_t a = lb[0].key >= 0 ? fc_.e_prime[lb[0].key] : grp_prime_h_[-1 - lb[0].key];
    if (a == b || copied[a] || in_list[a].size() != lb.size()) continue;
    bool same = true;
    for (size_t q = 0; q < lb.size() && same; ++q)
      same = lb[q].role == 1 && in_list[a][q].role == 0 && in_list[a][q].key == lb[q].key;
    if (same) alias_of[b] = a;
  }
  std::vector<int32_t> alias_ptr(nn + 1, 0), alias_list;
  for (int64_t b = 0; b < nn; ++b) if (alias_of[b] >= 0) alias_ptr[alias_of[b] + 1]++;
  for (int64_t n = 0; n < nn; ++n) alias_ptr[n + 1] += alias_ptr[n];
  alias_list.resize(alias_ptr[nn]);
  {
    std::vector<int32_t> fill(alias_ptr.begin(), alias_ptr.end() - 1);
    for (int64_t b = 0; b < nn; ++b) if (alias_of[b] >= 0) alias_list[fill[alias_of[b]]++] = (int32_t)b;
  }
  if (alias_list.empty()) alias_list.push_back(0);
  std::vector<int32_t> bwd_order;
  bwd_layer0_.assign(n_layers_ + 1, 0);
  bwd_layer_max_in_.assign(n_layers_, 0);
  for (int l = 0; l < n_layers_; ++l) {
    for (int i = layer_node0_[l]; i < layer_node0_[l + 1]; ++i)
      if (alias_of[order[i]] < 0 && !copied[order[i]]) {
        bwd_order.push_back(order[i]);
        bwd_layer_max_in_[l] = std::max(bwd_layer_max_in_[l], (int)(rec_ptr[order[i] + 1] - rec_ptr[order[i]]));
      }
    bwd_layer0_[l + 1] = (int)bwd_order.size();
  }
  d_alias_list_.upload(alias_list);
  d_bwd_order_.upload(bwd_order);
  {
    std::vector<int4> br(std::max<size_t>(bwd_order.size(), 1), int4{0, -1, 0, 0});
    std::vector<int2> ar(br.size(), int2{0, 0});
    for (size_t i = 0; i < bwd_order.size(); ++i) {
      const int32_t n = bwd_order[i];
      br[i] = int4{n, seed_of[n], rec_ptr[n], rec_ptr[n + 1]};
      ar[i] = int2{alias_ptr[n], alias_ptr[n + 1]};
    }
    d_bwd_rec_.upload(br);
    d_bwd_alias_.upload(ar);
  }
  build_group_runs();
  // normalisation groups over the sum parameters
  std::vector<int32_t> gp(1, 0), p2e;
  for (int64_t s : fc_.pargroup_sizes) gp.push_back(gp.back() + (int32_t)s);
  for (int64_t e : fc_.param2edge) p2e.push_back((int32_t)(e - 1));
  if (p2e.empty()) p2e.push_back(0);
  d_group_ptr_.upload(gp);
  d_param2edge_.upload(p2e);
}

int64_t SparseCircuit::size(int what) const {
  switch (what) {
    case 0: return (int64_t)fc_.param2edge.size() + (int64_t)fc_.leaf_logp.size();
    case 1: return (int64_t)fc_.param2edge.size();
    case 2: return fc_.n_nodes();
    case 3: return fc_.n_edges();
    case 4: return (int64_t)fc_.leaf_logp.size();
    case 5: return fc_.num_vars;
    case 6: return fc_.num_cats;
    case 7: return 0;
    case 8: return 0;
    case 9: return (int64_t)fc_.layer_ends.size();
    case 10: return (int64_t)fc_.pargroup_sizes.size();
    case 11: return (int64_t)fc_.input_nodes.size();
    case 12: return fc_.num_heads;
    case 13: return (int64_t)fc_.desc_node.size();
    case 14: return 0;
    case 15: return 1;
    case 16: return n_groups_;
    case 17: return n_layer_nodes_;
    case 18: return n_walk_levels_;
    default: fail(PCM_ERR_ARG, "unknown size selector %d", what);
  }
}

void SparseCircuit::index_table(int which, int64_t* out, int64_t n) const {
  auto copy = [&](const std::vector<int64_t>& v) {
    if ((int64_t)v.size() != n) fail(PCM_ERR_ARG, "index table %d has %lld entries, caller gave %lld", which,
                                     (long long)v.size(), (long long)n);
    std::copy(v.begin(), v.end(), out);
  };
  auto plus1 = [&](const std::vector<int32_t>& v) { std::vector<int64_t> r(v.size()); for (size_t i = 0; i < v.size(); ++i) r[i] = v[i] + 1; return r; };
  switch (which) {
    case 0: copy(fc_.edge2param); break;
    case 1: copy(fc_.param2edge); break;
    case 2: copy(fc_.param2group); break;
    case 3: copy(fc_.pargroup_sizes); break;
    case 4: { std::vector<int64_t> c(fc_.input_nodes.size()); for (size_t i = 0; i < c.size(); ++i) c[i] = (int64_t)(i + 1) * fc_.num_cats; copy(c); break; }
    case 5: copy(fc_.layer_ends); break;
    case 6: copy(plus1(fc_.e_parent)); break;
    case 7: copy(plus1(fc_.e_prime)); break;
    case 8: copy(plus1(fc_.e_sub)); break;
    case 9: copy(plus1(fc_.heads)); break;
    case 10: copy(plus1(fc_.desc_node)); break;
    case 11: copy(plus1(fc_.input_nodes)); break;
    default: fail(PCM_ERR_ARG, "unknown index table %d", which);
  }
}

static void fetch(std::vector<float>& h, const float* d, size_t n, hipStream_t s) {
  h.resize(n);
  if (!n) return;
  PCM_HIP(hipMemcpyAsync(h.data(), d, n * sizeof(float), hipMemcpyDeviceToHost, s));
  PCM_HIP(hipStreamSynchronize(s));
}

void SparseCircuit::vectorize(float* out, int64_t n) {
  if (n != size(0)) fail(PCM_ERR_ARG, "parameter vector has %lld entries, circuit has %lld", (long long)n, (long long)size(0));
  std::vector<float> lp, lf;
  fetch(lp, d_logp_.p, fc_.n_edges(), stream);
  fetch(lf, d_leaf_.p, fc_.leaf_logp.size(), stream);
  const size_t ns = fc_.param2edge.size();
  for (size_t i = 0; i < ns; ++i) out[i] = lp[fc_.param2edge[i] - 1];
  std::copy(lf.begin(), lf.end(), out + ns);
}

void SparseCircuit::update_parameters(const float* in, int64_t n) {
  if (n != size(0)) fail(PCM_ERR_ARG, "parameter vector has %lld entries, circuit has %lld", (long long)n, (long long)size(0));
  std::vector<float> lp;
  fetch(lp, d_logp_.p, fc_.n_edges(), stream);
  const size_t ns = fc_.param2edge.size();
  for (size_t i = 0; i < ns; ++i) lp[fc_.param2edge[i] - 1] = in[i];
  if (!lp.empty()) PCM_HIP(hipMemcpyAsync(d_logp_.p, lp.data(), lp.size() * sizeof(float), hipMemcpyHostToDevice, stream));
  if (!fc_.leaf_logp.empty())
    PCM_HIP(hipMemcpyAsync(d_leaf_.p, in + ns, fc_.leaf_logp.size() * sizeof(float), hipMemcpyHostToDevice, stream));
  PCM_HIP(hipStreamSynchronize(stream));
}

void SparseCircuit::ensure_batch(int batch) {
  if (batch <= cap_batch_) return;
  const int Bp = ceil_div(batch, 64) * 64;
  d_mars_.alloc((size_t)(fc_.n_nodes() + 1) * Bp);   // one more row, of zeros: the operand an edge does not have
  d_flows_.alloc((size_t)n_flow_rows() * Bp);
  cap_batch_ = Bp;
}

static SparseDev make_dev(const uint8_t* type, const int32_t* order, const int32_t* e0, const int32_t* e1,
                          const int32_t* ep, const int32_t* epr, const int32_t* es, const int32_t* in_var,
                          const int32_t* in_ptr, const int32_t* in_edge, const int4* in_rec, const int64_t* in_off, const float* logp,
                          const float* leaf, const uint8_t* xb, float* mars, float* flows, int B, int Bp, int C, int64_t n_nodes,
                          const int4* fwd_rec, const int4* bwd_rec, const int2* bwd_alias) {
  SparseDev d;
  d.fwd_rec = fwd_rec; d.bwd_rec = bwd_rec; d.bwd_alias = bwd_alias;
  d.type = type; d.order = order; d.node_e0 = e0; d.node_e1 = e1; d.e_parent = ep; d.e_prime = epr; d.e_sub = es;
  d.in_var = in_var; d.in_ptr = in_ptr; d.in_edge = in_edge; d.in_rec = in_rec; d.in_logp = nullptr; d.in_off = in_off;
  d.ev = nullptr; d.ev_se = d.ev_sv = d.ev_sc = 0; d.ev_idx = nullptr; d.logp = logp; d.leaf = leaf;
  d.xb = xb; d.mars = mars; d.flows = flows; d.B = B; d.Bp = Bp; d.C = C; d.n_nodes = n_nodes; d.n_flow_rows = n_nodes;
  d.norm = nullptr; d.inv_f = 1.f;
  return d;
}

// a layer kernel with rows through buffer descriptors where the value / flow arrays stay below 2 GiB (row offsets are
// signed 32-bit scalars)
#define PCM_LAYER_LAUNCH(kernel, EX_, W_, RUN_, grid, ...)                                                      \
  do {                                                                                                          \
    if ((int64_t)(n_flow_rows() + 1) * Bp * 4 < ((int64_t)1 << 31))                                             \
      hipLaunchKernelGGL((kernel<EX_, W_, RUN_, true>), grid, dim3((W_) * 64), 0, stream, __VA_ARGS__);         \
    else                                                                                                        \
      hipLaunchKernelGGL((kernel<EX_, W_, RUN_, false>), grid, dim3((W_) * 64), 0, stream, __VA_ARGS__);        \
  } while (0)

#define SPARSE_DEV(B_, Bp_, xb_) \
  make_dev(d_type_.p, d_order_.p, d_node_e0_.p, d_node_e1_.p, d_e_parent_.p, d_e_prime_.p, d_e_sub_.p, d_in_var_.p, \
           d_in_ptr_.p, d_in_edge_.p, d_in_rec_.p, d_in_off_.p, d_logp_.p, d_leaf_.p, xb_, d_mars_.p, d_flows_.p, B_, Bp_, fc_.num_cats, fc_.n_nodes(), d_fwd_rec_.p, d_bwd_rec_.p, d_bwd_alias_.p)

// input nodes grouped by variable
void SparseCircuit::ensure_var_tables() {
  if (d_var_ptr_.n) return;
  std::vector<int32_t> vp(fc_.num_vars + 1, 0), vn(fc_.input_nodes.size());
  for (int32_t n : fc_.input_nodes) vp[fc_.in_var[n] + 1]++;
  for (int v = 0; v < fc_.num_vars; ++v) vp[v + 1] += vp[v];
  std::vector<int32_t> fill(vp.begin(), vp.end() - 1);
  for (int32_t n : fc_.input_nodes) vn[fill[fc_.in_var[n]]++] = n;
  if (vn.empty()) vn.push_back(0);
  max_var_nodes_ = 1;
  for (int v = 0; v < fc_.num_vars; ++v) max_var_nodes_ = std::max(max_var_nodes_, vp[v + 1] - vp[v]);
  d_var_ptr_.upload(vp, stream);
  d_var_nodes_.upload(vn, stream);
}

void SparseCircuit::run_forward(const BatchRef* b, const SoftRef* s) {
  const int batch = b ? b->batch : s->batch;
  if (b ? !b->d_data : !s->d_ev) fail(PCM_ERR_ARG, "data pointer is null");
  if (batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", batch);
  ensure_batch(batch);
  const int Bp = ceil_div(batch, 64) * 64;
  // the staged categories live in a dedicated buffer
  d_visit_.ensure((size_t)std::max<int64_t>((int64_t)fc_.num_vars, fc_.n_nodes()) * Bp);
  uint8_t* xb = d_visit_.p;
  if (b) {
    pcm_stage(b->d_data, b->stride_ex, b->stride_var, b->d_idx, batch, Bp, fc_.num_vars, fc_.num_cats, xb, stream);
    check_launch("stage_batch");
  }
  SparseDev d = SPARSE_DEV(batch, Bp, xb);
  // the row of zeros sits behind the last node's row at this batch's row length (a smaller batch than the
  // arrays were sized for finds old values there)
  PCM_HIP(hipMemsetAsync(d_mars_.p + (size_t)fc_.n_nodes() * Bp, 0, (size_t)Bp * sizeof(float), stream));
  if (s) {
    d.ev = s->d_ev; d.ev_se = s->stride_ex; d.ev_sv = s->stride_var; d.ev_sc = s->stride_cat; d.ev_idx = s->d_idx;
    ensure_var_tables();
    hipLaunchKernelGGL(sparse_soft_input_kernel, dim3(fc_.num_vars, Bp / kSoftTile), dim3(256), 0, stream, d, d_var_ptr_.p,
                       d_var_nodes_.p);
  }
  refresh_group_w();
  if (n_groups_) {
    d_grp_m_.ensure((size_t)n_groups_ * Bp);
    d_grp_xm_.ensure(d_grp_rows_.n * (size_t)Bp);
  }
  size_t next_run = 0;
  for (int l = 0; l < n_layers_; ++l) {
    const int n0 = fwd_layer0_[l], cnt = fwd_layer0_[l + 1] - n0;
    while (next_run < group_runs_fwd_.size() && group_runs_fwd_[next_run].layer_first < l) ++next_run;
    if (next_run < group_runs_fwd_.size() && group_runs_fwd_[next_run].layer_first == l &&
        launch_group_walk(group_runs_fwd_[next_run], true, Bp, batch, false)) {
      l = group_runs_fwd_[next_run].layer_last;   // the run's layers hold nothing but these groups
      continue;
    }
    launch_groups(l, 0, Bp, batch);
    if (cnt == 0) continue;
    const int64_t pairs = (int64_t)cnt * (Bp / 64);
    if (l == 0 && layer0_inputs_only_ && cnt >= 4096) {
      if (!s) hipLaunchKernelGGL(sparse_input_kernel, dim3(ceil_div(cnt, 4)), dim3(256), 0, stream, d, n0, cnt);
      continue;   // (soft evidence: sparse_soft_input_kernel has filled the input rows)
    }
    if (layer_max_children_[l] <= kNarrowDegree) {
      if (pairs < kManyPairs) PCM_LAYER_LAUNCH(sparse_forward_kernel, 1, 1, 4, dim3(cnt, Bp / 64), d, n0);
      else PCM_LAYER_LAUNCH(sparse_forward_kernel, 4, 1, 4, dim3(cnt, ceil_div(Bp, 256)), d, n0);
    } else if (pairs < kSplitBelow) {
      PCM_LAYER_LAUNCH(sparse_forward_kernel, 1, kSplitWaves, kSplitRun, dim3(cnt, Bp / 64), d, n0);
    } else if (pairs < kSaturated) {
      PCM_LAYER_LAUNCH(sparse_forward_kernel, 1, 1, kWideRun, dim3(cnt, Bp / 64), d, n0);
    } else {
      PCM_LAYER_LAUNCH(sparse_forward_kernel, 2, 1, 8, dim3(cnt, ceil_div(Bp, 128)), d, n0);
    }
  }
  check_launch("sparse_forward");
  last_batch_ = batch;
  flow_batch_ = 0;       // the flow array belongs to an earlier batch
}

// root (or head) rows -> output; the root is the last node
void SparseCircuit::write_ll(int batch, float* d_ll) {
  const int Bp = ceil_div(batch, 64) * 64;
  if (fc_.heads.empty()) {
    PCM_HIP(hipMemcpyAsync(d_ll, d_mars_.p + (size_t)(fc_.n_nodes() - 1) * Bp, (size_t)batch * sizeof(float),
                           hipMemcpyDeviceToDevice, stream));
  } else {
    hipLaunchKernelGGL(sparse_copy_rows_kernel, dim3(ceil_div(batch, 256), (int)fc_.heads.size()), dim3(256), 0, stream,
                       d_mars_.p, Bp, batch, d_head_nodes_.p, (int)fc_.heads.size(), d_ll);
    check_launch("copy_rows");
  }
}

void SparseCircuit::loglikelihoods(const BatchRef& b, float* d_ll) {
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  run_forward(&b, nullptr);
  write_ll(b.batch, d_ll);
}

void SparseCircuit::loglikelihoods_soft(const SoftRef& s, float* d_ll) {
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  run_forward(nullptr, &s);
  write_ll(s.batch, d_ll);
}

void SparseCircuit::flows(const BatchRef& b, float rate, const float* d_head_mask, float* d_ll) {
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  // (a circuit with one root takes the mask as [1][batch]: the flow each example starts with at the root, i.e. the
  // per-example weights of reg_flow.jl:38-39,190-191 -- every flow is linear in it)
  if (!fc_.heads.empty() && !d_head_mask) fail(PCM_ERR_ARG, "a multi-head circuit needs a head_mask for its flows");
  run_forward(&b, nullptr);
  run_flows(b.batch, nullptr, rate, d_head_mask, d_ll);
}

void SparseCircuit::flows_soft(const SoftRef& s, float rate, const float* d_head_mask, float* d_ll) {
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  if (!fc_.heads.empty() && !d_head_mask) fail(PCM_ERR_ARG, "a multi-head circuit needs a head_mask for its flows");
  run_forward(nullptr, &s);
  run_flows(s.batch, &s, rate, d_head_mask, d_ll);
}

// accumulate = false: node flows only (d_flows_), the circuit's accumulators and d_ll are left alone
void SparseCircuit::run_flows(int batch, const SoftRef* soft, float rate, const float* d_head_mask, float* d_ll, bool accumulate) {
  const int Bp = ceil_div(batch, 64) * 64;
  const int64_t ne = fc_.n_edges();
  if (accumulate) {
    hipLaunchKernelGGL(sparse_scale_kernel, dim3(ceil_div(std::max<int64_t>(ne, 1), 256)), dim3(256), 0, stream, d_edge_aggr_.p, ne, rate);
    hipLaunchKernelGGL(sparse_scale_kernel, dim3(ceil_div((int64_t)fc_.leaf_logp.size(), 256)), dim3(256), 0, stream,
                       d_leaf_flow_.p, (int64_t)fc_.leaf_logp.size(), rate);
  }
  SparseDev d = SPARSE_DEV(batch, Bp, d_visit_.p);
  d.n_flow_rows = n_flow_rows();
  if (soft) { d.ev = soft->d_ev; d.ev_se = soft->stride_ex; d.ev_sv = soft->stride_var; d.ev_sc = soft->stride_cat; d.ev_idx = soft->d_idx; }
  SparseDev db = d;
  if (ne) {
    d_in_logp_.ensure(d_in_rec_.n);
    hipLaunchKernelGGL(sparse_gather_in_logp_kernel, dim3(ceil_div((int64_t)d_in_rec_.n, 256)), dim3(256), 0, stream,
                       d_in_rec_.p, d_logp_.p, (int64_t)d_in_rec_.n, fc_.n_nodes(), d_in_logp_.p);
    db.in_logp = d_in_logp_.p;
  }
  db.order = d_bwd_order_.p;   // the layers without the input nodes whose rows other nodes write
  const bool tempered = accumulate && flow_scale != 1.f;
  if (tempered) {
    d_norm_.ensure((size_t)(fc_.n_nodes() + 1) * Bp);
    db.inv_f = 1.f / flow_scale;
    db.norm = d_norm_.p;
    hipLaunchKernelGGL(sparse_tempered_norm_kernel, dim3((unsigned)(fc_.n_nodes() + 1), ceil_div(Bp, 256)), dim3(256), 0, stream, db,
                       d_norm_.p);
    refresh_group_w(db.inv_f);   // W^(1 / fscale) for this pass; the next forward pass puts W back
  }
  // edge flows summed over the batch: one row of partial sums per 64 examples, cleared first (an edge that
  // no wave visits must read as zero), added into the accumulators in row order after the walk
  const int n_parts = Bp / 64;
  if (ne) {
    d_edge_part_.ensure((size_t)n_parts * ne);
    hipLaunchKernelGGL(sparse_scale_kernel, dim3(ceil_div((int64_t)n_parts * ne, 256)), dim3(256), 0, stream, d_edge_part_.p,
                       (int64_t)n_parts * ne, 0.f);
  }
  int next_run = (int)group_runs_bwd_.size() - 1;
  for (int l = n_layers_ - 1; l >= 0; --l) {
    while (next_run >= 0 && group_runs_bwd_[next_run].layer_last > l) --next_run;
    if (next_run >= 0 && group_runs_bwd_[next_run].layer_last == l &&
        launch_group_walk(group_runs_bwd_[next_run], false, Bp, batch, tempered)) {
      l = group_runs_bwd_[next_run].layer_first;   // (the loop's --l moves on below the run)
      continue;
    }
    const int n0 = bwd_layer0_[l], cnt = bwd_layer0_[l + 1] - n0;
    const int64_t pairs = (int64_t)cnt * (Bp / 64);
#define PCM_BWD_ARGS db, n0, d_head_mask, d_edge_part_.p, ne, d_alias_list_.p
    if (cnt == 0) {   // (every node of the layer takes its flow from a group's row)
    } else if (tempered) {
      hipLaunchKernelGGL((sparse_backward_kernel<1, 1, 16, false, true>), dim3(cnt, Bp / 64), dim3(64), 0, stream, PCM_BWD_ARGS);
    } else if (bwd_layer_max_in_[l] <= kNarrowDegree) {
      if (pairs < kManyPairs) PCM_LAYER_LAUNCH(sparse_backward_kernel, 1, 1, 4, dim3(cnt, Bp / 64), PCM_BWD_ARGS);
      else   // (the rows of partial edge sums beyond a quarter stay as cleared)
        PCM_LAYER_LAUNCH(sparse_backward_kernel, 4, 1, 4, dim3(cnt, ceil_div(Bp, 256)), PCM_BWD_ARGS);
    } else if (pairs < kSplitBelow) {
      PCM_LAYER_LAUNCH(sparse_backward_kernel, 1, kSplitWaves, kSplitRun, dim3(cnt, Bp / 64), PCM_BWD_ARGS);
    } else if (pairs < kSaturated) {
      PCM_LAYER_LAUNCH(sparse_backward_kernel, 1, 1, kWideRun, dim3(cnt, Bp / 64), PCM_BWD_ARGS);
    } else {
      PCM_LAYER_LAUNCH(sparse_backward_kernel, 2, 1, 8, dim3(cnt, ceil_div(Bp, 128)), PCM_BWD_ARGS);
    }
#undef PCM_BWD_ARGS
    launch_groups(l, 1, Bp, batch, tempered);   // the layer's sums have their flows: on to their children's rows
  }
  if (!accumulate) {
    check_launch("sparse_backward");
    flow_batch_ = last_batch_;
    return;
  }
  launch_groups(-1, 2, Bp, batch, tempered);   // the groups' edge flows, into the same rows of partial sums
  if (tempered) refresh_group_w();   // (W itself again, for whatever reads the tables next)
  if (n_group_product_edges_)
    hipLaunchKernelGGL(sparse_product_edge_kernel, dim3(ceil_div(n_group_product_edges_, 4), Bp / 64), dim3(256), 0, stream,
                       d_grp_product_edges_.p, n_group_product_edges_, d_flows_.p, Bp, d_edge_part_.p, ne);
  if (ne)
    hipLaunchKernelGGL(sum_parts_kernel<false>, dim3(ceil_div(ne, 64)), dim3(256), 0, stream, d_edge_part_.p, n_parts, ne,
                       (const float*)nullptr, d_edge_aggr_.p);
  if (!fc_.input_nodes.empty()) {
    if (d_input_nodes_.n == 0) d_input_nodes_.upload(fc_.input_nodes, stream);
    if (soft)
      hipLaunchKernelGGL(sparse_leaf_flow_soft_kernel,
                         dim3(fc_.num_vars, ceil_div(fc_.num_cats, kSoftTile), ceil_div(max_var_nodes_, 4 * kFlowNodes)), dim3(256), 0,
                         stream, d, d_var_ptr_.p, d_var_nodes_.p, d_leaf_flow_.p);
    else
    {
      const int n_in = (int)fc_.input_nodes.size();
      if (n_in >= 4096 && batch <= 16384)   // (a wave per node: enough nodes to fill the device four to a workgroup)
        hipLaunchKernelGGL(sparse_leaf_flow_kernel<64>, dim3((unsigned)ceil_div(n_in, 4)), dim3(256), 0, stream, d,
                           d_input_nodes_.p, n_in, d_leaf_flow_.p);
      else
        hipLaunchKernelGGL(sparse_leaf_flow_kernel<256>, dim3((unsigned)n_in), dim3(256), 0, stream, d, d_input_nodes_.p, n_in,
                           d_leaf_flow_.p);
    }
  }
  check_launch("sparse_backward");
  if (fc_.heads.empty()) {
    PCM_HIP(hipMemcpyAsync(d_ll, d_mars_.p + (size_t)(fc_.n_nodes() - 1) * Bp, (size_t)batch * sizeof(float),
                           hipMemcpyDeviceToDevice, stream));
  } else {
    hipLaunchKernelGGL(sparse_head_mixture_kernel, dim3(ceil_div(batch, 64)), dim3(64 * kMixGroups), 0, stream, d_mars_.p, Bp, batch,
                       d_head_nodes_.p, (int)fc_.heads.size(), d_head_mask, d_ll);
    check_launch("head_mixture");
  }
  have_flows_ = true;
  flow_batch_ = last_batch_;
}

void SparseCircuit::em_update(float pseudocount, float inertia) {
  if (!have_flows_) fail(PCM_ERR_STATE, "pcm_em_update called before any pcm_flows");
  SparseDev d = SPARSE_DEV(0, 64, nullptr);
  hipLaunchKernelGGL(sparse_update_kernel, dim3(ceil_div(fc_.n_nodes(), 4)), dim3(256), 0, stream, d, (int)fc_.n_nodes(),
                     d_logp_.p, d_leaf_.p, d_edge_aggr_.p, d_leaf_flow_.p, pseudocount, inertia);
  check_launch("sparse_update");
}

void SparseCircuit::get_node_values(float* mars, float* flows, int64_t n) {
  if (!last_batch_) fail(PCM_ERR_STATE, "no batch has been evaluated yet");
  const int B = last_batch_, Bp = ceil_div(B, 64) * 64;
  if (n != fc_.n_nodes() * B) fail(PCM_ERR_ARG, "expected %lld values (nodes x batch), caller gave %lld",
                                   (long long)(fc_.n_nodes() * B), (long long)n);
  std::vector<float> h;
  for (int pass = 0; pass < 2; ++pass) {
    float* dst = pass ? flows : mars;
    if (!dst) continue;
    if (pass && !have_flows_) fail(PCM_ERR_STATE, "no flows have been computed yet");
    fetch(h, pass ? d_flows_.p : d_mars_.p, (size_t)fc_.n_nodes() * Bp, stream);
    for (int64_t i = 0; i < fc_.n_nodes(); ++i) std::copy(h.begin() + i * Bp, h.begin() + i * Bp + B, dst + i * B);
  }
}

// out[n] = sum over the examples of the last flow pass of flows[n][b] (one wave per node)
__global__ __launch_bounds__(256) void sparse_node_flow_sum_kernel(const float* __restrict__ flows, int64_t n_nodes, int B, int Bp,
                                                                   float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= n_nodes) return;
  const float* row = flows + n * Bp;
  float s = 0.f;
  for (int b = lane; b < B; b += 64) s += row[b];
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) out[n] = s;
}

void SparseCircuit::node_flow_sums(float* out, int64_t n) {
  if (!have_flows_ || !flow_batch_) fail(PCM_ERR_STATE, "the node flows of the last batch are gone (call pcm_flows first)");
  if (!out) fail(PCM_ERR_ARG, "output pointer is null");
  if (n != fc_.n_nodes()) fail(PCM_ERR_ARG, "circuit has %lld nodes, caller gave %lld", (long long)fc_.n_nodes(), (long long)n);
  const int B = flow_batch_, Bp = ceil_div(B, 64) * 64;
  d_node_sums_.ensure((size_t)n);
  hipLaunchKernelGGL(sparse_node_flow_sum_kernel, dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, stream, d_flows_.p, n, B, Bp,
                     d_node_sums_.p);
  check_launch("node_flow_sums");
  PCM_HIP(hipMemcpyAsync(out, d_node_sums_.p, n * sizeof(float), hipMemcpyDeviceToHost, stream));
  PCM_HIP(hipStreamSynchronize(stream));
}

void SparseCircuit::get_aggregates(float* edge_aggr, int64_t n_edges, float* leaf_flow, int64_t n_leaf) {
  if (!have_flows_) fail(PCM_ERR_STATE, "no flows have been computed yet");
  if (edge_aggr) {
    if (n_edges != fc_.n_edges()) fail(PCM_ERR_ARG, "circuit has %lld edges, caller gave %lld", (long long)fc_.n_edges(), (long long)n_edges);
    if (n_edges) { PCM_HIP(hipMemcpyAsync(edge_aggr, d_edge_aggr_.p, n_edges * sizeof(float), hipMemcpyDeviceToHost, stream)); }
  }
  if (leaf_flow) {
    if (n_leaf != (int64_t)fc_.leaf_logp.size()) fail(PCM_ERR_ARG, "circuit has %zu input parameters, caller gave %lld", fc_.leaf_logp.size(), (long long)n_leaf);
    PCM_HIP(hipMemcpyAsync(leaf_flow, d_leaf_flow_.p, n_leaf * sizeof(float), hipMemcpyDeviceToHost, stream));
  }
  PCM_HIP(hipStreamSynchronize(stream));
}

// ---- KL ---------------------------------------------------------------------------------

static SparseCircuit* same_structure(SparseCircuit* p, pcm_circuit* q) {
  auto* s = dynamic_cast<SparseCircuit*>(q);
  if (!s) fail(PCM_ERR_ARG, "the two circuits of a KL query must be of the same kind");
  if (s->flat().n_nodes() != p->flat().n_nodes() || s->flat().n_edges() != p->flat().n_edges() ||
      s->flat().e_prime != p->flat().e_prime || s->flat().e_sub != p->flat().e_sub || s->flat().num_cats != p->flat().num_cats)
    fail(PCM_ERR_SHAPE, "the two circuits of a KL query must share one structure");
  return s;
}

void SparseCircuit::kld_forward_device(SparseCircuit* q) {
  if (!fc_.heads.empty()) fail(PCM_ERR_UNSUPPORTED, "KL of multi-head circuits is not defined");
  d_kld_.ensure(fc_.n_nodes());
  d_edge_kld_.ensure(std::max<int64_t>(fc_.n_edges(), 1));
  SparseDev d = SPARSE_DEV(0, 64, nullptr);
  for (int l = 0; l < n_layers_; ++l) {
    const int n0 = layer_node0_[l], n1 = layer_node0_[l + 1];
    hipLaunchKernelGGL(sparse_kld_up_kernel, dim3(ceil_div(n1 - n0, 128)), dim3(128), 0, stream, d, n0, n1, q->d_logp_.p,
                       q->d_leaf_.p, d_kld_.p, d_edge_kld_.p);
  }
  check_launch("sparse_kld_up");
}

void SparseCircuit::kld(pcm_circuit* q, float* out) {
  SparseCircuit* s = same_structure(this, q);
  kld_forward_device(s);
  PCM_HIP(hipMemcpyAsync(out, d_kld_.p + fc_.n_nodes() - 1, sizeof(float), hipMemcpyDeviceToHost, stream));
  PCM_HIP(hipStreamSynchronize(stream));
}

void SparseCircuit::kld_backward_device(SparseCircuit* q, float* g1, float* g2, float* lg1, float* lg2) {
  kld_forward_device(q);
  d_grad_.ensure(fc_.n_nodes());
  SparseDev d = SPARSE_DEV(0, 64, nullptr);
  for (int l = n_layers_ - 1; l >= 0; --l) {
    const int n0 = layer_node0_[l], n1 = layer_node0_[l + 1];
    hipLaunchKernelGGL(sparse_kld_down_kernel, dim3(ceil_div(n1 - n0, 128)), dim3(128), 0, stream, d, n0, n1,
                       (int)fc_.n_nodes() - 1, d_grad_.p);
  }
  const int64_t ne = fc_.n_edges();
  if (ne) hipLaunchKernelGGL(sparse_kld_edge_grad_kernel, dim3(ceil_div(ne, 256)), dim3(256), 0, stream, d, ne, d_grad_.p,
                             d_edge_kld_.p, g1, g2);
  DevBuf<int32_t> inn;
  inn.upload(fc_.input_nodes, stream);
  const int64_t nl = (int64_t)fc_.leaf_logp.size();
  hipLaunchKernelGGL(sparse_kld_leaf_grad_kernel, dim3(ceil_div(nl, 256)), dim3(256), 0, stream, d, inn.p,
                     (int)fc_.input_nodes.size(), q->d_leaf_.p, d_grad_.p, lg1, lg2);
  check_launch("sparse_kld_backward");
  PCM_HIP(hipStreamSynchronize(stream));
}

void SparseCircuit::kld_backward(pcm_circuit* q, float* gp, float* gq, int64_t n) {
  SparseCircuit* s = same_structure(this, q);
  if (n != size(0)) fail(PCM_ERR_ARG, "gradient vectors have %lld entries, circuit has %lld parameters", (long long)n, (long long)size(0));
  if (!gp || !gq) fail(PCM_ERR_ARG, "gradient pointer is null");
  const int64_t ne = std::max<int64_t>(fc_.n_edges(), 1), nl = (int64_t)fc_.leaf_logp.size();
  DevBuf<float> g1, g2, l1, l2;
  g1.alloc(ne); g2.alloc(ne); l1.alloc(nl); l2.alloc(nl);
  kld_backward_device(s, g1.p, g2.p, l1.p, l2.p);
  std::vector<float> h1, h2;
  fetch(h1, g1.p, ne, stream); fetch(h2, g2.p, ne, stream);
  const size_t ns = fc_.param2edge.size();
  for (size_t i = 0; i < ns; ++i) { gp[i] = h1[fc_.param2edge[i] - 1]; gq[i] = h2[fc_.param2edge[i] - 1]; }
  fetch(h1, l1.p, nl, stream); fetch(h2, l2.p, nl, stream);
  std::copy(h1.begin(), h1.end(), gp + ns);
  std::copy(h2.begin(), h2.end(), gq + ns);
}

__global__ void sparse_gather_params_kernel(const int32_t* __restrict__ param2edge, int64_t n_sum,
                                            const float* __restrict__ edge_vals, const float* __restrict__ leaf_vals,
                                            int64_t n_leaf, float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_sum) out[i] = edge_vals[param2edge[i]];
  else if (i < n_sum + n_leaf) out[i] = leaf_vals[i - n_sum];
}

void SparseCircuit::kld_backward_dev(pcm_circuit* q, float* d_gp, float* d_gq, int64_t n) {
  SparseCircuit* s = same_structure(this, q);
  if (n != size(0)) fail(PCM_ERR_ARG, "gradient vectors have %lld entries, circuit has %lld parameters", (long long)n, (long long)size(0));
  if (!d_gp || !d_gq) fail(PCM_ERR_ARG, "gradient pointer is null");
  const int64_t ne = std::max<int64_t>(fc_.n_edges(), 1), nl = (int64_t)fc_.leaf_logp.size();
  d_g1_.ensure(ne); d_g2_.ensure(ne); d_l1_.ensure(nl); d_l2_.ensure(nl);
  kld_backward_device(s, d_g1_.p, d_g2_.p, d_l1_.p, d_l2_.p);
  const int64_t ns = (int64_t)fc_.param2edge.size();
  const unsigned blocks = (unsigned)ceil_div(ns + nl, 256);
  hipLaunchKernelGGL(sparse_gather_params_kernel, dim3(blocks), dim3(256), 0, stream, d_param2edge_.p, ns, d_g1_.p, d_l1_.p, nl, d_gp);
  hipLaunchKernelGGL(sparse_gather_params_kernel, dim3(blocks), dim3(256), 0, stream, d_param2edge_.p, ns, d_g2_.p, d_l2_.p, nl, d_gq);
  check_launch("gather_params");
}

// ---- sampling ---------------------------------------------------------------------------

void SparseCircuit::sample_with_slots(const float* d_node_noise, const int32_t* d_noise_slot, int64_t noise_stride,
                                      const float* d_leaf_noise, int32_t batch, uint8_t* d_out) {
  if (!d_node_noise || !d_leaf_noise || !d_out) fail(PCM_ERR_ARG, "null noise or output pointer");
  if (batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", batch);
  if (!fc_.heads.empty()) fail(PCM_ERR_UNSUPPORTED, "sampling from a multi-head circuit needs a head choice");
  const int Bp = ceil_div(batch, 64) * 64;
  d_visit_.ensure((size_t)std::max<int64_t>((int64_t)fc_.num_vars, fc_.n_nodes()) * Bp);
  const int64_t nv = fc_.n_nodes() * Bp;
  hipLaunchKernelGGL(sparse_fill_u8_kernel, dim3(ceil_div(nv, 256)), dim3(256), 0, stream, d_visit_.p, nv, (uint8_t)0);
  hipLaunchKernelGGL(sparse_set_row_u8_kernel, dim3(ceil_div(Bp, 256)), dim3(256), 0, stream,
                     d_visit_.p + (size_t)(fc_.n_nodes() - 1) * Bp, Bp, (uint8_t)1);
  hipLaunchKernelGGL(sparse_fill_u8_kernel, dim3(ceil_div((int64_t)batch * fc_.num_vars, 256)), dim3(256), 0, stream, d_out,
                     (int64_t)batch * fc_.num_vars, (uint8_t)255);
  DevBuf<int64_t> e2p;
  std::vector<int64_t> e2pv = fc_.edge2param;
  if (e2pv.empty()) e2pv.push_back(0);
  e2p.upload(e2pv, stream);
  SparseDev d = SPARSE_DEV(batch, Bp, nullptr);
  for (int l = n_layers_ - 1; l >= 0; --l) {
    const int n0 = layer_node0_[l], cnt = layer_node0_[l + 1] - n0;
    hipLaunchKernelGGL(sparse_sample_kernel, dim3(cnt, Bp / 64), dim3(64), 0, stream, d, n0, d_noise_slot, e2p.p,
                       noise_stride, d_node_noise, d_leaf_noise, fc_.num_vars, d_visit_.p, d_out);
  }
  check_launch("sparse_sample");
  PCM_HIP(hipStreamSynchronize(stream));
}

void SparseCircuit::sample(const float* d_node_noise, const float* d_leaf_noise, int32_t batch, uint8_t* d_out) {
  sample_with_slots(d_node_noise, nullptr, sample_noise_size(), d_leaf_noise, batch, d_out);
}

void SparseCircuit::sample_soft_with_slots(const float* d_node_noise, const int32_t* d_noise_slot, int64_t noise_stride,
                                           float temperature, int32_t batch, float* d_out) {
  if (!d_out) fail(PCM_ERR_ARG, "output pointer is null");
  if (batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", batch);
  if (!(temperature > 0.f)) fail(PCM_ERR_ARG, "temperature must be positive");
  if (!fc_.heads.empty()) fail(PCM_ERR_UNSUPPORTED, "sampling from a multi-head circuit needs a head choice");
  ensure_batch(batch);
  const int Bp = ceil_div(batch, 64) * 64;
  d_grad_.ensure((size_t)fc_.n_nodes() * Bp);   // normaliser sums; maxima go to the value array, td to the flow array
  ensure_var_tables();
  DevBuf<int64_t> e2p;
  std::vector<int64_t> e2pv = fc_.edge2param;
  if (e2pv.empty()) e2pv.push_back(0);
  e2p.upload(e2pv, stream);
  SparseDev d = SPARSE_DEV(batch, Bp, nullptr);
  const float inv_t = 1.f / temperature;
  hipLaunchKernelGGL(sparse_soft_norm_kernel, dim3((unsigned)fc_.n_nodes(), Bp / 64), dim3(64), 0, stream, d,
                     (int)fc_.n_nodes(), d_noise_slot, e2p.p, noise_stride, d_node_noise, inv_t, d_mars_.p, d_grad_.p);
  for (int l = n_layers_ - 1; l >= 0; --l) {
    const int n0 = layer_node0_[l], cnt = layer_node0_[l + 1] - n0;
    hipLaunchKernelGGL(sparse_soft_down_kernel, dim3(cnt, Bp / 64), dim3(64), 0, stream, d, n0, (int)fc_.n_nodes() - 1,
                       d_noise_slot, e2p.p, noise_stride, d_node_noise, inv_t, d_mars_.p, d_grad_.p, d_flows_.p);
  }
  hipLaunchKernelGGL(sparse_soft_leaf_kernel, dim3(fc_.num_vars, batch), dim3(std::min(256, ceil_div(fc_.num_cats, 64) * 64)),
                     0, stream, d, d_var_ptr_.p, d_var_nodes_.p, fc_.num_vars, d_flows_.p, d_out);
  check_launch("sparse_sample_soft");
  PCM_HIP(hipStreamSynchronize(stream));
  last_batch_ = 0;       // the value / flow arrays no longer hold a batch
  flow_batch_ = 0;
  have_flows_ = false;
}

void SparseCircuit::sample_soft(const float* d_node_noise, float temperature, int32_t batch, float* d_out) {
  sample_soft_with_slots(d_node_noise, nullptr, sample_noise_size(), temperature, batch, d_out);
}

// ---- Adam ---------------------------------------------------------------------------------

void SparseCircuit::adam_step(const float* d_grad, float* d_params, float* d_m, float* d_v, float lr, float b1,
                              float b2, float eps, int t) {
  if (!d_grad || !d_params || !d_m || !d_v) fail(PCM_ERR_ARG, "null optimiser array");
  if (t < 1) fail(PCM_ERR_ARG, "step count must start at 1, got %d", t);
  const int64_t ns = (int64_t)fc_.param2edge.size();
  if (!ns) return;
  const float c1 = 1.f - std::pow(b1, (float)t), c2 = 1.f - std::pow(b2, (float)t);
  hipLaunchKernelGGL(sparse_adam_kernel, dim3(ceil_div(ns, 256)), dim3(256), 0, stream, ns, d_grad, d_params, d_m, d_v, lr,
                     b1, b2, eps, c1, c2);
  const int ng = (int)fc_.pargroup_sizes.size();
  hipLaunchKernelGGL(sparse_normalize_kernel, dim3(ceil_div(ng, 128)), dim3(128), 0, stream, ng, d_group_ptr_.p,
                     d_param2edge_.p, d_params, d_logp_.p);
  check_launch("sparse_adam");
}


// ---- Adam from flows ------------------------------------------------------------------------
// src/sgd/adam.jl:305-311 and :27-61: edge flows / batch size minus exp(logp) times their sum over the sum node,
// one thread per normalisation group, written in parameter order.
__global__ void sparse_flow_grad_kernel(int n_groups, const int32_t* __restrict__ group_ptr,
                                        const int32_t* __restrict__ param2edge, const float* __restrict__ edge_aggr,
                                        const float* __restrict__ logp, float inv_batch, float* __restrict__ grad) {
  const int gi = blockIdx.x * blockDim.x + threadIdx.x;
  if (gi >= n_groups) return;
  const int p0 = group_ptr[gi], p1 = group_ptr[gi + 1];
  float s = 0.f;
  for (int p = p0; p < p1; ++p) s += edge_aggr[param2edge[p]] * inv_batch;
  for (int p = p0; p < p1; ++p) {
    const int e = param2edge[p];
    grad[p] = edge_aggr[e] * inv_batch - expf(logp[e]) * s;
  }
}

// src/sgd/adam.jl:218-242, a wave per input node: g = flow + exp(logp) * node flow (as the source has it); the
// steps go to the auxiliary copy, never into the circuit.
__global__ __launch_bounds__(256) void sparse_leaf_adam_kernel(int64_t n_inputs, int C, const float* __restrict__ leaf,
                                                               const float* __restrict__ leaf_flow, float* __restrict__ aux_p,
                                                               float* __restrict__ aux_m, float* __restrict__ aux_v, float lr,
                                                               float b1, float b2, float eps, float c1, float c2) {
  const int lane = threadIdx.x & 63;
  const int64_t q = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (q >= n_inputs) return;
  const float* fl = leaf_flow + q * C;
  float node_flow = 0.f;
  for (int c = lane; c < C; c += 64) node_flow += fl[c];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) node_flow += __shfl_xor(node_flow, o);
  for (int c = lane; c < C; c += 64) {
    const int64_t i = q * C + c;
    const float g = fl[c] + expf(leaf[i]) * node_flow;
    const float m = b1 * aux_m[i] + (1.f - b1) * g, v = b2 * aux_v[i] + (1.f - b2) * g * g;
    aux_m[i] = m;
    aux_v[i] = v;
    aux_p[i] += lr * ((m / c1) / (sqrtf(v / c2) + eps));
  }
}

void SparseCircuit::flow_gradients(int32_t batch_size, float* d_grad) {
  if (!have_flows_) fail(PCM_ERR_STATE, "no flows have been computed on this circuit yet");
  if (!d_grad) fail(PCM_ERR_ARG, "gradient pointer is null");
  if (batch_size < 1) fail(PCM_ERR_ARG, "batch size must be positive, got %d", batch_size);
  const int ng = (int)fc_.pargroup_sizes.size();
  if (!ng) return;
  hipLaunchKernelGGL(sparse_flow_grad_kernel, dim3(ceil_div(ng, 128)), dim3(128), 0, stream, ng, d_group_ptr_.p,
                     d_param2edge_.p, d_edge_aggr_.p, d_logp_.p, 1.f / (float)batch_size, d_grad);
  check_launch("sparse_flow_grad");
}

void SparseCircuit::leaf_adam(float* d_aux_p, float* d_aux_m, float* d_aux_v, float lr, float b1, float b2, float eps, int t) {
  if (!have_flows_) fail(PCM_ERR_STATE, "no flows have been computed on this circuit yet");
  if (!d_aux_p || !d_aux_m || !d_aux_v) fail(PCM_ERR_ARG, "null optimiser array");
  if (t < 1) fail(PCM_ERR_ARG, "step count must start at 1, got %d", t);
  const int64_t ni = (int64_t)fc_.input_nodes.size();
  const float c1 = 1.f - std::pow(b1, (float)t), c2 = 1.f - std::pow(b2, (float)t);
  hipLaunchKernelGGL(sparse_leaf_adam_kernel, dim3((unsigned)ceil_div(ni, 4)), dim3(256), 0, stream, ni, fc_.num_cats,
                     d_leaf_.p, d_leaf_flow_.p, d_aux_p, d_aux_m, d_aux_v, lr, b1, b2, eps, c1, c2);
  check_launch("sparse_leaf_adam");
}

}  // namespace pcm
