// Queries on a MATRIX of parameter rows: one structure, R parameter vectors, all rows in one pass.
//
// Reference: `kld(mbpc, params1[R, n], params2[R, n])` src/queries/kld.jl:6-206, `kld_backward` :212-649,
// `gumbel_sample(mbpc, params[R, n], ...)` src/queries/sample.jl:8-383, reached from Python through
// src/utils/cuda_preallocation.jl:47-78, :189-203 with one row per example.  `norm_params = true` there
// changes the LEAF lines only (leaf parameters are probabilities: src/nodes/fixable_categorical_dist.jl
// :182-186, :216-217; sample.jl:265-268); sum edges are log-parameters either way.
//
// Layout.  A row holds its parameters in parameter-vector order (sum edges in up-edge order, then the
// input nodes' C values), so a sum node's edges and an input node's categories are contiguous in a row.
// The kernels therefore put a group of 32 lanes on one (node, row) pair, lanes over the node's edges (or
// a wave over an input node's categories): every request is a contiguous run of one row, whatever R is.
// Matrices are taken with element strides; anything but unit stride along the parameters is first turned
// into that layout (the reference's column-major [R, n] arrays pass through a tiled transposition).
// Node quantities (KL, gradient, top-down probability) are [R][n_nodes]; the chain of layers is one
// launch per layer with the rows in the grid's second dimension.  Every sum is a fixed-order tree over
// the lanes: results do not depend on scheduling.
#include "sparse_engine.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>

namespace pcm {

namespace {

void check_launch_r(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

struct RowsDev {
  const uint8_t* type;
  const int32_t *order, *node_e0, *node_e1, *e_parent, *e_prime, *e_sub, *in_ptr, *in_edge, *e2p, *p2e, *input_nodes, *in_var;
  int64_t n_nodes, n_edges, n_sum, n_par;
  int32_t C, n_inputs;
};

constexpr int kGroup = 32;               // lanes per (node, row) pair
constexpr int kGroupsPerBlock = 8;
constexpr float kNormEps = 1e-8f;

template <typename T>
__device__ __forceinline__ T group_sum(T v) {
#pragma unroll
  for (int o = kGroup / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kGroup);
  return v;
}
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int o = kGroup / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kGroup));
  return v;
}

// ---- layout: [rows][n] with unit stride along n <-> any element strides -----------------------------
// kIn: dst[r * n + p] = src[r * sr + p * sp]; else src/dst swapped.  32 x 32 tiles through LDS, so both sides move in runs
// when one of the strides is 1.
template <bool kIn>
__global__ __launch_bounds__(256) void rows_relayout_kernel(float* __restrict__ packed, float* __restrict__ strided, int64_t sr,
                                                            int64_t sp, int rows, int64_t n) {
  __shared__ float tile[32][33];
  const int64_t p0 = (int64_t)blockIdx.x * 32;
  const int r0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  if (kIn) {
    // read with the row index fastest (good for sr == 1), write with p fastest
    for (int q = ty; q < 32; q += 8) {
      const int r = r0 + tx;
      const int64_t p = p0 + q;
      if (r < rows && p < n) tile[q][tx] = strided[(int64_t)r * sr + p * sp];
    }
    __syncthreads();
    for (int q = ty; q < 32; q += 8) {
      const int r = r0 + q;
      const int64_t p = p0 + tx;
      if (r < rows && p < n) packed[(int64_t)r * n + p] = tile[tx][q];
    }
  } else {
    for (int q = ty; q < 32; q += 8) {
      const int r = r0 + q;
      const int64_t p = p0 + tx;
      if (r < rows && p < n) tile[tx][q] = packed[(int64_t)r * n + p];
    }
    __syncthreads();
    for (int q = ty; q < 32; q += 8) {
      const int r = r0 + tx;
      const int64_t p = p0 + q;
      if (r < rows && p < n) strided[(int64_t)r * sr + p * sp] = tile[q][tx];
    }
  }
}

// ---- KL, bottom-up --------------------------------------------------------------------------------
// Leaf term, a wave per (input node, row): fixable_categorical_dist.jl:182-192.
template <bool kNorm>
__global__ __launch_bounds__(256) void rows_kld_leaf_kernel(RowsDev d, const float* __restrict__ P1, const float* __restrict__ P2,
                                                            float* __restrict__ klds) {
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int r = blockIdx.y;
  if (i >= d.n_inputs) return;
  const float* a = P1 + (size_t)r * d.n_par + d.n_sum + (size_t)i * d.C;
  const float* b = P2 + (size_t)r * d.n_par + d.n_sum + (size_t)i * d.C;
  float acc = 0.f;
  for (int c = lane; c < d.C; c += 64) {
    const float x = a[c], y = b[c];
    acc += kNorm ? x * (logf(x + kNormEps) - logf(y + kNormEps)) : expf(x) * (x - y);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) klds[(size_t)r * d.n_nodes + d.input_nodes[i]] = acc;
}

// One layer of inner nodes, a lane group per (node, row): kld.jl:95-128.
__global__ __launch_bounds__(kGroup * kGroupsPerBlock) void rows_kld_up_kernel(RowsDev d, int n0, int n1,
                                                                               const float* __restrict__ P1,
                                                                               const float* __restrict__ P2,
                                                                               float* __restrict__ klds,
                                                                               float* __restrict__ edge_klds) {
  const int l = threadIdx.x % kGroup;
  const int i = n0 + blockIdx.x * kGroupsPerBlock + threadIdx.x / kGroup;
  const int r = blockIdx.y;
  if (i >= n1) return;
  const int n = d.order[i];
  const bool issum = d.type[n] == kSum;
  const float* p1 = P1 + (size_t)r * d.n_par;
  const float* p2 = P2 + (size_t)r * d.n_par;
  float* kl = klds + (size_t)r * d.n_nodes;
  float acc = 0.f;
  for (int e = d.node_e0[n] + l; e < d.node_e1[n]; e += kGroup) {
    float k = kl[d.e_prime[e]];
    const int s = d.e_sub[e];
    if (s >= 0) k += kl[s];
    if (issum) {
      const int pid = d.e2p[e];
      const float a = p1[pid], b = p2[pid];
      k = expf(a) * (k + a - b);
    }
    if (edge_klds) edge_klds[(size_t)r * d.n_edges + e] = k;
    acc += k;
  }
  acc = group_sum(acc);
  if (l == 0) kl[n] = acc;
}

__global__ void rows_take_root_kernel(const float* __restrict__ node_vals, int64_t n_nodes, int rows, float* __restrict__ out) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < rows) out[r] = node_vals[(size_t)r * n_nodes + n_nodes - 1];
}

// ---- KL, top-down ---------------------------------------------------------------------------------
// Node gradients of one layer, a lane group per (node, row) over the node's incoming edges: kld.jl:262-300.
__global__ __launch_bounds__(kGroup * kGroupsPerBlock) void rows_kld_down_kernel(RowsDev d, int n0, int n1,
                                                                                 const float* __restrict__ P1,
                                                                                 float* __restrict__ grads) {
  const int l = threadIdx.x % kGroup;
  const int i = n0 + blockIdx.x * kGroupsPerBlock + threadIdx.x / kGroup;
  const int r = blockIdx.y;
  if (i >= n1) return;
  const int n = d.order[i];
  const float* p1 = P1 + (size_t)r * d.n_par;
  float* g = grads + (size_t)r * d.n_nodes;
  float acc = 0.f;
  for (int q = d.in_ptr[n] + l; q < d.in_ptr[n + 1]; q += kGroup) {
    const int e = d.in_edge[q] >> 1;
    const int p = d.e_parent[e];
    acc += g[p] * (d.type[p] == kSum ? expf(p1[d.e2p[e]]) : 1.f);
  }
  acc = group_sum(acc);
  if (l == 0) g[n] = acc + (n == d.n_nodes - 1 ? 1.f : 0.f);
}

// Gradients in parameter order.  Sum parameters: kld.jl:271-272; leaf parameters as the source writes them,
// fixable_categorical_dist.jl:216-219.
template <bool kNorm>
__global__ __launch_bounds__(256) void rows_kld_param_grad_kernel(RowsDev d, const float* __restrict__ P1,
                                                                  const float* __restrict__ P2, const float* __restrict__ grads,
                                                                  const float* __restrict__ edge_klds, float* __restrict__ G1,
                                                                  float* __restrict__ G2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int r = blockIdx.y;
  if (i >= d.n_par) return;
  const size_t at = (size_t)r * d.n_par + i;
  const float a = P1[at], b = P2[at];
  const float* g = grads + (size_t)r * d.n_nodes;
  if (i < d.n_sum) {
    const int e = d.p2e[i];
    const float gp = g[d.e_parent[e]], pr = expf(a);
    G1[at] = gp * (edge_klds[(size_t)r * d.n_edges + e] + pr);
    G2[at] = -gp * pr;
  } else {
    const float gn = g[d.input_nodes[(i - d.n_sum) / d.C]];
    if (kNorm) {
      G1[at] = gn * (logf(a + kNormEps) - logf(b + kNormEps) + 1.f);
      G2[at] = gn * a / (b + kNormEps);
    } else {
      G1[at] = gn * (a - b + 1.f);
      G2[at] = gn * expf(a - b);
    }
  }
}

// ---- relaxed sampling -------------------------------------------------------------------------------
// Normaliser of every sum node's edge weights exp((logp + g) / T), kept as (maximum, sum relative to it):
// sample.jl:37-51.  noise: [rows][n_sum] or null.
__global__ __launch_bounds__(kGroup * kGroupsPerBlock) void rows_soft_norm_kernel(RowsDev d, const float* __restrict__ P,
                                                                                  const float* __restrict__ noise, float inv_t,
                                                                                  float* __restrict__ emax,
                                                                                  float* __restrict__ esum) {
  const int l = threadIdx.x % kGroup;
  const int64_t n = (int64_t)blockIdx.x * kGroupsPerBlock + threadIdx.x / kGroup;
  const int r = blockIdx.y;
  if (n >= d.n_nodes || d.type[n] != kSum) return;
  const float* p = P + (size_t)r * d.n_par;
  const float* g = noise ? noise + (size_t)r * d.n_sum : nullptr;
  float m = -INFINITY;
  for (int e = d.node_e0[n] + l; e < d.node_e1[n]; e += kGroup) {
    const int pid = d.e2p[e];
    m = fmaxf(m, (p[pid] + (g ? g[pid] : 0.f)) * inv_t);
  }
  m = group_max(m);
  float s = 0.f;
  for (int e = d.node_e0[n] + l; e < d.node_e1[n]; e += kGroup) {
    const int pid = d.e2p[e];
    s += expf((p[pid] + (g ? g[pid] : 0.f)) * inv_t - m);
  }
  s = group_sum(s);
  if (l == 0) { emax[(size_t)r * d.n_nodes + n] = m; esum[(size_t)r * d.n_nodes + n] = s; }
}

// Top-down probabilities of one layer: sample.jl:105-140.
__global__ __launch_bounds__(kGroup * kGroupsPerBlock) void rows_soft_down_kernel(RowsDev d, int n0, int n1,
                                                                                  const float* __restrict__ P,
                                                                                  const float* __restrict__ noise, float inv_t,
                                                                                  const float* __restrict__ emax,
                                                                                  const float* __restrict__ esum,
                                                                                  float* __restrict__ td) {
  const int l = threadIdx.x % kGroup;
  const int i = n0 + blockIdx.x * kGroupsPerBlock + threadIdx.x / kGroup;
  const int r = blockIdx.y;
  if (i >= n1) return;
  const int n = d.order[i];
  const float* p = P + (size_t)r * d.n_par;
  const float* g = noise ? noise + (size_t)r * d.n_sum : nullptr;
  float* t = td + (size_t)r * d.n_nodes;
  const float* em = emax + (size_t)r * d.n_nodes;
  const float* es = esum + (size_t)r * d.n_nodes;
  float acc = 0.f;
  for (int q = d.in_ptr[n] + l; q < d.in_ptr[n + 1]; q += kGroup) {
    const int e = d.in_edge[q] >> 1;
    const int par = d.e_parent[e];
    float f = t[par];
    if (d.type[par] == kSum) {
      const int pid = d.e2p[e];
      f *= expf((p[pid] + (g ? g[pid] : 0.f)) * inv_t - em[par]) / es[par];
    }
    acc += f;
  }
  acc = group_sum(acc);
  if (l == 0) t[n] = acc + (n == d.n_nodes - 1 ? 1.f : 0.f);
}

// out[r][v][c] = sum over the variable's input nodes of td * (their distribution): sample.jl:262-284.
template <bool kNorm>
__global__ __launch_bounds__(256) void rows_soft_leaf_kernel(RowsDev d, const int32_t* __restrict__ var_ptr,
                                                             const int32_t* __restrict__ var_inputs, int V,
                                                             const float* __restrict__ P, const float* __restrict__ td,
                                                             float* __restrict__ out) {
  const int v = blockIdx.x, r = blockIdx.y;
  const float* p = P + (size_t)r * d.n_par + d.n_sum;
  const float* t = td + (size_t)r * d.n_nodes;
  for (int c = threadIdx.x; c < d.C; c += blockDim.x) {
    float acc = 0.f;
    for (int q = var_ptr[v]; q < var_ptr[v + 1]; ++q) {
      const int i = var_inputs[q];   // position among the input nodes
      const float x = p[(size_t)i * d.C + c];
      acc += t[d.input_nodes[i]] * (kNorm ? x : expf(x));
    }
    out[((size_t)r * V + v) * d.C + c] = acc;
  }
}

// ---- relaxed sampling, reverse pass --------------------------------------------------------------------
// Input nodes, a wave per (input node, row): gumbel_input_sample_up_kernel, sample.jl:531-598.  The leaf part
// of the gradient matrix is the gradient with respect to the PROBABILITY of the category (og * td), with
// probability-valued parameters or not, as the source writes it (:560-570); the node's own gradient is the
// output gradient weighted by its distribution.
template <bool kNorm>
__global__ __launch_bounds__(256) void rows_soft_back_leaf_kernel(RowsDev d, int V, const float* __restrict__ P,
                                                                  const float* __restrict__ td, const float* __restrict__ og,
                                                                  float* __restrict__ grads, float* __restrict__ G) {
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int r = blockIdx.y;
  if (i >= d.n_inputs) return;
  const int node = d.input_nodes[i];
  const size_t at = (size_t)r * d.n_par + d.n_sum + (size_t)i * d.C;
  const float* o = og + ((size_t)r * V + d.in_var[node]) * d.C;
  const float t = td[(size_t)r * d.n_nodes + node];
  float acc = 0.f;
  for (int c = lane; c < d.C; c += 64) {
    const float x = P[at + c], oc = o[c];
    G[at + c] = oc * t;
    acc += (kNorm ? x : expf(x)) * oc;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if (lane == 0) grads[(size_t)r * d.n_nodes + node] = acc;
}

// One layer of inner nodes, children first, a lane group per (node, row): gumbel_params_up_layer_kernel,
// sample.jl:391-480.  A sum node's edges share the node's probability as w = softmax((logp + g) / T); the
// gradient passes through that softmax: edge gradient (child_grad * td - sum_e' child_grad' * td * w') * w / T
// (without the last w when the gradient is wanted per probability, :466-469).  The group owns the node, so
// the two sums are lane reductions: nothing is accumulated in memory.
__global__ __launch_bounds__(kGroup * kGroupsPerBlock) void rows_soft_back_up_kernel(
    RowsDev d, int n0, int n1, const float* __restrict__ P, const float* __restrict__ noise, float inv_t,
    const float* __restrict__ emax, const float* __restrict__ esum, const float* __restrict__ td, int wrt_log,
    float* __restrict__ grads, float* __restrict__ G) {
  const int l = threadIdx.x % kGroup;
  const int i = n0 + blockIdx.x * kGroupsPerBlock + threadIdx.x / kGroup;
  const int r = blockIdx.y;
  if (i >= n1) return;
  const int n = d.order[i];
  const bool issum = d.type[n] == kSum;
  const float* p = P + (size_t)r * d.n_par;
  const float* g = noise ? noise + (size_t)r * d.n_sum : nullptr;
  float* gr = grads + (size_t)r * d.n_nodes;
  const float t = td[(size_t)r * d.n_nodes + n];
  const float em = issum ? emax[(size_t)r * d.n_nodes + n] : 0.f, es = issum ? esum[(size_t)r * d.n_nodes + n] : 1.f;
  float acc = 0.f, cum = 0.f;
  for (int e = d.node_e0[n] + l; e < d.node_e1[n]; e += kGroup) {
    float child = gr[d.e_prime[e]];
    const int s = d.e_sub[e];
    if (s >= 0) child += gr[s];
    if (issum) {
      const int pid = d.e2p[e];
      const float w = expf((p[pid] + (g ? g[pid] : 0.f)) * inv_t - em) / es;
      cum += child * t * w;
      child *= w;
    }
    acc += child;
  }
  acc = group_sum(acc);
  if (issum) {
    cum = group_sum(cum);
    float* out = G + (size_t)r * d.n_par;
    for (int e = d.node_e0[n] + l; e < d.node_e1[n]; e += kGroup) {
      float child = gr[d.e_prime[e]];
      const int s = d.e_sub[e];
      if (s >= 0) child += gr[s];
      const int pid = d.e2p[e];
      const float w = expf((p[pid] + (g ? g[pid] : 0.f)) * inv_t - em) / es;
      out[pid] = (child * t - cum) * (wrt_log ? w : 1.f) * inv_t;
    }
  }
  if (l == 0) gr[n] = acc;
}

}  // namespace

// ---- host -------------------------------------------------------------------------------------------

struct SparseCircuit::RowsState {
  DevBuf<int32_t> e2p, input_nodes, var_ptr, var_inputs;
  DevBuf<float> pk1, pk2, pg1, pg2;        // matrices re-laid out to unit parameter stride
  DevBuf<float> node_a, node_b, node_c, node_d, edge_a;   // [rows][n_nodes] x 4, [rows][n_edges]
};

SparseCircuit::~SparseCircuit() {}

static RowsDev rows_dev(const SparseCircuit& c, const FlatCircuit& fc, const SparseCircuit::RowsState& st,
                        const uint8_t* type, const int32_t* order, const int32_t* e0, const int32_t* e1, const int32_t* ep,
                        const int32_t* epr, const int32_t* es, const int32_t* in_ptr, const int32_t* in_edge,
                        const int32_t* p2e, const int32_t* in_var) {
  (void)c;
  RowsDev d;
  d.in_var = in_var;
  d.type = type; d.order = order; d.node_e0 = e0; d.node_e1 = e1; d.e_parent = ep; d.e_prime = epr; d.e_sub = es;
  d.in_ptr = in_ptr; d.in_edge = in_edge; d.e2p = st.e2p.p; d.p2e = p2e; d.input_nodes = st.input_nodes.p;
  d.n_nodes = fc.n_nodes(); d.n_edges = fc.n_edges(); d.n_sum = (int64_t)fc.param2edge.size();
  d.n_par = d.n_sum + (int64_t)fc.leaf_logp.size();
  d.C = fc.num_cats; d.n_inputs = (int32_t)fc.input_nodes.size();
  return d;
}

SparseCircuit::RowsState& SparseCircuit::rows_state() {
  if (!rows_) {
    rows_.reset(new RowsState);
    std::vector<int32_t> e2p(std::max<int64_t>(fc_.n_edges(), 1), -1);
    for (int64_t e = 0; e < fc_.n_edges(); ++e) e2p[e] = (int32_t)fc_.edge2param[e] - 1;
    rows_->e2p.upload(e2p, stream);
    rows_->input_nodes.upload(fc_.input_nodes, stream);
    std::vector<int32_t> vp(fc_.num_vars + 1, 0), vi(fc_.input_nodes.size());
    for (int32_t n : fc_.input_nodes) vp[fc_.in_var[n] + 1]++;
    for (int v = 0; v < fc_.num_vars; ++v) vp[v + 1] += vp[v];
    std::vector<int32_t> fill(vp.begin(), vp.end() - 1);
    for (size_t i = 0; i < fc_.input_nodes.size(); ++i) vi[fill[fc_.in_var[fc_.input_nodes[i]]]++] = (int32_t)i;
    if (vi.empty()) vi.push_back(0);
    rows_->var_ptr.upload(vp, stream);
    rows_->var_inputs.upload(vi, stream);
  }
  return *rows_;
}

#define ROWS_DEV(st)                                                                                              \
  rows_dev(*this, fc_, st, d_type_.p, d_order_.p, d_node_e0_.p, d_node_e1_.p, d_e_parent_.p, d_e_prime_.p, d_e_sub_.p, \
           d_in_ptr_.p, d_in_edge_.p, d_param2edge_.p, d_in_var_.p)

namespace {
void check_rows_args(const SparseCircuit& c, const FlatCircuit& fc, const void* p, int64_t sr, int64_t sp, int rows) {
  (void)c;
  if (!fc.heads.empty()) fail(PCM_ERR_UNSUPPORTED, "queries on parameter rows are defined for single-root circuits");
  if (!p) fail(PCM_ERR_ARG, "parameter matrix is null");
  if (rows < 1) fail(PCM_ERR_ARG, "need at least one parameter row, got %d", rows);
  if (rows > 65535) fail(PCM_ERR_UNSUPPORTED, "at most 65535 parameter rows per call, got %d", rows);
  if (sr == 0 || sp == 0) fail(PCM_ERR_ARG, "parameter matrix strides must not be zero");
}

const float* packed_in(const float* m, int64_t sr, int64_t sp, int rows, int64_t n, DevBuf<float>& tmp, hipStream_t s) {
  return rows_packed_in(m, sr, sp, rows, n, tmp, s);
}
}  // namespace

// the matrix with unit stride along the parameters: itself, or a re-laid-out copy in `tmp`
const float* rows_packed_in(const float* m, int64_t sr, int64_t sp, int rows, int64_t n, DevBuf<float>& tmp, hipStream_t s) {
  if (sp == 1 && sr == n) return m;
  tmp.ensure((size_t)rows * n);
  hipLaunchKernelGGL(rows_relayout_kernel<true>, dim3((unsigned)ceil_div(n, 32), ceil_div(rows, 32)), dim3(256), 0, s, tmp.p,
                     const_cast<float*>(m), sr, sp, rows, n);
  return tmp.p;
}

// ... and back: a packed [rows][n] result into the caller's matrix
void rows_unpack_out(float* packed, float* m, int64_t sr, int64_t sp, int rows, int64_t n, hipStream_t s) {
  hipLaunchKernelGGL(rows_relayout_kernel<false>, dim3((unsigned)ceil_div(n, 32), ceil_div(rows, 32)), dim3(256), 0, s, packed, m,
                     sr, sp, rows, n);
}

// klds [rows] on the device; with_edges keeps what the reverse pass needs
void SparseCircuit::kld_rows_forward(const float* p1, const float* p2, int rows, bool norm, bool with_edges) {
  RowsState& st = rows_state();
  const RowsDev d = ROWS_DEV(st);
  st.node_a.ensure((size_t)rows * d.n_nodes);
  if (with_edges) st.edge_a.ensure((size_t)rows * std::max<int64_t>(d.n_edges, 1));
  const dim3 lgrid(ceil_div(d.n_inputs, 4), rows);
  if (norm) hipLaunchKernelGGL(rows_kld_leaf_kernel<true>, lgrid, dim3(256), 0, stream, d, p1, p2, st.node_a.p);
  else hipLaunchKernelGGL(rows_kld_leaf_kernel<false>, lgrid, dim3(256), 0, stream, d, p1, p2, st.node_a.p);
  for (int l = 1; l < n_layers_; ++l) {
    const int n0 = layer_node0_[l], n1 = layer_node0_[l + 1];
    hipLaunchKernelGGL(rows_kld_up_kernel, dim3(ceil_div(n1 - n0, kGroupsPerBlock), rows), dim3(kGroup * kGroupsPerBlock), 0,
                       stream, d, n0, n1, p1, p2, st.node_a.p, with_edges ? st.edge_a.p : (float*)nullptr);
  }
  check_launch_r("rows_kld_up");
}

void SparseCircuit::kld_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm,
                             float* d_out) {
  check_rows_args(*this, fc_, d_p1, sr, sp, rows);
  if (!d_p2 || !d_out) fail(PCM_ERR_ARG, "parameter matrix or output pointer is null");
  if (fc_.layer[fc_.n_nodes() - 1] == 0) fail(PCM_ERR_UNSUPPORTED, "the circuit has no inner node");
  RowsState& st = rows_state();
  const int64_t n = size(0);
  const float* p1 = packed_in(d_p1, sr, sp, rows, n, st.pk1, stream);
  const float* p2 = packed_in(d_p2, sr, sp, rows, n, st.pk2, stream);
  kld_rows_forward(p1, p2, rows, norm, false);
  hipLaunchKernelGGL(rows_take_root_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, stream, st.node_a.p, fc_.n_nodes(), rows,
                     d_out);
  check_launch_r("rows_take_root");
}

void SparseCircuit::kld_backward_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm,
                                      float* d_g1, float* d_g2, float* d_klds) {
  check_rows_args(*this, fc_, d_p1, sr, sp, rows);
  if (!d_p2 || !d_g1 || !d_g2) fail(PCM_ERR_ARG, "parameter or gradient matrix is null");
  if (fc_.layer[fc_.n_nodes() - 1] == 0) fail(PCM_ERR_UNSUPPORTED, "the circuit has no inner node");
  RowsState& st = rows_state();
  const int64_t n = size(0);
  const float* p1 = packed_in(d_p1, sr, sp, rows, n, st.pk1, stream);
  const float* p2 = packed_in(d_p2, sr, sp, rows, n, st.pk2, stream);
  kld_rows_forward(p1, p2, rows, norm, true);
  if (d_klds)
    hipLaunchKernelGGL(rows_take_root_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, stream, st.node_a.p, fc_.n_nodes(), rows,
                       d_klds);
  const RowsDev d = ROWS_DEV(st);
  st.node_b.ensure((size_t)rows * d.n_nodes);
  for (int l = n_layers_ - 1; l >= 0; --l) {
    const int n0 = layer_node0_[l], n1 = layer_node0_[l + 1];
    hipLaunchKernelGGL(rows_kld_down_kernel, dim3(ceil_div(n1 - n0, kGroupsPerBlock), rows), dim3(kGroup * kGroupsPerBlock), 0,
                       stream, d, n0, n1, p1, st.node_b.p);
  }
  const bool direct = sp == 1 && sr == n;
  float* g1 = d_g1;
  float* g2 = d_g2;
  if (!direct) {
    st.pg1.ensure((size_t)rows * n);
    st.pg2.ensure((size_t)rows * n);
    g1 = st.pg1.p;
    g2 = st.pg2.p;
  }
  const dim3 pgrid((unsigned)ceil_div(n, 256), rows);
  if (norm) hipLaunchKernelGGL(rows_kld_param_grad_kernel<true>, pgrid, dim3(256), 0, stream, d, p1, p2, st.node_b.p, st.edge_a.p, g1, g2);
  else hipLaunchKernelGGL(rows_kld_param_grad_kernel<false>, pgrid, dim3(256), 0, stream, d, p1, p2, st.node_b.p, st.edge_a.p, g1, g2);
  if (!direct) {
    const dim3 tgrid((unsigned)ceil_div(n, 32), ceil_div(rows, 32));
    hipLaunchKernelGGL(rows_relayout_kernel<false>, tgrid, dim3(256), 0, stream, g1, d_g1, sr, sp, rows, n);
    hipLaunchKernelGGL(rows_relayout_kernel<false>, tgrid, dim3(256), 0, stream, g2, d_g2, sr, sp, rows, n);
  }
  check_launch_r("rows_kld_backward");
}

// emax / esum / td of every node and row (node_a, node_b, node_c): the top-down half both directions share
void SparseCircuit::soft_rows_down(const float* p, int rows, const float* d_noise, float inv_t) {
  RowsState& st = rows_state();
  const RowsDev d = ROWS_DEV(st);
  st.node_a.ensure((size_t)rows * d.n_nodes);
  st.node_b.ensure((size_t)rows * d.n_nodes);
  st.node_c.ensure((size_t)rows * d.n_nodes);
  hipLaunchKernelGGL(rows_soft_norm_kernel, dim3((unsigned)ceil_div(d.n_nodes, kGroupsPerBlock), rows),
                     dim3(kGroup * kGroupsPerBlock), 0, stream, d, p, d_noise, inv_t, st.node_a.p, st.node_b.p);
  for (int l = n_layers_ - 1; l >= 0; --l) {
    const int n0 = layer_node0_[l], n1 = layer_node0_[l + 1];
    hipLaunchKernelGGL(rows_soft_down_kernel, dim3(ceil_div(n1 - n0, kGroupsPerBlock), rows), dim3(kGroup * kGroupsPerBlock), 0,
                       stream, d, n0, n1, p, d_noise, inv_t, st.node_a.p, st.node_b.p, st.node_c.p);
  }
}

void SparseCircuit::gumbel_sample_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                       float temperature, bool norm, float* d_out) {
  check_rows_args(*this, fc_, d_params, sr, sp, rows);
  if (!d_out) fail(PCM_ERR_ARG, "output pointer is null");
  if (!(temperature > 0.f)) fail(PCM_ERR_ARG, "temperature must be positive");
  RowsState& st = rows_state();
  const int64_t n = size(0);
  const float* p = packed_in(d_params, sr, sp, rows, n, st.pk1, stream);
  soft_rows_down(p, rows, d_noise, 1.f / temperature);
  const RowsDev d = ROWS_DEV(st);
  const dim3 lgrid(fc_.num_vars, rows);
  const int threads = std::min(256, ceil_div(fc_.num_cats, 64) * 64);
  if (norm) hipLaunchKernelGGL(rows_soft_leaf_kernel<true>, lgrid, dim3(threads), 0, stream, d, st.var_ptr.p, st.var_inputs.p,
                               fc_.num_vars, p, st.node_c.p, d_out);
  else hipLaunchKernelGGL(rows_soft_leaf_kernel<false>, lgrid, dim3(threads), 0, stream, d, st.var_ptr.p, st.var_inputs.p,
                          fc_.num_vars, p, st.node_c.p, d_out);
  check_launch_r("rows_gumbel_sample");
}

void SparseCircuit::gumbel_sample_backward_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                                float temperature, bool norm, bool wrt_log, const float* d_out_grad,
                                                float* d_grads) {
  check_rows_args(*this, fc_, d_params, sr, sp, rows);
  if (!d_out_grad || !d_grads) fail(PCM_ERR_ARG, "gradient pointer is null");
  if (!(temperature > 0.f)) fail(PCM_ERR_ARG, "temperature must be positive");
  RowsState& st = rows_state();
  const int64_t n = size(0);
  const float* p = packed_in(d_params, sr, sp, rows, n, st.pk1, stream);
  const float inv_t = 1.f / temperature;
  soft_rows_down(p, rows, d_noise, inv_t);
  const RowsDev d = ROWS_DEV(st);
  st.node_d.ensure((size_t)rows * d.n_nodes);
  const bool direct = sp == 1 && sr == n;
  float* g = d_grads;
  if (!direct) {
    st.pg1.ensure((size_t)rows * n);
    g = st.pg1.p;
  }
  const dim3 lgrid(ceil_div(d.n_inputs, 4), rows);
  if (norm) hipLaunchKernelGGL(rows_soft_back_leaf_kernel<true>, lgrid, dim3(256), 0, stream, d, fc_.num_vars, p, st.node_c.p,
                               d_out_grad, st.node_d.p, g);
  else hipLaunchKernelGGL(rows_soft_back_leaf_kernel<false>, lgrid, dim3(256), 0, stream, d, fc_.num_vars, p, st.node_c.p,
                          d_out_grad, st.node_d.p, g);
  for (int l = 1; l < n_layers_; ++l) {
    const int n0 = layer_node0_[l], n1 = layer_node0_[l + 1];
    hipLaunchKernelGGL(rows_soft_back_up_kernel, dim3(ceil_div(n1 - n0, kGroupsPerBlock), rows), dim3(kGroup * kGroupsPerBlock), 0,
                       stream, d, n0, n1, p, d_noise, inv_t, st.node_a.p, st.node_b.p, st.node_c.p, wrt_log ? 1 : 0, st.node_d.p, g);
  }
  if (!direct) {
    const dim3 tgrid((unsigned)ceil_div(n, 32), ceil_div(rows, 32));
    hipLaunchKernelGGL(rows_relayout_kernel<false>, tgrid, dim3(256), 0, stream, g, d_grads, sr, sp, rows, n);
  }
  check_launch_r("rows_gumbel_sample_backward");
}

}  // namespace pcm
