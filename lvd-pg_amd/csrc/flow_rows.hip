// Per-example normalised flows and normalize_params on parameter rows: the first call of the reference's
// variational loop (src/models/pc_vae.py:77 -> `normalized_flows_with_prealloc`, src/utils/cuda_preallocation.jl:292-308).
//
//   per_sample_normalized_flows (src/queries/flow.jl:417-464): forward + backward pass of a batch without touching
//   the accumulators, then for every example a vector in parameter order:
//     sum parameter (map_flows_kernel, :496-528)        log(f / (g + 1e-8) + 1e-8), f the example's flow over the edge,
//                                                       g the flow over all edges of the same sum node
//     input parameter (map_input_flows_kernel, :549-593) log(f_c / sum_c f_c), where the node's flow sits in one slot
//                                                       (get_edge_flow, src/nodes/fixable_categorical_dist.jl:162-176)
//   The reference accumulates g with float atomics behind a block-level barrier; here a thread owns a (sum node,
//   example) pair and folds the node's edges itself.
//
//   normalize_params (src/misc.jl:448-498): every input node's entries exp'd and divided by their sum, every sum
//   node's entries minus the log of the sum of their exponentials; undo: input entries p > 0 -> log(p + 1e-6).
#include <hip/hip_runtime.h>

#include "sparse_engine.hpp"

namespace pcm {

static void check_launch_f(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

// thread = (sum node, example); the node's parameters are p0 .. p1-1, side by side in the parameter vector
__global__ __launch_bounds__(256) void flow_rows_sum_kernel(int n_groups, const int32_t* __restrict__ group_ptr,
                                                            const int32_t* __restrict__ param2edge,
                                                            const int32_t* __restrict__ e_parent, const int32_t* __restrict__ e_prime,
                                                            const int32_t* __restrict__ e_sub, const float* __restrict__ logp,
                                                            const float* __restrict__ mars, const float* __restrict__ flows,
                                                            int B, int Bp, float* __restrict__ out, int64_t sr, int64_t sp) {
  const int b = blockIdx.x * 64 + (threadIdx.x & 63);
  const int gi = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (gi >= n_groups || b >= B) return;
  const int p0 = group_ptr[gi], p1 = group_ptr[gi + 1];
  const int parent = e_parent[param2edge[p0]];
  const float fpar = flows[(size_t)parent * Bp + b], mpar = mars[(size_t)parent * Bp + b];
  auto edge_flow = [&](int p) {
    const int e = param2edge[p];
    const int sub = e_sub[e];
    float v = mars[(size_t)e_prime[e] * Bp + b] + logp[e];
    if (sub >= 0) v += mars[(size_t)sub * Bp + b];
    // a parent without flow (or of probability zero) passes none on, whatever its children's values
    return fpar > 0.f ? fpar * __expf(v - mpar) : 0.f;
  };
  float g = 1e-8f;
  for (int p = p0; p < p1; ++p) g += edge_flow(p);
  for (int p = p0; p < p1; ++p) out[(int64_t)b * sr + (int64_t)p * sp] = __logf(edge_flow(p) / g + 1e-8f);
}

// thread = (input node, example): C entries, one of them log(f / f), the others log(0 / f)
__global__ __launch_bounds__(256) void flow_rows_input_kernel(int n_inputs, const int32_t* __restrict__ input_nodes,
                                                              const int32_t* __restrict__ in_var, const uint8_t* __restrict__ xb,
                                                              const float* __restrict__ flows, int B, int Bp, int C, int as_written,
                                                              int64_t first, float* __restrict__ out, int64_t sr, int64_t sp) {
  const int b = blockIdx.x * 64 + (threadIdx.x & 63);
  const int i = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (i >= n_inputs || b >= B) return;
  const int n = input_nodes[i];
  const float f = flows[(size_t)n * Bp + b];
  const int x = xb[(size_t)in_var[n] * Bp + b];
  const int slot = as_written ? x - 1 : x;   // (the source compares the 0-based category with the 1-based parameter index)
  const float total = slot >= 0 ? f : 0.f;
  float* o = out + (int64_t)b * sr + (first + (int64_t)i * C) * sp;
  for (int c = 0; c < C; ++c) o[(int64_t)c * sp] = __logf((c == slot ? f : 0.f) / total);   // 0/0 = NaN where nothing lands
}

void SparseCircuit::normalized_flows(const BatchRef& b, float* d_out, int64_t sr, int64_t sp, bool as_written) {
  if (!d_out) fail(PCM_ERR_ARG, "output pointer is null");
  if (!fc_.heads.empty())
    fail(PCM_ERR_UNSUPPORTED, "per-example normalised flows are defined for single-root circuits (src/queries/flow.jl:417)");
  if (sr < 1 || sp < 1) fail(PCM_ERR_ARG, "strides must be positive");
  run_forward(&b, nullptr);
  run_flows(b.batch, nullptr, 0.f, nullptr, nullptr, false);
  const int Bp = ceil_div(b.batch, 64) * 64;
  const int ng = (int)fc_.pargroup_sizes.size();
  if (ng > 0) {
    hipLaunchKernelGGL(flow_rows_sum_kernel, dim3(Bp / 64, ceil_div(ng, 4)), dim3(256), 0, stream, ng, d_group_ptr_.p,
                       d_param2edge_.p, d_e_parent_.p, d_e_prime_.p, d_e_sub_.p, d_logp_.p, d_mars_.p, d_flows_.p, b.batch, Bp,
                       d_out, sr, sp);
    check_launch_f("flow_rows_sum");
  }
  const int ni = (int)fc_.input_nodes.size();
  if (ni > 0) {
    if (d_input_nodes_.n == 0) d_input_nodes_.upload(fc_.input_nodes, stream);
    hipLaunchKernelGGL(flow_rows_input_kernel, dim3(Bp / 64, ceil_div(ni, 4)), dim3(256), 0, stream, ni, d_input_nodes_.p,
                       d_in_var_.p, d_visit_.p, d_flows_.p, b.batch, Bp, fc_.num_cats, as_written ? 1 : 0,
                       (int64_t)fc_.param2edge.size(), d_out, sr, sp);
    check_launch_f("flow_rows_input");
  }
}

// thread = (group, row): a sum node's parameters (log-normalised) or an input node's entries (exp-normalised / undone)
__global__ __launch_bounds__(256) void normalize_rows_kernel(int n_groups, const int32_t* __restrict__ group_ptr, int n_inputs, int C,
                                                             int64_t first_input, int rows, int undo, float* __restrict__ params,
                                                             int64_t sr, int64_t sp) {
  const int r = blockIdx.x * 64 + (threadIdx.x & 63);
  const int gi = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (r >= rows || gi >= n_groups + n_inputs) return;
  float* row = params + (int64_t)r * sr;
  if (gi < n_groups) {   // preprocess_inner_params_kernel, misc.jl:403-446
    const int p0 = group_ptr[gi], p1 = group_ptr[gi + 1];
    float cum = 0.f;
    for (int p = p0; p < p1; ++p) cum += __expf(row[(int64_t)p * sp]);
    const float lc = __logf(cum);
    for (int p = p0; p < p1; ++p) row[(int64_t)p * sp] -= lc;
    return;
  }
  float* o = row + (first_input + (int64_t)(gi - n_groups) * C) * sp;
  if (!undo) {           // normalize_params_step, misc.jl:364-378
    float cum = 0.f;
    for (int c = 0; c < C; ++c) {
      const float e = __expf(o[(int64_t)c * sp]);
      o[(int64_t)c * sp] = e;
      cum += e;
    }
    for (int c = 0; c < C; ++c) o[(int64_t)c * sp] /= cum;
  } else {               // undo_normalize_params_step, misc.jl:380-393
    for (int c = 0; c < C; ++c) {
      const float p = o[(int64_t)c * sp];
      if (p > 0.f) o[(int64_t)c * sp] = __logf(p + 1e-6f);
    }
  }
}

void SparseCircuit::normalize_params_rows(float* d_params, int64_t sr, int64_t sp, int32_t rows, bool undo) {
  if (!d_params) fail(PCM_ERR_ARG, "parameter matrix is null");
  if (rows < 1) fail(PCM_ERR_ARG, "rows must be positive, got %d", rows);
  if (sr < 1 || sp < 1) fail(PCM_ERR_ARG, "strides must be positive");
  const int ng = (int)fc_.pargroup_sizes.size(), ni = (int)fc_.input_nodes.size();
  if (ng + ni == 0) return;
  hipLaunchKernelGGL(normalize_rows_kernel, dim3(ceil_div(rows, 64), ceil_div(ng + ni, 4)), dim3(256), 0, stream, ng, d_group_ptr_.p,
                     ni, fc_.num_cats, (int64_t)fc_.param2edge.size(), rows, undo ? 1 : 0, d_params, sr, sp);
  check_launch_f("normalize_rows");
}

}  // namespace pcm
