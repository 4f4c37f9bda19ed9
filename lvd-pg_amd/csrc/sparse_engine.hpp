// General engine: any circuit DAG, flattened into nodes + (prime, sub) edges and evaluated
// layer by layer.  It restates what the reference gets from ProbabilisticCircuits.jl
// `BitsProbCircuit` (un-vendored) plus src/bits_circuit.jl:39-113, with two layout changes
// for the GPU: node values are kept node-major with the example index fastest (coalesced
// over a wave), and every node owns a contiguous run of up-edges and a contiguous run of
// incoming (down) edges, so that a thread folds one node's edges sequentially and writes
// its result once -- no atomics on node values or flows.
#pragma once

#include <memory>

#include "common.hpp"

namespace pcm {

enum : uint8_t { kInput = 0, kSum = 1, kMul = 2 };

// Host-side flat circuit (also used by the HCLT engine to expose its general form).
struct FlatCircuit {
  int32_t num_vars = 0, num_cats = 0, num_heads = 0;
  std::vector<uint8_t> type;          // per node
  std::vector<int32_t> layer;         // per node: inputs 0, inner 1 + max over children
  std::vector<int32_t> in_var;        // per node (inputs)
  std::vector<int64_t> in_off;        // per node (inputs): offset into leaf arrays
  std::vector<int32_t> input_nodes;   // input node ids in creation order
  // up edges in the reference's order: by layer, then by parent id
  std::vector<int32_t> e_parent, e_prime, e_sub;   // sub = -1: none
  std::vector<float> e_logp;                         // 0 on product edges
  std::vector<int32_t> node_e0, node_e1;             // a node's run of up edges
  std::vector<int64_t> layer_ends;                   // edge count at the end of each up layer
  std::vector<float> leaf_logp;                      // [inputs * C]
  std::vector<int32_t> heads;                        // node ids of the heads (multi-head)
  std::vector<int32_t> desc_node;                    // per node of the description: its node id, -1 where it was folded into an edge or is unreachable
  // parameter tables (1-based, src/bits_circuit.jl:46-70)
  std::vector<int64_t> edge2param, param2edge, param2group, pargroup_sizes;
  int64_t n_nodes() const { return (int64_t)type.size(); }
  int64_t n_edges() const { return (int64_t)e_parent.size(); }
  void finish();   // derives node_e0/e1, layer_ends and the parameter tables from the edges
};

// Flattening of a DAG description (see pcm_circuit_create for the format).
FlatCircuit flatten_dag(int32_t num_nodes, const uint8_t* node_type, const int32_t* child_ptr,
                        const int32_t* child_idx, const float* sum_logp, const int32_t* input_var,
                        const float* input_logp, int32_t num_vars, int32_t num_cats, int32_t num_heads);

// Matrices of parameter rows arrive with element strides; the row kernels want unit stride along the parameters
// (param_rows.hip): the matrix itself, or a re-laid-out copy in `tmp`; and a packed result back into a strided matrix.
const float* rows_packed_in(const float* m, int64_t sr, int64_t sp, int rows, int64_t n, DevBuf<float>& tmp, hipStream_t s);
void rows_unpack_out(float* packed, float* m, int64_t sr, int64_t sp, int rows, int64_t n, hipStream_t s);

class SparseCircuit : public pcm_circuit {
 public:
  explicit SparseCircuit(FlatCircuit fc);
  ~SparseCircuit() override;

  int64_t size(int what) const override;
  void index_table(int which, int64_t* out, int64_t n) const override;
  void vectorize(float* out, int64_t n) override;
  void update_parameters(const float* in, int64_t n) override;
  void loglikelihoods(const BatchRef& b, float* d_ll) override;
  void flows(const BatchRef& b, float rate, const float* d_head_mask, float* d_ll) override;
  void loglikelihoods_soft(const SoftRef& s, float* d_ll) override;
  void flows_soft(const SoftRef& s, float rate, const float* d_head_mask, float* d_ll) override;
  void em_update(float pseudocount, float inertia) override;
  void kld(pcm_circuit* q, float* out) override;
  void kld_backward(pcm_circuit* q, float* gp, float* gq, int64_t n) override;
  void kld_backward_dev(pcm_circuit* q, float* d_gp, float* d_gq, int64_t n) override;
  int64_t sample_noise_size() const override { return (int64_t)fc_.param2edge.size(); }
  void sample(const float* d_node_noise, const float* d_leaf_noise, int32_t batch, uint8_t* d_out) override;
  void adam_step(const float* d_grad, float* d_params, float* d_m, float* d_v, float lr, float b1, float b2,
                 float eps, int t) override;
  void sample_soft(const float* d_node_noise, float temperature, int32_t batch, float* d_out) override;
  void flow_gradients(int32_t batch_size, float* d_grad) override;
  void leaf_adam(float* d_aux_p, float* d_aux_m, float* d_aux_v, float lr, float b1, float b2, float eps, int t) override;
  void sample_soft_with_slots(const float* d_node_noise, const int32_t* d_noise_slot, int64_t noise_stride,
                              float temperature, int32_t batch, float* d_out);
  void kld_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                float* d_out) override;
  void kld_backward_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                         float* d_g1, float* d_g2, float* d_klds) override;
  void gumbel_sample_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                          float temperature, bool norm_params, float* d_out) override;
  void gumbel_sample_backward_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                   float temperature, bool norm_params, bool grad_wrt_logparams, const float* d_out_grad,
                                   float* d_grads) override;
  void normalized_flows(const BatchRef& b, float* d_out, int64_t sr, int64_t sp, bool as_written) override;
  void normalize_params_rows(float* d_params, int64_t sr, int64_t sp, int32_t rows, bool undo) override;
  void soft_rows_down(const float* p, int rows, const float* d_noise, float inv_t);
  struct RowsState;   // tables and scratch of the parameter-row queries (param_rows.hip)

  void get_node_values(float* mars, float* flows, int64_t n);
  void get_aggregates(float* edge_aggr, int64_t n_edges, float* leaf_flow, int64_t n_leaf);
  void node_flow_sums(float* out, int64_t n);

  // device views for engines that embed a general circuit (the HCLT engine's KL / sampling)
  float* d_logp() { return d_logp_.p; }
  float* d_leaf() { return d_leaf_.p; }
  const FlatCircuit& flat() const { return fc_; }
  // noise_slot: optional device table (one entry per edge, up order) mapping a sum edge to its
  // column in the node-noise matrix; noise_stride: columns of that matrix
  void sample_with_slots(const float* d_node_noise, const int32_t* d_noise_slot, int64_t noise_stride,
                         const float* d_leaf_noise, int32_t batch, uint8_t* d_out);
  void kld_forward_device(SparseCircuit* q);          // leaves the result in d_kld_ (root last)
  void kld_backward_device(SparseCircuit* q, float* d_edge_g1, float* d_edge_g2, float* d_leaf_g1, float* d_leaf_g2);
  float* d_kld() { return d_kld_.p; }

 private:
  FlatCircuit fc_;
  int n_layers_ = 0;
  std::vector<int32_t> layer_node0_;   // nodes sorted by layer: ranges per layer
  DevBuf<uint8_t> d_type_;
  DevBuf<int32_t> d_order_, d_node_e0_, d_node_e1_, d_e_parent_, d_e_prime_, d_e_sub_, d_in_var_;
  DevBuf<int64_t> d_in_off_;
  DevBuf<float> d_logp_, d_leaf_, d_edge_aggr_, d_leaf_flow_, d_mars_, d_flows_, d_kld_, d_edge_kld_, d_grad_;
  // incoming edges per node (down direction)
  DevBuf<int32_t> d_in_ptr_, d_in_edge_;
  DevBuf<int4> d_in_rec_;
  DevBuf<float> d_in_logp_, d_edge_part_;
  DevBuf<int32_t> d_input_nodes_, d_alias_list_, d_bwd_order_;
  std::vector<int> bwd_layer0_;
  DevBuf<int4> d_fwd_rec_, d_bwd_rec_;   // per position of the forward / backward order: node and its ranges in one record
  DevBuf<int2> d_bwd_alias_;
  std::vector<int> layer_max_children_, bwd_layer_max_in_;   // per layer: most edges of a node going up / coming in
  // dense groups (sparse_groups.hip.hpp): sum nodes of a layer that share one list of children
  struct GroupLaunch { int layer, group0, count, gt, ct; int32_t pnode0, pslot0; int64_t pw0; };
  std::vector<GroupLaunch> group_launches_;   // per (layer, shape), sorted by layer: ranges of groups
  // runs of layers of groups that go as one walk launch (sparse_group_walk_kernel); level0: the run's layers in d_grp_levels_
  struct GroupRun { int layer_first, layer_last, gt, ct, group0, n_groups; int32_t pnode0, pslot0; int64_t pw0; int level0, n_levels, max_count; };
  std::vector<GroupRun> group_runs_fwd_, group_runs_bwd_;
  DevBuf<int2> d_grp_levels_;
  int64_t n_walk_levels_ = 0;                 // layers of groups inside forward runs
  void build_group_runs();
  bool launch_group_walk(const GroupRun& r, bool forward, int Bp, int batch, bool tempered);
  std::vector<GroupLaunch> group_stat_launches_;   // per shape: ranges of d_grp_order_ (layer and bases unused)
  std::vector<int> fwd_layer0_;               // ranges of d_fwd_rec_ per layer: the nodes no group computes
  bool layer0_inputs_only_ = true;            // the first layer holds input nodes and nothing else
  int64_t n_layer_nodes_ = 0;                 // nodes whose values the layer kernels compute (the others: the groups')
  int64_t n_group_slots_ = 0, n_groups_ = 0, n_group_elems_ = 0;   // children of all groups; groups; padded W entries
  DevBuf<int32_t> d_grp_node_, d_grp_edge_, d_grp_own_, d_grp_elem_, d_grp_order_;
  DevBuf<int4> d_grp_rec_, d_grp_rows_, d_grp_copies_;   // (a group's record is two int4)
  DevBuf<float> d_grp_wf_, d_grp_wb_, d_grp_m_, d_grp_xm_;
  DevBuf<float> d_norm_;                      // tempered flows: [n_nodes + 1][Bp], see sparse_tempered_norm_kernel
  DevBuf<int2> d_grp_product_edges_;          // {edge, parent}: product edges into nodes a group's kernel writes
  int n_group_product_edges_ = 0;
  std::vector<int32_t> grp_pslot_h_;          // host: where a slot's entry sits in the padded per-child tables
  std::vector<int32_t> grp_prime_h_;          // host copy: the prime of every slot
  std::vector<char> grp_expanded_;            // per node: a product that the groups using it compute themselves
  void refresh_group_w(float inv_f = 1.f);    // W = exp(log-parameter * inv_f): 1 / fscale for a tempered backward pass
  void build_groups(std::vector<int32_t>& group_of, std::vector<int32_t>& edge_slot);
  void launch_groups(int layer, int what, int Bp, int batch, bool tempered = false);   // what: 0 forward, 1 backward (one layer), 2 edge flows (all layers)
  int64_t n_flow_rows() const { return fc_.n_nodes() + n_group_slots_; }
  DevBuf<int32_t> d_head_nodes_;   // node ids of the heads
  DevBuf<int32_t> d_group_ptr_, d_param2edge_, d_var_ptr_, d_var_nodes_;
  DevBuf<uint8_t> d_visit_;
  DevBuf<float> d_g1_, d_g2_, d_l1_, d_l2_;   // KL gradients in edge / leaf order
  int cap_batch_ = 0, last_batch_ = 0, max_var_nodes_ = 1;
  bool have_flows_ = false;
  int flow_batch_ = 0;   // examples whose node flows d_flows_ holds (0: none)
  DevBuf<float> d_node_sums_;

  std::shared_ptr<RowsState> rows_;   // (shared_ptr: the type is complete only in param_rows.hip)
  RowsState& rows_state();
  void kld_rows_forward(const float* p1, const float* p2, int rows, bool norm, bool with_edges);
  void ensure_batch(int batch);
  void ensure_var_tables();
  void run_forward(const BatchRef* b, const SoftRef* s);
  void write_ll(int batch, float* d_ll);
  void run_flows(int batch, const SoftRef* soft, float rate, const float* d_head_mask, float* d_ll, bool accumulate = true);
};

}  // namespace pcm
