/*
 * pcmi355 -- C ABI of the MI355X probabilistic-circuit engine.
 *
 * Every entry point returns 0 on success and a negative pcm_status on failure;
 * pcm_last_error() then holds a message for the calling thread.  No exception crosses
 * this boundary.  Pointers named d_* are DEVICE pointers (hipMalloc'd or owned by any
 * framework on the current device); all other pointers are host memory owned by the
 * caller and only touched during the call.  Calls on one circuit are serialised by the
 * caller; distinct circuits are independent.  Work is queued on the circuit's stream
 * (default: the null stream) and entry points that return host data synchronise it.
 *
 * Citations name the reference interface each entry replaces; paths are relative to
 * VariationalJuice.jl/ in the reference tree.
 */
#ifndef PCMI355_H
#define PCMI355_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct pcm_circuit pcm_circuit;

enum pcm_status {
  PCM_OK = 0,
  PCM_ERR_ARG = -1,       /* null pointer, bad size, bad handle */
  PCM_ERR_SHAPE = -2,     /* tree / circuit description is malformed */
  PCM_ERR_UNSUPPORTED = -3,
  PCM_ERR_HIP = -4,       /* a HIP call failed; message names it */
  PCM_ERR_STATE = -5      /* call order violated (e.g. update before flows) */
};

/* Message of the last failure on this thread (never NULL). */
const char* pcm_last_error(void);
int pcm_version(void);

/* ---- compilation -------------------------------------------------------------- */

/*
 * Build the hidden Chow-Liu tree circuit of src/structures/hclts.jl:100-145
 * (`hclt_from_clt` with one observed variable per tree node and Categorical leaves) and
 * flatten it as ProbabilisticCircuits.jl `BitsProbCircuit` + src/bits_circuit.jl:39-113
 * (`CuMetaBitsProbCircuit`) do, into the dense per-tree-node block form the kernels use.
 * clt_parent[v] is the tree parent of variable v (-1 for the single root).
 * Parameters start uniform; set them with pcm_hclt_set_params or pcm_update_parameters.
 */
int pcm_hclt_create(const int32_t* clt_parent, int32_t num_vars, int32_t num_hidden_cats,
                    int32_t num_cats, pcm_circuit** out);

/*
 * A multi-head HCLT: the circuits `CuMultiHeadBitsProbCircuit(pcs)` (src-jl/multi_head_pc/bit_circuit.jl:14-56)
 * is given when the `pcs` are num_heads root sum nodes over the K products of one HCLT body (the patch
 * circuits of exps/progressive_growing/parallel_PG.jl:214-225 before pruning).  Runs on the block engine:
 * the body through the tree-walk kernels, the heads as an [H][K] block in two small kernels around them.
 * Needs num_hidden_cats 16 or 32 (PCM_ERR_UNSUPPORTED otherwise: describe the circuit to pcm_circuit_create
 * instead).  Parameter vector: the body's sum parameters in
 * the order of pcm_hclt_create without the root's row, then num_heads x K head parameters, then the input
 * nodes; the same order pcm_circuit_create gives the equivalent description.  pcm_loglikelihoods returns
 * [num_heads][batch], pcm_flows takes d_head_mask [num_heads][batch]; KL and sampling are not defined.
 */
int pcm_hclt_create_multihead(const int32_t* clt_parent, int32_t num_vars, int32_t num_hidden_cats, int32_t num_cats,
                              int32_t num_heads, pcm_circuit** out);

/*
 * Many multi-head HCLTs over one batch as ONE handle: the 64 patch circuits of
 * exps/progressive_growing/parallel_PG.jl:214-225, each of which the reference trains with its own
 * `mini_batch_em_for_multihead_pc` call (src-jl/multi_head_pc/em.jl:1-99) on its own columns of the same
 * images.  clt_parent is a forest over the num_vars variables of the batch: every -1 entry roots a tree
 * (trees are numbered by their root's variable index), every tree has at least two variables and gets
 * num_heads heads.  The handle is a container for running them together -- one launch per kernel for
 * all trees, the walks' sixteen waves filled with nodes of different trees -- and computes per tree the
 * bits a handle of pcm_hclt_create_multihead over that tree's variables (numbered in the same relative
 * order: a node's children are added up in variable order) would:
 *   pcm_loglikelihoods  d_ll_out [num_trees][num_heads][batch]
 *   pcm_flows           d_head_mask [num_trees][num_heads][batch], d_ll_out [num_trees][batch]
 *   pcm_em_update, pcm_set_stream, pcm_set_timing  (pcm_em_step has no head mask: not for multi-head circuits)
 *   pcm_hclt_set_params / get_params / get_flows  (per-variable blocks: rows of trees stay apart)
 *   pcm_hclt_set_heads / get_heads, pcm_size
 * Everything a single circuit defines beyond that (parameter vector and index tables, KL, sampling, soft
 * evidence, Adam) returns PCM_ERR_UNSUPPORTED: move a tree's blocks and heads to a handle of its own for those.
 * Needs num_hidden_cats 16 or 32 and trees the lean walk kernels take (at most three children per tree
 * node), PCM_ERR_UNSUPPORTED otherwise.
 */
int pcm_hclt_create_forest(const int32_t* clt_parent, int32_t num_vars, int32_t num_hidden_cats, int32_t num_cats,
                           int32_t num_heads, pcm_circuit** out);

/*
 * Missing values.  The reference's data may hold `missing` where a variable was not observed: the leaf then
 * counts as probability 1 (src/regularization/reg_likelihood.jl:40-47, :76-83), its flow goes to the input node's
 * `missing_flow`, and the update spreads that flow over the categories as the leaf's own distribution
 * (src/nodes/fixable_categorical_dist.jl:223-248).  uint8 data has no such value, so a circuit that is to see
 * missing values is created with one category more than the data has, and this call (HCLT, forest and multi-head
 * HCLT handles on the block kernels; on != 0) declares that last category, num_cats - 1, the marker: a binding
 * writes it where the reference has `missing`.  The marker's row of every leaf table is pinned to log-probability
 * 0 and left out of the normalisation, the pseudocount is shared by the num_cats - 1 real categories, and the
 * marker's row of the leaf statistics (pcm_hclt_get_flows) is the missing_flow.  Likelihoods, flows and EM
 * are defined on such a circuit; KL, sampling, soft evidence and Adam return PCM_ERR_UNSUPPORTED.
 */
int pcm_set_missing_category(pcm_circuit* c, int32_t on);

/*
 * `soft_reg`, `soft_reg_width` of mini_batch_em_with_reg / probs_flows_circuit_with_reg
 * (src/regularization/reg_em.jl:208-213, reg_flow.jl:276-282) for HCLT handles on the block kernels: from this call
 * on, categorical batches (pcm_loglikelihoods, pcm_flows, pcm_em_step) see every leaf at the smoothed value
 * soft_loglikelihood = log((1 - soft_reg) p[x] + soft_reg mean(p[c], c in the window of x))
 * (src/regularization/reg_likelihood.jl:4-14; window: c_start = max(0, x - width / 2), c_end = min(c_start + width - 1,
 * num_cats - 1)), and an example's leaf flow is shared out over x and its window as soft_flow does
 * (reg_flow.jl:3-22).  as_written != 0: the shares as that source line computes them, with the heap's
 * LOG-probabilities where probabilities are meant -- (1 - s) logp[x] F / base and s / n logp[c] F / base with
 * base = (1 - s) logp[x] + s mean(p) -- for parity with the reference as it runs; as_written == 0: the derivative of
 * the smoothed value, the same lines with probabilities (the form of soft_flow_params,
 * src/nodes/fixable_categorical_dist.jl:141-160).  soft_reg = 0 switches the smoothing off.  Inner flows and
 * likelihoods do not depend on as_written.  PCM_ERR_UNSUPPORTED for hidden sizes without block kernels and circuits with
 * a missing-value category (those smooth through the soft-evidence entry points).
 */
int pcm_set_soft_reg(pcm_circuit* c, float soft_reg, int32_t soft_reg_width, int32_t as_written);

/*
 * `fscale` of mini_batch_em_beta (VariationalJuice.jl/src-jl/learning/em.jl:289-296, scaled_probs_flows_circuit
 * flow.jl:367-373): from this call on, pcm_flows / pcm_flows_soft / pcm_em_step hand every sum node's flow to its
 * edges in shares proportional to (posterior share)^(1 / fscale) -- scale_flows_kernel flow.jl:120-175 computes the
 * sum of those per node, reg_layer_down_kernel :204-300 the edge flows -- instead of the posterior shares themselves;
 * likelihoods, per-example normalised flows and every other query are not touched.  fscale = 1 (the default) is the
 * ordinary pass.  Any handle but a forest or a circuit with a missing-value category (PCM_ERR_UNSUPPORTED); HCLT
 * handles run these passes on their layered form (kernels per layer, dense groups on the matrix cores), with the
 * statistics and the flow memory held there until pcm_em_update.  Per-example weights / head masks scale the
 * flows as always (the reference's tempered pass reads its `weights` argument only at the input nodes).
 * Together with pcm_set_soft_reg (mini_batch_em_beta passes both on, em.jl:366-368): the layered form has no smoothed
 * leaf table, so the library turns every categorical batch into the soft evidence that gives the leaves the smoothed
 * values (batch x num_vars x num_cats floats of device memory) and runs the tempered soft-evidence pass on it; the leaf
 * flows are those of as_written == 0, and as_written != 0 makes such a pass fail with PCM_ERR_UNSUPPORTED.
 * PCM_ERR_ARG unless fscale is positive and finite.
 */
int pcm_set_flow_scale(pcm_circuit* c, float fscale);

/* Head log-parameters of a multi-head HCLT or a forest, [num_trees][num_heads][num_hidden_cats] on the host:
 * the `params` of the head sum nodes (src-jl/multi_head_pc/bit_circuit.jl:14-56 keeps them in the heads'
 * edges), row h of a tree being the head that row h of its head mask seeds. */
int pcm_hclt_set_heads(pcm_circuit* c, const float* heads);
int pcm_hclt_get_heads(pcm_circuit* c, float* heads);

/*
 * Compile a general circuit given as a DAG in topological order (children before
 * parents, root last), the flat form a binding obtains by walking a `ProbCircuit`:
 * replaces `CuMetaBitsProbCircuit(pc)` (src/bits_circuit.jl:39) and, with num_heads > 0,
 * `CuMultiHeadBitsProbCircuit(pcs)` (src-jl/multi_head_pc/bit_circuit.jl:14-56; the last
 * num_heads nodes are the heads and no fake root is needed).
 * node_type: 0 input, 1 sum, 2 product.  child_ptr[n..n+1] delimits node n's children in
 * child_idx; sum_logp is parallel to child_idx (ignored under products).  Input node n
 * reads variable input_var[n] (0-based) and owns num_cats log-probabilities; input_logp holds
 * them for the input nodes in the order they appear in the description.  The compiled
 * circuit numbers its nodes, edges and parameters as the reference's flattening does
 * (depth-first from the root, children in order); nodes unreachable from the root or the
 * heads are dropped.
 */
int pcm_circuit_create(int32_t num_nodes, const uint8_t* node_type, const int32_t* child_ptr,
                       const int32_t* child_idx, const float* sum_logp, const int32_t* input_var,
                       const float* input_logp, int32_t num_vars, int32_t num_cats,
                       int32_t num_heads, pcm_circuit** out);

/* Releases the circuit and all device memory it owns.  The library keeps a table of the handles it
 * has given out: every entry point answers PCM_ERR_ARG, without touching the pointer, for a handle
 * that is null, was freed before or was not created by this library. */
int pcm_free(pcm_circuit* c);

/* Queue this circuit's work on the given hipStream_t (NULL = null stream). */
int pcm_set_stream(pcm_circuit* c, void* hip_stream);

/* ---- sizes and index tables --------------------------------------------------- */

/* `num_parameters(mbpc)`, `num_nodes`, `num_edges`, `num_input_params`
 * (src/bits_circuit.jl:119-131).  what: 0 parameters, 1 sum parameters, 2 nodes,
 * 3 edges, 4 input parameters, 5 variables, 6 categories, 7 hidden categories (0 if not an
 * HCLT), 8 inner tree nodes (HCLT), 9 up layers, 10 parameter groups, 11 input nodes,
 * 12 heads (0 for a single-root circuit), 13 nodes of the description the circuit was
 * built from (0 for an HCLT built from its tree), 14 which kernels run likelihoods and flows:
 * 0 per-layer kernels, 1 lean tree walks, 2 general tree walks, 3 wide block kernels, 15 trees (1 unless
 * the handle is a forest), 16 dense groups of a pcm_circuit_create circuit: sets of sum nodes of one layer with one
 * and the same list of children, which run as blocks on the matrix cores instead of edge by edge (0 for an HCLT
 * handle, and for every circuit created while PCMI355_DENSE_GROUPS=0 is in the environment: a switch for comparisons,
 * results agree to rounding), 17 nodes whose values the per-layer kernels compute (the others are the groups'), 18 layers
 * of groups that go inside walk launches: runs of consecutive layers that hold groups of one shape and nothing else take
 * one launch per direction where their groups are few (PCMI355_GROUP_WALK=0 at creation: a launch per layer, the same
 * bits). */
int64_t pcm_size(const pcm_circuit* c, int32_t what);

/* Index tables of src/bits_circuit.jl:9-36, 1-based as the reference holds them.
 * which: 0 edge2param [edges], 1 param2edge [sum parameters], 2 param2group [sum
 * parameters], 3 pargroup_sizes [groups], 4 innode2ncumparam [input nodes],
 * 5 up-layer ends [layers], 6 edge parent ids, 7 edge prime ids, 8 edge sub ids (0: none)
 * [edges, up order], 9 head node ids (`root_ids`, src-jl/multi_head_pc/bit_circuit.jl:38-51)
 * [heads], 10 node id of every node of the description given to pcm_circuit_create, 0 where
 * the node was folded into an edge or cannot be reached from a root (the inverse of the
 * reference's `bpc.nodes_map`, used by src-jl/multi_head_pc/prune.jl:38-57 and
 * transformation.jl:132-135) [description nodes], 11 input node ids in parameter order
 * (`bpc.input_node_ids`) [input nodes].  n must equal the table length. */
int pcm_index_table(const pcm_circuit* c, int32_t which, int64_t* out, int64_t n);

/* ---- parameters --------------------------------------------------------------- */

/* `vectorize_parameters(mbpc, params)` (src/misc.jl:5-40): sum-edge log-parameters in
 * up-edge order, then every input node's log-probabilities in creation order. */
int pcm_vectorize_parameters(pcm_circuit* c, float* out, int64_t n);
/* `update_parameters(mbpc, params)` (src/misc.jl:73-102). */
int pcm_update_parameters(pcm_circuit* c, const float* params, int64_t n);

/* HCLT block form.  theta is [num_vars][K][K] log-parameters (row k: sum node k of the
 * tree node, column j: hidden state j; rows of leaf tree nodes are ignored and only row 0
 * of the root is used, hclts.jl:137); leaf is [num_vars][K][num_cats] log-probabilities of
 * `joined_leaves[v, j]` (hclts.jl:147-156).  Either pointer may be NULL to skip it. */
int pcm_hclt_set_params(pcm_circuit* c, const float* theta, const float* leaf);
int pcm_hclt_get_params(pcm_circuit* c, float* theta, float* leaf);
/* Sufficient statistics of the last pcm_flows / pcm_em_step in the same block form:
 * edge_aggr [num_vars][K][K] (the reference's `edge_aggr`, src/queries/flow.jl:73-81) and
 * leaf_flow [num_vars][K][num_cats] (the heap's flow slots,
 * src/nodes/fixable_categorical_dist.jl:121-130). */
int pcm_hclt_get_flows(pcm_circuit* c, float* edge_aggr, float* leaf_flow);

/* ---- queries ------------------------------------------------------------------ */

/*
 * Forward pass: `loglikelihoods(bpc, data; batch_size)` / `loglikelihoods_probcat`
 * (src/regularization/reg_likelihood.jl:139-162) for one batch.  d_data holds uint8
 * categories; element (example e, variable v) is d_data[e*stride_ex + v*stride_var].
 * d_example_ids (may be NULL = 0..batch-1) selects the batch rows, 0-based, like the
 * reference's `example_ids`.  d_ll_out receives `batch` floats (mars[:, end]).
 * For a multi-head circuit d_ll_out receives [num_heads][batch]
 * (src-jl/multi_head_pc/likelihood.jl:3-18 with head_mask = nothing).
 */
int pcm_loglikelihoods(pcm_circuit* c, const uint8_t* d_data, int64_t stride_ex,
                       int64_t stride_var, const int32_t* d_example_ids, int32_t batch,
                       float* d_ll_out);

/*
 * Forward + backward + leaf flows: `probs_flows_circuit_with_reg` with soft_reg = 0
 * (src/regularization/reg_flow.jl:276-282) == `probs_flows_circuit`
 * (src/queries/flow.jl:228-234).  The circuit's edge_aggr and leaf flow accumulators are
 * first scaled by `rate` (0 clears them; src/regularization/reg_em.jl:276-284) and then
 * receive this batch.  d_head_mask (multi-head circuits, else NULL) is
 * [num_heads][batch] and seeds the head flows (src-jl/multi_head_pc/flow.jl:141-176);
 * d_ll_out then receives `batch` floats, the mask-weighted mixture
 * logsumexp_h(mars[head_h] + log mask_h) - log sum_h mask_h
 * (src-jl/multi_head_pc/likelihood.jl:3-12).
 * Per-example weights (the `weights` of reg_flow.jl:38-39,190-191, which multiply an example's edge and
 * leaf flows): every flow is linear in the flow its example starts with, so for a multi-head circuit they
 * are a factor of the mask's column, and a single-root circuit (pcm_circuit_create without heads,
 * pcm_hclt_create) takes them as a mask [1][batch]; d_ll_out is not weighted.  Masks and weights must be
 * finite and >= 0: the library does not look at them on the host (they are device memory), a binding does.
 */
int pcm_flows(pcm_circuit* c, const uint8_t* d_data, int64_t stride_ex, int64_t stride_var,
              const int32_t* d_example_ids, int32_t batch, float rate, const float* d_head_mask,
              float* d_ll_out);

/*
 * Parameter update from the accumulated flows, the four calls of
 * src/regularization/reg_em.jl:292-299: add_pseudocount, aggr_node_flows,
 * update_params(inertia), update_input_node_params(pseudocount, inertia).
 */
int pcm_em_update(pcm_circuit* c, float pseudocount, float inertia);

/* pcm_flows followed by pcm_em_update: one iteration of the batch loop of
 * `mini_batch_em_with_reg` (src/regularization/reg_em.jl:272-300). */
int pcm_em_step(pcm_circuit* c, const uint8_t* d_data, int64_t stride_ex, int64_t stride_var,
                const int32_t* d_example_ids, int32_t batch, float rate, float pseudocount,
                float inertia, float* d_ll_out);

/* General circuits: host copies of per-batch node values / flows of the last pcm_flows,
 * [num_nodes][batch] (the reference's `mars` / `flows`, transposed), and of the
 * accumulators: edge_aggr [edges, up order], leaf_flow [input parameters]. */
int pcm_get_node_values(pcm_circuit* c, float* mars, float* flows, int64_t n);
/* General circuits: out[n] = sum over the examples of the last pcm_flows batch of the flow of
 * node n, host array [num_nodes] (`sum(flows[1:batch, :]; dims = 1)`,
 * src-jl/multi_head_pc/transformation.jl:121). */
int pcm_node_flow_sums(pcm_circuit* c, float* out, int64_t n);
int pcm_get_aggregates(pcm_circuit* c, float* edge_aggr, int64_t n_edges, float* leaf_flow,
                       int64_t n_leaf);

/*
 * KL(p || q) of two parameterisations of one structure: `kld(mbpc, params1, params2)`
 * with norm_params = false (src/queries/kld.jl:177-206).  p and q must have been compiled
 * from the same description.  *out receives klds[:, end].
 */
int pcm_kld(pcm_circuit* p, pcm_circuit* q, float* out);
/* `kld_backward(mbpc, params1, params2; grad_wrt_logparams = true)`
 * (src/queries/kld.jl:593-649): gradients in parameter-vector order. */
int pcm_kld_backward(pcm_circuit* p, pcm_circuit* q, float* grad_p, float* grad_q, int64_t n);
/* The same with the two gradient vectors left in device memory (the reference copies them to
 * the host, src/queries/kld.jl:640-648, and its optimiser takes them back to the device,
 * src/sgd/adam.jl:318): the form pcm_adam_step consumes.  Queued on the circuit's stream. */
int pcm_kld_backward_dev(pcm_circuit* p, pcm_circuit* q, float* d_grad_p, float* d_grad_q, int64_t n);

/*
 * Gumbel-max ancestral sampling from supplied noise: the temperature -> 0 limit of
 * `gumbel_sample` (src/queries/sample.jl:338-383), which itself draws its noise in-kernel
 * (:45) and has no counterpart taking a noise tensor.  d_node_noise is
 * [batch][pcm_sample_noise_size()] (HCLT: [batch][inner tree nodes in bottom-up
 * order][K], indexed by the hidden state chosen; general: one float per sum parameter),
 * d_leaf_noise is [batch][num_vars][num_cats], d_out [batch][num_vars] uint8.  Both noise
 * pointers must be 16-byte aligned (PCM_ERR_ARG otherwise).
 */
int64_t pcm_sample_noise_size(const pcm_circuit* c);
int pcm_sample(pcm_circuit* c, const float* d_node_noise, const float* d_leaf_noise,
               int32_t batch, uint8_t* d_out);

/*
 * Relaxed sampling at a positive temperature: `gumbel_sample(mbpc, params, ...; temperature,
 * no_gumbel)` (src/queries/sample.jl:338-383) for one parameter row per circuit, with the
 * noise supplied instead of drawn in the kernel (:45).  d_node_noise is laid out as for
 * pcm_sample, or NULL for no_gumbel = true; d_out receives the soft assignment
 * [batch][num_vars][num_cats]: every variable's top-down probabilities times its input
 * nodes' distributions (:262-284).  On an HCLT the sum nodes of one tree node share their
 * noise column per hidden state; compile the circuit with pcm_circuit_create for one
 * independent draw per sum edge.  On an HCLT with block kernels d_node_noise and d_out must be
 * 16-byte aligned (PCM_ERR_ARG otherwise).
 */
int pcm_sample_soft(pcm_circuit* c, const float* d_node_noise, float temperature, int32_t batch,
                    float* d_out);

/*
 * The same three queries on a MATRIX of parameter rows -- one structure, `rows` parameter vectors, all
 * rows in one pass -- as the reference's own signatures have them: `kld(mbpc, params1, params2;
 * norm_params)` (src/queries/kld.jl:164-206), `kld_backward(mbpc, params1, params2; norm_params,
 * grad_wrt_logparams = true)` (:593-649) and `gumbel_sample(mbpc, params, num_vars, par_buffer_size;
 * temperature, no_gumbel, norm_params)` (src/queries/sample.jl:338-383), called with one row per example
 * by src/utils/cuda_preallocation.jl:47-78, :189-203.  The circuit gives the structure only; its own
 * parameters are not read.  Element (row r, parameter i) of a matrix is at d_x[r * stride_row + i *
 * stride_param], parameters in pcm_vectorize_parameters order; Julia's column-major [rows, n] array is
 * (1, rows), a row-major tensor (n, 1).  Unit stride along the parameters is the layout the kernels work
 * in; anything else is re-laid-out on the way in and out.  norm_params != 0: the LEAF parameters are
 * probabilities, not log-probabilities (src/nodes/fixable_categorical_dist.jl:182-186, :216-217;
 * sample.jl:265-268); sum parameters are log-parameters either way, as in the reference.
 *
 * pcm_kld_rows: d_klds [rows] (device) receives klds[:, end].
 * pcm_kld_backward_rows: d_grads1 / d_grads2 (device, the strides of the parameter matrices) receive the
 * gradients with respect to the rows of params1 / params2; d_klds may be NULL.
 * pcm_gumbel_sample_rows: d_noise is [rows][num sum parameters] (dense, one draw per sum edge) or NULL for
 * no_gumbel = true; d_out [rows][num_vars][num_cats].
 * pcm_gumbel_sample_backward_rows: the reverse pass of pcm_gumbel_sample_rows, `gumbel_sample_backward(mbpc,
 * params, input_aggr_params, input_aggr_grads, temperature; norm_params, grad_wrt_logparams)`
 * (src/queries/sample.jl:389-650; src/utils/cuda_preallocation.jl:205-218).  d_out_grads [rows][num_vars][num_cats]
 * is the gradient of a loss with respect to the soft output; d_param_grads (the strides of the parameter matrix)
 * receives its gradient with respect to every parameter, for the same d_params, d_noise and temperature as the
 * forward call (the top-down probabilities are rebuilt, nothing is kept between the two calls).  Sum parameters:
 * with respect to the log-parameter, or divided by the edge's share of its node when grad_wrt_logparams == 0
 * (:466-469).  Leaf parameters: with respect to the PROBABILITY of the category, whatever norm_params says, as
 * the source writes it (:560-570).
 * All of these queue their work on the circuit's stream and do not wait for it.  At most 65535 rows per call.
 * On a single-root HCLT handle with block kernels (hidden size 16, 32 or 64) the four of them run on the block form, the
 * row as a grid dimension (fastest with 16-byte aligned matrices and a category count divisible by 4: otherwise the
 * two gradients take the per-layer kernels of the general form, which every other circuit uses).
 */
int pcm_kld_rows(pcm_circuit* c, const float* d_params1, const float* d_params2, int64_t stride_row, int64_t stride_param,
                 int32_t rows, int32_t norm_params, float* d_klds);
int pcm_kld_backward_rows(pcm_circuit* c, const float* d_params1, const float* d_params2, int64_t stride_row,
                          int64_t stride_param, int32_t rows, int32_t norm_params, float* d_grads1, float* d_grads2,
                          float* d_klds);
int pcm_gumbel_sample_rows(pcm_circuit* c, const float* d_params, int64_t stride_row, int64_t stride_param, int32_t rows,
                           const float* d_noise, float temperature, int32_t norm_params, float* d_out);
int pcm_gumbel_sample_backward_rows(pcm_circuit* c, const float* d_params, int64_t stride_row, int64_t stride_param,
                                    int32_t rows, const float* d_noise, float temperature, int32_t norm_params,
                                    int32_t grad_wrt_logparams, const float* d_out_grads, float* d_param_grads);

/*
 * Per-example normalised flows: `per_sample_normalized_flows(mbpc, data; batch_size)` (src/queries/flow.jl:417-464)
 * for one batch, what `normalized_flows_with_prealloc` (src/utils/cuda_preallocation.jl:292-308, called by
 * src/models/pc_vae.py:77) starts from.  A forward and a backward pass that leave the circuit's accumulators alone;
 * row r of d_out (element (r, i) at d_out[r * stride_row + i * stride_param], parameters in
 * pcm_vectorize_parameters order; Julia's [batch, n] array: 1, batch) belongs to example r of the batch:
 *   sum parameters (`map_flows_kernel`, flow.jl:496-528):  log(f / (g + 1e-8) + 1e-8), f the example's flow over the
 *     edge and g its flow over all edges of the same sum node (the edge's posterior share, guarded as the source does);
 *   input parameters (`map_input_flows_kernel`, :549-593): log(f_c / sum_c f_c) of the node's per-example edge flows,
 *     which hold the node's flow in one slot: 0 there, -inf in the other slots, NaN (0/0) in all of them where the
 *     node has no flow.  as_written != 0 places the flow as `get_edge_flow` does
 *     (src/nodes/fixable_categorical_dist.jl:162-176: it compares the 0-based category x with the 1-based parameter
 *     index, so the flow of category x sits in the slot of category x - 1 and category 0 fills no slot: NaN);
 *     as_written == 0 places it in the slot of the observed category (src/conditional_pc/flow.jl:244).
 * Single-root circuits (PCM_ERR_UNSUPPORTED with heads or for a forest); an HCLT handle answers on its general form.
 * Queued on the circuit's stream; the call does not wait for it.
 *
 * pcm_normalize_params_rows: `normalize_params(mbpc, params; undo)` (src/misc.jl:448-498) in place on a matrix of
 * parameter rows (the circuit gives the structure only): undo == 0: an input node's entries become exp(entry) / their
 * sum (probabilities, :364-378) and a sum node's entries logp - log(sum of exp(logp)) (:403-446); undo != 0: input
 * entries p > 0 become log(p + 1e-6) (:380-393), the sum parameters are normalised as before.
 */
int pcm_normalized_flows(pcm_circuit* c, const uint8_t* d_data, int64_t stride_ex, int64_t stride_var,
                         const int32_t* d_example_ids, int32_t batch, int32_t as_written, float* d_out, int64_t stride_row,
                         int64_t stride_param);
int pcm_normalize_params_rows(pcm_circuit* c, float* d_params, int64_t stride_row, int64_t stride_param, int32_t rows,
                              int32_t undo);

/*
 * Soft evidence: the same two queries with a three-dimensional data argument, as the reference
 * dispatches on `data isa CuArray{Float32,3}` (`init_mar!_with_reg_cat_kernel`
 * src/regularization/reg_likelihood.jl:51-91, `input_flows_circuit_with_reg_cat_kernel`
 * src/regularization/reg_flow.jl:50-82; the top-level circuits of
 * exps/LVD_for_imagenet/src/train_PG_top_level_pcs.jl are trained on per-cluster patch
 * log-likelihoods this way).  d_evidence[row * stride_ex + var * stride_var + cat * stride_cat]
 * is the log-evidence of category `cat` (element strides; Julia's [N, V, C] array: 1, N, N*V).
 * A leaf's value is logsumexp_c(evidence_c + logp_c) and its flow is shared among the categories
 * in proportion to exp(evidence_c + logp_c - value).  pcm_em_update afterwards as usual.
 */
int pcm_loglikelihoods_soft(pcm_circuit* c, const float* d_evidence, int64_t stride_ex, int64_t stride_var,
                            int64_t stride_cat, const int32_t* d_example_ids, int32_t batch, float* d_ll);
int pcm_flows_soft(pcm_circuit* c, const float* d_evidence, int64_t stride_ex, int64_t stride_var, int64_t stride_cat,
                   const int32_t* d_example_ids, int32_t batch, float rate, const float* d_head_mask, float* d_ll);

/*
 * Structure learning, the step before pcm_hclt_create: what `hclt(data, num_hidden_cats; pseudocount)`
 * (src/structures/hclts.jl:7-24) obtains from `learn_chow_liu_tree` and `clt_edges2graphs`.
 *
 * pcm_pairwise_mi: `pairwise_MI_chunked` (src/utils/information.jl:97-141 with the marginals of
 * :43-95): mutual information of every pair of variables of a device-resident uint8 data set
 * (element strides as in pcm_loglikelihoods; any number of examples in one call), counts smoothed with
 * pseudocount/C per category and pseudocount/C^2 per cell.  d_mi: device, [num_vars][num_vars],
 * symmetric, diagonal included.  Synchronous on `stream` (NULL: the default stream).
 *
 * pcm_chow_liu_tree: host matrix [num_vars][num_vars] -> maximum spanning tree (ties: lowest
 * index), directed away from the lowest-numbered centre of the tree; clt_parent[v] = parent
 * of v, -1 at the root: the argument of pcm_hclt_create.
 */
int pcm_pairwise_mi(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t num_examples,
                    int32_t num_vars, int32_t num_cats, float pseudocount, float* d_mi, void* stream);
int pcm_chow_liu_tree(const float* mi, int32_t num_vars, int32_t* clt_parent);

/*
 * pcm_pairwise_mi without any allocation.  No counterpart in the reference: it is for callers that
 * cannot call hipMalloc (code under HIP graph capture, tight serving loops, harnesses that forbid
 * it).  Same arguments, kernels and results as pcm_pairwise_mi; the staging buffer and the two
 * tables the kernels need live in a fixed 16.6 MiB array of the library's code object, held by every
 * GPU the library runs on until the process ends.  Limits (PCM_ERR_UNSUPPORTED beyond them):
 * num_examples <= 65535, num_vars <= 4096, num_vars * ceil64(num_examples) <= 16 MiB (e.g. 4096
 * examples of 3072 variables).  The work is queued on `stream` and the call does NOT wait for it.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two
 * threads) race; calls queued on one stream do not.  The first call on a device resolves the array's
 * address (hipGetSymbolAddress) and raises the kernels' LDS limit: make it before any stream capture
 * begins; later calls only query a device attribute and launch.
 */
int pcm_pairwise_mi_static(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t num_examples,
                           int32_t num_vars, int32_t num_cats, float pseudocount, float* d_mi, void* stream);

/*
 * Adam ascent step on the sum parameters followed by per-sum-node normalisation
 * (src/sgd/adam.jl:63-86, :88-127, :318-319).  d_grad, d_params (unnormalised
 * log-parameters), d_m, d_v are device vectors in parameter-vector order over the sum
 * parameters; the circuit's log-parameters become params - log(sum exp(params)) per node.
 */
int pcm_adam_step(pcm_circuit* c, const float* d_grad, float* d_params, float* d_m, float* d_v,
                  float lr, float beta1, float beta2, float eps, int32_t t);

/*
 * The `adam` trainer's step from the flows of a batch (src/sgd/adam.jl:244-344), after pcm_flows with rate 0:
 * pcm_flow_gradients: d_grad [num sum parameters] (device, parameter-vector order) receives
 *   edge_aggr / batch_size - exp(logp) * (sum of the sum node's edge_aggr / batch_size)
 * (`edge_aggr ./= batch_size` :310, `compute_gradients` :27-61), the gradient of the mean log-likelihood with
 * respect to the unnormalised log-parameters.
 * pcm_adam_flow_step: that gradient, then the sum-parameter step of pcm_adam_step (:318-325, :63-127), and --
 * if d_leaf_params is not NULL -- `update_input_node_params_adam` (:218-242) on the three device arrays
 * [num input parameters] that stand for the reference's auxiliary heap (a copy of the leaf log-parameters that
 * takes the steps, and its two moments): g = flow + exp(logp) * node_flow as the source writes it.  Like the
 * source, it never writes the stepped leaf values back into the circuit.
 */
int pcm_flow_gradients(pcm_circuit* c, int32_t batch_size, float* d_grad);
int pcm_adam_flow_step(pcm_circuit* c, int32_t batch_size, float* d_params, float* d_m, float* d_v, float* d_leaf_params,
                       float* d_leaf_m, float* d_leaf_v, float lr, float beta1, float beta2, float eps, int32_t t);

/* ---- instrumentation ----------------------------------------------------------- */

/* Per-kernel timing, the role of `debug = true` -> `CUDA.@time` around each launch
 * (src/queries/likelihood.jl:86-92, src/queries/flow.jl:127-133).  When on, the
 * forward / backward / statistics launches of pcm_flows carry a start and a stop event
 * on their own dispatches (nothing is put between the kernels, nothing synchronises);
 * pcm_get_timing synchronises and returns the mean milliseconds over the calls since
 * the previous read of each (n <= 4 values: forward, backward, statistics, reserved).
 * `on`: 0 off, 1 all three phases, otherwise a mask of phases (2 forward, 4 backward,
 * 8 statistics): a timed dispatch costs a few microseconds, so a measurement of one
 * kernel inside a throughput run times that kernel only; phases not timed read 0. */
int pcm_set_timing(pcm_circuit* c, int32_t on);
int pcm_get_timing(pcm_circuit* c, float* ms, int32_t n);

/* A plain streaming kernel, for bench.py's `hbm_stream_mix` workload: no counterpart in the reference, a
 * measuring instrument.  One launch reads `reads` streams of `lanes` x 16 bytes from d_src (laid out one after
 * the other) and writes `writes` such streams to d_dst, every access 16 bytes per lane and non-temporal, on a
 * grid of `grid` workgroups of 256 threads; (reads, writes) is one of (1,0) (0,1) (1,1) (4,3) (1,3) (6,1) --
 * the last three are the mixes of the backward walk, the forward walk and the statistics kernel of the EM step.
 * Queued on `stream`, not waited for.  With writes = 0, d_dst still needs 16 valid bytes. */
int pcm_stream_probe(const void* d_src, void* d_dst, int64_t lanes, int32_t reads, int32_t writes, int32_t grid, void* stream);

#ifdef __cplusplus
}
#endif
#endif
