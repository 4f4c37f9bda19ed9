// Dense-block engine for hidden Chow-Liu tree circuits.
//
// An HCLT (reference: src/structures/hclts.jl:100-145) has one K x K block of sum edges
// per non-leaf tree node v:  O_v[b,k] = logsumexp_j(theta_v[k,j] + Z_v[b,j]) with
// Z_v[b,j] = leaf_v[j][x_b,v] + sum over tree children c of (O_c[b,j] or leaf_c[j][x_b,c]).
// The engine never materialises the K^2 product nodes per block; it keeps one K-vector of
// node values (and one of flows) per tree node and example.
#pragma once

#include <memory>

#include "common.hpp"
#include "sparse_engine.hpp"

namespace pcm {

constexpr int kSlice = 16;       // examples per tile
constexpr double kWideNodeUs = 1.2, kWalk64StepUs = 7.6;   // measured costs behind the choice of walk kernels at K = 64
constexpr int kWalkWaves = 16;   // waves per workgroup (= items per step) in the tree-walk kernels
constexpr int kInlineOps = 4;    // static operands held in a step item
constexpr int kInlineLds = 3;    // LDS-resident operands held in a step item
constexpr uint32_t kOpLeaf = 0x80000000u;    // operand is a leaf-table row of variable id
constexpr uint32_t kOpIdMask = 0x003fffffu;  // else: value tile of inner node id
constexpr uint32_t kOpNone = 0x40000000u;    // absent operand: reads as zeros
constexpr int kXSelShift = 28;               // leaf operand: which byte of the packed categories (2 bits)
constexpr int kSlotShift = 22;               // LDS operand: (slot + 1) << kSlotShift | inner id
constexpr int kItemRoot = 1, kItemHasInnerChild = 2, kItemOverflow = 4, kItemSpillOut = 8;
constexpr int kPre = 3;          // static operand tiles a wave requests one step ahead

struct HcltNode {     // one non-leaf tree node, device-resident
  int32_t var;        // its observed variable
  int32_t parent;     // inner id of the tree parent, -1 for the root
  int32_t ic_off, ic_cnt;  // non-leaf tree children (inner ids) in child_inner
  int32_t lc_off, lc_cnt;  // leaf tree children (variable ids) in child_leaf
  int32_t is_root;
  int32_t has_inner_child;
};

// What one wave does in one step of a tree walk (or, for the statistics kernel, what a
// workgroup needs to know about its node).  64 bytes, read with scalar loads.
struct StepItem {
  int32_t node;       // inner id (tile index); idle waves get the trash tile
  int32_t out_slot;   // LDS slot receiving the produced tile (trash slot if nobody reads it)
  int32_t in_slot;    // backward: LDS slot of the parent's flow tile, -1: read it from HBM
  int32_t parent;     // inner id of the tree parent
  int32_t flags;      // kItemRoot | kItemHasInnerChild | kItemOverflow | kItemSpillOut
  int32_t n_g, n_l;   // inline static operands / inline LDS operands
  int32_t ext_off;    // static operands beyond the inline list: ext_ops[ext_off .. +ext_cnt)
  int32_t ext_cnt;
  uint32_t g[kInlineOps];   // static operands, most urgent first
  uint32_t l[kInlineLds];   // forward: inner children as (slot + 1) << kSlotShift | inner id
};
static_assert(sizeof(StepItem) == 64, "StepItem is read as 16 dwords");

// Field rows of a walk schedule (see SchedChunk in the kernels).  kFNode is the tile whose
// value the item reads ahead (backward: its own O tile; idle: the zero tile), kFStore the
// tile index it writes (idle: the trash tile).  kFL0..2: forward: the inner children's
// (slot + 1) << kSlotShift | id; backward: kFL0 = LDS slot of the parent's flow tile (-1:
// in HBM), kFL1 = inner id of the parent.  kFFlags = item flags | n_l << 8.
enum { kFNode = 0, kFWnode, kFG0, kFG1, kFG2, kFStore, kFOutSlot, kFFlags, kFL0, kFL1, kFL2, kSchedFields };

// What a wave has to request ahead for an item: its value tile / parameter block ids and
// its first kPre static operands (absent ones name the zero tile).
struct PreItem {
  int32_t node;    // tile index of the item's own node (idle: the zero tile)
  int32_t wnode;   // parameter block to fetch (idle: block 0)
  uint32_t g[kPre];
  int32_t pad[3];
};
static_assert(sizeof(PreItem) == 32, "PreItem is read as 8 dwords");

// A node as the lean statistics kernel sees it.
struct StatNode {
  int32_t var;        // the node's own variable
  int32_t c[3];       // children: -1 none, leaf child: variable << 3 | 1 | category byte << 1, inner child: node << 3
  int32_t n_hist;     // variables to histogram: own + leaf children
  int32_t hvar[4];    // ... their ids; entry i uses category byte i
  int32_t node;       // the node's index (the records are in the order the workgroups draw them: costliest first)
  int32_t pad[6];
};
static_assert(sizeof(StatNode) == 64, "StatNode is read with scalar loads");

// One slot of a wide walk's schedule: what one of the two groups of waves does in one step (hclt_wide.hip).
struct WideSlot {
  uint32_t op[6];      // operands requested a slot ahead.  0: none; leaf row: bit 31 | category selector << 24 | variable; value tile: bit 30 | node
  int32_t node;        // -1: the group idles this step
  int32_t parent;      // the parent's node, -1 at the root
  int32_t flags;       // bit 0: the root; bit 1: the tile of the group's previous slot is an operand (still in registers)
  int32_t extra_off, extra_cnt;   // operands fetched at the point of use
};
constexpr int kWideRoot = 1, kWidePrev = 2;

// Everything the kernels need, passed by value.
struct HcltDev {
  const HcltNode* nodes;
  const int32_t* child_inner;
  const int32_t* child_leaf;
  const uint32_t* ext_ops;
  const float* leaf;      // [V][C][K] log-probabilities, hidden state fastest
  const float* logtheta;  // [n_inner][K][K]
  const float* Wf;        // exp(theta) laid out per MFMA operand, forward contraction
  const float* Wb;        // same values, operand layout of the backward contraction
  const uint8_t* xb;      // [V][Bp] batch categories, example fastest
  const uint32_t* xn;     // [n_inner][Bp] packed categories of a node's own variable and leaf children
  float* O;               // [n_inner][nslices][16*K] node values, tile-native layout
  float* R;               // [n_inner][nslices][16*K] flow / value ratios of the sum nodes
  float* G;               // child-flow tiles that found no LDS slot (same layout), or null
  float* M;               // [n_inner + 1][Bp] row maxima of the forward walk (row n_inner: idle waves of the lean kernels)
  int* err;               // host-visible word a walk kernel sets when a wave gave up waiting for a tile
  int* err_dev;           // the same in device memory: the update kernels skip their work after such a pass
  const float* w;         // [B] flow every example starts with at a single root (per-example weights), or null: 1
  int32_t B, Bp, nslices, C, n_inner, V;
  uint32_t leaf_stride;   // bytes per variable in the leaf table (C*K*4)
  uint32_t leaf_slice;    // 0; soft evidence: the "leaf table" holds one row per example ([V][Bp][K], the
                          // categories are the example's rank in its slice) and a slice's rows start this many bytes on
  uint32_t tile_stride;   // bytes per node in O / R / G: its slices' tiles, plus one unused tile where that makes the count odd
};

#define PCM_DISPATCH_K(K_, ...)                         \
  switch (K_) {                                         \
    case 16: { constexpr int KK = 16; __VA_ARGS__; break; } \
    case 32: { constexpr int KK = 32; __VA_ARGS__; break; } \
    case 64: { constexpr int KK = 64; __VA_ARGS__; break; } \
    default: fail(PCM_ERR_UNSUPPORTED, "hidden size %d not supported by the block engine", K_); \
  }

// the parameter kernels also serve the wide block sizes
#define PCM_DISPATCH_PARAM_K(K_, ...)                   \
  switch (K_) {                                         \
    case 16: { constexpr int KK = 16; __VA_ARGS__; break; } \
    case 32: { constexpr int KK = 32; __VA_ARGS__; break; } \
    case 64: { constexpr int KK = 64; __VA_ARGS__; break; } \
    case 128: { constexpr int KK = 128; __VA_ARGS__; break; } \
    default: fail(PCM_ERR_UNSUPPORTED, "hidden size %d not supported by the block engine", K_); \
  }

class HcltCircuit : public pcm_circuit {
 public:
  // num_heads > 0: a multi-head circuit, num_heads sum nodes over the root's K products instead of one.
  // forest: `parent` may hold several roots; every tree is a multi-head circuit of its own over the same batch
  // (num_heads heads each), and the handle runs flows and EM for all of them with one launch per kernel.
  HcltCircuit(const int32_t* parent, int V, int K, int C, int num_heads = 0, bool forest = false);
  ~HcltCircuit() override;

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
  int64_t sample_noise_size() const override { return (int64_t)n_user_inner_ * K_; }
  void sample(const float* d_node_noise, const float* d_leaf_noise, int32_t batch,
              uint8_t* d_out) override;
  void adam_step(const float* d_grad, float* d_params, float* d_m, float* d_v, float lr, float b1,
                 float b2, float eps, int t) override;
  void sample_soft(const float* d_node_noise, float temperature, int32_t batch, float* d_out) override;
  void flow_gradients(int32_t batch_size, float* d_grad) override;
  void leaf_adam(float* d_aux_p, float* d_aux_m, float* d_aux_v, float lr, float b1, float b2, float eps, int t) override;
  // Parameter-row queries: the KL recursion and its gradient on the block form with the row as a grid dimension
  // (hclt_kld.hip) for single-root circuits with block kernels; everything else on the circuit's general form (its
  // structure; the rows bring the parameters).
  void kld_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                float* d_out) override;
  void kld_backward_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                         float* d_g1, float* d_g2, float* d_klds) override;
  void kld_rows_block(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm, float* d_klds,
                      float* d_g1, float* d_g2);
  void gumbel_sample_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                          float temperature, bool norm_params, float* d_out) override;
  void gumbel_sample_backward_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                   float temperature, bool norm_params, bool grad_wrt_logparams, const float* d_out_grad,
                                   float* d_grads) override;

  // (both on the general form: the first with the circuit's own parameters, the second on the rows alone)
  void normalized_flows(const BatchRef& b, float* d_out, int64_t sr, int64_t sp, bool as_written) override {
    general()->normalized_flows(b, d_out, sr, sp, as_written);
  }
  void normalize_params_rows(float* d_params, int64_t sr, int64_t sp, int32_t rows, bool undo) override {
    general_structure()->normalize_params_rows(d_params, sr, sp, rows, undo);
  }

  bool sample_soft_block(const float* d_node_noise, float temperature, int32_t batch, float* d_out);
  void set_block_params(const float* theta, const float* leaf);
  // head log-parameters [trees][H][K] (host); a tree's heads are in the order of its head mask rows
  void set_heads(const float* heads);
  void get_heads(float* heads);
  int num_trees() const { return T_; }
  // The last of the num_cats categories becomes the marker of a missing value (see pin_missing_marker).
  void set_missing_category(bool on);
  // soft_reg > 0: categorical batches are smoothed as reg_likelihood.jl:4-14 has it; as_written: leaf statistics as
  // reg_flow.jl:12-17 computes them (log-probabilities in the shares) instead of the derivative of the smoothed value
  void set_soft_reg(float soft_reg, int width, bool as_written);
  // tempered flows run on the circuit's layered form: not for forests and circuits with a missing-value category
  void check_flow_scale(float fscale) {
    if (fscale == 1.f) return;
    no_forest("tempered flows");
    no_missing("tempered flows");
  }
  void get_block_params(float* theta, float* leaf);
  void get_block_flows(float* edge_aggr, float* leaf_flow);

  // Kernel timing: the launches of the phases in the mask (bit 0 forward, 1 backward, 2 statistics) carry a
  // start and a stop event on their own dispatch (no synchronisation); read_timing synchronises and
  // averages the calls recorded since the previous read (at most kTimingRing of them).
  static constexpr int kTimingRing = 64;
  int timing = 0;
  void set_timing(int mask) {
    timing = mask;
    n_timed_ = 0;
  }
  void read_timing(float* ms, int n);

 private:
  int V_, K_, C_, n_inner_, root_;
  int Vu_ = 0;                     // the caller's variables; V_ - Vu_ auxiliary ones behind them (forests only)
  void split_wide_nodes();
  std::vector<std::vector<int32_t>> uchildren_;   // the caller's tree (children of every variable) where nodes were split
  // soft evidence on the block form reads evidence per variable of the stored tree; with auxiliary nodes in it
  // that query takes the general form of the caller's circuit instead
  bool block_queries() const { return block_ && V_ == Vu_; }
  bool forest_ = false;
  int T_ = 1;                      // trees (1 unless a forest)
  int n_groups_ = 1;               // groups of trees the walk kernels take side by side (blockIdx.y)
  // a forest's walk schedules with more, smaller groups of trees, for batches whose slices do not fill the device
  struct LeanPlan {
    int n_groups = 1, n_fwd_steps = 0, fwd_stride = 0, n_bwd_steps = 0, bwd_stride = 0;
    DevBuf<int32_t> fwd, bwd;
  };
  std::vector<std::unique_ptr<LeanPlan>> fine_plans_;
  const LeanPlan* fine_plan(int nslices) const;
  std::vector<int32_t> roots_;     // root variable of every tree, in variable order
  std::vector<int32_t> tree_of_inner_;   // tree of every inner node
  // inner nodes of the caller's tree, and every node's index among them (auxiliary nodes keep the post-order of the
  // caller's nodes as it would be without them): the sampling noise is indexed by this
  int n_user_inner_ = 0;
  std::vector<int32_t> user_index_;
  DevBuf<int32_t> d_user_index_;
  DevBuf<float> d_noise_x_;
  // the sampling noise as the block kernels index it: the caller's array, or a copy with room for the auxiliary nodes
  const float* kernel_noise(const float* d_node_noise, int32_t batch);
  DevBuf<int32_t> d_root_node_;    // ... their nodes
  // what only a single circuit defines (parameter vector order, the general form and the queries on it)
  bool missing_ = false;           // the last category is the marker of a missing value
  void pin_missing_marker();
  // soft_reg smoothing of categorical data on the block kernels (see hclt_leaf_smooth_kernel)
  float soft_reg_ = 0.f;
  int soft_width_ = 1;
  bool soft_written_ = false;
  DevBuf<float> d_leaf_smooth_, d_leaf_hist_;
  DevBuf<float> d_soft_reg_ev_;                 // a smoothed batch as soft evidence, for tempered flows on the layered form
  void leaf_changed();                          // after anything that rewrites the leaf table
  float* stats_leaf_out() { return soft_reg_ > 0.f ? d_leaf_hist_.p : d_leaf_flow_.p; }
  float stats_leaf_rate(float rate) const { return soft_reg_ > 0.f ? 0.f : rate; }
  void soft_reg_counts(float rate);             // histogram by shown category -> leaf statistics
  void no_missing(const char* what) const {
    if (missing_)
      fail(PCM_ERR_UNSUPPORTED, "%s is not defined for a circuit with a missing-value category (likelihoods, flows and EM are)",
           what);
  }
  void no_forest(const char* what) const {
    if (forest_) fail(PCM_ERR_UNSUPPORTED, "%s is not defined for a forest handle: use one handle per tree", what);
  }
  int H_ = 0, Hp_ = 0;             // heads, and heads rounded up to whole operand tiles
  DevBuf<float> d_head_wf_, d_head_wb_;   // head block [Hp][K] in the two operand layouts
  DevBuf<int> d_flow_shift_;              // ceil(log2) of the largest flow one example carried in the last flow pass
  float* head_logp() { return d_logtheta_.p + (size_t)n_inner_ * K_ * K_; }   // [trees][H][K], behind the blocks
  float* head_aggr() { return d_edge_aggr_.p + (size_t)n_inner_ * K_ * K_; }
  void rebuild_heads();
  void heads_forward(const HcltDev& d, const float* d_mask, float* d_ll_heads, float* d_ll_mix, bool flows_follow = false,
                     float rate = 0.f);
  bool block_ = true;   // the hidden size has walk kernels (block tiles in registers)
  bool wide_ = false;   // the hidden size has the wide block kernels (likelihoods, flows, EM); neither: layered engine
  std::vector<int32_t> parent_, inner_of_var_, var_of_inner_, height_, depth_;
  std::vector<std::vector<int32_t>> children_;
  int n_fwd_steps_ = 0, n_bwd_steps_ = 0, lds_slots_ = 0, max_lds_ = 0, n_cus_ = 1;
  bool fwd_spill_ = false, bwd_spill_ = false;
  // parameter-vector order (reference numbering, see build_param_order)
  std::vector<int64_t> sum_param_src_;   // param i -> index into logtheta [n_inner][K][K]
  std::vector<int32_t> sum_group_size_;  // sizes of the normalisation groups, in order
  std::vector<int32_t> input_order_;     // i-th input node -> v*K + j
  std::vector<int64_t> edge2param_, edge_parent_, edge_prime_, edge_sub_, layer_ends_;
  int64_t n_nodes_ = 0, n_edges_ = 0;

  DevBuf<HcltNode> d_nodes_;
  DevBuf<int32_t> d_child_inner_, d_child_leaf_;
  DevBuf<StepItem> d_fwd_sched_, d_bwd_sched_, d_stat_items_;
  DevBuf<int32_t> d_fwd_fields_, d_bwd_fields_, d_fwd_lean_, d_bwd_lean_;
  bool fwd_lean_ = false, bwd_lean_ = false, stat_lean_ = false;   // each lean kernel could run this tree ...
  bool lean_ = false;   // ... and all three do (they share the stored row maxima, so it is all or none)
  DevBuf<float> d_M_;
  int* walk_err_ = nullptr;    // pinned host word the walk kernels raise (HcltDev::err); checked by check_walks()
  void check_walks();
  void sync_checked();   // waits for the stream, then check_walks()
  DevBuf<int32_t> d_walk_void_;   // device copy of the word: non-zero after a void pass, read by the update kernels
  int walk_chunk(int batch) const;
  static BatchRef chunk_of(const BatchRef& b, int off, int chunk);
  // Floats per node in the tile arrays.  The walk engines keep an odd number of tiles per node: with a power
  // of two (a batch of 4096), the tiles that one step reads from different nodes at equal slice offsets fell on
  // the same memory channels (the backward walk ran 4 % slower).  The wide kernels index by slice count.
  size_t tile_floats(int ns) const { return (size_t)((wide_ || wide_walk_) ? ns : (ns | 1)) * kSlice * K_; }
  int stat_lean_hists_ = 1;   // histograms the lean statistics kernel holds in LDS per pass
  DevBuf<StatNode> d_stat_lean_;
  DevBuf<uint32_t> d_stat_claim_;   // the statistics workgroups draw their nodes from this counter; zero between launches
  int fwd_stride_ = 0, bwd_stride_ = 0;
  DevBuf<uint32_t> d_ext_ops_;
  DevBuf<float> d_leaf_, d_logtheta_, d_Wf_, d_Wb_, d_edge_aggr_, d_leaf_flow_, d_O_, d_R_, d_G_;
  DevBuf<uint8_t> d_xb_;
  DevBuf<uint32_t> d_xn_;
  DevBuf<float> d_leaf_kc_;      // [V][K][C] copy for sampling
  DevBuf<float> d_kld_;          // scratch of the KL recursion
  DevBuf<uint8_t> d_state_;      // [batch][n_inner] hidden states of a batch of samples
  DevBuf<int32_t> d_soft_tabs_;     // relaxed sampler: parents | leaf-feeding nodes | nodes by depth | level offsets
  DevBuf<float> d_soft_w_;          // ... exp(theta / T) in the two operand layouts
  int soft_levels_ = 0;
  DevBuf<int32_t> d_sample_tabs_;   // sampler tables: parent of every inner node | state-giving node of every variable | level order
  DevBuf<int32_t> d_sample_passes_;   // the sampler's levels from the root in records of 64 {node, parent} pairs
  int sample_passes_ = 0;
  DevBuf<int64_t> d_sum_param_src_;
  DevBuf<int32_t> d_in_pos_;   // input node (v, j) -> its position among the input nodes of the parameter vector
  DevBuf<float> d_param_vec_;  // a parameter vector on its way to or from the host
  DevBuf<float> d_part_;       // rows of partial sums (head statistics per slice, soft leaf counts per split)
  DevBuf<float> d_row_sum_;    // Adam from flows: per-sum-node / per-input-node flow totals
  DevBuf<int32_t> d_input_order_;   // i-th input node of the parameter vector -> v*K + j
  int cap_slices_ = 0;
  bool have_flows_ = false;
  // soft evidence on the block kernels (single head, K <= 64)
  bool soft_block_ok() const { return block_queries() && !wide_ && H_ == 0; }
  HcltDev soft_stage(const SoftRef& s);
  DevBuf<float> d_soft_lv_, d_soft_m_;   // value table [V][Bp][K] and largest evidence [V][Bp] of the batch
  DevBuf<int32_t> d_soft_gnode_;
  bool force_general_walks_ = false;
  bool wide_walk_ = false;            // forward / backward / statistics run on the node-at-a-time wide kernels
  bool flows_in_general_ = false;   // the last flows were computed by the layered engine (soft evidence)
  std::vector<hipEvent_t> ev_;   // kTimingRing sets of 6 events: start and stop of the forward, backward, statistics phase
  int n_timed_ = 0;
  hipEvent_t* ev_set();

  FlatCircuit flat_;                       // the same circuit in general form (structure only)
  std::vector<int32_t> noise_slot_;       // per up edge: column of the compact sampling noise
  std::unique_ptr<SparseCircuit> general_; // built on first use by the KL / sampling / Adam queries
  bool general_stale_ = true;
  SparseCircuit* general();
  SparseCircuit* general_structure();   // the same object without bringing its parameters up to date
  // KL recursion on the block form
  DevBuf<int32_t> d_kl_up_, d_kl_down_;   // chain steps (KlItem records) bottom-up / top-down
  DevBuf<int32_t> d_blk2par_;             // entry of the [n_inner][K][K] blocks -> parameter (-1: no such edge), for the row queries
  DevBuf<float> d_rows_scratch_, d_rows_pk1_, d_rows_pk2_, d_rows_pg1_, d_rows_pg2_;   // row queries: per-row arrays; re-laid-out matrices
  DevBuf<int32_t> d_kl_tabs_;             // parent of every inner node | h-giving node of every variable | input-node positions
  DevBuf<int32_t> d_kl_pos_;              // chain slot of every inner node: upward | downward
  DevBuf<float> d_kl_leaf_, d_kl_vec_, d_kl_par_;
  DevBuf<int32_t> d_kl_ext_;              // chain slots of the children past the second, of nodes with more than three
  int kl_up_steps_ = 0, kl_down_steps_ = 0;
  int kl_ring_slots_ = 0;                 // slots of the chains' LDS ring; 0: levels too wide, the ring is the whole chain in device memory
  HcltCircuit* same_tree(pcm_circuit* q);
  void build_kld_tables();
  void kld_device(HcltCircuit* q, bool with_down);
  void pull_from_general();
  void build_structure();
  void build_schedules();
  void build_param_order();
  void ensure_batch(int batch);
  HcltDev dev(int batch) const;
  void stage_batch(const BatchRef& b);
  void rebuild_w();
  void run_forward(const HcltDev& d, float* d_ll);
  void run_backward(const HcltDev& d);
  void run_stats(const HcltDev& d, float rate);
  // wide block kernels
  DevBuf<float> d_wide_rs_, d_wide_es_;   // R and E of every node in the operand layout of the statistics contraction
  DevBuf<int32_t> d_wide_state_node_;     // per variable: the inner node whose flow tile feeds its leaf histogram
  DevBuf<WideSlot> d_wide_fwd_, d_wide_bwd_;   // [steps][2 groups]
  int wide_steps_f_ = 0, wide_steps_b_ = 0;
  DevBuf<uint32_t> d_wide_extra_;
  void build_wide_tables();
  void wide_forward(const HcltDev& d, float* d_ll);
  void wide_backward_stats(const HcltDev& d, float rate, bool soft = false);
};

}  // namespace pcm
