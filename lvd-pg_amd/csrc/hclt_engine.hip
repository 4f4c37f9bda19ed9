// Host side of the dense-block HCLT engine: structure, schedules, parameter order,
// launches.
#include <hip/hip_ext.h>

#include "hclt_engine.hpp"

#include <algorithm>
#include <cmath>
#include <functional>
#include <numeric>

#include "hclt_walk_lean.hip.hpp"
#include "hclt_soft_sample.hip.hpp"
#include "hclt_heads.hip.hpp"
#include "lean_schedule_check.hpp"
#include "hclt_soft_evidence.hip.hpp"

namespace pcm {

// the lean walk kernels exist for the hidden sizes whose blocks fit the register file
#define PCM_DISPATCH_LEAN_K(K_, ...)                    \
  switch (K_) {                                         \
    case 16: { constexpr int KK = 16; __VA_ARGS__; break; } \
    case 32: { constexpr int KK = 32; __VA_ARGS__; break; } \
    default: fail(PCM_ERR_STATE, "no lean walk kernel for hidden size %d", K_); \
  }

// A launch of one of the three timed phases (0 forward, 1 backward, 2 statistics).  With timing on, the phase's
// start / stop events ride on the kernel's own dispatch: events recorded between the kernels of a step are
// packets of their own that keep the next kernel waiting (measured: about 6 us each).
#define PCM_LAUNCH_PHASE(phase, kernel, grid, block, lds, ...)                                                       \
  do {                                                                                                               \
    if (timing & (1 << (phase))) {                                                                                   \
      hipEvent_t* ev__ = ev_set() + 2 * (phase);                                                                     \
      hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)(lds), stream, ev__[0], ev__[1], 0, __VA_ARGS__);        \
    } else {                                                                                                         \
      hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                                             \
    }                                                                                                                \
  } while (0)

static void check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

HcltCircuit::HcltCircuit(const int32_t* parent, int V, int K, int C, int num_heads, bool forest)
    : V_(V), K_(K), C_(C), forest_(forest) {
  if (num_heads < 0 || num_heads > 4096) fail(PCM_ERR_SHAPE, "num_heads must be in 0..4096, got %d", num_heads);
  if (forest && num_heads < 1) fail(PCM_ERR_SHAPE, "the trees of a forest are multi-head circuits: num_heads must be positive");
  H_ = num_heads;
  Hp_ = ceil_div(num_heads, 16) * 16;
  if (!parent) fail(PCM_ERR_ARG, "clt_parent is null");
  if (V < 2) fail(PCM_ERR_SHAPE, "an HCLT needs at least 2 variables, got %d", V);
  if (K < 1 || K > 1024) fail(PCM_ERR_SHAPE, "num_hidden_cats must be in 1..1024, got %d", K);
  // hidden sizes without block kernels run every query on the layered engine over the
  // circuit's general form; the block-form parameter interface stays the same
  block_ = K == 16 || K == 32 || K == 64;
  wide_ = K == 128;
  if (C < 1 || C > 256) fail(PCM_ERR_SHAPE, "num_cats must be in 1..256 (uint8 data), got %d", C);
  parent_.assign(parent, parent + V);
  Vu_ = V;
  // (single circuits too, where the lean kernels exist: otherwise one node with four children would put the whole
  // circuit on the general walk kernels, 1.4 x slower on the 3072-variable tree)
  if (forest_ || K == 16 || K == 32) split_wide_nodes();
  build_structure();
  // K = 64: a parameter block and its prefetched successor do not fit the 128 registers a wave of the 16-wave
  // walk kernels has, so those kernels spill (6 us per step); the node-at-a-time wide kernels take about
  // kWideNodeUs per node instead and win unless the tree is bushy enough to fill the 16 waves of a step
  wide_walk_ = wide_ || (K == 64 && (double)n_inner_ * kWideNodeUs < (double)(n_fwd_steps_ + n_bwd_steps_) * 0.5 * kWalk64StepUs);
  if (H_ > 0 && !(block_ && K <= 32))
    fail(PCM_ERR_UNSUPPORTED, "multi-head block kernels need K = 16 or 32; compile this circuit with pcm_circuit_create");
  if (forest_ && !lean_)
    fail(PCM_ERR_UNSUPPORTED, "a forest needs trees the lean walk kernels take (at most three children per node, "
                              "every tile in LDS); use one handle per tree");
  if (!forest_) build_param_order();

  // uniform parameters
  std::vector<float> theta((size_t)Vu_ * K_ * K_, -std::log((float)K_));
  std::vector<float> leaf((size_t)Vu_ * K_ * C_, -std::log((float)C_));
  d_leaf_.alloc((size_t)V_ * C_ * K_);
  d_logtheta_.alloc((size_t)n_inner_ * K_ * K_ + (size_t)T_ * H_ * K_);   // the head rows sit behind the blocks
  d_Wf_.alloc((size_t)n_inner_ * K_ * K_);
  d_Wb_.alloc((size_t)n_inner_ * K_ * K_);
  d_edge_aggr_.alloc((size_t)n_inner_ * K_ * K_ + (size_t)T_ * H_ * K_);
  if (H_ > 0) {
    d_head_wf_.alloc((size_t)T_ * Hp_ * K_);
    d_head_wb_.alloc((size_t)T_ * Hp_ * K_);
    std::vector<int32_t> rn;
    for (int r : roots_) rn.push_back(inner_of_var_[r]);
    d_root_node_.upload(rn);
    std::vector<float> hl((size_t)T_ * H_ * K_, -std::log((float)K_));
    PCM_HIP(hipMemcpy(head_logp(), hl.data(), hl.size() * sizeof(float), hipMemcpyHostToDevice));
  }
  d_flow_shift_.alloc(1);
  d_leaf_flow_.alloc((size_t)V_ * C_ * K_);
  d_edge_aggr_.zero();
  d_leaf_flow_.zero();
  set_block_params(theta.data(), leaf.data());
}

// The lean walk kernels hold three children per tree node.  A forest meets that by construction: a node with
// more children hands the last two or three of them to an auxiliary node below it, a tree node over a variable
// of its own that nobody observes (variables Vu_ .. V_-1: one category with probability 1, so its leaf row adds
// nothing) with the identity as its block (so its sum nodes ARE its products: the value of the K products
// the children form goes up unchanged, the flow goes down unchanged).  The update kernels leave the auxiliary
// blocks and leaf rows alone, and the caller's arrays never show them.  It is the same circuit: a product of
// five factors written as a product of three, one of which is a product of three.
void HcltCircuit::split_wide_nodes() {
  for (int v = 0; v < Vu_; ++v)
    if (parent_[v] >= Vu_ || parent_[v] == v) fail(PCM_ERR_SHAPE, "clt_parent[%d] = %d is out of range", v, parent_[v]);
  std::vector<std::vector<int32_t>>& ch = uchildren_;
  ch.assign(Vu_, {});
  for (int v = 0; v < Vu_; ++v)
    if (parent_[v] >= 0) ch[parent_[v]].push_back(v);
  for (int v = 0; v < Vu_; ++v) {
    std::vector<int32_t> c = ch[v];
    while (c.size() > 3) {
      const size_t take = std::min<size_t>(3, c.size() - 2);
      const int u = (int)parent_.size();
      parent_.push_back(v);
      for (size_t i = c.size() - take; i < c.size(); ++i) parent_[c[i]] = u;
      c.resize(c.size() - take);
      c.push_back(u);
    }
  }
  V_ = (int)parent_.size();
}

void HcltCircuit::build_structure() {
  children_.assign(V_, {});
  root_ = -1;
  roots_.clear();
  for (int v = 0; v < V_; ++v) {
    int p = parent_[v];
    if (p < 0) {
      if (root_ >= 0 && !forest_) fail(PCM_ERR_SHAPE, "clt_parent has more than one root (%d and %d)", root_, v);
      if (root_ < 0) root_ = v;
      roots_.push_back(v);
    } else {
      if (p >= V_ || p == v) fail(PCM_ERR_SHAPE, "clt_parent[%d] = %d is out of range", v, p);
      children_[p].push_back(v);
    }
  }
  if (root_ < 0) fail(PCM_ERR_SHAPE, "clt_parent has no root (-1 entry)");
  // bottom-up order by iterative post-order; detects cycles / unreachable nodes
  std::vector<int32_t> order;
  order.reserve(V_);
  std::vector<std::pair<int32_t, int32_t>> st;
  depth_.assign(V_, -1);
  T_ = (int)roots_.size();
  for (int r : roots_) {   // tree after tree
    if (children_[r].empty()) fail(PCM_ERR_SHAPE, "variable %d is a tree of its own: a tree needs at least 2 variables", r);
    st.push_back({r, 0});
    depth_[r] = 0;
    while (!st.empty()) {
      auto& top = st.back();
      int v = top.first;
      if (top.second < (int)children_[v].size()) {
        int c = children_[v][top.second++];
        depth_[c] = depth_[v] + 1;
        st.push_back({c, 0});
      } else {
        order.push_back(v);
        st.pop_back();
      }
    }
  }
  if ((int)order.size() != V_) fail(PCM_ERR_SHAPE, "clt_parent is not a tree: %d of %d variables reach a root",
                                    (int)order.size(), V_);
  inner_of_var_.assign(V_, -1);
  var_of_inner_.clear();
  height_.assign(V_, 0);
  for (int v : order) {
    if (children_[v].empty()) continue;
    inner_of_var_[v] = (int)var_of_inner_.size();
    var_of_inner_.push_back(v);
    int h = 0;
    for (int c : children_[v]) h = std::max(h, height_[c]);
    height_[v] = h + 1;
  }
  n_inner_ = (int)var_of_inner_.size();
  user_index_.assign(n_inner_, -1);
  n_user_inner_ = 0;
  for (int n = 0; n < n_inner_; ++n)
    if (var_of_inner_[n] < Vu_) user_index_[n] = n_user_inner_++;
  // post-order goes tree after tree: a node's tree is the number of roots before it
  tree_of_inner_.assign(n_inner_, 0);
  for (int n = 0, t = 0; n < n_inner_; ++n) {
    tree_of_inner_[n] = t;
    if (parent_[var_of_inner_[n]] < 0) ++t;
  }

  std::vector<HcltNode> nodes(n_inner_);
  std::vector<int32_t> ci, cl;
  for (int n = 0; n < n_inner_; ++n) {
    int v = var_of_inner_[n];
    HcltNode& nd = nodes[n];
    nd.var = v;
    nd.parent = parent_[v] < 0 ? -1 : inner_of_var_[parent_[v]];
    nd.is_root = v >= Vu_ ? 2 : parent_[v] < 0;   // (2: an auxiliary node, whose identity block no update touches)
    nd.ic_off = (int)ci.size();
    nd.lc_off = (int)cl.size();
    for (int c : children_[v]) {
      if (children_[c].empty()) cl.push_back(c); else ci.push_back(inner_of_var_[c]);
    }
    nd.ic_cnt = (int)ci.size() - nd.ic_off;
    nd.lc_cnt = (int)cl.size() - nd.lc_off;
    nd.has_inner_child = nd.ic_cnt > 0;
  }
  if (ci.empty()) ci.push_back(0);
  if (cl.empty()) cl.push_back(0);
  d_nodes_.upload(nodes);
  d_child_inner_.upload(ci);
  d_child_leaf_.upload(cl);

  if (block_) build_schedules();
}

// Step schedules of the two tree walks.  Every step holds at most kWalkWaves nodes whose
// dependencies were produced in earlier steps; among the ready nodes those with the longest
// remaining chain go first (for unit-time tasks on a tree this greedy rule gives the fewest
// steps).  The host also places every produced tile into one of the LDS slots, for as long
// as a later step still reads it.
void HcltCircuit::build_schedules() {
  if (!walk_err_) {
    PCM_HIP(hipHostMalloc((void**)&walk_err_, sizeof(int), hipHostMallocMapped));
    *walk_err_ = 0;
    d_walk_void_.upload(std::vector<int32_t>(1, 0));
  }
  int dev_id = 0;
  PCM_HIP(hipGetDevice(&dev_id));
  PCM_HIP(hipDeviceGetAttribute(&max_lds_, hipDeviceAttributeMaxSharedMemoryPerBlock, dev_id));
  PCM_HIP(hipDeviceGetAttribute(&n_cus_, hipDeviceAttributeMultiprocessorCount, dev_id));
  const int tile_bytes = kSlice * K_ * (int)sizeof(float);
  // (the lean walks keep one state word per slot behind the slots)
  lds_slots_ = std::min((max_lds_ - kLeanFlagWords * 4) / tile_bytes, (1 << (31 - kSlotShift)) - 2);
  if (lds_slots_ < 3) fail(PCM_ERR_UNSUPPORTED, "device offers %d bytes of LDS, a value tile needs %d", max_lds_, tile_bytes);
  const int trash_slot = lds_slots_ - 1;          // idle waves and childless nodes write here

  std::vector<std::vector<int32_t>> ic(n_inner_), lc(n_inner_);
  std::vector<int32_t> par(n_inner_, -1), hin(n_inner_, 0);   // hin: longest chain of inner nodes below
  for (int n = 0; n < n_inner_; ++n) {
    const int v = var_of_inner_[n];
    if (parent_[v] >= 0) par[n] = inner_of_var_[parent_[v]];
    for (int c : children_[v]) {
      if (children_[c].empty()) lc[n].push_back(c);
      else { ic[n].push_back(inner_of_var_[c]); hin[n] = std::max(hin[n], hin[inner_of_var_[c]] + 1); }
    }
  }
  std::vector<uint32_t> ext;
  // a leaf child's row operand: its category is byte 1 + i of the node's packed word (the
  // word holds the first three leaf children; later ones only occur beyond the kPre
  // requested-ahead operands, where the category is fetched on the spot)
  auto leaf_child_op = [&](int var, size_t i) {
    return kOpLeaf | (uint32_t)var | ((uint32_t)std::min<size_t>(i + 1, 3) << kXSelShift);
  };
  auto fill_ops = [&](StepItem& it, PreItem& q, const std::vector<uint32_t>& ops) {
    it.n_g = (int32_t)std::min<size_t>(ops.size(), kInlineOps);
    for (int i = 0; i < kInlineOps; ++i) it.g[i] = i < it.n_g ? ops[i] : 0;
    for (int i = 0; i < kPre; ++i) q.g[i] = i < (int)ops.size() ? ops[i] : kOpNone;
    it.ext_off = (int32_t)ext.size();
    it.ext_cnt = 0;
    if (ops.size() > (size_t)kPre) it.flags |= kItemOverflow;
    if (ops.size() > (size_t)kInlineOps) {
      it.ext_cnt = (int32_t)(ops.size() - kInlineOps);
      ext.insert(ext.end(), ops.begin() + kInlineOps, ops.end());
    }
  };
  auto blank = [&](int n) {
    StepItem it;
    std::memset(&it, 0, sizeof it);
    it.node = n;
    it.out_slot = trash_slot; it.in_slot = trash_slot; it.parent = n >= 0 ? par[n] : -1;
    if (n >= 0) it.flags = (par[n] < 0 ? kItemRoot : 0) | (ic[n].empty() ? 0 : kItemHasInnerChild);
    return it;
  };
  auto blank_pre = [&](int n) {
    PreItem q;
    std::memset(&q, 0, sizeof q);
    q.node = n;
    q.wnode = n;
    for (int i = 0; i < kPre; ++i) q.g[i] = kOpNone;
    return q;
  };
  // field rows [field][wave][stride] with 64 idle steps of padding (a chunk refill reads
  // 64 steps starting anywhere below n_steps)
  auto make_fields = [&](std::vector<StepItem>& sched, std::vector<PreItem>& pre, bool forward, int& stride,
                         DevBuf<int32_t>& dst) {
    const int n_steps = (int)sched.size() / kWalkWaves;
    for (int i = 0; i < 64 * kWalkWaves; ++i) { sched.push_back(blank(-1)); pre.push_back(blank_pre(-1)); }
    stride = n_steps + 64;
    std::vector<int32_t> f((size_t)kSchedFields * kWalkWaves * stride, 0);
    for (int s = 0; s < stride; ++s)
      for (int w = 0; w < kWalkWaves; ++w) {
        const StepItem& it = sched[(size_t)s * kWalkWaves + w];
        const PreItem& q = pre[(size_t)s * kWalkWaves + w];
        auto put = [&](int field, int32_t v) { f[((size_t)field * kWalkWaves + w) * stride + s] = v; };
        put(kFNode, q.node); put(kFWnode, q.wnode);
        put(kFG0, (int32_t)q.g[0]); put(kFG1, (int32_t)q.g[1]); put(kFG2, (int32_t)q.g[2]);
        put(kFStore, it.node); put(kFOutSlot, it.out_slot);
        put(kFFlags, it.flags | (it.n_l << 8));
        if (forward) { put(kFL0, (int32_t)it.l[0]); put(kFL1, (int32_t)it.l[1]); put(kFL2, (int32_t)it.l[2]); }
        else { put(kFL0, it.in_slot); put(kFL1, it.parent < 0 ? 0 : it.parent); put(kFL2, 0); }
      }
    dst.upload(f);
  };
  // lean schedule rows (see hclt_walk_lean.hip.hpp) from the padded items of a walk, or none
  // if some node has more operands than the lean kernels hold
  const size_t leaf_stride = (size_t)C_ * K_ * sizeof(float);
  // (backward: ratio_slot[n] is the LDS slot in which node n finds its ratio tile, left there by its parent)
  auto make_lean = [&](const std::vector<StepItem>& sched, bool forward, int stride, std::vector<int32_t>& dst,
                       const std::vector<int32_t>* ratio_slot = nullptr) -> bool {
    if (K_ > 32 || lds_slots_ > 255 || (size_t)V_ * leaf_stride >= ((size_t)1 << 31)) return false;
    const size_t f0 = dst.size();   // (the rows of a further group of trees go behind those of the groups before)
    dst.resize(f0 + (size_t)kLeanFields * kWalkWaves * stride, 0);
    int32_t* f = dst.data() + f0;
    // how often each slot has been filled so far: a step's reads see the fills of earlier steps only, so the
    // readers of a step are numbered before its writers
    std::vector<int32_t> fills(256, 0);
    for (int s = 0; s < stride; ++s) {
      for (int pass = 0; pass < 2; ++pass)
        for (int w = 0; w < kWalkWaves; ++w) {
          const StepItem& it = sched[(size_t)s * kWalkWaves + w];
          if (it.node < 0) continue;
          int32_t& turns = f[((size_t)kLTurns * kWalkWaves + w) * stride + s];
          if (!forward) {   // a node reads the slot its parent filled and fills one per inner child
            const int n = it.node;
            if (pass == 0) {
              if (par[n] >= 0) turns |= (fills[(*ratio_slot)[n]] - 1) & 0x7f;
            } else {
              int q = 0;
              for (int c : ic[n]) turns |= (fills[(*ratio_slot)[c]]++ & 0x7f) << (8 * ++q);
            }
            continue;
          }
          if (pass == 0) {
            for (int c = 0; c < it.n_l; ++c) {
              const int sl = (int)(it.l[c] >> kSlotShift) - 1;
              if (sl >= 0) turns |= ((fills[sl] - 1) & 0x7f) << (8 * (c + 1));
            }
          } else if (it.out_slot != trash_slot) {
            turns |= fills[it.out_slot]++ & 0x7f;
          }
        }
    }
    for (int s = 0; s < stride; ++s)
      for (int w = 0; w < kWalkWaves; ++w) {
        const StepItem& it = sched[(size_t)s * kWalkWaves + w];
        auto put = [&](int field, int32_t v) { f[((size_t)field * kWalkWaves + w) * stride + s] = v; };
        const int n = it.node;
        put(kLA1, -1); put(kLA2, -1); put(kLA3, -1);
        if (n < 0) {   // idle: trash tile, trash slot, block and leaf rows of node / variable 0
          put(kLNode, n_inner_);
          put(kLSlots, (int32_t)(0xffffff00u | (uint32_t)trash_slot));
          continue;
        }
        put(kLW, (int32_t)((size_t)n * K_ * K_ * sizeof(float)));
        put(kLA0, (int32_t)((size_t)var_of_inner_[n] * leaf_stride));
        put(kLNode, n);
        put(kLFlags, par[n] < 0 ? (H_ > 0 ? 3 : 1) : 0);
        if (forward) {
          if (lc[n].size() > 3 || ic[n].size() > 3) return false;
          for (size_t i = 0; i < lc[n].size(); ++i) put(kLA1 + (int)i, (int32_t)((size_t)lc[n][i] * leaf_stride));
          uint32_t slots = (uint32_t)it.out_slot | 0xffffff00u;
          for (int c = 0; c < it.n_l; ++c) {
            const int sl = (int)(it.l[c] >> kSlotShift) - 1;
            if (sl < 0) return false;
            slots = (slots & ~(0xffu << (8 * (c + 1)))) | ((uint32_t)sl << (8 * (c + 1)));
          }
          put(kLSlots, (int32_t)slots);
        } else {
          if (lc[n].size() + ic[n].size() > 3) return false;
          int q = 0;
          uint32_t slots = (uint32_t)(par[n] < 0 ? trash_slot : (*ratio_slot)[n]) | 0xffffff00u;
          for (int c : ic[n]) {
            slots = (slots & ~(0xffu << (8 * (q + 1)))) | ((uint32_t)(*ratio_slot)[c] << (8 * (q + 1)));
            put(kLA1 + q++, c << 3);
          }
          for (size_t i = 0; i < lc[n].size(); ++i)
            put(kLA1 + q++, (int32_t)((size_t)lc[n][i] * leaf_stride) | 1 | (int32_t)((i + 1) << 1));
          put(kLSlots, (int32_t)slots);
        }
      }
    // the waits and posts of all waves, replayed: a schedule on which a wave would wait for ever is refused here
    static_assert(kLeanCheckA1 == kLA1 && kLeanCheckSlots == kLSlots && kLeanCheckTurns == kLTurns &&
                  kLeanCheckFields == kLeanFields && kLeanCheckWaves == kWalkWaves, "lean_schedule_check.hpp follows the lean field rows");
    const int stuck = lean_schedule_stuck_at(f, stride, stride, forward, trash_slot);
    if (stuck >= 0)
      fail(PCM_ERR_STATE, "%s walk schedule is unsound: wave %d would wait for ever in step %d", forward ? "forward" : "backward",
           stuck % kWalkWaves, stuck / kWalkWaves);
    return true;
  };
  auto depth_of = [&](int n) { return depth_[var_of_inner_[n]]; };

  // A forest's trees are walked in groups side by side (blockIdx.y of the walk kernels): each group of whole trees
  // has a schedule of its own, so that a batch too small to fill the device with its slices (1024 examples are 64
  // workgroups) still does.  Groups are node ranges (post-order goes tree after tree) of about equal size.
  auto make_groups = [&](int G) {
    std::vector<std::pair<int, int>> gr;
    int n0 = 0;
    for (int g = 0; g < G && n0 < n_inner_; ++g) {
      // up to the end of the tree in which this group's share of the nodes is reached
      const int want = (int)((int64_t)n_inner_ * (g + 1) / G);
      int n1 = std::max(n0 + 1, want);
      while (n1 < n_inner_ && tree_of_inner_[n1] == tree_of_inner_[n1 - 1]) ++n1;
      if (g == G - 1) n1 = n_inner_;
      gr.push_back({n0, n1});
      n0 = n1;
    }
    return gr;
  };
  const std::vector<std::pair<int, int>> groups = make_groups(forest_ ? std::max(1, std::min(4, T_ / 8)) : 1);
  n_groups_ = (int)groups.size();

  // ---- forward -----------------------------------------------------------------------
  auto schedule_forward = [&](int g0, int g1, std::vector<StepItem>& sched, std::vector<PreItem>& pre) {
    std::vector<int32_t> pending(n_inner_), slot(n_inner_, -1), free_slots;
    for (int s = trash_slot - 1; s >= 0; --s) free_slots.push_back(s);
    // max-heap: deeper first, then lower id (post-order).  In a forest the earlier tree goes first whatever the
    // depth: the trees then pass through the waves one behind the other, a few at a time, and the tiles that wait
    // for a parent in LDS are those of a few trees instead of all.
    auto cmp = [&](int a, int b) {
      if (tree_of_inner_[a] != tree_of_inner_[b]) return tree_of_inner_[a] > tree_of_inner_[b];
      return depth_of(a) != depth_of(b) ? depth_of(a) < depth_of(b) : a > b;
    };
    // ... and a node without inner children, which fills a slot and frees none, only starts while more than a
    // step's worth of slots is free (or nothing else can run)
    const int producer_reserve = T_ > 1 ? kWalkWaves : 0;
    std::vector<int32_t> ready;
    for (int n = g0; n < g1; ++n) { pending[n] = (int)ic[n].size(); if (!pending[n]) ready.push_back(n); }
    std::make_heap(ready.begin(), ready.end(), cmp);
    int done = 0;
    while (done < g1 - g0) {
      // nodes whose flow tile needs an LDS slot wait while none is free (their turn comes
      // when children of earlier nodes have drained); only if nothing else is ready does a
      // tile go through HBM instead
      std::vector<int32_t> step, deferred;
      int slots_left = (int)free_slots.size();
      while (!ready.empty() && (int)step.size() < kWalkWaves) {
        std::pop_heap(ready.begin(), ready.end(), cmp);
        const int n = ready.back();
        ready.pop_back();
        if (T_ > 1) {
          if (par[n] >= 0) {
            if (slots_left <= (ic[n].empty() ? producer_reserve : 0)) { deferred.push_back(n); continue; }
            --slots_left;
          }
        } else if (!ic[n].empty()) {
          if (slots_left == 0) { deferred.push_back(n); continue; }
          --slots_left;
        }
        step.push_back(n);
      }
      if (step.empty() && !deferred.empty()) {
        // nothing fits: the first of the waiting nodes in heap order (a forest) / the last (one tree) goes anyway
        const size_t pick = T_ > 1 ? 0 : deferred.size() - 1;
        step.push_back(deferred[pick]);
        deferred.erase(deferred.begin() + (std::ptrdiff_t)pick);
      }
      for (int n : deferred) { ready.push_back(n); std::push_heap(ready.begin(), ready.end(), cmp); }
      if (step.empty()) fail(PCM_ERR_SHAPE, "forward schedule stalled (tree is inconsistent)");
      for (int w = 0; w < kWalkWaves; ++w) {
        if (w >= (int)step.size()) { sched.push_back(blank(-1)); pre.push_back(blank_pre(-1)); continue; }
        const int n = step[w];
        StepItem it = blank(n);
        PreItem q = blank_pre(n);
        std::vector<uint32_t> ops;
        ops.push_back(kOpLeaf | (uint32_t)var_of_inner_[n]);
        for (size_t i = 0; i < lc[n].size(); ++i) ops.push_back(leaf_child_op(lc[n][i], i));
        it.n_l = 0;
        for (int c : ic[n]) {
          if (it.n_l < kInlineLds) {
            it.l[it.n_l++] = ((uint32_t)(slot[c] + 1) << kSlotShift) | (uint32_t)c;
          } else {
            // read back from HBM, and only at the point of use: the child may have been
            // produced in the step before this one, when the requests ahead were already out
            while (ops.size() < (size_t)kPre) ops.push_back(kOpNone);
            ops.push_back((uint32_t)c);
            fwd_spill_ = true;
          }
          if (slot[c] < 0) fwd_spill_ = true;
        }
        fill_ops(it, q, ops);
        if (par[n] >= 0 && !free_slots.empty()) { slot[n] = free_slots.back(); free_slots.pop_back(); }
        if (slot[n] >= 0) it.out_slot = slot[n];
        sched.push_back(it);
        pre.push_back(q);
      }
      for (int n : step) {
        for (int c : ic[n]) if (slot[c] >= 0) free_slots.push_back(slot[c]);
        if (par[n] >= 0 && --pending[par[n]] == 0) { ready.push_back(par[n]); std::push_heap(ready.begin(), ready.end(), cmp); }
        ++done;
      }
    }
  };
  // The lean backward walk hands every inner child its own tile: a slot per (parent, inner child) pair, taken
  // in the parent's step and free again from the step after the child's.  False if the slots run out.
  auto assign_ratio_slots = [&](const std::vector<StepItem>& sched, std::vector<int32_t>& ratio_slot) {
    const int g_steps = (int)sched.size() / kWalkWaves;
    std::vector<int32_t> fs;
    for (int sl = trash_slot - 1; sl >= 0; --sl) fs.push_back(sl);
    for (int st = 0; st < g_steps; ++st) {
      std::vector<int32_t> freed;
      for (int w = 0; w < kWalkWaves; ++w) {
        const int n = sched[(size_t)st * kWalkWaves + w].node;
        if (n < 0) continue;
        if (par[n] >= 0) freed.push_back(ratio_slot[n]);
        for (int c : ic[n]) {
          if (fs.empty()) return false;
          ratio_slot[c] = fs.back();
          fs.pop_back();
        }
      }
      fs.insert(fs.end(), freed.begin(), freed.end());
    }
    return true;
  };
  auto pad_steps = [&](std::vector<StepItem>& sched, std::vector<PreItem>& pre, int steps) {
    while ((int)sched.size() < steps * kWalkWaves) { sched.push_back(blank(-1)); pre.push_back(blank_pre(-1)); }
  };
  {
    fwd_spill_ = false;
    std::vector<std::vector<StepItem>> sched(n_groups_);
    std::vector<std::vector<PreItem>> pre(n_groups_);
    n_fwd_steps_ = 0;
    for (int g = 0; g < n_groups_; ++g) {
      schedule_forward(groups[g].first, groups[g].second, sched[g], pre[g]);
      n_fwd_steps_ = std::max(n_fwd_steps_, (int)sched[g].size() / kWalkWaves);
    }
    std::vector<int32_t> lean_rows;
    fwd_lean_ = !fwd_spill_;
    for (int g = 0; g < n_groups_; ++g) {
      pad_steps(sched[g], pre[g], n_fwd_steps_);   // the shorter groups idle at the end
      if (g == 0) make_fields(sched[g], pre[g], true, fwd_stride_, d_fwd_fields_);
      else pad_steps(sched[g], pre[g], fwd_stride_);
      fwd_lean_ = fwd_lean_ && make_lean(sched[g], true, fwd_stride_, lean_rows);
    }
    if (fwd_lean_) d_fwd_lean_.upload(lean_rows);
    d_fwd_sched_.upload(sched[0]);
  }
  // ---- backward ----------------------------------------------------------------------
  // Oldest-ready first (ties: longest chain below first): a parent's flow tile then leaves
  // its LDS slot a few steps after it was produced, so the number of live tiles stays near
  // the width of the tree instead of growing with every postponed short subtree.
  auto schedule_backward = [&](int g0, int g1, std::vector<StepItem>& sched, std::vector<PreItem>& pre) {
    std::vector<int32_t> remaining(n_inner_), slot(n_inner_, -1), ready_at(n_inner_, 0), free_slots;
    for (int s = trash_slot - 1; s >= 0; --s) free_slots.push_back(s);
    std::vector<int32_t> ready;
    for (int n = g0; n < g1; ++n) { remaining[n] = (int)ic[n].size(); if (par[n] < 0) ready.push_back(n); }
    int done = 0, step_no = 0, ratio_live = 0;
    while (done < g1 - g0) {
      std::sort(ready.begin(), ready.end(), [&](int a, int b) {
        if (tree_of_inner_[a] != tree_of_inner_[b]) return tree_of_inner_[a] < tree_of_inner_[b];   // a forest: tree after tree
        if (ready_at[a] != ready_at[b]) return ready_at[a] < ready_at[b];
        return hin[a] != hin[b] ? hin[a] > hin[b] : a > b;
      });
      // a node whose flow tile needs a slot waits while none is free; only if nothing else
      // is ready does a tile go through HBM instead
      std::vector<int32_t> step, rest;
      int slots_left = (int)free_slots.size();
      for (int n : ready) {
        // a forest also counts the ratio tiles of the lean walk while it schedules (one per inner child, from the
        // parent's step to the end of the child's): a node only runs if its children's tiles fit, and a new tree
        // only starts while half the slots are free, so that the trees under way can finish
        const int need = (int)ic[n].size();
        const bool ratio_ok = T_ == 1 || ratio_live + need <= (par[n] < 0 ? trash_slot / 2 : trash_slot);
        if ((int)step.size() < kWalkWaves && (ic[n].empty() || slots_left > 0) && ratio_ok) {
          step.push_back(n);
          if (!ic[n].empty()) --slots_left;
          ratio_live += need;
        } else {
          rest.push_back(n);
        }
      }
      if (step.empty()) {
        if (rest.empty()) fail(PCM_ERR_SHAPE, "backward schedule stalled (tree is inconsistent)");
        step.push_back(rest.front());
        rest.erase(rest.begin());
      }
      ready.swap(rest);
      for (int w = 0; w < kWalkWaves; ++w) {
        if (w >= (int)step.size()) { sched.push_back(blank(-1)); pre.push_back(blank_pre(-1)); continue; }
        const int n = step[w];
        StepItem it = blank(n);
        PreItem q = blank_pre(n);
        std::vector<uint32_t> ops;
        ops.push_back(kOpLeaf | (uint32_t)var_of_inner_[n]);
        for (int c : ic[n]) ops.push_back((uint32_t)c);
        for (size_t i = 0; i < lc[n].size(); ++i) ops.push_back(leaf_child_op(lc[n][i], i));
        fill_ops(it, q, ops);
        if (par[n] >= 0) it.in_slot = slot[par[n]];   // -1: the parent's tile went to HBM
        if (!ic[n].empty()) {
          if (!free_slots.empty()) { slot[n] = free_slots.back(); free_slots.pop_back(); it.out_slot = slot[n]; }
          else { bwd_spill_ = true; it.flags |= kItemSpillOut; }
        }
        sched.push_back(it);
        pre.push_back(q);
      }
      ++step_no;
      for (int n : step) {
        if (par[n] >= 0) --ratio_live;
        if (par[n] >= 0 && --remaining[par[n]] == 0 && slot[par[n]] >= 0) free_slots.push_back(slot[par[n]]);
        for (int c : ic[n]) { ready.push_back(c); ready_at[c] = step_no; }
        ++done;
      }
    }
  };
  {
    bwd_spill_ = false;
    std::vector<std::vector<StepItem>> scheds(n_groups_);
    std::vector<std::vector<PreItem>> pres(n_groups_);
    n_bwd_steps_ = 0;
    for (int g = 0; g < n_groups_; ++g) {
      schedule_backward(groups[g].first, groups[g].second, scheds[g], pres[g]);
      n_bwd_steps_ = std::max(n_bwd_steps_, (int)scheds[g].size() / kWalkWaves);
    }
    std::vector<int32_t> ratio_slot(n_inner_, -1);
    bool slots_ok = true;
    for (int g = 0; g < n_groups_ && slots_ok; ++g) slots_ok = assign_ratio_slots(scheds[g], ratio_slot);
    std::vector<int32_t> lean_rows;
    bwd_lean_ = slots_ok;
    for (int g = 0; g < n_groups_; ++g) {
      pad_steps(scheds[g], pres[g], n_bwd_steps_);
      if (g == 0) make_fields(scheds[g], pres[g], false, bwd_stride_, d_bwd_fields_);
      else pad_steps(scheds[g], pres[g], bwd_stride_);
      bwd_lean_ = bwd_lean_ && make_lean(scheds[g], false, bwd_stride_, lean_rows, &ratio_slot);
    }
    if (bwd_lean_) d_bwd_lean_.upload(lean_rows);
    d_bwd_sched_.upload(scheds[0]);
  }
  // ---- a forest's finer plans --------------------------------------------------------------
  // The same walks with two and four times as many, smaller groups of trees, for batches whose slices times the
  // groups above leave most of the device idle (256 examples are 16 slices): the walk then takes the plan with
  // the most groups that still gives every workgroup a compute unit of its own.  A tree's arithmetic does not
  // depend on the group it is walked in, so the results are the same bits under every plan.
  fine_plans_.clear();
  if (forest_ && fwd_lean_ && bwd_lean_) {
    const bool keep_fwd_spill = fwd_spill_, keep_bwd_spill = bwd_spill_;
    for (int G = 2 * n_groups_; G <= 4 * n_groups_ && G <= T_ / 4; G *= 2) {
      const std::vector<std::pair<int, int>> gr = make_groups(G);
      if ((int)gr.size() <= (fine_plans_.empty() ? n_groups_ : fine_plans_.back()->n_groups)) break;
      std::unique_ptr<LeanPlan> plan(new LeanPlan);
      plan->n_groups = (int)gr.size();
      bool ok = true;
      std::vector<int32_t> rows;
      {
        fwd_spill_ = false;
        std::vector<std::vector<StepItem>> sched(gr.size());
        std::vector<std::vector<PreItem>> pre(gr.size());
        for (size_t g = 0; g < gr.size(); ++g) {
          schedule_forward(gr[g].first, gr[g].second, sched[g], pre[g]);
          plan->n_fwd_steps = std::max(plan->n_fwd_steps, (int)sched[g].size() / kWalkWaves);
        }
        ok = !fwd_spill_;
        plan->fwd_stride = plan->n_fwd_steps + 64;
        for (size_t g = 0; g < gr.size() && ok; ++g) {
          pad_steps(sched[g], pre[g], plan->fwd_stride);
          ok = make_lean(sched[g], true, plan->fwd_stride, rows);
        }
        if (ok) plan->fwd.upload(rows);
      }
      if (ok) {
        bwd_spill_ = false;
        std::vector<std::vector<StepItem>> sched(gr.size());
        std::vector<std::vector<PreItem>> pre(gr.size());
        for (size_t g = 0; g < gr.size(); ++g) {
          schedule_backward(gr[g].first, gr[g].second, sched[g], pre[g]);
          plan->n_bwd_steps = std::max(plan->n_bwd_steps, (int)sched[g].size() / kWalkWaves);
        }
        ok = !bwd_spill_;
        std::vector<int32_t> ratio_slot(n_inner_, -1);
        for (size_t g = 0; g < gr.size() && ok; ++g) ok = assign_ratio_slots(sched[g], ratio_slot);
        plan->bwd_stride = plan->n_bwd_steps + 64;
        rows.clear();
        for (size_t g = 0; g < gr.size() && ok; ++g) {
          pad_steps(sched[g], pre[g], plan->bwd_stride);
          ok = make_lean(sched[g], false, plan->bwd_stride, rows, &ratio_slot);
        }
        if (ok) plan->bwd.upload(rows);
      }
      if (!ok) break;
      fine_plans_.push_back(std::move(plan));
    }
    fwd_spill_ = keep_fwd_spill;
    bwd_spill_ = keep_bwd_spill;
  }
  // ---- statistics: the static operands of every node ------------------------------------
  {
    std::vector<StepItem> items;
    for (int n = 0; n < n_inner_; ++n) {
      StepItem it = blank(n);
      PreItem q = blank_pre(n);
      std::vector<uint32_t> ops;
      ops.push_back(kOpLeaf | (uint32_t)var_of_inner_[n]);
      for (int c : ic[n]) ops.push_back((uint32_t)c);
      for (size_t i = 0; i < lc[n].size(); ++i) ops.push_back(leaf_child_op(lc[n][i], i));
      fill_ops(it, q, ops);
      for (int i = 0; i < kPre; ++i) it.g[i] = q.g[i];   // absent operands name the zero tile
      items.push_back(it);
    }
    d_stat_items_.upload(items);
    // the same for the lean statistics kernel (nodes with at most three children)
    stat_lean_ = K_ <= 32;
    std::vector<StatNode> sn(n_inner_);
    for (int n = 0; n < n_inner_ && stat_lean_; ++n) {
      StatNode& q = sn[n];
      std::memset(&q, 0, sizeof q);
      if (ic[n].size() + lc[n].size() > 3) { stat_lean_ = false; break; }
      q.var = var_of_inner_[n];
      q.node = n;
      q.c[0] = q.c[1] = q.c[2] = -1;
      int k = 0;
      for (int c : ic[n]) q.c[k++] = c << 3;
      q.n_hist = 1;
      q.hvar[0] = q.var;
      for (size_t i = 0; i < lc[n].size(); ++i) {
        q.c[k++] = (lc[n][i] << 3) | 1 | (int32_t)((i + 1) << 1);
        q.hvar[q.n_hist++] = lc[n][i];
      }
    }
    {   // its LDS: two histograms if they fit, else one (or the parked edge-flow blocks, if larger) | per-wave pads
      const size_t hist = 2 * (size_t)C_ * K_, park = (size_t)kStatLeanWaves * K_ * K_, pads = (size_t)kStatLeanWaves * kSlice * K_;
      stat_lean_hists_ = (std::max(2 * hist, park) + pads) * 4 <= (size_t)max_lds_ ? 2 : 1;
      if ((std::max(hist, park) + pads) * 4 > (size_t)max_lds_) stat_lean_ = false;
    }
    if (stat_lean_) {
      // The workgroups draw the records in this order, and the kernel ends when the last drawn node is done: the
      // costliest nodes (passes over the batch, then histograms, then operands) go first, so that what is left for
      // the end are the short ones.
      const int nh_pass = stat_lean_hists_;
      auto cost = [&](const StatNode& q) {
        const int children = (q.c[0] >= 0) + (q.c[1] >= 0) + (q.c[2] >= 0);
        return ((q.n_hist + nh_pass - 1) / nh_pass) * 100 + std::min(q.n_hist, nh_pass) * 10 + children;
      };
      std::stable_sort(sn.begin(), sn.end(), [&](const StatNode& a, const StatNode& b) { return cost(a) > cost(b); });
      d_stat_lean_.upload(sn);
      d_stat_claim_.upload(std::vector<uint32_t>(1, 0u));
    }
  }
  lean_ = fwd_lean_ && bwd_lean_ && stat_lean_;
  if (ext.empty()) ext.push_back(0);
  d_ext_ops_.upload(ext);
  if (getenv("PCM_VERBOSE"))
    fprintf(stderr, "[pcmi355] hclt V=%d K=%d C=%d inner=%d trees=%d groups=%d: forward %d steps%s%s, backward %d steps%s%s, statistics%s, "
            "%d LDS slots\n",
            V_, K_, C_, n_inner_, T_, n_groups_, n_fwd_steps_, fwd_spill_ ? " (spills)" : "", fwd_lean_ ? " (lean)" : "", n_bwd_steps_,
            bwd_spill_ ? " (spills)" : "", bwd_lean_ ? " (lean)" : "", stat_lean_ ? " (lean)" : "", lds_slots_);
  if (getenv("PCM_VERBOSE"))
    for (const auto& p : fine_plans_)
      fprintf(stderr, "[pcmi355]   finer plan: %d groups, forward %d steps, backward %d steps\n", p->n_groups, p->n_fwd_steps,
              p->n_bwd_steps);
}

// Numbering the reference would give this circuit.  Nodes are created in depth-first
// post-order from the root sum node (children in order, prime before sub); the sum node
// (v, k) is reached from its tree parent's edge j = k, so the first visit of tree node v is
// through (v, 0), which creates, for j = 0..K-1: [children circuits at state j], [the
// K-ary product if v has several children], input leaf_v[j]; then sum (v, 0); later visits
// create only (v, k).  Up edges are ordered by layer, then by parent id
// (reference: test/bits_circuit_tests.jl:13-24, test/misc_tests.jl:39-62 for the pinned
// part; src/bits_circuit.jl:46-70 for the tables).
void HcltCircuit::build_param_order() {
  const int K = K_;
  // the caller's tree: auxiliary nodes (split_wide_nodes) are no part of the circuit the reference would number
  const std::vector<std::vector<int32_t>>& children_ = V_ > Vu_ ? uchildren_ : this->children_;
  const int V_ = Vu_;
  std::vector<int64_t> sum_id((size_t)V_ * K, -1), mul_id((size_t)V_ * K, -1), in_id((size_t)V_ * K, -1);
  std::vector<int64_t> rprod_id(K, -1);
  int64_t next = 0;
  input_order_.clear();
  // explicit stack machine for visit(v, k)
  struct Frame { int v, k, j, c; };
  std::vector<Frame> st;
  auto create_input = [&](int v, int j) {
    if (in_id[(size_t)v * K + j] < 0) {
      in_id[(size_t)v * K + j] = next++;
      input_order_.push_back(v * K + j);
    }
  };
  st.push_back({root_, 0, 0, 0});
  std::vector<char> expanded(V_, 0);
  while (!st.empty()) {
    Frame& f = st.back();
    const int v = f.v;
    if (sum_id[(size_t)v * K + f.k] >= 0) { st.pop_back(); continue; }
    if (expanded[v] == 2) {   // subtree already created: only this sum node is new
      sum_id[(size_t)v * K + f.k] = next++;
      st.pop_back();
      continue;
    }
    expanded[v] = 1;
    if (f.j < K) {
      if (f.c < (int)children_[v].size()) {
        int c = children_[v][f.c++];
        if (children_[c].empty()) create_input(c, f.j);
        else if (sum_id[(size_t)c * K + f.j] < 0) st.push_back({c, f.j, 0, 0});
        continue;
      }
      // a product of exactly two circuits stays an unnumbered (prime, sub) pair until the
      // product above it (with leaf_v[j]) needs it as a node, i.e. after the leaf
      if (children_[v].size() > 2) mul_id[(size_t)v * K + f.j] = next++;
      create_input(v, f.j);
      if (children_[v].size() == 2) mul_id[(size_t)v * K + f.j] = next++;
      // multi-head: the root's product (children x leaf) is shared by all heads, so it is a node of its own
      if (H_ > 0 && v == root_) rprod_id[f.j] = next++;
      f.j++;
      f.c = 0;
      continue;
    }
    expanded[v] = 2;
    sum_id[(size_t)v * K + f.k] = next++;
    st.pop_back();
  }
  n_nodes_ = next + (H_ > 0 ? H_ - 1 : 0);   // multi-head: the root's sum node is head 0, the other heads follow it
  const int64_t head0 = next - 1;

  // layers
  std::vector<int> vlayer(V_, 0);   // layer of the sum nodes of v (0 for leaves = inputs)
  std::vector<int> mlayer(V_, 0);
  for (int n = 0; n < n_inner_; ++n) {
    int v = var_of_inner_[n];
    if (v >= Vu_) continue;
    int lc = 0;
    for (int c : children_[v]) lc = std::max(lc, vlayer[c]);
    if (children_[v].size() > 1) { mlayer[v] = lc + 1; lc = lc + 1; }
    vlayer[v] = lc + 1;
  }
  // edge records (parent id, layer) -> sorted
  struct Rec { int layer; int64_t parent; int kind; int v, k; };   // kind 0 mul, 1 sum
  std::vector<Rec> recs;
  for (int n = 0; n < n_inner_; ++n) {
    int v = var_of_inner_[n];
    if (v >= Vu_) continue;
    if (children_[v].size() > 1)
      for (int j = 0; j < K; ++j) recs.push_back({mlayer[v], mul_id[(size_t)v * K + j], 0, v, j});
    int nk = v == root_ ? (H_ > 0 ? 0 : 1) : K;
    for (int k = 0; k < nk; ++k) recs.push_back({vlayer[v], sum_id[(size_t)v * K + k], 1, v, k});
  }
  if (H_ > 0) {
    for (int j = 0; j < K; ++j) recs.push_back({vlayer[root_], rprod_id[j], 3, root_, j});   // kind 3: a root product
    for (int h = 0; h < H_; ++h) recs.push_back({vlayer[root_] + 1, head0 + h, 2, root_, h});   // kind 2: a head
  }
  std::sort(recs.begin(), recs.end(), [](const Rec& a, const Rec& b) {
    return a.layer != b.layer ? a.layer < b.layer : a.parent < b.parent;
  });
  sum_param_src_.clear();
  sum_group_size_.clear();
  edge2param_.clear(); edge_parent_.clear(); edge_prime_.clear(); edge_sub_.clear(); layer_ends_.clear();
  auto circ_id = [&](int c, int j) -> int64_t {
    return children_[c].empty() ? in_id[(size_t)c * K + j] : sum_id[(size_t)c * K + j];
  };
  int cur_layer = recs.empty() ? 0 : recs[0].layer;
  for (const Rec& r : recs) {
    if (r.layer != cur_layer) { layer_ends_.push_back((int64_t)edge_parent_.size()); cur_layer = r.layer; }
    const auto& ch = children_[r.v];
    if (r.kind == 0) {
      for (size_t q = 0; q < ch.size(); q += 2) {
        edge_parent_.push_back(r.parent + 1);
        edge_prime_.push_back(circ_id(ch[q], r.k) + 1);
        edge_sub_.push_back(q + 1 < ch.size() ? circ_id(ch[q + 1], r.k) + 1 : 0);
        edge2param_.push_back(0);
      }
    } else if (r.kind == 3) {   // root product of a multi-head circuit: (children's circuit, leaf) at state r.k
      edge_parent_.push_back(r.parent + 1);
      edge_prime_.push_back((ch.size() > 1 ? mul_id[(size_t)r.v * K + r.k] : circ_id(ch[0], r.k)) + 1);
      edge_sub_.push_back(in_id[(size_t)r.v * K + r.k] + 1);
      edge2param_.push_back(0);
    } else if (r.kind == 2) {   // head r.k over the K root products
      for (int j = 0; j < K; ++j) {
        edge_parent_.push_back(r.parent + 1);
        edge_prime_.push_back(rprod_id[j] + 1);
        edge_sub_.push_back(0);
        sum_param_src_.push_back(((int64_t)n_inner_ * K + r.k) * K + j);   // head rows sit behind the blocks
        edge2param_.push_back((int64_t)sum_param_src_.size());
      }
      sum_group_size_.push_back(K);
    } else {
      const int n = inner_of_var_[r.v];
      for (int j = 0; j < K; ++j) {
        edge_parent_.push_back(r.parent + 1);
        int64_t prime = ch.size() > 1 ? mul_id[(size_t)r.v * K + j] : circ_id(ch[0], j);
        edge_prime_.push_back(prime + 1);
        edge_sub_.push_back(in_id[(size_t)r.v * K + j] + 1);
        sum_param_src_.push_back(((int64_t)n * K + r.k) * K + j);
        edge2param_.push_back((int64_t)sum_param_src_.size());
      }
      sum_group_size_.push_back(K);
    }
  }
  layer_ends_.push_back((int64_t)edge_parent_.size());
  n_edges_ = (int64_t)edge_parent_.size();
  d_sum_param_src_.upload(sum_param_src_);
  {
    std::vector<int32_t> pos((size_t)V_ * K_, 0);
    for (size_t q = 0; q < input_order_.size(); ++q) pos[(size_t)input_order_[q]] = (int32_t)q;
    d_in_pos_.upload(pos);
  }

  // the same circuit in general form, for the queries that run on the general engine
  flat_ = FlatCircuit();
  flat_.num_vars = V_; flat_.num_cats = C_; flat_.num_heads = H_;
  flat_.type.assign(n_nodes_, kInput);
  flat_.layer.assign(n_nodes_, 0);
  flat_.in_var.assign(n_nodes_, -1);
  flat_.in_off.assign(n_nodes_, -1);
  flat_.input_nodes.resize(input_order_.size());
  for (size_t q = 0; q < input_order_.size(); ++q) {
    const int v = input_order_[q] / K, j = input_order_[q] % K;
    const int64_t id = in_id[(size_t)v * K + j];
    flat_.input_nodes[q] = (int32_t)id;
    flat_.in_var[id] = v;
    flat_.in_off[id] = (int64_t)q * C_;
  }
  for (int n = 0; n < n_inner_; ++n) {
    const int v = var_of_inner_[n];
    if (v >= Vu_) continue;
    for (int k = 0; k < K; ++k) {
      if (mul_id[(size_t)v * K + k] >= 0) { flat_.type[mul_id[(size_t)v * K + k]] = kMul; flat_.layer[mul_id[(size_t)v * K + k]] = mlayer[v]; }
      if (sum_id[(size_t)v * K + k] >= 0) { flat_.type[sum_id[(size_t)v * K + k]] = kSum; flat_.layer[sum_id[(size_t)v * K + k]] = vlayer[v]; }
    }
  }
  for (int h = 0; h < H_; ++h) {
    flat_.type[head0 + h] = kSum;
    flat_.layer[head0 + h] = vlayer[root_] + 1;
    flat_.heads.push_back((int32_t)(head0 + h));
  }
  if (H_ > 0)
    for (int j = 0; j < K; ++j) { flat_.type[rprod_id[j]] = kMul; flat_.layer[rprod_id[j]] = vlayer[root_]; }
  flat_.leaf_logp.assign((size_t)V_ * K * C_, 0.f);
  noise_slot_.assign(n_edges_, 0);
  for (int64_t ed = 0; ed < n_edges_; ++ed) {
    flat_.e_parent.push_back((int32_t)(edge_parent_[ed] - 1));
    flat_.e_prime.push_back((int32_t)(edge_prime_[ed] - 1));
    flat_.e_sub.push_back((int32_t)(edge_sub_[ed] - 1));
    flat_.e_logp.push_back(0.f);
    if (edge2param_[ed]) {
      const int64_t src = sum_param_src_[edge2param_[ed] - 1];
      if (src < (int64_t)n_inner_ * K * K) noise_slot_[ed] = (int32_t)(user_index_[src / ((int64_t)K * K)] * K + src % K);
    }
  }
  flat_.finish();
}

int64_t HcltCircuit::size(int what) const {
  switch (what) {
    case 0: return (int64_t)sum_param_src_.size() + (int64_t)Vu_ * K_ * C_;
    case 1: return (int64_t)sum_param_src_.size();
    case 2: return n_nodes_;
    case 3: return n_edges_;
    case 4: return (int64_t)Vu_ * K_ * C_;
    case 5: return Vu_;
    case 6: return C_;
    case 7: return K_;
    case 8: return n_user_inner_;
    case 9: return (int64_t)layer_ends_.size();
    case 10: return (int64_t)sum_group_size_.size();
    case 11: return (int64_t)Vu_ * K_;
    case 12: return H_;
    case 13: return 0;
    case 14: return wide_walk_ ? 3 : !block_ ? 0 : lean_ ? 1 : 2;
    case 15: return T_;
    case 16: return 0;
    case 17: return 0;
    case 18: return 0;
    default: fail(PCM_ERR_ARG, "unknown size selector %d", what);
  }
}

void HcltCircuit::index_table(int which, int64_t* out, int64_t n) const {
  no_forest("an index table");
  auto copy = [&](const std::vector<int64_t>& v) {
    if ((int64_t)v.size() != n) fail(PCM_ERR_ARG, "index table %d has %lld entries, caller gave %lld",
                                     which, (long long)v.size(), (long long)n);
    std::copy(v.begin(), v.end(), out);
  };
  switch (which) {
    case 0: copy(edge2param_); break;
    case 1: {
      std::vector<int64_t> p2e;
      for (size_t e = 0; e < edge2param_.size(); ++e) if (edge2param_[e]) p2e.push_back((int64_t)e + 1);
      copy(p2e); break;
    }
    case 2: {
      std::vector<int64_t> p2g;
      for (size_t gi = 0; gi < sum_group_size_.size(); ++gi)
        for (int i = 0; i < sum_group_size_[gi]; ++i) p2g.push_back((int64_t)gi + 1);
      copy(p2g); break;
    }
    case 3: copy(std::vector<int64_t>(sum_group_size_.begin(), sum_group_size_.end())); break;
    case 4: {
      std::vector<int64_t> cum((size_t)Vu_ * K_);
      for (size_t i = 0; i < cum.size(); ++i) cum[i] = (int64_t)(i + 1) * C_;
      copy(cum); break;
    }
    case 5: copy(layer_ends_); break;
    case 6: copy(edge_parent_); break;
    case 7: copy(edge_prime_); break;
    case 8: copy(edge_sub_); break;
    case 9: {
      std::vector<int64_t> hd;
      for (int h = 0; h < H_; ++h) hd.push_back(n_nodes_ - H_ + h + 1);
      copy(hd); break;
    }
    default: fail(PCM_ERR_ARG, "unknown index table %d", which);
  }
}

// ---- parameters -------------------------------------------------------------------

void HcltCircuit::rebuild_w() {
  if (!block_ && !wide_) return;
  const int64_t tot = (int64_t)n_inner_ * K_ * K_;
  PCM_DISPATCH_PARAM_K(K_, hipLaunchKernelGGL(hclt_rebuild_w_kernel<KK>, dim3(ceil_div(tot, 256)), dim3(256), 0,
                                        stream, d_logtheta_.p, d_Wf_.p, d_Wb_.p, n_inner_));
  check_launch("rebuild_w");
  rebuild_heads();
}

void HcltCircuit::rebuild_heads() {
  if (H_ == 0) return;
  hipLaunchKernelGGL(hclt_heads_rebuild_kernel, dim3(ceil_div((int64_t)Hp_ * K_, 256), T_), dim3(256), 0, stream, head_logp(),
                     H_, Hp_, K_, d_head_wf_.p, d_head_wb_.p);
  check_launch("rebuild_heads");
}

// head values from the root tile the forward walk has left (identity block: the root's Z)
void HcltCircuit::heads_forward(const HcltDev& d, const float* d_mask, float* d_ll_heads, float* d_ll_mix, bool flows_follow,
                                float rate) {
  PCM_DISPATCH_LEAN_K(K_, hipLaunchKernelGGL(hclt_heads_forward_kernel<KK>, dim3(d.nslices, T_), dim3(kHeadWaves * 64), 0,
                                             stream, d.O, d.M, d.Bp, d_root_node_.p, (int64_t)(d.tile_stride / 4), d_head_wf_.p,
                                             H_, Hp_, d.B, d_mask, d_ll_heads, d_ll_mix,
                                             flows_follow ? head_aggr() : (float*)nullptr, rate, d_flow_shift_.p));
  check_launch("heads_forward");
}

void HcltCircuit::set_block_params(const float* theta, const float* leaf) {
  const int K = K_, C = C_;
  if (theta) {
    std::vector<float> lt((size_t)n_inner_ * K * K);
    for (int n = 0; n < n_inner_; ++n) {
      float* dst = lt.data() + (size_t)n * K * K;
      if (var_of_inner_[n] >= Vu_) {   // auxiliary node: identity
        for (int i = 0; i < K * K; ++i) dst[i] = (i / K == i % K) ? 0.f : -INFINITY;
        continue;
      }
      const float* src = theta + (size_t)var_of_inner_[n] * K * K;
      std::copy(src, src + (size_t)K * K, dst);
      if (parent_[var_of_inner_[n]] < 0) {
        if (H_ > 0) {   // multi-head: identity block, the heads have their own rows
          for (int i = 0; i < K * K; ++i) dst[i] = (i / K == i % K) ? 0.f : -INFINITY;
        } else {
          for (int i = K; i < K * K; ++i) dst[i] = -INFINITY;   // the root keeps one sum node
        }
      }
    }
    PCM_HIP(hipMemcpyAsync(d_logtheta_.p, lt.data(), lt.size() * sizeof(float), hipMemcpyHostToDevice, stream));
    PCM_HIP(hipStreamSynchronize(stream));
    rebuild_w();
  }
  general_stale_ = true;
  if (leaf) {
    std::vector<float> t((size_t)V_ * C * K, 0.f);   // (auxiliary variables: log 1 whatever the category)
    for (int v = 0; v < Vu_; ++v)
      for (int j = 0; j < K; ++j)
        for (int c = 0; c < C; ++c) t[((size_t)v * C + c) * K + j] = leaf[((size_t)v * K + j) * C + c];
    PCM_HIP(hipMemcpyAsync(d_leaf_.p, t.data(), t.size() * sizeof(float), hipMemcpyHostToDevice, stream));
    PCM_HIP(hipStreamSynchronize(stream));
    leaf_changed();
  }
}

// The marker of a missing value is a table row like the categories', with log-probability 0 for every hidden state:
// a missing observation then multiplies every leaf by 1 (src/regularization/reg_likelihood.jl:40-47), its flow
// collects in the marker's row of the leaf statistics, and no walk or statistics kernel knows about it.
void HcltCircuit::pin_missing_marker() {
  if (!missing_) return;
  PCM_HIP(hipMemset2DAsync(d_leaf_.p + (size_t)(C_ - 1) * K_, (size_t)C_ * K_ * sizeof(float), 0, (size_t)K_ * sizeof(float),
                           (size_t)V_, stream));
  general_stale_ = true;
}

void HcltCircuit::set_missing_category(bool on) {
  if (on && !(block_ || wide_))
    fail(PCM_ERR_UNSUPPORTED, "a missing-value category needs the block kernels (K = 16, 32, 64 or 128)");
  if (on && C_ < 2) fail(PCM_ERR_SHAPE, "a circuit with a missing-value category needs at least one real category");
  if (on && soft_reg_ > 0.f) fail(PCM_ERR_UNSUPPORTED, "soft_reg smoothing and a missing-value category together");
  missing_ = on;
  pin_missing_marker();
}

void HcltCircuit::leaf_changed() {
  pin_missing_marker();
  if (soft_reg_ > 0.f) {
    const int64_t total = (int64_t)V_ * C_ * K_;
    hipLaunchKernelGGL(hclt_leaf_smooth_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, stream, d_leaf_.p,
                       d_leaf_smooth_.p, total, C_, K_, soft_reg_, soft_width_);
    check_launch("leaf_smooth");
  }
}

void HcltCircuit::set_soft_reg(float soft_reg, int width, bool as_written) {
  if (!(soft_reg >= 0.f && soft_reg < 1.f)) fail(PCM_ERR_ARG, "soft_reg must lie in [0, 1), got %g", (double)soft_reg);
  if (width < 1) fail(PCM_ERR_ARG, "soft_reg_width must be at least 1, got %d", width);
  if (soft_reg > 0.f) {
    if (!(block_ || wide_)) fail(PCM_ERR_UNSUPPORTED, "soft_reg smoothing in the kernels needs the block kernels (K = 16, 32, 64 or 128)");
    if (missing_) fail(PCM_ERR_UNSUPPORTED, "soft_reg smoothing and a missing-value category together");
    if (flows_in_general_) fail(PCM_ERR_STATE, "the flows of this circuit are held by the layered engine");
    d_leaf_smooth_.ensure((size_t)V_ * C_ * K_);
    d_leaf_hist_.ensure((size_t)V_ * C_ * K_);
  }
  soft_reg_ = soft_reg;
  soft_width_ = width;
  soft_written_ = as_written;
  leaf_changed();
}

// the statistics kernels have left the histogram by shown category in d_leaf_hist_
void HcltCircuit::soft_reg_counts(float rate) {
  if (!(soft_reg_ > 0.f)) return;
  const int64_t total = (int64_t)V_ * C_ * K_;
  hipLaunchKernelGGL(hclt_soft_counts_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, stream, d_leaf_.p,
                     d_leaf_smooth_.p, d_leaf_hist_.p, d_leaf_flow_.p, total, C_, K_, soft_reg_, soft_width_, rate,
                     soft_written_ ? 1 : 0);
  check_launch("soft_counts");
}

void HcltCircuit::set_heads(const float* heads) {
  if (H_ == 0) fail(PCM_ERR_STATE, "a single-head circuit has no head parameters");
  if (!heads) fail(PCM_ERR_ARG, "head parameters are null");
  PCM_HIP(hipMemcpyAsync(head_logp(), heads, (size_t)T_ * H_ * K_ * sizeof(float), hipMemcpyHostToDevice, stream));
  PCM_HIP(hipStreamSynchronize(stream));
  rebuild_heads();
  general_stale_ = true;
}

void HcltCircuit::get_heads(float* heads) {
  if (H_ == 0) fail(PCM_ERR_STATE, "a single-head circuit has no head parameters");
  if (!heads) fail(PCM_ERR_ARG, "head parameters are null");
  PCM_HIP(hipMemcpyAsync(heads, head_logp(), (size_t)T_ * H_ * K_ * sizeof(float), hipMemcpyDeviceToHost, stream));
  sync_checked();
}

static void fetch(std::vector<float>& h, const float* d, size_t n, hipStream_t s) {
  h.resize(n);
  PCM_HIP(hipMemcpyAsync(h.data(), d, n * sizeof(float), hipMemcpyDeviceToHost, s));
  PCM_HIP(hipStreamSynchronize(s));
}

void HcltCircuit::get_block_params(float* theta, float* leaf) {
  sync_checked();   // (a void pass is reported before anything that came after it is handed out)
  const int K = K_, C = C_;
  std::vector<float> h;
  if (theta) {
    fetch(h, d_logtheta_.p, d_logtheta_.n, stream);
    std::fill(theta, theta + (size_t)Vu_ * K * K, 0.f);
    for (int n = 0; n < n_inner_; ++n)
      if (var_of_inner_[n] < Vu_)
        std::copy(h.begin() + (size_t)n * K * K, h.begin() + (size_t)(n + 1) * K * K,
                  theta + (size_t)var_of_inner_[n] * K * K);
  }
  if (leaf) {
    fetch(h, d_leaf_.p, d_leaf_.n, stream);
    for (int v = 0; v < Vu_; ++v)
      for (int j = 0; j < K; ++j)
        for (int c = 0; c < C; ++c) leaf[((size_t)v * K + j) * C + c] = h[((size_t)v * C + c) * K + j];
  }
}

void HcltCircuit::get_block_flows(float* edge_aggr, float* leaf_flow) {
  sync_checked();
  if (!have_flows_) fail(PCM_ERR_STATE, "no flows have been computed on this circuit yet");
  const int K = K_, C = C_;
  std::vector<float> h;
  if (flows_in_general_ || (!block_ && !wide_)) {   // from the layered engine's accumulators: up-edge / input-node order -> blocks
    std::vector<float> ea((size_t)n_edges_), lf((size_t)Vu_ * K * C);
    general_->get_aggregates(ea.data(), n_edges_, lf.data(), (int64_t)lf.size());
    if (edge_aggr) {
      std::fill(edge_aggr, edge_aggr + (size_t)Vu_ * K * K, 0.f);
      for (int64_t e = 0; e < n_edges_; ++e)
        if (edge2param_[e]) {
          const int64_t src = sum_param_src_[edge2param_[e] - 1];
          edge_aggr[(size_t)var_of_inner_[src / ((int64_t)K * K)] * K * K + src % ((int64_t)K * K)] = ea[e];
        }
    }
    if (leaf_flow)
      for (size_t q = 0; q < input_order_.size(); ++q)
        std::copy(lf.begin() + q * C, lf.begin() + (q + 1) * C, leaf_flow + (size_t)input_order_[q] * C);
    return;
  }
  if (edge_aggr) {
    fetch(h, d_edge_aggr_.p, d_edge_aggr_.n, stream);
    std::fill(edge_aggr, edge_aggr + (size_t)Vu_ * K * K, 0.f);
    for (int n = 0; n < n_inner_; ++n)
      if (var_of_inner_[n] < Vu_)
        std::copy(h.begin() + (size_t)n * K * K, h.begin() + (size_t)(n + 1) * K * K,
                  edge_aggr + (size_t)var_of_inner_[n] * K * K);
  }
  if (leaf_flow) {
    fetch(h, d_leaf_flow_.p, d_leaf_flow_.n, stream);
    for (int v = 0; v < Vu_; ++v)
      for (int j = 0; j < K; ++j)
        for (int c = 0; c < C; ++c) leaf_flow[((size_t)v * K + j) * C + c] = h[((size_t)v * C + c) * K + j];
  }
}

void HcltCircuit::vectorize(float* out, int64_t n) {
  no_forest("the parameter vector");
  sync_checked();
  if (n != size(0)) fail(PCM_ERR_ARG, "parameter vector has %lld entries, circuit has %lld", (long long)n,
                         (long long)size(0));
  if (!out) fail(PCM_ERR_ARG, "parameter vector is null");
  const int64_t ns = (int64_t)sum_param_src_.size();
  d_param_vec_.ensure((size_t)n);
  if (ns > 0)
    hipLaunchKernelGGL(hclt_params_gather_kernel, dim3((unsigned)ceil_div(ns, 256)), dim3(256), 0, stream, ns,
                       d_sum_param_src_.p, d_logtheta_.p, d_param_vec_.p);
  hipLaunchKernelGGL(hclt_leaf_vector_kernel<true>, dim3(Vu_, ceil_div(C_, kLeafVecCats)), dim3(256),
                     (size_t)kLeafVecCats * (K_ + 1) * sizeof(float), stream, d_leaf_.p, d_in_pos_.p, K_, C_,
                     d_param_vec_.p + ns);
  check_launch("vectorize");
  PCM_HIP(hipMemcpyAsync(out, d_param_vec_.p, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, stream));
  PCM_HIP(hipStreamSynchronize(stream));
}

void HcltCircuit::update_parameters(const float* in, int64_t n) {
  no_forest("the parameter vector");
  if (n != size(0)) fail(PCM_ERR_ARG, "parameter vector has %lld entries, circuit has %lld", (long long)n,
                         (long long)size(0));
  if (!in) fail(PCM_ERR_ARG, "parameter vector is null");
  const int64_t ns = (int64_t)sum_param_src_.size();
  d_param_vec_.ensure((size_t)n);
  PCM_HIP(hipMemcpyAsync(d_param_vec_.p, in, (size_t)n * sizeof(float), hipMemcpyHostToDevice, stream));
  if (ns > 0)
    hipLaunchKernelGGL(hclt_params_scatter_kernel, dim3((unsigned)ceil_div(ns, 256)), dim3(256), 0, stream, ns,
                       d_sum_param_src_.p, d_param_vec_.p, d_logtheta_.p);
  hipLaunchKernelGGL(hclt_leaf_vector_kernel<false>, dim3(Vu_, ceil_div(C_, kLeafVecCats)), dim3(256),
                     (size_t)kLeafVecCats * (K_ + 1) * sizeof(float), stream, d_leaf_.p, d_in_pos_.p, K_, C_,
                     d_param_vec_.p + ns);
  check_launch("update_parameters");
  PCM_HIP(hipStreamSynchronize(stream));   // the caller's vector is free again
  rebuild_w();
  general_stale_ = true;
  leaf_changed();
}

// ---- batches ------------------------------------------------------------------------

void HcltCircuit::ensure_batch(int batch) {
  const int ns = ceil_div(batch, kSlice);
  if (ns <= cap_slices_) return;
  const size_t tile = tile_floats(ns);
  if (wide_) {
    d_O_.alloc((size_t)n_inner_ * tile);
    d_G_.alloc((size_t)n_inner_ * tile);
    d_wide_rs_.alloc((size_t)n_inner_ * tile);
    d_wide_es_.alloc((size_t)n_inner_ * tile);
    d_M_.alloc((size_t)(n_inner_ + 1) * ns * kSlice);
    d_xb_.alloc((size_t)V_ * ns * kSlice);
    d_xn_.alloc((size_t)(n_inner_ + 1) * ns * kSlice);
    d_xn_.zero(stream);
    cap_slices_ = ns;
    return;
  }
  d_O_.alloc((size_t)(n_inner_ + 1) * tile);   // row n_inner: trash tile of idle waves
  d_R_.alloc((size_t)(n_inner_ + 1) * tile);
  if (bwd_spill_ || wide_walk_) d_G_.alloc((size_t)n_inner_ * tile);
  if (wide_walk_) {
    d_wide_rs_.alloc((size_t)n_inner_ * tile);
    d_wide_es_.alloc((size_t)n_inner_ * tile);
  }
  d_M_.alloc((size_t)(n_inner_ + 1) * ns * kSlice);   // row maxima of the forward walk
  d_xb_.alloc((size_t)V_ * ns * kSlice);
  if (V_ > Vu_) d_xb_.zero(stream);   // the category of an auxiliary variable is always 0
  d_xn_.alloc((size_t)(n_inner_ + 1) * ns * kSlice);
  d_xn_.zero(stream);
  cap_slices_ = ns;
}

HcltDev HcltCircuit::dev(int batch) const {
  HcltDev d;
  d.nodes = d_nodes_.p;
  d.child_inner = d_child_inner_.p;
  d.child_leaf = d_child_leaf_.p;
  d.leaf = soft_reg_ > 0.f ? d_leaf_smooth_.p : d_leaf_.p;   // (the smoothed table: categorical batches under soft_reg)
  d.logtheta = d_logtheta_.p;
  d.Wf = d_Wf_.p;
  d.Wb = d_Wb_.p;
  d.xb = d_xb_.p;
  d.xn = d_xn_.p;
  d.O = d_O_.p;
  d.R = d_R_.p;
  d.G = d_G_.p;
  d.M = d_M_.p;
  d.err = walk_err_;
  d.err_dev = d_walk_void_.p;
  d.w = nullptr;
  d.ext_ops = d_ext_ops_.p;
  d.B = batch;
  d.nslices = ceil_div(batch, kSlice);
  d.Bp = d.nslices * kSlice;
  d.C = C_;
  d.n_inner = n_inner_;
  d.V = V_;
  d.leaf_stride = (uint32_t)C_ * K_ * 4;
  d.leaf_slice = 0;
  d.tile_stride = (uint32_t)(tile_floats(d.nslices) * 4);
  return d;
}

// A walk workgroup (16 examples) fills a compute unit, and the walks run fastest with exactly one workgroup per
// unit: with 8192 examples on 256 units a step took 4.60 ms, as two halves 3.47 (the second round's workgroups no
// longer share parameter blocks and leaf tables in time with the first's).  So a larger batch of a single-head
// circuit on the walk kernels goes through in chunks of that size -- which also keeps the tile arrays at one chunk's
// size whatever the batch.  Returns the chunk size, or 0 for a batch that goes through as it is.
int HcltCircuit::walk_chunk(int batch) const {
  const int chunk = n_cus_ * kSlice;
  return (H_ == 0 && block_ && !wide_walk_ && batch > chunk) ? chunk : 0;
}

BatchRef HcltCircuit::chunk_of(const BatchRef& b, int off, int chunk) {
  BatchRef part = b;
  part.batch = std::min(chunk, b.batch - off);
  if (b.d_idx) part.d_idx = b.d_idx + off;
  else part.d_data = b.d_data + (int64_t)off * b.stride_ex;
  return part;
}

void HcltCircuit::stage_batch(const BatchRef& b) {
  check_walks();
  if (!b.d_data) fail(PCM_ERR_ARG, "data pointer is null");
  if (b.batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", b.batch);
  ensure_batch(b.batch);
  const int Bp = ceil_div(b.batch, kSlice) * kSlice;
  pcm_stage(b.d_data, b.stride_ex, b.stride_var, b.d_idx, b.batch, Bp, Vu_, C_, d_xb_.p, stream);   // (auxiliary rows stay 0)
  check_launch("stage_batch");
  hipLaunchKernelGGL(hclt_pack_x_kernel, dim3(ceil_div(Bp, 1024), n_inner_), dim3(256), 0, stream, d_nodes_.p,
                     d_child_leaf_.p, d_xb_.p, n_inner_, Bp, d_xn_.p);
  check_launch("pack_x");
}

// The finer plan a batch of `nslices` slices walks a forest with, or null for the plan of the constructor: the
// most groups whose workgroups still get a compute unit each.
const HcltCircuit::LeanPlan* HcltCircuit::fine_plan(int nslices) const {
  const LeanPlan* best = nullptr;
  for (const auto& p : fine_plans_)
    if ((int64_t)nslices * p->n_groups <= n_cus_) best = p.get();
  return best;
}

void HcltCircuit::run_forward(const HcltDev& d, float* d_ll) {
  const size_t lds = (size_t)lds_slots_ * kSlice * K_ * sizeof(float);
  auto launch = [&](auto kernel) {
    PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    PCM_LAUNCH_PHASE(0, kernel, dim3(d.nslices), dim3(kWalkWaves * 64), lds, d, d_fwd_fields_.p, fwd_stride_,
                     d_fwd_sched_.p, n_fwd_steps_, d_ll);
  };
  // the lean kernels address every array with 32-bit offsets from one descriptor
  const bool small = (size_t)(n_inner_ + 1) * d.tile_stride < ((size_t)1 << 31);
  if (lean_ && small && !force_general_walks_) {
    const size_t lean_lds = lds + kLeanFlagWords * 4;   // the slots' state words sit behind the slots
    PCM_DISPATCH_LEAN_K(K_, {
      PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hclt_forward_lean_kernel<KK>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lean_lds));
      const LeanPlan* fp = fine_plan(d.nslices);
      if (fp)
        PCM_LAUNCH_PHASE(0, hclt_forward_lean_kernel<KK>, dim3(d.nslices, fp->n_groups), dim3(kWalkWaves * 64), lean_lds, d,
                         fp->fwd.p, fp->fwd_stride, fp->n_fwd_steps, d_ll, lds_slots_);
      else
        PCM_LAUNCH_PHASE(0, hclt_forward_lean_kernel<KK>, dim3(d.nslices, n_groups_), dim3(kWalkWaves * 64), lean_lds, d,
                         d_fwd_lean_.p, fwd_stride_, n_fwd_steps_, d_ll, lds_slots_);
    });
  } else {
    PCM_DISPATCH_K(K_, {
      if (fwd_spill_) launch(&hclt_forward_kernel<KK, true>); else launch(&hclt_forward_kernel<KK, false>);
    });
  }
  check_launch("hclt_forward");
}

void HcltCircuit::run_backward(const HcltDev& d) {
  const size_t lds = (size_t)lds_slots_ * kSlice * K_ * sizeof(float);
  auto launch = [&](auto kernel) {
    PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    PCM_LAUNCH_PHASE(1, kernel, dim3(d.nslices), dim3(kWalkWaves * 64), lds, d, d_bwd_fields_.p, bwd_stride_,
                     d_bwd_sched_.p, n_bwd_steps_);
  };
  const bool small = (size_t)(n_inner_ + 1) * d.tile_stride < ((size_t)1 << 31);
  if (lean_ && small && !force_general_walks_) {
    const size_t lean_lds = lds + kLeanFlagWords * 4;
    auto launch_lean = [&](auto kernel) {
      PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lean_lds));
      const LeanPlan* fp = fine_plan(d.nslices);
      if (fp)
        PCM_LAUNCH_PHASE(1, kernel, dim3(d.nslices, fp->n_groups), dim3(kWalkWaves * 64), lean_lds, d, fp->bwd.p,
                         fp->bwd_stride, fp->n_bwd_steps, lds_slots_);
      else
        PCM_LAUNCH_PHASE(1, kernel, dim3(d.nslices, n_groups_), dim3(kWalkWaves * 64), lean_lds, d, d_bwd_lean_.p, bwd_stride_,
                         n_bwd_steps_, lds_slots_);
    };
    PCM_DISPATCH_LEAN_K(K_, {
      if (H_ > 0) launch_lean(&hclt_backward_lean_kernel<KK, true>); else launch_lean(&hclt_backward_lean_kernel<KK, false>);
    });
  } else {
    PCM_DISPATCH_K(K_, {
      if (H_ > 0) {
        if (bwd_spill_) launch(&hclt_backward_kernel<KK, true, true>); else launch(&hclt_backward_kernel<KK, false, true>);
      } else {
        if (bwd_spill_) launch(&hclt_backward_kernel<KK, true, false>); else launch(&hclt_backward_kernel<KK, false, false>);
      }
    });
  }
  check_launch("hclt_backward");
}

void HcltCircuit::run_stats(const HcltDev& d, float rate) {
  if (soft_reg_ > 0.f) PCM_HIP(hipMemsetAsync(d_leaf_hist_.p, 0, d_leaf_hist_.n * sizeof(float), stream));   // (the kernels add to rate x what is there)
  // fixed-point split of the flows: limb sums over the padded batch must stay below 2^32
  int bits = 0;
  while ((1 << bits) < d.Bp) ++bits;
  const int limb = std::min(24, 32 - bits);
  if (limb < 12) fail(PCM_ERR_UNSUPPORTED, "batch of %d examples is too large for one call", d.B);
  const size_t hist = 2 * (size_t)C_ * (K_ + 1);                    // words per histogram (two limbs)
  const bool small = (size_t)(n_inner_ + 1) * d.tile_stride < ((size_t)1 << 31);
  if (lean_ && small && !force_general_walks_) {
    // LDS: the histograms of a pass (or the parked edge-flow blocks, whichever is larger) | per-wave pads
    const size_t park = (size_t)kStatLeanWaves * K_ * K_;
    const size_t hw = std::max((size_t)stat_lean_hists_ * 2 * C_ * K_, park);
    const size_t lds = (hw + (size_t)kStatLeanWaves * kSlice * K_) * 4;
    {
      PCM_DISPATCH_LEAN_K(K_, {
        PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hclt_stats_lean_kernel<KK>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        // one workgroup fills a compute unit; they draw nodes from d_stat_claim_, which every launch leaves at zero
        PCM_LAUNCH_PHASE(2, hclt_stats_lean_kernel<KK>, dim3(std::min(n_inner_, n_cus_)), dim3(kStatLeanWaves * 64), lds,
                         d, d_stat_lean_.p, d_edge_aggr_.p, stats_leaf_out(), rate, (int)hw, stat_lean_hists_, limb,
                         (H_ > 0 || d.w) ? (const int*)d_flow_shift_.p : (const int*)nullptr, d_stat_claim_.p, n_inner_);
      });
      check_launch("hclt_stats_lean");
      soft_reg_counts(rate);
      return;
    }
  }
  // LDS layout of hclt_stats_kernel
  const size_t pads = (size_t)kStatWaves * kSlice * (K_ + 16);
  auto hist_words = [&](int nh) { return std::max((((size_t)nh * hist + 3) & ~(size_t)3), (size_t)K_ * K_); };
  int nh = 3;
  while (nh > 1 && (hist_words(nh) + pads) * 4 > (size_t)max_lds_) --nh;
  const size_t lds = (hist_words(nh) + pads) * 4;
  if (lds > (size_t)max_lds_)
    fail(PCM_ERR_UNSUPPORTED, "statistics kernel needs %zu bytes of LDS, device offers %d", lds, max_lds_);
  auto launch = [&](auto kernel) {
    PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    PCM_LAUNCH_PHASE(2, kernel, dim3(n_inner_), dim3(kStatWaves * 64), lds, d, d_stat_items_.p, d_edge_aggr_.p,
                     stats_leaf_out(), rate, nh, (int)hist_words(nh), limb, (H_ > 0 || d.w) ? (const int*)d_flow_shift_.p : (const int*)nullptr);
  };
  PCM_DISPATCH_K(K_, {
    if (d.leaf_slice != 0) launch(&hclt_stats_kernel<KK, true>); else launch(&hclt_stats_kernel<KK, false>);
  });
  check_launch("hclt_stats");
  soft_reg_counts(rate);
}

void HcltCircuit::loglikelihoods(const BatchRef& b, float* d_ll) {
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  if (!block_ && !wide_) return general()->loglikelihoods(b, d_ll);
  if (const int chunk = walk_chunk(b.batch)) {
    for (int off = 0; off < b.batch; off += chunk) loglikelihoods(chunk_of(b, off, chunk), d_ll + off);
    return;
  }
  stage_batch(b);
  if (wide_walk_) return wide_forward(dev(b.batch), d_ll);
  if (H_ > 0) {   // per-head values [H][batch]
    const HcltDev d = dev(b.batch);
    run_forward(d, nullptr);   // (the head kernel reads the root tiles and the row maxima)
    heads_forward(d, nullptr, d_ll, nullptr);
    return;
  }
  run_forward(dev(b.batch), d_ll);
}

// Soft evidence (src/regularization/reg_likelihood.jl:51-91, reg_flow.jl:50-82) runs on the layered
// engine over the circuit's general form for every hidden size.
// Single-head circuits with K <= 64 take it on the block kernels: a value table [V][Bp][K] of the
// batch stands in for the leaf table (hclt_soft_evidence.hip.hpp).
HcltDev HcltCircuit::soft_stage(const SoftRef& s) {
  if (!s.d_ev) fail(PCM_ERR_ARG, "evidence pointer is null");
  if (s.batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", s.batch);
  ensure_batch(s.batch);
  HcltDev d = dev(s.batch);
  if ((size_t)d.Bp * K_ * 4 >= ((size_t)1 << 31)) fail(PCM_ERR_UNSUPPORTED, "batch of %d examples is too large for one call", s.batch);
  const int64_t nx = (int64_t)V_ * d.Bp;
  hipLaunchKernelGGL(hclt_soft_x_kernel, dim3(ceil_div(nx, 256)), dim3(256), 0, stream, d_xb_.p, nx);
  hipLaunchKernelGGL(hclt_pack_x_kernel, dim3(ceil_div(d.Bp, 1024), n_inner_), dim3(256), 0, stream, d_nodes_.p,
                     d_child_leaf_.p, d_xb_.p, n_inner_, d.Bp, d_xn_.p);
  check_launch("soft pack_x");
  const int Bp64 = ceil_div(d.Bp, kEvExamples) * kEvExamples;
  d_soft_lv_.ensure((size_t)V_ * Bp64 * K_);
  d_soft_m_.ensure((size_t)V_ * Bp64);
  const int Cp = (C_ + 3) & ~3;
  const size_t lds = ((size_t)kEvExamples * (Cp + 4) + (size_t)Cp * (K_ + 16) + kEvExamples) * sizeof(float);
  PCM_DISPATCH_K(K_, {
    PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hclt_soft_leafval_kernel<KK>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(hclt_soft_leafval_kernel<KK>, dim3(ceil_div(V_, kEvVars), Bp64 / kEvExamples), dim3(4 * (KK / 16) * 64), lds,
                       stream, s, d_leaf_.p, C_, V_, s.batch, Bp64, d_soft_lv_.p, d_soft_m_.p);
  });
  check_launch("soft_leafval");
  d.leaf = d_soft_lv_.p;
  d.leaf_stride = (uint32_t)((size_t)Bp64 * K_ * 4);
  d.leaf_slice = (uint32_t)kSlice * K_ * 4;
  return d;
}

void HcltCircuit::loglikelihoods_soft(const SoftRef& s, float* d_ll) {
  if (soft_reg_ > 0.f) fail(PCM_ERR_STATE, "soft_reg smoothing is for categorical batches; switch it off for soft evidence");
  no_forest("soft evidence");
  no_missing("soft evidence");
  if (!soft_block_ok()) return general()->loglikelihoods_soft(s, d_ll);
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  const HcltDev d = soft_stage(s);
  if (wide_walk_) return wide_forward(d, d_ll);
  force_general_walks_ = true;
  run_forward(d, d_ll);
  force_general_walks_ = false;
}

void HcltCircuit::flows_soft(const SoftRef& s, float rate, const float* d_head_mask, float* d_ll) {
  if (soft_reg_ > 0.f) fail(PCM_ERR_STATE, "soft_reg smoothing is for categorical batches; switch it off for soft evidence");
  no_forest("soft evidence");
  no_missing("soft evidence");
  // (per-example weights on soft evidence -- a mask for a single-head circuit -- go to the layered engine)
  if (soft_block_ok() && !(H_ == 0 && d_head_mask) && flow_scale == 1.f) {   // (tempered flows: the layered engine)
    if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
    if (flows_in_general_ && rate != 0.f) fail(PCM_ERR_STATE, "flow memory cannot carry over from the layered engine");
    const HcltDev d = soft_stage(s);
    if (d_soft_gnode_.n == 0) {   // the tile that carries the flow of a variable's leaves: its own node's, or its parent's
      std::vector<int32_t> gn(V_);
      for (int v = 0; v < V_; ++v)
        for (int c : children_[v]) gn[c] = inner_of_var_[v];
      for (int v = 0; v < V_; ++v)
        if (inner_of_var_[v] >= 0) gn[v] = inner_of_var_[v];
      d_soft_gnode_.upload(gn);
    }
    const float* g_tiles = d.R;   // where the statistics pass leaves the child-flow tiles
    if (wide_walk_) {
      wide_forward(d, d_ll);
      wide_backward_stats(d, rate, true);
      g_tiles = d_G_.p;
    } else {
      force_general_walks_ = true;
      run_forward(d, d_ll);
      run_backward(d);
      run_stats(d, rate);
      force_general_walks_ = false;
    }
    const int Bp64 = ceil_div(d.Bp, kEvExamples) * kEvExamples;
    // old statistics times the flow memory rate first; then the batch's counts.  Small tables are split over the
    // examples (in chunks of 64) until about 512 workgroups run; the splits' shares are added in order afterwards
    const int64_t n_leaf = (int64_t)V_ * C_ * K_;
    hipLaunchKernelGGL(hclt_soft_scale_kernel, dim3(ceil_div(n_leaf, 256)), dim3(256), 0, stream, d_leaf_flow_.p, n_leaf, rate);
    const int chunks = ceil_div(s.batch, kEvExamples);
    const int want = std::max(1, ceil_div(512, (int64_t)V_ * ceil_div(C_, kEvCats)));
    const int split = ceil_div(chunks, std::min(chunks, want)) * kEvExamples;      // examples per split
    const int n_split = ceil_div(s.batch, split);
    if (n_split > 1) d_part_.ensure((size_t)n_split * n_leaf);
    PCM_DISPATCH_K(K_, hipLaunchKernelGGL(hclt_soft_leafflow_kernel<KK>, dim3(ceil_div(C_, kEvCats), V_, n_split),
                                          dim3(256), 0, stream, s, d_leaf_.p, d_soft_lv_.p, d_soft_m_.p, g_tiles,
                                          d_soft_gnode_.p, C_, s.batch, Bp64, (size_t)d.tile_stride / 4, split,
                                          d_leaf_flow_.p, n_split > 1 ? d_part_.p : (float*)nullptr));
    if (n_split > 1)
      hipLaunchKernelGGL(sum_parts_kernel<false>, dim3(ceil_div(n_leaf, 64)), dim3(256), 0, stream, d_part_.p, n_split, n_leaf,
                         (const float*)nullptr, d_leaf_flow_.p);
    check_launch("soft_leafflow");
    have_flows_ = true;
    flows_in_general_ = false;
    if (timing) ++n_timed_;
    return;
  }
  if (have_flows_ && !flows_in_general_ && rate != 0.f && (block_ || wide_))
    fail(PCM_ERR_STATE, "flow memory cannot carry over from categorical batches to soft-evidence batches");
  general()->flow_scale = flow_scale;
  general()->flows_soft(s, rate, d_head_mask, d_ll);
  have_flows_ = true;
  flows_in_general_ = true;
}

void HcltCircuit::flows(const BatchRef& b, float rate, const float* d_head_mask, float* d_ll) {
  // a single-head circuit takes the mask as [1][batch]: the flow every example starts with at the root, i.e. the
  // per-example weights of reg_flow.jl:38-39,190-191 (every flow is linear in it)
  const float* weights = H_ == 0 ? d_head_mask : nullptr;
  if (H_ > 0 && !d_head_mask) fail(PCM_ERR_ARG, "a multi-head circuit needs a head_mask for its flows");
  if (!d_ll) fail(PCM_ERR_ARG, "output pointer is null");
  if (flow_scale != 1.f && (block_ || wide_)) {
    // tempered flows (fscale of mini_batch_em_beta) are the layered engine's: the block kernels keep S, not the sum of
    // the shares to the power 1 / fscale
    if (soft_reg_ > 0.f && soft_written_)
      fail(PCM_ERR_UNSUPPORTED, "tempered flows with the leaf flows of soft_reg as the source writes them: that form is the block kernels'");
    if (have_flows_ && !flows_in_general_ && rate != 0.f)
      fail(PCM_ERR_STATE, "flow memory cannot carry over from ordinary flows on the block kernels to tempered flows");
    SparseCircuit* g = general();
    g->flow_scale = flow_scale;
    if (soft_reg_ > 0.f) {
      // soft_reg and fscale together (scaled_probs_flows_circuit, src-jl/learning/flow.jl:366-372): the layered form
      // has no smoothed leaf table, it takes the batch as the soft evidence that gives its leaves the smoothed values
      no_forest("soft_reg with tempered flows");
      const int64_t total = (int64_t)b.batch * Vu_ * C_;
      d_soft_reg_ev_.ensure((size_t)total);
      hipLaunchKernelGGL(hclt_soft_reg_evidence_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, stream, b, Vu_, C_,
                         soft_reg_, soft_width_, d_soft_reg_ev_.p);
      check_launch("soft_reg_evidence");
      const SoftRef ev{d_soft_reg_ev_.p, (int64_t)Vu_ * C_, C_, 1, nullptr, b.batch};
      g->flows_soft(ev, rate, d_head_mask, d_ll);
    } else {
      g->flows(b, rate, d_head_mask, d_ll);
    }
    have_flows_ = true;
    flows_in_general_ = true;
    return;
  }
  if (flows_in_general_ && rate != 0.f && (block_ || wide_))
    fail(PCM_ERR_STATE, "flow memory cannot carry over from soft-evidence batches to categorical batches");
  flows_in_general_ = false;
  if (!block_ && !wide_) {
    general()->flow_scale = flow_scale;
    general()->flows(b, rate, weights, d_ll);
    have_flows_ = true;
    return;
  }
  if (const int chunk = walk_chunk(b.batch)) {
    // the accumulators take the first chunk scaled by `rate` and the others on top
    for (int off = 0; off < b.batch; off += chunk)
      flows(chunk_of(b, off, chunk), off == 0 ? rate : 1.f, weights ? weights + off : nullptr, d_ll + off);
    return;
  }
  stage_batch(b);
  HcltDev d = dev(b.batch);
  d.w = weights;
  if (weights) {   // bound on the flow of one example, as a power of two, for the statistics' fixed-point counters
    hipLaunchKernelGGL(hclt_weight_shift_kernel, dim3(1), dim3(256), 0, stream, weights, b.batch, d_flow_shift_.p);
    check_launch("weight_shift");
  }
  if (H_ > 0) {
    run_forward(d, nullptr);
    heads_forward(d, d_head_mask, nullptr, d_ll, true, rate);
    const size_t lds = ((size_t)16 * Hp_ + 16 * K_ + (size_t)kHeadWaves * 16 * K_ + (size_t)kHeadWaves * 16) * sizeof(float);
    d_part_.ensure((size_t)T_ * d.nslices * H_ * K_);
    PCM_DISPATCH_LEAN_K(K_, hipLaunchKernelGGL(hclt_heads_backward_kernel<KK>, dim3(d.nslices, T_), dim3(kHeadWaves * 64), lds,
                                               stream, d.O, d.R, d_root_node_.p, (int64_t)(d.tile_stride / 4), d_head_wf_.p,
                                               d_head_wb_.p, H_, Hp_, d.B, d_head_mask, d_part_.p, d_flow_shift_.p));
    hipLaunchKernelGGL(sum_parts_kernel<true>, dim3(ceil_div((int64_t)H_ * K_, 64), T_), dim3(256), 0, stream, d_part_.p,
                       d.nslices, (int64_t)H_ * K_, head_logp(), head_aggr());
    check_launch("heads_backward");
    run_backward(d);
    run_stats(d, rate);
    have_flows_ = true;
    if (timing) ++n_timed_;
    return;
  }
  if (wide_walk_) {
    wide_forward(d, d_ll);
    wide_backward_stats(d, rate);
    have_flows_ = true;
    if (timing) ++n_timed_;
    return;
  }
  run_forward(d, d_ll);
  run_backward(d);
  run_stats(d, rate);
  have_flows_ = true;
  if (timing) ++n_timed_;
}

// Relaxed sampling on the block form; false: this hidden size / temperature goes to the layered engine.
const float* HcltCircuit::kernel_noise(const float* d_node_noise, int32_t batch) {
  if (V_ == Vu_ || !d_node_noise) return d_node_noise;
  if (K_ % 4) fail(PCM_ERR_STATE, "noise rows of %d floats do not move as 16-byte words", K_);
  if (d_user_index_.n == 0) d_user_index_.upload(user_index_, stream);
  const int64_t total = (int64_t)batch * n_inner_ * (K_ / 4);
  d_noise_x_.ensure((size_t)total * 4);
  hipLaunchKernelGGL(hclt_expand_noise_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, stream,
                     reinterpret_cast<const float4*>(d_node_noise), d_user_index_.p, n_inner_, n_user_inner_, K_ / 4, total,
                     reinterpret_cast<float4*>(d_noise_x_.p));
  check_launch("expand_noise");
  return d_noise_x_.p;
}

bool HcltCircuit::sample_soft_block(const float* d_node_noise, float temperature, int32_t batch, float* d_out) {
  if (!block_ || !(temperature >= kSoftMinTemperature)) return false;
  if (!d_out) fail(PCM_ERR_ARG, "output pointer is null");
  if (batch < 1) fail(PCM_ERR_ARG, "batch must be positive, got %d", batch);
  if ((reinterpret_cast<uintptr_t>(d_node_noise) | reinterpret_cast<uintptr_t>(d_out)) & 15)
    fail(PCM_ERR_ARG, "noise and output pointers must be 16-byte aligned (rows move as 16-byte words)");
  if (d_soft_tabs_.n == 0) {
    // parent of every inner node | per variable the node whose probabilities reach its leaf |
    // inner nodes by depth | level offsets
    std::vector<int32_t> t((size_t)n_inner_ + V_);
    for (int n = 0; n < n_inner_; ++n) {
      const int v = var_of_inner_[n];
      t[n] = parent_[v] < 0 ? -1 : inner_of_var_[parent_[v]];
    }
    for (int v = 0; v < V_; ++v) t[(size_t)n_inner_ + v] = children_[v].empty() ? inner_of_var_[parent_[v]] : inner_of_var_[v];
    std::vector<std::vector<int32_t>> by_depth;
    for (int n = 0; n < n_inner_; ++n) {
      const size_t dep = (size_t)depth_[var_of_inner_[n]];
      if (by_depth.size() <= dep) by_depth.resize(dep + 1);
      by_depth[dep].push_back(n);
    }
    std::vector<int32_t> ptr(1, 0);
    for (const auto& lvl : by_depth) {
      t.insert(t.end(), lvl.begin(), lvl.end());
      ptr.push_back(ptr.back() + (int32_t)lvl.size());
    }
    soft_levels_ = (int)by_depth.size();
    t.insert(t.end(), ptr.begin(), ptr.end());
    d_soft_tabs_.upload(t, stream);
  }
  ensure_batch(batch);                       // the flow-ratio tiles double as the probability tiles
  const int ns = ceil_div(batch, kSlice);
  d_soft_w_.ensure((size_t)2 * n_inner_ * K_ * K_);
  float* Af = d_soft_w_.p;
  float* Ab = Af + (size_t)n_inner_ * K_ * K_;
  const float inv_t = 1.f / temperature;
  const int32_t* parent_of = d_soft_tabs_.p;
  const int32_t* state_node = parent_of + n_inner_;
  const int32_t* order = state_node + V_;
  const int32_t* level_ptr = order + n_inner_;
  PCM_DISPATCH_K(K_, {
    hipLaunchKernelGGL(hclt_soft_w_kernel<KK>, dim3(ceil_div((int64_t)n_inner_ * K_, 128)), dim3(128), 0, stream, d_logtheta_.p,
                       inv_t, n_inner_, Af, Ab);
    hipLaunchKernelGGL(hclt_soft_walk_kernel<KK>, dim3(ns), dim3(soft_walk_waves(KK) * 64), 0, stream, Af, Ab, parent_of, order,
                       level_ptr, soft_levels_, kernel_noise(d_node_noise, batch), n_inner_, batch, ns, inv_t, d_R_.p);
    const int nchunks = ceil_div(C_, kSoftLeafCats);
    const int use_rows = (C_ & 3) == 0 ? 1 : 0;   // rows of whole 16-byte words leave through an LDS pad
    const int run_slices = soft_leaf_run_slices((int64_t)Vu_ * nchunks, ns);
    const dim3 lgrid(Vu_, ceil_div(nchunks * ceil_div(ns, run_slices), 4));   // (the caller's variables)
    const size_t pad_bytes = use_rows ? (size_t)4 * kSlice * (kSoftLeafCats + 4) * sizeof(float) : 0;   // 65 KB
    PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&hclt_soft_leaves_kernel<KK>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)pad_bytes));
    hipLaunchKernelGGL(hclt_soft_leaves_kernel<KK>, lgrid, dim3(256), pad_bytes, stream, d_leaf_.p, state_node, d_R_.p, Vu_,
                       C_, batch, ns, nchunks, run_slices, use_rows, d_out);
  });
  check_launch("hclt_sample_soft");
  PCM_HIP(hipStreamSynchronize(stream));
  return true;
}

HcltCircuit::~HcltCircuit() {
  for (hipEvent_t e : ev_) (void)hipEventDestroy(e);
  if (walk_err_) (void)hipHostFree(walk_err_);
}

// A walk kernel whose wave ran out of polls waiting for a tile has raised the word (its results are
// void); seen here at the next call that looks.
// The same kernel raises a word in device memory, which the update kernels look at: they leave the parameters
// alone after a void pass, whether or not the host has looked in between (pcm_em_step queues flows and update
// without waiting).  Reporting also puts the device word and the statistics kernel's node counter back to zero
// (a launch that followed a void walk may have ended before all its tickets were drawn).
void HcltCircuit::check_walks() {
  if (walk_err_ && *walk_err_) {
    (void)hipStreamSynchronize(stream);
    *walk_err_ = 0;
    if (d_walk_void_.p) (void)hipMemsetAsync(d_walk_void_.p, 0, sizeof(int32_t), stream);
    if (d_stat_claim_.p) (void)hipMemsetAsync(d_stat_claim_.p, 0, sizeof(uint32_t), stream);
    have_flows_ = false;
    fail(PCM_ERR_HIP, "a tree-walk kernel gave up waiting for a tile of an earlier step; the results of that pass are void");
  }
}

void HcltCircuit::sync_checked() {
  PCM_HIP(hipStreamSynchronize(stream));
  check_walks();
}

hipEvent_t* HcltCircuit::ev_set() {
  if (ev_.empty()) {
    ev_.resize((size_t)kTimingRing * 6, nullptr);
    for (auto& e : ev_) PCM_HIP(hipEventCreate(&e));
  }
  return ev_.data() + (size_t)(n_timed_ % kTimingRing) * 6;
}

void HcltCircuit::read_timing(float* ms, int n) {
  for (int i = 0; i < n; ++i) ms[i] = 0.f;
  const int cnt = std::min(n_timed_, (int)kTimingRing);
  if (cnt == 0) return;
  sync_checked();
  for (int s = 0; s < cnt; ++s)
    for (int i = 0; i < std::min(n, 3); ++i) {
      if (!(timing & (1 << i))) continue;
      float t = 0.f;
      PCM_HIP(hipEventElapsedTime(&t, ev_[(size_t)s * 6 + 2 * i], ev_[(size_t)s * 6 + 2 * i + 1]));
      ms[i] += t / cnt;
    }
  n_timed_ = 0;
}

void HcltCircuit::em_update(float pseudocount, float inertia) {
  check_walks();   // (a pass already known to be void is reported before its statistics are used)
  if (!have_flows_) fail(PCM_ERR_STATE, "pcm_em_update called before any pcm_flows");
  if (flows_in_general_ || (!block_ && !wide_)) {
    general_->em_update(pseudocount, inertia);
    PCM_HIP(hipStreamSynchronize(stream));
    pull_from_general();
    return;
  }
  // the leaf tables first, the parameter blocks last: what the next forward walk reads most often is then
  // what the caches saw last (the blocks are read by every workgroup, a leaf table row by sixteen examples)
  // 32 category groups per workgroup; a thread holds its group's share of the categories (8 of 256)
  {
    const int threads = 1024, cats = ceil_div(C_, threads / 32);
    auto launch = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(Vu_, ceil_div(K_, 32)), dim3(threads), 0, stream, d_leaf_.p, d_leaf_flow_.p, C_, K_,
                         pseudocount, inertia, missing_ ? 1 : 0, (const int32_t*)d_walk_void_.p);
    };
    if (cats <= 8) launch(&hclt_leaf_update_kernel<8>);
    else if (cats <= 16) launch(&hclt_leaf_update_kernel<16>);
    else launch(&hclt_leaf_update_kernel<32>);
  }
  check_launch("leaf_update");
  leaf_changed();   // (the smoothed table of soft_reg follows the leaf table)
  PCM_DISPATCH_PARAM_K(K_, {
    constexpr int rows_per_block = 256 / (KK < 64 ? KK : 64);
    hipLaunchKernelGGL(hclt_theta_update_kernel<KK>, dim3(ceil_div((int64_t)n_inner_ * K_, rows_per_block)), dim3(256), 0,
                       stream, d_nodes_.p, d_logtheta_.p, d_Wf_.p, d_Wb_.p, d_edge_aggr_.p, n_inner_, pseudocount, inertia,
                       H_ > 0 ? 1 : 0, (const int32_t*)d_walk_void_.p);
  });
  check_launch("theta_update");
  if (H_ > 0) {
    hipLaunchKernelGGL(hclt_heads_update_kernel, dim3(ceil_div(H_, 4), T_), dim3(256), 0, stream, head_logp(), head_aggr(), H_,
                       Hp_, K_, pseudocount, inertia, d_head_wf_.p, d_head_wb_.p, (const int32_t*)d_walk_void_.p);
  }
  general_stale_ = true;
}

}  // namespace pcm
