/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's probabilistic-circuit
 * arithmetic (forward, flows, mini-batch EM update, KL recursion, Gumbel sampling).
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may load this file's
 * library; the product never does.
 *
 * The circuit is given in the reference's own flat form: nodes in topological order
 * (root last) and "up" edges grouped by parent, each edge carrying a prime child, an
 * optional sub child (-1 if none) and, for sum edges, a log-parameter.  Every function
 * names the reference lines whose arithmetic it repeats (paths are relative to
 * VariationalJuice.jl/src).  Arithmetic is done in REAL (float by default, the
 * reference's type; build with -DREAL=double for the high-precision twin used to pin
 * the float build by finite differences and closed forms).
 *
 * Pinned by tests/test_oracle_pinning.py: brute-force latent enumeration on tiny HCLTs,
 * closed forms quoted from the reference's own tests, finite-difference checks of the
 * flows (= dLL/dlogtheta) and of the KL gradient, exact M-step properties, statistics
 * of exact samples, the closed form theta^(1/T) / sum theta^(1/T) and the cold limit of the
 * relaxed sampler.  The two leaf lines of orc_kld_backward in their as-written form
 * (analytic == 0; nodes/fixable_categorical_dist.jl:219, not the analytic derivative) are
 * pinned through their fixed ratio to the finite-difference-checked analytic form and by a
 * literal worked by hand.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL float
#endif

#define NODE_INPUT 0
#define NODE_SUM 1
#define NODE_MUL 2

int orc_max_threads(void);

#if defined(_OPENMP)
#include <omp.h>
#endif

/* ProbabilisticCircuits.jl `logsumexp(x::Float32, y::Float32)` (un-vendored dependency,
 * used at queries/likelihood.jl:101-102 and regularization/reg_likelihood.jl:127-128):
 * max + log1p(exp(-|x-y|)) when both finite, else max. */
static inline REAL lse2f(REAL x, REAL y) {
  if (isfinite(x) && isfinite(y)) {
    REAL m = x > y ? x : y;
    REAL d = x > y ? x - y : y - x;
    if (sizeof(REAL) == 4) return m + log1pf(expf(-(float)d));
    return m + (REAL)log1p(exp(-(double)d));
  }
  return x > y ? x : y;
}

/*
 * Forward pass for a chunk of examples.
 *   leaf init  : regularization/reg_likelihood.jl:16-49 with soft_reg = 0 (categorical
 *                lookup heap[heap_start + value], nodes/fixable_categorical_dist.jl:87-88);
 *                sums start at -Inf, products at 0.
 *   inner nodes: queries/likelihood.jl:29-48 -- child_prob = mars[prime] (+ mars[sub])
 *                (+ logp for a sum edge); first edge of a parent starts the accumulator,
 *                later edges fold in with logsumexp (sum) or + (product).
 * mars is [n_nodes][B] (example fastest).  data is [N][V] uint8, row idx[b] is example b.
 */
void orc_forward(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                 const int32_t* prime, const int32_t* sub, const REAL* logp,
                 const int32_t* in_var, const int64_t* in_off, const REAL* leaf_logp,
                 const uint8_t* data, int64_t V, const int32_t* idx, int B, REAL* mars) {
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    const uint8_t* row = data + (int64_t)idx[b] * V;
    for (int n = 0; n < n_nodes; ++n) {
      REAL* out = mars + (int64_t)n * B + b;
      if (type[n] == NODE_INPUT) {
        *out = leaf_logp[in_off[n] + row[in_var[n]]];
        continue;
      }
      int issum = type[n] == NODE_SUM;
      REAL acc = issum ? (REAL)-INFINITY : (REAL)0;
      for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
        REAL child = mars[(int64_t)prime[e] * B + b];
        if (sub[e] >= 0) child += mars[(int64_t)sub[e] * B + b];
        if (issum) child += logp[e];
        if (e == edge_ptr[n]) acc = child;
        else if (issum) acc = lse2f(acc, child);
        else acc += child;
      }
      *out = acc;
    }
  }
}

/*
 * Backward flows for a chunk of examples.
 *   init       : queries/flow.jl:140-143 -- flows = 0, root (last node) = 1; if
 *                root_flow != NULL the listed nodes start from root_flow[h][b] instead
 *                (multi-head seeding, src-jl/multi_head_pc/flow.jl:141-176).
 *   inner nodes: queries/flow.jl:49-60 -- edge_flow = flows[parent] for a product edge;
 *                for a sum edge child_prob = mars[prime] + logp (+ mars[sub]) and
 *                edge_flow = flows[parent] * exp(child_prob - mars[parent]);
 *                flows[prime] += edge_flow, flows[sub] += edge_flow (:62-68, :84-99);
 *                edge_aggr[e] += sum_b edge_flow (:73-81).
 *   skip[e]!=0 : edge left out of the downward pass (tag bit 4 of the multi-head fake
 *                root, src-jl/multi_head_pc/flow.jl:45).
 * Parents are visited in reverse topological order, so flows[parent] is complete when
 * its edges are expanded, as with the reference's down layers.
 * edge_aggr is accumulated in double across examples and added to the REAL array.
 */
void orc_backward(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                  const int32_t* prime, const int32_t* sub, const REAL* logp,
                  const uint8_t* skip, const REAL* mars, int B, REAL* flows,
                  REAL* edge_aggr, int n_roots, const int32_t* root_ids,
                  const REAL* root_flow) {
  int n_edges = edge_ptr[n_nodes];
  int nthreads = orc_max_threads();
  if (nthreads > B) nthreads = B;
  double* aggr = (double*)calloc((size_t)n_edges * nthreads, sizeof(double));
  /* examples are independent: each thread owns a contiguous range of them */
#pragma omp parallel for schedule(static) num_threads(nthreads)
  for (int t = 0; t < nthreads; ++t) {
    int b0 = (int)((int64_t)B * t / nthreads), b1 = (int)((int64_t)B * (t + 1) / nthreads);
    double* my = aggr + (size_t)t * n_edges;
    for (int n = 0; n < n_nodes; ++n)
      for (int b = b0; b < b1; ++b) flows[(int64_t)n * B + b] = 0;
    if (n_roots == 0) {
      for (int b = b0; b < b1; ++b) flows[(int64_t)(n_nodes - 1) * B + b] = 1;
    } else {
      for (int h = 0; h < n_roots; ++h)
        for (int b = b0; b < b1; ++b)
          flows[(int64_t)root_ids[h] * B + b] = root_flow[(int64_t)h * B + b];
    }
    for (int n = n_nodes - 1; n >= 0; --n) {
      if (type[n] == NODE_INPUT) continue;
      int issum = type[n] == NODE_SUM;
      for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
        if (skip && skip[e]) continue;
        double s = 0;
        for (int b = b0; b < b1; ++b) {
          REAL ef = flows[(int64_t)n * B + b];
          if (issum) {
            REAL child = mars[(int64_t)prime[e] * B + b] + logp[e];
            if (sub[e] >= 0) child += mars[(int64_t)sub[e] * B + b];
            REAL d = child - mars[(int64_t)n * B + b];
            ef = ef * (sizeof(REAL) == 4 ? (REAL)expf((float)d) : (REAL)exp((double)d));
          }
          flows[(int64_t)prime[e] * B + b] += ef;
          if (sub[e] >= 0) flows[(int64_t)sub[e] * B + b] += ef;
          s += ef;
        }
        my[e] += s;
      }
    }
  }
  if (edge_aggr)
    for (int e = 0; e < n_edges; ++e) {
      double s = 0;
      for (int t = 0; t < nthreads; ++t) s += aggr[(size_t)t * n_edges + e];
      edge_aggr[e] += (REAL)s;
    }
  free(aggr);
}

/*
 * Tempered flows of mini_batch_em_beta (fscale), VariationalJuice.jl/src-jl/learning/flow.jl:
 *   :120-175 scale_flows_kernel -- per sum node and example the logsumexp over its edges of
 *            (child - parent) / fscale, folded pairwise in edge order (the node-owned path, flows_buf = acc);
 *   :204-300 reg_layer_down_kernel -- edge flow = flows[parent] * exp((child - parent) / fscale - that logsumexp)
 *            for a sum edge, flows[parent] for a product edge; children and edge_aggr as in orc_backward.
 * The root's flow (flows[:, end] = 1, :344) or root_flow as in orc_backward.
 */
void orc_backward_scaled(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                         const int32_t* prime, const int32_t* sub, const REAL* logp,
                         const uint8_t* skip, const REAL* mars, int B, REAL* flows,
                         REAL* edge_aggr, int n_roots, const int32_t* root_ids,
                         const REAL* root_flow, REAL fscale) {
  int n_edges = edge_ptr[n_nodes];
  double* aggr = (double*)calloc((size_t)n_edges, sizeof(double));
  REAL* norm = (REAL*)malloc((size_t)B * sizeof(REAL));
  for (int64_t i = 0; i < (int64_t)n_nodes * B; ++i) flows[i] = 0;
  if (n_roots == 0) {
    for (int b = 0; b < B; ++b) flows[(int64_t)(n_nodes - 1) * B + b] = 1;
  } else {
    for (int h = 0; h < n_roots; ++h)
      for (int b = 0; b < B; ++b) flows[(int64_t)root_ids[h] * B + b] = root_flow[(int64_t)h * B + b];
  }
  for (int n = n_nodes - 1; n >= 0; --n) {
    if (type[n] == NODE_INPUT) continue;
    int issum = type[n] == NODE_SUM;
    if (issum)
      for (int b = 0; b < B; ++b) {
        int first = 1;
        REAL acc = 0;
        for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
          if (skip && skip[e]) continue;
          REAL child = mars[(int64_t)prime[e] * B + b] + logp[e];
          if (sub[e] >= 0) child += mars[(int64_t)sub[e] * B + b];
          REAL d = (child - mars[(int64_t)n * B + b]) / fscale;
          acc = first ? d : lse2f(acc, d);
          first = 0;
        }
        norm[b] = acc;
      }
    for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
      if (skip && skip[e]) continue;
      double s = 0;
      for (int b = 0; b < B; ++b) {
        REAL ef = flows[(int64_t)n * B + b];
        if (issum) {
          REAL child = mars[(int64_t)prime[e] * B + b] + logp[e];
          if (sub[e] >= 0) child += mars[(int64_t)sub[e] * B + b];
          REAL d = (child - mars[(int64_t)n * B + b]) / fscale - norm[b];
          ef = ef * (sizeof(REAL) == 4 ? (REAL)expf((float)d) : (REAL)exp((double)d));
        }
        flows[(int64_t)prime[e] * B + b] += ef;
        if (sub[e] >= 0) flows[(int64_t)sub[e] * B + b] += ef;
        s += ef;
      }
      aggr[e] += s;
    }
  }
  if (edge_aggr)
    for (int e = 0; e < n_edges; ++e) edge_aggr[e] += (REAL)aggr[e];
  free(norm);
  free(aggr);
}

/*
 * Leaf sufficient statistics: queries/flow.jl:165-195 with the categorical `flow`
 * of nodes/fixable_categorical_dist.jl:121-130: counts[node][value] += flows[b, node].
 * leaf_flow has the same indexing as leaf_logp (in_off[n] + category).
 */
void orc_input_flows(int n_nodes, const uint8_t* type, const int32_t* in_var,
                     const int64_t* in_off, const uint8_t* data, int64_t V,
                     const int32_t* idx, int B, const REAL* flows, REAL* leaf_flow) {
  for (int n = 0; n < n_nodes; ++n) {
    if (type[n] != NODE_INPUT) continue;
    for (int b = 0; b < B; ++b) {
      int x = data[(int64_t)idx[b] * V + in_var[n]];
      leaf_flow[in_off[n] + x] += flows[(int64_t)n * B + b];
    }
  }
}

/*
 * Soft evidence: data is a [B][V][C] array of log-evidence instead of one category per variable.
 *   leaf value : regularization/reg_likelihood.jl:51-91 -- logsumexp_c(data[b,v,c] + logp_c),
 *                folded pairwise from -inf in category order
 *   leaf flows : regularization/reg_flow.jl:50-82 -- counts[c] += exp(data[b,v,c] + logp_c - value) * flow
 * Inner nodes are those of orc_forward / orc_backward.
 */
void orc_forward_soft(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                      const int32_t* prime, const int32_t* sub, const REAL* logp,
                      const int32_t* in_var, const int64_t* in_off, int C, const REAL* leaf_logp,
                      const REAL* ev, int64_t V, int B, REAL* mars) {
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    for (int n = 0; n < n_nodes; ++n) {
      REAL* out = mars + (int64_t)n * B + b;
      if (type[n] == NODE_INPUT) {
        const REAL* e = ev + ((int64_t)b * V + in_var[n]) * C;
        REAL acc = (REAL)-INFINITY;
        for (int c = 0; c < C; ++c) acc = lse2f(acc, e[c] + leaf_logp[in_off[n] + c]);
        *out = acc;
        continue;
      }
      int issum = type[n] == NODE_SUM;
      REAL acc = issum ? (REAL)-INFINITY : (REAL)0;
      for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
        REAL child = mars[(int64_t)prime[e] * B + b];
        if (sub[e] >= 0) child += mars[(int64_t)sub[e] * B + b];
        if (issum) child += logp[e];
        if (e == edge_ptr[n]) acc = child;
        else if (issum) acc = lse2f(acc, child);
        else acc += child;
      }
      *out = acc;
    }
  }
}

void orc_input_flows_soft(int n_nodes, const uint8_t* type, const int32_t* in_var,
                          const int64_t* in_off, int C, const REAL* leaf_logp, const REAL* ev,
                          int64_t V, int B, const REAL* mars, const REAL* flows, REAL* leaf_flow) {
  for (int n = 0; n < n_nodes; ++n) {
    if (type[n] != NODE_INPUT) continue;
    for (int b = 0; b < B; ++b) {
      const REAL* e = ev + ((int64_t)b * V + in_var[n]) * C;
      REAL value = mars[(int64_t)n * B + b], f = flows[(int64_t)n * B + b];
      for (int c = 0; c < C; ++c) {
        REAL t = e[c] + leaf_logp[in_off[n] + c];
        if (t > (REAL)-INFINITY) leaf_flow[in_off[n] + c] += (REAL)exp((double)(t - value)) * f;
      }
    }
  }
}

/*
 * Mini-batch EM parameter update, in the reference's call order
 * (regularization/reg_em.jl:292-299):
 *   add_pseudocount : edge_aggr[e] += pseudocount / #sum-edges(parent)
 *                     (pretrain/mini_batch_warmup.jl:4-17 without its 1e-8 guard, which
 *                     the un-vendored original called by reg_em.jl:292 does not have)
 *   aggr_node_flows : node_aggr[parent] = sum_e edge_aggr[e]
 *   update_params   : logp = log(inertia*exp(logp) + (1-inertia)*edge_aggr/node_aggr),
 *                     skipped for a sum node with a single edge
 *                     (pretrain/mini_batch_warmup.jl:54-70)
 *   leaf update     : nodes/fixable_categorical_dist.jl:223-248 (missing_flow = 0 unless `missing`).
 * edge_aggr is modified in place (the pseudocount stays in it, as in the reference).
 */
void orc_em_update(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                   REAL* logp, REAL* edge_aggr, const int64_t* in_off, int C,
                   REAL* leaf_logp, const REAL* leaf_flow, REAL pseudocount, REAL inertia, int missing) {
  for (int n = 0; n < n_nodes; ++n) {
    if (type[n] == NODE_SUM) {
      int e0 = edge_ptr[n], e1 = edge_ptr[n + 1];
      REAL nsib = (REAL)(e1 - e0);
      REAL node_aggr = 0;
      for (int e = e0; e < e1; ++e) {
        edge_aggr[e] += pseudocount / nsib;
        node_aggr += edge_aggr[e];
      }
      if (e1 - e0 == 1) continue;
      for (int e = e0; e < e1; ++e) {
        REAL oldv = inertia * (REAL)exp((double)logp[e]);
        REAL newv = ((REAL)1 - inertia) * edge_aggr[e] / node_aggr;
        logp[e] = (REAL)log((double)(oldv + newv));
      }
    } else if (type[n] == NODE_INPUT) {
      REAL* lp = leaf_logp + in_off[n];
      const REAL* fl = leaf_flow + in_off[n];
      /* missing != 0: the last of the C table rows is not a category but the marker of a missing value
       * (log-probability 0, never updated); its flow is the reference's missing_flow (:233-241) */
      const int num_cats = missing ? C - 1 : C;
      const REAL missing_flow = missing ? fl[C - 1] : (REAL)0;
      REAL node_flow = 0;
      REAL cat_pc = pseudocount / (REAL)num_cats;
      for (int i = 0; i < num_cats; ++i) node_flow += fl[i];
      node_flow += missing_flow + pseudocount;
      for (int i = 0; i < num_cats; ++i) {
        REAL oldp = (REAL)exp((double)lp[i]);
        REAL oldv = inertia * oldp;
        REAL newv = ((REAL)1 - inertia) * (fl[i] + cat_pc + missing_flow * oldp) / node_flow;
        lp[i] = (REAL)log((double)(oldv + newv));
      }
    }
  }
}

/*
 * KL(p || q) between two parameterisations of one structure, bottom-up.
 *   leaves : nodes/fixable_categorical_dist.jl:187-192 (log-parameter form):
 *            kld = sum_c exp(p1_c) * (p1_c - p2_c)
 *   edges  : queries/kld.jl:95-107 -- kld = klds[prime] (+ klds[sub]); for a sum edge
 *            kld = exp(p1) * (kld + p1 - p2); a parent adds up its edges (:113-128).
 * klds is [n_nodes]; edge_klds [n_edges] (may be NULL).
 * norm_params != 0: the LEAF arrays hold probabilities instead of log-probabilities and the
 * leaf term is nodes/fixable_categorical_dist.jl:182-186,
 *            kld = sum_c p1_c * (log(p1_c + 1e-8) - log(p2_c + 1e-8));
 * the sum edges are in log space either way (queries/kld.jl:103-107 has no such switch).
 */
void orc_kld(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
             const int32_t* prime, const int32_t* sub, const REAL* logp1,
             const REAL* logp2, const int64_t* in_off, int C, const REAL* leaf1,
             const REAL* leaf2, REAL* klds, REAL* edge_klds, int norm_params) {
  for (int n = 0; n < n_nodes; ++n) {
    if (type[n] == NODE_INPUT) {
      REAL k = 0;
      for (int i = 0; i < C; ++i) {
        REAL a = leaf1[in_off[n] + i], b = leaf2[in_off[n] + i];
        if (norm_params) k += a * ((REAL)log((double)(a + (REAL)1e-8)) - (REAL)log((double)(b + (REAL)1e-8)));
        else k += (REAL)exp((double)a) * (a - b);
      }
      klds[n] = k;
      continue;
    }
    REAL acc = 0;
    for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
      REAL k = klds[prime[e]];
      if (sub[e] >= 0) k += klds[sub[e]];
      if (type[n] == NODE_SUM) k = (REAL)exp((double)logp1[e]) * (k + logp1[e] - logp2[e]);
      if (edge_klds) edge_klds[e] = k;
      acc = (e == edge_ptr[n]) ? k : acc + k;
    }
    klds[n] = acc;
  }
}

/*
 * Reverse pass of the KL recursion with respect to the log-parameters.
 *   init   : queries/kld.jl:476-479 -- grads = 0, root = 1
 *   edges  : queries/kld.jl:262-281 -- for a sum edge p1 = exp(logp1):
 *            grad_edge1 = g_parent * (edge_kld + p1), grad_edge2 = -g_parent * p1,
 *            the child receives g_parent * p1; a product edge passes g_parent on.
 *   leaves : queries/kld.jl:528-535 with nodes/fixable_categorical_dist.jl:219
 *            (written exactly as the source has it, which is not the analytic
 *            derivative: grad1_c = g * (p1_c - p2_c + 1), grad2_c = g * exp(p1_c - p2_c)).
 * If analytic != 0 the leaf lines use the true derivatives
 *   grad1_c = g * exp(p1_c) * (p1_c - p2_c + 1), grad2_c = -g * exp(p1_c)
 * (used only to pin the recursion against finite differences).
 * analytic == 2: the leaf arrays hold probabilities (norm_params = true) and the leaf lines are
 * those of nodes/fixable_categorical_dist.jl:216-217, as written:
 *   grad1_c = g * (log(p1_c + 1e-8) - log(p2_c + 1e-8) + 1), grad2_c = g * p1_c / (p2_c + 1e-8).
 */
void orc_kld_backward(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                      const int32_t* prime, const int32_t* sub, const REAL* logp1,
                      const REAL* logp2, const int64_t* in_off, int C, const REAL* leaf1,
                      const REAL* leaf2, const REAL* edge_klds, REAL* grads,
                      REAL* edge_g1, REAL* edge_g2, REAL* leaf_g1, REAL* leaf_g2,
                      int analytic) {
  (void)logp2;
  memset(grads, 0, sizeof(REAL) * (size_t)n_nodes);
  grads[n_nodes - 1] = 1;
  for (int n = n_nodes - 1; n >= 0; --n) {
    REAL g = grads[n];
    if (type[n] == NODE_INPUT) {
      for (int i = 0; i < C; ++i) {
        REAL a = leaf1[in_off[n] + i], b = leaf2[in_off[n] + i];
        if (analytic == 2) {
          leaf_g1[in_off[n] + i] = g * ((REAL)log((double)(a + (REAL)1e-8)) - (REAL)log((double)(b + (REAL)1e-8)) + 1);
          leaf_g2[in_off[n] + i] = g * a / (b + (REAL)1e-8);
        } else if (analytic) {
          leaf_g1[in_off[n] + i] = g * (REAL)exp((double)a) * (a - b + 1);
          leaf_g2[in_off[n] + i] = -g * (REAL)exp((double)a);
        } else {
          leaf_g1[in_off[n] + i] = g * (a - b + 1);
          leaf_g2[in_off[n] + i] = g * (REAL)exp((double)(a - b));
        }
      }
      continue;
    }
    for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
      REAL eg = g;
      if (type[n] == NODE_SUM) {
        REAL p1 = (REAL)exp((double)logp1[e]);
        eg = g * p1;
        edge_g1[e] = g * (edge_klds[e] + p1);
        edge_g2[e] = -g * p1;
      } else {
        edge_g1[e] = 0;
        edge_g2[e] = 0;
      }
      grads[prime[e]] += eg;
      if (sub[e] >= 0) grads[sub[e]] += eg;
    }
  }
}

/*
 * Gumbel-max ancestral sampling with supplied noise: the temperature -> 0 limit of
 * queries/sample.jl:37-51 (u = exp((logp + g)/T), normalised over the sum node's
 * edges) and :105-140 (top-down probability pushed to prime and sub), and of the leaf
 * step :233-260.  A visited sum node keeps the edge maximising logp + g (first maximum
 * wins: strict > scan in edge order); a visited product node visits every edge; a
 * visited leaf emits argmax_c(leaf_logp[c] + g_leaf[c]).
 * Noise indexing: edge_noise[b][e] for sum edge e (dense form), or, when
 * noise_slot != NULL, edge_noise[b][noise_slot[e]] (compact form shared by sum nodes
 * that can never be visited together); leaf_noise[b][var][c].
 * out is [B][V] uint8; variables not reached keep 255.
 */
void orc_sample(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                const int32_t* prime, const int32_t* sub, const REAL* logp,
                const int32_t* in_var, const int64_t* in_off, int C, const REAL* leaf_logp,
                const int64_t* noise_slot, int64_t noise_stride, const REAL* edge_noise,
                const REAL* leaf_noise, int64_t V, int B, uint8_t* out) {
#pragma omp parallel
  {
    uint8_t* visit = (uint8_t*)malloc((size_t)n_nodes);
#pragma omp for schedule(static)
    for (int b = 0; b < B; ++b) {
      memset(visit, 0, (size_t)n_nodes);
      visit[n_nodes - 1] = 1;
      memset(out + (int64_t)b * V, 255, (size_t)V);
      const REAL* en = edge_noise + (int64_t)b * noise_stride;
      for (int n = n_nodes - 1; n >= 0; --n) {
        if (!visit[n]) continue;
        if (type[n] == NODE_INPUT) {
          const REAL* lp = leaf_logp + in_off[n];
          const REAL* g = leaf_noise + ((int64_t)b * V + in_var[n]) * C;
          int best = 0;
          REAL bv = lp[0] + g[0];
          for (int c = 1; c < C; ++c) {
            REAL v = lp[c] + g[c];
            if (v > bv) { bv = v; best = c; }
          }
          out[(int64_t)b * V + in_var[n]] = (uint8_t)best;
        } else if (type[n] == NODE_SUM) {
          int e0 = edge_ptr[n], e1 = edge_ptr[n + 1];
          int best = e0;
          REAL bv = logp[e0] + en[noise_slot ? noise_slot[e0] : e0];
          for (int e = e0 + 1; e < e1; ++e) {
            REAL v = logp[e] + en[noise_slot ? noise_slot[e] : e];
            if (v > bv) { bv = v; best = e; }
          }
          visit[prime[best]] = 1;
          if (sub[best] >= 0) visit[sub[best]] = 1;
        } else {
          for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
            visit[prime[e]] = 1;
            if (sub[e] >= 0) visit[sub[e]] = 1;
          }
        }
      }
    }
    free(visit);
  }
}

/*
 * Soft (Gumbel-softmax) top-down pass with supplied noise, one parameter row:
 * queries/sample.jl:37-51 (unnormalised edge weight exp((logp + g)/T), group sum per
 * sum node), :105-140 (td_prob[child] += td_prob[parent] * w / group_sum; products pass
 * td_prob on to prime and sub) and the categorical leaf step :262-284
 * (out[var][c] += td_prob * exp(leaf_logp[c])).  g may be NULL (no_gumbel = true).
 * norm_params != 0: the leaf array holds probabilities and is added without the exp (:265-268).
 */
void orc_gumbel_soft(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                     const int32_t* prime, const int32_t* sub, const REAL* logp,
                     const int32_t* in_var, const int64_t* in_off, int C,
                     const REAL* leaf_logp, const REAL* g, REAL temperature, int64_t V,
                     REAL* td, REAL* out, int norm_params) {
  memset(td, 0, sizeof(REAL) * (size_t)n_nodes);
  memset(out, 0, sizeof(REAL) * (size_t)(V * C));
  td[n_nodes - 1] = 1;
  for (int n = n_nodes - 1; n >= 0; --n) {
    if (type[n] == NODE_INPUT) {
      for (int c = 0; c < C; ++c)
        out[(int64_t)in_var[n] * C + c] +=
            td[n] * (norm_params ? leaf_logp[in_off[n] + c] : (REAL)exp((double)leaf_logp[in_off[n] + c]));
      continue;
    }
    int e0 = edge_ptr[n], e1 = edge_ptr[n + 1];
    REAL cum = 0;
    if (type[n] == NODE_SUM)
      for (int e = e0; e < e1; ++e)
        cum += (REAL)exp((double)((logp[e] + (g ? g[e] : 0)) / temperature));
    for (int e = e0; e < e1; ++e) {
      REAL p = td[n];
      if (type[n] == NODE_SUM)
        p *= (REAL)exp((double)((logp[e] + (g ? g[e] : 0)) / temperature)) / cum;
      td[prime[e]] += p;
      if (sub[e] >= 0) td[sub[e]] += p;
    }
  }
}

/*
 * Reverse pass of the relaxed sampler, VariationalJuice.jl/src/queries/sample.jl:389-650
 * (gumbel_input_sample_up_kernel :531-598, gumbel_params_up_layer_kernel :391-480,
 * gumbel_sample_backward :620-640), one example.  og[var][c]: gradient of the loss with
 * respect to the soft output of orc_gumbel_soft; td: the top-down probabilities that
 * call left behind.  Nodes are walked children first.
 *   input node (:560-570)  leaf_grad[c] = og[var][c] * td[node]  -- with respect to the
 *       PROBABILITY of category c, with or without norm_params, as the source writes it;
 *       grads[node] = sum_c prob(c) * og[var][c]
 *   sum edge (:421-436)    w = exp((logp + g)/T) / cum;  param_grad = child_grad * td[parent];
 *       cum_grad += param_grad * w;  grads[parent] += child_grad * w
 *       then (:463-470)    edge_grad = (param_grad - cum_grad) * w / T   (grad_wrt_logparams)
 *                                     (param_grad - cum_grad) / T       (otherwise)
 *   product edge           grads[parent] += child_grad
 * with child_grad = grads[prime] (+ grads[sub]).  Product edges get edge_grad 0.
 */
void orc_gumbel_soft_backward(int n_nodes, const uint8_t* type, const int32_t* edge_ptr,
                              const int32_t* prime, const int32_t* sub, const REAL* logp,
                              const int32_t* in_var, const int64_t* in_off, int C,
                              const REAL* leaf_logp, const REAL* g, REAL temperature,
                              const REAL* td, const REAL* og, int norm_params,
                              int grad_wrt_logparams, REAL* grads, REAL* edge_grad,
                              REAL* leaf_grad) {
  for (int n = 0; n < n_nodes; ++n) {
    if (type[n] == NODE_INPUT) {
      REAL acc = 0;
      for (int c = 0; c < C; ++c) {
        REAL o = og[(int64_t)in_var[n] * C + c], x = leaf_logp[in_off[n] + c];
        leaf_grad[in_off[n] + c] = o * td[n];
        acc += (norm_params ? x : (REAL)exp((double)x)) * o;
      }
      grads[n] = acc;
      continue;
    }
    int e0 = edge_ptr[n], e1 = edge_ptr[n + 1];
    REAL acc = 0;
    if (type[n] != NODE_SUM) {
      for (int e = e0; e < e1; ++e) {
        acc += grads[prime[e]] + (sub[e] >= 0 ? grads[sub[e]] : 0);
        edge_grad[e] = 0;
      }
      grads[n] = acc;
      continue;
    }
    REAL cum = 0, cum_grad = 0;
    for (int e = e0; e < e1; ++e)
      cum += (REAL)exp((double)((logp[e] + (g ? g[e] : 0)) / temperature));
    for (int e = e0; e < e1; ++e) {
      REAL w = (REAL)exp((double)((logp[e] + (g ? g[e] : 0)) / temperature)) / cum;
      REAL child = grads[prime[e]] + (sub[e] >= 0 ? grads[sub[e]] : 0);
      REAL pg = child * td[n];
      edge_grad[e] = pg;
      cum_grad += pg * w;
      acc += child * w;
    }
    for (int e = e0; e < e1; ++e) {
      REAL w = (REAL)exp((double)((logp[e] + (g ? g[e] : 0)) / temperature)) / cum;
      edge_grad[e] = grad_wrt_logparams ? (edge_grad[e] - cum_grad) * w / temperature
                                        : (edge_grad[e] - cum_grad) / temperature;
    }
    grads[n] = acc;
  }
}

/*
 * Adam ascent step on unnormalised log-parameters, then per-sum-node normalisation
 * into the circuit's log-parameters, as the reference's training loop does it:
 *   sgd/adam.jl:318-319  m = b1*m + (1-b1)*g ; v = b2*v + (1-b2)*g^2
 *   sgd/adam.jl:63-76    mhat = m/(1-b1^t), vhat = v/(1-b2^t),
 *                        params += lr * mhat / (sqrt(vhat) + eps)   (ascent)
 *   sgd/adam.jl:88-127   node_aggr = sum exp(params) over the sum node's edges,
 *                        logp = params - log(node_aggr); `params` itself stays
 *                        unnormalised; a sum node with a single edge keeps its logp.
 * group_ptr delimits the sum nodes over the parameter vector; logp_out receives the
 * normalised values.
 */
void orc_adam_step(int64_t n, REAL* params, const REAL* grad, REAL* m, REAL* v, REAL lr,
                   REAL b1, REAL b2, REAL eps, int t, int n_groups, const int64_t* group_ptr,
                   REAL* logp_out) {
  REAL c1 = (REAL)1 - (REAL)pow((double)b1, (double)t);
  REAL c2 = (REAL)1 - (REAL)pow((double)b2, (double)t);
  for (int64_t i = 0; i < n; ++i) {
    m[i] = b1 * m[i] + ((REAL)1 - b1) * grad[i];
    v[i] = b2 * v[i] + ((REAL)1 - b2) * grad[i] * grad[i];
    REAL mh = m[i] / c1, vh = v[i] / c2;
    params[i] += lr * (mh / ((REAL)sqrt((double)vh) + eps));
  }
  for (int gi = 0; gi < n_groups; ++gi) {
    int64_t i0 = group_ptr[gi], i1 = group_ptr[gi + 1];
    if (i1 - i0 == 1) continue;
    REAL s = 0;
    for (int64_t i = i0; i < i1; ++i) s += (REAL)exp((double)params[i]);
    REAL l = (REAL)log((double)s);
    for (int64_t i = i0; i < i1; ++i) logp_out[i] = params[i] - l;
  }
}

/*
 * Gradient of the mean log-likelihood with respect to the unnormalised log-parameters of the sum
 * edges, from the accumulated edge flows: sgd/adam.jl:305-311 (edge_aggr ./= batch_size) and :27-61
 * (`compute_gradients`: node_aggr[parent] = sum of the parent's edge flows, then
 * edge_aggr[e] -= exp(logp_e) * node_aggr[parent]).  Product edges are left as they are.
 * edge_aggr is [n_edges] in CSR order and is overwritten with the gradient.
 */
void orc_flow_gradients(int n_nodes, const uint8_t* type, const int32_t* edge_ptr, const REAL* logp,
                        REAL* edge_aggr, REAL batch_size) {
  for (int n = 0; n < n_nodes; ++n) {
    if (type[n] != NODE_SUM) continue;
    REAL node_aggr = 0;
    for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e) {
      edge_aggr[e] /= batch_size;
      node_aggr += edge_aggr[e];
    }
    for (int e = edge_ptr[n]; e < edge_ptr[n + 1]; ++e)
      edge_aggr[e] -= (REAL)exp((double)logp[e]) * node_aggr;
  }
}

/*
 * Adam on the input nodes as sgd/adam.jl:218-242 writes it (`update_params_adam` of a categorical
 * leaf), one call per input node with its C log-probabilities `lp` (read only: the source never
 * writes the stepped values back into the circuit), its C flows, and its slice of the auxiliary
 * heap: aux_p (a copy of the parameters that takes the steps), aux_m, aux_v.
 *   node_flow = sum_i flow_i;  g_i = flow_i + exp(lp_i) * node_flow   (the sign is the source's)
 *   m = b1*m + (1-b1)*g;  v = b2*v + (1-b2)*g^2;  aux_p += lr * (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps)
 */
void orc_leaf_adam(int64_t n_inputs, int C, const REAL* leaf_logp, const REAL* leaf_flow, REAL* aux_p,
                   REAL* aux_m, REAL* aux_v, REAL lr, REAL b1, REAL b2, REAL eps, int t) {
  REAL c1 = (REAL)1 - (REAL)pow((double)b1, (double)t);
  REAL c2 = (REAL)1 - (REAL)pow((double)b2, (double)t);
  for (int64_t q = 0; q < n_inputs; ++q) {
    const REAL* lp = leaf_logp + q * C;
    const REAL* fl = leaf_flow + q * C;
    REAL node_flow = 0;
    for (int i = 0; i < C; ++i) node_flow += fl[i];
    for (int i = 0; i < C; ++i) {
      REAL p = (REAL)exp((double)lp[i]);
      REAL g = fl[i] + p * node_flow;
      REAL m = b1 * aux_m[q * C + i] + ((REAL)1 - b1) * g;
      REAL v = b2 * aux_v[q * C + i] + ((REAL)1 - b2) * g * g;
      aux_m[q * C + i] = m;
      aux_v[q * C + i] = v;
      aux_p[q * C + i] += lr * ((m / c1) / ((REAL)sqrt((double)(v / c2)) + eps));
    }
  }
}

int orc_real_size(void) { return (int)sizeof(REAL); }
int orc_max_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}
