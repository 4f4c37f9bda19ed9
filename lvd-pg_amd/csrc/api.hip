// C ABI of pcmi355: argument checks, exception -> status translation.
#include <algorithm>
#include <mutex>
#include <new>
#include <unordered_set>

#include "common.hpp"
#include "hclt_engine.hpp"
#include "sparse_engine.hpp"

namespace {
thread_local std::string g_last_error;

template <typename F>
int guarded(F&& f) {
  try {
    f();
    return PCM_OK;
  } catch (const pcm::Error& e) {
    g_last_error = e.what();
    return e.status;
  } catch (const std::bad_alloc&) {
    g_last_error = "out of host memory";
    return PCM_ERR_ARG;
  } catch (const std::exception& e) {
    g_last_error = e.what();
    return PCM_ERR_ARG;
  }
}

// Every handle the library has given out and not yet freed.  A call with any other pointer (freed
// twice, never created here) is turned down before it is dereferenced.
std::mutex g_handles_mu;
std::unordered_set<const pcm_circuit*> g_handles;

void adopt(pcm_circuit* c) {
  std::lock_guard<std::mutex> lock(g_handles_mu);
  g_handles.insert(c);
}

pcm_circuit* need(pcm_circuit* c) {
  if (!c) pcm::fail(PCM_ERR_ARG, "circuit handle is null");
  std::lock_guard<std::mutex> lock(g_handles_mu);
  if (!g_handles.count(c)) pcm::fail(PCM_ERR_ARG, "not a live circuit handle (already freed, or not created by this library)");
  return c;
}

pcm_circuit* release(pcm_circuit* c) {
  if (!c) pcm::fail(PCM_ERR_ARG, "circuit handle is null");
  std::lock_guard<std::mutex> lock(g_handles_mu);
  if (!g_handles.erase(c)) pcm::fail(PCM_ERR_ARG, "not a live circuit handle (already freed, or not created by this library)");
  return c;
}

pcm::HcltCircuit* need_hclt(pcm_circuit* c) {
  auto* h = dynamic_cast<pcm::HcltCircuit*>(need(c));
  if (!h) pcm::fail(PCM_ERR_ARG, "circuit was not created by pcm_hclt_create");
  return h;
}

pcm::BatchRef batch_ref(const uint8_t* d, int64_t se, int64_t sv, const int32_t* idx, int32_t b) {
  return pcm::BatchRef{d, se, sv, idx, b};
}
}  // namespace

extern "C" {

const char* pcm_last_error(void) { return g_last_error.c_str(); }
int pcm_version(void) { return 1; }

int pcm_hclt_create(const int32_t* clt_parent, int32_t num_vars, int32_t num_hidden_cats, int32_t num_cats,
                    pcm_circuit** out) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    *out = nullptr;
    adopt(*out = new pcm::HcltCircuit(clt_parent, num_vars, num_hidden_cats, num_cats));
  });
}

int pcm_hclt_create_multihead(const int32_t* clt_parent, int32_t num_vars, int32_t num_hidden_cats, int32_t num_cats,
                              int32_t num_heads, pcm_circuit** out) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    *out = nullptr;
    if (num_heads < 1) pcm::fail(PCM_ERR_SHAPE, "num_heads must be positive, got %d", num_heads);
    adopt(*out = new pcm::HcltCircuit(clt_parent, num_vars, num_hidden_cats, num_cats, num_heads));
  });
}

int pcm_circuit_create(int32_t num_nodes, const uint8_t* node_type, const int32_t* child_ptr,
                       const int32_t* child_idx, const float* sum_logp, const int32_t* input_var,
                       const float* input_logp, int32_t num_vars, int32_t num_cats, int32_t num_heads,
                       pcm_circuit** out) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    *out = nullptr;
    adopt(*out = new pcm::SparseCircuit(pcm::flatten_dag(num_nodes, node_type, child_ptr, child_idx, sum_logp, input_var,
                                                         input_logp, num_vars, num_cats, num_heads)));
  });
}

int pcm_free(pcm_circuit* c) {
  return guarded([&] { delete release(c); });
}

int pcm_set_stream(pcm_circuit* c, void* s) {
  return guarded([&] { need(c)->stream = reinterpret_cast<hipStream_t>(s); });
}

int64_t pcm_size(const pcm_circuit* c, int32_t what) {
  int64_t r = -1;
  guarded([&] { r = need(const_cast<pcm_circuit*>(c))->size(what); });
  return r;
}

int pcm_index_table(const pcm_circuit* c, int32_t which, int64_t* out, int64_t n) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    need(const_cast<pcm_circuit*>(c))->index_table(which, out, n);
  });
}

int pcm_vectorize_parameters(pcm_circuit* c, float* out, int64_t n) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    need(c)->vectorize(out, n);
  });
}

int pcm_update_parameters(pcm_circuit* c, const float* p, int64_t n) {
  return guarded([&] {
    if (!p) pcm::fail(PCM_ERR_ARG, "params is null");
    need(c)->update_parameters(p, n);
  });
}

int pcm_hclt_create_forest(const int32_t* clt_parent, int32_t num_vars, int32_t num_hidden_cats, int32_t num_cats,
                           int32_t num_heads, pcm_circuit** out) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    *out = nullptr;
    if (num_heads < 1) pcm::fail(PCM_ERR_SHAPE, "num_heads must be positive, got %d", num_heads);
    adopt(*out = new pcm::HcltCircuit(clt_parent, num_vars, num_hidden_cats, num_cats, num_heads, true));
  });
}

int pcm_hclt_set_heads(pcm_circuit* c, const float* heads) {
  return guarded([&] { need_hclt(c)->set_heads(heads); });
}
int pcm_hclt_get_heads(pcm_circuit* c, float* heads) {
  return guarded([&] { need_hclt(c)->get_heads(heads); });
}

int pcm_set_missing_category(pcm_circuit* c, int32_t on) {
  return guarded([&] { need_hclt(c)->set_missing_category(on != 0); });
}

int pcm_set_soft_reg(pcm_circuit* c, float soft_reg, int32_t soft_reg_width, int32_t as_written) {
  return guarded([&] { need_hclt(c)->set_soft_reg(soft_reg, soft_reg_width, as_written != 0); });
}

int pcm_set_flow_scale(pcm_circuit* c, float fscale) {
  return guarded([&] {
    pcm_circuit* h = need(c);
    if (!(fscale > 0.f) || !std::isfinite(fscale)) pcm::fail(PCM_ERR_ARG, "fscale must be positive and finite, got %g", (double)fscale);
    if (auto* hc = dynamic_cast<pcm::HcltCircuit*>(h)) hc->check_flow_scale(fscale);
    h->flow_scale = fscale;
  });
}

int pcm_hclt_set_params(pcm_circuit* c, const float* theta, const float* leaf) {
  return guarded([&] { need_hclt(c)->set_block_params(theta, leaf); });
}
int pcm_hclt_get_params(pcm_circuit* c, float* theta, float* leaf) {
  return guarded([&] { need_hclt(c)->get_block_params(theta, leaf); });
}
int pcm_hclt_get_flows(pcm_circuit* c, float* edge_aggr, float* leaf_flow) {
  return guarded([&] { need_hclt(c)->get_block_flows(edge_aggr, leaf_flow); });
}

int pcm_loglikelihoods(pcm_circuit* c, const uint8_t* d_data, int64_t se, int64_t sv, const int32_t* idx,
                       int32_t batch, float* d_ll) {
  return guarded([&] { need(c)->loglikelihoods(batch_ref(d_data, se, sv, idx, batch), d_ll); });
}

int pcm_flows(pcm_circuit* c, const uint8_t* d_data, int64_t se, int64_t sv, const int32_t* idx, int32_t batch,
              float rate, const float* d_head_mask, float* d_ll) {
  return guarded([&] { need(c)->flows(batch_ref(d_data, se, sv, idx, batch), rate, d_head_mask, d_ll); });
}

int pcm_em_update(pcm_circuit* c, float pseudocount, float inertia) {
  return guarded([&] { need(c)->em_update(pseudocount, inertia); });
}

int pcm_em_step(pcm_circuit* c, const uint8_t* d_data, int64_t se, int64_t sv, const int32_t* idx, int32_t batch,
                float rate, float pseudocount, float inertia, float* d_ll) {
  return guarded([&] {
    need(c)->flows(batch_ref(d_data, se, sv, idx, batch), rate, nullptr, d_ll);
    c->em_update(pseudocount, inertia);
  });
}

int pcm_get_node_values(pcm_circuit* c, float* mars, float* flows, int64_t n) {
  return guarded([&] {
    auto* s = dynamic_cast<pcm::SparseCircuit*>(need(c));
    if (!s) pcm::fail(PCM_ERR_UNSUPPORTED, "node values are kept only by circuits from pcm_circuit_create");
    s->get_node_values(mars, flows, n);
  });
}
int pcm_node_flow_sums(pcm_circuit* c, float* out, int64_t n) {
  return guarded([&] {
    auto* s = dynamic_cast<pcm::SparseCircuit*>(need(c));
    if (!s) pcm::fail(PCM_ERR_UNSUPPORTED, "node flows exist only for circuits built from a description (pcm_circuit_create)");
    s->node_flow_sums(out, n);
  });
}

int pcm_get_aggregates(pcm_circuit* c, float* edge_aggr, int64_t n_edges, float* leaf_flow, int64_t n_leaf) {
  return guarded([&] {
    auto* s = dynamic_cast<pcm::SparseCircuit*>(need(c));
    if (!s) pcm::fail(PCM_ERR_UNSUPPORTED, "use pcm_hclt_get_flows on an HCLT circuit");
    s->get_aggregates(edge_aggr, n_edges, leaf_flow, n_leaf);
  });
}

int pcm_kld(pcm_circuit* p, pcm_circuit* q, float* out) {
  return guarded([&] {
    if (!out) pcm::fail(PCM_ERR_ARG, "out is null");
    need(q);
    need(p)->kld(q, out);
  });
}
int pcm_kld_backward(pcm_circuit* p, pcm_circuit* q, float* gp, float* gq, int64_t n) {
  return guarded([&] {
    need(q);
    need(p)->kld_backward(q, gp, gq, n);
  });
}

int pcm_kld_backward_dev(pcm_circuit* p, pcm_circuit* q, float* d_grad_p, float* d_grad_q, int64_t n) {
  return guarded([&] { need(p)->kld_backward_dev(need(q), d_grad_p, d_grad_q, n); });
}

int64_t pcm_sample_noise_size(const pcm_circuit* c) {
  int64_t r = -1;
  guarded([&] { r = need(const_cast<pcm_circuit*>(c))->sample_noise_size(); });
  return r;
}
int pcm_sample(pcm_circuit* c, const float* d_node_noise, const float* d_leaf_noise, int32_t batch, uint8_t* d_out) {
  return guarded([&] { need(c)->sample(d_node_noise, d_leaf_noise, batch, d_out); });
}

int pcm_sample_soft(pcm_circuit* c, const float* d_node_noise, float temperature, int32_t batch, float* d_out) {
  return guarded([&] { need(c)->sample_soft(d_node_noise, temperature, batch, d_out); });
}

int pcm_adam_step(pcm_circuit* c, const float* d_grad, float* d_params, float* d_m, float* d_v, float lr,
                  float b1, float b2, float eps, int32_t t) {
  return guarded([&] { need(c)->adam_step(d_grad, d_params, d_m, d_v, lr, b1, b2, eps, t); });
}

int pcm_flow_gradients(pcm_circuit* c, int32_t batch_size, float* d_grad) {
  return guarded([&] { need(c)->flow_gradients(batch_size, d_grad); });
}

int pcm_adam_flow_step(pcm_circuit* c, int32_t batch_size, float* d_params, float* d_m, float* d_v, float* d_leaf_params,
                       float* d_leaf_m, float* d_leaf_v, float lr, float b1, float b2, float eps, int32_t t) {
  return guarded([&] {
    if (!d_params || !d_m || !d_v) pcm::fail(PCM_ERR_ARG, "null optimiser array");
    const int64_t ns = need(c)->size(1);
    // the gradient takes the place the reference gives it: edge_aggr itself (src/sgd/adam.jl:305-319)
    pcm::DevBuf<float> grad;
    grad.alloc((size_t)std::max<int64_t>(ns, 1));
    c->flow_gradients(batch_size, grad.p);
    if (d_leaf_params) c->leaf_adam(d_leaf_params, d_leaf_m, d_leaf_v, lr, b1, b2, eps, t);   // reads the leaves before the sum step, as :319-325
    c->adam_step(grad.p, d_params, d_m, d_v, lr, b1, b2, eps, t);
    PCM_HIP(hipStreamSynchronize(c->stream));
  });
}

int pcm_kld_rows(pcm_circuit* c, const float* d_params1, const float* d_params2, int64_t stride_row, int64_t stride_param,
                 int32_t rows, int32_t norm_params, float* d_klds) {
  return guarded([&] { need(c)->kld_rows(d_params1, d_params2, stride_row, stride_param, rows, norm_params != 0, d_klds); });
}

int pcm_kld_backward_rows(pcm_circuit* c, const float* d_params1, const float* d_params2, int64_t stride_row,
                          int64_t stride_param, int32_t rows, int32_t norm_params, float* d_grads1, float* d_grads2,
                          float* d_klds) {
  return guarded([&] {
    need(c)->kld_backward_rows(d_params1, d_params2, stride_row, stride_param, rows, norm_params != 0, d_grads1, d_grads2,
                               d_klds);
  });
}

int pcm_gumbel_sample_rows(pcm_circuit* c, const float* d_params, int64_t stride_row, int64_t stride_param, int32_t rows,
                           const float* d_noise, float temperature, int32_t norm_params, float* d_out) {
  return guarded([&] {
    need(c)->gumbel_sample_rows(d_params, stride_row, stride_param, rows, d_noise, temperature, norm_params != 0, d_out);
  });
}

int pcm_gumbel_sample_backward_rows(pcm_circuit* c, const float* d_params, int64_t stride_row, int64_t stride_param,
                                    int32_t rows, const float* d_noise, float temperature, int32_t norm_params,
                                    int32_t grad_wrt_logparams, const float* d_out_grads, float* d_param_grads) {
  return guarded([&] {
    need(c)->gumbel_sample_backward_rows(d_params, stride_row, stride_param, rows, d_noise, temperature, norm_params != 0,
                                         grad_wrt_logparams != 0, d_out_grads, d_param_grads);
  });
}

int pcm_normalized_flows(pcm_circuit* c, const uint8_t* d_data, int64_t se, int64_t sv, const int32_t* idx, int32_t batch,
                         int32_t as_written, float* d_out, int64_t stride_row, int64_t stride_param) {
  return guarded([&] {
    need(c)->normalized_flows(batch_ref(d_data, se, sv, idx, batch), d_out, stride_row, stride_param, as_written != 0);
  });
}

int pcm_normalize_params_rows(pcm_circuit* c, float* d_params, int64_t stride_row, int64_t stride_param, int32_t rows,
                              int32_t undo) {
  return guarded([&] { need(c)->normalize_params_rows(d_params, stride_row, stride_param, rows, undo != 0); });
}

int pcm_loglikelihoods_soft(pcm_circuit* c, const float* d_evidence, int64_t stride_ex, int64_t stride_var,
                            int64_t stride_cat, const int32_t* d_example_ids, int32_t batch, float* d_ll) {
  return guarded([&] {
    need(c)->loglikelihoods_soft(pcm::SoftRef{d_evidence, stride_ex, stride_var, stride_cat, d_example_ids, batch}, d_ll);
  });
}

int pcm_flows_soft(pcm_circuit* c, const float* d_evidence, int64_t stride_ex, int64_t stride_var, int64_t stride_cat,
                   const int32_t* d_example_ids, int32_t batch, float rate, const float* d_head_mask, float* d_ll) {
  return guarded([&] {
    need(c)->flows_soft(pcm::SoftRef{d_evidence, stride_ex, stride_var, stride_cat, d_example_ids, batch}, rate,
                        d_head_mask, d_ll);
  });
}

int pcm_pairwise_mi(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t num_examples,
                    int32_t num_vars, int32_t num_cats, float pseudocount, float* d_mi, void* stream) {
  return guarded([&] {
    pcm::pairwise_mi(d_data, stride_ex, stride_var, num_examples, num_vars, num_cats, pseudocount, d_mi,
                     static_cast<hipStream_t>(stream));
  });
}

int pcm_pairwise_mi_static(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t num_examples,
                           int32_t num_vars, int32_t num_cats, float pseudocount, float* d_mi, void* stream) {
  return guarded([&] {
    pcm::pairwise_mi_static(d_data, stride_ex, stride_var, num_examples, num_vars, num_cats, pseudocount, d_mi,
                            static_cast<hipStream_t>(stream));
  });
}

int pcm_chow_liu_tree(const float* mi, int32_t num_vars, int32_t* clt_parent) {
  return guarded([&] { pcm::chow_liu_tree(mi, num_vars, clt_parent); });
}

int pcm_stream_probe(const void* d_src, void* d_dst, int64_t lanes, int32_t reads, int32_t writes, int32_t grid, void* stream) {
  return guarded([&] { pcm::stream_probe(d_src, d_dst, lanes, reads, writes, grid, static_cast<hipStream_t>(stream)); });
}

int pcm_set_timing(pcm_circuit* c, int32_t on) {
  return guarded([&] {
    if (on < 0 || on > 15) pcm::fail(PCM_ERR_ARG, "timing mode %d outside 0..15", on);
    need_hclt(c)->set_timing(on == 1 ? 7 : on >> 1);
  });
}
int pcm_get_timing(pcm_circuit* c, float* ms, int32_t n) {
  return guarded([&] {
    if (!ms || n < 0 || n > 4) pcm::fail(PCM_ERR_ARG, "ms is null or n outside 0..4");
    need_hclt(c)->read_timing(ms, n);
  });
}

}  // extern "C"
