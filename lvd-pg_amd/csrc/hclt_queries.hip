// KL recursion, Gumbel-max sampling and Adam for HCLT circuits.  These queries have no batch
// of examples to slice (KL: one parameter row; sampling: a top-down choice per example), so
// they run on the general engine over the circuit's general form; parameters are exchanged
// in parameter-vector order, which both forms share.
#include "hclt_engine.hpp"

namespace pcm {

SparseCircuit* HcltCircuit::general() {
  if (!general_) {
    general_.reset(new SparseCircuit(flat_));
    general_->stream = stream;
    general_stale_ = true;
  }
  general_->stream = stream;
  if (general_stale_) {
    std::vector<float> p((size_t)size(0));
    vectorize(p.data(), (int64_t)p.size());
    general_->update_parameters(p.data(), (int64_t)p.size());
    general_stale_ = false;
  }
  return general_.get();
}

void HcltCircuit::pull_from_general() {
  std::vector<float> p((size_t)size(0));
  general_->vectorize(p.data(), (int64_t)p.size());
  update_parameters(p.data(), (int64_t)p.size());
  general_stale_ = false;
}

static HcltCircuit* as_hclt(pcm_circuit* q) {
  auto* h = dynamic_cast<HcltCircuit*>(q);
  if (!h) fail(PCM_ERR_ARG, "the two circuits of a KL query must be of the same kind");
  return h;
}

void HcltCircuit::kld(pcm_circuit* q, float* out) { general()->kld(as_hclt(q)->general(), out); }

void HcltCircuit::kld_backward(pcm_circuit* q, float* gp, float* gq, int64_t n) {
  general()->kld_backward(as_hclt(q)->general(), gp, gq, n);
}

void HcltCircuit::sample(const float* d_node_noise, const float* d_leaf_noise, int32_t batch, uint8_t* d_out) {
  SparseCircuit* g = general();
  DevBuf<int32_t> slots;
  slots.upload(noise_slot_, stream);
  g->sample_with_slots(d_node_noise, slots.p, sample_noise_size(), d_leaf_noise, batch, d_out);
}

void HcltCircuit::sample_soft(const float* d_node_noise, float temperature, int32_t batch, float* d_out) {
  SparseCircuit* g = general();
  DevBuf<int32_t> slots;
  slots.upload(noise_slot_, stream);
  g->sample_soft_with_slots(d_node_noise, slots.p, sample_noise_size(), temperature, batch, d_out);
}

void HcltCircuit::adam_step(const float* d_grad, float* d_params, float* d_m, float* d_v, float lr, float b1,
                            float b2, float eps, int t) {
  general()->adam_step(d_grad, d_params, d_m, d_v, lr, b1, b2, eps, t);
  PCM_HIP(hipStreamSynchronize(stream));
  pull_from_general();
}

}  // namespace pcm
