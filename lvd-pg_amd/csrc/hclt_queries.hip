// KL recursion, Gumbel-max sampling and Adam on the dense-block HCLT engine.
#include "hclt_engine.hpp"

namespace pcm {

void HcltCircuit::kld(pcm_circuit*, float*) { fail(PCM_ERR_UNSUPPORTED, "kld: not built yet"); }
void HcltCircuit::kld_backward(pcm_circuit*, float*, float*, int64_t) {
  fail(PCM_ERR_UNSUPPORTED, "kld_backward: not built yet");
}
void HcltCircuit::sample(const float*, const float*, int32_t, uint8_t*) {
  fail(PCM_ERR_UNSUPPORTED, "sample: not built yet");
}
void HcltCircuit::adam_step(const float*, float*, float*, float*, float, float, float, float, int) {
  fail(PCM_ERR_UNSUPPORTED, "adam_step: not built yet");
}

}  // namespace pcm
