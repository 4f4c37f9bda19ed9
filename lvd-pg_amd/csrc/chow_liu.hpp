// Internal interface of the pairwise mutual-information kernels (chow_liu.hip).
#pragma once

#include "common.hpp"

namespace pcm {

// Device memory the pair kernels need beyond their input and output.
struct MiScratch {
  uint8_t* xb;     // [V][Np] staged categories
  double* stat;    // [V][2]
  long long* g;    // [N + 1] the count table (fixed point)
};

struct MiShape {
  int N, V, C;
  int64_t Np;
};

// Argument checks shared by the entry points; throws pcm::Error.
MiShape mi_check(const uint8_t* d_data, int64_t n_examples, int num_vars, int num_cats, float pseudocount, const float* d_mi);

// Queues staging, marginals, the count table and the pair kernel on `stream`; allocates nothing and
// does not wait.  w.xb holds V * Np bytes, w.stat 2 * V doubles, w.g N + 1 64-bit integers.
void mi_launch(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, const MiShape& sh, float pseudocount,
               const MiScratch& w, float* d_mi, hipStream_t stream);

}  // namespace pcm
