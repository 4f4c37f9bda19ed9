// pcm_pairwise_mi_static: pairwise mutual information for callers that cannot allocate device
// memory (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The same
// kernels as pcm_pairwise_mi (chow_liu.hip); their working memory is a fixed array of this code object.
#include "chow_liu.hpp"

#include <mutex>

namespace pcm {

// Its working memory is one array in the code object, so every device the library runs on holds
// kMiStaticBytes of it until the process ends.  Layout: staged categories | stat | g.
constexpr size_t kMiStaticStage = 16u << 20;                      // num_vars * ceil64(num_examples) bytes
constexpr int kMiStaticVars = 4096;                                // stat: 2 doubles per variable
constexpr int kMiStaticExamples = 65535;                           // g: one 64-bit integer per count
constexpr size_t kMiStaticStatOff = kMiStaticStage;
constexpr size_t kMiStaticGOff = kMiStaticStatOff + (size_t)kMiStaticVars * 2 * sizeof(double);
constexpr size_t kMiStaticBytes = kMiStaticGOff + ((size_t)kMiStaticExamples + 1) * sizeof(long long);

static __device__ __align__(256) unsigned char scratch[kMiStaticBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char* g_scratch_ptr[kMaxDevices] = {};

// The array's address on the current device (`scratch` itself is only a host-side stand-in for it).
unsigned char* mi_static_scratch() {
  int dev = 0;
  PCM_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) fail(PCM_ERR_UNSUPPORTED, "device ordinal %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    PCM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) fail(PCM_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
    g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
  }
  return g_scratch_ptr[dev];
}
}  // namespace

void pairwise_mi_static(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t n_examples, int num_vars,
                        int num_cats, float pseudocount, float* d_mi, hipStream_t stream) {
  const MiShape sh = mi_check(d_data, n_examples, num_vars, num_cats, pseudocount, d_mi);
  if (sh.N > kMiStaticExamples)
    fail(PCM_ERR_UNSUPPORTED, "pcm_pairwise_mi_static takes at most %d examples, got %d (use pcm_pairwise_mi)",
         kMiStaticExamples, sh.N);
  if (sh.V > kMiStaticVars)
    fail(PCM_ERR_UNSUPPORTED, "pcm_pairwise_mi_static takes at most %d variables, got %d (use pcm_pairwise_mi)",
         kMiStaticVars, sh.V);
  if ((size_t)sh.V * (size_t)sh.Np > kMiStaticStage)
    fail(PCM_ERR_UNSUPPORTED,
         "pcm_pairwise_mi_static stages num_vars * ceil64(num_examples) = %zu bytes, its static buffer holds %zu "
         "(use pcm_pairwise_mi)", (size_t)sh.V * (size_t)sh.Np, kMiStaticStage);
  unsigned char* base = mi_static_scratch();
  // every byte the kernels read from the array is written earlier in the same call: nothing to clear
  const MiScratch w{base, reinterpret_cast<double*>(base + kMiStaticStatOff), reinterpret_cast<long long*>(base + kMiStaticGOff)};
  mi_launch(d_data, stride_ex, stride_var, sh, pseudocount, w, d_mi, stream);
}

}  // namespace pcm
