// Shared host-side plumbing of the pcmi355 library: error reporting, device buffers,
// and the abstract engine every compiled circuit implements.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/pcmi355.h"

namespace pcm {

// Error carried from anywhere below the C ABI to the entry point that reports it.
struct Error : std::runtime_error {
  int status;
  Error(int s, const std::string& m) : std::runtime_error(m), status(s) {}
};

[[noreturn]] inline void fail(int status, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  throw Error(status, buf);
}

#define PCM_HIP(expr)                                                                   \
  do {                                                                                  \
    hipError_t e__ = (expr);                                                            \
    if (e__ != hipSuccess)                                                              \
      ::pcm::fail(PCM_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__),  \
                  __FILE__, __LINE__);                                                  \
  } while (0)

// Owning device array.
template <typename T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  DevBuf() = default;
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  ~DevBuf() { release(); }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    n = 0;
  }
  void alloc(size_t count) {
    release();
    if (count) PCM_HIP(hipMalloc((void**)&p, count * sizeof(T)));
    n = count;
  }
  void ensure(size_t count) {
    if (count > n) alloc(count);
  }
  void upload(const std::vector<T>& h, hipStream_t s = nullptr) {
    alloc(h.size());
    if (!h.empty()) {
      PCM_HIP(hipMemcpyAsync(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice, s));
      PCM_HIP(hipStreamSynchronize(s));
    }
  }
  // On a stream of the caller's the clear is queued like any other work; without one (set-up code) it has
  // finished when the call returns, so work queued later on any stream finds the memory cleared.
  void zero(hipStream_t s = nullptr) {
    if (!n) return;
    PCM_HIP(hipMemsetAsync(p, 0, n * sizeof(T), s));
    if (!s) PCM_HIP(hipStreamSynchronize(nullptr));
  }
};

// dst[i] = keep * dst[i] + w(i) * (part[0][i] + part[1][i] + ...); w(i) = exp(logw[i]) or 1; keep < 0 stands for
// keep = 1 (plain accumulation), keep = 0 never reads dst.  Kernels that share one sum out
// among workgroups leave their parts in rows of `part` and this kernel puts them together: no atomics, the same
// bits on every run.  A workgroup takes 64 elements; its four waves each add up every fourth row in order, and
// the four subtotals are added in order too (the order is fixed, just not row after row).
template <bool kExpWeight>
__global__ __launch_bounds__(256) void sum_parts_kernel(const float* __restrict__ part, int n_parts, int64_t n,
                                                        const float* __restrict__ logw, float* __restrict__ dst,
                                                        float keep = -1.f) {
  __shared__ float sub[4][64];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int64_t i = (int64_t)blockIdx.x * 64 + lane;
  // blockIdx.y: one of several independent sums laid out one behind the other (the trees of a forest)
  part += (size_t)blockIdx.y * n_parts * n;
  dst += (size_t)blockIdx.y * n;
  if (kExpWeight) logw += (size_t)blockIdx.y * n;
  float s = 0.f;
  if (i < n)
    for (int q = g; q < n_parts; q += 4) s += part[(size_t)q * n + i];
  sub[g][lane] = s;
  __syncthreads();
  if (g == 0 && i < n) {
    s = ((sub[0][lane] + sub[1][lane]) + sub[2][lane]) + sub[3][lane];
    const float old = keep < 0.f ? dst[i] : keep != 0.f ? keep * dst[i] : 0.f;
    dst[i] = old + (kExpWeight ? __expf(logw[i]) * s : s);
  }
}

// A batch of soft evidence: log-evidence per (example, variable, category) with element strides.
struct SoftRef {
  const float* d_ev;
  int64_t stride_ex, stride_var, stride_cat;
  const int32_t* d_idx;
  int32_t batch;
};

inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

struct BatchRef {
  const uint8_t* d_data;
  int64_t stride_ex, stride_var;
  const int32_t* d_idx;
  int32_t batch;
};

// structure learning (chow_liu.hip)
void pairwise_mi(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t n_examples, int num_vars,
                 int num_cats, float pseudocount, float* d_mi, hipStream_t stream);
void stream_probe(const void* d_src, void* d_dst, int64_t lanes, int reads, int writes, int grid, hipStream_t stream);
void pairwise_mi_static(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t n_examples, int num_vars,
                        int num_cats, float pseudocount, float* d_mi, hipStream_t stream);
void chow_liu_tree(const float* mi, int num_vars, int32_t* parent_out);

}  // namespace pcm

// The opaque handle of the C ABI.
struct pcm_circuit {
  hipStream_t stream = nullptr;
  // fscale of mini_batch_em_beta (src-jl/learning/em.jl:293, flow.jl:120-370): flows that feed the accumulators hand
  // a sum node's flow down in shares proportional to (posterior share)^(1 / flow_scale); 1: the ordinary flows
  float flow_scale = 1.f;
  virtual ~pcm_circuit() {}
  virtual int64_t size(int what) const = 0;
  virtual void index_table(int which, int64_t* out, int64_t n) const = 0;
  virtual void vectorize(float* out, int64_t n) = 0;
  virtual void update_parameters(const float* in, int64_t n) = 0;
  virtual void loglikelihoods(const pcm::BatchRef& b, float* d_ll) = 0;
  virtual void flows(const pcm::BatchRef& b, float rate, const float* d_head_mask, float* d_ll) = 0;
  virtual void loglikelihoods_soft(const pcm::SoftRef& s, float* d_ll) = 0;
  virtual void flows_soft(const pcm::SoftRef& s, float rate, const float* d_head_mask, float* d_ll) = 0;
  virtual void em_update(float pseudocount, float inertia) = 0;
  virtual void kld(pcm_circuit* q, float* out) = 0;
  virtual void kld_backward(pcm_circuit* q, float* gp, float* gq, int64_t n) = 0;
  virtual void kld_backward_dev(pcm_circuit* q, float* d_gp, float* d_gq, int64_t n) = 0;
  virtual int64_t sample_noise_size() const = 0;
  virtual void sample(const float* d_node_noise, const float* d_leaf_noise, int32_t batch,
                      uint8_t* d_out) = 0;
  virtual void sample_soft(const float* d_node_noise, float temperature, int32_t batch, float* d_out) = 0;
  virtual void adam_step(const float* d_grad, float* d_params, float* d_m, float* d_v, float lr,
                         float b1, float b2, float eps, int t) = 0;
  // gradient of the mean log-likelihood w.r.t. the unnormalised sum log-parameters, from the accumulated edge flows
  virtual void flow_gradients(int32_t batch_size, float* d_grad) = 0;
  // Adam on the input nodes' auxiliary parameter copy, from the accumulated leaf flows
  virtual void leaf_adam(float* d_aux_p, float* d_aux_m, float* d_aux_v, float lr, float b1, float b2, float eps, int t) = 0;
  // queries on a matrix of parameter rows (element strides sr, sp), all rows in one pass
  virtual void kld_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows, bool norm_params,
                        float* d_out) = 0;
  virtual void kld_backward_rows(const float* d_p1, const float* d_p2, int64_t sr, int64_t sp, int32_t rows,
                                 bool norm_params, float* d_g1, float* d_g2, float* d_klds) = 0;
  virtual void gumbel_sample_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                  float temperature, bool norm_params, float* d_out) = 0;
  virtual void gumbel_sample_backward_rows(const float* d_params, int64_t sr, int64_t sp, int32_t rows, const float* d_noise,
                                           float temperature, bool norm_params, bool grad_wrt_logparams,
                                           const float* d_out_grad, float* d_grads) = 0;
  // per-example normalised flows [batch][parameters] (element strides sr, sp); normalize_params on parameter rows
  virtual void normalized_flows(const pcm::BatchRef& b, float* d_out, int64_t sr, int64_t sp, bool as_written) = 0;
  virtual void normalize_params_rows(float* d_params, int64_t sr, int64_t sp, int32_t rows, bool undo) = 0;
};
