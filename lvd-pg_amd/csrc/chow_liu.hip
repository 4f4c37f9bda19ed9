// Chow-Liu structure learning: pairwise mutual information of categorical data on the device,
// maximum spanning tree and rooting on the host.
//
// Reference: src/utils/information.jl:3-95 (pairwise and single marginals with a pseudocount
// spread as pc/C per category and pc/C^2 per cell, normalised by Z = N + pc) and :97-141
//   MI[u,v] = sum_{a,b} ( xlogx(P_uv[a,b]) - xlogy(P_uv[a,b], P_u[a] * P_v[b]) ).
// The tree is what src/structures/hclts.jl:17-18 asks ChowLiuTrees.jl / ProbabilisticCircuits.jl
// for: a maximum spanning tree of MI, directed away from the centre of the tree.
//
// The reference fills a dense [V][V][C][C] table with float atomics and reduces it on the host.
// Here a pair never leaves the workgroup.  With c(a,b) the count of a cell, s = pc/C^2,
// p(c) = (c + s)/Z, la[u][a] = log P_u[a]:
//   MI[u,v] = sum over non-empty cells of g(c(cell))  -  M_u - M_v  +  C^2 * xlogx(p(0))  -  p(0) * C * (L_u + L_v)
//   g(c) = xlogx(p(c)) - xlogx(p(0)),   M_u = (1/Z) sum_e la[u][x_eu],   L_u = sum_a la[u][a]
// (the empty cells' terms are the closed-form remainder), so a pair costs two passes over its N examples against a
// C x C table of counters in LDS -- count; then every example takes its cell's count away with it, and the one that
// finds a count there adds the cell's term -- and no pass over the table itself.  Up to 65535
// examples the counters are 16 bits wide and the whole table fits; beyond, they are 32 bits wide
// and the table is walked in bands of rows.
#include "common.hpp"
#include "chow_liu.hpp"
#include "stage_kernel.hip.hpp"

#include <algorithm>
#include <cmath>
#include <queue>

namespace pcm {

static void check_launch_c(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) fail(PCM_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
}

// Single marginals of one variable per workgroup: with la[a] = log((count_a + pc/C)/Z),
//   stat[v] = {M_v, L_v}
__global__ __launch_bounds__(256) void mi_single_kernel(const uint8_t* __restrict__ xb, int N, int64_t Np, int C, float pc,
                                                        double* __restrict__ stat) {
  __shared__ unsigned cnt[256];
  __shared__ double red[256];
  const int v = blockIdx.x, t = threadIdx.x;
  cnt[t] = 0u;
  __syncthreads();
  const uint8_t* row = xb + (size_t)v * Np;
  for (int64_t b = t; b < N; b += 256) atomicAdd(&cnt[row[b]], 1u);
  __syncthreads();
  const double Z = (double)N + (double)pc;
  double l = 0.0, m = 0.0;
  if (t < C) {
    const double p = ((double)cnt[t] + (double)pc / C) / Z;
    const double lg = p > 0.0 ? log(p) : -INFINITY;
    l = lg;                                        // -inf if a category is empty and pc = 0: only used with pc > 0
    m = cnt[t] ? (double)cnt[t] * lg / Z : 0.0;
  }
  red[t] = m;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) { if (t < o) red[t] += red[t + o]; __syncthreads(); }
  const double M = red[0];
  __syncthreads();
  red[t] = l;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) { if (t < o) red[t] += red[t + o]; __syncthreads(); }
  if (t == 0) { stat[2 * v] = M; stat[2 * v + 1] = red[0]; }
}

// g(c) = xlogx(p(c)) - xlogx(p(0)) for c = 0 .. N, the term of a cell that holds c examples, as a fixed-point integer of
// kMiFrac fractional bits: |g| < 0.37, a pair adds at most N < 2^17 of them into 64 bits, and integer sums do not
// depend on which thread adds which term (2^-44 per term is far below the float the sum ends as).
constexpr int kMiFrac = 44;
__global__ void mi_table_kernel(int N, int C, float pc, long long* __restrict__ g) {
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c > N) return;
  const double Z = (double)N + (double)pc, s = (double)pc / ((double)C * C);
  const double p0 = s / Z, x0 = p0 > 0.0 ? p0 * log(p0) : 0.0;
  const double p = ((double)c + s) / Z;
  g[c] = c ? llrint(ldexp(p * log(p) - x0, kMiFrac)) : 0ll;
}

constexpr int kMiThreads = 1024;

// Calls fn(a, b) for every example of a pair of staged rows; thread t owns examples 4t .. 4t+3
// (+ 4096 per further round).
template <typename F>
__device__ __forceinline__ void mi_each_example(const uint8_t* __restrict__ xu, const uint8_t* __restrict__ xv, int N, int t,
                                                F&& fn) {
  for (int64_t b4 = 4 * (int64_t)t; b4 < N; b4 += 4 * kMiThreads) {
    const uint32_t wu = *reinterpret_cast<const uint32_t*>(xu + b4), wv = *reinterpret_cast<const uint32_t*>(xv + b4);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (b4 + i < N) fn((int)((wu >> (8 * i)) & 0xffu), (int)((wv >> (8 * i)) & 0xffu));
  }
}

// The same with the words of the thread's first R rounds already in registers (R = 1, 2, 4 or 8: the host picks the
// smallest that covers the examples; rounds are masked, not branched around): a pair's three passes read them
// once, all of them requested before the first is used (a loop of a load and its use per round waits out one memory
// latency per round and pass), and the next pair's are requested while this pair's passes run -- a persistent workgroup
// owns its compute unit (the table fills the LDS), so nothing else hides the latency of its rows.
template <int R>
struct MiWords { uint32_t u[R], v[R]; };

template <int R>
__device__ __forceinline__ void mi_load_words(const uint8_t* __restrict__ xu, const uint8_t* __restrict__ xv, int N, int t,
                                              MiWords<R>& w) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t b4 = 4 * (int64_t)t + (int64_t)r * 4 * kMiThreads;
    w.u[r] = w.v[r] = 0u;
    if (b4 < N) {   // (the rows are padded to whole words past N)
      w.u[r] = *reinterpret_cast<const uint32_t*>(xu + b4);
      w.v[r] = *reinterpret_cast<const uint32_t*>(xv + b4);
    }
  }
}

template <int R, typename F>
__device__ __forceinline__ void mi_each_example_from(const MiWords<R>& w, const uint8_t* __restrict__ xu,
                                                     const uint8_t* __restrict__ xv, int N, int t, F&& fn) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t b4 = 4 * (int64_t)t + (int64_t)r * 4 * kMiThreads;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (b4 + i < N) fn((int)((w.u[r] >> (8 * i)) & 0xffu), (int)((w.v[r] >> (8 * i)) & 0xffu));
  }
  for (int64_t b4 = 4 * (int64_t)t + (int64_t)R * 4 * kMiThreads; b4 < N; b4 += 4 * kMiThreads) {
    const uint32_t wu = *reinterpret_cast<const uint32_t*>(xu + b4), wv = *reinterpret_cast<const uint32_t*>(xv + b4);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (b4 + i < N) fn((int)((wu >> (8 * i)) & 0xffu), (int)((wv >> (8 * i)) & 0xffu));
  }
}

// Sum of acc over the workgroup, then the closed-form remainder; thread 0 writes both halves of the matrix.  su, sv: the
// two variables' constants (M, L), read when the pair began -- read here they kept the whole workgroup waiting for
// thread 0's trip to memory.  No barrier behind thread 0: whoever writes `red` next has passed a barrier that thread 0
// reaches only after this.
struct MiStat { double m, l; };
__device__ __forceinline__ void mi_finish_pair(long long acc, long long* red, int t, int u, int v, int V, int C, double p0,
                                               double x0, MiStat su, MiStat sv, float* __restrict__ mi) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if ((t & 63) == 0) red[t >> 6] = acc;
  __syncthreads();
  if (t == 0) {
    long long sum = 0;
    for (int w = 0; w < kMiThreads / 64; ++w) sum += red[w];
    const double tot = ldexp((double)sum, -kMiFrac);
    double val = tot - su.m - sv.m + (double)C * C * x0;
    if (p0 > 0.0) val -= p0 * C * (su.l + sv.l);
    mi[(size_t)u * V + v] = (float)val;
    mi[(size_t)v * V + u] = (float)val;
  }
}

// Pairs (u <= v) in row-major order of the upper triangle, dealt round-robin to persistent
// workgroups.  At most 65535 examples: a cell's count fits 16 bits, two cells per LDS word.
template <int R>
__global__ __launch_bounds__(kMiThreads) void mi_pair_kernel(const uint8_t* __restrict__ xb, int N, int64_t Np, int V, int C,
                                                             float pc, const long long* __restrict__ g, int g_lds,
                                                             const double* __restrict__ stat, float* __restrict__ mi) {
  extern __shared__ unsigned cells[];   // C*C 16-bit counters, two per word | 16 sums | the first g_lds entries of g
  const int t = threadIdx.x;
  const int words = (C * C + 1) / 2;
  long long* red = reinterpret_cast<long long*>(cells + ((words + 1) & ~1));
  long long* gl = red + kMiThreads / 64;   // what the LDS has left holds the table over counts from its start: a lookup
  for (int i = t; i < words; i += kMiThreads) cells[i] = 0u;   // is then no trip to memory (counts past it are rare)
  for (int i = t; i < g_lds; i += kMiThreads) gl[i] = g[i];
  __syncthreads();
  const int64_t n_pairs = (int64_t)V * (V + 1) / 2;
  const double Z = (double)N + (double)pc, s = (double)pc / ((double)C * C);
  const double p0 = s / Z, x0 = p0 > 0.0 ? p0 * log(p0) : 0.0;
  // row u of the triangle starts at pair u*V - u*(u-1)/2
  int u = 0, un = 0;          // rows of this pair and of the workgroup's next one
  int64_t row0 = 0, rown = 0;
  MiWords<R> cur, nxt;
  if ((int64_t)blockIdx.x < n_pairs) {
    while ((int64_t)blockIdx.x >= rown + (V - un)) { rown += V - un; ++un; }
    mi_load_words(xb + (size_t)un * Np, xb + (size_t)(un + (int)(blockIdx.x - rown)) * Np, N, t, cur);
  }
  for (int64_t p = blockIdx.x; p < n_pairs; p += gridDim.x) {
    while (p >= row0 + (V - u)) { row0 += V - u; ++u; }
    const int v = u + (int)(p - row0);
    const uint8_t* xu = xb + (size_t)u * Np;
    const uint8_t* xv = xb + (size_t)v * Np;
    const MiStat su{stat[2 * u], stat[2 * u + 1]}, sv{stat[2 * v], stat[2 * v + 1]};
    long long acc = 0;
    mi_each_example_from(cur, xu, xv, N, t, [&](int a, int b) {
      const int key = a * C + b;
      atomicAdd(&cells[key >> 1], 1u << (16 * (key & 1)));
    });
    // the next pair's words, on their way while this pair is looked up and cleared
    const int64_t pn = p + gridDim.x;
    if (pn < n_pairs) {
      while (pn >= rown + (V - un)) { rown += V - un; ++un; }
      mi_load_words(xb + (size_t)un * Np, xb + (size_t)(un + (int)(pn - rown)) * Np, N, t, nxt);
    }
    __syncthreads();
    // look up and clear in one: the first of a cell's examples to come takes the cell's count with it and adds the
    // cell's term, the others find it empty (the sums are integers: who adds what does not show in the result)
    mi_each_example_from(cur, xu, xv, N, t, [&](int a, int b) {
      const int key = a * C + b, sh = 16 * (key & 1);
      const int cnt = (int)((atomicAnd(&cells[key >> 1], ~(0xffffu << sh)) >> sh) & 0xffffu);
      if (cnt) acc += cnt < g_lds ? gl[cnt] : g[cnt];
    });
    mi_finish_pair(acc, red, t, u, v, V, C, p0, x0, su, sv, mi);   // (its barrier also ends the clearing)
    cur = nxt;
  }
}

// The same for any number of examples: 32-bit cells.  A C x C table of them can exceed the LDS, so
// the categories of u are cut into bands of `band` rows and the three passes run once per band over
// the examples whose u-category falls into it.
__global__ __launch_bounds__(kMiThreads) void mi_pair_wide_kernel(const uint8_t* __restrict__ xb, int N, int64_t Np, int V,
                                                                  int C, int band, float pc, const long long* __restrict__ g,
                                                                  const double* __restrict__ stat, float* __restrict__ mi) {
  extern __shared__ unsigned cells[];   // band*C counters | 16 sums
  const int t = threadIdx.x;
  const int words = band * C;
  long long* red = reinterpret_cast<long long*>(cells + ((words + 1) & ~1));
  for (int i = t; i < words; i += kMiThreads) cells[i] = 0u;
  __syncthreads();
  const int64_t n_pairs = (int64_t)V * (V + 1) / 2;
  const double Z = (double)N + (double)pc, s = (double)pc / ((double)C * C);
  const double p0 = s / Z, x0 = p0 > 0.0 ? p0 * log(p0) : 0.0;
  int u = 0;
  int64_t row0 = 0;
  for (int64_t p = blockIdx.x; p < n_pairs; p += gridDim.x) {
    while (p >= row0 + (V - u)) { row0 += V - u; ++u; }
    const int v = u + (int)(p - row0);
    const uint8_t* xu = xb + (size_t)u * Np;
    const uint8_t* xv = xb + (size_t)v * Np;
    const MiStat su{stat[2 * u], stat[2 * u + 1]}, sv{stat[2 * v], stat[2 * v + 1]};
    long long acc = 0;
    for (int a0 = 0; a0 < C; a0 += band) {
      mi_each_example(xu, xv, N, t, [&](int a, int b) {
        if ((unsigned)(a - a0) < (unsigned)band) atomicAdd(&cells[(a - a0) * C + b], 1u);
      });
      __syncthreads();
      mi_each_example(xu, xv, N, t, [&](int a, int b) {   // look up and clear in one, as above
        if ((unsigned)(a - a0) < (unsigned)band) {
          const unsigned cnt = atomicExch(&cells[(a - a0) * C + b], 0u);
          if (cnt) acc += g[cnt];
        }
      });
      __syncthreads();
    }
    mi_finish_pair(acc, red, t, u, v, V, C, p0, x0, su, sv, mi);
  }
}

MiShape mi_check(const uint8_t* d_data, int64_t n_examples, int num_vars, int num_cats, float pseudocount, const float* d_mi) {
  if (!d_data || !d_mi) fail(PCM_ERR_ARG, "data or output pointer is null");
  if (n_examples < 1 || n_examples > 2147483584LL)
    fail(PCM_ERR_ARG, "pairwise MI takes 1..2147483584 examples per call, got %lld", (long long)n_examples);
  if (num_vars < 1) fail(PCM_ERR_SHAPE, "num_vars must be positive, got %d", num_vars);
  if (num_cats < 1 || num_cats > 256) fail(PCM_ERR_SHAPE, "num_cats must be in 1..256 (uint8 data), got %d", num_cats);
  if (pseudocount < 0.f) fail(PCM_ERR_ARG, "pseudocount must not be negative");
  MiShape s;
  s.N = (int)n_examples;
  s.V = num_vars;
  s.C = num_cats;
  s.Np = (n_examples + 63) / 64 * 64;
  return s;
}

// Queues staging, marginals, the count table and the pair kernel on `stream`; allocates nothing.
void mi_launch(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, const MiShape& sh, float pseudocount,
               const MiScratch& w, float* d_mi, hipStream_t stream) {
  const int N = sh.N, V = sh.V, C = sh.C;
  int dev = 0, cus = 0, max_lds = 0;
  PCM_HIP(hipGetDevice(&dev));
  PCM_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  PCM_HIP(hipDeviceGetAttribute(&max_lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev));
  const size_t red_bytes = (kMiThreads / 64) * sizeof(double);
  const bool narrow = N <= 65535;
  int band = C;
  size_t lds;
  int g_lds = 0;
  if (narrow) {
    const int words = (C * C + 1) / 2;
    lds = ((size_t)((words + 1) & ~1)) * 4 + red_bytes;
    // the rest of the LDS -- of half of it where two workgroups fit a compute unit -- holds the start of the g table
    const size_t whole = std::min<size_t>((size_t)max_lds, 160 * 1024), share = lds <= whole / 4 ? whole / 2 : whole;
    g_lds = (int)std::min<size_t>((size_t)N + 1, (share - lds) / sizeof(double));
    lds += (size_t)g_lds * sizeof(long long);
  } else {
    const size_t budget = std::min<size_t>((size_t)max_lds, 160 * 1024) - red_bytes - 8;
    band = (int)std::min<size_t>((size_t)C, budget / ((size_t)C * 4));
    if (band < 1) fail(PCM_ERR_UNSUPPORTED, "one row of the pair table does not fit %d bytes of LDS", max_lds);
    band = ceil_div(C, ceil_div(C, band));         // equal bands
    lds = ((size_t)((band * C + 1) & ~1)) * 4 + red_bytes;
  }
  if (lds > (size_t)max_lds) fail(PCM_ERR_UNSUPPORTED, "pair table needs %zu bytes of LDS, device offers %d", lds, max_lds);
  pcm_stage(d_data, stride_ex, stride_var, nullptr, N, sh.Np, V, C, w.xb, stream);
  hipLaunchKernelGGL(mi_single_kernel, dim3(V), dim3(256), 0, stream, w.xb, N, sh.Np, C, pseudocount, w.stat);
  hipLaunchKernelGGL(mi_table_kernel, dim3(ceil_div((int64_t)N + 1, 256)), dim3(256), 0, stream, N, C, pseudocount, w.g);
  const int64_t n_pairs = (int64_t)V * (V + 1) / 2;
  const int per_cu = std::max<int>(1, (int)(std::min<size_t>((size_t)max_lds, 160 * 1024) / lds));
  const int grid = (int)std::min<int64_t>(n_pairs, (int64_t)cus * std::min(per_cu, 2));
  if (narrow) {
    auto pairs = [&](auto kernel) {
      PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(kMiThreads), lds, stream, w.xb, N, sh.Np, V, C, pseudocount, w.g, g_lds, w.stat,
                         d_mi);
    };
    // rounds of 4 * kMiThreads examples whose words a thread keeps in registers
    if (N <= 4 * kMiThreads) pairs(&mi_pair_kernel<1>);
    else if (N <= 8 * kMiThreads) pairs(&mi_pair_kernel<2>);
    else if (N <= 16 * kMiThreads) pairs(&mi_pair_kernel<4>);
    else pairs(&mi_pair_kernel<8>);
  } else {
    PCM_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&mi_pair_wide_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(mi_pair_wide_kernel, dim3(grid), dim3(kMiThreads), lds, stream, w.xb, N, sh.Np, V, C, band,
                       pseudocount, w.g, w.stat, d_mi);
  }
  check_launch_c("pairwise_mi");
}

void pairwise_mi(const uint8_t* d_data, int64_t stride_ex, int64_t stride_var, int64_t n_examples, int num_vars,
                 int num_cats, float pseudocount, float* d_mi, hipStream_t stream) {
  const MiShape sh = mi_check(d_data, n_examples, num_vars, num_cats, pseudocount, d_mi);
  DevBuf<uint8_t> xb;
  DevBuf<double> stat;
  DevBuf<long long> g;
  xb.alloc((size_t)sh.V * sh.Np);
  stat.alloc((size_t)2 * sh.V);
  g.alloc((size_t)sh.N + 1);
  mi_launch(d_data, stride_ex, stride_var, sh, pseudocount, MiScratch{xb.p, stat.p, g.p}, d_mi, stream);
  PCM_HIP(hipStreamSynchronize(stream));   // the scratch arrays die with this call
}

// Maximum spanning tree of a dense symmetric weight matrix (Prim; among equal weights the
// lowest vertex index wins), rooted at the lowest-numbered centre of the tree (the vertex of
// least eccentricity), as a parent array with -1 at the root.
void chow_liu_tree(const float* mi, int V, int32_t* parent_out) {
  if (!mi || !parent_out) fail(PCM_ERR_ARG, "matrix or output pointer is null");
  if (V < 1) fail(PCM_ERR_SHAPE, "num_vars must be positive, got %d", V);
  std::vector<float> best(V, -INFINITY);
  std::vector<int32_t> link(V, -1);
  std::vector<char> in(V, 0);
  std::vector<std::vector<int32_t>> adj(V);
  in[0] = 1;
  for (int v = 1; v < V; ++v) { best[v] = mi[v]; link[v] = 0; }
  for (int it = 1; it < V; ++it) {
    int pick = -1;
    for (int v = 0; v < V; ++v)
      if (!in[v] && (pick < 0 || best[v] > best[pick])) pick = v;
    if (!(best[pick] > -INFINITY)) fail(PCM_ERR_ARG, "mutual information matrix holds NaN or -inf in row %d", pick);
    in[pick] = 1;
    adj[pick].push_back(link[pick]);
    adj[link[pick]].push_back(pick);
    const float* row = mi + (size_t)pick * V;
    for (int v = 0; v < V; ++v)
      if (!in[v] && row[v] > best[v]) { best[v] = row[v]; link[v] = pick; }
  }
  for (auto& a : adj) std::sort(a.begin(), a.end());
  // centre: peel leaves layer by layer; the last one or two vertices are the centres
  std::vector<int> deg(V);
  std::vector<int32_t> layer, next;
  int left = V;
  for (int v = 0; v < V; ++v) { deg[v] = (int)adj[v].size(); if (deg[v] <= 1) layer.push_back(v); }
  while (left > 2) {
    left -= (int)layer.size();
    next.clear();
    for (int32_t v : layer)
      for (int32_t w : adj[v])
        if (--deg[w] == 1) next.push_back(w);
    layer.swap(next);
  }
  const int root = *std::min_element(layer.begin(), layer.end());
  std::fill(parent_out, parent_out + V, -2);
  std::queue<int32_t> q;
  parent_out[root] = -1;
  q.push(root);
  while (!q.empty()) {
    const int32_t v = q.front();
    q.pop();
    for (int32_t w : adj[v])
      if (parent_out[w] == -2) { parent_out[w] = v; q.push(w); }
  }
}

}  // namespace pcm
