// Soft evidence on the block engine (reference: src/regularization/reg_likelihood.jl:51-91,
// reg_flow.jl:50-82: with data [examples, variables, categories] of log-evidence a leaf's value
// is logsumexp_c(evidence_c + logp_c) and its flow is shared among the categories in proportion
// to exp(evidence_c + logp_c - value)).
//
// Both steps factor through the example's largest evidence m_b = max_c ev[b,v,c]:
//   value[b,k]  = m_b + log sum_c E[b,c] P[c,k],        E = exp(ev - m_b), P = exp(leaf[v])
//   counts[c,k] += P[c,k] sum_b E[b,c] Gs[b,k],         Gs[b,k] = flow[b,k] exp(m_b - value[b,k])
// i.e. one [examples x categories] x [categories x states] product per variable going up and one
// [categories x examples] x [examples x states] product going down, instead of an exponential per
// (example, category, state).  The sum over c always contains the term of the largest evidence,
// E = 1, so it can only get small where that category is all but impossible under the leaf; where
// the sum drops below e^-60 the value is recomputed in log space, and the flow of such an
// (example, state) is shared out term by term (slow paths that ordinary parameters never take).
//
// The values land in a table [V][Bp][K] that the walk kernels read as if it were the leaf table:
// one row per example instead of one per category, the "category" of example b being its rank
// in its 16-example slice and every slice's rows starting 16*K*4 bytes further on.
#pragma once

#include "hclt_kernels.hip.hpp"

namespace pcm {

constexpr int kEvExamples = 64;   // examples per evidence tile
constexpr int kEvCats = 64;       // categories per tile of the flow kernel
constexpr int kEvVars = 1;        // variables a workgroup of the value kernel takes in turn (more: longer contiguous rows, fewer workgroups; no gain measured)
constexpr int kEvBatch = 16;      // evidence requests a thread keeps in flight while staging a tile
constexpr float kEvTiny = 1e-26f;     // e^-60: below it the factored sum has lost its footing
constexpr float kEvFar = 59.f;        // value more than this below the largest evidence: exact flow

// categories of the walk kernels under soft evidence: the example's rank in its slice
__global__ void hclt_soft_x_kernel(uint8_t* __restrict__ xb, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) xb[i] = (uint8_t)(i & (kSlice - 1));
}

__device__ __forceinline__ float soft_ev(const SoftRef& s, int b, int v, int c) {
  const int64_t e = s.d_idx ? s.d_idx[b] : b;
  return s.d_ev[e * s.stride_ex + (int64_t)v * s.stride_var + (int64_t)c * s.stride_cat];
}

// value table and per-example maxima of one batch; grid (ceil(V / kEvVars), Bp / 64), 4 * K/16 waves.
// LDS: E tile [64][LD] | P = exp(leaf[v]) [Cp][K + 16] | row maxima [64]; Cp = C rounded up to 4.
// Wave w contracts examples 16*(w%4).. against states 16*(w/4).. on the matrix cores
// (v_mfma_f32_16x16x4_f32: A = E, rows examples; B = P, columns states; 4 categories a step).
// Many short waves rather than four long ones: every phase is a chain of LDS round trips.
template <int K>
__global__ __launch_bounds__(4 * (K / 16) * 64) void hclt_soft_leafval_kernel(SoftRef s, const float* __restrict__ leaf, int C,
                                                                              int V, int B, int Bp, float* __restrict__ LV,
                                                                              float* __restrict__ M) {
  extern __shared__ __align__(16) float smem[];
  constexpr int KT = K / 16, LDP = K + 16, NW = 4 * KT, NT = NW * 64, TPE = NT / kEvExamples;   // threads per example
  const int Cp = (C + 3) & ~3, LD = Cp + 4;
  float* tile = smem;
  float* Pt = tile + kEvExamples * LD;
  float* rmax = Pt + (size_t)Cp * LDP;
  const int b0 = blockIdx.y * kEvExamples;
  const bool cat_fast = s.stride_cat == 1;
  const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // a run of kEvVars variables per workgroup: with [examples][variables][categories] evidence the
  // rows it reads are kEvVars * C contiguous floats each, and neighbouring workgroups continue them
  for (int v = blockIdx.x * kEvVars; v < min((int)(blockIdx.x + 1) * kEvVars, V); ++v) {
  if (v != (int)blockIdx.x * kEvVars) __syncthreads();   // the previous variable's tiles are still being read
  // Evidence tile: lanes run along whichever of (category, example) is contiguous in memory, waves
  // along the other; no division by the run-time C, kEvBatch requests in flight per thread.
  {
    const int n_fast = cat_fast ? C : kEvExamples, n_slow = cat_fast ? kEvExamples : C;
    for (int f0 = 0; f0 < n_fast; f0 += 64) {
      const int f = f0 + lane;
      for (int s0 = w; s0 < n_slow; s0 += NW * kEvBatch) {
        float tmp[kEvBatch];
#pragma unroll
        for (int u = 0; u < kEvBatch; ++u) {
          const int sl = s0 + NW * u;
          const int e = cat_fast ? sl : f, c = cat_fast ? f : sl;
          tmp[u] = (f < n_fast && sl < n_slow && b0 + e < B) ? soft_ev(s, b0 + e, v, c) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kEvBatch; ++u) {
          const int sl = s0 + NW * u;
          const int e = cat_fast ? sl : f, c = cat_fast ? f : sl;
          if (f < n_fast && sl < n_slow) tile[e * LD + c] = tmp[u];
        }
      }
    }
  }
  for (int i0 = threadIdx.x; i0 < Cp * K; i0 += NT * 8) {
    float tmp[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * NT;
      tmp[u] = i < C * K ? leaf[(size_t)v * C * K + i] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * NT;
      if (i < Cp * K) Pt[(i / K) * LDP + i % K] = __expf(tmp[u]);
    }
  }
  __syncthreads();
  {
    // TPE threads per example: row maximum, then E = exp(ev - m) in place (columns C..Cp-1: 0)
    const int e = threadIdx.x / TPE, sub = threadIdx.x % TPE;
    float m = -INFINITY;
    for (int c = sub; c < C; c += TPE) m = fmaxf(m, tile[e * LD + c]);
#pragma unroll
    for (int o = 1; o < TPE; o <<= 1) m = fmaxf(m, __shfl_xor(m, o));
    if (!(m > -INFINITY)) m = 0.f;
    for (int c = sub; c < Cp; c += TPE) tile[e * LD + c] = c < C ? __expf(tile[e * LD + c] - m) : 0.f;
    if (sub == 0) rmax[e] = m;
  }
  __syncthreads();
  const int r = lane & 15, g = lane >> 4, bt = w & 3, kt = w >> 2;
  v4f acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0;   // two chains
  const float* arow = tile + (16 * bt + r) * LD + g;
  const float* brow = Pt + g * LDP + kt * 16 + r;
  int c0 = 0;
  for (; c0 + 8 <= Cp; c0 += 8) {
    acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(arow[c0], brow[c0 * LDP], acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(arow[c0 + 4], brow[(c0 + 4) * LDP], acc1, 0, 0, 0);
  }
  if (c0 < Cp) acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(arow[c0], brow[c0 * LDP], acc0, 0, 0, 0);
  const v4f acc = acc0 + acc1;
  // accumulator element i: example 16*bt + 4g + i, state kt*16 + r
  const int k = kt * 16 + r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = 16 * bt + 4 * g + i, b = b0 + e;
    const float m = rmax[e];
    float val = 0.f;
    if (b < B) {
      val = m + __logf(acc[i]);
      if (!(acc[i] > kEvTiny)) {            // the favoured category is all but impossible under this leaf
        float mx = -INFINITY, sm = 0.f;
        for (int c = 0; c < C; ++c) {
          const float t = soft_ev(s, b, v, c) + leaf[((size_t)v * C + c) * K + k];
          if (t > mx) { sm = sm * __expf(mx - t) + 1.f; mx = t; }
          else if (t > -INFINITY) sm += __expf(t - mx);
        }
        val = mx > -INFINITY ? mx + __logf(sm) : -INFINITY;
      }
    }
    LV[((size_t)v * Bp + b) * K + k] = val;
    if (kt == 0 && r == 0) M[(size_t)v * Bp + b] = b < B ? m : 0.f;
  }
  }
}

// leaf_flow *= rate (0: cleared) ahead of a flow kernel that adds into it
__global__ void hclt_soft_scale_kernel(float* __restrict__ p, int64_t n, float rate) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = rate != 0.f ? p[i] * rate : 0.f;
}

// leaf_flow[v][c][k] += P[c,k] * sum_b E[b,c] Gs[b,k] over the examples of split blockIdx.z;
// grid (ceil(C / 64), V, splits), 256 threads.  With one split the sum goes straight into leaf_flow; with
// several, split z leaves its share in row z of part_all [splits][V * C * K] for sum_parts_kernel.
// G: the child-flow tiles the statistics pass left behind; g_node[v]: the tree node whose tile
// carries the flow of variable v's leaves (its own node, or its parent's).
// LDS: E tile [64 examples][68] | Gs [64 examples][K + 4].  Wave w contracts categories
// c0 + 16w .. +15 against all K states over the examples on the matrix cores (A = E^T, B = Gs).
// The (example, state) pairs whose value lies too far below the largest evidence are left out
// of Gs and shared out term by term afterwards, from memory.
template <int K>
__global__ __launch_bounds__(256) void hclt_soft_leafflow_kernel(SoftRef s, const float* __restrict__ leaf,
                                                                 const float* __restrict__ LV, const float* __restrict__ M,
                                                                 const float* __restrict__ G, const int32_t* __restrict__ g_node,
                                                                 int C, int B, int Bp, size_t node_floats, int split_examples,
                                                                 float* __restrict__ leaf_flow, float* __restrict__ part_all) {
  constexpr int KT = K / 16, ELD = kEvCats + 4, LDG = K + 4;
  float* part = part_all ? part_all + (size_t)blockIdx.z * gridDim.y * C * K : nullptr;
  __shared__ __align__(16) float Et[kEvExamples * ELD];
  __shared__ __align__(16) float Gs[kEvExamples * LDG];
  __shared__ int any_slow;
  const int v = blockIdx.y, c0 = blockIdx.x * kEvCats;
  const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g4 = lane >> 4;
  const bool cat_fast = s.stride_cat == 1;
  const float* g = G + (size_t)g_node[v] * node_floats;
  const int b_begin = blockIdx.z * split_examples, b_end = min(B, b_begin + split_examples);
  v4f acc[KT], accD[KT];   // accD: exact-path terms, which already contain the leaf probability
#pragma unroll
  for (int kt = 0; kt < KT; ++kt) acc[kt] = accD[kt] = v4f{0.f, 0.f, 0.f, 0.f};
  for (int b0 = b_begin; b0 < b_end; b0 += kEvExamples) {
    if (threadIdx.x == 0) any_slow = 0;
    __syncthreads();
    for (int i0 = threadIdx.x; i0 < kEvExamples * kEvCats; i0 += 256 * kEvBatch) {
      float tmp[kEvBatch], mb[kEvBatch];
#pragma unroll
      for (int u = 0; u < kEvBatch; ++u) {
        const int i = i0 + u * 256;
        const int e = cat_fast ? i / kEvCats : i % kEvExamples, cc = cat_fast ? i % kEvCats : i / kEvExamples;
        const bool ok = b0 + e < b_end && c0 + cc < C;
        tmp[u] = ok ? soft_ev(s, b0 + e, v, c0 + cc) : -INFINITY;
        mb[u] = ok ? M[(size_t)v * Bp + b0 + e] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < kEvBatch; ++u) {
        const int i = i0 + u * 256;
        const int e = cat_fast ? i / kEvCats : i % kEvExamples, cc = cat_fast ? i % kEvCats : i / kEvExamples;
        Et[e * ELD + cc] = __expf(tmp[u] - mb[u]);
      }
    }
    // the chunk's four slices of G, tile-native: float4 (kt, lane) of a slice holds states
    // kt*16 + 4*(lane/16) + 0..3 of example lane%16
    constexpr int NG = KT;   // float4 units of G per thread and chunk
    v4f gf[NG], glv[NG];
    float gm[NG];
#pragma unroll
    for (int u = 0; u < NG; ++u) {
      const int i = threadIdx.x + u * 256;
      const int sl = i / (KT * 64), kt = (i / 64) % KT, ln = i % 64;
      const int e = sl * 16 + (ln & 15), k = kt * 16 + 4 * (ln >> 4), b = b0 + e;
      gf[u] = glv[u] = v4f{0.f, 0.f, 0.f, 0.f};
      gm[u] = 0.f;
      if (b < b_end) {
        gf[u] = *reinterpret_cast<const v4f*>(g + ((size_t)(b0 / kSlice + sl) * kSlice * K) + (size_t)(kt * 64 + ln) * 4);
        glv[u] = *reinterpret_cast<const v4f*>(LV + ((size_t)v * Bp + b) * K + k);
        gm[u] = M[(size_t)v * Bp + b];
      }
    }
#pragma unroll
    for (int u = 0; u < NG; ++u) {
      const int i = threadIdx.x + u * 256;
      const int sl = i / (KT * 64), kt = (i / 64) % KT, ln = i % 64;
      const int e = sl * 16 + (ln & 15), k = kt * 16 + 4 * (ln >> 4);
      v4f f = gf[u];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (!(f[j] > 0.f)) f[j] = 0.f;
        else if (gm[u] - glv[u][j] > kEvFar) { f[j] = 0.f; any_slow = 1; }
        else f[j] *= __expf(gm[u] - glv[u][j]);
      }
      *reinterpret_cast<v4f*>(&Gs[e * LDG + k]) = f;
    }
    __syncthreads();
    {
      const float* arow = Et + g4 * ELD + 16 * w + r;
      const float* brow = Gs + g4 * LDG + r;
#pragma unroll 4
      for (int e0 = 0; e0 < kEvExamples; e0 += 4) {
        const float a = arow[e0 * ELD];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
          acc[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, brow[e0 * LDG + kt * 16], acc[kt], 0, 0, 0);
      }
    }
    if (any_slow) {
      // accumulator element i of tile kt: category c0 + 16w + 4*g4 + i, state kt*16 + r
      for (int e = 0; e < kEvExamples && b0 + e < b_end; ++e) {
        const int b = b0 + e;
        const float m = M[(size_t)v * Bp + b];
        const float* gt = g + (size_t)(b / kSlice) * kSlice * K;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
          const int k = kt * 16 + r;
          const float fl = gt[(size_t)(kt * 64 + 16 * ((k % 16) / 4) + (b % kSlice)) * 4 + k % 4];
          const float lv = LV[((size_t)v * Bp + b) * K + k];
          if (fl > 0.f && m - lv > kEvFar) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int c = c0 + 16 * w + 4 * g4 + i;
              if (c < C) accD[kt][i] += fl * __expf(soft_ev(s, b, v, c) + leaf[((size_t)v * C + c) * K + k] - lv);
            }
          }
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + 16 * w + 4 * g4 + i;
    if (c >= C) continue;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const size_t o = ((size_t)v * C + c) * K + kt * 16 + r;
      const float add = __expf(leaf[o]) * acc[kt][i] + accD[kt][i];
      if (part) part[o] = add;       // this workgroup is the only writer of the cell either way
      else leaf_flow[o] += add;
    }
  }
}

}  // namespace pcm
