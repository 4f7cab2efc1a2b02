// The router's epilogue in one pass over the logits: sigmoid gate values, top-k experts per token and the
// entropy regulariser of the mean expert usage; and its backward pass.  One wave per token row, a lane owns the
// experts lane, lane + 64, ...  (PER of them: 1, 2, 4 or 8, the kernels are instantiated per count).
#pragma once
#include "common.h"

namespace amoe {

constexpr int kSelPerLane = 8;            // experts per lane: E <= 512
constexpr int kSelRowsPerWave = 8;        // rows a wave walks through; its usage sums stay in registers meanwhile

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += wave_shfl_xor(v, d);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, wave_shfl_xor(v, d));
  return v;
}

// The gate value as the tensor expression sigmoid(logits) holds it: computed in fp32, stored in T.
template <typename T>
__device__ __forceinline__ float gate_value(float x) {
  return Elem<T>::to_f32(Elem<T>::cvt(1.0f / (1.0f + expf(-x))));
}

// sel_val / sel_idx [rows, k]: the k largest gate values of each row in descending order, ties to the lower
// expert id.  prob_partial [gridDim.x, E] (optional): per workgroup, sum over its rows of softmax(logits[row]).
template <typename T, int PER>
__global__ __launch_bounds__(kThreads) void select_fwd_kernel(const T* __restrict__ logits, long long rows, int E, int k,
                                                               T* __restrict__ sel_val, int64_t* __restrict__ sel_idx,
                                                               float* __restrict__ prob_partial) {
  __shared__ float sProb[4][64 * PER];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float kNegInf = -__builtin_inff();
  float usage[PER];
#pragma unroll
  for (int j = 0; j < PER; j++) usage[j] = 0.f;
  const long long first = ((long long)blockIdx.x * 4 + wave) * kSelRowsPerWave;
  for (int rr = 0; rr < kSelRowsPerWave; rr++) {
    const long long row = first + rr;
    if (row >= rows) break;                       // the same for the whole wave
    const T* __restrict__ src = logits + row * (long long)E;
    float x[PER], s[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) {
      const int e = lane + 64 * j;
      x[j] = e < E ? Elem<T>::load(src + e) : kNegInf;
      s[j] = e < E ? gate_value<T>(x[j]) : kNegInf;
    }
    if (prob_partial != nullptr) {
      float m = kNegInf;
#pragma unroll
      for (int j = 0; j < PER; j++) m = fmaxf(m, x[j]);
      m = wave_max(m);
      float ex[PER], sum = 0.f;
#pragma unroll
      for (int j = 0; j < PER; j++) {
        ex[j] = expf(x[j] - m);                   // exp(-inf) = 0 for the slots past E
        sum += ex[j];
      }
      const float inv = 1.0f / wave_sum(sum);
#pragma unroll
      for (int j = 0; j < PER; j++) usage[j] += ex[j] * inv;
    }
    for (int t = 0; t < k; t++) {
      float bv = kNegInf;
      int bi = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < PER; j++) {     // ascending expert id within the lane: the first maximum wins
        const bool better = s[j] > bv;
        bv = better ? s[j] : bv;
        bi = better ? lane + 64 * j : bi;
      }
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) {
        const float ov = wave_shfl_xor(bv, d);
        const int oi = wave_shfl_xor(bi, d);
        const bool take = ov > bv || (ov == bv && oi < bi);
        bv = take ? ov : bv;
        bi = take ? oi : bi;
      }
#pragma unroll
      for (int j = 0; j < PER; j++)
        if (lane + 64 * j == bi) s[j] = kNegInf;  // taken
      if (lane == 0) {
        sel_val[row * k + t] = Elem<T>::cvt(bv);
        sel_idx[row * k + t] = bi;
      }
    }
  }
  if (prob_partial != nullptr) {
#pragma unroll
    for (int j = 0; j < PER; j++) sProb[wave][lane + 64 * j] = usage[j];
    __syncthreads();
    for (int e = tid; e < E; e += kThreads)
      prob_partial[(long long)blockIdx.x * E + e] = (sProb[0][e] + sProb[1][e]) + (sProb[2][e] + sProb[3][e]);
  }
}

// First level of the usage sum: workgroup g adds the partial rows [g * chunk, (g + 1) * chunk) into out[g, :].
// (One workgroup walking all of them would wait for one memory latency per four rows.)
constexpr int kSelSumChunk = 64;
__global__ __launch_bounds__(kThreads) void select_usage_sum_kernel(const float* __restrict__ prob_partial, int blocks,
                                                                     int E, float* __restrict__ out) {
  __shared__ float sSum[4][64 * kSelPerLane];
  const int tid = threadIdx.x, lane = tid & 63, slice = tid >> 6;
  const int lo = blockIdx.x * kSelSumChunk;
  const int hi = lo + kSelSumChunk < blocks ? lo + kSelSumChunk : blocks;
  float s[kSelPerLane];
#pragma unroll
  for (int j = 0; j < kSelPerLane; j++) s[j] = 0.f;
#pragma unroll 4
  for (int b = lo + slice; b < hi; b += 4) {
#pragma unroll
    for (int j = 0; j < kSelPerLane; j++)
      if (lane + 64 * j < E) s[j] += prob_partial[(long long)b * E + lane + 64 * j];
  }
#pragma unroll
  for (int j = 0; j < kSelPerLane; j++) sSum[slice][lane + 64 * j] = s[j];
  __syncthreads();
  for (int e = tid; e < E; e += kThreads)
    out[(long long)blockIdx.x * E + e] = (sSum[0][e] + sSum[1][e]) + (sSum[2][e] + sSum[3][e]);
}

// reg = sum_e pbar_e * log(pbar_e), pbar = mean over the rows of softmax(logits); reg_c[e] = 1 + log(pbar_e) is
// d reg / d pbar_e, kept for the backward pass.  One workgroup; fixed summation order.
__global__ __launch_bounds__(kThreads) void select_reg_kernel(const float* __restrict__ prob_partial, int blocks, int E,
                                                               long long rows, float* __restrict__ reg,
                                                               float* __restrict__ reg_c) {
  __shared__ float sSum[4][64 * kSelPerLane];
  __shared__ float red[kThreads];
  const int tid = threadIdx.x, lane = tid & 63, slice = tid >> 6;
  // wave `slice` adds the workgroups slice, slice + 4, ...; a lane owns the experts lane, lane + 64, ...
  float s[kSelPerLane];
#pragma unroll
  for (int j = 0; j < kSelPerLane; j++) s[j] = 0.f;
#pragma unroll 4
  for (int b = slice; b < blocks; b += 4) {
#pragma unroll
    for (int j = 0; j < kSelPerLane; j++)
      if (lane + 64 * j < E) s[j] += prob_partial[(long long)b * E + lane + 64 * j];
  }
#pragma unroll
  for (int j = 0; j < kSelPerLane; j++) sSum[slice][lane + 64 * j] = s[j];
  __syncthreads();
  float mine = 0.f;
  for (int e = tid; e < E; e += kThreads) {
    const float pbar = ((sSum[0][e] + sSum[1][e]) + (sSum[2][e] + sSum[3][e])) / (float)rows;
    const float lp = logf(pbar);
    reg_c[e] = 1.0f + lp;
    mine += pbar * lp;
  }
  red[tid] = mine;
  __syncthreads();
  for (int d = kThreads / 2; d >= 1; d >>= 1) {
    if (tid < d) red[tid] += red[tid + d];
    __syncthreads();
  }
  if (tid == 0) *reg = red[0];
}

// grad_logits[row, e] = grad_reg / rows * p_e * (c_e - sum_e' p_e' c_e')          (regulariser, p = softmax)
//                     + grad_val[row, t] * s * (1 - s)  where e == sel_idx[row, t]  (sigmoid gate of a chosen expert)
template <typename T, int PER>
__global__ __launch_bounds__(kThreads) void select_bwd_kernel(const T* __restrict__ logits, long long rows, int E, int k,
                                                               const int64_t* __restrict__ sel_idx,
                                                               const T* __restrict__ grad_val,
                                                               const float* __restrict__ reg_c,
                                                               const float* __restrict__ grad_reg,
                                                               T* __restrict__ grad_logits) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float kNegInf = -__builtin_inff();
  const T* __restrict__ src = logits + row * (long long)E;
  float x[PER], g[PER];
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int e = lane + 64 * j;
    x[j] = e < E ? Elem<T>::load(src + e) : kNegInf;
    g[j] = 0.f;
  }
  if (reg_c != nullptr && grad_reg != nullptr) {
    float m = kNegInf;
#pragma unroll
    for (int j = 0; j < PER; j++) m = fmaxf(m, x[j]);
    m = wave_max(m);
    float pr[PER], c[PER], sum = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      pr[j] = expf(x[j] - m);
      sum += pr[j];
      c[j] = lane + 64 * j < E ? reg_c[lane + 64 * j] : 0.f;
    }
    const float inv = 1.0f / wave_sum(sum);
    float dot = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      pr[j] *= inv;
      dot += pr[j] * c[j];
    }
    dot = wave_sum(dot);
    const float scale = *grad_reg / (float)rows;
#pragma unroll
    for (int j = 0; j < PER; j++) g[j] = scale * pr[j] * (c[j] - dot);
  }
  if (grad_val != nullptr) {
    for (int t = 0; t < k; t++) {
      const int idx = (int)sel_idx[row * k + t];
      const float gv = Elem<T>::load(grad_val + row * k + t);
#pragma unroll
      for (int j = 0; j < PER; j++) {
        if (lane + 64 * j == idx) {
          const float s = gate_value<T>(x[j]);
          g[j] += gv * s * (1.0f - s);
        }
      }
    }
  }
  T* __restrict__ dst = grad_logits + row * (long long)E;
#pragma unroll
  for (int j = 0; j < PER; j++)
    if (lane + 64 * j < E) dst[lane + 64 * j] = Elem<T>::cvt(g[j]);
}

}  // namespace amoe
