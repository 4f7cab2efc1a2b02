// Weight-side companions of a hardware-aware training step: the weight modifier of a training forward
// (discretise to levels of max |W|, add Gaussian noise in units of max |W|), the standard deviation behind
// the Gaussian weight clip, and the clamp itself.  Streaming kernels: every weight is read once and, where
// it changes, written once.
#pragma once
#include "common.h"
#include "misc_kernels.h"

namespace amoe {

// The value v as an element of type T would hold it (bf16: round to nearest even; fp32: unchanged).
template <typename T>
__device__ __forceinline__ float rnd_to(float v) { return Elem<T>::to_f32(Elem<T>::cvt(v)); }

// CH consecutive fp32 per-column values (missing ones read as `fill`); vec: 16-byte aligned and complete.
template <int CH>
__device__ __forceinline__ void load_cols(const float* __restrict__ p, int nv, bool vec, float fill, float (&o)[CH]) {
  if (vec && nv == CH) {
#pragma unroll
    for (int j = 0; j < CH / 4; j++) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(p + 4 * j);
#pragma unroll
      for (int i = 0; i < 4; i++) o[4 * j + i] = t[i];
    }
  } else {
#pragma unroll
    for (int q = 0; q < CH; q++) o[q] = q < nv ? p[q] : fill;
  }
}

struct ModifyParams {
  const void* w; void* out;
  const float* wmax;          // [E] (wmax_cols == 1) or [E, N]
  const float* noise;         // optional standard normals [E, K, N]; nullptr: drawn here
  long long rows;             // E * K
  int K, N, wmax_cols;
  float inv_states;           // > 0: discretise to multiples of wmax * inv_states (= wmax / n_states)
  float std_dev;              // > 0: add std_dev * wmax * normal
  int round_noise;            // the normals are elements of type T (rounded before use)
  uint64_t seed; const uint64_t* seed_dev;
  int vec, cvec;              // 16-byte access allowed on w / out, on wmax
};

constexpr int kModifierStream = 0x4D4F44;   // keeps these draws apart from the output noise of the same seed

// out = modified copy of w.  Every intermediate is rounded to T where an element-wise expression on tensors
// of type T would round it, so that bf16 results equal those of the expression evaluated op by op:
//   res = wmax * (1 / n_states);  q = round(w / res) * res;  out = q + (std_dev * wmax) * z
// (a tensor divided by a host scalar is multiplied by the scalar's fp32 reciprocal on the GPU, hence res).
template <typename T>
__global__ __launch_bounds__(kThreads) void modify_weight_kernel(const ModifyParams p) {
  constexpr int CH = Elem<T>::kChunk;
  const int chunks = (p.N + CH - 1) / CH;
  const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (idx >= p.rows * chunks) return;
  const long long row = idx / chunks;
  const int d = (int)(idx % chunks) * CH;
  const int nv = p.N - d < CH ? p.N - d : CH;
  const int e = (int)(row / p.K);
  const long long at = row * (long long)p.N + d;
  float v[CH], wm[CH];
  raw_unpack<T>(raw_load<T>(static_cast<const T*>(p.w) + at, nv, p.vec != 0), v);
  if (p.wmax_cols == 1) {
    const float we = p.wmax[e];
#pragma unroll
    for (int q = 0; q < CH; q++) wm[q] = we;
  } else {
    load_cols<CH>(p.wmax + (long long)e * p.N + d, nv, p.cvec != 0, 1.f, wm);
  }
  if (p.inv_states > 0.f) {
#pragma unroll
    for (int q = 0; q < CH; q++) {
      const float res = rnd_to<T>(wm[q] * p.inv_states);
      const float t = rnd_to<T>(v[q] / res);
      v[q] = rnd_to<T>(rintf(t) * res);
    }
  }
  if (p.std_dev > 0.f) {
    float z[CH];
    if (p.noise) {
#pragma unroll
      for (int q = 0; q < CH; q++) z[q] = q < nv ? p.noise[at + q] : 0.f;
    } else {
      const uint64_t seed = p.seed + (p.seed_dev ? *p.seed_dev : 0ull);
      const NoiseKey key = noise_key(seed, kModifierStream);
      const uint32_t rk = noise_row_key(key, (uint32_t)row);
#pragma unroll
      for (int j = 0; j < CH / 2; j++) noise_pair(key, rk, (uint32_t)(d / 2 + j), z[2 * j], z[2 * j + 1]);
    }
#pragma unroll
    for (int q = 0; q < CH; q++) {
      const float s = rnd_to<T>(p.std_dev * wm[q]);
      const float zz = p.round_noise ? rnd_to<T>(z[q]) : z[q];
      v[q] = rnd_to<T>(v[q] + rnd_to<T>(s * zz));
    }
  }
  T* out = static_cast<T*>(p.out) + at;
  if (p.vec && nv == CH) {
    *reinterpret_cast<Raw*>(out) = raw_pack<T>(v);
  } else {
    for (int q = 0; q < nv; q++) out[q] = Elem<T>::cvt(v[q]);
  }
}

// ---- unbiased standard deviation ------------------------------------------------------------------------
// Sums of (w - pivot) and (w - pivot)^2 in double, pivot = the first element of what is reduced: the shift
// keeps the one-pass formula (S2 - S1^2 / n) / (n - 1) free of cancellation for weights with a large mean.
constexpr int kStdMaxSlices = 64;

// Per expert: workgroup (slice, e) sums one slice of expert e into partial[(e * gridDim.x + slice) * 2 + {0, 1}].
template <typename T>
__global__ __launch_bounds__(kThreads) void weight_moments_kernel(const T* __restrict__ w, long long per_expert,
                                                                   double* __restrict__ partial, int vec) {
  __shared__ double red[4];
  const int tid = threadIdx.x;
  const T* base = w + (long long)blockIdx.y * per_expert;
  long long span = (per_expert + gridDim.x - 1) / gridDim.x;
  span = (span + 15) / 16 * 16;             // keep slices 16-byte aligned
  const long long lo = (long long)blockIdx.x * span;
  const long long hi = lo + span < per_expert ? lo + span : per_expert;
  constexpr int CH = Elem<T>::kChunk;
  const double pivot = (double)Elem<T>::load(base);
  double s1 = 0.0, s2 = 0.0;
  for (long long i = lo + (long long)tid * CH; i < hi; i += (long long)kThreads * CH) {
    const int nv = hi - i < CH ? (int)(hi - i) : CH;
    float v[CH];
    raw_unpack<T>(raw_load<T>(base + i, nv, vec != 0), v);
#pragma unroll
    for (int q = 0; q < CH; q++) {
      const double dv = q < nv ? (double)v[q] - pivot : 0.0;
      s1 += dv;
      s2 += dv * dv;
    }
  }
  s1 = block_sum_double(s1, red);
  s2 = block_sum_double(s2, red);
  if (tid == 0) {
    double* o = partial + ((long long)blockIdx.y * gridDim.x + blockIdx.x) * 2;
    o[0] = s1;
    o[1] = s2;
  }
}

__device__ __forceinline__ float std_from_moments(double s1, double s2, double n) {
  const double var = (s2 - s1 * s1 / n) / (n - 1.0);              // n == 1: 0 / 0, as the two-pass estimate gives
  return (float)sqrt(var < 0.0 ? 0.0 : var);
}

__global__ __launch_bounds__(kThreads) void weight_std_finalize_kernel(const double* __restrict__ partial, int slices,
                                                                        long long per_expert, int E,
                                                                        float* __restrict__ out) {
  const int e = blockIdx.x * kThreads + threadIdx.x;
  if (e >= E) return;
  double s1 = 0.0, s2 = 0.0;
  for (int s = 0; s < slices; s++) {
    s1 += partial[((long long)e * slices + s) * 2];
    s2 += partial[((long long)e * slices + s) * 2 + 1];
  }
  out[e] = std_from_moments(s1, s2, (double)per_expert);
}

// Per channel: std over k of w[e, k, c].  Same work split as the per-channel abs-max: a lane owns one 16-byte chunk
// of columns, `width` lanes cover a row, the wave's other lanes and the other waves take further rows of the
// workgroup's K slice; the slice's sums meet in LDS in a fixed order and go to
// partial[((e * slices + slice) * N + c) * 2 + {0, 1}].  The pivot of column c is w[e, 0, c].
template <typename T>
__global__ __launch_bounds__(kThreads) void weight_col_moments_kernel(const T* __restrict__ w, int K, int N, int width,
                                                                       double* __restrict__ partial, int vec) {
  constexpr int CH = Elem<T>::kChunk;
  __shared__ double red[kThreads][2 * CH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rows_per_wave = 64 / width;
  const int chunk = blockIdx.x * 64 + (lane % width);
  const int row_in_block = wave * rows_per_wave + lane / width;
  const int rows_per_block = 4 * rows_per_wave;
  const int d = chunk * CH;
  const int nv = N - d < CH ? N - d : CH;
  const int e = blockIdx.z;
  double s1[CH], s2[CH];
#pragma unroll
  for (int q = 0; q < CH; q++) s1[q] = s2[q] = 0.0;
  if (nv > 0) {
    const T* base = w + (long long)e * K * N + d;
    float pv[CH];
    raw_unpack<T>(raw_load<T>(base, nv, vec != 0), pv);
    for (int k = blockIdx.y * rows_per_block + row_in_block; k < K; k += gridDim.y * rows_per_block) {
      float v[CH];
      raw_unpack<T>(raw_load<T>(base + (long long)k * N, nv, vec != 0), v);
#pragma unroll
      for (int q = 0; q < CH; q++) {
        const double dv = (double)v[q] - (double)pv[q];
        s1[q] += dv;
        s2[q] += dv * dv;
      }
    }
  }
#pragma unroll
  for (int q = 0; q < CH; q++) {
    red[tid][2 * q] = s1[q];
    red[tid][2 * q + 1] = s2[q];
  }
  __syncthreads();
  if (row_in_block == 0 && nv > 0) {
    for (int r = 1; r < rows_per_block; r++) {
      const int other = (r / rows_per_wave) * 64 + (r % rows_per_wave) * width + (lane % width);
#pragma unroll
      for (int q = 0; q < CH; q++) {
        s1[q] += red[other][2 * q];
        s2[q] += red[other][2 * q + 1];
      }
    }
    double* o = partial + (((long long)e * gridDim.y + blockIdx.y) * N + d) * 2;
    for (int q = 0; q < nv; q++) {
      o[2 * q] = s1[q];
      o[2 * q + 1] = s2[q];
    }
  }
}

__global__ __launch_bounds__(kThreads) void weight_col_std_finalize_kernel(const double* __restrict__ partial, int slices,
                                                                            int K, int N, int E, float* __restrict__ out) {
  const long long i = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (i >= (long long)E * N) return;
  const int e = (int)(i / N), c = (int)(i % N);
  double s1 = 0.0, s2 = 0.0;
  for (int s = 0; s < slices; s++) {
    const double* o = partial + (((long long)e * slices + s) * N + c) * 2;
    s1 += o[0];
    s2 += o[1];
  }
  out[i] = std_from_moments(s1, s2, (double)K);
}

// w = clamp(w, -bound, +bound) in place; bound is [E] (cols == 1) or [E, N].
template <typename T>
__global__ __launch_bounds__(kThreads) void clamp_weights_kernel(T* __restrict__ w, const float* __restrict__ bound,
                                                                  long long rows, int K, int N, int cols, int vec,
                                                                  int cvec) {
  constexpr int CH = Elem<T>::kChunk;
  const int chunks = (N + CH - 1) / CH;
  const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (idx >= rows * chunks) return;
  const long long row = idx / chunks;
  const int d = (int)(idx % chunks) * CH;
  const int nv = N - d < CH ? N - d : CH;
  const int e = (int)(row / K);
  T* at = w + row * (long long)N + d;
  float v[CH];
  raw_unpack<T>(raw_load<T>(at, nv, vec != 0), v);
  float bd[CH];
  if (cols == 1) {
    const float be = bound[e];
#pragma unroll
    for (int q = 0; q < CH; q++) bd[q] = be;
  } else {
    load_cols<CH>(bound + (long long)e * N + d, nv, cvec != 0, 0.f, bd);
  }
  bool changed = false;
#pragma unroll
  for (int q = 0; q < CH; q++) {
    const float b = bd[q];
    const float c = fminf(fmaxf(v[q], -b), b);
    changed |= (q < nv) && (c != v[q]);
    v[q] = c;
  }
  if (!changed) return;                      // a Gaussian clip at 2-3 sigma leaves most chunks as they are
  if (vec && nv == CH) {
    *reinterpret_cast<Raw*>(at) = raw_pack<T>(v);
  } else {
    for (int q = 0; q < nv; q++) at[q] = Elem<T>::cvt(v[q]);
  }
}

}  // namespace amoe
