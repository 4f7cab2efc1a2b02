// Row-wise companions of the CVMM calls: gate-weighted reduction over the k heads, k-sum,
// gate gradient, abs-max of rows and of weights, per-expert segment sums and standard
// deviation.  All are bandwidth-bound streaming kernels with fixed summation order.
#pragma once
#include "common.h"

namespace amoe {

// The step counter of the generated noise moves on in the launch that follows the last kernel drawing from it: stream
// order puts every read of the old value before this addition (one lane, a vector-memory atomic).
__device__ __forceinline__ void bump_counter(long long* counter, long long add) {
  if (counter != nullptr && blockIdx.x == 0 && threadIdx.x == 0)
    atomicAdd(reinterpret_cast<unsigned long long*>(counter), (unsigned long long)add);
}

// y[t, d] = sum_j gate[t*k+j] * z[(t*k+j), d]   (gate == nullptr: plain sum over j).
// One thread per (row, 16-byte chunk); fp32 accumulation in ascending j.
template <typename T>
__global__ __launch_bounds__(kThreads) void head_reduce_kernel(const T* __restrict__ z, const T* __restrict__ gate,
                                                                T* __restrict__ y, long long rows, int k, int D,
                                                                int vec, long long* counter, long long counter_add) {
  constexpr int CH = Elem<T>::kChunk;
  const int chunks = (D + CH - 1) / CH;
  bump_counter(counter, counter_add);
  const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (idx >= rows * chunks) return;
  const long long t = idx / chunks;
  const int d = (int)(idx % chunks) * CH;
  const int nv = D - d < CH ? D - d : CH;
  float acc[CH];
#pragma unroll
  for (int q = 0; q < CH; q++) acc[q] = 0.f;
  for (int j = 0; j < k; j++) {
    float v[CH];
    raw_unpack<T>(raw_load_streaming<T>(z + (t * k + j) * (long long)D + d, nv, vec != 0), v);
    const float gt = gate ? Elem<T>::load(gate + t * k + j) : 1.f;
#pragma unroll
    for (int q = 0; q < CH; q++) acc[q] += gt * v[q];
  }
  T* out = y + t * (long long)D + d;
  if (vec && nv == CH) {
    store_streaming(out, raw_pack<T>(acc));
  } else {
    for (int q = 0; q < nv; q++) out[q] = Elem<T>::cvt(acc[q]);
  }
}

// Wave sums of eight per-lane values in ten exchanges instead of forty-eight: at distance 32 a lane hands over the
// four values its partner keeps, at 16 two, at 8 one; three more steps finish the one left.  Returns the sum of
// v[lane / 8] (the same in the eight lanes of a group); fixed order.
__device__ __forceinline__ float wave_sum8(const float (&v)[8], int lane) {
  const bool b5 = (lane & 32) != 0, b4 = (lane & 16) != 0, b3 = (lane & 8) != 0;
  float w4[4], w2[2];
#pragma unroll
  for (int i = 0; i < 4; i++) w4[i] = (b5 ? v[4 + i] : v[i]) + wave_shfl_xor(b5 ? v[i] : v[4 + i], 32);
#pragma unroll
  for (int i = 0; i < 2; i++) w2[i] = (b4 ? w4[2 + i] : w4[i]) + wave_shfl_xor(b4 ? w4[i] : w4[2 + i], 16);
  float w1 = (b3 ? w2[1] : w2[0]) + wave_shfl_xor(b3 ? w2[0] : w2[1], 8);
#pragma unroll
  for (int s = 4; s >= 1; s >>= 1) w1 += wave_shfl_xor(w1, s);
  return w1;
}

// grad_gate[t*k+j] = <z[t*k+j, :], dy[t, :]>.  One wave per token: a lane's chunk of dy[t] is loaded once and
// meets the same chunk of up to 8 head rows, whose loads are all in flight together.  Per row the sum runs
// over the lane's chunks in ascending order, then over the lanes in a fixed order: independent of k.
template <typename T>
__global__ __launch_bounds__(kThreads) void gate_grad_kernel(const T* __restrict__ z, const T* __restrict__ dy,
                                                              T* __restrict__ out, long long tokens, int k, int D,
                                                              int vec) {
  constexpr int CH = Elem<T>::kChunk, JB = 8;
  const int lane = threadIdx.x & 63;
  const long long t = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= tokens) return;
  const T* dr = dy + t * (long long)D;
  for (int j0 = 0; j0 < k; j0 += JB) {
    float s[JB];
#pragma unroll
    for (int jj = 0; jj < JB; jj++) s[jj] = 0.f;
    for (int d = lane * CH; d < D; d += 64 * CH) {
      const int nv = D - d < CH ? D - d : CH;
      Raw ra[JB];
#pragma unroll
      for (int jj = 0; jj < JB; jj++)
        ra[jj] = j0 + jj < k ? raw_load_streaming<T>(z + (t * k + j0 + jj) * (long long)D + d, nv, vec != 0) : raw_zero();
      float b[CH];
      raw_unpack<T>(raw_load<T>(dr + d, nv, vec != 0), b);
#pragma unroll
      for (int jj = 0; jj < JB; jj++) {
        float a[CH];
        raw_unpack<T>(ra[jj], a);
#pragma unroll
        for (int q = 0; q < CH; q++) s[jj] += a[q] * b[q];
      }
    }
    const float v = wave_sum8(s, lane);
    if ((lane & 7) == 0 && j0 + (lane >> 3) < k) out[t * k + j0 + (lane >> 3)] = Elem<T>::cvt(v);
  }
}

// ---- the same two companions for a k-head tensor stored as ADC codes -----------------------------------------
// z[r, d] = ((code[r, d] - 128) * scale[e][0]) * scale[e][1], e = sel[r] (the expert of flat row r = t*k + j).
__device__ __forceinline__ int code_row_expert(const void* sel, int sel_is_i64, long long r) {
  return sel_is_i64 ? (int)static_cast<const long long*>(sel)[r] : static_cast<const int32_t*>(sel)[r];
}
__device__ __forceinline__ void codes_unpack16(const Raw& r, float a, float b, float (&v)[16]) {
#pragma unroll
  for (int w = 0; w < 4; w++)
#pragma unroll
    for (int i = 0; i < 4; i++) v[4 * w + i] = (((float)((r[w] >> (8 * i)) & 0xffu) - 128.0f) * a) * b;
}

// One thread per (token, 16 codes): y[t, d] = sum_j gate[t*k+j] * z[t*k+j, d], fp32, ascending j.  D % 16 == 0.
template <typename T>
__global__ __launch_bounds__(kThreads) void head_reduce_codes_kernel(const uint8_t* __restrict__ codes,
                                                                      const float* __restrict__ scale,
                                                                      const void* __restrict__ sel, int sel_is_i64,
                                                                      const T* __restrict__ gate, T* __restrict__ y,
                                                                      long long rows, int k, int D,
                                                                      long long* counter, long long counter_add) {
  const int chunks = D / 16;
  bump_counter(counter, counter_add);
  const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (idx >= rows * chunks) return;
  const long long t = idx / chunks;
  const int d = (int)(idx % chunks) * 16;
  float acc[16];
#pragma unroll
  for (int q = 0; q < 16; q++) acc[q] = 0.f;
  for (int j = 0; j < k; j++) {
    const long long r = t * k + j;
    const Raw c = __builtin_nontemporal_load(reinterpret_cast<const Raw*>(codes + r * (long long)D + d));
    const int e = code_row_expert(sel, sel_is_i64, r);
    float v[16];
    codes_unpack16(c, scale[2 * e], scale[2 * e + 1], v);
    const float gt = Elem<T>::load(gate + r);
#pragma unroll
    for (int q = 0; q < 16; q++) acc[q] += gt * v[q];
  }
  T* out = y + t * (long long)D + d;
  if constexpr (sizeof(T) == 2) {
    float lo[8], hi[8];
#pragma unroll
    for (int q = 0; q < 8; q++) { lo[q] = acc[q]; hi[q] = acc[8 + q]; }
    store_streaming(out, raw_pack<T>(lo));
    store_streaming(out + 8, raw_pack<T>(hi));
  } else {
#pragma unroll
    for (int q = 0; q < 16; q += 4) {
      float f[4] = {acc[q], acc[q + 1], acc[q + 2], acc[q + 3]};
      store_streaming(out + q, raw_pack<T>(f));
    }
  }
}

// grad_gate[t*k+j] = <z[t*k+j, :], dy[t, :]>.  A wave takes kCodeTokens tokens at once (their loads are all in
// flight together); a lane owns runs of 16 columns.  Each term (c - 128) * dy is formed as fma(c, dy, -128 * dy) on
// the byte as it is: -128 * dy is exact, so the fused operation rounds the exact product (c - 128) * dy once, as a
// multiplication by the signed code would (no large common part that cancels afterwards).  The row's two scale
// factors multiply the finished sum.  D % 16 == 0.
constexpr int kCodeTokens = 2;
template <typename T>
__global__ __launch_bounds__(kThreads) void gate_grad_codes_kernel(const uint8_t* __restrict__ codes,
                                                                    const float* __restrict__ scale,
                                                                    const void* __restrict__ sel, int sel_is_i64,
                                                                    const T* __restrict__ dy, T* __restrict__ out,
                                                                    long long tokens, int k, int D) {
  constexpr int JB = 8, TK = kCodeTokens;
  const int lane = threadIdx.x & 63;
  const long long t0 = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * TK;
  if (t0 >= tokens) return;
  for (int j0 = 0; j0 < k; j0 += JB) {
    float s[TK][JB];
#pragma unroll
    for (int u = 0; u < TK; u++) {
#pragma unroll
      for (int jj = 0; jj < JB; jj++) s[u][jj] = 0.f;
    }
    for (int d = lane * 16; d < D; d += 64 * 16) {
      Raw rc[TK][JB], rd[TK][sizeof(T) == 2 ? 2 : 4];
#pragma unroll
      for (int u = 0; u < TK; u++) {
        const long long t = t0 + u < tokens ? t0 + u : t0;        // a wave past the end repeats its first token
#pragma unroll
        for (int jj = 0; jj < JB; jj++)
          rc[u][jj] = j0 + jj < k ? __builtin_nontemporal_load(reinterpret_cast<const Raw*>(codes + (t * k + j0 + jj) * (long long)D + d))
                                  : raw_zero();
#pragma unroll
        for (int q = 0; q < (sizeof(T) == 2 ? 2 : 4); q++)
          rd[u][q] = *reinterpret_cast<const Raw*>(dy + t * (long long)D + d + q * (16 / (int)sizeof(T)));
      }
#pragma unroll
      for (int u = 0; u < TK; u++) {
        float b[16];
        if constexpr (sizeof(T) == 2) {
          float lo[8], hi[8];
          raw_unpack<T>(rd[u][0], lo);
          raw_unpack<T>(rd[u][1], hi);
#pragma unroll
          for (int q = 0; q < 8; q++) { b[q] = lo[q]; b[8 + q] = hi[q]; }
        } else {
#pragma unroll
          for (int q = 0; q < 4; q++)
#pragma unroll
            for (int i = 0; i < 4; i++) b[4 * q + i] = as_f32(rd[u][q][i]);
        }
        float nb[16];
#pragma unroll
        for (int q = 0; q < 16; q++) nb[q] = -128.0f * b[q];
#pragma unroll
        for (int jj = 0; jj < JB; jj++) {
          float acc = 0.f;
#pragma unroll
          for (int w = 0; w < 4; w++)
#pragma unroll
            for (int i = 0; i < 4; i++)
              acc += fmaf((float)((rc[u][jj][w] >> (8 * i)) & 0xffu), b[4 * w + i], nb[4 * w + i]);
          s[u][jj] += acc;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < TK; u++) {
      const float v = wave_sum8(s[u], lane);
      const int jj = lane >> 3;
      if ((lane & 7) == 0 && j0 + jj < k && t0 + u < tokens) {
        const long long r = (t0 + u) * k + j0 + jj;
        const int e = code_row_expert(sel, sel_is_i64, r);
        out[r] = Elem<T>::cvt((v * scale[2 * e]) * scale[2 * e + 1]);
      }
    }
  }
}

// ---- the sum over the k heads of a per-head input gradient, with the input-range clip applied on the way -----
// The clip mask of row r = t*k + j is |x[t, d]| < ir[e_r, tile(d)]: it depends on the token's input row, shared by
// the k heads, and on one number per (expert, K-tile).  Applied here, the input row is read once per token instead
// of once per head inside the GEMM that makes `full`, and that GEMM keeps no mask tile (cvmm.py:848-893, regrouped;
// the reference masks the rounded product as well):
//   out[t, d]        = sum_j [|x| < ir_j] full[t*k+j, d]                       fp32, ascending j
//   row_part[tile][r] = sum_{d in tile} min([x >= ir] f, 0) - max([x <= -ir] f, 0)   lane's chunks in ascending d, then
//                                                                                   over the lanes in a fixed order
//   count[workgroup]  = number of (r, d) with |x| < ir
// One wave per token (grid-stride); a lane owns 16-byte chunks; the k <= 8 head rows of a chunk are in flight together.
// Tile bounds are multiples of the chunk.
struct HeadClipParams {
  const void* full; const void* x; long long ldx; void* out;
  const void* sel; int sel_is_i64;
  const float* ir; int n_tiles; int bounds[kMaxTiles + 1];
  float* row_part; int32_t* count;
  long long tokens; int k, D;
};

template <typename T>
__global__ __launch_bounds__(kThreads, 4) void head_sum_clip_kernel(const HeadClipParams p) {
  constexpr int CH = Elem<T>::kChunk, JB = 8;
  __shared__ int sCnt[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* __restrict__ FULL = static_cast<const T*>(p.full);
  const T* __restrict__ X = static_cast<const T*>(p.x);
  T* __restrict__ OUT = static_cast<T*>(p.out);
  const int k = p.k, D = p.D;
  const long long M = p.tokens * k;
  int cnt = 0;
  for (long long t = (long long)blockIdx.x * 4 + wave; t < p.tokens; t += (long long)gridDim.x * 4) {
    int ej[JB];
#pragma unroll
    for (int jj = 0; jj < JB; jj++) ej[jj] = jj < k ? code_row_expert(p.sel, p.sel_is_i64, t * k + jj) : 0;
    for (int tile = 0; tile < p.n_tiles; tile++) {
      const int lo = p.bounds[tile], hi = p.bounds[tile + 1];
      float irj[JB], part[JB];
#pragma unroll
      for (int jj = 0; jj < JB; jj++) {
        irj[jj] = p.ir[(long long)ej[jj] * p.n_tiles + tile];
        part[jj] = 0.f;
      }
      for (int d0 = lo; d0 < hi; d0 += 64 * CH) {      // (the same trip count in every lane: the vote below is wave-wide)
        const int d = d0 + lane * CH;
        const bool in = d < hi;
        Raw rf[JB], rx = raw_zero();
#pragma unroll
        for (int jj = 0; jj < JB; jj++)
          rf[jj] = (in && jj < k)
                       ? __builtin_nontemporal_load(reinterpret_cast<const Raw*>(FULL + (t * k + jj) * (long long)D + d))
                       : raw_zero();
        if (in) rx = *reinterpret_cast<const Raw*>(X + t * p.ldx + d);
        float xv[CH], acc[CH];
        raw_unpack<T>(rx, xv);
#pragma unroll
        for (int q = 0; q < CH; q++) {
          acc[q] = 0.f;
          if (!in) xv[q] = __builtin_inff();   // a lane past the tile: clipped everywhere, and its zeros add nothing
        }
#pragma unroll
        for (int jj = 0; jj < JB; jj++) {
          if (jj < k) {
            float v[CH];
            raw_unpack<T>(rf[jj], v);
#pragma unroll
            for (int q = 0; q < CH; q++) {
              const bool clipped = fabsf(xv[q]) >= irj[jj];
              const float toward = as_f32(as_u32(v[q]) ^ (as_u32(xv[q]) & 0x80000000u));   // f * sign(x)
              part[jj] += (clipped && toward < 0.f) ? toward : 0.f;                        // min([clipped] toward, 0)
              cnt += popc64(wave_ballot(!clipped));                                          // (scalar unit; every lane votes)
              acc[q] += clipped ? 0.f : v[q];
            }
          }
        }
        if (in) store_streaming(OUT + t * (long long)D + d, raw_pack<T>(acc));
      }
      const float w1 = wave_sum8(part, lane);          // row lane / 8
      if ((lane & 7) == 0 && (lane >> 3) < k) p.row_part[(long long)tile * M + t * k + (lane >> 3)] = w1;
    }
  }
  if (lane == 0) sCnt[wave] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) p.count[blockIdx.x] = sCnt[0] + sCnt[1] + sCnt[2] + sCnt[3];
}

template <typename T>
__global__ __launch_bounds__(kThreads) void row_abs_max_kernel(const T* __restrict__ x, long long ldx, long long rows,
                                                                int K, float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  float m = 0.f;
  if (row < rows)
    for (int d = lane; d < K; d += 64) m = fmaxf(m, fabsf(Elem<T>::load(x + row * ldx + d)));
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, wave_shfl_xor(m, d));
  if (row < rows && lane == 0) out[row] = m;
}

// cols == N: wmax[e, c] = max_k |w[e, k, c]|.  Workgroup (column block, K slice, expert): a lane owns one 16-byte
// chunk of columns, `width` lanes cover a row (or 64 chunks of it), the rest of the wave and the other three
// waves take further rows; the slice's maxima meet in LDS and merge into the zero-filled output with an atomic
// max on the bit pattern.
template <typename T>
__global__ __launch_bounds__(kThreads) void weight_col_abs_max_kernel(const T* __restrict__ w, int K, int N, int width,
                                                                       float* __restrict__ out, int vec) {
  constexpr int CH = Elem<T>::kChunk;
  __shared__ float red[kThreads][CH + 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rows_per_wave = 64 / width;
  const int chunk = blockIdx.x * 64 + (lane % width);
  const int row_in_block = wave * rows_per_wave + lane / width;
  const int rows_per_block = 4 * rows_per_wave;
  const int d = chunk * CH;
  const int nv = N - d < CH ? N - d : CH;
  const int e = blockIdx.z;
  float m[CH];
#pragma unroll
  for (int q = 0; q < CH; q++) m[q] = 0.f;
  if (nv > 0) {
    const T* base = w + (long long)e * K * N + d;
    for (int k = blockIdx.y * rows_per_block + row_in_block; k < K; k += gridDim.y * rows_per_block) {
      float v[CH];
      raw_unpack<T>(raw_load<T>(base + (long long)k * N, nv, vec != 0), v);
#pragma unroll
      for (int q = 0; q < CH; q++) m[q] = fmaxf(m[q], fabsf(v[q]));
    }
  }
#pragma unroll
  for (int q = 0; q < CH; q++) red[tid][q] = m[q];
  __syncthreads();
  if (row_in_block == 0 && nv > 0) {
    for (int r = 1; r < rows_per_block; r++) {
      const int other = (r / rows_per_wave) * 64 + (r % rows_per_wave) * width + (lane % width);
#pragma unroll
      for (int q = 0; q < CH; q++) m[q] = fmaxf(m[q], red[other][q]);
    }
    for (int q = 0; q < nv; q++) atomicMax(reinterpret_cast<uint32_t*>(out) + (long long)e * N + d + q, as_u32(m[q]));
  }
}
// cols == 1: wmax[e] = max |w[e]|.  grid (chunks, E): every workgroup reduces one slice and
// merges with an atomic max on the bit pattern (non-negative floats order like integers), so the
// output must be zero-filled first (fill_zero_kernel).
__global__ __launch_bounds__(kThreads) void fill_zero_kernel(uint32_t* __restrict__ p, int n) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) p[i] = 0u;
}
__global__ __launch_bounds__(kThreads) void fill_zero2_kernel(uint32_t* __restrict__ a, int na,
                                                               uint32_t* __restrict__ b, int nb) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < na) a[i] = 0u;
  if (i < nb) b[i] = 0u;
}
// fill_zero2_kernel that also makes the two fp32 input-range tables of a layer from its parameter
// ir [2, E, ir_cols] of element type T: ir_up [E, n_up] = ir[0, :, :n_up], ir_dn [E, n_dn] = ir[1, :, :n_dn].
template <typename T>
__global__ __launch_bounds__(kThreads) void layer_tables_prep_kernel(uint32_t* __restrict__ a, uint32_t* __restrict__ b, int E,
                                                                      const T* __restrict__ ir, int ir_cols, int n_up,
                                                                      float* __restrict__ ir_up, int n_dn,
                                                                      float* __restrict__ ir_dn) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < E) { a[i] = 0u; b[i] = 0u; }
  if (ir != nullptr) {
    if (i < E * n_up) ir_up[i] = Elem<T>::to_f32(ir[(long long)(i / n_up) * ir_cols + i % n_up]);
    if (i < E * n_dn) ir_dn[i] = Elem<T>::to_f32(ir[(long long)(E + i / n_dn) * ir_cols + i % n_dn]);
  }
}
// (blockIdx.z picks one of two weight tensors of the same expert count: both tables of a layer from one launch)
template <typename T>
__global__ __launch_bounds__(kThreads) void weight_abs_max_kernel(const T* __restrict__ w, long long per_expert,
                                                                   float* __restrict__ out, int vec,
                                                                   const T* __restrict__ w2 = nullptr,
                                                                   long long per_expert2 = 0,
                                                                   float* __restrict__ out2 = nullptr, int vec2 = 0) {
  __shared__ float red[4];
  const int tid = threadIdx.x, lane = tid & 63;
  if (blockIdx.z == 1) { w = w2; per_expert = per_expert2; out = out2; vec = vec2; }
  const T* base = w + (long long)blockIdx.y * per_expert;
  long long span = (per_expert + gridDim.x - 1) / gridDim.x;
  span = (span + 15) / 16 * 16;             // keep slices 16-byte aligned
  const long long lo = (long long)blockIdx.x * span;
  const long long hi = lo + span < per_expert ? lo + span : per_expert;
  constexpr int CH = Elem<T>::kChunk;
  float m = 0.f;
  // four pieces per thread in flight at a time (the weights are read once: what matters is the loads' latency)
  constexpr int U = 4;
  for (long long i0 = lo + (long long)tid * CH; i0 < hi; i0 += (long long)U * kThreads * CH) {
    Raw r[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const long long i = i0 + (long long)u * kThreads * CH;
      const long long left = hi - i;
      const int nv = left < 0 ? 0 : (left < CH ? (int)left : CH);
      r[u] = raw_load<T>(base + (nv > 0 ? i : lo), nv, vec != 0);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      float v[CH];
      raw_unpack<T>(r[u], v);
#pragma unroll
      for (int q = 0; q < CH; q++) m = fmaxf(m, fabsf(v[q]));
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, wave_shfl_xor(m, d));
  if (lane == 0) red[tid >> 6] = m;
  __syncthreads();
  if (tid == 0) {
    const float r = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    atomicMax(reinterpret_cast<uint32_t*>(out) + blockIdx.y, as_u32(r));
  }
}

// out[e, t] = sum_{i in [offsets[e], offsets[e+1])} v[i, t], one workgroup per (expert, column); columns from n_tiles
// on (gridDim.y may exceed n_tiles) receive zero.  T: element type of out (one rounding of the fp32 sum).
template <typename T>
__global__ __launch_bounds__(kThreads) void segment_sum_kernel(const float* __restrict__ v,
                                                                const int32_t* __restrict__ offsets, int n_tiles,
                                                                T* __restrict__ out, long long ldout) {
  __shared__ float red[4];
  const int e = blockIdx.x, t = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63;
  float s = 0.f;
  if (t < n_tiles)
    for (int i = offsets[e] + tid; i < offsets[e + 1]; i += kThreads) s += v[(long long)i * n_tiles + t];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) s += wave_shfl_xor(s, d);
  if (lane == 0) red[tid >> 6] = s;
  __syncthreads();
  if (tid == 0) out[(long long)e * ldout + t] = Elem<T>::cvt((red[0] + red[1]) + (red[2] + red[3]));
}

__device__ __forceinline__ double block_sum_double(double v, double* red /* LDS [4] */) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += wave_shfl_xor(v, d);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// Two-pass unbiased std over all elements of the rows of one expert (one workgroup per expert).
template <typename T>
__global__ __launch_bounds__(kThreads) void expert_std_kernel(const T* __restrict__ x, long long ldx, int K,
                                                               const int32_t* __restrict__ in_index,
                                                               const int32_t* __restrict__ offsets,
                                                               float* __restrict__ out) {
  __shared__ double red[4];
  const int e = blockIdx.x, tid = threadIdx.x;
  const int lo = offsets[e], hi = offsets[e + 1];
  const long long n = (long long)(hi - lo) * K;
  double s = 0.0;
  for (long long i = tid; i < n; i += kThreads) {
    const int r = lo + (int)(i / K), c = (int)(i % K);
    s += (double)Elem<T>::load(x + (long long)in_index[r] * ldx + c);
  }
  s = block_sum_double(s, red);
  const double mean = n > 0 ? s / (double)n : 0.0;
  double ss = 0.0;
  for (long long i = tid; i < n; i += kThreads) {
    const int r = lo + (int)(i / K), c = (int)(i % K);
    const double d = (double)Elem<T>::load(x + (long long)in_index[r] * ldx + c) - mean;
    ss += d * d;
  }
  ss = block_sum_double(ss, red);
  if (tid == 0) out[e] = (n == 0) ? -0.0f : (float)sqrt(ss / (double)(n - 1));
}

}  // namespace amoe
