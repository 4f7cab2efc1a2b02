// Segmented weight gradient of the CVMM path:
//     grad_w[e][kk][n] = sum_{i in expert e} clamp(x[in_index[i]][kk], +-ir[i,t]) * g[g_index[i]][n]
// One workgroup owns one 128 (kk) x 128 (n) tile of one expert and walks that expert's sorted
// rows in order, so the result needs no atomics, no pre-zeroing and has a fixed summation order.
// Both operands are staged token-major ("RC": [token][feature], as they lie in memory) and
// fed to the matrix unit through the transposing LDS read (bf16) or plain reads (fp32); the
// gradient fragment is the A operand, so a lane holds one kk and runs of 4 consecutive n.
#pragma once
#include "common.h"

namespace amoe {

struct WgradParams {
  int M, N, K, E;
  const void* x; int64_t ldx;
  const void* g; int64_t ldg;
  void* grad_w;
  const int32_t* offsets; const int32_t* in_index; const int32_t* g_index;
  const float* ir; int ir_by_expert; const void* g_scale; int n_tiles; int bounds[kMaxTiles + 1];
  int n_k_blocks, n_n_blocks;
  int x_vec, g_vec, out_vec;
};

template <typename T>
__global__ __launch_bounds__(kThreads) void gemm_wgrad_kernel(const WgradParams p) {
  using EL = Elem<T>;
  constexpr int CH = EL::kChunk, MMAK = EL::kMmaK;
  constexpr int BT = EL::kBK;                     // tokens per step
  constexpr int LD = kTileCols + EL::kPadRC;
  constexpr int CPR = kTileCols / CH, RPP = kThreads / CPR;
  constexpr bool IS_BF16 = sizeof(T) == 2;
  static_assert(BT == 4 * RPP, "staging expects 4 passes");

  __shared__ __attribute__((aligned(16))) T sX[BT * LD];
  __shared__ __attribute__((aligned(16))) T sG[BT * LD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave >> 1, wk = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  int b = blockIdx.x;
  const int nb = b % p.n_n_blocks; b /= p.n_n_blocks;
  const int kb = b % p.n_k_blocks;
  const int e = b / p.n_k_blocks;
  const ColBlock kcol = find_col_block(p.bounds, p.n_tiles, kb);
  const int kc0 = kcol.c0, kc1 = kcol.c1;
  const int n0 = nb * kTileCols, n1 = (n0 + kTileCols < p.N) ? n0 + kTileCols : p.N;
  const int seg0 = p.offsets[e], seg1 = p.offsets[e + 1];

  const T* __restrict__ X = static_cast<const T*>(p.x);
  const T* __restrict__ G = static_cast<const T*>(p.g);
  const T* __restrict__ GS = static_cast<const T*>(p.g_scale);
  const bool has_ir = p.ir != nullptr;
  const int chunk = tid % CPR;

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][c][i] = 0.f;

  Chunk<T> rx[4], rg[4];
  auto load_step = [&](int i0) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int r = i0 + tid / CPR + RPP * i;
      const bool ok = r < seg1;
      const int xi = ok ? p.in_index[r] : 0;
      const int gi = ok ? (p.g_index ? p.g_index[r] : xi) : 0;
      const int kk = kc0 + chunk * CH;
      int nvx = ok ? kc1 - kk : 0;
      nvx = nvx < 0 ? 0 : (nvx > CH ? CH : nvx);
      rx[i] = chunk_load<T>(X + (int64_t)xi * p.ldx + kk, nvx, p.x_vec != 0);
      if (has_ir && ok) {
        const float rng = p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.n_tiles + kcol.tile];
#pragma unroll
        for (int j = 0; j < CH; j++) {
          float v = rx[i].v[j];
          v = v > rng ? rng : v;
          v = v < -rng ? -rng : v;
          rx[i].v[j] = v;
        }
      }
      const int n = n0 + chunk * CH;
      int nvg = ok ? n1 - n : 0;
      nvg = nvg < 0 ? 0 : (nvg > CH ? CH : nvg);
      rg[i] = chunk_load<T>(G + (int64_t)gi * p.ldg + n, nvg, p.g_vec != 0);
      if (GS != nullptr && ok) {
        const float sc = Elem<T>::load(GS + xi);
#pragma unroll
        for (int j = 0; j < CH; j++) rg[i].v[j] *= sc;
      }
    }
  };

  if (seg0 < seg1) load_step(seg0);
  for (int i0 = seg0; i0 < seg1; i0 += BT) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      chunk_store_lds<T>(&sX[(tid / CPR + RPP * i) * LD + chunk * CH], rx[i]);
      chunk_store_lds<T>(&sG[(tid / CPR + RPP * i) * LD + chunk * CH], rg[i]);
    }
    __syncthreads();
    if (i0 + BT < seg1) load_step(i0 + BT);
#pragma unroll
    for (int kk = 0; kk < BT; kk += MMAK) {
      if constexpr (IS_BF16) {
        const int R = lane & 15, gq = (lane >> 4) & 1;
        const int roff = (kk + 8 * lh + (R >> 2)) * LD + 16 * gq + 4 * (R & 3);
        u32x4 gf[2], xf[2];
#pragma unroll
        for (int f = 0; f < 2; f++) {
          const uint16_t* bg = reinterpret_cast<const uint16_t*>(&sG[roff + wn * 64 + f * 32]);
          const uint16_t* bx = reinterpret_cast<const uint16_t*>(&sX[roff + wk * 64 + f * 32]);
          u32x2 glo = lds_read_tr16_b64(bg), ghi = lds_read_tr16_b64(bg + 4 * LD);
          u32x2 xlo = lds_read_tr16_b64(bx), xhi = lds_read_tr16_b64(bx + 4 * LD);
          gf[f] = u32x4{glo[0], glo[1], ghi[0], ghi[1]};
          xf[f] = u32x4{xlo[0], xlo[1], xhi[0], xhi[1]};
        }
#pragma unroll
        for (int fn = 0; fn < 2; fn++)
#pragma unroll
          for (int fk = 0; fk < 2; fk++) acc[fn][fk] = mfma_32x32x16_bf16(gf[fn], xf[fk], acc[fn][fk]);
      } else {
        float gf[2], xf[2];
#pragma unroll
        for (int f = 0; f < 2; f++) {
          gf[f] = sG[(kk + lh) * LD + wn * 64 + f * 32 + l32];
          xf[f] = sX[(kk + lh) * LD + wk * 64 + f * 32 + l32];
        }
#pragma unroll
        for (int fn = 0; fn < 2; fn++)
#pragma unroll
          for (int fk = 0; fk < 2; fk++) acc[fn][fk] = mfma_32x32x2_f32(gf[fn], xf[fk], acc[fn][fk]);
      }
    }
    __syncthreads();
  }

  T* __restrict__ GW = static_cast<T*>(p.grad_w) + (int64_t)e * p.K * p.N;
#pragma unroll
  for (int fk = 0; fk < 2; fk++) {
    const int kk = kc0 + wk * 64 + fk * 32 + l32;
    if (kk >= kc1) continue;
#pragma unroll
    for (int fn = 0; fn < 2; fn++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int n = n0 + wn * 64 + fn * 32 + 8 * q + 4 * lh;
        int nv = n1 - n;
        nv = nv < 0 ? 0 : (nv > 4 ? 4 : nv);
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = acc[fn][fk][4 * q + j];
        if (nv > 0) store4<T>(GW + (int64_t)kk * p.N + n, v, nv, p.out_vec != 0);
      }
    }
  }
}

}  // namespace amoe
