// Segmented weight gradient of the CVMM path:
//     grad_w[e][kk][n] = sum_{i in expert e} clamp(x[in_index[i]][kk], +-ir[i,t]) * g[g_index[i]][n]
// One workgroup owns one 128 (kk) x 128 (n) tile of one expert and walks that expert's sorted
// rows in order, so the result needs no atomics, no pre-zeroing and has a fixed summation order.
// Both operands are staged token-major ("RC": [token][feature], as they lie in memory) and
// fed to the matrix unit through the transposing LDS read (bf16) or plain reads (fp32); the
// gradient fragment is the A operand, so a lane holds one kk and runs of 4 consecutive n.
#pragma once
#include "common.h"
#include "gemm_rows.h"

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
__global__ __launch_bounds__(kThreads, 2) void gemm_wgrad_kernel(const WgradParams p) {
  using EL = Elem<T>;
  constexpr int CH = EL::kChunk, MMAK = EL::kMmaK;
  constexpr int BT = EL::kBK;                     // tokens per step
  constexpr int LD = kTileCols + EL::kPadRC;
  constexpr int STAGE = BT * LD;
  constexpr int CPR = kTileCols / CH, RPP = kThreads / CPR;
  constexpr bool IS_BF16 = sizeof(T) == 2;
  static_assert(BT == 4 * RPP, "staging expects 4 passes");

  __shared__ __attribute__((aligned(16))) T sX[2 * STAGE];   // two stages
  __shared__ __attribute__((aligned(16))) T sG[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave >> 1, wk = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  int b = xcd_contiguous_id(blockIdx.x, gridDim.x);
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
  const float ir_expert = (has_ir && p.ir_by_expert) ? p.ir[(int64_t)e * p.n_tiles + kcol.tile] : 1.f;

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][c][i] = 0.f;

  // rows of the step after the one being loaded: indices are fetched one step ahead of the data
  int nx_xi[4], nx_gi[4];
  float nx_ir[4];
  bool nx_ok[4];
  auto load_index = [&](int i0) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int r = i0 + tid / CPR + RPP * i;
      nx_ok[i] = r < seg1;
      nx_xi[i] = nx_ok[i] ? p.in_index[r] : 0;
      nx_gi[i] = nx_ok[i] ? (p.g_index ? p.g_index[r] : nx_xi[i]) : 0;
      nx_ir[i] = (has_ir && !p.ir_by_expert && nx_ok[i]) ? p.ir[(int64_t)r * p.n_tiles + kcol.tile] : ir_expert;
    }
  };
  Raw rx[4], rg[4];
  float st_ir[4], st_gs[4];
  auto load_step = [&]() {                   // global -> registers, rows from nx_*
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int kk = kc0 + chunk * CH;
      int nvx = nx_ok[i] ? kc1 - kk : 0;
      nvx = nvx < 0 ? 0 : (nvx > CH ? CH : nvx);
      rx[i] = raw_load<T>(X + (int64_t)nx_xi[i] * p.ldx + kk, nvx, p.x_vec != 0);
      const int n = n0 + chunk * CH;
      int nvg = nx_ok[i] ? n1 - n : 0;
      nvg = nvg < 0 ? 0 : (nvg > CH ? CH : nvg);
      rg[i] = raw_load<T>(G + (int64_t)nx_gi[i] * p.ldg + n, nvg, p.g_vec != 0);
      st_ir[i] = nx_ir[i];
      st_gs[i] = (GS != nullptr && nx_ok[i]) ? Elem<T>::load(GS + nx_xi[i]) : 1.f;
    }
  };
  // Interior steps (all BT tokens exist, full 128-column tiles, aligned rows): unconditional loads.
  const bool tile_fast = p.x_vec != 0 && p.g_vec != 0 && (kc1 - kc0) == kTileCols && (n1 - n0) == kTileCols;
  auto load_fast = [&]() {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      rx[i] = *reinterpret_cast<const Raw*>(X + (int64_t)nx_xi[i] * p.ldx + kc0 + chunk * CH);
      rg[i] = *reinterpret_cast<const Raw*>(G + (int64_t)nx_gi[i] * p.ldg + n0 + chunk * CH);
      st_ir[i] = nx_ir[i];
      st_gs[i] = GS != nullptr ? Elem<T>::load(GS + nx_xi[i]) : 1.f;
    }
  };
  auto store_step = [&](int buf) {           // registers -> LDS, clip / gate scaling on the way
    T* __restrict__ dX = sX + buf * STAGE;
    T* __restrict__ dG = sG + buf * STAGE;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      Raw x = rx[i], g = rg[i];
      if (has_ir) {
        float v[CH];
        raw_unpack<T>(x, v);
        const float rng = st_ir[i];
#pragma unroll
        for (int j = 0; j < CH; j++) {
          v[j] = v[j] > rng ? rng : v[j];
          v[j] = v[j] < -rng ? -rng : v[j];
        }
        x = raw_pack<T>(v);
      }
      if (GS != nullptr) {
        float v[CH];
        raw_unpack<T>(g, v);
#pragma unroll
        for (int j = 0; j < CH; j++) v[j] *= st_gs[i];
        g = raw_pack<T>(v);
      }
      *reinterpret_cast<Raw*>(&dX[(tid / CPR + RPP * i) * LD + chunk * CH]) = x;
      *reinterpret_cast<Raw*>(&dG[(tid / CPR + RPP * i) * LD + chunk * CH]) = g;
    }
  };

  if (seg0 < seg1) {
    load_index(seg0);
    if (tile_fast && seg0 + BT <= seg1) load_fast(); else load_step();
    load_index(seg0 + BT);
    store_step(0);
  }
  __syncthreads();
  int cur = 0;
  for (int i0 = seg0; i0 < seg1; i0 += BT) {
    const bool more = i0 + BT < seg1;
    if (more) {
      if (tile_fast && i0 + 2 * BT <= seg1) load_fast(); else load_step();
      load_index(i0 + 2 * BT);
    }
    const T* __restrict__ cX = sX + cur * STAGE;
    const T* __restrict__ cG = sG + cur * STAGE;
#pragma unroll
    for (int kk = 0; kk < BT; kk += MMAK) {
      if constexpr (IS_BF16) {
        const int R = lane & 15, gq = (lane >> 4) & 1;
        const int roff = (kk + 8 * lh + (R >> 2)) * LD + 16 * gq + 4 * (R & 3);
        u32x4 gf[2], xf[2];
#pragma unroll
        for (int f = 0; f < 2; f++) {
          const uint16_t* bg = reinterpret_cast<const uint16_t*>(&cG[roff + wn * 64 + f * 32]);
          const uint16_t* bx = reinterpret_cast<const uint16_t*>(&cX[roff + wk * 64 + f * 32]);
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
          gf[f] = cG[(kk + lh) * LD + wn * 64 + f * 32 + l32];
          xf[f] = cX[(kk + lh) * LD + wk * 64 + f * 32 + l32];
        }
#pragma unroll
        for (int fn = 0; fn < 2; fn++)
#pragma unroll
          for (int fk = 0; fk < 2; fk++) acc[fn][fk] = mfma_32x32x2_f32(gf[fn], xf[fk], acc[fn][fk]);
      }
    }
    if (more) store_step(cur ^ 1);
    __syncthreads();
    cur ^= 1;
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
