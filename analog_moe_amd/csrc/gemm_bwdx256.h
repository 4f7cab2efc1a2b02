// Input gradient of the CVMM path for the usual training shapes (bf16 or fp16, every tile interior, one input range per
// expert and K-tile): the 128 x 256 counterpart of MODE_BWDX in gemm_rows.h, same arithmetic in the same order.
//     G = g[g_index[i], :] @ W[e]^T                  (contraction over the forward's output features, which are
//                                                      contiguous in W: both operands are staged k-contiguous)
//     masks, input-range partial sums, gate scaling   (cvmm.py:848-888), from the forward-input tile behind them
// A gathered gradient row is fetched once per 256 output columns.  The forward-input tile the masks need
// (128 x 256 values) passes through LDS in two halves of 64 rows next to the staged output half; its loads are
// issued during the last K step (first half) and during the first half's output stage (second half).
#pragma once
#include <type_traits>

#include "gemm_fwd256.h"

namespace amoe {

// MASKS: the forward input is read for the clip mask against the input range (infinite if there is none) and, with
// RELU, for the ReLU mask.  XC: also leave gate * clamp(x, +-ir) at the rows of x (needs MASKS).  The optional gate
// scales the result in every variant.
template <typename T, bool MASKS, bool RELU, bool XC, int COLS = kFCols>
__global__ __launch_bounds__(kThreads, COLS == 128 ? 3 : 2) void bwdx256_kernel(const RowsParams p) {
  static_assert(sizeof(T) == 2, "16-bit elements: bf16 (as bits) or fp16");
  static_assert(COLS == 128 || COLS == 256, "output columns per workgroup tile");
  constexpr int BK = kFBK, CH = 8;
  constexpr int LDA = BK + 8, LDB = BK + 8;
  constexpr int A_ELEMS = kTileRows * LDA, B_ELEMS = COLS * LDB;
  constexpr int STAGE = A_ELEMS + B_ELEMS;            // 256 columns: 15360 elements = 30 KB
  constexpr int NB = COLS / 64;                       // rows of W per thread and step; 32-column blocks per wave
  constexpr int WCOLS = COLS / 2;                     // columns per wave
  constexpr int CPR = COLS / CH, RPP = kThreads / CPR;   // 16-byte pieces per row of a staged half tile; rows per pass
  constexpr int LDO = COLS + 8;
  constexpr int HALF_ROWS = 64;
  constexpr int HALF = HALF_ROWS * LDO;               // one staged half tile: 33 KB
  constexpr int LDS_ELEMS = (2 * STAGE > 2 * HALF) ? 2 * STAGE : 2 * HALF;
  static_assert((!XC && !RELU) || MASKS, "the clipped input and the ReLU mask are made from the mask tile");

  __shared__ __attribute__((aligned(16))) T sStage[LDS_ELEMS];
  __shared__ float sRed[2][kTileRows];
  __shared__ int sOrow[kTileRows];
  __shared__ int sXrow[kTileRows];
  __shared__ int sDesc[kMaxDesc][4];
  __shared__ int sCnt[4];
  __shared__ int sWave[4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;
  const int ncb = p.n_col_blocks;

  // ---- this workgroup's work items (row tile, column block), as in gemm_rows_kernel ------------------------
  const int per = (p.E + kThreads - 1) / kThreads;
  const int e_first = tid * per;
  int mine = 0;
  for (int j = 0; j < per; j++) {
    const int e = e_first + j;
    if (e < p.E) mine += (p.offsets[e + 1] - p.offsets[e] + kTileRows - 1) / kTileRows;
  }
  int incl = mine;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = wave_shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == 63) sWave[wave] = incl;
  __syncthreads();
  int tiles_before = incl - mine;
  for (int w = 0; w < wave; w++) tiles_before += sWave[w];
  const int total_rt = sWave[0] + sWave[1] + sWave[2] + sWave[3];
  const int total_work = total_rt * ncb;
  const int lb = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int G = (int)gridDim.x;
  const int n_my = lb < total_work ? (total_work - lb + G - 1) / G : 0;
  {
    int t = tiles_before;
    for (int j = 0; j < per; j++) {
      const int e = e_first + j;
      if (e < p.E) {
        const int lo = p.offsets[e], hi = p.offsets[e + 1];
        const int nt = (hi - lo + kTileRows - 1) / kTileRows;
        if (nt > 0) {
          const int wlo = t * ncb, whi = (t + nt) * ncb;
          int i = wlo > lb ? (wlo - lb + G - 1) / G : 0;
          for (; i < n_my && i < kMaxDesc && lb + i * G < whi; i++) {
            const int rt = (lb + i * G) / ncb;
            const int r0 = lo + (rt - t) * kTileRows;
            sDesc[i][0] = e;
            sDesc[i][1] = r0;
            sDesc[i][2] = r0 + kTileRows < hi ? r0 + kTileRows : hi;
          }
        }
        t += nt;
      }
    }
  }
  __syncthreads();

  const T* __restrict__ A = static_cast<const T*>(p.a);
  T* __restrict__ OUT = static_cast<T*>(p.out);
  const T* __restrict__ XF = static_cast<const T*>(p.xf);
  const T* __restrict__ GATE = static_cast<const T*>(p.gate);
  const BufRsrc rsrcA = make_rsrc(A);
  const bool use_ir = MASKS && p.ir != nullptr;
  const float kInf = __builtin_inff();
  int cnt = 0;                                  // un-clipped inputs seen by this wave

  const int a_row = tid >> 2, a_chunk = tid & 3;          // A: rows a_row, a_row + 64; B: rows a_row + 64 * i, i < 4
  int n_idx[2] = {0, 0}, n_orow = -1, n_xrow = 0;
  auto fetch_rows = [&](int i) {
    if (i >= n_my) return;
    const int r0 = sDesc[i][1], r1 = sDesc[i][2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const int r = r0 + a_row + 64 * q;
      n_idx[q] = p.a_index[r < r1 ? r : r0];
    }
    if (tid < kTileRows) {
      const int r = r0 + tid;
      n_orow = r < r1 ? p.out_index[r] : -1;
      if (MASKS) n_xrow = p.xf_index[r < r1 ? r : r0];
    }
  };
  fetch_rows(0);

  for (int it = 0; it < n_my; it++) {
    const int w = lb + it * G;
    const int rt = w / ncb, cb = w - rt * ncb;
    const int e = wave_uniform(sDesc[it][0]), row0 = wave_uniform(sDesc[it][1]), row_end = wave_uniform(sDesc[it][2]);
    uint32_t a_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) a_off[i] = (uint32_t)(((int64_t)n_idx[i] * p.lda + a_chunk * CH) * 2);
    if (tid < kTileRows) {
      sOrow[tid] = n_orow;
      if (MASKS) sXrow[tid] = n_xrow;
    }
    fetch_rows(it + 1);
    const ColBlock colb = find_col_block(p.col_bounds, p.n_col_tiles, cb, COLS);
    const int c0 = colb.c0;
    const T* __restrict__ W = static_cast<const T*>(p.w) + (int64_t)e * p.w_se;
    const BufRsrc rsrcW = make_rsrc(W);
    uint32_t w_off[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) w_off[i] = (uint32_t)(((int64_t)(c0 + a_row + 64 * i) * p.w_snd + a_chunk * CH) * 2);

    f32x16 acc[NB][2];
#pragma unroll
    for (int a = 0; a < NB; a++)
#pragma unroll
      for (int b = 0; b < 2; b++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

    const int nsteps = p.KD / BK;
    Raw ra[2], rb[NB];
    auto load_step = [&](int s) {
#pragma unroll
      for (int i = 0; i < 2; i++) ra[i] = buffer_load_b128(rsrcA, a_off[i], s * (BK * 2));
#pragma unroll
      for (int i = 0; i < NB; i++) rb[i] = buffer_load_b128(rsrcW, w_off[i], s * (BK * 2));
    };
    auto store_step = [&](int buf) {
      T* __restrict__ dA = sStage + buf * STAGE;
      T* __restrict__ dB = dA + A_ELEMS;
#pragma unroll
      for (int i = 0; i < 2; i++) *reinterpret_cast<Raw*>(&dA[(a_row + 64 * i) * LDA + a_chunk * CH]) = ra[i];
#pragma unroll
      for (int i = 0; i < NB; i++) *reinterpret_cast<Raw*>(&dB[(a_row + 64 * i) * LDB + a_chunk * CH]) = rb[i];
    };
    auto multiply_group = [&](const T* __restrict__ cA, const T* __restrict__ cB, int kk) {
      u32x4 xf[2], wf[NB];
#pragma unroll
      for (int ti = 0; ti < 2; ti++)
        xf[ti] = *reinterpret_cast<const u32x4*>(&cA[(wr * 64 + ti * 32 + l32) * LDA + kk + 8 * lh]);
#pragma unroll
      for (int fi = 0; fi < NB; fi++)
        wf[fi] = *reinterpret_cast<const u32x4*>(&cB[(wc * WCOLS + fi * 32 + l32) * LDB + kk + 8 * lh]);
#pragma unroll
      for (int fi = 0; fi < NB; fi++)
#pragma unroll
        for (int ti = 0; ti < 2; ti++) acc[fi][ti] = mfma_32x32x16<T>(wf[fi], xf[ti], acc[fi][ti]);
    };
    // the forward-input rows of one half of the tile: 64 rows x CPR pieces, 64 / RPP per thread (rows tid / CPR + RPP i)
    constexpr int NX = HALF_ROWS / RPP;
    Raw xr[MASKS ? NX : 1];
    auto load_x_half = [&](int h) {
      if constexpr (MASKS) {
#pragma unroll
        for (int i = 0; i < NX; i++) {
          const int rl = tid / CPR + RPP * i;
          const int rt = (rl >> 5) * 64 + h * 32 + (rl & 31);
          const Raw* src = reinterpret_cast<const Raw*>(XF + (int64_t)sXrow[rt] * p.ldxf + c0 + (tid % CPR) * CH);
          // (with the clipped input written back, every row of x belongs to one sorted position: read once)
          xr[i] = XC ? __builtin_nontemporal_load(src) : *src;
        }
      }
    };
    auto park_x_half = [&](T* __restrict__ sX) {
      if constexpr (MASKS) {
#pragma unroll
        for (int i = 0; i < NX; i++)
          *reinterpret_cast<Raw*>(&sX[(tid / CPR + RPP * i) * LDO + (tid % CPR) * CH]) = xr[i];
      }
    };

    load_step(0);
    store_step(0);
    __syncthreads();
    if (nsteps > 1) load_step(1);
    for (int s = 0; s + 1 < nsteps; s++) {
      const T* __restrict__ cA = sStage + (s & 1) * STAGE;
      multiply_group(cA, cA + A_ELEMS, 0);
      multiply_group(cA, cA + A_ELEMS, 16);
      store_step((s + 1) & 1);
      if (s + 2 < nsteps) load_step(s + 2);
      __syncthreads();
    }
    {
      const T* __restrict__ cA = sStage + ((nsteps - 1) & 1) * STAGE;
      load_x_half(0);                             // the staging registers of the operands are idle now
      multiply_group(cA, cA + A_ELEMS, 0);
      multiply_group(cA, cA + A_ELEMS, 16);
      __syncthreads();
    }

    // ---- output stage: the first 32-row block of every wave, then the second (all four waves work in both) ------
    // Row j of a staged half tile is row (j / 32) * 64 + h * 32 + j % 32 of the tile.
    T* __restrict__ sX = sStage;                 // forward-input half tile (then: its clipped, gate-scaled image)
    T* __restrict__ sO = sStage + HALF;          // staged output half tile
    const float ir_r = use_ir ? p.ir[(int64_t)e * p.ir_cols + colb.tile] : kInf;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if constexpr (MASKS) {
        park_x_half(sX);
        __syncthreads();
      }
      {
        const int rl = wr * 32 + l32;                         // row within the half
        const int rt = wr * 64 + h * 32 + l32;                // row within the tile
        const bool valid = row0 + rt < row_end;
        const int orow = valid ? sOrow[rt] : 0;
        const float gate_r = (valid && GATE != nullptr) ? Elem<T>::load(GATE + orow) : 1.f;
        const uint64_t valid_lanes = wave_ballot(valid);
        float part = 0.f;
#pragma unroll
        for (int fi = 0; fi < NB; fi++) {
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int cl = wc * WCOLS + fi * 32 + 8 * q + 4 * lh;
            float v[4];
            if constexpr (MASKS) {
              float xv[4];
              load4<T>(&sX[rl * LDO + cl], xv, 4, true);
#pragma unroll
              for (int j = 0; j < 4; j++) {
                // A clipped input passes no gradient on; the gate-scaled gradient it would have passed goes to
                // the input range instead: min(gs, 0) above the range, -max(gs, 0) = min(-gs, 0) below it.
                const float gs = acc[fi][h][4 * q + j] * gate_r;
                const bool clipped = fabsf(xv[j]) >= ir_r;
                const float toward = as_f32(as_u32(gs) ^ (as_u32(xv[j]) & 0x80000000u));     // gs * sign(x)
                part += fminf(clipped ? toward : 0.f, 0.f);
                cnt += popc64(wave_ballot(!clipped) & valid_lanes);                            // (scalar unit)
                const bool keep = RELU ? (!clipped && xv[j] > 0.f) : !clipped;
                v[j] = keep ? gs : 0.f;
              }
              if constexpr (XC) {
#pragma unroll
                for (int j = 0; j < 4; j++) xv[j] = clamp_sym(xv[j], ir_r) * gate_r;
                store4<T>(&sX[rl * LDO + cl], xv, 4, true);
              }
            } else {
#pragma unroll
              for (int j = 0; j < 4; j++) v[j] = acc[fi][h][4 * q + j] * gate_r;
            }
            store4<T>(&sO[rl * LDO + cl], v, 4, true);
          }
        }
        if (use_ir) {
          part += wave_shfl_xor(part, 32);
          if (lh == 0) sRed[wc][rt] = part;
        }
      }
      if (MASKS && h == 0) load_x_half(1);        // in flight while the first half leaves
      __syncthreads();
      {
        constexpr int OCPR = CPR, ORPP = RPP;
#pragma unroll
        for (int i0 = 0; i0 < HALF_ROWS / ORPP; i0 += 4) {
          Raw seg[4], segx[XC ? 4 : 1];
          int orow[4], xrow[4];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int rl = tid / OCPR + ORPP * (i0 + i);
            const int rt = (rl >> 5) * 64 + h * 32 + (rl & 31);
            orow[i] = sOrow[rt];
            seg[i] = *reinterpret_cast<const Raw*>(&sO[rl * LDO + (tid % OCPR) * CH]);
            if constexpr (XC) {
              xrow[i] = sXrow[rt];
              segx[i] = *reinterpret_cast<const Raw*>(&sX[rl * LDO + (tid % OCPR) * CH]);
            }
          }
#pragma unroll
          for (int i = 0; i < 4; i++) {
            if (orow[i] >= 0) {
              store_streaming(OUT + (int64_t)orow[i] * p.ldo + c0 + (tid % OCPR) * CH, seg[i]);
              if constexpr (XC)
                store_streaming(static_cast<T*>(p.xc_out) + (int64_t)xrow[i] * p.ldxc + c0 + (tid % OCPR) * CH, segx[i]);
            }
          }
        }
      }
      __syncthreads();
    }
    if (use_ir) {
      if (tid < kTileRows && row0 + tid < row_end)
        p.irg_partial[(int64_t)cb * p.M + row0 + tid] = sRed[0][tid] + sRed[1][tid];
      __syncthreads();
    }
  }

  if (use_ir) {
    if (lane == 0) sCnt[wave] = cnt;
    __syncthreads();
    if (tid == 0) p.notclip_count[blockIdx.x] = sCnt[0] + sCnt[1] + sCnt[2] + sCnt[3];
  }
}

}  // namespace amoe
