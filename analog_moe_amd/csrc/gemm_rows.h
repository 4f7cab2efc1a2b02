// Row-gather GEMM of the CVMM path: for every sorted position i of expert e
//     out[out_index[i], :] = epilogue( prologue(a[a_index[i], :]) @ W[e] )
// One kernel serves the analog forward (DAC prologue; noise / ADC / rescale epilogue, optional
// K-tile split) and the input gradient (plain prologue; clip mask, input-range gradient and
// gate scaling in the epilogue).
//
// Workgroup = 256 threads = 2 x 2 waves over a 128 (rows) x 128 (columns) output tile; each
// wave owns 64 x 64 = 2 x 2 MFMA 32x32 tiles.  The matrix instruction is issued with the
// weight fragment as its A operand and the token fragment as its B operand, so a lane ends up
// holding ONE token row (lane % 32) and runs of 4 consecutive output columns: per-row scalars
// (input range, abs-max, gate, scatter row) are per-lane scalars and stores are 4-wide.
//
// LDS layouts:  "KC" [row][k] for operands whose contraction index is contiguous in memory
// (read with one 16-byte ds_read per fragment), "RC" [k][col] for weights whose output column
// is contiguous (bf16: read with the transposing ds_read_b64_tr_b16; fp32: plain reads).
#pragma once
#include "common.h"

namespace amoe {

enum { MODE_FWD = 0, MODE_FWD_SPLIT = 1, MODE_BWDX = 2 };

// DAC code of a value already clamped to +-r: round((x / r) / res) to nearest even, bit-identical to the two
// correctly rounded divisions of the reference's tensor expression (cvmm.py:150-167).  fp32 operands take the two
// divisions.  bf16 operands -- whose gathered rows pass this stage once per block of output columns, where ten
// instructions per element held the vector ALU longer than the matrix instructions hold the matrix pipe -- take one
// multiplication by kq = (1 / r) * (1 / res); the product is within 6 * 2^-24 (relative) of the double-rounded
// quotient, so the two can only round differently when the product lies within 6 * 2^-24 * (1 / res + 1) of a
// half-integer.  dac_code() tracks the largest distance from the rounded code it has seen; when that exceeds
// dac_tie_margin(1 / res) the caller redoes its values with dac_code_exact (one chunk in ten thousand for 8 bits).
__device__ __forceinline__ float dac_tie_margin(float resinv) { return 0.5f - 4.0e-7f * (resinv + 1.0f); }
__device__ __forceinline__ float dac_code_exact(float x, float r, float rinv, float res, float resinv) {
  return rintf(div_by(div_by(x, r, rinv), res, resinv));
}
template <bool IS_BF16>
__device__ __forceinline__ float dac_code(float x, float r, float rinv, float res, float resinv, float kq,
                                          float& tie_dist) {
  if constexpr (IS_BF16) {
    const float q = x * kq, c = rintf(q);
    tie_dist = fmaxf(tie_dist, fabsf(q - c));
    return c;
  } else {
    return dac_code_exact(x, r, rinv, res, resinv);
  }
}

struct RowsParams {
  int M, E;
  int KD, ND;                       // contraction length, output columns
  const void* a; int64_t lda;       // gathered operand rows [*, KD]
  const void* w; int64_t w_se, w_skd, w_snd;  // element strides of W[e][kd][nd]
  void* out; int64_t ldo;           // [*, ND]
  const int32_t* offsets; const int32_t* a_index; const int32_t* out_index;
  int n_kd_tiles; int kd_bounds[kMaxTiles + 1];   // contraction split (forward K-tiles)
  int n_col_tiles; int col_bounds[kMaxTiles + 1]; // column split (input gradient: K-tiles of x)
  int n_col_blocks;
  // forward
  const float* ir; int ir_cols; int ir_by_expert; const float* abs_max; float inp_res;
  const float* noise; int64_t noise_ts, ldnoise; float noise_std; uint64_t seed; const uint64_t* seed_dev;
  const float* wmax; int wmax_cols; float out_bound, out_half_states; int relu;
  int32_t* range_flag;
  void* xq_out; int64_t ldxq; const float* xq_ir; float xq_inp_res; int xq_stage, xq_vec;  // DAC image of the result
  int a_prequant;                    // the gathered operand already is such an image: no input stage
  uint8_t* code_out; int64_t ldcode; float* code_scale_out;   // the result as ADC codes + 128 (gemm_fwd256.h)
  // input gradient
  const void* xf; int64_t ldxf; const int32_t* xf_index; const void* gate;
  float* irg_partial; int32_t* notclip_count; int relu_mask;
  void* xc_out; int64_t ldxc; int xc_vec;   // gate * clamp(x): the weight gradient's x operand, made once here
  // vector-access permissions (alignment checked on the host)
  int a_vec, w_vec, out_vec, out_stage, noise_vec, xf_vec;   // out_stage: 16-byte row segments
  int buf_ok;   // operands small enough for 32-bit byte offsets (buffer loads in the interior path)
};

// Workgroups are handed to the 8 XCDs round-robin; this maps the hardware id to a logical id so
// that each XCD (one L2) works on a contiguous range of logical tiles.
__device__ __forceinline__ int xcd_contiguous_id(int b, int grid) {
  const int q = grid >> 3, r = grid & 7;
  const int xcd = b & 7, idx = b >> 3;
  return xcd * q + (xcd < r ? xcd : r) + idx;
}

constexpr int kMaxDesc = 64;   // row tiles one workgroup can own (the host sizes the grid for it)

// Persistent workgroups: the work items (row tile, column block), column block fastest, are dealt
// round-robin to the workgroups (item w goes to logical workgroup w % gridDim.x).  Neighbouring
// workgroups -- which the id remap keeps on one XCD -- therefore work on the column blocks of
// the SAME row tile at the same time, so the gathered rows are read from HBM once and found in
// that XCD's L2 by the others; the same holds for the weight tiles of consecutive row tiles.
//
// FAST instantiations serve launches whose every tile is interior (the host checks: 16-byte
// aligned operands, column tiles that are multiples of 128, K tiles that are multiples of the K
// step, 32-bit addressable operands, no per-row abs-max scaling); they carry none of the
// element-wise edge code.
template <typename T, bool W_KC, int MODE, bool FAST>
__global__ __launch_bounds__(kThreads, 2) void gemm_rows_kernel(const RowsParams p) {
  using EL = Elem<T>;
  constexpr int BK = EL::kBK, CH = EL::kChunk, MMAK = EL::kMmaK;
  constexpr int LDA = BK + EL::kPadKC;
  constexpr int LDB = W_KC ? (BK + EL::kPadKC) : (kTileCols + EL::kPadRC);
  constexpr int A_ELEMS = kTileRows * LDA;
  constexpr int B_ELEMS = W_KC ? kTileCols * LDB : BK * LDB;
  constexpr int STAGE = A_ELEMS + B_ELEMS;
  constexpr bool IS_BF16 = sizeof(T) == 2;
  constexpr bool FWD = MODE != MODE_BWDX;
  // output staging in LDS: rows of 128 columns + 16 bytes, as many rows per pass as one stage holds
  constexpr int LDO = kTileCols + 16 / (int)sizeof(T);
  constexpr int OUT_PASSES = IS_BF16 ? 1 : 2;
  constexpr int OUT_ROWS = kTileRows / OUT_PASSES;
  static_assert(OUT_ROWS * LDO <= (IS_BF16 ? STAGE : 2 * STAGE), "output staging must fit the stage buffers");

  __shared__ __attribute__((aligned(16))) T sStage[2 * STAGE];
  __shared__ __attribute__((aligned(16))) float sCol[4][kTileCols];
  __shared__ float sRed[2][kTileRows];
  __shared__ int sOrow[kTileRows];
  __shared__ int sXrow[kTileRows];                // rows of the forward input of the tile (MODE_BWDX)
  __shared__ int sDesc[kMaxDesc][4];
  __shared__ int sCnt[4];
  __shared__ int sWave[4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;
  const int ncb = p.n_col_blocks;

  // ---- this workgroup's range of work items ----------------------------------------------------
  // tiles per expert -> exclusive prefix (thread tid owns experts [tid*per, (tid+1)*per))
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
  const int n_my = lb < total_work ? (total_work - lb + G - 1) / G : 0;   // items lb, lb+G, ...
  int cnt = 0;                                       // un-clipped inputs seen by this lane (MODE_BWDX)
  {
    // descriptors (expert, first sorted position, end position) of the row tiles of my items
    int t = tiles_before;
    for (int j = 0; j < per; j++) {
      const int e = e_first + j;
      if (e < p.E) {
        const int lo = p.offsets[e], hi = p.offsets[e + 1];
        const int nt = (hi - lo + kTileRows - 1) / kTileRows;
        if (nt > 0) {
          // items whose row tile lies in [t, t+nt): w in [t*ncb, (t+nt)*ncb)
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
  const bool has_ir = FWD && p.ir != nullptr;
  const bool has_amax = !FAST && FWD && p.abs_max != nullptr;
  const bool quant = FWD && p.inp_res > 0.f;
  const bool prequant = FWD && p.a_prequant != 0;          // the caller did the input stage already
  const bool dac = (has_ir || has_amax || quant) && !prequant;
  const bool dac_ir_quant = has_ir && quant && !has_amax && !prequant;   // the common analog case: tight code
  const bool codes_mode = IS_BF16 && quant;   // feed integer codes, scale the accumulator
  const bool adc_clip = FWD && p.out_bound > 0.f;
  const bool adc_quant = adc_clip && p.out_half_states > 0.f;
  const bool gen_noise = FWD && p.noise == nullptr && p.noise_std > 0.f;
  const uint64_t seed = p.seed + ((gen_noise && p.seed_dev != nullptr) ? *p.seed_dev : 0);
  const float inv_res = quant ? 1.0f / p.inp_res : 0.f;
  const float tie_margin = dac_tie_margin(inv_res);
  const bool use_ir_bw = !FWD && p.ir != nullptr;
  // no analog output stage at all: the K-tile result is the accumulator itself
  const bool plain_epi = !codes_mode && p.noise == nullptr && !gen_noise && !adc_clip && !has_amax && !has_ir;

  const int a_chunk = tid & 7;
  constexpr int CPR = kTileCols / CH, RPP = kThreads / CPR;
  static_assert(BK == 4 * RPP, "RC staging expects 4 passes");

  // state of the current row tile
  int e = 0, row0 = 0, row_end = 0, cur_rt = -1;
  const T* a_row[4];
  uint32_t a_off[4];                      // byte offset of (row, chunk) from A, interior path
  bool a_ok[4];
  float a_amax[4], a_amax_inv[4];
#pragma unroll
  for (int i = 0; i < 4; i++) { a_row[i] = A; a_off[i] = 0; a_ok[i] = false; a_amax[i] = a_amax_inv[i] = 1.f; }
  const BufRsrc rsrcA = make_rsrc(A);

  // row indices of the next item, fetched while the current one is multiplied
  int n_idx[4] = {0, 0, 0, 0}, n_orow = -1, n_xrow = 0;
  // input gradient, bf16, edge-free: the forward-input tile behind the clip / ReLU masks is read as
  // whole row segments during the last K step and handed to the epilogue through LDS
  const bool xf_stage = FAST && IS_BF16 && !FWD && p.xf != nullptr;
  auto fetch_rows = [&](int i) {
    if (i >= n_my) return;
    const int r0 = sDesc[i][1], r1 = sDesc[i][2];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int r = r0 + (tid >> 3) + 32 * q;
      // rows past the tile read the tile's first row: safe to load, never stored
      n_idx[q] = p.a_index[r < r1 ? r : r0];
    }
    if (tid < kTileRows) {
      const int r = r0 + tid;
      n_orow = r < r1 ? (p.out_index ? p.out_index[r] : p.a_index[r]) : -1;
      if (xf_stage) n_xrow = p.xf_index[r < r1 ? r : r0];
    }
  };
  fetch_rows(0);

  for (int it = 0; it < n_my; it++) {
    const int w = lb + it * G;
    const int rt = w / ncb, cb = w - rt * ncb;
    {                                       // this item's row tile: gather pointers, scatter rows
      cur_rt = rt;
      // (the same for every lane: kept in scalar registers, and so is everything derived from them)
      e = wave_uniform(sDesc[it][0]); row0 = wave_uniform(sDesc[it][1]); row_end = wave_uniform(sDesc[it][2]);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int r = row0 + (tid >> 3) + 32 * i;
        a_ok[i] = r < row_end;
        a_row[i] = A + (int64_t)n_idx[i] * p.lda;
        a_off[i] = (uint32_t)(((int64_t)n_idx[i] * p.lda + a_chunk * CH) * (int64_t)sizeof(T));
        a_amax[i] = (has_amax && a_ok[i]) ? p.abs_max[n_idx[i]] : 1.f;
        a_amax_inv[i] = has_amax ? 1.0f / a_amax[i] : 1.f;
      }
      if (tid < kTileRows) {
        sOrow[tid] = n_orow;
        if (xf_stage) sXrow[tid] = n_xrow;
      }
      fetch_rows(it + 1);
    }
    const ColBlock colb = find_col_block(p.col_bounds, p.n_col_tiles, cb);
    const int c0 = colb.c0, c1 = colb.c1;
    const T* __restrict__ W = static_cast<const T*>(p.w) + (int64_t)e * p.w_se;

    // per-column constants of the forward epilogue (last read before the barrier that ended the
    // previous item)
    // (with one max |W| per expert they are the same for every column: scalars, no LDS traffic)
    const bool col_uniform = FWD && p.wmax_cols <= 1;
    float u_nz = 0.f, u_bound = 0.f, u_q = 0.f, u_qinv = 0.f;
    if (col_uniform) {
      const float wm = p.wmax != nullptr ? p.wmax[(int64_t)e * p.wmax_cols] : 1.f;
      u_nz = p.noise_std * wm;
      u_bound = p.out_bound * wm;
      u_q = adc_quant ? p.out_half_states / u_bound : 0.f;
      u_qinv = adc_quant ? u_bound / p.out_half_states : 0.f;
    }
    if (FWD && !col_uniform && tid < kTileCols) {
      const int col = c0 + tid;
      float wm = 1.f;
      if (p.wmax != nullptr && col < c1) wm = p.wmax[(int64_t)e * p.wmax_cols + (p.wmax_cols > 1 ? col : 0)];
      const float bound = p.out_bound * wm;
      sCol[0][tid] = p.noise_std * wm;
      sCol[1][tid] = bound;
      sCol[2][tid] = adc_quant ? p.out_half_states / bound : 0.f;
      sCol[3][tid] = adc_quant ? bound / p.out_half_states : 0.f;
    }

    f32x16 acc[2][2];
    f32x16 total[2][2];
    if (MODE == MODE_FWD_SPLIT) {
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
          for (int i = 0; i < 16; i++) total[a][b][i] = 0.f;
    }

    for (int t = 0; t < p.n_kd_tiles; t++) {
      const int klo = p.kd_bounds[t], khi = p.kd_bounds[t + 1];
      const int nsteps = (khi - klo + BK - 1) / BK;
      float a_ir[4], a_ir_inv[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int r = row0 + (tid >> 3) + 32 * i;
        a_ir[i] = (has_ir && a_ok[i]) ? p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.ir_cols + t] : 1.f;
        a_ir_inv[i] = has_ir ? 1.0f / a_ir[i] : 1.f;
      }
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
          for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

      Raw ra0[4], rb0[4];
      // Interior tiles (every chunk complete and 16-byte aligned) take unconditional vector loads.
      const bool fast_shape = p.a_vec != 0 && p.w_vec != 0 && (c1 - c0) == kTileCols && (khi - klo) % BK == 0;
      // the interior path addresses both operands with 32-bit byte offsets through buffer
      // resources: per lane a fixed offset, per step a wave-uniform one
      const bool fast = FAST || (fast_shape && p.buf_ok != 0);
      const BufRsrc rsrcW = make_rsrc(W);
      uint32_t w_off[4];
#pragma unroll
      for (int i = 0; i < 4; i++)
        w_off[i] = W_KC ? (uint32_t)((((int64_t)(c0 + (tid >> 3) + 32 * i)) * p.w_snd + a_chunk * CH) * (int64_t)sizeof(T))
                        : (uint32_t)((((int64_t)(tid / CPR + RPP * i)) * p.w_skd + c0 + (tid % CPR) * CH) * (int64_t)sizeof(T));
      const uint32_t a_step = BK * (uint32_t)sizeof(T);
      const uint32_t w_step = (uint32_t)((W_KC ? (int64_t)BK : (int64_t)BK * p.w_skd) * (int64_t)sizeof(T));
      const uint32_t a_base = (uint32_t)klo * (uint32_t)sizeof(T);
      const uint32_t w_base = (uint32_t)((W_KC ? (int64_t)klo : (int64_t)klo * p.w_skd) * (int64_t)sizeof(T));
      auto load_fast = [&](int s, Raw (&ra)[4], Raw (&rb)[4]) {
#pragma unroll
        for (int i = 0; i < 4; i++) ra[i] = buffer_load_b128(rsrcA, a_off[i], a_base + s * a_step);
#pragma unroll
        for (int i = 0; i < 4; i++) rb[i] = buffer_load_b128(rsrcW, w_off[i], w_base + s * w_step);
      };
      auto load_step = [&](int s, Raw (&ra)[4], Raw (&rb)[4]) {   // global -> registers, any shape
        const int k0 = klo + s * BK;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int kpos = k0 + a_chunk * CH;
          int nv = a_ok[i] ? khi - kpos : 0;
          nv = nv < 0 ? 0 : (nv > CH ? CH : nv);
          ra[i] = raw_load<T>(a_row[i] + kpos, nv, p.a_vec != 0);
        }
        if (W_KC) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int col = c0 + (tid >> 3) + 32 * i;
            const int kpos = k0 + a_chunk * CH;
            int nv = col < c1 ? khi - kpos : 0;
            nv = nv < 0 ? 0 : (nv > CH ? CH : nv);
            rb[i] = raw_load<T>(W + (int64_t)col * p.w_snd + kpos, nv, p.w_vec != 0);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int kd = k0 + tid / CPR + RPP * i;
            const int col = c0 + (tid % CPR) * CH;
            int nv = kd < khi ? c1 - col : 0;
            nv = nv < 0 ? 0 : (nv > CH ? CH : nv);
            rb[i] = raw_load<T>(W + (int64_t)kd * p.w_skd + col, nv, p.w_vec != 0);
          }
        }
      };
      auto store_step = [&](int buf, Raw (&ra)[4], Raw (&rb)[4]) {   // registers -> LDS stage, DAC stage on the way
        T* __restrict__ dA = sStage + buf * STAGE;
        T* __restrict__ dB = dA + A_ELEMS;
        if (FWD && dac_ir_quant) {      // the usual input stage: clip, scale, round (one branch for all chunks)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float v[CH];
            raw_unpack<T>(ra[i], v);
            const float r = a_ir[i], rinv = a_ir_inv[i];
            const float kq = rinv * inv_res;
            float tie = 0.f;
            float xc[CH];
#pragma unroll
            for (int j = 0; j < CH; j++) {
              xc[j] = clamp_sym(v[j], r);
              const float c = dac_code<IS_BF16>(xc[j], r, rinv, p.inp_res, inv_res, kq, tie);
              v[j] = IS_BF16 ? c : c * p.inp_res;
            }
            if (IS_BF16 && tie > tie_margin) {      // rare: a product next to a rounding tie
#pragma unroll
              for (int j = 0; j < CH; j++) v[j] = dac_code_exact(xc[j], r, rinv, p.inp_res, inv_res);
            }
            if constexpr (IS_BF16) ra[i] = raw_pack_codes<T>(v);
            else ra[i] = raw_pack<T>(v);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
          Raw a = ra[i];
          if (!FAST && FWD && dac && !dac_ir_quant) {
            float v[CH];
            raw_unpack<T>(a, v);
            bool out_of_range = false;
#pragma unroll
            for (int j = 0; j < CH; j++) {
              float x = v[j];
              if (has_ir) {
                const float r = a_ir[i];
                x = x > r ? r : x;
                x = x < -r ? -r : x;
                x = div_by(x, r, a_ir_inv[i]);
              }
              if (has_amax) x = div_by(x, a_amax[i], a_amax_inv[i]);
              if (quant) {
                out_of_range |= !(fabsf(x) <= 1.0f);
                x = rintf(div_by(x, p.inp_res, inv_res));
                if (!IS_BF16) x = x * p.inp_res;
              }
              v[j] = x;
            }
            if (quant && out_of_range && a_ok[i] && p.range_flag != nullptr) atomicOr(p.range_flag, 1);
            if constexpr (IS_BF16) a = codes_mode ? raw_pack_codes<T>(v) : raw_pack<T>(v);
            else a = raw_pack<T>(v);
          }
          *reinterpret_cast<Raw*>(&dA[((tid >> 3) + 32 * i) * LDA + a_chunk * CH]) = a;
          if (W_KC) *reinterpret_cast<Raw*>(&dB[((tid >> 3) + 32 * i) * LDB + a_chunk * CH]) = rb[i];
          else *reinterpret_cast<Raw*>(&dB[(tid / CPR + RPP * i) * LDB + (tid % CPR) * CH]) = rb[i];
        }
      };

      auto load_any = [&](int s, Raw (&ra)[4], Raw (&rb)[4]) {
        if constexpr (FAST) {
          load_fast(s, ra, rb);
        } else {
          if (fast) load_fast(s, ra, rb); else load_step(s, ra, rb);
        }
      };
      auto multiply_stage = [&](int cur) {     // acc += stage `cur` of LDS
        const T* __restrict__ cA = sStage + cur * STAGE;
        const T* __restrict__ cB = cA + A_ELEMS;
#pragma unroll
        for (int kk = 0; kk < BK; kk += MMAK) {
          if constexpr (IS_BF16) {
            u32x4 xf[2], wf[2];
#pragma unroll
            for (int ti = 0; ti < 2; ti++)
              xf[ti] = *reinterpret_cast<const u32x4*>(&cA[(wr * 64 + ti * 32 + l32) * LDA + kk + 8 * lh]);
#pragma unroll
            for (int fi = 0; fi < 2; fi++) {
              if (W_KC) {
                wf[fi] = *reinterpret_cast<const u32x4*>(&cB[(wc * 64 + fi * 32 + l32) * LDB + kk + 8 * lh]);
              } else {
                const int R = lane & 15, g = (lane >> 4) & 1;
                const uint16_t* base = reinterpret_cast<const uint16_t*>(
                    &cB[(kk + 8 * lh + (R >> 2)) * LDB + wc * 64 + fi * 32 + 16 * g + 4 * (R & 3)]);
                u32x2 lo = lds_read_tr16_b64(base);
                u32x2 hi = lds_read_tr16_b64(base + 4 * LDB);
                wf[fi] = u32x4{lo[0], lo[1], hi[0], hi[1]};
              }
            }
#pragma unroll
            for (int fi = 0; fi < 2; fi++)
#pragma unroll
              for (int ti = 0; ti < 2; ti++) acc[fi][ti] = mfma_32x32x16<T>(wf[fi], xf[ti], acc[fi][ti]);
          } else {
            float xf[2], wf[2];
#pragma unroll
            for (int ti = 0; ti < 2; ti++) xf[ti] = cA[(wr * 64 + ti * 32 + l32) * LDA + kk + lh];
#pragma unroll
            for (int fi = 0; fi < 2; fi++)
              wf[fi] = W_KC ? cB[(wc * 64 + fi * 32 + l32) * LDB + kk + lh]
                            : cB[(kk + lh) * LDB + wc * 64 + fi * 32 + l32];
#pragma unroll
            for (int fi = 0; fi < 2; fi++)
#pragma unroll
              for (int ti = 0; ti < 2; ti++) acc[fi][ti] = mfma_32x32x2_f32(wf[fi], xf[ti], acc[fi][ti]);
          }
        }
      };
      load_any(0, ra0, rb0);
      store_step(0, ra0, rb0);
      __syncthreads();
      for (int s = 0; s < nsteps; s++) {
        if (s + 1 < nsteps) {
          load_any(s + 1, ra0, rb0);
        } else if (xf_stage) {                // last step: the staging registers fetch the mask tile
          const T* __restrict__ XF = static_cast<const T*>(p.xf);
#pragma unroll
          for (int i = 0; i < 8; i++) {
            const int rl = tid / 16 + 16 * i;
            // (when the clipped input is written back, every row of x belongs to one sorted position and its
            // segment is read by this item only; token rows shared by k positions are better kept in the L2)
            const Raw* src = reinterpret_cast<const Raw*>(XF + (int64_t)sXrow[rl] * p.ldxf + c0 + (tid % 16) * CH);
            const Raw v = p.xc_out != nullptr ? __builtin_nontemporal_load(src) : *src;
            if (i < 4) ra0[i] = v; else rb0[i - 4] = v;
          }
        }
        multiply_stage(s & 1);
        if (s + 1 < nsteps) {
          store_step((s + 1) & 1, ra0, rb0);
        } else if (xf_stage) {                // ... and park it in the stage that is idle now
          T* __restrict__ sXF = sStage + ((s + 1) & 1) * STAGE;
#pragma unroll
          for (int i = 0; i < 8; i++)
            *reinterpret_cast<Raw*>(&sXF[(tid / 16 + 16 * i) * LDO + (tid % 16) * CH]) = i < 4 ? ra0[i] : rb0[i - 4];
        }
        __syncthreads();
      }

      // ---- per-K-tile analog output stage (forward) ----------------------------------------------
      if (FWD && plain_epi) {
        if (MODE == MODE_FWD_SPLIT) {
#pragma unroll
          for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++) total[a][b] += acc[a][b];
        }
      } else if (FWD && FAST && codes_mode && gen_noise && adc_quant && col_uniform && has_ir) {
        // The usual training configuration on edge-free tiles -- DAC codes, noise drawn here, ADC with one
        // max |W| per expert, input range -- as straight-line code: same operations in the same order as the
        // general stage below, without a branch around every 4 values.
        const NoiseKey key = noise_key(seed, t);
        uint32_t col_key[2];
#pragma unroll
        for (int fi = 0; fi < 2; fi++) col_key[fi] = noise_col_key(key, (uint32_t)(c0 + wc * 64 + fi * 32 + l32));
        const float u_nzs = u_nz * kNoiseScale;
#pragma unroll
        for (int ti = 0; ti < 2; ti++) {
          const int rl = wr * 64 + ti * 32 + l32;
          const int r = row0 + rl;
          const bool valid = r < row_end;
          const int orow = valid ? sOrow[rl] : 0;
          const float ir_r = valid ? p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.ir_cols + t] : 1.f;
          const uint32_t row_key = noise_row_key(key, (uint32_t)orow);
#pragma unroll
          for (int fi = 0; fi < 2; fi++) {
            // the block's noise: one 8-bit matrix instruction (same slot layout as acc[fi][ti])
            const i32x16 zi = noise_block(row_key, col_key[fi], (uint32_t)(c0 + wc * 64 + fi * 32) >> 5,
                                          (uint32_t)(row0 + wr * 64 + ti * 32), lh);
#pragma unroll
            for (int q = 0; q < 4; q++) {
#pragma unroll
              for (int j = 0; j < 4; j++) {
                float v = acc[fi][ti][4 * q + j] * p.inp_res;
                v = fmaf((float)zi[4 * q + j], u_nzs, v);
                v = clamp_sym(v, u_bound);
                v = rintf(v * u_q) * u_qinv;
                v *= ir_r;
                if (MODE == MODE_FWD_SPLIT) total[fi][ti][4 * q + j] += v;
                else acc[fi][ti][4 * q + j] = v;
              }
            }
          }
        }
      } else if (FWD) {
        const NoiseKey key = noise_key(seed, t);
#pragma unroll
        for (int ti = 0; ti < 2; ti++) {
          const int rl = wr * 64 + ti * 32 + l32;
          const int r = row0 + rl;
          const bool valid = r < row_end;
          const int orow = valid ? sOrow[rl] : 0;
          const float ir_r = (has_ir && valid) ? p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.ir_cols + t] : 1.f;
          const float am_r = (has_amax && valid) ? p.abs_max[p.a_index[r]] : 1.f;
          const uint32_t row_key = gen_noise ? noise_row_key(key, (uint32_t)orow) : 0u;
#pragma unroll
          for (int fi = 0; fi < 2; fi++) {
            i32x16 zi;
            if (gen_noise) {
              const int cb0 = c0 + wc * 64 + fi * 32;
              zi = noise_block(row_key, noise_col_key(key, (uint32_t)(cb0 + l32)), (uint32_t)cb0 >> 5,
                               (uint32_t)(row0 + wr * 64 + ti * 32), lh);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
              const int cl = wc * 64 + fi * 32 + 8 * q + 4 * lh;
              const int col = c0 + cl;
              int nv = valid ? c1 - col : 0;
              nv = nv < 0 ? 0 : (nv > 4 ? 4 : nv);
              if (FAST) nv = valid ? 4 : 0;
              float v[4];
#pragma unroll
              for (int j = 0; j < 4; j++) v[j] = acc[fi][ti][4 * q + j];
              if (codes_mode) {
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] *= p.inp_res;
              }
              if (p.noise != nullptr) {
                float nz[4];
                load4<float>(p.noise + (int64_t)t * p.noise_ts + (int64_t)orow * p.ldnoise + col, nz, nv,
                             FAST || p.noise_vec != 0);
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] += nz[j];
              } else if (gen_noise) {
#pragma unroll
                for (int j = 0; j < 4; j++)
                  v[j] = fmaf((float)zi[4 * q + j], (col_uniform ? u_nz : sCol[0][cl + j]) * kNoiseScale, v[j]);
              }
              if (adc_clip && col_uniform) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                  v[j] = clamp_sym(v[j], u_bound);
                  if (adc_quant) v[j] = rintf(v[j] * u_q) * u_qinv;
                }
              } else if (adc_clip) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                  const float b = sCol[1][cl + j];
                  v[j] = fminf(fmaxf(v[j], -b), b);
                  if (adc_quant) v[j] = rintf(v[j] * sCol[2][cl + j]) * sCol[3][cl + j];
                }
              }
#pragma unroll
              for (int j = 0; j < 4; j++) {
                if (has_amax) v[j] *= am_r;
                if (has_ir) v[j] *= ir_r;
                if (MODE == MODE_FWD_SPLIT) total[fi][ti][4 * q + j] += v[j];
                else acc[fi][ti][4 * q + j] = v[j];
              }
            }
          }
        }
      }
    }

    // ---- final values of the tile (in acc), then the store ------------------------------------
    if (FWD) {
      if (MODE == MODE_FWD_SPLIT) {
#pragma unroll
        for (int fi = 0; fi < 2; fi++)
#pragma unroll
          for (int ti = 0; ti < 2; ti++) acc[fi][ti] = total[fi][ti];
      }
      if (p.relu) {
#pragma unroll
        for (int fi = 0; fi < 2; fi++)
#pragma unroll
          for (int ti = 0; ti < 2; ti++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[fi][ti][i] = fmaxf(acc[fi][ti][i], 0.f);
      }
    } else {
      // input gradient: clip mask, input-range gradient partial sums, gate
      const T* __restrict__ XF = static_cast<const T*>(p.xf);
      const T* __restrict__ GATE = static_cast<const T*>(p.gate);
      if (xf_stage) {
        // Edge-free, mask tile parked in LDS: straight-line code.  A stage that is switched off works with a
        // neutral constant (infinite range, threshold -inf, gate 1) instead of a branch around every 4 values.
        T* __restrict__ sXF = sStage + (((p.kd_bounds[1] - p.kd_bounds[0] + BK - 1) / BK) & 1) * STAGE;
        const float kInf = __builtin_inff();
        const float relu_thr = p.relu_mask ? 0.f : -kInf;
#pragma unroll
        for (int ti = 0; ti < 2; ti++) {
          const int rl = wr * 64 + ti * 32 + l32;
          const int r = row0 + rl;
          const bool valid = r < row_end;
          const int orow = valid ? sOrow[rl] : 0;
          const float gate_r = (valid && GATE != nullptr) ? Elem<T>::load(GATE + orow) : 1.f;
          const float ir_r = (use_ir_bw && valid) ? p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.ir_cols + colb.tile]
                                                  : kInf;
          float part = 0.f;
          int seen = 0;
#pragma unroll
          for (int fi = 0; fi < 2; fi++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
              float xv[4];
              load4<T>(&sXF[rl * LDO + wc * 64 + fi * 32 + 8 * q + 4 * lh], xv, 4, true);
#pragma unroll
              for (int j = 0; j < 4; j++) {
                float g = acc[fi][ti][4 * q + j];
                const float gs = g * gate_r;
                part += xv[j] >= ir_r ? fminf(gs, 0.f) : 0.f;
                part -= xv[j] <= -ir_r ? fmaxf(gs, 0.f) : 0.f;
                const bool not_clip = fabsf(xv[j]) < ir_r;
                seen += not_clip ? 1 : 0;
                g = not_clip ? g : 0.f;
                g = xv[j] > relu_thr ? g : 0.f;
                acc[fi][ti][4 * q + j] = g * gate_r;
              }
            }
          }
          cnt += valid ? seen : 0;
          if (use_ir_bw) {
            part += wave_shfl_xor(part, 32);
            if (lh == 0) sRed[wc][rl] = part;
          }
        }
        if (p.xc_out != nullptr) {      // the clipped, gate-scaled input for the weight gradient, in place
#pragma unroll
          for (int ti = 0; ti < 2; ti++) {
            const int rl = wr * 64 + ti * 32 + l32;
            const int r = row0 + rl;
            const bool valid = r < row_end;
            const float gate_r = (valid && GATE != nullptr) ? Elem<T>::load(GATE + sOrow[rl]) : 1.f;
            const float ir_r = (use_ir_bw && valid) ? p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.ir_cols + colb.tile]
                                                    : kInf;
#pragma unroll
            for (int fi = 0; fi < 2; fi++) {
#pragma unroll
              for (int q = 0; q < 4; q++) {
                T* __restrict__ at = &sXF[rl * LDO + wc * 64 + fi * 32 + 8 * q + 4 * lh];
                float xv[4];
                load4<T>(at, xv, 4, true);
#pragma unroll
                for (int j = 0; j < 4; j++) xv[j] = clamp_sym(xv[j], ir_r) * gate_r;
                store4<T>(at, xv, 4, true);
              }
            }
          }
        }
      } else if (XF != nullptr || GATE != nullptr) {
#pragma unroll
      for (int ti = 0; ti < 2; ti++) {
        const int rl = wr * 64 + ti * 32 + l32;
        const int r = row0 + rl;
        const bool valid = r < row_end;
        const int orow = valid ? sOrow[rl] : 0;
        const int xrow = (valid && XF != nullptr) ? p.xf_index[r] : 0;
        const float gate_r = (valid && GATE != nullptr) ? Elem<T>::load(GATE + orow) : 1.f;
        const float ir_r = (use_ir_bw && valid) ? p.ir[(int64_t)(p.ir_by_expert ? e : r) * p.ir_cols + colb.tile]
                                                : 0.f;
        float part = 0.f;
#pragma unroll
        for (int fi = 0; fi < 2; fi++) {
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int col = c0 + wc * 64 + fi * 32 + 8 * q + 4 * lh;
            int nv = valid ? c1 - col : 0;
            nv = nv < 0 ? 0 : (nv > 4 ? 4 : nv);
            if (FAST) nv = valid ? 4 : 0;
            float xv[4] = {0.f, 0.f, 0.f, 0.f};
            if (XF != nullptr && nv > 0) {
              load4<T>(XF + (int64_t)xrow * p.ldxf + col, xv, nv, FAST || p.xf_vec != 0);
            }
            if (p.xc_out != nullptr) {      // the clipped, gate-scaled input for the weight gradient
              float pc[4];
#pragma unroll
              for (int j = 0; j < 4; j++) pc[j] = (use_ir_bw ? clamp_sym(xv[j], ir_r) : xv[j]) * gate_r;
              if (nv > 0) {
                store4<T>(static_cast<T*>(p.xc_out) + (int64_t)xrow * p.ldxc + col, pc, nv, p.xc_vec != 0);
              }
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
              float g = acc[fi][ti][4 * q + j];
              if (j < nv) {
                if (use_ir_bw) {
                  const float gs = g * gate_r;
                  if (xv[j] >= ir_r) part += fminf(gs, 0.f);
                  if (xv[j] <= -ir_r) part -= fmaxf(gs, 0.f);
                  const bool not_clip = fabsf(xv[j]) < ir_r;
                  cnt += not_clip ? 1 : 0;
                  g = not_clip ? g : 0.f;
                }
                if (p.relu_mask) g = xv[j] > 0.f ? g : 0.f;
              }
              acc[fi][ti][4 * q + j] = g * gate_r;
            }
          }
        }
        if (use_ir_bw) {
          part += wave_shfl_xor(part, 32);
          if (lh == 0) sRed[wc][rl] = part;
        }
      }
      }
    }

    // The tile leaves once as the result and, when the caller wants it (forward), a second time as
    // the DAC image of the result for the projection that follows: clamp / scale / round of the
    // value as stored in T, so that projection's input stage has nothing left to do.
    const float q_r = (FWD && p.xq_out != nullptr) ? p.xq_ir[e] : 1.f;
    const float q_rinv = 1.0f / q_r, q_res = p.xq_inp_res, q_resinv = 1.0f / p.xq_inp_res;
    const float q_kq = q_rinv * q_resinv;
    const float q_tie_margin = dac_tie_margin(q_resinv);
    auto as_codes = [&](float (&v)[4]) {
      float tie = 0.f;
      float xc[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float x = v[j];
        if constexpr (IS_BF16) x = Elem<T>::to_f32(Elem<T>::cvt(x));
        xc[j] = clamp_sym(x, q_r);
        const float c = dac_code<IS_BF16>(xc[j], q_r, q_rinv, q_res, q_resinv, q_kq, tie);
        v[j] = IS_BF16 ? c : c * q_res;
      }
      if (IS_BF16 && tie > q_tie_margin) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = dac_code_exact(xc[j], q_r, q_rinv, q_res, q_resinv);
      }
    };
    const int n_out = (FWD && p.xq_out != nullptr) ? 2 : 1;
    for (int pass = 0; pass < n_out; pass++) {
    T* __restrict__ DST = pass == 0 ? OUT : static_cast<T*>(p.xq_out);
    const int64_t ldd = pass == 0 ? p.ldo : p.ldxq;
    const bool staged = FAST || ((pass == 0 ? p.out_stage : p.xq_stage) != 0 && (c1 - c0) == kTileCols);
    if (staged) {
      // registers -> LDS tile -> whole 256-byte (bf16) row segments to global memory
      // (the input gradient may still be reading the parked mask tile from the other stage)
      T* __restrict__ sOut = sStage + ((!FWD && ((p.kd_bounds[1] - p.kd_bounds[0] + BK - 1) / BK) % 2 == 0) ? STAGE : 0);
#pragma unroll
      for (int h = 0; h < OUT_PASSES; h++) {
        if (OUT_PASSES == 1 || wr == h) {
#pragma unroll
          for (int ti = 0; ti < 2; ti++) {
            const int rl = (OUT_PASSES == 1 ? wr * 64 : 0) + ti * 32 + l32;
#pragma unroll
            for (int fi = 0; fi < 2; fi++)
#pragma unroll
              for (int q = 0; q < 4; q++) {
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = acc[fi][ti][4 * q + j];
                if (pass == 1) as_codes(v);
                store4<T>(&sOut[rl * LDO + wc * 64 + fi * 32 + 8 * q + 4 * lh], v, 4, true);
              }
          }
        }
        __syncthreads();
        constexpr int OCPR = kTileCols / CH;            // 16-byte chunks per row
        constexpr int ORPP = kThreads / OCPR;
        // (all LDS reads of a thread first, then its stores: one wait instead of one per row)
        constexpr int NROW = OUT_ROWS / ORPP;
        {
          Raw seg[NROW];
          int orow[NROW];
#pragma unroll
          for (int i = 0; i < NROW; i++) {
            const int rl = tid / OCPR + ORPP * i;
            orow[i] = sOrow[h * OUT_ROWS + rl];
            seg[i] = *reinterpret_cast<const Raw*>(&sOut[rl * LDO + (tid % OCPR) * CH]);
          }
#pragma unroll
          for (int i = 0; i < NROW; i++)
            if (orow[i] >= 0) store_streaming(DST + (int64_t)orow[i] * ldd + c0 + (tid % OCPR) * CH, seg[i]);
        }
        if (xf_stage && p.xc_out != nullptr) {     // the parked input tile, clipped and scaled in place
          const T* __restrict__ sXF = sStage + (sOut == sStage ? STAGE : 0);
          Raw seg[NROW];
          int xrow[NROW];
#pragma unroll
          for (int i = 0; i < NROW; i++) {
            const int rl = tid / OCPR + ORPP * i;
            xrow[i] = row0 + rl < row_end ? sXrow[rl] : -1;
            seg[i] = *reinterpret_cast<const Raw*>(&sXF[rl * LDO + (tid % OCPR) * CH]);
          }
#pragma unroll
          for (int i = 0; i < NROW; i++)
            if (xrow[i] >= 0)
              store_streaming(static_cast<T*>(p.xc_out) + (int64_t)xrow[i] * p.ldxc + c0 + (tid % OCPR) * CH, seg[i]);
        }
        __syncthreads();
      }
    } else if constexpr (!FAST) {
#pragma unroll
      for (int ti = 0; ti < 2; ti++) {
        const int rl = wr * 64 + ti * 32 + l32;
        const int orow = sOrow[rl];
#pragma unroll
        for (int fi = 0; fi < 2; fi++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int col = c0 + wc * 64 + fi * 32 + 8 * q + 4 * lh;
            int nv = orow >= 0 ? c1 - col : 0;
            nv = nv < 0 ? 0 : (nv > 4 ? 4 : nv);
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = acc[fi][ti][4 * q + j];
            if (pass == 1) as_codes(v);
            if (nv > 0) store4<T>(DST + (int64_t)orow * ldd + col, v, nv, (pass == 0 ? p.out_vec : p.xq_vec) != 0);
          }
      }
      __syncthreads();
    }
    }
    if (use_ir_bw) {     // sRed was written before the barriers above
      if (tid < kTileRows && row0 + tid < row_end)
        p.irg_partial[(int64_t)cb * p.M + row0 + tid] = sRed[0][tid] + sRed[1][tid];
      __syncthreads();
    }
  }

  if (use_ir_bw) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) cnt += wave_shfl_xor(cnt, d);
    if (lane == 0) sCnt[wave] = cnt;
    __syncthreads();
    if (tid == 0) p.notclip_count[blockIdx.x] = sCnt[0] + sCnt[1] + sCnt[2] + sCnt[3];
  }
}

// Sum the column-block partials into ir_grad[M, n_tiles] and apply the scaling and decay rules.
struct IrFinalizeParams {
  int M, n_tiles, KD_total;      // KD_total = columns of x (for the un-clipped fraction)
  int block_cols;                // width of the column blocks the partial sums were made over
  int col_bounds[kMaxTiles + 1];
  const float* irg_partial; const int32_t* notclip_count; int n_blocks;
  const int32_t* row_index;      // optional: the partial sums of sorted position r lie at row row_index[r]
  const float* ir; int ir_by_expert; const int32_t* offsets; int E; float* ir_grad;
  int relative; float scale, decay, min_pct;
};

__global__ __launch_bounds__(kThreads) void ir_grad_finalize_kernel(const IrFinalizeParams p) {
  __shared__ long long sTot[4];
  __shared__ int sOff[kSelMaxExperts];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // the segment starts come to LDS in the same round trip as the counts: the search below then runs on LDS
  // instead of on a chain of dependent global loads (E <= kSelMaxExperts: the entry points check it)
  if (p.ir_by_expert)
    for (int i = tid; i < p.E; i += kThreads) sOff[i] = p.offsets[i];
  long long c = 0;
  if (p.decay > 0.f)
    for (int i = tid; i < p.n_blocks; i += kThreads) c += p.notclip_count[i];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) c += wave_shfl_xor(c, d);
  if (lane == 0) sTot[wave] = c;
  __syncthreads();
  float flag = 0.f;
  if (p.decay > 0.f) {
    const long long tot = sTot[0] + sTot[1] + sTot[2] + sTot[3];
    const float pct = (float)tot / (float)((long long)p.M * (long long)p.KD_total);
    flag = pct > p.min_pct ? 1.f : 0.f;
  }
  const int r = blockIdx.x * kThreads + tid;
  if (r >= p.M) return;
  int ir_row = r;
  if (p.ir_by_expert) {  // expert of sorted position r: last e with offsets[e] <= r
    int lo = 0, hi = p.E - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (sOff[mid] <= r) lo = mid; else hi = mid - 1;
    }
    ir_row = lo;
  }
  const int pr = p.row_index ? p.row_index[r] : r;
  int cb = 0;
  for (int t = 0; t < p.n_tiles; t++) {
    const int nb = (p.col_bounds[t + 1] - p.col_bounds[t] + p.block_cols - 1) / p.block_cols;
    float s = 0.f;
    for (int b = 0; b < nb; b++) s += p.irg_partial[(int64_t)(cb + b) * p.M + pr];
    cb += nb;
    const float irv = p.ir[(int64_t)ir_row * p.n_tiles + t];
    if (p.relative) s = s * irv * p.scale;
    if (p.decay > 0.f) s = s + p.decay * irv * flag;
    p.ir_grad[(int64_t)r * p.n_tiles + t] = s;
  }
}

}  // namespace amoe
