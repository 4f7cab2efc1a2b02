// Forward row-gather GEMM of the CVMM path for the usual training shapes: bf16 or fp16, every tile interior, one
// input range per expert and K-tile, one max |W| per expert.  Same arithmetic, in the same order, as the
// general kernel of gemm_rows.h (which keeps serving every other case); what differs is the shape of the work:
//
//  * 128 (rows) x 256 (columns) output tile per workgroup, 2 x 2 waves of 64 x 128 (2 x 4 matrix tiles of
//    32 x 32).  A gathered row passes the DAC stage once per 256 output columns instead of once per 128, and
//    the stage's vector work per matrix instruction halves with it -- to about six instructions, which a wave
//    issues in the shadow of its own matrix instructions.
//  * 32-deep K steps, two LDS stages, two workgroups per CU.  The rows of step s + 1 are fetched at the end
//    of step s - 1, pass the DAC stage between the matrix instructions of step s and reach LDS at its end.
//  * every feature is a template parameter: no uniform branch keeps a dead alternative's registers alive.
//  * with two K-tiles and an output quantiser, the first tile's result is kept as its ADC codes, four to a
//    register (32 registers instead of a second set of 128 accumulators).
#pragma once
#include <type_traits>

#include "gemm_rows.h"

namespace amoe {

constexpr int kFCols = 256;                 // output columns per workgroup tile
constexpr int kFBK = 32;                    // contraction elements per step

enum { FA_PLAIN = 0, FA_DAC = 1, FA_CODES = 2 };   // what the gathered operand is: values as they are; values
                                                   // that take the clip / scale / round stage; codes already

// A_MODE: see above.  ANALOG: ADC with rounding + rescale by the input range, after the generated noise if NOISE;
// otherwise the accumulator leaves as it is (times inp_res * ir for code operands).  SPLIT2: exactly two K-tiles
// (needs ANALOG).  ZCODES: the result leaves as its ADC codes + 128, one byte each (and the expert's step and input
// range go to code_scale_out), instead of as values.
template <typename T, int A_MODE, bool ANALOG, bool NOISE, bool SPLIT2, bool ZCODES = false>
__global__ __launch_bounds__(kThreads, 2) void fwd256_kernel(const RowsParams p) {
  static_assert(sizeof(T) == 2, "16-bit elements: bf16 (as bits) or fp16");
  constexpr int BK = kFBK, CH = 8;
  constexpr int LDA = BK + 8;                       // 80-byte rows: 16 consecutive rows hit 16 disjoint bank groups
  constexpr int LDB = kFCols + 32;                  // 576-byte rows: the four rows of a transposing read are disjoint
  constexpr int A_ELEMS = kTileRows * LDA, B_ELEMS = BK * LDB;
  constexpr int STAGE = A_ELEMS + B_ELEMS;
  constexpr int LDO = kFCols + 8;                   // staged output rows: 256 columns + 16 bytes
  // the whole 128-row tile is staged at once (all four waves write, one barrier, all threads store): 66 KB, ten more
  // than the two K-loop stages it overlays, still two workgroups per CU
  constexpr int OUT_ELEMS = kTileRows * LDO;
  constexpr int LDS_ELEMS = OUT_ELEMS > 2 * STAGE ? OUT_ELEMS : 2 * STAGE;
  static_assert((!SPLIT2 || ANALOG) && (!NOISE || ANALOG), "the packed first tile holds ADC codes");
  static_assert(!ZCODES || (ANALOG && !SPLIT2), "a result leaves as ADC codes only after a single output quantiser");
  constexpr bool CODES = A_MODE != FA_PLAIN;        // the matrix unit sees integer codes: scale the accumulator

  __shared__ __attribute__((aligned(16))) T sStage[LDS_ELEMS];
  __shared__ int sOrow[kTileRows];
  __shared__ int sDesc[kMaxDesc][4];
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
  const BufRsrc rsrcA = make_rsrc(A);
  const uint64_t seed = p.seed + ((NOISE && p.seed_dev != nullptr) ? *p.seed_dev : 0);
  const float inv_res = CODES ? 1.0f / p.inp_res : 0.f;
  const float tie_margin = dac_tie_margin(inv_res);
  const bool want_xq = p.xq_out != nullptr;

  // staging maps: A 128 rows x 4 chunks (2 per thread), B 32 k-rows x 32 chunks (4 per thread)
  const int a_row = tid >> 2, a_chunk = tid & 3;          // rows a_row, a_row + 64
  const int b_row = tid >> 5, b_chunk = tid & 31;         // k-rows b_row + 8 * i

  int n_idx[2] = {0, 0}, n_orow = -1;
  auto fetch_rows = [&](int i) {
    if (i >= n_my) return;
    const int r0 = sDesc[i][1], r1 = sDesc[i][2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const int r = r0 + a_row + 64 * q;
      n_idx[q] = p.a_index[r < r1 ? r : r0];            // rows past the tile read its first row: never stored
    }
    if (tid < kTileRows) {
      const int r = r0 + tid;
      n_orow = r < r1 ? (p.out_index ? p.out_index[r] : p.a_index[r]) : -1;
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
    if (tid < kTileRows) sOrow[tid] = n_orow;
    fetch_rows(it + 1);
    const int c0 = cb * kFCols;
    const T* __restrict__ W = static_cast<const T*>(p.w) + (int64_t)e * p.w_se;
    const BufRsrc rsrcW = make_rsrc(W);
    uint32_t w_off[4];
#pragma unroll
    for (int i = 0; i < 4; i++) w_off[i] = (uint32_t)(((int64_t)(b_row + 8 * i) * p.w_skd + c0 + b_chunk * CH) * 2);
    const uint32_t w_step = (uint32_t)((int64_t)BK * p.w_skd * 2);

    // epilogue constants of the expert (scalars)
    const float wm = (ANALOG && p.wmax != nullptr) ? p.wmax[e] : 1.f;
    const float u_nzs = (p.noise_std * wm) * kNoiseScale;
    const float u_bound = p.out_bound * wm;
    const float u_q = ANALOG ? p.out_half_states / u_bound : 0.f;
    const float u_qinv = ANALOG ? u_bound / p.out_half_states : 0.f;

    f32x16 acc[4][2];                       // [column block fi][row block ti]
    uint32_t packed[SPLIT2 ? 4 : 1][2][4];  // ADC codes + 128 of the first K-tile, four to a word
    float ir_first = 1.f;

    constexpr int NT = SPLIT2 ? 2 : 1;
#pragma unroll 1
    for (int t = 0; t < NT; t++) {     // (one copy of the K loop's code: unrolled, the two tiles compete for registers)
      const int klo = p.kd_bounds[t], khi = p.kd_bounds[t + 1];
      const int nsteps = (khi - klo) / BK;
      const float ir_t = (A_MODE != FA_PLAIN || ANALOG) ? p.ir[(int64_t)e * p.ir_cols + t] : 1.f;
      const float ir_inv = 1.0f / ir_t;
      const float kq = ir_inv * inv_res;
#pragma unroll
      for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
          for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

      Raw ra[2], rb[4];
      const uint32_t a_base = (uint32_t)klo * 2, w_base = (uint32_t)((int64_t)klo * p.w_skd * 2);
      auto load_step = [&](int s) {
#pragma unroll
        for (int i = 0; i < 2; i++) ra[i] = buffer_load_b128(rsrcA, a_off[i], a_base + s * (BK * 2));
#pragma unroll
        for (int i = 0; i < 4; i++) rb[i] = buffer_load_b128(rsrcW, w_off[i], w_base + s * w_step);
      };
      auto dac_step = [&]() {                 // clip, scale, round the gathered chunks in their registers
        if constexpr (A_MODE == FA_DAC) {
#pragma unroll
          for (int i = 0; i < 2; i++) {
            float v[CH], xc[CH];
            raw_unpack<T>(ra[i], v);
            float tie = 0.f;
#pragma unroll
            for (int j = 0; j < CH; j++) {
              xc[j] = clamp_sym(v[j], ir_t);
              v[j] = dac_code<true>(xc[j], ir_t, ir_inv, p.inp_res, inv_res, kq, tie);
            }
            if (tie > tie_margin) {
#pragma unroll
              for (int j = 0; j < CH; j++) v[j] = dac_code_exact(xc[j], ir_t, ir_inv, p.inp_res, inv_res);
            }
            ra[i] = raw_pack_codes<T>(v);
          }
        }
      };
      auto store_step = [&](int buf) {
        T* __restrict__ dA = sStage + buf * STAGE;
        T* __restrict__ dB = dA + A_ELEMS;
#pragma unroll
        for (int i = 0; i < 2; i++) *reinterpret_cast<Raw*>(&dA[(a_row + 64 * i) * LDA + a_chunk * CH]) = ra[i];
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<Raw*>(&dB[(b_row + 8 * i) * LDB + b_chunk * CH]) = rb[i];
      };
      auto multiply_group = [&](const T* __restrict__ cA, const T* __restrict__ cB, int kk) {
        u32x4 xf[2], wf[4];
#pragma unroll
        for (int ti = 0; ti < 2; ti++)
          xf[ti] = *reinterpret_cast<const u32x4*>(&cA[(wr * 64 + ti * 32 + l32) * LDA + kk + 8 * lh]);
        const int R = lane & 15, g = (lane >> 4) & 1;
#pragma unroll
        for (int fi = 0; fi < 4; fi++) {
          const uint16_t* base = reinterpret_cast<const uint16_t*>(
              &cB[(kk + 8 * lh + (R >> 2)) * LDB + wc * 128 + fi * 32 + 16 * g + 4 * (R & 3)]);
          const u32x2 lo = lds_read_tr16_b64(base), hi = lds_read_tr16_b64(base + 4 * LDB);
          wf[fi] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
#pragma unroll
        for (int fi = 0; fi < 4; fi++)
#pragma unroll
          for (int ti = 0; ti < 2; ti++) acc[fi][ti] = mfma_32x32x16<T>(wf[fi], xf[ti], acc[fi][ti]);
      };

      load_step(0);
      dac_step();
      store_step(0);
      __syncthreads();
      if (nsteps > 1) load_step(1);
      for (int s = 0; s < nsteps; s++) {
        const T* __restrict__ cA = sStage + (s & 1) * STAGE;
        const T* __restrict__ cB = cA + A_ELEMS;
        multiply_group(cA, cB, 0);
        if (s + 1 < nsteps) dac_step();          // vector work of step s + 1 between the matrix instructions of s
        multiply_group(cA, cB, 16);
        if (s + 1 < nsteps) {
          store_step((s + 1) & 1);
          if (s + 2 < nsteps) load_step(s + 2);
        }
        __syncthreads();
      }

      // ---- output stage of this K-tile ------------------------------------------------------------------------
      if constexpr (ANALOG) {
        const NoiseKey key = noise_key(seed, t);
#pragma unroll
        for (int ti = 0; ti < 2; ti++) {
          const int rl = wr * 64 + ti * 32 + l32;
          const bool valid = row0 + rl < row_end;
          const int orow = valid ? sOrow[rl] : 0;
          const uint32_t row_key = NOISE ? noise_row_key(key, (uint32_t)orow) : 0u;
#pragma unroll
          for (int fi = 0; fi < 4; fi++) {
            i32x16 zi;
            if constexpr (NOISE) {
              zi = noise_block(row_key, noise_col_key(key, (uint32_t)(c0 + wc * 128 + fi * 32 + l32)),
                               (uint32_t)(c0 + wc * 128 + fi * 32) >> 5,
                               (uint32_t)(row0 + wr * 64 + ti * 32), lh);
            }
            auto code_of = [&](int i) {       // the ADC code of accumulator element i of this block
              float v = acc[fi][ti][i];
              if (CODES) v *= p.inp_res;
              if constexpr (NOISE) v = fmaf((float)zi[i], u_nzs, v);
              v = clamp_sym(v, u_bound);
              return rintf(v * u_q);
            };
            // (the tile test stays outside the element loops: inside them the compiler keeps one branch and one
            // copy of the accumulator block per element)
            if (SPLIT2 && t == 0) {
#pragma unroll
              for (int q = 0; q < 4; q++) {
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) word = cvt_pk_u8_f32(code_of(4 * q + j) + 128.0f, j, word);
                packed[SPLIT2 ? fi : 0][ti][q] = word;
              }
            } else if constexpr (SPLIT2) {
#pragma unroll
              for (int q = 0; q < 4; q++) {
                const uint32_t word = packed[fi][ti][q];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                  const float first = (float)((word >> (8 * j)) & 0xffu) - 128.0f;
                  acc[fi][ti][4 * q + j] = (first * u_qinv) * ir_first + (code_of(4 * q + j) * u_qinv) * ir_t;
                }
              }
            } else if constexpr (ZCODES) {  // straight to the staged tile (the stage buffers are idle by now)
#pragma unroll
              for (int q = 0; q < 4; q++) {
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) word = cvt_pk_u8_f32(code_of(4 * q + j) + 128.0f, j, word);
                *reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(sStage) + rl * (kFCols + 16) + wc * 128 +
                                             fi * 32 + 8 * q + 4 * lh) = word;
              }
            } else {
#pragma unroll
              for (int i = 0; i < 16; i++) acc[fi][ti][i] = (code_of(i) * u_qinv) * ir_t;
            }
          }
        }
        if (SPLIT2 && t == 0) ir_first = ir_t;
        if constexpr (ZCODES) {
          if (tid == 0 && cb == 0 && row0 == p.offsets[e]) {     // once per expert that has rows
            p.code_scale_out[2 * e] = u_qinv;
            p.code_scale_out[2 * e + 1] = ir_t;
          }
        }
      } else if constexpr (CODES) {
        const float s1 = p.inp_res;
#pragma unroll
        for (int fi = 0; fi < 4; fi++)
#pragma unroll
          for (int ti = 0; ti < 2; ti++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[fi][ti][i] = (acc[fi][ti][i] * s1) * ir_t;
      }
    }

    if constexpr (ZCODES) {
      // one byte per result: rows of 256 bytes (+ 16) through LDS, whole 256-byte row segments out
      constexpr int LDC = kFCols + 16;
      const uint8_t* __restrict__ sC = reinterpret_cast<const uint8_t*>(sStage);   // filled by the output stage
      __syncthreads();
      constexpr int CPRC = kFCols / 16;            // 16 chunks of 16 bytes per row
      constexpr int RPPC = kThreads / CPRC;        // 16 rows per pass
#pragma unroll
      for (int i0 = 0; i0 < kTileRows / RPPC; i0 += 4) {
        Raw seg[4];
        int orow[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int rl = tid / CPRC + RPPC * (i0 + i);
          orow[i] = sOrow[rl];
          seg[i] = *reinterpret_cast<const Raw*>(&sC[rl * LDC + (tid % CPRC) * 16]);
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (orow[i] >= 0) store_streaming(p.code_out + (int64_t)orow[i] * p.ldcode + c0 + (tid % CPRC) * 16, seg[i]);
      }
      __syncthreads();
      continue;
    }
    if (p.relu) {
#pragma unroll
      for (int fi = 0; fi < 4; fi++)
#pragma unroll
        for (int ti = 0; ti < 2; ti++)
#pragma unroll
          for (int i = 0; i < 16; i++) acc[fi][ti][i] = fmaxf(acc[fi][ti][i], 0.f);
    }

    // ---- store: the result and, if asked for, the DAC image of it for the projection that follows ----------
    const float q_r = want_xq ? p.xq_ir[e] : 1.f;
    const float q_rinv = 1.0f / q_r, q_res = p.xq_inp_res, q_resinv = 1.0f / p.xq_inp_res;
    const float q_kq = q_rinv * q_resinv, q_tie_margin = dac_tie_margin(q_resinv);
    auto as_codes = [&](float (&v)[4]) {
      float tie = 0.f, xc[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float x = Elem<T>::to_f32(Elem<T>::cvt(v[j]));
        xc[j] = clamp_sym(x, q_r);
        v[j] = dac_code<true>(xc[j], q_r, q_rinv, q_res, q_resinv, q_kq, tie);
      }
      if (tie > q_tie_margin) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = dac_code_exact(xc[j], q_r, q_rinv, q_res, q_resinv);
      }
    };
    auto emit = [&](auto pass_tag) {
      constexpr int pass = decltype(pass_tag)::value;
      T* __restrict__ DST = pass == 0 ? OUT : static_cast<T*>(p.xq_out);
      const int64_t ldd = pass == 0 ? p.ldo : p.ldxq;
      T* __restrict__ sOut = sStage;
#pragma unroll
      for (int ti = 0; ti < 2; ti++) {
        const int rl = wr * 64 + ti * 32 + l32;
#pragma unroll
        for (int fi = 0; fi < 4; fi++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = acc[fi][ti][4 * q + j];
            if (pass == 1) as_codes(v);
            store4<T>(&sOut[rl * LDO + wc * 128 + fi * 32 + 8 * q + 4 * lh], v, 4, true);
          }
      }
      __syncthreads();
      constexpr int OCPR = kFCols / CH;          // 32 chunks per row
      constexpr int ORPP = kThreads / OCPR;      // 8 rows per pass of the workgroup
      constexpr int NROW = 4;                    // rows in flight per thread (the accumulators are still live)
#pragma unroll
      for (int i0 = 0; i0 < kTileRows / ORPP; i0 += NROW) {
        Raw seg[NROW];
        int orow[NROW];
#pragma unroll
        for (int i = 0; i < NROW; i++) {
          const int rl = tid / OCPR + ORPP * (i0 + i);
          orow[i] = sOrow[rl];
          seg[i] = *reinterpret_cast<const Raw*>(&sOut[rl * LDO + (tid % OCPR) * CH]);
        }
#pragma unroll
        for (int i = 0; i < NROW; i++)
          if (orow[i] >= 0) store_streaming(DST + (int64_t)orow[i] * ldd + c0 + (tid % OCPR) * CH, seg[i]);
      }
      __syncthreads();
    };
    emit(std::integral_constant<int, 0>{});
    if (want_xq) emit(std::integral_constant<int, 1>{});
  }
}

}  // namespace amoe
