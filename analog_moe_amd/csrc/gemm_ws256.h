// Row-gather GEMM of the CVMM path with the WEIGHTS HELD IN REGISTERS, for launches whose contraction is exactly 256
// elements long (the down-projection's forward and the up-projection's input gradient of an expert size of 256):
//     out[out_index[i], :] = epilogue( a[a_index[i], :] @ W[e] )             a [*, 256], W[e] [256, ND]
//
// The kernels of gemm_fwd256.h / gemm_bwdx256.h keep the output tile in registers and stream both operands through
// LDS, 32 contraction elements at a time; with a contraction of 256 an output tile lives for eight such steps only,
// and every matrix instruction costs 0.75 KB of LDS fragment reads, 0.4 KB of stage stores and a sixteenth of a
// workgroup barrier.  Here the roles are turned round.  A wave owns CW output columns of one expert and loads the
// 256 x CW block of W[e] behind them into registers ONCE (as matrix-instruction fragments: 128 registers for 64
// columns, 256 for 128); the expert's rows then stream past it in blocks of 32: a block is 16 KB in LDS, shared by
// the four waves of the workgroup, each of which reads its 16 fragments (0.5 / 0.25 KB per matrix instruction) and
// issues 16 * CW / 32 matrix instructions.  One workgroup barrier per block; no weight traffic in the loop at all.
//
// The 32-row blocks of all experts form one list; the workgroups of a column group (4 * CW columns) take equal runs
// of it, and the workgroups that work on the same run for different column groups are neighbours, so that they run
// side by side behind one L2 and the rows are fetched from memory once.
#pragma once
#include <type_traits>

#include "gemm_fwd256.h"

namespace amoe {

constexpr int kWsK = 256;          // contraction length
constexpr int kWsRows = 32;        // rows per block
constexpr uint32_t kWsOutLimit = 0x80000000u;   // the output must be smaller than this many bytes

enum { WS_PLAIN = 0, WS_SCALE = 1, WS_ZCODES = 2 };
// WS_PLAIN : the accumulator leaves as it is, rounded to T.
// WS_SCALE : the gathered operand holds DAC codes: the accumulator is scaled by inp_res * ir[e] (no output stage).
// WS_ZCODES: codes in; generated noise (if NOISE), ADC; the result leaves as its ADC codes + 128, one byte each.

template <typename T, bool W_KC, int CW, int EPI, bool NOISE>
__global__ __launch_bounds__(kThreads, CW == 128 ? 1 : 2) void ws256_kernel(const RowsParams p) {
  static_assert(sizeof(T) == 2, "16-bit elements: bf16 (as bits) or fp16");
  static_assert(CW == 64 || CW == 128, "columns per wave");
  constexpr int KS = kWsK / 16;                  // matrix-instruction steps over the contraction
  constexpr int CB = CW / 32;                    // 32-column blocks per wave
  constexpr int WGC = 4 * CW;                    // columns per workgroup
  constexpr int CH = 8;
  constexpr int LDA = kWsK + 8;                  // 528-byte rows: 16 consecutive rows start on 16 disjoint bank groups
  constexpr int A_STAGE = kWsRows * LDA;         // elements
  constexpr bool BYTES = EPI == WS_ZCODES;
  constexpr int ROW_B = BYTES ? WGC : 2 * WGC;   // bytes of one staged output row
  constexpr int LDO_B = ROW_B + 16;
  constexpr int O_STAGE_B = kWsRows * LDO_B;
  constexpr int LDB = WGC + 32;                  // weight staging (W_KC == false): rows of WGC columns + 64 bytes
  constexpr int W_STAGE_B = 2 * 32 * LDB * 2;    // two buffers
  constexpr int LOOP_B = 2 * A_STAGE * 2 + 2 * O_STAGE_B;
  constexpr int LDS_B = LOOP_B > W_STAGE_B ? LOOP_B : W_STAGE_B;
  constexpr int OCPR = ROW_B / 16;               // 16-byte pieces per staged output row
  constexpr int ORPP = kThreads / OCPR;          // rows per pass of the workgroup
  constexpr int NPASS = kWsRows / ORPP;
  static_assert(!NOISE || EPI == WS_ZCODES, "noise belongs to the analog output stage");

  __shared__ __attribute__((aligned(16))) unsigned char sMem[LDS_B];
  __shared__ int sDesc[kMaxDesc][4];
  __shared__ int sWave[4];

  T* __restrict__ sA = reinterpret_cast<T*>(sMem);
  unsigned char* __restrict__ sO = sMem + 2 * A_STAGE * 2;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int ncg = p.n_col_blocks;                // column groups of WGC columns

  // ---- this workgroup's share of the work --------------------------------------------------------------------
  // The rows of every expert are cut into blocks of 32; the blocks of all experts, in expert order, form one list,
  // and the gridDim.x / ncg workgroups of a column group take equal contiguous runs of that list.  A run that
  // crosses an expert boundary is worked off as several segments (the weights are reloaded at the boundary), so the
  // load is balanced to one block whatever the experts' sizes are.  sDesc[b] describes the segment that starts at
  // block b of the run: (expert, first sorted position, end position, blocks).
  const int per = (p.E + kThreads - 1) / kThreads;
  const int e_first = tid * per;
  int mine = 0;
  for (int j = 0; j < per; j++) {
    const int e = e_first + j;
    if (e < p.E) mine += (p.offsets[e + 1] - p.offsets[e] + kWsRows - 1) / kWsRows;
  }
  int incl = mine;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = wave_shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == 63) sWave[wave] = incl;
  __syncthreads();
  int blocks_before = incl - mine;
  for (int w = 0; w < wave; w++) blocks_before += sWave[w];
  const int total_blocks = sWave[0] + sWave[1] + sWave[2] + sWave[3];
  const int lb = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int runs = (int)gridDim.x / ncg;         // (the host makes the grid a multiple of ncg)
  const int run = lb / ncg, cg = lb - run * ncg;
  const int run_first = (int)((long long)total_blocks * run / runs);
  const int run_end = (int)((long long)total_blocks * (run + 1) / runs);
  {
    int t = blocks_before;
    for (int j = 0; j < per; j++) {
      const int e = e_first + j;
      if (e < p.E) {
        const int lo = p.offsets[e], hi = p.offsets[e + 1];
        const int nb = (hi - lo + kWsRows - 1) / kWsRows;
        const int b0 = t > run_first ? t : run_first, b1 = t + nb < run_end ? t + nb : run_end;
        if (b0 < b1 && b0 - run_first < kMaxDesc) {
          const int r1 = lo + (b1 - t) * kWsRows;
          sDesc[b0 - run_first][0] = e;
          sDesc[b0 - run_first][1] = lo + (b0 - t) * kWsRows;
          sDesc[b0 - run_first][2] = r1 < hi ? r1 : hi;
          sDesc[b0 - run_first][3] = b1 - b0;
        }
        t += nb;
      }
    }
  }
  __syncthreads();

  const T* __restrict__ A = static_cast<const T*>(p.a);
  const BufRsrc rsrcA = make_rsrc(A);
  const BufRsrc rsrcI = make_rsrc(p.a_index), rsrcOI = make_rsrc(p.out_index ? p.out_index : p.a_index);
  // stores go through a buffer resource of kWsOutLimit bytes (the host checks that the output is smaller): a store
  // at kDropOffset falls outside it and is dropped
  constexpr uint32_t kDropOffset = kWsOutLimit;
  const BufRsrc rsrcO = make_rsrc_sized(EPI == WS_ZCODES ? static_cast<void*>(p.code_out) : p.out, kWsOutLimit);
  const uint64_t seed = p.seed + ((NOISE && p.seed_dev != nullptr) ? *p.seed_dev : 0);

  const int a_chunk = tid & 31, a_row = tid >> 5;       // staging of a block: rows a_row + 8 i, 16-byte piece a_chunk
  const int o_chunk = tid % OCPR, o_row = tid / OCPR;   // leaving of a block: rows o_row + ORPP i

  const int c0 = cg * WGC;
  for (int seg_at = 0; seg_at < run_end - run_first;) {
    const int e = wave_uniform(sDesc[seg_at][0]), row0 = wave_uniform(sDesc[seg_at][1]),
              row_end = wave_uniform(sDesc[seg_at][2]), nblk = wave_uniform(sDesc[seg_at][3]);
    seg_at += nblk;
    const T* __restrict__ W = static_cast<const T*>(p.w) + (int64_t)e * p.w_se;

    // ---- the expert's 256 x CW weight block of this wave, as matrix-instruction fragments ----------------------
    u32x4 wf[KS][CB];
    if constexpr (W_KC) {
      // contraction-contiguous weights: a fragment is 16 bytes of one output column's row, straight from memory
      const BufRsrc rsrcW = make_rsrc(W);
#pragma unroll
      for (int c = 0; c < CB; c++) {
        const uint32_t off = (uint32_t)(((int64_t)(c0 + wave * CW + c * 32 + l32) * p.w_snd + 8 * lh) * 2);
#pragma unroll
        for (int s = 0; s < KS; s++) wf[s][c] = buffer_load_b128(rsrcW, off, s * 32);
      }
    } else {
      // column-contiguous weights: 32 contraction rows at a time through LDS, read back transposed
      T* __restrict__ sB = reinterpret_cast<T*>(sMem);
      const BufRsrc rsrcW = make_rsrc(W);
      constexpr int CPRW = WGC / CH, RPPW = kThreads / CPRW, NLD = 32 / RPPW;
      const int R = lane & 15, g = (lane >> 4) & 1;
      // (two staging buffers: the loads of pass ps + 1 are in flight while pass ps is read back, one barrier per pass)
      auto load_pass = [&](int ps, Raw (&rb)[NLD]) {
#pragma unroll
        for (int i = 0; i < NLD; i++)
          rb[i] = buffer_load_b128(
              rsrcW, (uint32_t)(((int64_t)(tid / CPRW + RPPW * i) * p.w_skd + c0 + (tid % CPRW) * CH) * 2),
              (uint32_t)((int64_t)ps * 32 * p.w_skd * 2));
      };
      Raw rb[2][NLD];
      load_pass(0, rb[0]);
#pragma unroll
      for (int ps = 0; ps < kWsK / 32; ps++) {
        T* __restrict__ sBp = sB + (ps & 1) * 32 * LDB;
        if (ps + 1 < kWsK / 32) load_pass(ps + 1, rb[(ps + 1) & 1]);
#pragma unroll
        for (int i = 0; i < NLD; i++)
          *reinterpret_cast<Raw*>(&sBp[(tid / CPRW + RPPW * i) * LDB + (tid % CPRW) * CH]) = rb[ps & 1][i];
        __syncthreads();                                 // (the buffer written next was read two passes ago)
#pragma unroll
        for (int kk = 0; kk < 32; kk += 16)
#pragma unroll
          for (int c = 0; c < CB; c++) {
            const uint16_t* base = reinterpret_cast<const uint16_t*>(
                &sBp[(kk + 8 * lh + (R >> 2)) * LDB + wave * CW + c * 32 + 16 * g + 4 * (R & 3)]);
            const u32x2 lo = lds_read_tr16_b64(base), hi = lds_read_tr16_b64(base + 4 * LDB);
            wf[2 * ps + kk / 16][c] = u32x4{lo[0], lo[1], hi[0], hi[1]};
          }
      }
      __syncthreads();                                   // the staging area becomes the block stages
    }

    // ---- constants of the expert's output stage ---------------------------------------------------------------
    const float ir_e = (EPI != WS_PLAIN) ? p.ir[(int64_t)e * p.ir_cols] : 1.f;
    const float wm = (EPI == WS_ZCODES && p.wmax != nullptr) ? p.wmax[e] : 1.f;
    const float u_nzs = (p.noise_std * wm) * kNoiseScale;
    const float u_bound = p.out_bound * wm;
    const float u_q = EPI == WS_ZCODES ? p.out_half_states / u_bound : 0.f;
    const NoiseKey key = noise_key(seed, 0);
    if constexpr (EPI == WS_ZCODES) {
      if (tid == 0 && cg == 0 && row0 == p.offsets[e]) {       // once per expert that has rows (its first segment)
        p.code_scale_out[2 * e] = u_bound / p.out_half_states;
        p.code_scale_out[2 * e + 1] = ir_e;
      }
    }

    // ---- the row blocks ------------------------------------------------------------------------------------------
    // Iteration b: (1) fragments of block b from its stage, (2) block b - 1's staged results leave, (3) multiply,
    // (4) block b + 1 (in registers since the previous iteration) goes to the other stage and the loads of block
    // b + 2 are issued, (5) output stage of block b into its staging tile; one barrier.
    //
    // The loop body is straight-line code on purpose.  The wait counter of vector memory operations counts loads and
    // stores alike, in issue order; a wait for a load can name how many YOUNGER operations may stay in flight only
    // if it is certain that they were issued.  One operation issued under a condition (rows past the end of the
    // chunk, a block that does not exist) turns every later wait into a wait for everything, which puts the whole
    // latency of the loads and stores just issued into every iteration.  So nothing is conditional: rows and
    // blocks past the end are clamped to the chunk's first row (loaded, never used), and a store for a row that
    // does not exist gets an offset beyond the buffer, which the hardware's range check drops.
    auto row_of = [&](int b, int r) {                    // sorted position of row r of block b, clamped to the chunk
      const int pos = row0 + b * kWsRows + r;
      return pos < row_end ? pos : row0;
    };
    Raw ra[4];
    int idx_n[4];                                        // gathered rows of the block whose loads are issued next
    uint32_t orow_n[NPASS], ooff_c[NPASS];               // output rows fetched ahead; byte offsets of the pieces this
                                                         // thread sends off
    int my_orow_n = 0, my_orow_c = 0;                    // output row of the token row this lane holds (noise key)
    auto load_block = [&]() {
#pragma unroll
      for (int i = 0; i < 4; i++)
        ra[i] = buffer_load_b128(rsrcA, (uint32_t)(((int64_t)idx_n[i] * p.lda + a_chunk * CH) * 2), 0);
    };
    // (index loads go through buffer resources: 32-bit offsets, no 64-bit address arithmetic in the loop)
    auto fetch_idx = [&](int b) {
#pragma unroll
      for (int i = 0; i < 4; i++) idx_n[i] = (int)buffer_load_b32(rsrcI, (uint32_t)row_of(b, a_row + 8 * i) * 4u);
    };
    // The output rows of a block are only LOADED here; what is made of them (byte offsets, the noise key) is made an
    // iteration later, by use_orow: computing on a value right after its load would put the load's latency here.
    auto fetch_orow = [&](int b) {
#pragma unroll
      for (int i = 0; i < NPASS; i++) orow_n[i] = buffer_load_b32(rsrcOI, (uint32_t)row_of(b, o_row + ORPP * i) * 4u);
      if constexpr (NOISE) my_orow_n = (int)buffer_load_b32(rsrcOI, (uint32_t)row_of(b, l32) * 4u);
    };
    auto use_orow = [&](int b) {                         // block b's rows, fetched during the previous iteration
#pragma unroll
      for (int i = 0; i < NPASS; i++) {
        const uint32_t off = BYTES ? orow_n[i] * (uint32_t)p.ldcode + (uint32_t)(c0 + o_chunk * 16)
                                   : (orow_n[i] * (uint32_t)p.ldo + (uint32_t)(c0 + o_chunk * CH)) * 2u;
        ooff_c[i] = row0 + b * kWsRows + o_row + ORPP * i < row_end ? off : kDropOffset;
      }
      my_orow_c = my_orow_n;
    };
    auto store_block = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 4; i++)
        *reinterpret_cast<Raw*>(&sA[buf * A_STAGE + (a_row + 8 * i) * LDA + a_chunk * CH]) = ra[i];
    };
    auto send_off = [&](const Raw (&seg)[NPASS]) {
#pragma unroll
      for (int i = 0; i < NPASS; i++) buffer_store_b128_nt(rsrcO, seg[i], ooff_c[i]);
    };

    fetch_idx(0);
    load_block();
    fetch_orow(0);
    fetch_idx(1);
    store_block(0);                                      // (waits for block 0)
    load_block();
    fetch_idx(2);
#pragma unroll
    for (int i = 0; i < NPASS; i++) ooff_c[i] = kDropOffset;
    __syncthreads();

    for (int b = 0; b < nblk; b++) {
      // (1) + (3): the fragments are read PF steps ahead of the matrix instructions that use them; the scheduling
      // fences keep the compiler from collapsing that into read, wait, multiply (which it does to save registers)
      const T* __restrict__ cA = sA + (b & 1) * A_STAGE + l32 * LDA + 8 * lh;
      constexpr int PF = 4;
      f32x16 acc[CB];
      u32x4 xf[KS];
#pragma unroll
      for (int s = 0; s < PF; s++) xf[s] = *reinterpret_cast<const u32x4*>(cA + 16 * s);
#pragma unroll
      for (int c = 0; c < CB; c++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[c][i] = 0.f;
      // (2) the previous block leaves while the first fragments arrive: its pieces are read here and stored a few
      // steps into the multiplication (before the first block there is nothing: the offsets drop the stores)
      Raw seg[NPASS];
      {
        const unsigned char* __restrict__ src = sO + ((b + 1) & 1) * O_STAGE_B;
#pragma unroll
        for (int i = 0; i < NPASS; i++)
          seg[i] = *reinterpret_cast<const Raw*>(src + (o_row + ORPP * i) * LDO_B + o_chunk * 16);
      }
#pragma unroll
      for (int s = 0; s < KS; s++) {
        if (s + PF < KS) xf[s + PF] = *reinterpret_cast<const u32x4*>(cA + 16 * (s + PF));
        sched_fence();
#pragma unroll
        for (int c = 0; c < CB; c++) acc[c] = mfma_32x32x16<T>(wf[s][c], xf[s], acc[c]);
        sched_fence();
        if (s == 3) send_off(seg);
      }
      // (4)
      store_block((b + 1) & 1);
      use_orow(b);
      // (5)
      unsigned char* __restrict__ dst = sO + (b & 1) * O_STAGE_B + l32 * LDO_B;
      if constexpr (EPI == WS_ZCODES) {
        const uint32_t row_key = NOISE ? noise_row_key(key, (uint32_t)my_orow_c) : 0u;
#pragma unroll
        for (int c = 0; c < CB; c++) {
          const int col = c0 + wave * CW + c * 32;
          i32x16 zi;
          if constexpr (NOISE)
            zi = noise_block(row_key, noise_col_key(key, (uint32_t)(col + l32)), (uint32_t)col >> 5,
                             (uint32_t)(row0 + b * kWsRows), lh);
#pragma unroll
          for (int q = 0; q < 4; q++) {
            uint32_t word = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
              float v = acc[c][4 * q + j] * p.inp_res;
              if constexpr (NOISE) v = fmaf((float)zi[4 * q + j], u_nzs, v);
              v = clamp_sym(v, u_bound);
              word = cvt_pk_u8_f32(rintf(v * u_q) + 128.0f, j, word);
            }
            *reinterpret_cast<uint32_t*>(dst + wave * CW + c * 32 + 8 * q + 4 * lh) = word;
          }
        }
      } else {
#pragma unroll
        for (int c = 0; c < CB; c++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
              v[j] = acc[c][4 * q + j];
              if constexpr (EPI == WS_SCALE) v[j] = (v[j] * p.inp_res) * ir_e;
            }
            store4<T>(reinterpret_cast<T*>(dst) + wave * CW + c * 32 + 8 * q + 4 * lh, v, 4, true);
          }
      }
      // (4), second half: the loads of block b + 2 and the rows of the blocks after it (issued after the output stage,
      // whose registers the loaded values would otherwise take)
      load_block();
      fetch_idx(b + 3);
      fetch_orow(b + 1);
      __syncthreads();
    }
    {                                                    // the last block leaves
      const unsigned char* __restrict__ src = sO + ((nblk + 1) & 1) * O_STAGE_B;
      Raw seg[NPASS];
#pragma unroll
      for (int i = 0; i < NPASS; i++)
        seg[i] = *reinterpret_cast<const Raw*>(src + (o_row + ORPP * i) * LDO_B + o_chunk * 16);
      send_off(seg);
    }
    __syncthreads();                                     // the stages are free for the next segment's weights
  }
}

}  // namespace amoe
