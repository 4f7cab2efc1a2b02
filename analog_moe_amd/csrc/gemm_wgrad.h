// Segmented weight gradient of the CVMM path:
//     grad_w[e][kk][n] = sum_{i in expert e} clamp(x[in_index[i]][kk], +-ir[i,t]) * g[g_index[i]][n]
// One workgroup owns one 128 (kk) x 128 (n) tile of one expert and walks that expert's sorted
// rows in order, so the result needs no atomics, no pre-zeroing and has a fixed summation order.
// Both operands are staged token-major ("RC": [token][feature], as they lie in memory) and
// fed to the matrix unit through the transposing LDS read (bf16) or plain reads (fp32); the
// gradient fragment is the A operand, so a lane holds one kk and runs of 4 consecutive n.
// With a workspace, an expert with more than two chunks' worth of rows is cut into chunks of
// rows_per_chunk rows that different workgroups sum (few experts, or a few heavy ones, would
// otherwise leave most of the chip idle); those workgroups leave fp32 partial tiles, which
// wgrad_reduce_kernel adds in chunk order in a second launch: no atomics, a fixed summation order.
// The clip and the optional per-row scale (the gate of the fused layer) are applied to the x
// operand on its way into LDS; the finished tile leaves through LDS as whole row segments.
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
  int x_vec, g_vec, out_vec, out_stage;
  int buf_ok;   // x and g small enough for 32-bit byte offsets (buffer loads on interior steps)
  int rows_per_chunk;            // 0: one workgroup per (expert, tile) walks all rows
  float* partial;                // [slots][tiles][128*128] fp32 partial tiles of multi-chunk experts
};

// chunks of an expert with `rows` rows
__device__ __host__ inline int wgrad_chunks(int rows, int rows_per_chunk) {
  return (rows_per_chunk > 0 && rows > 2 * rows_per_chunk) ? (rows + rows_per_chunk - 1) / rows_per_chunk : 1;
}

constexpr int kWgradTileElems = kTileRows * kTileCols;

template <typename T>
__global__ __launch_bounds__(kThreads, 2) void gemm_wgrad_kernel(const WgradParams p) {
  using EL = Elem<T>;
  constexpr int CH = EL::kChunk, MMAK = EL::kMmaK;
  // tokens per step.  (bf16: 64 fills the LDS budget of two workgroups per CU.  With 32, four fit and the kernel
  // alone runs about a tenth faster, but it then leaves no registers for the row-wise kernels the layer runs next to
  // it on a second stream, and the training step as a whole gets slower.)
  constexpr int BT = EL::kBK;
  constexpr int LD = kTileCols + EL::kPadRC;
  constexpr int STAGE = BT * LD;
  constexpr int CPR = kTileCols / CH, RPP = kThreads / CPR;
  constexpr bool IS_BF16 = sizeof(T) == 2;
  constexpr int NP = BT / RPP;                    // staging passes per step
  static_assert(BT == NP * RPP && 4 * BT <= kThreads, "whole staging passes; one metadata lane per row and item");

  constexpr int LDO = kTileCols + 16 / (int)sizeof(T);       // staged output tile, rows of 128 + 16 bytes
  static_assert(kTileRows * LDO <= 4 * STAGE, "the output tile must fit the stage buffers");
  __shared__ __attribute__((aligned(16))) T sS[4 * STAGE];   // two stages of each operand
  T* const sX = sS;
  T* const sG = sS + 2 * STAGE;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave >> 1, wk = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // Workgroup ids go to the 8 XCDs round-robin.  All tiles of one chunk of rows run on one XCD
  // (they share those rows through that L2) and consecutive chunks / experts go to different
  // XCDs, so that a few heavy experts -- skewed routing -- do not pile up behind one L2.
  // (scratch for the chunk search and the arrival flag lives in the stage buffers, which are idle then)
  int* const sScanA = reinterpret_cast<int*>(sS);
  int* const sScanB = sScanA + 4;
  int* const sFound = sScanA + 8;
  const int tiles_per_expert = p.n_k_blocks * p.n_n_blocks;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int cg = xcd + 8 * (slot / tiles_per_expert);      // index of the (expert, chunk) pair
  const int tile_id = slot % tiles_per_expert;
  int e = cg, chunk_id = 0, n_chunks = 1, part_slot = 0;
  if (p.rows_per_chunk > 0) {
    // chunks per expert -> exclusive prefix; thread tid owns experts [tid*per, (tid+1)*per)
    const int R = p.rows_per_chunk;
    const int per = (p.E + kThreads - 1) / kThreads;
    int mineA = 0, mineB = 0;
    for (int j = 0; j < per; j++) {
      const int ee = tid * per + j;
      if (ee < p.E) {
        const int rows = p.offsets[ee + 1] - p.offsets[ee];
        const int c = wgrad_chunks(rows, R);
        mineA += c;
        mineB += c > 1 ? c : 0;
      }
    }
    int inclA = mineA, inclB = mineB;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int ua = wave_shfl_up(inclA, d), ub = wave_shfl_up(inclB, d);
      if (lane >= d) { inclA += ua; inclB += ub; }
    }
    if (lane == 63) { sScanA[wave] = inclA; sScanB[wave] = inclB; }
    if (tid == 0) sFound[0] = -1;
    __syncthreads();
    int beforeA = inclA - mineA, beforeB = inclB - mineB;
    for (int w = 0; w < wave; w++) { beforeA += sScanA[w]; beforeB += sScanB[w]; }
    for (int j = 0; j < per; j++) {
      const int ee = tid * per + j;
      if (ee < p.E) {
        const int rows = p.offsets[ee + 1] - p.offsets[ee];
        const int c = wgrad_chunks(rows, R);
        if (cg >= beforeA && cg < beforeA + c) {
          sFound[0] = ee; sFound[1] = cg - beforeA; sFound[2] = c; sFound[3] = beforeB;
        }
        beforeA += c;
        beforeB += c > 1 ? c : 0;
      }
    }
    __syncthreads();
    // (wave-uniform by construction; telling the compiler keeps the tile bookkeeping in scalar registers)
    e = wave_uniform(sFound[0]); chunk_id = wave_uniform(sFound[1]); n_chunks = wave_uniform(sFound[2]);
    part_slot = wave_uniform(sFound[3]) + chunk_id;
    if (e < 0) return;
    __syncthreads();                       // the scratch is stage memory again from here on
  } else if (e >= p.E) {
    return;
  }
  const int nb = tile_id % p.n_n_blocks, kb = tile_id / p.n_n_blocks;
  const ColBlock kcol = find_col_block(p.bounds, p.n_tiles, kb);
  const int kc0 = kcol.c0, kc1 = kcol.c1;
  const int n0 = nb * kTileCols, n1 = (n0 + kTileCols < p.N) ? n0 + kTileCols : p.N;
  int seg0 = p.offsets[e], seg1 = p.offsets[e + 1];
  if (p.rows_per_chunk > 0 && n_chunks > 1) {
    seg0 += chunk_id * p.rows_per_chunk;
    seg1 = seg0 + p.rows_per_chunk < seg1 ? seg0 + p.rows_per_chunk : seg1;
  }

  const T* __restrict__ X = static_cast<const T*>(p.x);
  const T* __restrict__ G = static_cast<const T*>(p.g);
  const T* __restrict__ GS = static_cast<const T*>(p.g_scale);
  const bool has_ir = p.ir != nullptr;
  const int chunk = tid % CPR;
  // (without input ranges the clip below runs against an infinite range: no branch per row group)
  const float ir_expert = (has_ir && p.ir_by_expert) ? p.ir[(int64_t)e * p.n_tiles + kcol.tile] : __builtin_inff();

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][c][i] = 0.f;

  // Per-row metadata of a step (x row, g row, scale, input range) is fetched by ONE lane per row
  // and item -- thread group tid / BT picks the item -- two steps ahead of use, and handed to the
  // other threads through the padding columns of the x stage rows: 16 bytes behind the 128
  // operand columns of row j of a stage buffer.
  auto meta = [&](int buf, int row) -> int* {
    return reinterpret_cast<int*>(&sX[buf * STAGE + row * LD + kTileCols]);
  };
  const int m_item = tid / BT, m_row = tid % BT;
  int m_val = 0;
  auto fetch_meta = [&](int i0) {            // global -> register, rows of the step that starts at i0
    const int r = i0 + m_row;
    const bool ok = r < seg1;
    if (m_item == 0) m_val = ok ? p.in_index[r] : 0;
    else if (m_item == 1) m_val = ok ? (p.g_index ? p.g_index[r] : p.in_index[r]) : 0;
    else if (m_item == 2) m_val = (int)as_u32((GS != nullptr && ok) ? Elem<T>::load(GS + r) : 1.f);
    else if (m_item == 3)
      m_val = (int)as_u32((has_ir && !p.ir_by_expert && ok) ? p.ir[(int64_t)r * p.n_tiles + kcol.tile] : ir_expert);
  };
  auto publish_meta = [&](int buf) {
    if (m_item < 4) meta(buf, m_row)[m_item] = m_val;
  };

  Raw rx[NP], rg[NP];
  auto load_step = [&](int i0, int mbuf) {   // global -> registers, any shape; rows from the metadata
#pragma unroll
    for (int i = 0; i < NP; i++) {
      const int j = tid / CPR + RPP * i;
      const bool ok = i0 + j < seg1;
      const int* m = meta(mbuf, j);
      const int kk = kc0 + chunk * CH;
      int nvx = ok ? kc1 - kk : 0;
      nvx = nvx < 0 ? 0 : (nvx > CH ? CH : nvx);
      rx[i] = raw_load<T>(X + (int64_t)m[0] * p.ldx + kk, nvx, p.x_vec != 0);
      const int n = n0 + chunk * CH;
      int nvg = ok ? n1 - n : 0;
      nvg = nvg < 0 ? 0 : (nvg > CH ? CH : nvg);
      rg[i] = raw_load<T>(G + (int64_t)m[1] * p.ldg + n, nvg, p.g_vec != 0);
    }
  };
  // Interior steps (all BT tokens exist, full 128-column tiles, aligned rows, 32-bit addressable
  // operands): unconditional buffer loads, one 32-bit multiply per row address.
  const bool tile_fast = p.x_vec != 0 && p.g_vec != 0 && p.buf_ok != 0 && (kc1 - kc0) == kTileCols &&
                         (n1 - n0) == kTileCols;
  const BufRsrc rsX = make_rsrc(X), rsG = make_rsrc(G);
  const uint32_t x_row_bytes = (uint32_t)(p.ldx * (int64_t)sizeof(T)), g_row_bytes = (uint32_t)(p.ldg * (int64_t)sizeof(T));
  const uint32_t x_col_bytes = (uint32_t)((kc0 + chunk * CH) * (int)sizeof(T));
  const uint32_t g_col_bytes = (uint32_t)((n0 + chunk * CH) * (int)sizeof(T));
  auto load_fast = [&](int mbuf) {
#pragma unroll
    for (int i = 0; i < NP; i++) {
      const int* m = meta(mbuf, tid / CPR + RPP * i);
      rx[i] = buffer_load_b128(rsX, (uint32_t)m[0] * x_row_bytes + x_col_bytes, 0);
      rg[i] = buffer_load_b128(rsG, (uint32_t)m[1] * g_row_bytes + g_col_bytes, 0);
    }
  };
  auto load_rows = [&](int i0, int mbuf) {
    if (tile_fast && i0 + BT <= seg1) load_fast(mbuf); else load_step(i0, mbuf);
  };
  auto store_step = [&](int buf, int mbuf) {  // registers -> LDS, clip / row scaling of x on the way
    T* __restrict__ dX = sX + buf * STAGE;
    T* __restrict__ dG = sG + buf * STAGE;
    if (has_ir || GS != nullptr) {           // one branch for the whole step; a stage that is off is neutral
#pragma unroll
      for (int i = 0; i < NP; i++) {
        const int* m = meta(mbuf, tid / CPR + RPP * i);
        const float scale = as_f32((uint32_t)m[2]), rng = as_f32((uint32_t)m[3]);
        float v[CH];
        raw_unpack<T>(rx[i], v);
#pragma unroll
        for (int q = 0; q < CH; q++) v[q] = clamp_sym(v[q], rng) * scale;
        rx[i] = raw_pack<T>(v);
      }
    }
#pragma unroll
    for (int i = 0; i < NP; i++) {
      const int j = tid / CPR + RPP * i;
      *reinterpret_cast<Raw*>(&dX[j * LD + chunk * CH]) = rx[i];
      *reinterpret_cast<Raw*>(&dG[j * LD + chunk * CH]) = rg[i];
    }
  };

  // Pipeline, step s (rows seg0 + s*BT ...): data of step s is in stage s&1; the metadata of step
  // s+1 sits in the padding of stage s&1 and that of step s+2 is published, at the end of step
  // s, into the padding of stage (s+1)&1 together with the data of step s+1.
  const int nsteps = (seg1 - seg0 + BT - 1) / BT;
  if (nsteps > 0) {
    fetch_meta(seg0);
    publish_meta(1);                          // metadata of step 0, parked in stage 1
    __syncthreads();
    load_rows(seg0, 1);
    fetch_meta(seg0 + BT);
    __syncthreads();                          // every thread has read its step-0 metadata
    // (the scale / range of step 0 are still in stage 1's padding, which nothing has overwritten)
    store_step(0, 1);
    __syncthreads();                          // ... before the metadata of step 1 replaces it
    publish_meta(0);
    __syncthreads();
  }
  for (int s = 0; s < nsteps; s++) {
    const int cur = s & 1;
    const bool more = s + 1 < nsteps;
    if (more) {
      load_rows(seg0 + (s + 1) * BT, cur);    // rows of step s+1: metadata in stage cur's padding
      fetch_meta(seg0 + (s + 2) * BT);
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
          for (int fk = 0; fk < 2; fk++) acc[fn][fk] = mfma_32x32x16<T>(gf[fn], xf[fk], acc[fn][fk]);
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
    if (more) {
      // the scale / range of step s+1 are read from stage cur's padding; the metadata of step
      // s+2 goes to the padding of the stage that receives the data of step s+1
      store_step(cur ^ 1, cur);
      publish_meta(cur ^ 1);
    }
    __syncthreads();
  }

  if (n_chunks > 1) {
    // leave this chunk's tile in fp32 for wgrad_reduce_kernel
    float* __restrict__ mine = p.partial + ((int64_t)part_slot * tiles_per_expert + tile_id) * kWgradTileElems;
#pragma unroll
    for (int fk = 0; fk < 2; fk++)
#pragma unroll
      for (int fn = 0; fn < 2; fn++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          f32x4 v;
#pragma unroll
          for (int j = 0; j < 4; j++) v[j] = acc[fn][fk][4 * q + j];
          *reinterpret_cast<f32x4*>(&mine[(wk * 64 + fk * 32 + l32) * kTileCols + wn * 64 + fn * 32 + 8 * q + 4 * lh]) = v;
        }
    return;
  }
  T* __restrict__ GW = static_cast<T*>(p.grad_w) + (int64_t)e * p.K * p.N;
  if (p.out_stage != 0 && (kc1 - kc0) == kTileCols && (n1 - n0) == kTileCols) {
    // registers -> LDS tile -> whole 256-byte (bf16) / 512-byte (fp32) row segments.  The barrier
    // that ended the last step has retired every read of the stage buffers.
    T* __restrict__ sOut = sS;
#pragma unroll
    for (int fk = 0; fk < 2; fk++)
#pragma unroll
      for (int fn = 0; fn < 2; fn++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; j++) v[j] = acc[fn][fk][4 * q + j];
          store4<T>(&sOut[(wk * 64 + fk * 32 + l32) * LDO + wn * 64 + fn * 32 + 8 * q + 4 * lh], v, 4, true);
        }
    __syncthreads();
    constexpr int OCPR = kTileCols / CH, ORPP = kThreads / OCPR;
#pragma unroll
    for (int i = 0; i < kTileRows / ORPP; i++) {
      const int rl = tid / OCPR + ORPP * i;
      store_streaming(GW + (int64_t)(kc0 + rl) * p.N + n0 + (tid % OCPR) * CH,
                      *reinterpret_cast<const Raw*>(&sOut[rl * LDO + (tid % OCPR) * CH]));
    }
    return;
  }
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

// Second launch of a row-chunked weight gradient: kWgradReduceSplit workgroups per (expert, tile), each
// with its share of the tile's rows, add the fp32 partial tiles of a multi-chunk expert in chunk order and
// write the tile of grad_w.
constexpr int kWgradReduceSplit = 8;
template <typename T>
__global__ __launch_bounds__(kThreads) void wgrad_reduce_kernel(const WgradParams p) {
  __shared__ int sSum[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tiles = p.n_k_blocks * p.n_n_blocks;
  const int part = blockIdx.x % kWgradReduceSplit, et = blockIdx.x / kWgradReduceSplit;
  const int e = et / tiles, tile_id = et % tiles;
  const int R = p.rows_per_chunk;
  const int n_chunks = wgrad_chunks(p.offsets[e + 1] - p.offsets[e], R);
  if (n_chunks <= 1) return;
  int before = 0;                          // partial slots of the multi-chunk experts before e
  for (int ee = tid; ee < e; ee += kThreads) {
    const int c = wgrad_chunks(p.offsets[ee + 1] - p.offsets[ee], R);
    before += c > 1 ? c : 0;
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) before += wave_shfl_xor(before, d);
  if (lane == 0) sSum[wave] = before;
  __syncthreads();
  const int slot0 = sSum[0] + sSum[1] + sSum[2] + sSum[3];
  const int nb = tile_id % p.n_n_blocks, kb = tile_id / p.n_n_blocks;
  const ColBlock kcol = find_col_block(p.bounds, p.n_tiles, kb);
  const int n0 = nb * kTileCols;
  const float* __restrict__ first = p.partial + ((int64_t)slot0 * tiles + tile_id) * kWgradTileElems;
  T* __restrict__ GW = static_cast<T*>(p.grad_w) + (int64_t)e * p.K * p.N;
  constexpr int kIters = kWgradTileElems / (4 * kThreads * kWgradReduceSplit);
  const int64_t cstride = (int64_t)tiles * kWgradTileElems;
  for (int it = 0; it < kIters; it++) {
    const int idx = ((part * kIters + it) * kThreads + tid) * 4;
    const int row = idx / kTileCols, col = idx % kTileCols;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    int c = 0;
    for (; c + 4 <= n_chunks; c += 4) {      // four loads in flight, added in chunk order
      f32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const f32x4*>(&first[(c + u) * cstride + idx]);
#pragma unroll
      for (int u = 0; u < 4; u++) sum += v[u];
    }
    for (; c < n_chunks; c++) sum += *reinterpret_cast<const f32x4*>(&first[c * cstride + idx]);
    const int kk = kcol.c0 + row, n = n0 + col;
    int nv = kk < kcol.c1 ? p.N - n : 0;
    nv = nv < 0 ? 0 : (nv > 4 ? 4 : nv);
    float v[4] = {sum[0], sum[1], sum[2], sum[3]};
    if (nv > 0) store4<T>(GW + (int64_t)kk * p.N + n, v, nv, p.out_vec != 0);
  }
}

}  // namespace amoe
