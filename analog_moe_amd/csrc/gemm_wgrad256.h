// Segmented weight gradient for the usual training shapes (bf16 or fp16; 16-byte aligned operands, 32-bit
// addressable; K-tiles and N multiples of 256): the 256 (kk) x 256 (n) counterpart of gemm_wgrad_kernel, same
// arithmetic, same fixed summation order along the rows.
//     grad_w[e][kk][n] = sum_{i in expert e} scale_i * clamp(x[in_index[i]][kk], +-ir) * g[g_index[i]][n]
// One workgroup of 512 threads (4 x 2 waves of 64 x 128: half the LDS fragment traffic per matrix instruction of the
// 128 x 128 kernel, and every operand row is read once per 256 instead of per 128 columns of the other operand) owns
// one 256 x 256 tile of one expert, or of one chunk of its rows; one workgroup per CU (144 KB of LDS stages).  Row chunks, their partial
// tiles (laid out as the four 128 x 128 tiles they cover, so that wgrad_reduce_kernel adds them unchanged) and the
// placement of the tiles of one chunk on one XCD are those of gemm_wgrad_kernel.
#pragma once
#include "gemm_wgrad.h"

namespace amoe {

constexpr int kW256Threads = 512;
constexpr int kW256Tile = 256;

// index, among the 128-column blocks of all K-tiles, of the block that starts at column c0 of K-tile `tile`
__device__ __forceinline__ int find_block128(const int32_t* bounds, int tile, int c0) {
  int n = 0;
  for (int t = 0; t < tile; t++) n += (bounds[t + 1] - bounds[t] + kTileCols - 1) / kTileCols;
  return n + (c0 - bounds[tile]) / kTileCols;
}

template <typename T>
__global__ __launch_bounds__(kW256Threads, 2) void wgrad256_kernel(const WgradParams p) {
  static_assert(sizeof(T) == 2, "16-bit elements: bf16 (as bits) or fp16");
  constexpr int CH = 8, NT = kW256Threads;
  constexpr int BT = 64;                          // tokens per step (32: 4-5 % slower, 10 % with skewed routing)
  constexpr int NP = BT / 16;                     // staging passes: 16 rows of 32 pieces per pass
  constexpr int LD = kW256Tile + 32;              // 576-byte rows: the rows of a transposing read are disjoint
  constexpr int STAGE = BT * LD;                  // one operand, one stage: 36 KB (144 KB in all: one workgroup per CU)
  constexpr int LDO = kW256Tile + 8, OUT_ROWS = 64;
  static_assert(OUT_ROWS * LDO <= 4 * STAGE, "the staged output rows must fit the stage buffers");
  __shared__ __attribute__((aligned(16))) T sS[4 * STAGE];
  T* const sX = sS;
  T* const sG = sS + 2 * STAGE;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wk = wave >> 1, wn = wave & 1;        // kk rows wk * 64 .., n columns wn * 128 ..
  const int l32 = lane & 31, lh = lane >> 5;

  int* const sScanA = reinterpret_cast<int*>(sS);
  int* const sScanB = sScanA + 8;
  int* const sFound = sScanA + 16;
  // tiles of 256 x 256 per expert; the reduce kernel and the partial buffer count tiles of 128 x 128
  const int kb256 = p.n_k_blocks / 2, nb256 = p.n_n_blocks / 2;
  const int tiles_per_expert = kb256 * nb256;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int cg = xcd + 8 * (slot / tiles_per_expert);      // index of the (expert, chunk) pair
  const int tile_id = slot % tiles_per_expert;
  int e = cg, chunk_id = 0, n_chunks = 1, part_slot = 0;
  if (p.rows_per_chunk > 0) {
    const int R = p.rows_per_chunk;
    const int per = (p.E + NT - 1) / NT;
    int mineA = 0, mineB = 0;
    for (int j = 0; j < per; j++) {
      const int ee = tid * per + j;
      if (ee < p.E) {
        const int c = wgrad_chunks(p.offsets[ee + 1] - p.offsets[ee], R);
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
        const int c = wgrad_chunks(p.offsets[ee + 1] - p.offsets[ee], R);
        if (cg >= beforeA && cg < beforeA + c) {
          sFound[0] = ee; sFound[1] = cg - beforeA; sFound[2] = c; sFound[3] = beforeB;
        }
        beforeA += c;
        beforeB += c > 1 ? c : 0;
      }
    }
    __syncthreads();
    e = wave_uniform(sFound[0]); chunk_id = wave_uniform(sFound[1]); n_chunks = wave_uniform(sFound[2]);
    part_slot = wave_uniform(sFound[3]) + chunk_id;
    if (e < 0) return;
    __syncthreads();                       // the scratch is stage memory again from here on
  } else if (e >= p.E) {
    return;
  }
  const int nb = tile_id % nb256, kb = tile_id / nb256;
  const ColBlock kcol = find_col_block(p.bounds, p.n_tiles, kb, kW256Tile);
  const int kc0 = kcol.c0;
  const int n0 = nb * kW256Tile;
  int seg0 = p.offsets[e], seg1 = p.offsets[e + 1];
  if (p.rows_per_chunk > 0 && n_chunks > 1) {
    seg0 += chunk_id * p.rows_per_chunk;
    seg1 = seg0 + p.rows_per_chunk < seg1 ? seg0 + p.rows_per_chunk : seg1;
  }

  const T* __restrict__ X = static_cast<const T*>(p.x);
  const T* __restrict__ G = static_cast<const T*>(p.g);
  const T* __restrict__ GS = static_cast<const T*>(p.g_scale);
  const bool has_ir = p.ir != nullptr;
  const float ir_expert = has_ir ? p.ir[(int64_t)e * p.n_tiles + kcol.tile] : __builtin_inff();   // (per expert only)

  f32x16 acc[4][2];                              // [n block fn][kk block fk]
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][c][i] = 0.f;

  // per-row metadata (x row, g row, scale) of a step: one lane per row and item fetches it two steps ahead and
  // hands it over through the padding behind the 256 operand columns of the x stage rows
  auto meta = [&](int buf, int row) -> int* { return reinterpret_cast<int*>(&sX[buf * STAGE + row * LD + kW256Tile]); };
  const int m_item = tid / BT, m_row = tid % BT;
  int m_val = 0;
  auto fetch_meta = [&](int i0) {
    const int r = i0 + m_row;
    const bool ok = r < seg1;
    if (m_item == 0) m_val = ok ? p.in_index[r] : -1;                       // -1: no such row, the chunk reads as zero
    else if (m_item == 1) m_val = ok ? (p.g_index ? p.g_index[r] : p.in_index[r]) : 0;
    else if (m_item == 2) m_val = (int)as_u32((GS != nullptr && ok) ? Elem<T>::load(GS + r) : 1.f);
  };
  auto publish_meta = [&](int buf) {
    if (m_item < 3) meta(buf, m_row)[m_item] = m_val;
  };

  const int chunk = tid & 31, srow = tid >> 5;                 // staging: rows srow, srow + 16; 16-byte piece `chunk`
  const BufRsrc rsX = make_rsrc(X), rsG = make_rsrc(G);
  const uint32_t x_row_bytes = (uint32_t)(p.ldx * 2), g_row_bytes = (uint32_t)(p.ldg * 2);
  const uint32_t x_col_bytes = (uint32_t)((kc0 + chunk * CH) * 2), g_col_bytes = (uint32_t)((n0 + chunk * CH) * 2);
  Raw rx[NP], rg[NP];
  auto load_rows = [&](int mbuf) {
#pragma unroll
    for (int i = 0; i < NP; i++) {
      const int* m = meta(mbuf, srow + 16 * i);
      const int xr = m[0];
      rx[i] = raw_zero();
      rg[i] = raw_zero();
      if (xr >= 0) {
        rx[i] = buffer_load_b128(rsX, (uint32_t)xr * x_row_bytes + x_col_bytes, 0);
        rg[i] = buffer_load_b128(rsG, (uint32_t)m[1] * g_row_bytes + g_col_bytes, 0);
      }
    }
  };
  auto store_step = [&](int buf, int mbuf) {  // registers -> LDS, clip / row scaling of x on the way
    T* __restrict__ dX = sX + buf * STAGE;
    T* __restrict__ dG = sG + buf * STAGE;
    if (has_ir || GS != nullptr) {
#pragma unroll
      for (int i = 0; i < NP; i++) {
        const float scale = as_f32((uint32_t)meta(mbuf, srow + 16 * i)[2]);
        float v[CH];
        raw_unpack<T>(rx[i], v);
#pragma unroll
        for (int q = 0; q < CH; q++) v[q] = clamp_sym(v[q], ir_expert) * scale;
        rx[i] = raw_pack<T>(v);
      }
    }
#pragma unroll
    for (int i = 0; i < NP; i++) {
      *reinterpret_cast<Raw*>(&dX[(srow + 16 * i) * LD + chunk * CH]) = rx[i];
      *reinterpret_cast<Raw*>(&dG[(srow + 16 * i) * LD + chunk * CH]) = rg[i];
    }
  };

  // Pipeline as in gemm_wgrad_kernel: data of step s in stage s & 1; the metadata of step s + 1 in the padding of
  // stage s & 1, that of step s + 2 published at the end of step s into stage (s + 1) & 1 with the data of s + 1.
  const int nsteps = (seg1 - seg0 + BT - 1) / BT;
  if (nsteps > 0) {
    fetch_meta(seg0);
    publish_meta(1);
    __syncthreads();
    load_rows(1);
    fetch_meta(seg0 + BT);
    __syncthreads();
    store_step(0, 1);
    __syncthreads();
    publish_meta(0);
    __syncthreads();
  }
  for (int s = 0; s < nsteps; s++) {
    const int cur = s & 1;
    const bool more = s + 1 < nsteps;
    if (more) {
      load_rows(cur);
      fetch_meta(seg0 + (s + 2) * BT);
    }
    const T* __restrict__ cX = sX + cur * STAGE;
    const T* __restrict__ cG = sG + cur * STAGE;
#pragma unroll
    for (int kk = 0; kk < BT; kk += 16) {
      const int R = lane & 15, gq = (lane >> 4) & 1;
      const int roff = (kk + 8 * lh + (R >> 2)) * LD + 16 * gq + 4 * (R & 3);
      u32x4 gf[4], xf[2];
#pragma unroll
      for (int f = 0; f < 2; f++) {
        const uint16_t* bx = reinterpret_cast<const uint16_t*>(&cX[roff + wk * 64 + f * 32]);
        const u32x2 lo = lds_read_tr16_b64(bx), hi = lds_read_tr16_b64(bx + 4 * LD);
        xf[f] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
#pragma unroll
      for (int f = 0; f < 4; f++) {
        const uint16_t* bg = reinterpret_cast<const uint16_t*>(&cG[roff + wn * 128 + f * 32]);
        const u32x2 lo = lds_read_tr16_b64(bg), hi = lds_read_tr16_b64(bg + 4 * LD);
        gf[f] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
#pragma unroll
      for (int fn = 0; fn < 4; fn++)
#pragma unroll
        for (int fk = 0; fk < 2; fk++) acc[fn][fk] = mfma_32x32x16<T>(gf[fn], xf[fk], acc[fn][fk]);
    }
    if (more) {
      store_step(cur ^ 1, cur);
      publish_meta(cur ^ 1);
    }
    __syncthreads();
  }

  if (n_chunks > 1) {
    // this chunk's tile in fp32, as the four 128 x 128 tiles wgrad_reduce_kernel knows: this wave's rows and
    // columns lie in tile (2 kb + wk / 2, 2 nb + wn)
    const int tiles128 = p.n_k_blocks * p.n_n_blocks;
    const int kb128 = find_block128(p.bounds, kcol.tile, kc0) + (wk >> 1);
    const int t128 = kb128 * p.n_n_blocks + 2 * nb + wn;
    float* __restrict__ mine = p.partial + ((int64_t)part_slot * tiles128 + t128) * kWgradTileElems;
#pragma unroll
    for (int fk = 0; fk < 2; fk++)
#pragma unroll
      for (int fn = 0; fn < 4; fn++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          f32x4 v;
#pragma unroll
          for (int j = 0; j < 4; j++) v[j] = acc[fn][fk][4 * q + j];
          *reinterpret_cast<f32x4*>(&mine[((wk & 1) * 64 + fk * 32 + l32) * kTileCols + fn * 32 + 8 * q + 4 * lh]) = v;
        }
    return;
  }
  // registers -> LDS -> whole 512-byte row segments, 64 rows (one wk) at a time
  T* __restrict__ GW = static_cast<T*>(p.grad_w) + (int64_t)e * p.K * p.N;
  T* __restrict__ sOut = sS;
#pragma unroll 1
  for (int pass = 0; pass < 4; pass++) {
    if (wk == pass) {
#pragma unroll
      for (int fk = 0; fk < 2; fk++)
#pragma unroll
        for (int fn = 0; fn < 4; fn++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = acc[fn][fk][4 * q + j];
            store4<T>(&sOut[(fk * 32 + l32) * LDO + wn * 128 + fn * 32 + 8 * q + 4 * lh], v, 4, true);
          }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int rl = srow + 16 * i;
      store_streaming(GW + (int64_t)(kc0 + pass * 64 + rl) * p.N + n0 + chunk * CH,
                      *reinterpret_cast<const Raw*>(&sOut[rl * LDO + chunk * CH]));
    }
    __syncthreads();
  }
}

}  // namespace amoe
