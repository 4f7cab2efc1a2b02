// Shared device helpers: element types, bf16 conversion, vector load/store, tile lookup.
#pragma once
#include <gfx950_intrin.h>
#include <stdint.h>

namespace amoe {

constexpr int kThreads = 256;   // 4 waves per workgroup, arranged 2 x 2 over the output tile
constexpr int kTileRows = 128;  // token rows per workgroup tile
constexpr int kTileCols = 128;  // feature columns per workgroup tile
constexpr int kMaxTiles = 16;
constexpr int kSelMaxExperts = 2048;   // experts the sort, the per-expert tables and their LDS copies are sized for

// Bit casts through by-value helpers (a bit cast applied directly to a vector element
// reads element 0 with this compiler).
__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---- bf16 <-> fp32 (round to nearest even), on raw bits -----------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return as_f32((uint32_t)h << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return (uint16_t)(pack_bf16x2(f, 0.f) & 0xffffu);   // hardware conversion, ties to even
}

// ---- fp16 <-> fp32 (round to nearest even) ----------------------------------------------------
// The element type of fp16 tensors is f16_t; bf16 tensors are handled as their bits (uint16_t).
typedef _Float16 f16_t;
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_v;
  typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_v;
  const f32x2_v v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_v));
}
__device__ __forceinline__ void unpack_f16x2(uint32_t w, float& lo, float& hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_v;
  typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_v;
  const f32x2_v v = __builtin_convertvector(__builtin_bit_cast(f16x2_v, w), f32x2_v);
  lo = v[0];
  hi = v[1];
}
template <typename T> constexpr bool kIsF16 = false;
template <> constexpr bool kIsF16<f16_t> = true;
// the 16 bits of one element, whatever its type
template <typename T> __device__ __forceinline__ uint32_t elem_bits16(T v) {
  return (uint32_t)__builtin_bit_cast(uint16_t, v);
}

// Element traits.  Chunk = 16 bytes of elements, the unit of global and LDS vector access.
template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int kChunk = 4;     // elements per 16 bytes
  static constexpr int kBK = 32;       // contraction elements staged per step (128 B per row)
  static constexpr int kMmaK = 2;      // contraction elements per matrix instruction
  static constexpr int kPadKC = 4;     // row padding of the k-contiguous LDS layout
  static constexpr int kPadRC = 4;     // row padding of the row-contiguous LDS layout
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ float cvt(float v) { return v; }
  static __device__ __forceinline__ float to_f32(float v) { return v; }
};
template <> struct Elem<uint16_t> {    // bf16 bits
  static constexpr int kChunk = 8;
  static constexpr int kBK = 64;
  static constexpr int kMmaK = 16;
  static constexpr int kPadKC = 8;
  static constexpr int kPadRC = 32;     // row stride 320 B: the four rows x two 16-column groups of a
                                       // transposing read land on disjoint LDS banks
  static __device__ __forceinline__ float load(const uint16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ uint16_t cvt(float v) { return f32_to_bf16(v); }
  static __device__ __forceinline__ float to_f32(uint16_t v) { return bf16_to_f32(v); }
};

template <> struct Elem<f16_t> : Elem<uint16_t> {    // same tiling as bf16
  static __device__ __forceinline__ float load(const f16_t* p) { return (float)*p; }
  static __device__ __forceinline__ f16_t cvt(float v) { return (f16_t)v; }
  static __device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
};

// 32 x 32 x 16 matrix instruction on 16-bit operands of type T
template <typename T>
__device__ __forceinline__ f32x16 mfma_32x32x16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (kIsF16<T>) return mfma_32x32x16_f16(a, b, c);
  else return mfma_32x32x16_bf16(a, b, c);
}

// ---- 16-byte chunks --------------------------------------------------------------------------
// Operands travel global -> registers -> LDS as raw 16-byte chunks; only the gathered rows of
// the analog forward are unpacked to fp32 (for the DAC stage) on the way.
typedef u32x4 Raw;

__device__ __forceinline__ Raw raw_zero() { return Raw{0u, 0u, 0u, 0u}; }

// Store one chunk of an output that this kernel does not read again, with the non-temporal hint: a tile of results
// is written once, in whole 128-byte lines, and is far larger than the L2 in total; as ordinary stores the lines
// stay in the L2 until they are evicted, and the launches whose output is large against their arithmetic (four K
// steps per 128 x 128 tile) spent a quarter of their time on that (0.184 -> 0.147 ms for the plain forward).
template <typename T>
__device__ __forceinline__ void store_streaming(T* p, const Raw& v) {
  __builtin_nontemporal_store(v, reinterpret_cast<Raw*>(p));
}

// Load one chunk starting at p (elements [0, n_valid) exist; the rest read as zero).
// vec: p is 16-byte aligned and the caller allows vector access.
template <typename T>
__device__ __forceinline__ Raw raw_load(const T* p, int n_valid, bool vec) {
  constexpr int C = Elem<T>::kChunk;
  if (vec && n_valid >= C) return *reinterpret_cast<const Raw*>(p);
  Raw r = raw_zero();
  if (n_valid <= 0) return r;
  if constexpr (sizeof(T) == 2) {
    // a complete bf16 chunk that is only 8- or 4-byte aligned (row strides that are multiples of 4
    // or 2 elements): two or four loads instead of eight
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
    if (n_valid >= C && (addr & 7) == 0) {
      const u32x2 lo = *reinterpret_cast<const u32x2*>(p), hi = *reinterpret_cast<const u32x2*>(p + 4);
      return Raw{lo[0], lo[1], hi[0], hi[1]};
    }
    if (n_valid >= C && (addr & 3) == 0) {
      const uint32_t* q = reinterpret_cast<const uint32_t*>(p);
      return Raw{q[0], q[1], q[2], q[3]};
    }
  }
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int j = 0; j < 4; j++) r[j] = (j < n_valid) ? as_u32(p[j]) : 0u;
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t lo = (2 * j < n_valid) ? elem_bits16(p[2 * j]) : 0u;
      const uint32_t hi = (2 * j + 1 < n_valid) ? elem_bits16(p[2 * j + 1]) : 0u;
      r[j] = lo | (hi << 16);
    }
  }
  return r;
}

// raw_load for operands that are read exactly once by the whole launch (the k-head tensors of the row-wise
// companions): a complete, aligned chunk is fetched with the non-temporal hint, so that it does not push the
// operand tiles of a GEMM launch running beside it out of the L2.
template <typename T>
__device__ __forceinline__ Raw raw_load_streaming(const T* p, int n_valid, bool vec) {
  if (vec && n_valid >= Elem<T>::kChunk) return __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p));
  return raw_load<T>(p, n_valid, vec);
}

template <typename T>
__device__ __forceinline__ void raw_unpack(const Raw& r, float (&v)[Elem<T>::kChunk]) {
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = as_f32(r[j]);
  } else if constexpr (kIsF16<T>) {
#pragma unroll
    for (int j = 0; j < 4; j++) unpack_f16x2(r[j], v[2 * j], v[2 * j + 1]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j] = as_f32(r[j] << 16);
      v[2 * j + 1] = as_f32(r[j] & 0xffff0000u);
    }
  }
}

// fp32 -> T with round to nearest even.
template <typename T>
__device__ __forceinline__ Raw raw_pack(const float (&v)[Elem<T>::kChunk]) {
  Raw r;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int j = 0; j < 4; j++) r[j] = as_u32(v[j]);
  } else if constexpr (kIsF16<T>) {
#pragma unroll
    for (int j = 0; j < 4; j++) r[j] = pack_f16x2(v[2 * j], v[2 * j + 1]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) r[j] = pack_bf16x2(v[2 * j], v[2 * j + 1]);
  }
  return r;
}

// fp32 values that are exactly representable in bf16 (small integers): plain truncation.
__device__ __forceinline__ Raw raw_pack_exact_bf16(const float (&v)[8]) {
  Raw r;
#pragma unroll
  for (int j = 0; j < 4; j++) r[j] = pack_high_halves(as_u32(v[2 * j + 1]), as_u32(v[2 * j]));
  return r;
}
// DAC codes as 16-bit elements of T.  Exact only while the type holds the integers: |code| <= 256 in bf16 (the
// truncation below drops nothing then), <= 2048 in fp16; the host rejects finer input quantisers for these types.
template <typename T>
__device__ __forceinline__ Raw raw_pack_codes(const float (&v)[8]) {
  if constexpr (kIsF16<T>) return raw_pack<T>(v);
  else return raw_pack_exact_bf16(v);
}

// a / b given y = 1/b (correctly rounded): one multiply and two fused multiply-adds give the
// correctly rounded quotient (checked against IEEE division over 4e8 random operand pairs of
// the DAC stage's value ranges, including all-ones and near-power-of-two divisors).
__device__ __forceinline__ float div_by(float a, float b, float y) {
  const float q0 = a * y;
  const float r = fmaf(-q0, b, a);
  return fmaf(r, y, q0);
}

// Store 4 consecutive fp32 values as T to global memory at p; n_valid of them exist.
template <typename T>
__device__ __forceinline__ void store4(T* p, const float (&v)[4], int n_valid, bool vec) {
  if (vec && n_valid >= 4) {
    if constexpr (sizeof(T) == 4) {
      f32x4 o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4*>(p) = o;
    } else {
      u32x2 o;
      o[0] = kIsF16<T> ? pack_f16x2(v[0], v[1]) : pack_bf16x2(v[0], v[1]);
      o[1] = kIsF16<T> ? pack_f16x2(v[2], v[3]) : pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<u32x2*>(p) = o;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (j < n_valid) p[j] = Elem<T>::cvt(v[j]);
  }
}

// Load 4 consecutive elements of T from global memory as fp32.
template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&v)[4], int n_valid, bool vec) {
  if (vec && n_valid >= 4) {
    if constexpr (sizeof(T) == 4) {
      f32x4 o = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
      for (int j = 0; j < 4; j++) v[j] = o[j];
    } else if constexpr (kIsF16<T>) {
      u32x2 o = *reinterpret_cast<const u32x2*>(p);
      unpack_f16x2(o[0], v[0], v[1]);
      unpack_f16x2(o[1], v[2], v[3]);
    } else {
      u32x2 o = *reinterpret_cast<const u32x2*>(p);
      v[0] = as_f32(o[0] << 16);
      v[1] = as_f32(o[0] & 0xffff0000u);
      v[2] = as_f32(o[1] << 16);
      v[3] = as_f32(o[1] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = (j < n_valid) ? Elem<T>::load(p + j) : 0.f;
  }
}

// ---- row-tile lookup -------------------------------------------------------------------------
// Sorted positions are cut into tiles of kTileRows rows that never cross an expert boundary.
// Tile `tile` of the whole list -> (expert, first sorted position, end position).  Every
// thread of the workgroup calls this; info[0] < 0 means the tile does not exist.
__device__ __forceinline__ void find_row_tile(const int32_t* __restrict__ offsets, int E, int tile,
                                              int* info /* LDS int[8] */, int* wave_sums /* LDS int[4] */) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = (E + kThreads - 1) / kThreads;
  const int e0 = tid * per;
  int mine = 0;
  for (int j = 0; j < per; j++) {
    int e = e0 + j;
    if (e < E) mine += (offsets[e + 1] - offsets[e] + kTileRows - 1) / kTileRows;
  }
  int incl = mine;  // inclusive scan over the wave
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int up = wave_shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (tid == 0) info[0] = -1;
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; w++) base += wave_sums[w];
  int excl = base + incl - mine;
  if (tile >= excl && tile < excl + mine) {
    int t = excl;
    for (int j = 0; j < per; j++) {
      int e = e0 + j;
      if (e < E) {
        int lo = offsets[e], hi = offsets[e + 1];
        int nt = (hi - lo + kTileRows - 1) / kTileRows;
        if (tile < t + nt) {
          int r0 = lo + (tile - t) * kTileRows;
          info[0] = e;
          info[1] = r0;
          info[2] = (r0 + kTileRows < hi) ? r0 + kTileRows : hi;
          break;
        }
        t += nt;
      }
    }
  }
  __syncthreads();
}

// Feature blocks of `width` columns (kTileCols unless said otherwise) that restart at every K-tile bound, so that one block
// lies inside one K-tile.  Block b -> (first column, end column, K-tile).
struct ColBlock { int c0, c1, tile; };
__device__ __host__ inline int count_col_blocks(const int32_t* bounds, int n_tiles, int width = kTileCols) {
  int n = 0;
  for (int t = 0; t < n_tiles; t++) n += (bounds[t + 1] - bounds[t] + width - 1) / width;
  return n;
}
__device__ __forceinline__ ColBlock find_col_block(const int32_t* bounds, int n_tiles, int b, int width = kTileCols) {
  ColBlock r{0, 0, 0};
  for (int t = 0; t < n_tiles; t++) {
    int nb = (bounds[t + 1] - bounds[t] + width - 1) / width;
    if (b < nb) {
      r.c0 = bounds[t] + b * width;
      r.c1 = (r.c0 + width < bounds[t + 1]) ? r.c0 + width : bounds[t + 1];
      r.tile = t;
      return r;
    }
    b -= nb;
  }
  return r;
}

// ---- counter-based Gaussian noise ---------------------------------------------------------------
// Pure function of (seed, K-tile, output row, column pair): one 32-bit hash per pair, its two
// 16-bit halves drive one Box-Muller transform.
__device__ __host__ inline uint32_t fmix32(uint32_t h) {
  h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  return h;
}
struct NoiseKey { uint32_t ka, kb, seed_hi; };
__device__ __host__ inline NoiseKey noise_key(uint64_t seed, int tile) {
  NoiseKey k;
  k.ka = fmix32(((uint32_t)seed ^ 0x9E3779B9u) + (uint32_t)tile * 0x632BE5ABu);
  k.kb = fmix32(((uint32_t)(seed >> 32) ^ 0x85EBCA77u) + (uint32_t)tile * 0x27D4EB2Fu);
  k.seed_hi = (uint32_t)(seed >> 32);
  return k;
}
// Key of an output row (once per row and K tile), then the pair of normals of column pair p.
__device__ __forceinline__ uint32_t noise_row_key(const NoiseKey& key, uint32_t row) { return fmix32(row ^ key.ka); }
__device__ __forceinline__ void noise_pair(const NoiseKey& key, uint32_t row_key, uint32_t pair, float& z0, float& z1) {
  uint32_t h = row_key + pair * 0x9E3779B9u;
  h ^= h >> 16; h *= 0x85EBCA6Bu; h += key.kb; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  const float u1 = fmaf((float)(h >> 16), 1.0f / 65536.0f, 0.5f / 65536.0f);   // exact: (b + 0.5) / 65536
  const float u2 = (float)(h & 0xffffu) * (1.0f / 65536.0f);
  const float r = fast_sqrt(-1.3862943611f * fast_log2(u1));     // sqrt(-2 ln u1)
  z0 = r * fast_cos_rev(u2);
  z1 = r * fast_sin_rev(u2);
}

// ---- counter-based Gaussian noise of the forward output stage, drawn on the matrix unit ---------------------
// The noise of a 32 x 32 block of outputs is the product of two 32 x 32 matrices of pseudo-random signed bytes,
// one row per output row and one per output column:  z[row][col] = sum_k a[row][k] * b[col][k] - 8, an integer
// with mean 0 and standard deviation sqrt(32) * 5461.5, approximately normal (excess kurtosis 0.01; entries of a
// block are uncorrelated, blocks are independent).  One 8-bit matrix instruction per block replaces a hash and a
// Box-Muller transform per output; what is left per output is one integer-to-float conversion.
//   a[row] : the 8 words of the key  row_key ^ (col / 32) * 0x632BE5AB,   row_key = fmix32(out_row ^ ka)
//   b[col] : the 8 words of the key  col_key ^ block_start * 0x27D4EB2F,  col_key = fmix32(col * 0x9E3779B1 ^ kb)
// (xor, not add: keys that differ by a constant give words that differ by a constant, hence correlated bytes)
// block_start = sorted position of the block's first row: blocks are the 32-row groups counted from the first
// sorted position of the expert.  Byte i of word j is contraction index 4 * j + i (any pairing gives the same sum).
constexpr float kNoiseScale = (float)(1.0 / (5.656854249492380195 * 5461.5));
// word j (0 .. 7) of a key's vector: words 0 .. 3 from the key, words 4 .. 7 from key ^ kNoiseHalfKey, each
// (k mod 2^24) * c_(j mod 4) + k followed by one xor-shift.  (Unrelated odd 24-bit multipliers: with multipliers in
// arithmetic progression the words are in arithmetic progression too, which shows as an excess kurtosis of 0.1.
// The four multipliers are the same for every lane, so they live in scalar registers.)
constexpr uint32_t kNoiseHalfKey = 0x5BD1E995u;
constexpr uint32_t kNoiseMul0 = 0x9E3779u, kNoiseMul1 = 0x85EBCBu, kNoiseMul2 = 0xC2B2AFu, kNoiseMul3 = 0x27D4EBu;
__device__ __forceinline__ uint32_t noise_word(uint32_t key, uint32_t cj) {
  uint32_t w = mul_u24(key, cj) + key;
  return w ^ (w >> 15);
}
__device__ __forceinline__ u32x4 noise_words(uint32_t key) {
  return u32x4{noise_word(key, kNoiseMul0), noise_word(key, kNoiseMul1), noise_word(key, kNoiseMul2),
               noise_word(key, kNoiseMul3)};
}
__device__ __forceinline__ uint32_t noise_col_key(const NoiseKey& key, uint32_t col) {
  return fmix32((col * 0x9E3779B1u) ^ key.kb);
}
// Integer noise of the block whose rows this wave's lanes l % 32 name by row_key and whose columns they name by
// col_key; lane l gets the 16 values of its accumulator slots (the layout of an fp32 32 x 32 tile whose first
// operand is the column side).  half = l / 32 picks the lane's 16 of the 32 contraction indices.
__device__ __forceinline__ i32x16 noise_block(uint32_t row_key, uint32_t col_key, uint32_t col_block,
                                              uint32_t block_start, int half) {
  const uint32_t hk = half ? kNoiseHalfKey : 0u;
  const uint32_t ak = row_key ^ (col_block * 0x632BE5ABu) ^ hk;
  const uint32_t bk = col_key ^ (block_start * 0x27D4EB2Fu) ^ hk;
  const u32x4 aw = noise_words(ak), bw = noise_words(bk);
  i32x16 c;
#pragma unroll
  for (int i = 0; i < 16; i++) c[i] = -8;
  return mfma_i32_32x32x32_i8(bw, aw, c);
}

}  // namespace amoe
