// CPU stand-ins for the gfx950 instruction wrappers (see the device header of the same name
// for the operand layouts these reproduce).  Test build only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace amoe {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

struct BufRsrc { const unsigned char* base; uint32_t bytes; };
inline BufRsrc make_rsrc(const void* base) { return BufRsrc{static_cast<const unsigned char*>(base), 0xffffffffu}; }
inline BufRsrc make_rsrc_sized(void* base, uint32_t bytes) { return BufRsrc{static_cast<const unsigned char*>(base), bytes}; }
inline u32x4 buffer_load_b128(BufRsrc r, uint32_t lane_off, uint32_t uniform_off) {
  u32x4 v;
  std::memcpy(&v, r.base + (size_t)lane_off + (size_t)uniform_off, 16);
  return v;
}
inline uint32_t buffer_load_b32(BufRsrc r, uint32_t lane_off) {
  uint32_t v;
  std::memcpy(&v, r.base + (size_t)lane_off, 4);
  return v;
}
// out-of-range stores are dropped, as the hardware's range check does
inline void buffer_store_b128_nt(BufRsrc r, u32x4 v, uint32_t lane_off) {
  if ((uint64_t)lane_off + 16 <= r.bytes) std::memcpy(const_cast<unsigned char*>(r.base) + lane_off, &v, 16);
}
inline uint32_t pack_high_halves(uint32_t hi, uint32_t lo) { return (hi & 0xffff0000u) | (lo >> 16); }
// scheduling fences mean nothing to a host compiler
inline void sched_fence() {}

inline int lane_id() { return threadIdx.x & 63; }

template <class V> inline V emu_exchange(V v, int src) {
  static_assert(sizeof(V) <= 64, "slot too small");
  EmuWave* w = emu_wave;
  std::memcpy(w->slot[lane_id()], &v, sizeof(V));
  w->bar.arrive_and_wait();
  V r;
  std::memcpy(&r, w->slot[src & 63], sizeof(V));
  w->bar.arrive_and_wait();
  return r;
}
template <class V> inline V wave_shfl_xor(V v, int mask) { return emu_exchange(v, lane_id() ^ mask); }
template <class V> inline V wave_shfl(V v, int src) { return emu_exchange(v, src); }
template <class V> inline V wave_shfl_up(V v, int d) {
  int l = lane_id();
  return emu_exchange(v, l >= d ? l - d : l);
}
inline uint64_t wave_ballot(bool p) {
  EmuWave* w = emu_wave;
  w->slot[lane_id()][0] = p ? 1 : 0;
  w->bar.arrive_and_wait();
  uint64_t m = 0;
  for (int i = 0; i < 64; i++) m |= (uint64_t)(w->slot[i][0] & 1) << i;
  w->bar.arrive_and_wait();
  return m;
}
inline int popc64(uint64_t v) { return __builtin_popcountll(v); }
inline void wave_sync() { emu_wave->bar.arrive_and_wait(); }

inline float emu_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

inline f32x16 mfma_32x32x16_bf16(u32x4 a, u32x4 b, f32x16 c) {
  struct Ops { uint16_t a[8], b[8]; } mine;
  std::memcpy(mine.a, &a, 16);
  std::memcpy(mine.b, &b, 16);
  EmuWave* w = emu_wave;
  const int l = lane_id();
  std::memcpy(w->slot[l], &mine, sizeof(mine));
  w->bar.arrive_and_wait();
  const int col = l % 32;
  for (int i = 0; i < 16; i++) {
    const int row = 8 * (i / 4) + 4 * (l / 32) + (i % 4);
    float s = c[i];
    for (int k = 0; k < 16; k++) {
      const Ops* pa = (const Ops*)w->slot[row + 32 * (k / 8)];
      const Ops* pb = (const Ops*)w->slot[col + 32 * (k / 8)];
      s += emu_bf16(pa->a[k % 8]) * emu_bf16(pb->b[k % 8]);
    }
    c[i] = s;
  }
  w->bar.arrive_and_wait();
  return c;
}

inline f32x16 mfma_32x32x16_f16(u32x4 a, u32x4 b, f32x16 c) {
  struct Ops { _Float16 a[8], b[8]; } mine;
  std::memcpy(mine.a, &a, 16);
  std::memcpy(mine.b, &b, 16);
  EmuWave* w = emu_wave;
  const int l = lane_id();
  std::memcpy(w->slot[l], &mine, sizeof(mine));
  w->bar.arrive_and_wait();
  const int col = l % 32;
  for (int i = 0; i < 16; i++) {
    const int row = 8 * (i / 4) + 4 * (l / 32) + (i % 4);
    float s = c[i];
    for (int k = 0; k < 16; k++) {
      const Ops* pa = (const Ops*)w->slot[row + 32 * (k / 8)];
      const Ops* pb = (const Ops*)w->slot[col + 32 * (k / 8)];
      s += (float)pa->a[k % 8] * (float)pb->b[k % 8];
    }
    c[i] = s;
  }
  w->bar.arrive_and_wait();
  return c;
}

typedef __attribute__((ext_vector_type(16))) int i32x16;
inline i32x16 mfma_i32_32x32x32_i8(u32x4 a, u32x4 b, i32x16 c) {
  struct Ops { int8_t a[16], b[16]; } mine;
  std::memcpy(mine.a, &a, 16);
  std::memcpy(mine.b, &b, 16);
  EmuWave* w = emu_wave;
  const int l = lane_id();
  std::memcpy(w->slot[l], &mine, sizeof(mine));
  w->bar.arrive_and_wait();
  const int col = l % 32;
  for (int i = 0; i < 16; i++) {
    const int row = 8 * (i / 4) + 4 * (l / 32) + (i % 4);
    int s = c[i];
    for (int k = 0; k < 32; k++) {
      const Ops* pa = (const Ops*)w->slot[row + 32 * (k / 16)];
      const Ops* pb = (const Ops*)w->slot[col + 32 * (k / 16)];
      s += (int)pa->a[k % 16] * (int)pb->b[k % 16];
    }
    c[i] = s;
  }
  w->bar.arrive_and_wait();
  return c;
}
inline uint32_t mul_u24(uint32_t a, uint32_t b) { return (uint32_t)((uint64_t)(a & 0xffffffu) * (uint64_t)(b & 0xffffffu)); }

inline uint32_t cvt_pk_u8_f32(float v, int sel, uint32_t old) {
  const float r = nearbyintf(v);
  const uint32_t b = r <= 0.f ? 0u : (r >= 255.f ? 255u : (uint32_t)r);
  return (old & ~(0xffu << (8 * sel))) | (b << (8 * sel));
}

inline f32x16 mfma_32x32x2_f32(float a, float b, f32x16 c) {
  struct Ops { float a, b; } mine{a, b};
  EmuWave* w = emu_wave;
  const int l = lane_id();
  std::memcpy(w->slot[l], &mine, sizeof(mine));
  w->bar.arrive_and_wait();
  const int col = l % 32;
  for (int i = 0; i < 16; i++) {
    const int row = 8 * (i / 4) + 4 * (l / 32) + (i % 4);
    float s = c[i];
    for (int k = 0; k < 2; k++) {
      const Ops* pa = (const Ops*)w->slot[row + 32 * k];
      const Ops* pb = (const Ops*)w->slot[col + 32 * k];
      s += pa->a * pb->b;
    }
    c[i] = s;
  }
  w->bar.arrive_and_wait();
  return c;
}

inline u32x2 lds_read_tr16_b64(const uint16_t* p) {
  EmuWave* w = emu_wave;
  const int l = lane_id();
  w->ptr[l] = p;
  w->bar.arrive_and_wait();
  const int base = l & ~15, i = l & 15;
  uint16_t r[4];
  for (int j = 0; j < 4; j++) {
    const uint16_t* row = (const uint16_t*)w->ptr[base + i / 4 + 4 * j];
    r[j] = row[i % 4];
  }
  w->bar.arrive_and_wait();
  u32x2 out;
  std::memcpy(&out, r, 8);
  return out;
}

inline uint32_t emu_f32_to_bf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
inline uint32_t pack_bf16x2(float lo, float hi) { return emu_f32_to_bf16(lo) | (emu_f32_to_bf16(hi) << 16); }

inline float clamp_sym(float x, float r) { return x != x ? -r : (x > r ? r : (x < -r ? -r : x)); }
inline float fast_sin_rev(float x) { return sinf(6.283185307179586f * x); }
inline float fast_cos_rev(float x) { return cosf(6.283185307179586f * x); }
inline int wave_uniform(int v) { return v; }
inline float fast_log2(float x) { return log2f(x); }
inline float fast_sqrt(float x) { return sqrtf(x); }
inline uint32_t umulhi32(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }

}  // namespace amoe
