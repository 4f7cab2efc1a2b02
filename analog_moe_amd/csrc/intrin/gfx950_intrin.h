// gfx950 (CDNA4) instruction wrappers used by the CVMM kernels.
//
// Operand layouts of the two matrix instructions used here, for lane l of a 64-wide wave
// (measured on MI355X with one-hot operands):
//   v_mfma_f32_32x32x16_bf16: A lane l holds A[l%32][8*(l/32) .. +7], B lane l holds
//     B[8*(l/32) .. +7][l%32]; D lane l holds D[8*(i/4) + 4*(l/32) + i%4][l%32], i = 0..15.
//   v_mfma_f32_32x32x2_f32:   A lane l holds A[l%32][l/32], B lane l holds B[l/32][l%32];
//     D as above.
//   ds_read_b64_tr_b16: within each group of 16 lanes, lane R supplies the address of four
//     consecutive 16-bit elements (a "row"); lane i receives element (i%4) of rows
//     i/4, i/4+4, i/4+8, i/4+12.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace amoe {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;

__device__ __forceinline__ f32x16 mfma_32x32x16_bf16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// the same tile on fp16 operands (same operand layout)
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
__device__ __forceinline__ f32x16 mfma_32x32x16_f16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// 32x32x32 signed 8-bit product, 32-bit integer accumulate: lane l supplies 16 bytes of row l%32 of each
// operand (contraction indices 16*(l/32) .. +15); D as for the fp32 tiles.
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
__device__ __forceinline__ i32x16 mfma_i32_32x32x32_i8(u32x4 a, u32x4 b, i32x16 c) {
  return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, b), c, 0, 0, 0);
}
// (a mod 2^24) * (b mod 2^24) mod 2^32: a full-rate multiply (the 32-bit one runs at a quarter of the rate)
__device__ __forceinline__ uint32_t mul_u24(uint32_t a, uint32_t b) { return __umul24(a, b); }

// byte `sel` (0..3) of `old` replaced by v converted to an unsigned 8-bit integer (v integral, 0 .. 255 here)
__device__ __forceinline__ uint32_t cvt_pk_u8_f32(float v, int sel, uint32_t old) {
  return __builtin_amdgcn_cvt_pk_u8_f32(v, (uint32_t)sel, old);
}

__device__ __forceinline__ f32x16 mfma_32x32x2_f32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// Transposing 64-bit LDS read of 16-bit elements; p is this lane's row address in LDS.
__device__ __forceinline__ u32x2 lds_read_tr16_b64(const uint16_t* p) {
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (s16x4 __attribute__((address_space(3)))*)(p));
  return __builtin_bit_cast(u32x2, v);
}

// Raw buffer resource over [base, base + 4 GiB): loads take a per-lane 32-bit byte offset plus a
// wave-uniform 32-bit byte offset, so the hot loops carry no 64-bit address arithmetic.
typedef __amdgpu_buffer_rsrc_t BufRsrc;
__device__ __forceinline__ BufRsrc make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
}
__device__ __forceinline__ u32x4 buffer_load_b128(BufRsrc r, uint32_t lane_off, uint32_t uniform_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, uniform_off, 0);
}
__device__ __forceinline__ uint32_t buffer_load_b32(BufRsrc r, uint32_t lane_off) {
  return __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, 0, 0);
}
// Resource over [base, base + bytes): an access at a byte offset >= bytes is out of range; out-of-range stores are
// dropped by the hardware, which makes a store conditional without a branch around it.
__device__ __forceinline__ BufRsrc make_rsrc_sized(void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)bytes, 0x00020000);
}
// 16-byte store with the non-temporal hint (the data is not read again by this launch)
__device__ __forceinline__ void buffer_store_b128_nt(BufRsrc r, u32x4 v, uint32_t lane_off) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_off, 0, 2);
}

// Nothing is scheduled across this point (the compiler otherwise re-orders a software pipeline to save registers).
__device__ __forceinline__ void sched_fence() { __builtin_amdgcn_sched_barrier(0); }

// the high halves of two words as one word: hi's in the upper half, lo's in the lower (one byte permute)
__device__ __forceinline__ uint32_t pack_high_halves(uint32_t hi, uint32_t lo) {
  return __builtin_amdgcn_perm(hi, lo, 0x07060302u);
}

// value held by the first active lane, as a scalar
__device__ __forceinline__ int wave_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

template <typename V>
__device__ __forceinline__ V wave_shfl_xor(V v, int mask) { return __shfl_xor(v, mask, 64); }
template <typename V>
__device__ __forceinline__ V wave_shfl(V v, int src) { return __shfl(v, src, 64); }
template <typename V>
__device__ __forceinline__ V wave_shfl_up(V v, int d) { return __shfl_up(v, d, 64); }
__device__ __forceinline__ uint64_t wave_ballot(bool p) { return __ballot(p); }
__device__ __forceinline__ int popc64(uint64_t v) { return __popcll(v); }
// Orders this wave's LDS accesses before the barrier against those after it.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Two fp32 -> packed bf16 (round to nearest even), one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// clamp(x, -r, r) for r >= 0 as one v_med3_f32 (a NaN input gives -r or r instead of NaN).
__device__ __forceinline__ float clamp_sym(float x, float r) { return __builtin_amdgcn_fmed3f(x, -r, r); }

// sin / cos of 2*pi*x (x in revolutions), natural log, sqrt: single hardware instructions.
__device__ __forceinline__ float fast_sin_rev(float x) { return __builtin_amdgcn_sinf(x); }
__device__ __forceinline__ float fast_cos_rev(float x) { return __builtin_amdgcn_cosf(x); }
// log2 of a normal positive number (no denormal handling)
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ uint32_t umulhi32(uint32_t a, uint32_t b) { return __umulhi(a, b); }

}  // namespace amoe
