// Expert sort of the CVMM path: stable counting sort of expert ids with wavefront ballots.
//   pass 1  per-wave histograms of 1024-element units (LDS atomics)
//   pass 2  a wave per expert scans its unit counts (bases in place), then one workgroup scans
//           the per-expert totals -> offsets[E+1]
//   pass 3  per wave: rank every element among equal keys of its 64-lane batch with a
//           match-any built from ballots over the key bits, add the running per-key base kept
//           in LDS, scatter (sorted id, flat index, flat index / k)
// (small tables: passes 2 and 3 are one launch, sel_scan_scatter_kernel)
// Stable by construction: batches, units and lanes are all visited in ascending flat index.
#pragma once
#include "common.h"

namespace amoe {

constexpr int kSelUnitMax = 1024;   // elements per wave: 64 .. 1024, fewer for short inputs so that
                                    // the sort still spreads over the chip (see sel_unit)
__host__ __device__ inline int sel_unit(long long M) {
  int u = 64;
  while (u < kSelUnitMax && M / u > 2048) u <<= 1;   // aim at <= 2048 units
  return u < 256 ? 256 : u;
}

struct SelParams {
  const void* sel; int sel_is_i64;
  long long M; int E, k, n_units, key_bits, unit;
  int32_t* sel_sorted; int32_t* perm; int32_t* in_index; int32_t* offsets; int32_t* bad_flag;
  int32_t* unit_hist;               // workspace [n_units][E]
};

__device__ __forceinline__ int sel_key(const SelParams& p, long long i, bool& bad) {
  long long v = p.sel_is_i64 ? static_cast<const long long*>(p.sel)[i]
                             : (long long)static_cast<const int32_t*>(p.sel)[i];
  bad = v < 0 || v >= p.E;
  if (v < 0) v = 0;                      // out-of-range ids are flagged and clamped
  if (v >= p.E) v = p.E - 1;
  return (int)v;
}

__global__ __launch_bounds__(kThreads) void sel_hist_kernel(const SelParams p) {
  __shared__ int hist[4 * kSelMaxExperts];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 4 * p.E; i += kThreads) hist[i] = 0;
  __syncthreads();
  const int unit = blockIdx.x * 4 + wave;
  bool any_bad = false;
  if (unit < p.n_units) {
    for (int it = 0; it < p.unit / 64; it++) {
      const long long i = (long long)unit * p.unit + it * 64 + lane;
      if (i < p.M) {
        bool bad;
        const int key = sel_key(p, i, bad);
        any_bad |= bad;
        atomicAdd(&hist[wave * p.E + key], 1);
      }
    }
  }
  if (any_bad && p.bad_flag != nullptr) atomicOr(p.bad_flag, 1);
  __syncthreads();
  for (int w = 0; w < 4; w++) {
    const int u = blockIdx.x * 4 + w;
    if (u < p.n_units)
      for (int e = tid; e < p.E; e += kThreads) p.unit_hist[(long long)u * p.E + e] = hist[w * p.E + e];
  }
}

// pass 2a: one wave per expert turns its column of unit counts into unit bases relative to the
// expert's segment start and writes the expert's total to offsets[e + 1].
__global__ __launch_bounds__(kThreads) void sel_unit_scan_kernel(const SelParams p) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= p.E) return;
  int carry = 0;
  for (int u0 = 0; u0 < p.n_units; u0 += 64) {
    const int u = u0 + lane;
    const int c = u < p.n_units ? p.unit_hist[(long long)u * p.E + e] : 0;
    int incl = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = wave_shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (u < p.n_units) p.unit_hist[(long long)u * p.E + e] = carry + incl - c;
    carry += wave_shfl(incl, 63);
  }
  if (lane == 0) p.offsets[e + 1] = carry;
}

// pass 2b: one workgroup turns the per-expert totals (in offsets[1..E]) into offsets[0..E].
__global__ __launch_bounds__(kThreads) void sel_offsets_kernel(const SelParams p) {
  constexpr int kPer = kSelMaxExperts / kThreads;
  __shared__ int wave_sums[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e0 = tid * kPer;
  int c[kPer];
  int mine = 0;
#pragma unroll
  for (int j = 0; j < kPer; j++) {
    c[j] = e0 + j < p.E ? p.offsets[e0 + j + 1] : 0;
    mine += c[j];
  }
  int incl = mine;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = wave_shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();                     // also orders every read of the totals before the writes below
  int run = incl - mine;
  for (int w = 0; w < wave; w++) run += wave_sums[w];
#pragma unroll
  for (int j = 0; j < kPer; j++) {
    if (e0 + j < p.E) p.offsets[e0 + j] = run;
    run += c[j];
  }
  if (tid == 0) p.offsets[p.E] = (int)p.M;
}

__global__ __launch_bounds__(kThreads) void sel_scatter_kernel(const SelParams p) {
  __shared__ int base[4 * kSelMaxExperts];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int w = 0; w < 4; w++) {
    const int u = blockIdx.x * 4 + w;
    if (u < p.n_units)
      for (int e = tid; e < p.E; e += kThreads) base[w * p.E + e] = p.offsets[e] + p.unit_hist[(long long)u * p.E + e];
  }
  __syncthreads();
  const int unit = blockIdx.x * 4 + wave;
  int* my_base = &base[wave * p.E];
  const uint64_t lt_mask = ((uint64_t)1 << lane) - 1;
  for (int it = 0; it < p.unit / 64; it++) {
    const long long i = (long long)unit * p.unit + it * 64 + lane;
    const bool valid = unit < p.n_units && i < p.M;
    bool bad;
    const int key = valid ? sel_key(p, i, bad) : 0;
    uint64_t same = wave_ballot(valid);
    for (int b = 0; b < p.key_bits; b++) {
      const bool bit = (key >> b) & 1;
      const uint64_t bal = wave_ballot(valid && bit);
      same &= bit ? bal : ~bal;
    }
    const int rank = popc64(same & lt_mask);
    const int count = popc64(same);
    int pos = 0;
    if (valid) pos = my_base[key] + rank;
    wave_sync();
    if (valid && rank == 0) my_base[key] += count;
    wave_sync();
    if (valid) {
      p.sel_sorted[pos] = key;
      p.perm[pos] = (int)i;
      p.in_index[pos] = (int)(i / p.k);
    }
  }
}

// Passes 2 and 3 in one launch, for tables small enough that every workgroup can afford to read all of it
// (n_units * E <= kSelFuseMax counts, E <= kThreads): each workgroup sums the whole table of unit counts itself --
// per expert: the total, and the part that belongs to the units before its own four -- scans the totals into the
// experts' segment starts, and scatters its units as sel_scatter_kernel does.  Workgroup 0 also writes offsets.
// Two launches and no pass over the table in between: the sort is on the path to the first GEMM of every step.
constexpr int kSelFuseMax = 32768;
__global__ __launch_bounds__(kThreads) void sel_scan_scatter_kernel(const SelParams p) {
  __shared__ int base[4 * kThreads];          // [wave][expert]: where the next element of that expert goes
  __shared__ __attribute__((aligned(16))) int part_total[4 * kThreads], part_before[4 * kThreads];
  __shared__ int wave_sums[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int E = p.E;
  const int first_unit = blockIdx.x * 4;
  // per expert: the total over all units and the part before this workgroup's first unit.  The table is read in rows
  // (one unit's counts), several rows per pass of the workgroup, four experts per thread where E allows it.
  int my_total = 0, my_before = 0;                  // thread e < E: the expert's two sums
  if ((E & 3) == 0) {
    typedef __attribute__((ext_vector_type(4))) int i32x4v;
    const int tpr = E >> 2;                         // threads per row (<= 64)
    const int rpp = kThreads / tpr;                 // rows per pass
    const int c4 = tid % tpr, row = tid / tpr;
    i32x4v tot = {0, 0, 0, 0}, bef = {0, 0, 0, 0};
    if (row < rpp) {
      for (int u = row; u < p.n_units; u += rpp) {
        const i32x4v c = *reinterpret_cast<const i32x4v*>(p.unit_hist + (long long)u * E + 4 * c4);
        tot += c;
        if (u < first_unit) bef += c;
      }
      *reinterpret_cast<i32x4v*>(&part_total[row * E + 4 * c4]) = tot;
      *reinterpret_cast<i32x4v*>(&part_before[row * E + 4 * c4]) = bef;
    }
    __syncthreads();
    if (tid < E)
      for (int r = 0; r < rpp; r++) {
        my_total += part_total[r * E + tid];
        my_before += part_before[r * E + tid];
      }
  } else {
    int epad = 1;
    while (epad < E) epad <<= 1;
    const int groups = kThreads / epad;
    const int e = tid & (epad - 1), grp = tid / epad;
    int total = 0, before = 0;
    if (e < E) {
      for (int u = grp; u < p.n_units; u += groups) {
        const int c = p.unit_hist[(long long)u * E + e];
        total += c;
        before += u < first_unit ? c : 0;
      }
    }
    part_total[tid] = total;
    part_before[tid] = before;
    __syncthreads();
    if (tid < E)
      for (int g = 0; g < groups; g++) {
        my_total += part_total[g * epad + tid];
        my_before += part_before[g * epad + tid];
      }
  }
  // exclusive scan of the totals over the experts (thread = expert)
  int incl = my_total;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = wave_shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();
  int start = incl - my_total;
  for (int w = 0; w < wave; w++) start += wave_sums[w];
  if (tid < E) {
    if (blockIdx.x == 0) {
      p.offsets[tid] = start;
      if (tid == E - 1) p.offsets[E] = (int)p.M;
    }
    int run = start + my_before;
    for (int w = 0; w < 4; w++) {
      base[w * kThreads + tid] = run;
      const int u = first_unit + w;
      if (u < p.n_units) run += p.unit_hist[(long long)u * E + tid];
    }
  }
  __syncthreads();
  const int unit = first_unit + wave;
  int* my_base = &base[wave * kThreads];
  const uint64_t lt_mask = ((uint64_t)1 << lane) - 1;
  for (int it = 0; it < p.unit / 64; it++) {
    const long long i = (long long)unit * p.unit + it * 64 + lane;
    const bool valid = unit < p.n_units && i < p.M;
    bool bad;
    const int key = valid ? sel_key(p, i, bad) : 0;
    uint64_t same = wave_ballot(valid);
    for (int b = 0; b < p.key_bits; b++) {
      const bool bit = (key >> b) & 1;
      const uint64_t bal = wave_ballot(valid && bit);
      same &= bit ? bal : ~bal;
    }
    const int rank = popc64(same & lt_mask);
    const int count = popc64(same);
    int pos = 0;
    if (valid) pos = my_base[key] + rank;
    wave_sync();
    if (valid && rank == 0) my_base[key] += count;
    wave_sync();
    if (valid) {
      p.sel_sorted[pos] = key;
      p.perm[pos] = (int)i;
      p.in_index[pos] = (int)(i / p.k);
    }
  }
}

// offsets[E+1] from sorted ids: position i owns every expert in (sel[i-1], sel[i]].
__global__ __launch_bounds__(kThreads) void offsets_from_sorted_kernel(const int32_t* __restrict__ sel,
                                                                        long long M, int E,
                                                                        int32_t* __restrict__ offsets) {
  const long long i = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (i > M) return;
  const int prev = (i == 0) ? -1 : sel[i - 1];
  int cur = (i == M) ? E : sel[i];
  if (cur > E) cur = E;
  for (int e = prev + 1; e <= cur; e++)
    if (e >= 0) offsets[e] = (int)i;
}

}  // namespace amoe
