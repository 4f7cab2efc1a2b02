// CPU stand-in for <hip/hip_runtime.h>, used ONLY by the host-compiled test build of the
// kernels (tests/emu).  One std::thread per GPU thread, blocks run one after another, so the
// kernels' own index arithmetic, masking and LDS traffic run unchanged under the host
// AddressSanitizer.  Nothing in the shipped library includes this file.
#pragma once
#include <atomic>
#include <barrier>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <sched.h>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct EmuIdx { unsigned x = 0, y = 0, z = 0; };
inline thread_local EmuIdx threadIdx, blockIdx, blockDim, gridDim;

typedef int hipError_t;
typedef void* hipStream_t;
enum { hipSuccess = 0 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emu"; }
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 0 };
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
// a "device" array is ordinary host memory here, and its address is the symbol's own
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))
template <class T> inline hipError_t hipGetSymbolAddress(void** p, T* sym) { *p = (void*)sym; return hipSuccess; }
// a 3-CU device: the persistent kernels then run few workgroups with several work items each
inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 3; return hipSuccess; }

// Barrier for heavily oversubscribed threads (256 per workgroup on a few cores): waiters give up the core instead of
// sleeping on a futex, which costs two system calls and a wake-up per thread and barrier.
struct EmuBarrier {
  explicit EmuBarrier(int n_) : n(n_) {}
  void arrive_and_wait() {
    const unsigned g = gen.load(std::memory_order_acquire);
    if (count.fetch_add(1, std::memory_order_acq_rel) + 1 == n) {
      count.store(0, std::memory_order_relaxed);
      gen.fetch_add(1, std::memory_order_release);
    } else {
      while (gen.load(std::memory_order_acquire) == g) sched_yield();
    }
  }
  const int n;
  std::atomic<int> count{0};
  std::atomic<unsigned> gen{0};
};

struct EmuWave {
  EmuBarrier bar{64};
  alignas(64) unsigned char slot[64][64];
  const void* ptr[64];
};
struct EmuBlock {
  EmuBarrier* bar;
};
inline thread_local EmuWave* emu_wave = nullptr;
inline thread_local EmuBlock* emu_block = nullptr;

inline void __syncthreads() { emu_block->bar->arrive_and_wait(); }

template <class T> inline T atomicAdd(T* p, T v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
inline float atomicAdd(float* p, float v) {
  std::atomic_ref<float> r(*p);
  float old = r.load();
  while (!r.compare_exchange_weak(old, old + v)) {}
  return old;
}
inline void __threadfence() { __atomic_thread_fence(__ATOMIC_SEQ_CST); }
template <class T> inline T atomicOr(T* p, T v) { return __atomic_fetch_or(p, v, __ATOMIC_RELAXED); }
template <class T> inline T atomicMax(T* p, T v) {
  T old = __atomic_load_n(p, __ATOMIC_RELAXED);
  while (old < v && !__atomic_compare_exchange_n(p, &old, v, true, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {}
  return old;
}

template <class K, class... A>
inline void emu_launch(K kernel, dim3 grid, dim3 block, A... args) {
  const unsigned nthreads = block.x;
  assert(nthreads % 64 == 0 && block.y == 1 && block.z == 1);
  for (unsigned bz = 0; bz < grid.z; bz++)
  for (unsigned by = 0; by < grid.y; by++)
  for (unsigned bx = 0; bx < grid.x; bx++) {
    EmuBarrier bar((int)nthreads);
    EmuBlock blk{&bar};
    std::unique_ptr<EmuWave[]> waves(new EmuWave[nthreads / 64]);
    std::vector<std::thread> th;
    th.reserve(nthreads);
    for (unsigned t = 0; t < nthreads; t++) {
      th.emplace_back([&, t]() {
        threadIdx.x = t;
        blockIdx.x = bx; blockIdx.y = by; blockIdx.z = bz;
        blockDim.x = nthreads; blockDim.y = blockDim.z = 1;
        gridDim.x = grid.x; gridDim.y = grid.y; gridDim.z = grid.z;
        emu_wave = &waves[t / 64];
        emu_block = &blk;
        kernel(args...);
      });
    }
    for (auto& x : th) x.join();
  }
}
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) emu_launch(kernel, grid, block, __VA_ARGS__)
