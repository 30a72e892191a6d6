// Host stand-in for <hip/hip_runtime.h>: test infrastructure, never part of the library that ships.
//
// With this directory first on the include path, daemon.hip and runtime.hip compile as plain C++ for the host
// (clang++ -x c++), and the daemon kernel runs on the CPU: one OS thread per GPU thread, a pthread barrier per
// workgroup for __syncthreads() and one per wave for the cross-lane operations.  The point is not speed but
// what host tools can then see in the kernel's own code:
//   * every __syncthreads() records its source line, and a workgroup whose threads meet at barriers of different
//     lines is reported at once (on the GPU that is a workgroup out of step, which ends in a hang);
//   * ThreadSanitizer sees LDS as ordinary shared memory ordered by those barriers only, so a flag that one wave
//     rewrites before the others have read it is a reported data race;
//   * AddressSanitizer sees every global-memory access of the kernel (hipMalloc is malloc here);
//   * a watchdog prints where every thread of every workgroup is waiting when nothing moves any more.
// All atomics are sequentially consistent here and scopes are ignored: the emulation checks control flow, LDS
// discipline and addresses, not the GPU's memory model.
#pragma once

#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <atomic>
#include <functional>
#include <memory>
#include <mutex>
#include <vector>

// ---- language extensions
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define DFCCL_GLOBAL  // no address spaces on the host
#define DFCCL_EMUL 1

namespace emul {

constexpr int kWaveSize = 64;
constexpr int kLdsBytes = 160 * 1024;

struct Dim3 {
  unsigned x = 1, y = 1, z = 1;
  Dim3() {}
  Dim3(unsigned x_, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

struct Wave {
  pthread_barrier_t bar;
  uint64_t slot[kWaveSize];
};

// where a thread is, for the watchdog: > 0 waiting at the __syncthreads() of that line, 0 running,
// -1 returned from the kernel, < -1 waiting inside the cross-lane operation of line -value
struct Workgroup {
  pthread_barrier_t bar;
  int nThreads = 0;
  std::vector<Wave> waves;
  std::vector<int> lines[2];           // line of the barrier every thread is at, for even and odd barrier numbers
  std::vector<std::atomic<int>> where;
  alignas(256) unsigned char lds[kLdsBytes];
  size_t ldsUsed = 0;
};

struct ThreadCtx {
  Dim3 tIdx, bIdx, bDim, gDim;
  Workgroup* wg = nullptr;
  unsigned barriers = 0;  // __syncthreads() passed so far
};
extern thread_local ThreadCtx tls;

// progress counter of the watchdog: bumped by every barrier and cross-lane operation
extern std::atomic<uint64_t> gProgress;

void barrierMismatch(int tid, int line, int line0);

// EMUL_JITTER=<per mille>: after a barrier a thread sleeps for a random short time with that probability, so
// that waves leave barriers far apart, as they can on the GPU, and different interleavings get explored
extern int gJitterPerMille;
void jitterSleep();
inline void jitter() {
  if (gJitterPerMille > 0) jitterSleep();
}

inline void syncthreads(int line) {
  ThreadCtx& t = tls;
  Workgroup* wg = t.wg;
  const int tid = (int)t.tIdx.x;
  const unsigned k = t.barriers++ & 1u;
  wg->lines[k][tid] = line;
  wg->where[tid].store(line, std::memory_order_relaxed);
  pthread_barrier_wait(&wg->bar);
  wg->where[tid].store(0, std::memory_order_relaxed);
  gProgress.fetch_add(1, std::memory_order_relaxed);
  // slot k is written again two barriers from now, which nobody reaches before everybody has left this one
  // and arrived at the next
  const int line0 = wg->lines[k][0];
  if (line0 != line) barrierMismatch(tid, line, line0);
  jitter();
}

inline Wave& myWave() { return tls.wg->waves[tls.tIdx.x / kWaveSize]; }
inline int myLane() { return (int)(tls.tIdx.x % kWaveSize); }
inline void waveSync(int line) {
  ThreadCtx& t = tls;
  t.wg->where[t.tIdx.x].store(-line, std::memory_order_relaxed);
  pthread_barrier_wait(&myWave().bar);
  t.wg->where[t.tIdx.x].store(0, std::memory_order_relaxed);
}

// The cross-lane operations assume what the kernel guarantees: all 64 lanes of the wave call them together.
inline uint64_t ballot(bool p, int line) {
  Wave& w = myWave();
  w.slot[myLane()] = p ? 1u : 0u;
  waveSync(line);
  uint64_t m = 0;
  for (int i = 0; i < kWaveSize; i++) m |= (w.slot[i] & 1ull) << i;
  waveSync(line);
  gProgress.fetch_add(1, std::memory_order_relaxed);
  return m;
}
template <typename T>
inline T shflFrom(T v, int src, int line) {
  static_assert(sizeof(T) <= 8, "64-bit values at most");
  Wave& w = myWave();
  uint64_t bits = 0;
  memcpy(&bits, &v, sizeof(T));
  w.slot[myLane()] = bits;
  waveSync(line);
  const uint64_t r = w.slot[src & (kWaveSize - 1)];
  waveSync(line);
  T out;
  memcpy(&out, &r, sizeof(T));
  return out;
}

// A value the kernel declares to be the same in every lane of the wave (on the GPU it is moved to scalar
// registers with v_readfirstlane, and the wave then branches on it as one): here every lane compares its own
// value with lane 0's, and a lane that disagrees ends the run with both values and the source line.
void notUniform(int line, uint64_t mine, uint64_t first);
template <typename T>
inline T uniformChecked(T v, int line) {
  const T first = shflFrom(v, 0, line);
  uint64_t a = 0, b = 0;
  memcpy(&a, &v, sizeof(T));
  memcpy(&b, &first, sizeof(T));
  if (a != b) notUniform(line, a, b);
  return first;
}

void* wgSharedMem(size_t bytes);  // the workgroup's LDS block (the same address for all its threads)

struct Job;     // one kernel launch: its threads
struct Stream;  // launches in order
struct Event;

void launch(Stream* s, unsigned grid, unsigned block, std::function<void()> body);

}  // namespace emul

// lanes of a wave that talk to each other through LDS rely on running in lockstep: a barrier of the wave here
#define DFCCL_WAVE_LDS_SYNC() ::emul::waveSync(__LINE__)

#define DFCCL_WAVE_UNIFORM(x) ::emul::shflFrom((x), 0, __LINE__)
#define DFCCL_UNIFORM(x) ::emul::uniformChecked((x), __LINE__)
#define DFCCL_FRESH_PER_ROUND(v) ((void)0)  // (a hint for the GPU compiler's register allocation)

// EMUL_NEVER_LEAVE=1: the daemon's workgroups ignore every reason to leave (see DFCCL_TEST_NEVER_LEAVES in daemon.hip)
namespace emul { extern bool gNeverLeave; }
#define DFCCL_TEST_NEVER_LEAVES() (::emul::gNeverLeave)

// the one LDS object of the daemon kernel
#define DFCCL_WG_SHARED(T, name) T& name = *reinterpret_cast<T*>(::emul::wgSharedMem(sizeof(T)))

#define threadIdx (::emul::tls.tIdx)
#define blockIdx (::emul::tls.bIdx)
#define blockDim (::emul::tls.bDim)
#define gridDim (::emul::tls.gDim)
typedef ::emul::Dim3 dim3;

#define __syncthreads() ::emul::syncthreads(__LINE__)
#define __ballot(p) ::emul::ballot((p), __LINE__)
#define __shfl(v, src) ::emul::shflFrom((v), (src), __LINE__)
#define __shfl_xor(v, mask) ::emul::shflFrom((v), ::emul::myLane() ^ (mask), __LINE__)

// ---- compiler builtins of the target
#define __builtin_amdgcn_readfirstlane(x) (x)  // only ever applied to values that are the same in every lane
#define __builtin_amdgcn_readlane(x, srcLane) ::emul::shflFrom((x), (srcLane), __LINE__)
#define __builtin_amdgcn_fence(order, scope) __atomic_thread_fence(__ATOMIC_SEQ_CST)
#define __builtin_amdgcn_s_sleep(n) sched_yield()
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __HIP_MEMORY_SCOPE_SYSTEM 0
#define __hip_atomic_load(p, order, scope) __atomic_load_n((p), __ATOMIC_SEQ_CST)
#define __hip_atomic_store(p, v, order, scope) __atomic_store_n((p), (v), __ATOMIC_SEQ_CST)
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add((p), (v), __ATOMIC_SEQ_CST)

inline uint64_t wall_clock64() {  // 100 MHz
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (uint64_t)ts.tv_sec * 100000000ull + (uint64_t)ts.tv_nsec / 10u;
}
inline uint32_t __float_as_uint(float f) { return __builtin_bit_cast(uint32_t, f); }
inline float __uint_as_float(uint32_t u) { return __builtin_bit_cast(float, u); }

// ---- runtime API (the part the library and its native driver use)
typedef int hipError_t;
enum : int { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorNotReady = 600 };
typedef emul::Stream* hipStream_t;
typedef emul::Event* hipEvent_t;
typedef void* hipDeviceptr_t;
enum hipMemcpyKind { hipMemcpyHostToHost = 0, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum : unsigned { hipHostMallocCoherent = 1u, hipHostMallocMapped = 2u, hipStreamNonBlocking = 1u, hipEventBlockingSync = 1u,
                  hipEventDisableTiming = 2u };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 16 };

hipError_t hipMalloc(void** p, size_t bytes);
hipError_t hipFree(void* p);
hipError_t hipHostMalloc(void** p, size_t bytes, unsigned flags = 0);
hipError_t hipHostFree(void* p);
hipError_t hipMemset(void* p, int value, size_t bytes);
hipError_t hipMemsetD8(hipDeviceptr_t p, unsigned char value, size_t count);
hipError_t hipMemsetD16(hipDeviceptr_t p, unsigned short value, size_t count);
hipError_t hipMemsetD32(hipDeviceptr_t p, int value, size_t count);
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind);
hipError_t hipSetDevice(int device);
hipError_t hipGetDevice(int* device);
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t attr, int device);
hipError_t hipGetLastError();
const char* hipGetErrorString(hipError_t e);
hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned flags);
hipError_t hipStreamDestroy(hipStream_t s);
hipError_t hipStreamSynchronize(hipStream_t s);
hipError_t hipDeviceSynchronize();
hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned flags);
hipError_t hipEventDestroy(hipEvent_t e);
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s);
hipError_t hipEventSynchronize(hipEvent_t e);

template <typename K>
inline hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int* n, K, int, size_t) {
  *n = 1;
  return hipSuccess;
}

template <typename K, typename... Args>
inline void hipLaunchKernelGGL(K kernel, dim3 grid, dim3 block, size_t, hipStream_t stream, Args... args) {
  emul::launch(stream, grid.x, block.x, [=]() { kernel(args...); });
}
