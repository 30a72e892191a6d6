// The persistent daemon kernel of the DFCCL data path for gfx950.
//
// One launch serves every virtual rank of a device: workgroup (slot, channel)
// is channel `channel` of the rank context in slot `slot`.  Each workgroup runs
// the scheduler of the reference's daemonKernel
// (src/collectives_ofccl/device/enqueue_ofccl_dev.cu:1026-1483) on its own:
//
//   poll submissions -> append to the task queue -> find the collectives that can
//   move -> visit them: load the context, run steps until the collective is done
//   or a bounded wait expires, save the context (preemption) or post the
//   completion -> repeat; leave after a long idle period, or when told to.
//
// What is shaped by the hardware rather than by the reference:
//  * only the rank's leader workgroup (channel 0) reads the host-coherent
//    submission ring; one wave fetches up to 15 entries per poll (four lanes per
//    entry, each word validated by its own tag) and mirrors them into an HBM ring
//    the other channels read, so PCIe sees one poller per rank;
//  * every blocking point is a WaitDesc ("these counters have reached this
//    value"); wave 0 evaluates it with one lane per counter and a ballot, and the
//    same descriptor, saved with the context, lets the scheduler test 64 parked
//    collectives per wave instruction instead of loading and spinning on each;
//  * two data protocols: the reference's FIFO ring (slices staged through HBM
//    FIFOs between neighbours) and a direct protocol in which the virtual ranks,
//    whose buffers share one HBM, read each other's send buffers and write each
//    other's receive buffers in place, keeping the ring's accumulation order;
//    its buffers are announced when a submission is ingested, so ranks never
//    wait for each other before the data has moved;
//  * an idle leader keeps several polls of the host ring in flight, and a small
//    collective (one tile of a few KiB) is run by wave 0 alone, without a single
//    workgroup barrier between its waits and its data movement;
//  * completions go to a host-coherent ring with a device-side ticket, no
//    compare-and-swap over PCIe;
//  * the collective's plan and resumable position live in LDS while it runs.
#include <hip/hip_runtime.h>

#include "dfccl_common.h"
#include "reduce_copy_wg.h"

// This file is compiled twice: as it is (the kernel that normally runs), and with DFCCL_TRACED_BUILD defined, which
// adds the timeline stamps and gives the kernel and its launcher names of their own; the runtime launches the
// traced kernel when DFCCL_TRACE=1 asks for a timeline.
#ifdef DFCCL_TRACED_BUILD
#define DFCCL_DAEMON_KERNEL dfcclDaemonKernelTraced
#define DFCCL_DAEMON_LAUNCH dfcclLaunchDaemonTraced
#define DFCCL_DAEMON_OCCUPANCY dfcclDaemonOccupancyTraced
#else
#define DFCCL_DAEMON_KERNEL dfcclDaemonKernel
#define DFCCL_DAEMON_LAUNCH dfcclLaunchDaemon
#define DFCCL_DAEMON_OCCUPANCY dfcclDaemonOccupancy
#endif

namespace dfccl {

#ifdef DFCCL_TRACED_BUILD
constexpr bool kTracedBuild = true;
#else
constexpr bool kTracedBuild = false;
#endif

// Rows (of one 128-bit access per thread) the FIFO movers keep in flight per thread and source.  A daemon
// workgroup has its compute unit to itself and a FIFO step reads at most two sources, so one row would leave
// 16 KiB in flight per compute unit, half of what the one-shot reduce-copy kernel keeps there with its two
// workgroups; two rows match it.  The movers of scaled sums keep one row (their integer divisions need the
// registers), and the kernel's register count is bounded by a test of the compiler's resource remarks.
constexpr int kFifoUnroll = 2;
constexpr int kFifoUnrollScaled = 1;
constexpr int kReadyWords = (kMaxColls + 63) / 64;
constexpr int kSoftWaitSpins = 2;       // polls of a wait of the direct protocol while other collectives are queued
constexpr int kSoloMaxBytes = 4096;  // largest own chunk of a one-tile collective that wave 0 runs by itself (see runDirect)
constexpr int kIdleRounds = 8;  // x 4 polls of the host ring before an idle leader goes round its main loop again
enum RunStatus : int { kRunDone = 0, kRunPreempted = 1 };

// Geometry of the direct all-reduce sweeps: loop l covers elements [l * loop, (l + 1) * loop), split into
// nChannels * n chunks of `real` elements; every loop but the last uses the nominal chunk.
struct SweepGeom {
  int64_t count, loop, chunkElems, lastReal, L;
  int64_t T;                         // tiles (one rank's chunk of one channel slot of one loop) per rank: L * C
  uint64_t instBase;                 // value of the rank's tile counter when this instance began
  uint64_t ctr;                      // the rank's tile counter
  int n, C, ch, es;                  // n: sources folded (1 = plain copy)
  int me, dtype, op, nd;             // nd: destinations written
  int tn, tme, scaleKind, pad1;      // a loop holds C * tn chunks, mine is number tme of every channel slot
  uint64_t scaleBits;                // scaled sums (see Scale in reduce_ops.h): the divisor of kScalePost
  uint64_t src[kMaxDirectRanks];     // the send buffers in fold order: in[me + 1], in[me + 2], ..., in[me]
  uint64_t dst[kMaxDirectRanks];     // every rank's receive buffer
};
// Scheduler state that only wave 0 uses, kept in registers: every lane of wave 0 holds the same values (they come
// from ballots and from loads that all lanes make of one address) and applies the same updates to them, so none
// of it goes through LDS, where every step of one lane's bookkeeping was a round trip of its own.  (The other
// waves carry a copy that nobody looks at.)
struct Wave0Regs {
  uint64_t frontier;       // next submission ticket this workgroup reads from the mirror ring
  uint64_t hostFrontier;   // leader: next ticket to fetch from the host ring (== mirror tail)
  uint64_t publishedHead;  // leader: last value written to the host's head word
  int64_t idle;            // consecutive rounds without work or progress
  uint32_t round;          // scheduler rounds since launch
  uint32_t statsReqSeen;   // leader: last request number passed on to the other workgroups
  int32_t numActive;       // this round's copy of the task queue's length (LDS holds it for the other waves)
  int32_t ingested;        // entries taken from the submission queue this round
  int32_t allFresh;        // every collective of the task queue was ingested this round (nothing is parked)
  int32_t rankBusy;        // leader: other channels of the rank still have work in flight
  int32_t finalQuit;       // a quit entry has been read
  int32_t numReady;        // collectives that can move this round
};

struct WgShared {
  // scheduler state the waves share
  int32_t numActive;
  int32_t numReady;
  int32_t exitKind;
  int32_t progressedRound;
  int32_t loadedColl;      // collective whose plan and position are in LDS, -1: none
  uint32_t statsEpoch;     // last request for the counters this workgroup has answered
  uint32_t traceCount;
  uint32_t wgIndex;
  uint64_t cqNext;         // single-channel ranks: next completion ticket
  Wave0Regs w0;            // wave 0's registers, set aside while the workgroup moves data (see the run phase)
  // collective being run
  int32_t waitOk;
  int32_t progressed;
  int32_t peersLoaded;
  int32_t released;        // the results of this visit are already visible to the system
  int64_t threshold;
  CollPlan plan;
  DynCtx dyn;
  WgStats stats;
  SweepGeom sweep;         // arguments of the direct protocol's sweeps
  uint64_t sweepScale[kMaxDirectRanks];  // pre-multiplied sums: the scalar that belongs to sweep.src[t] (see runDirect)
  uint64_t ticket[2];      // tile numbers handed from thread 0 to the workgroup (two slots, used alternately)
  uint64_t ready[kReadyWords];
  uint64_t readySolo[kReadyWords];  // those of `ready` that wave 0 runs alone (see visit)
  uint16_t taskq[kMaxColls];
  // of every collective of this rank (from the plans, at launch): its channels in the low bits, kCollSolo if
  // wave 0 runs it alone
  uint8_t collChannels[kMaxColls];
};
constexpr uint8_t kCollSolo = 0x80;
static_assert(kMaxChannels < kCollSolo, "the channel count shares a byte with the flag");

// the workgroup's one LDS object (a host build that emulates workgroups with threads supplies its own definition)
#ifndef DFCCL_WG_SHARED
#define DFCCL_WG_SHARED(T, name) __shared__ T name
#endif

// Marks the places where the lanes of one wave hand values to each other through LDS (one lane writes, the
// others read afterwards, or the other way round).  The hardware runs the lanes of a wave in lockstep and its LDS
// accesses in order, but the compiler knows nothing of that: to it the lanes are independent threads without
// synchronisation, and it has been seen to place the other lanes' read of a flag before the branch in which
// lane 0 writes it (so that lane 0 saw a failed wait and the other 63 lanes a successful one).  The barrier of
// the wave is a convergent operation: every lane's earlier accesses stay before it and every later access after
// it, and it is not moved into either side of a branch.  It costs no instruction.  (A host build that runs
// every lane as a thread makes it a real barrier of the wave.)
#ifndef DFCCL_WAVE_LDS_SYNC
#define DFCCL_WAVE_LDS_SYNC()                               \
  do {                                                      \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  \
    __builtin_amdgcn_wave_barrier();                        \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");  \
  } while (0)
#endif
// A value that has to be the same in every lane of the wave because the wave branches on it: scheduler state
// that all lanes load from one address in LDS or global memory.  Every lane takes the first lane's copy
// (v_readfirstlane: the value lives in scalar registers from there on and the branch is a scalar one), so the
// lanes of a wave cannot disagree about the way to go, whatever order their loads were performed in.
#ifndef DFCCL_WAVE_UNIFORM
__device__ __forceinline__ uint32_t waveUniform(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ int32_t waveUniform(int32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t waveUniform(uint64_t v) {
  return (uint64_t)waveUniform((uint32_t)v) | ((uint64_t)waveUniform((uint32_t)(v >> 32)) << 32);
}
__device__ __forceinline__ int64_t waveUniform(int64_t v) { return (int64_t)waveUniform((uint64_t)v); }
template <typename T>
__device__ __forceinline__ T* waveUniform(T* p) {
  return (T*)(uintptr_t)waveUniform((uint64_t)(uintptr_t)p);
}
#define DFCCL_WAVE_UNIFORM(x) ::dfccl::waveUniform(x)
#endif
// A value that IS the same in every lane of the wave by construction: read from LDS after a barrier of the
// workgroup, or computed from such values.  Everything read from LDS arrives in vector registers, and the
// compiler cannot know that all lanes hold the same: it would keep the whole state of the scheduler and of the
// running collective (dozens of counters, sizes and pointers) once per lane, and treat every branch on them as
// divergent.  Taking lane 0's copy tells it: the value lives in scalar registers from there on (64 of them fit
// one vector register when they have to be set aside), and the branch is a scalar one.  Only at places that
// all lanes of the wave reach together.  (A host build that runs every lane as a thread checks that the lanes do
// hold the same value.)
#ifndef DFCCL_UNIFORM
#define DFCCL_UNIFORM(x) ::dfccl::waveUniform(x)
#endif

// The scheduler is one endless loop with all of the data movement inlined into it.  Left alone, the compiler
// moves everything that does not change from round to round out of that loop: every expression in the thread
// number (lane masks, byte offsets of the thread's packs, comparisons of the lane with constants, for each of
// the inlined movers) is computed once at the kernel's entry and then kept in registers for the kernel's whole
// life, dozens of vector registers and as many scalar pairs that are live across everything.  Passing the
// thread number through an empty asm statement at the head of every round makes it a new value per round as far
// as the compiler can tell, so those expressions are computed where they are used and die there.
#ifndef DFCCL_FRESH_PER_ROUND
#define DFCCL_FRESH_PER_ROUND(v) asm volatile("" : "+v"(v))
#endif

// Test hook of the host build: a workgroup that never leaves (it ignores the host's requests, quit entries and
// the idle limit while it keeps running through its own bounded waits), to exercise the host's handling of a
// kernel that stays resident.  Nothing on the GPU.
#ifndef DFCCL_TEST_NEVER_LEAVES
#define DFCCL_TEST_NEVER_LEAVES() false
#endif

#define DFCCL_AGENT __HIP_MEMORY_SCOPE_AGENT
#define DFCCL_SYSTEM __HIP_MEMORY_SCOPE_SYSTEM

// Everything the daemon touches outside LDS is global memory.  Pointers that were loaded from memory have the
// generic address space as far as the compiler can tell, and accesses through them would be flat instructions
// (slower, and they stop the compiler from keeping several loads in flight); these helpers say what they are.
template <typename T>
__device__ __forceinline__ DFCCL_GLOBAL T* G(T* p) {
  return (DFCCL_GLOBAL T*)p;
}
template <typename T>
__device__ __forceinline__ void loadStruct(T& dst, const T* src) {
  static_assert(sizeof(T) % 8 == 0, "copied in 64-bit words");
  const DFCCL_GLOBAL uint64_t* s = (const DFCCL_GLOBAL uint64_t*)src;
  uint64_t* d = (uint64_t*)&dst;
#pragma unroll
  for (unsigned i = 0; i < sizeof(T) / 8; i++) d[i] = s[i];
}
template <typename T>
__device__ __forceinline__ void storeStruct(T* dst, const T& src) {
  static_assert(sizeof(T) % 8 == 0, "copied in 64-bit words");
  DFCCL_GLOBAL uint64_t* d = (DFCCL_GLOBAL uint64_t*)dst;
  const uint64_t* s = (const uint64_t*)&src;
#pragma unroll
  for (unsigned i = 0; i < sizeof(T) / 8; i++) d[i] = s[i];
}

// The value lane `srcLane` of the wave holds (srcLane is the same in every lane): a register read, no LDS.
__device__ __forceinline__ uint64_t readLane64(uint64_t v, int srcLane) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, srcLane);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), srcLane);
  return (uint64_t)lo | ((uint64_t)hi << 32);
}

// A 64-bit value that is the same in every lane, into scalar registers (the first lane's copy).
__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (uint64_t)lo | ((uint64_t)hi << 32);
}

__device__ __forceinline__ uint64_t waveMin64(uint64_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    uint64_t other = __shfl_xor(v, o);
    v = other < v ? other : v;
  }
  return v;
}

__device__ __forceinline__ WaitDesc noWait() {
  WaitDesc w;
  w.ptr = 0;
  w.value = 0;
  w.stride = 0;
  w.count = 0;
  return w;
}
__device__ __forceinline__ WaitDesc waitFor(const void* ptr, uint64_t value, int stride, int count) {
  WaitDesc w;
  w.ptr = (uint64_t)(uintptr_t)ptr;
  w.value = value;
  w.stride = stride;
  w.count = count;
  return w;
}

// The scalar of a PreMulSum operator that lives in device memory: one element of `es` bytes, read afresh
// (the caller may have written it with a copy or a kernel since the previous instance).
__device__ __forceinline__ uint64_t loadScalar(const void* p, int es) {
  switch (es) {
    case 1: return __hip_atomic_load((const DFCCL_GLOBAL uint8_t*)p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    case 2: return __hip_atomic_load((const DFCCL_GLOBAL uint16_t*)p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    case 4: return __hip_atomic_load((const DFCCL_GLOBAL uint32_t*)p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    default: return __hip_atomic_load((const DFCCL_GLOBAL uint64_t*)p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  }
}

// One thread: tell the peers where this rank's buffers of instance `inst` of a direct collective are.  The two
// words carry their own instance tag, so no ordering between them is needed, and the buffers' contents were
// made visible by whoever wrote them before the submission.  A scalar in device memory (scalePtr) is read now
// and handed over with the buffers: it has to be visible to whoever sees the tags, hence the release.
__device__ __forceinline__ void publishBuffers(PeerPub* myPub, uint64_t sendbuff, uint64_t recvbuff, uint64_t inst,
                                               const void* scalePtr, int elemSize) {
  const uint64_t tag = pubTag(inst);
  if (scalePtr != nullptr) {
    __hip_atomic_store(G(&myPub->scale), loadScalar(scalePtr, elemSize), __ATOMIC_RELAXED, DFCCL_AGENT);
    __hip_atomic_store(G(&myPub->send), sendbuff | tag, __ATOMIC_RELEASE, DFCCL_AGENT);
    __hip_atomic_store(G(&myPub->recv), recvbuff | tag, __ATOMIC_RELEASE, DFCCL_AGENT);
  } else {
    __hip_atomic_store(G(&myPub->send), sendbuff | tag, __ATOMIC_RELAXED, DFCCL_AGENT);
    __hip_atomic_store(G(&myPub->recv), recvbuff | tag, __ATOMIC_RELAXED, DFCCL_AGENT);
  }
}

// One record of the optional timeline (one thread per workgroup calls this).  The stamps are only compiled into
// the traced build of this file (see kTracedBuild): the kernel that runs otherwise carries none of it.
__device__ __forceinline__ void trace(const DaemonArgs& A, WgShared& sh, uint32_t ev, uint32_t arg) {
  if constexpr (!kTracedBuild) return;
  if (A.trace == nullptr) return;
  const uint32_t i = sh.traceCount++;
  DFCCL_GLOBAL uint64_t* rec = G(A.trace) + ((size_t)sh.wgIndex * kTraceRecords + (i % kTraceRecords)) * 2;
  rec[0] = (uint64_t)ev | ((uint64_t)arg << 32);
  rec[1] = wall_clock64();
}

// Writes the workgroup's counters to host-coherent memory (thread 0), marked as the answer to request `epoch`.
__device__ __forceinline__ void flushStats(const RankDev& R, WgShared& sh, int ch, uint32_t epoch) {
  DFCCL_GLOBAL WgStats* out = G(&R.stats[ch]);
  __hip_atomic_store(&out->sqesRead, sh.stats.sqesRead, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->cqesWritten, sh.stats.cqesWritten, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->ctxSaves, sh.stats.ctxSaves, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->ctxLoads, sh.stats.ctxLoads, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->voluntaryQuits, sh.stats.voluntaryQuits, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->forcedQuits, sh.stats.forcedQuits, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->slicesMoved, sh.stats.slicesMoved, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->spins, sh.stats.spins, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->epoch, (uint64_t)epoch, __ATOMIC_RELEASE, DFCCL_SYSTEM);
}

// One thread: what the head of the task queue is parked on, for the host's diagnosis (see WgStats::stuck).
__device__ __forceinline__ void reportStuck(const RankDev& R, WgShared& sh, int ch) {
  DFCCL_GLOBAL WgStats* out = G(&R.stats[ch]);
  const uint32_t coll = sh.taskq[0];
  if (coll >= (uint32_t)R.nColls) return;
  DynCtx d;
  if ((int32_t)coll == sh.loadedColl) {
    d = sh.dyn;
  } else {
    loadStruct(d, &R.dyn[(size_t)ch * R.nColls + coll]);
  }
  uint64_t seen = 0;
  if ((d.wait[0].count & (kWaitTagged - 1)) > 0)
    seen = __hip_atomic_load((const DFCCL_GLOBAL uint64_t*)(uintptr_t)d.wait[0].ptr, __ATOMIC_RELAXED, DFCCL_AGENT);
  const uint64_t n = __hip_atomic_load(&out->stuck[0], __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[1],
                     (uint64_t)coll | ((uint64_t)(uint8_t)d.step << 32) | ((uint64_t)(uint8_t)d.slice << 40) |
                         ((uint64_t)(uint16_t)sh.numActive << 48),
                     __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[2], d.instance, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[3], d.wait[0].ptr, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[4], (d.wait[0].value & 0xffffffffffffull) | ((uint64_t)(uint16_t)d.wait[0].count << 48),
                     __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[5], seen, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[6], d.wait[1].ptr, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->stuck[0], n + 1, __ATOMIC_RELEASE, DFCCL_SYSTEM);
}

// Wave 0: append the entries held one per lane (lanes < avail) to the task queue if this channel takes part
// in them; a quit entry ends the batch.  (Role of checkSQ7TidyTaskQ, enqueue_ofccl_dev.cu:491-627.)
__device__ __forceinline__ void ingestEntries(const DaemonArgs& A, const RankDev& R, WgShared& sh, Wave0Regs& st, int ch,
                                              int lane, int avail, uint64_t sendbuff, uint64_t recvbuff, uint32_t coll,
                                              uint32_t flags) {
  // buffers named by the new entries may have been written by the host, a copy engine or another kernel
  // before the submission
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
  const int base = st.numActive;
  bool isQuit = false, mine = false;
  if (lane < avail) {
    isQuit = (flags & kSqeFlagQuit) != 0;
    if (!isQuit && coll < (uint32_t)R.nColls) mine = ch < (int)(sh.collChannels[coll] & (kCollSolo - 1));
  }
  const uint64_t qm = __ballot(isQuit);
  const int q = qm ? (int)__builtin_ctzll(qm) : 64;
  const int take = avail < q ? avail : q;
  const uint64_t mm = __ballot(mine && lane < take);
  const int pos = __builtin_popcountll(mm & ((1ull << lane) - 1ull));
  if (mine && lane < take && base + pos < kMaxColls) {
    DFCCL_GLOBAL DynCtx* d = G(&R.dyn[(size_t)ch * R.nColls + coll]);
    d->sendbuff = sendbuff;
    d->recvbuff = recvbuff;
    d->active = 1;
    if ((int32_t)coll == sh.loadedColl) {
      // the collective whose context is resident starts its next instance: bring the resident copy up to date
      sh.dyn.sendbuff = sendbuff;
      sh.dyn.recvbuff = recvbuff;
      sh.dyn.active = 1;
      sh.peersLoaded = 0;
      if (sh.plan.proto == kProtoDirect && sh.dyn.slice == 0) {
        // and tell the peers at once where its buffers are, instead of when the scheduler gets to it
        publishBuffers(&sh.plan.pubs[(size_t)sh.plan.rank * sh.plan.nChannels + ch], sendbuff, recvbuff,
                       sh.dyn.instance, sh.plan.scalePtr, sh.plan.elemSize);
        sh.dyn.slice = 1;
      }
    } else {
      // Any other all-reduce of the direct protocol publishes its buffers here as well, straight from the
      // context in HBM: its peers can then fold it whenever they get to it, whatever this workgroup is busy
      // with, so that ranks which work through their collectives in different orders never wait for each
      // other before the data has moved.
      const DFCCL_GLOBAL CollPlan* pl = G(&R.plans[coll]);
      if (pl->proto == kProtoDirect &&
          __hip_atomic_load(G(&d->slice), __ATOMIC_RELAXED, DFCCL_AGENT) == 0) {
        publishBuffers(&pl->pubs[(size_t)pl->rank * pl->nChannels + ch], sendbuff, recvbuff,
                       __hip_atomic_load(G(&d->instance), __ATOMIC_RELAXED, DFCCL_AGENT), pl->scalePtr, pl->elemSize);
        d->slice = 1;
      }
    }
    sh.taskq[base + pos] = (uint16_t)coll;
  }
  int added = __builtin_popcountll(mm);
  if (added > kMaxColls - base) added = kMaxColls - base;  // (only the entries that were stored above)
  const int consumed = take + (q < avail ? 1 : 0);
  st.numActive = base + added;
  st.frontier += (uint64_t)consumed;
  if (q < avail) st.finalQuit = 1;
  st.ingested = consumed;
  st.allFresh = (base == 0) ? 1 : 0;
  if (lane == 0) {
    sh.numActive = base + added;
    sh.stats.sqesRead += (uint64_t)consumed;
    if (R.nChannels > 1) __hip_atomic_store(G(&R.wgFrontier[ch]), st.frontier, __ATOMIC_RELAXED, DFCCL_AGENT);
    trace(A, sh, kTrIngested, (uint32_t)consumed);
  }
  DFCCL_WAVE_LDS_SYNC();  // (the lanes' task queue entries are in place before any lane reads the queue)
}

// Leader, wave 0: fetch submissions from the host ring (four lanes per entry, each word validated by its own
// tag), hand them to the other channels through the HBM mirror, take them into the own task queue straight
// from the registers, and pick up the host's control word.  (Role of sqRead, enqueue_ofccl_dev.cu:85-173.)
__device__ __forceinline__ void pollHost(const DaemonArgs& A, const RankDev& R, WgShared& sh, Wave0Regs& st, int lane) {
  const uint64_t base = st.hostFrontier;
  const int32_t numActive = st.numActive;
  // With an empty task queue the leader has nothing to do but watch the ring's next entry and the control word
  // (lanes 0..3 and lane 60, one load instruction).  It keeps four such polls in flight, so that a new
  // entry is seen a fraction of a PCIe round trip after it lands rather than up to a whole one; the other
  // entries of a burst are fetched by the next, ordinary poll.
  // Not while other channels of the rank are still moving data, though: reads of host memory that are in
  // flight hold up the memory requests of every workgroup on the same XCD.  The rank is busy while it has
  // posted fewer completions than it has fetched submissions; then the leader polls once, and rarely.
  const int idleRounds = (int)A.knobs.idlePollRounds;
  bool busy = false;
  if (numActive == 0 && R.nChannels > 1)
    busy = DFCCL_WAVE_UNIFORM(__hip_atomic_load(G(R.cqTicket), __ATOMIC_RELAXED, DFCCL_AGENT)) < base;
  st.rankBusy = busy ? 1 : 0;
  const bool idleMode = numActive == 0 && idleRounds > 0 && !busy;
  const int nlanes = idleMode ? kSqeWords : kSqesPerPoll * kSqeWords;
  // every lane loads (the lanes without a word of their own re-read lane 0's, which costs nothing: it is the
  // same request), so that no load is conditional and several can stay in flight
  const uint64_t* pw = R.sq + ((base & (kSqRing - 1)) * kSqeWords);
  if (lane < nlanes) {
    pw = R.sq + (((base + (uint64_t)(lane >> 2)) & (kSqRing - 1)) * kSqeWords + (lane & 3));
  } else if (lane == 60) {
    pw = (const uint64_t*)R.ctrl;  // the control word's allocation is 64 bytes long
  }
  const DFCCL_GLOBAL uint64_t* p = (const DFCCL_GLOBAL uint64_t*)pw;
  const uint64_t tagWant = sqeTag(base + (uint64_t)(lane >> 2));
  uint64_t w;
  if (!idleMode) {
    w = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  } else {
    uint64_t q0 = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    __builtin_amdgcn_s_sleep(4);
    uint64_t q1 = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    __builtin_amdgcn_s_sleep(4);
    uint64_t q2 = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    __builtin_amdgcn_s_sleep(4);
    uint64_t q3 = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    int polls = 0;
    // one step: look at the oldest poll in flight; if it shows nothing, issue it again
#define DFCCL_IDLE_STEP(q)                                                                                    \
  {                                                                                                           \
    w = q;                                                                                                    \
    polls++;                                                                                                  \
    const bool some = (lane < kSqeWords) ? ((w & ~kPtrMask) == tagWant) : (lane == 60 && (uint32_t)w != 0);   \
    const uint64_t m = __ballot(some);                                                                        \
    if ((m & 0xfull) == 0xfull || (m >> 60) != 0) break;                                                      \
    __builtin_amdgcn_s_sleep(2);                                                                              \
    q = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);                                                 \
  }
    // the trip count is a constant on purpose: the unrolled loop keeps its four loads in flight, a rolled one
    // waits for all of them at its head
#pragma unroll
    for (int it = 0; it < kIdleRounds; it++) {
      DFCCL_IDLE_STEP(q0)
      DFCCL_IDLE_STEP(q1)
      DFCCL_IDLE_STEP(q2)
      DFCCL_IDLE_STEP(q3)
    }
#undef DFCCL_IDLE_STEP
    if (polls > 1) st.idle += polls - 1;  // (the same count in every lane: the loop ends on a ballot)
  }
  const bool valid = lane < nlanes && (w & ~kPtrMask) == tagWant;
  const uint64_t ctrlWord = readLane64(w, 60);  // (into scalar registers: the wave branches on it)
  const uint32_t ctrl = (uint32_t)ctrlWord, statsReq = (uint32_t)(ctrlWord >> 32);
  if (statsReq != st.statsReqSeen) {
    st.statsReqSeen = statsReq;
    if (lane == 0) __hip_atomic_store(G(&A.devFlags[2]), statsReq, __ATOMIC_RELAXED, DFCCL_AGENT);
  }
  if (ctrl != 0 && lane == 0) {
    if (ctrl & kCtrlQuitRequest) __hip_atomic_store(G(&A.devFlags[0]), 1u, __ATOMIC_RELAXED, DFCCL_AGENT);
    if (ctrl & kCtrlAbort) __hip_atomic_store(G(&A.devFlags[1]), 1u, __ATOMIC_RELAXED, DFCCL_AGENT);
  }
  const uint64_t vm = __ballot(valid);
  int n = 0;
  while (n < kSqesPerPoll && ((vm >> (4 * n)) & 0xfull) == 0xfull) n++;
  if (n == 0) {
    st.ingested = 0;
  } else {
    // lane k < n takes entry k
    const int srcLane = (lane * 4) & 63;
    const uint64_t w0 = __shfl(w, srcLane);
    const uint64_t w1 = __shfl(w, srcLane + 1);
    const uint64_t w2 = __shfl(w, srcLane + 2);
    const uint64_t sendbuff = w0 & kPtrMask, recvbuff = w1 & kPtrMask;
    const uint32_t coll = (uint32_t)(w2 & 0xffffffffull), flags = (uint32_t)((w2 >> 32) & 0xffffull);
    if (R.nChannels > 1) {
      if (lane < n) {
        const uint64_t ticket = base + (uint64_t)lane;
        DFCCL_GLOBAL DevSqe* e = G(&R.mirror[ticket & (kSqRing - 1)]);
        e->sendbuff = sendbuff;
        e->recvbuff = recvbuff;
        e->coll = coll;
        e->flags = flags;
        e->ticket = ticket;
      }
      // every lane's entry is written before lane 0 publishes the new tail
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      DFCCL_WAVE_LDS_SYNC();  // (the wave's fence covers all its lanes' stores)
      if (lane == 0) __hip_atomic_store(G(R.mirrorTail), base + (uint64_t)n, __ATOMIC_RELAXED, DFCCL_AGENT);
    }
    st.hostFrontier = base + (uint64_t)n;
    if (lane == 0) trace(A, sh, kTrSqeFetched, (uint32_t)n);
    ingestEntries(A, R, sh, st, 0, lane, n, sendbuff, recvbuff, coll, flags);
  }
  // The host may reuse entries every workgroup of the rank has consumed. It only looks at the head when the
  // ring seems full, so the head is published now and then, not on every poll.
  const uint64_t fetched = st.hostFrontier, published = st.publishedHead;
  if (fetched - published >= 64 || (n == 0 && fetched != published)) {
    uint64_t f = st.frontier;
    if (R.nChannels > 1) {
      f = ~0ull;
      if (lane < R.nChannels) f = __hip_atomic_load(G(&R.wgFrontier[lane]), __ATOMIC_RELAXED, DFCCL_AGENT);
      f = uniform64(waveMin64(f));
    }
    if (f != published) {
      if (lane == 0) __hip_atomic_store(G(R.sqHead), f, __ATOMIC_RELAXED, DFCCL_SYSTEM);
      st.publishedHead = f;
    }
  }
}

// Wave 0 of the other channels: take new entries from the mirror ring, one lane per entry.
__device__ __forceinline__ void ingestMirror(const DaemonArgs& A, const RankDev& R, WgShared& sh, Wave0Regs& st, int ch,
                                             int lane) {
  const uint64_t f = st.frontier;
  // polled with a relaxed load: an acquire would invalidate the L2 on every poll of every idle workgroup
  const uint64_t tail = DFCCL_WAVE_UNIFORM(__hip_atomic_load(G(R.mirrorTail), __ATOMIC_RELAXED, DFCCL_AGENT));
  const int avail = (int)((tail - f) < 64 ? (tail - f) : 64);
  if (avail <= 0) {
    st.ingested = 0;
    return;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  DevSqe e;
  e.sendbuff = e.recvbuff = 0;
  e.coll = 0;
  e.flags = 0;
  if (lane < avail) loadStruct(e, &R.mirror[(f + (uint64_t)lane) & (kSqRing - 1)]);
  ingestEntries(A, R, sh, st, ch, lane, avail, e.sendbuff, e.recvbuff, e.coll, e.flags);
}

// One lane: is this parked collective's wait condition met?
__device__ __forceinline__ bool descMet(const WaitDesc& w) {
  const bool tagged = (w.count & kWaitTagged) != 0;
  const int count = w.count & (kWaitTagged - 1);
  for (int i = 0; i < count; i++) {
    const DFCCL_GLOBAL uint64_t* p = (const DFCCL_GLOBAL uint64_t*)(uintptr_t)(w.ptr + (uint64_t)((int64_t)i * w.stride));
    if (!waitReached(__hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_AGENT), w.value, tagged)) return false;
  }
  return true;
}

// Wave 0: mark the collectives of the task queue that can move, 64 per pass, one
// lane per collective, from the wait descriptors saved with their contexts; and which of them wave 0 runs alone.
__device__ __forceinline__ void scanReady(const RankDev& R, WgShared& sh, Wave0Regs& st, int ch, int lane) {
  const int n = st.numActive;
  if (n == 0) {
    st.numReady = 0;
    if (lane == 0) sh.numReady = 0;
    return;
  }
  const bool fresh = st.allFresh && st.ingested > 0 && n <= 64;  // nothing is parked: everything arrived this round
  int total = 0;
  for (int base = 0; base < n; base += 64) {
    const int i = base + lane;
    bool ready = false, solo = false;
    if (i < n) {
      const uint32_t coll = sh.taskq[i];
      solo = (sh.collChannels[coll] & kCollSolo) != 0;
      if (fresh) {
        ready = true;
      } else {
        WaitDesc w0, w1;
        const DynCtx* d = &R.dyn[(size_t)ch * R.nColls + coll];
        loadStruct(w0, &d->wait[0]);
        loadStruct(w1, &d->wait[1]);
        ready = descMet(w0) && descMet(w1);
      }
    }
    const uint64_t m = __ballot(ready), ms = __ballot(ready && solo);
    if (lane == 0) {
      sh.ready[base >> 6] = m;
      sh.readySolo[base >> 6] = ms;
    }
    total += __builtin_popcountll(m);
  }
  st.numReady = total;
  if (lane == 0) sh.numReady = total;
}

// Outcome of a bounded wait.  `ok` comes from a ballot, so every lane of the wave holds the same value in a
// register: the wave's own code branches on that, never on a copy in LDS (a flag that lane 0 writes and the
// other lanes of the same wave read back is a data race as far as the compiler can tell, and it has been seen to
// place the other lanes' read before lane 0's write).  The other waves of the workgroup read sh.waitOk, after a
// workgroup barrier.
struct WaitResult {
  bool ok;
  uint64_t word;  // the word this lane saw last
};

// Wave 0: wait until both conditions hold.  Lanes 0..31 watch the counters of
// w0, lanes 32..63 those of w1; the ballot decides for the whole wave.  The wait
// is bounded: when the budget is spent the collective is preempted.  (Role of
// waitPeer, src/collectives_ofccl/device/ofccl_prims_simple.h:90-198.)
// `threshold` is the visit's spin budget, held in registers by every lane (all lanes update it alike);
// `slicesSinceLoad` is what the visit has moved so far (only the forced-preemption hook looks at it).
__device__ __forceinline__ WaitResult waitDescs(const DaemonArgs& A, WgShared& sh, int lane, const WaitDesc& w0,
                                                const WaitDesc& w1, bool adapt, int64_t& threshold,
                                                int64_t slicesSinceLoad, int64_t cap = 0) {
  bool ok;
  int64_t spins = 0;
  uint64_t seen = 0;
  if (lane == 0) trace(A, sh, kTrWaitBegin, (uint32_t)((w0.count + w1.count) & 0xffff));
  const int64_t forceEvery = A.knobs.forceQuitEvery;
  const bool forced = forceEvery > 0 && slicesSinceLoad >= forceEvery;
  if (forced) {
    ok = false;
  } else {
    const WaitDesc& w = (lane < 32) ? w0 : w1;
    const int idx = lane & 31;
    const bool tagged = (w.count & kWaitTagged) != 0;
    const DFCCL_GLOBAL uint64_t* p = nullptr;
    if (idx < (w.count & (kWaitTagged - 1)))
      p = (const DFCCL_GLOBAL uint64_t*)(uintptr_t)(w.ptr + (uint64_t)((int64_t)idx * w.stride));
    const uint64_t need = w.value;
    bool ready = (p == nullptr);
    const int64_t limit = (cap > 0 && cap < threshold) ? cap : threshold;
    for (;;) {
      if (!ready) {
        seen = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_AGENT);
        ready = waitReached(seen, need, tagged);
      }
      if (__ballot(!ready) == 0) { ok = true; break; }
      if (++spins >= limit) { ok = false; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    if (ok) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  if (ok && adapt && cap == 0) {
    const int64_t t = A.knobs.recvSuccessFactor * spins;
    if (t > threshold) threshold = t;
  }
  if (lane == 0) {
    trace(A, sh, kTrWaitEnd, (uint32_t)((ok ? 1u : 0u) | ((uint32_t)spins << 1)));
    sh.waitOk = ok ? 1 : 0;
    sh.stats.spins += (uint64_t)spins;
    if (forced) sh.stats.forcedQuits++;
    if (!ok) {
      sh.dyn.wait[0] = w0;
      sh.dyn.wait[1] = w1;
    }
  }
  WaitResult r;
  r.ok = ok;
  r.word = seen;
  return r;
}

// ---------------------------------------------------------------- data movement

template <int DT, int OP>
__device__ __forceinline__ void moveReduce(const void* s0, const void* s1, void* d0, void* d1, size_t nbytes, int tid) {
  const void* s[2] = {s0, s1};
  if (d1 != nullptr) {
    void* d[2] = {d0, d1};
    reduceCopyWG<DT, OP, 2, 2, kFifoUnroll, true, false, false>(s, d, nbytes, tid, kWgThreads);
  } else {
    void* d[1] = {d0};
    reduceCopyWG<DT, OP, 2, 1, kFifoUnroll, true, false, false>(s, d, nbytes, tid, kWgThreads);
  }
}

template <int DT>
__device__ __forceinline__ void moveReduceOp(int op, const void* s0, const void* s1, void* d0, void* d1, size_t nbytes,
                                             int tid) {
  switch (op) {
    case kSum: moveReduce<DT, kSum>(s0, s1, d0, d1, nbytes, tid); break;
    case kProd: moveReduce<DT, kProd>(s0, s1, d0, d1, nbytes, tid); break;
    case kMax: moveReduce<DT, kMax>(s0, s1, d0, d1, nbytes, tid); break;
    default: moveReduce<DT, kMin>(s0, s1, d0, d1, nbytes, tid); break;
  }
}

__device__ __forceinline__ void copySlice(const void* s0, void* d0, void* d1, size_t nbytes, int tid) {
  const void* s[1] = {s0};
  if (d1 != nullptr) {
    void* d[2] = {d0, d1};
    reduceCopyWG<kI8, kSum, 1, 2, kFifoUnroll, true, false, false>(s, d, nbytes, tid, kWgThreads);
  } else {
    void* d[1] = {d0};
    reduceCopyWG<kI8, kSum, 1, 1, kFifoUnroll, true, false, false>(s, d, nbytes, tid, kWgThreads);
  }
}

// Expands CALL once for every element type of ncclDataType_t, with DT the type's number as a constant.
#define DFCCL_FOR_DTYPE(dtype, CALL)                        \
  switch (dtype) {                                          \
    case kF32: { constexpr int DT = kF32; CALL; } break;    \
    case kBF16: { constexpr int DT = kBF16; CALL; } break;  \
    case kF16: { constexpr int DT = kF16; CALL; } break;    \
    case kI32: { constexpr int DT = kI32; CALL; } break;    \
    case kI8: { constexpr int DT = kI8; CALL; } break;      \
    case kU8: { constexpr int DT = kU8; CALL; } break;      \
    case kU32: { constexpr int DT = kU32; CALL; } break;    \
    case kI64: { constexpr int DT = kI64; CALL; } break;    \
    case kU64: { constexpr int DT = kU64; CALL; } break;    \
    default: { constexpr int DT = kF64; CALL; } break;      \
  }

// One slice: 1 or 2 sources into 1 or 2 destinations (s1 / d1 may be null).
__device__ __forceinline__ void moveSlice(int dtype, int op, const void* s0, const void* s1, void* d0, void* d1,
                                          size_t nbytes, int tid) {
  if (s1 == nullptr) {
    copySlice(s0, d0, d1, nbytes, tid);
    return;
  }
  DFCCL_FOR_DTYPE(dtype, moveReduceOp<DT>(op, s0, s1, d0, d1, nbytes, tid));
}

// The same for a slice of a scaled sum (ncclAvg, PreMulSum) that reads a user input or produces the final value:
// source 0 is the user's buffer whenever a step has one (su.preMask says whether it is multiplied).
template <int DT>
__device__ __forceinline__ void moveScaled(const void* s0, const void* s1, void* d0, void* d1, size_t nbytes, int tid,
                                           const ScaleUse& su) {
  if (s1 != nullptr) {
    const void* s[2] = {s0, s1};
    if (d1 != nullptr) {
      void* d[2] = {d0, d1};
      reduceCopyWG<DT, kSum, 2, 2, kFifoUnrollScaled, true, true, false>(s, d, nbytes, tid, kWgThreads, su);
    } else {
      void* d[1] = {d0};
      reduceCopyWG<DT, kSum, 2, 1, kFifoUnrollScaled, true, true, false>(s, d, nbytes, tid, kWgThreads, su);
    }
  } else {
    const void* s[1] = {s0};
    if (d1 != nullptr) {
      void* d[2] = {d0, d1};
      reduceCopyWG<DT, kSum, 1, 2, kFifoUnrollScaled, true, true, false>(s, d, nbytes, tid, kWgThreads, su);
    } else {
      void* d[1] = {d0};
      reduceCopyWG<DT, kSum, 1, 1, kFifoUnrollScaled, true, true, false>(s, d, nbytes, tid, kWgThreads, su);
    }
  }
}
__device__ __forceinline__ void moveSliceScaled(int dtype, const void* s0, const void* s1, void* d0, void* d1,
                                                size_t nbytes, int tid, const ScaleUse& su) {
  DFCCL_FOR_DTYPE(dtype, moveScaled<DT>(s0, s1, d0, d1, nbytes, tid, su));
}

// Direct protocol data movement.  A "tile" is one rank's chunk of one loop.

// dst[k][off..] = src[0][off..] (op) src[1][off..] ... (op) src[n-1][off..] for every k < nd, folded left to
// right with every step rounded to the storage type: with src = in[c+1], in[c+2], ..., in[c] this is the ring's
// order for a chunk owned by rank c.  n <= NS <= kMaxDirectRanks (NS = 1: plain copy); the NS - n surplus loads
// re-read src[0] (they hit in cache) so that every array element is defined: predicated loads made the compiler
// keep the packs in scratch.  A destination may be one of the sources (in place): each thread reads a pack
// before it writes it, and no other thread touches that pack.
// SC: a scaled sum (OP is kSum): every source is a user input and is multiplied by its rank's scalar first
// (kScalePre; lane j of `scaleV` holds the scalar that belongs to src[j]), or the result is divided by the group
// size (kScalePost, integer types).
template <int DT, int OP, int NS, bool SC = false>
__device__ __forceinline__ void foldTile(const uint64_t (&src)[kMaxDirectRanks], const uint64_t (&dst)[kMaxDirectRanks],
                                         int n, int nd, int64_t byteOff, size_t nbytes, int tid, int nthr,
                                         int scaleKind, uint64_t scaleV, uint64_t scaleBits) {
  constexpr int ES = typeSize(DT);
  const bool pre = SC && scaleKind == kScalePre;
  const bool post = SC && !isFloatType(DT) && scaleKind == kScalePost;
  const int divisor = (int)scaleBits;
  // lane j of every wave holds the scalar that belongs to src[j] (all lanes are here: the call is uniform)
  uint64_t scale[NS];
#pragma unroll
  for (int j = 0; j < NS; j++) {
    if constexpr (SC) scale[j] = readLane64(scaleV, j);
    else scale[j] = 0;
  }
  uint64_t align = (uint64_t)byteOff;
#pragma unroll
  for (int j = 0; j < NS; j++) align |= (j < n ? src[j] : 0);
#pragma unroll
  for (int j = 0; j < kMaxDirectRanks; j++) align |= (j < nd ? dst[j] : 0);
  size_t doneBytes = 0;
  if ((align & 15u) == 0) {
    const size_t npacks = nbytes >> 4;
#pragma clang loop vectorize(disable) interleave(disable) unroll(disable)
    for (size_t i = tid; i < npacks; i += nthr) {
      u32x4 v[NS];
#pragma unroll
      for (int j = 0; j < NS; j++) v[j] = loadPack<true>((const char*)(j < n ? src[j] : src[0]) + byteOff, i);
      if (pre) {
#pragma unroll
        for (int j = 0; j < NS; j++) v[j] = packOp<DT, kProd>(v[j], splatScalar<DT>(scale[j]));
      }
      u32x4 acc = v[0];
#pragma unroll
      for (int j = 1; j < NS; j++)
        if (j < n) acc = packOp<DT, OP>(acc, v[j]);
      if (post) acc = packPostDiv<DT>(acc, divisor);
#pragma unroll
      for (int j = 0; j < kMaxDirectRanks; j++)
        if (j < nd) storePack<false>((char*)dst[j] + byteOff, i, acc);
    }
    doneBytes = npacks << 4;
  }
  const size_t first = doneBytes / ES, nelem = nbytes / ES;
#pragma clang loop vectorize(disable) interleave(disable) unroll(disable)
  for (size_t i = first + tid; i < nelem; i += nthr) {
    uint64_t acc = loadElem<ES>((const char*)src[0] + byteOff, i);
    if (pre) acc = elemPreMul<DT>(acc, scale[0]);
#pragma unroll
    for (int j = 1; j < NS; j++)
      if (j < n) {
        uint64_t v = loadElem<ES>((const char*)src[j] + byteOff, i);
        if (pre) v = elemPreMul<DT>(v, scale[j]);
        acc = elemOp<DT, OP>(acc, v);
      }
    if (post) acc = elemPostDiv<DT>(acc, divisor);
#pragma unroll
    for (int j = 0; j < kMaxDirectRanks; j++)
      if (j < nd) storeElem<ES>((char*)dst[j] + byteOff, i, acc);
  }
}

// Which fold a sweep uses, as one number: the plain folds by (element type, operator, sources held in registers: 2, 4
// or 8), then the scaled sums by (element type, sources), then the plain copy.
constexpr int kFoldScaledBase = 10 * 4 * 3;
constexpr int kFoldCopy = kFoldScaledBase + 10 * 3;
__device__ __forceinline__ int foldVariant(const SweepGeom& g) {
  if (g.n <= 1) return kFoldCopy;  // plain copy, whatever the type
  const int held = g.n <= 2 ? 0 : (g.n <= 4 ? 1 : 2);
  if (g.scaleKind != kScaleNone) return kFoldScaledBase + g.dtype * 3 + held;  // ncclAvg / PreMulSum: a sum with a scale
  return (g.dtype * 4 + g.op) * 3 + held;
}

#define DFCCL_FOLD_ARGS g.src, g.dst, g.n, g.nd, byteOff, nbytes, tid, nthr, g.scaleKind, scaleV, g.scaleBits
#define DFCCL_FOLD_CASES_HELD(BASE, DT, OP, SC)                            \
  case (BASE) + 0: foldTile<DT, OP, 2, SC>(DFCCL_FOLD_ARGS); break;        \
  case (BASE) + 1: foldTile<DT, OP, 4, SC>(DFCCL_FOLD_ARGS); break;        \
  case (BASE) + 2: foldTile<DT, OP, 8, SC>(DFCCL_FOLD_ARGS); break;
#define DFCCL_FOLD_CASES_TYPE(DT)                                          \
  DFCCL_FOLD_CASES_HELD((DT * 4 + kSum) * 3, DT, kSum, false)              \
  DFCCL_FOLD_CASES_HELD((DT * 4 + kProd) * 3, DT, kProd, false)            \
  DFCCL_FOLD_CASES_HELD((DT * 4 + kMax) * 3, DT, kMax, false)              \
  DFCCL_FOLD_CASES_HELD((DT * 4 + kMin) * 3, DT, kMin, false)              \
  DFCCL_FOLD_CASES_HELD(kFoldScaledBase + DT * 3, DT, kSum, true)
__device__ __forceinline__ void foldTileAny(int variant, const SweepGeom& g, uint64_t scaleV, int64_t byteOff,
                                            size_t nbytes, int tid, int nthr) {
  static_assert(kI8 == 0 && kBF16 == 9, "the variants are numbered by the element types 0..9");
  switch (variant) {
    DFCCL_FOLD_CASES_TYPE(kI8)
    DFCCL_FOLD_CASES_TYPE(kU8)
    DFCCL_FOLD_CASES_TYPE(kI32)
    DFCCL_FOLD_CASES_TYPE(kU32)
    DFCCL_FOLD_CASES_TYPE(kI64)
    DFCCL_FOLD_CASES_TYPE(kU64)
    DFCCL_FOLD_CASES_TYPE(kF16)
    DFCCL_FOLD_CASES_TYPE(kF32)
    DFCCL_FOLD_CASES_TYPE(kF64)
    DFCCL_FOLD_CASES_TYPE(kBF16)
    default: foldTile<kI8, kSum, 1, false>(DFCCL_FOLD_ARGS); break;
  }
}
#undef DFCCL_FOLD_CASES_TYPE
#undef DFCCL_FOLD_CASES_HELD
#undef DFCCL_FOLD_ARGS

// The sweep of the direct protocol.  A tile is my rank's chunk in one channel slot of one loop: tile t lies in
// loop t / C, slot t % C, at l * loop + (slot * tn + tme) * real (tn = ranks that share the index space, tme = my
// place among them).  For every tile it takes, the workgroup folds the chunk from the n sources and writes the
// result into the nd destinations.  Tiles are handed out low to
// high, so at any instant the accesses of the whole grid fall into a narrow window of every buffer.
//  * With one channel the workgroup takes the tiles in order; `pos` is the next tile.
//  * With several channels the first loop is static (workgroup ch takes tile ch; pos 0 = not done yet) and the
//    rest is handed out by the rank's tile counter, whichever workgroup is free next: workgroups do not finish
//    at the same moment otherwise (HBM channels are not equally fast for all of them), and the slowest one
//    decides when the collective is done.  The next tile is requested while the current one is folded.  Every
//    workgroup draws exactly one number past the end per instance, so the counter advances by exactly T.
// At most maxTiles tiles are processed; `finished` says that no tile is left.
// `variant` (foldVariant) picks the fold for the element type, the operator and the number of sources; it is
// looked up once per tile (one indexed branch), so that the loop around it exists once and not once per variant.
__device__ __forceinline__ void sweepTiles(const SweepGeom& g, int variant, uint64_t scaleV, uint64_t* slots,
                                           int64_t& posInOut, int64_t maxTiles, int tid, int nthr, int64_t& tilesDone,
                                           bool& finished) {
  const bool dynamic = g.C > 1;
  DFCCL_GLOBAL uint64_t* ctr = (DFCCL_GLOBAL uint64_t*)(uintptr_t)g.ctr;
  int64_t pos = posInOut, done = 0;
  bool fin = false, have = false;
  uint64_t tile = 0;
  uint32_t par = 0;
  while (done < maxTiles) {
    if (!have) {
      if (!dynamic) {
        tile = (uint64_t)pos++;
      } else if (pos == 0) {
        tile = (uint64_t)g.ch;
        pos = 1;
      } else {
        if (tid == 0)
          slots[par] = __hip_atomic_fetch_add(ctr, 1ull, __ATOMIC_RELAXED, DFCCL_AGENT) - g.instBase + (uint64_t)g.C;
        __syncthreads();
        tile = DFCCL_UNIFORM(slots[par]);
        par ^= 1u;
      }
    }
    have = false;
    if (tile >= (uint64_t)g.T) {
      fin = true;
      break;
    }
    const bool prefetch = dynamic && done + 1 < maxTiles;
    uint64_t nxt = 0;
    if (prefetch && tid == 0)
      nxt = __hip_atomic_fetch_add(ctr, 1ull, __ATOMIC_RELAXED, DFCCL_AGENT) - g.instBase + (uint64_t)g.C;
    const uint32_t l = (uint32_t)tile / (uint32_t)g.C, slot = (uint32_t)tile % (uint32_t)g.C;
    const int64_t real = ((int64_t)l == g.L - 1) ? g.lastReal : g.chunkElems;
    const int64_t off = (int64_t)l * g.loop + ((int64_t)slot * g.tn + g.tme) * real;
    const int64_t nelem = (g.count - off < real) ? g.count - off : real;
    if (nelem > 0) foldTileAny(variant, g, scaleV, off * g.es, (size_t)(nelem * g.es), tid, nthr);
    done++;
    if (prefetch) {
      if (tid == 0) slots[par] = nxt;
      __syncthreads();
      tile = DFCCL_UNIFORM(slots[par]);
      par ^= 1u;
      have = true;
    }
  }
  posInOut = pos;
  tilesDone = done;
  finished = fin;
}

// `tid` of `nthr` threads take part (the whole workgroup, or wave 0 alone); the geometry is the same in all of them.
// `scaleV`: pre-multiplied sums only; lane t of every wave holds the scalar of the rank whose input is g.src[t].
__device__ __forceinline__ void sweepFoldAny(const SweepGeom& g, uint64_t scaleV, uint64_t* slots, int64_t& pos,
                                             int64_t maxTiles, int tid, int nthr, int64_t& tilesDone, bool& finished) {
  sweepTiles(g, foldVariant(g), scaleV, slots, pos, maxTiles, tid, nthr, tilesDone, finished);
}

// ------------------------------------------------------------- FIFO ring protocol

// Runs the loaded collective from its saved position until it is done or a wait
// expires.  Every thread takes the same path: all decisions come from LDS after
// a barrier.  (Role of the resumable runRing bodies and genericOp; see
// ring_schedule.h for the per-step roles.)
__device__ __forceinline__ int runFifo(const DaemonArgs& A, WgShared& sh, int ch, int tid) {
  const int lane = tid & 63, wave = DFCCL_UNIFORM(tid >> 6);
  // the plan and the position, taken from LDS into scalar registers (see DFCCL_UNIFORM)
  struct {
    int kind, dtype, op, root, nRanks, rank, slicesPerChunk, fifoSlots, scaleKind;
    int64_t chunkElems, alignElems, sliceElems, slotBytes;
    ConnFlags *sendFlags, *recvFlags;
  } P;
  P.kind = DFCCL_UNIFORM(sh.plan.kind);
  P.dtype = DFCCL_UNIFORM(sh.plan.dtype);
  P.op = DFCCL_UNIFORM(sh.plan.op);
  P.root = DFCCL_UNIFORM(sh.plan.root);
  P.nRanks = DFCCL_UNIFORM(sh.plan.nRanks);
  P.rank = DFCCL_UNIFORM(sh.plan.rank);
  P.slicesPerChunk = DFCCL_UNIFORM(sh.plan.slicesPerChunk);
  P.fifoSlots = DFCCL_UNIFORM(sh.plan.fifoSlots);
  P.scaleKind = DFCCL_UNIFORM(sh.plan.scaleKind);
  P.chunkElems = DFCCL_UNIFORM(sh.plan.chunkElems);
  P.alignElems = DFCCL_UNIFORM(sh.plan.alignElems);
  P.sliceElems = DFCCL_UNIFORM(sh.plan.sliceElems);
  P.slotBytes = DFCCL_UNIFORM(sh.plan.slotBytes);
  P.sendFlags = DFCCL_UNIFORM(sh.plan.sendFlags);
  P.recvFlags = DFCCL_UNIFORM(sh.plan.recvFlags);
  const int kind = P.kind, n = P.nRanks, C = DFCCL_UNIFORM(sh.plan.nChannels), es = DFCCL_UNIFORM(sh.plan.elemSize);
  const int64_t count = DFCCL_UNIFORM(sh.plan.count);
  const int64_t loop = loopElems(kind, n, C, P.chunkElems);
  const int nsteps = stepsPerLoop(kind, n);
  const char* sendbuff = (const char*)DFCCL_UNIFORM(sh.dyn.sendbuff);
  char* recvbuff = (char*)DFCCL_UNIFORM(sh.dyn.recvbuff);
  const int64_t fifoChanStride = DFCCL_UNIFORM(sh.plan.fifoChanStride);
  char* sendFifo = DFCCL_UNIFORM(sh.plan.sendFifo) + (int64_t)ch * fifoChanStride;
  const char* recvFifo = DFCCL_UNIFORM(sh.plan.recvFifo) + (int64_t)ch * fifoChanStride;
  int inPlace;
  if (kind == kAllGather) {
    inPlace = (sendbuff == recvbuff + (int64_t)P.rank * count * es);
  } else {
    inPlace = (sendbuff == recvbuff);
  }
  // this rank's scalar of a scaled sum: from the plan, or read from device memory at every visit of an instance
  // (a value that changes while the instance runs is the caller's affair, as in the reference)
  uint64_t scaleBits = DFCCL_UNIFORM(sh.plan.scaleBits);
  if (P.scaleKind == kScalePre) {
    const void* scalePtr = DFCCL_UNIFORM(sh.plan.scalePtr);
    if (scalePtr != nullptr) scaleBits = uniform64(loadScalar(scalePtr, es));
    if (n == 1) inPlace = 0;  // a one-rank communicator still multiplies: its copy may not be skipped
  }

  int64_t grid = DFCCL_UNIFORM(sh.dyn.gridOffset);
  int step0 = DFCCL_UNIFORM(sh.dyn.step), slice0 = DFCCL_UNIFORM(sh.dyn.slice);
  uint64_t sendStep = DFCCL_UNIFORM(sh.dyn.sendStep), recvStep = DFCCL_UNIFORM(sh.dyn.recvStep);
  int64_t threshold = DFCCL_UNIFORM(sh.threshold);  // the visit's spin budget (every thread keeps the same copy)
  int64_t slicesSinceLoad = 0;                      // slices this visit has moved over a link

  for (; grid < count; grid += loop, step0 = 0) {
    const int64_t real = realChunkElems(kind, n, C, P.chunkElems, P.alignElems, count, grid);
    for (int s = step0; s < nsteps; ++s, slice0 = 0) {
      const StepDesc d = describeStep(kind, n, P.rank, P.root, C, ch, count, grid, real, s, inPlace);
      if (d.nelem <= 0) continue;
      const int64_t sliceE = sliceElemsFor(d.nelem, P.slicesPerChunk, P.sliceElems);
      for (int sl = slice0; (int64_t)sl * sliceE < d.nelem; ++sl) {
        const int64_t off = (int64_t)sl * sliceE;
        const int64_t len = (d.nelem - off < sliceE) ? d.nelem - off : sliceE;
        if (d.recv || d.send) {
          // receive: the slot is filled (tail >= recvStep + 1); send: a slot is free (head + slots >= sendStep + 1)
          const WaitDesc w0 = d.recv ? waitFor(&P.recvFlags[ch].tail, recvStep + 1, 0, 1) : noWait();
          const uint64_t needHead = (sendStep + 1 > (uint64_t)P.fifoSlots) ? sendStep + 1 - (uint64_t)P.fifoSlots : 0;
          const WaitDesc w1 = d.send ? waitFor(&P.sendFlags[ch].head, needHead, 0, 1) : noWait();
          bool ok = true;
          if (wave == 0) ok = waitDescs(A, sh, lane, w0, w1, d.recv != 0, threshold, slicesSinceLoad).ok;
          __syncthreads();
          if (wave != 0) ok = DFCCL_UNIFORM(sh.waitOk) != 0;
          if (!ok) {
            if (tid == 0) {
              sh.dyn.gridOffset = grid;
              sh.dyn.step = s;
              sh.dyn.slice = sl;
              sh.dyn.sendStep = sendStep;
              sh.dyn.recvStep = recvStep;
            }
            return kRunPreempted;
          }
        }
        const void* s0 = nullptr;
        const void* s1 = nullptr;
        void* d0 = nullptr;
        void* d1 = nullptr;
        const void* fifoIn = d.recv ? recvFifo + (int64_t)(recvStep % (uint64_t)P.fifoSlots) * P.slotBytes : nullptr;
        void* fifoOut = d.send ? sendFifo + (int64_t)(sendStep % (uint64_t)P.fifoSlots) * P.slotBytes : nullptr;
        if (d.useIn) {
          s0 = sendbuff + (d.inOff + off) * es;
          s1 = fifoIn;
        } else {
          s0 = fifoIn;
        }
        if (d.useOut) {
          d0 = recvbuff + (d.outOff + off) * es;
          d1 = fifoOut;
        } else {
          d0 = fifoOut;
        }
        if (s0 != nullptr && d0 != nullptr) {
          // a scaled sum (ncclAvg / PreMulSum) multiplies the user's input where it enters (source 0 of a step that
          // reads it) and divides where the final value is produced
          const bool scaledStep = (P.scaleKind == kScalePre && d.useIn) || (P.scaleKind == kScalePost && d.post);
          if (scaledStep) {
            ScaleUse su;
            su.scale.kind = P.scaleKind;
            su.scale.bits = scaleBits;
            su.preMask = d.useIn ? 1u : 0u;
            su.post = d.post != 0;
            moveSliceScaled(P.dtype, s0, s1, d0, d1, (size_t)(len * es), tid, su);
          } else {
            moveSlice(P.dtype, P.op, s0, s1, d0, d1, (size_t)(len * es), tid);
          }
        }
        if (d.recv || d.send) {
          __syncthreads();  // every thread's loads and stores of this slice are done
          if (tid == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            if (d.send) __hip_atomic_store(G(&P.sendFlags[ch].tail), sendStep + 1, __ATOMIC_RELAXED, DFCCL_AGENT);
            if (d.recv) __hip_atomic_store(G(&P.recvFlags[ch].head), recvStep + 1, __ATOMIC_RELAXED, DFCCL_AGENT);
            trace(A, sh, kTrPosted, (uint32_t)s);
            sh.progressed = 1;
            sh.stats.slicesMoved++;
          }
          slicesSinceLoad++;
          sendStep += d.send ? 1 : 0;
          recvStep += d.recv ? 1 : 0;
        } else if (tid == 0) {
          sh.progressed = 1;
          sh.stats.slicesMoved++;
        }
      }
    }
  }
  // (only if a slice has gone over a link: its barrier then lies between the other threads' reading of the
  // counters at the top and this; a visit that finds nothing left to do must not write what slower threads may
  // still be reading, even though it would write the same values)
  if (tid == 0 && slicesSinceLoad > 0) {
    sh.dyn.sendStep = sendStep;
    sh.dyn.recvStep = recvStep;
  }
  return kRunDone;
}

// ----------------------------------------------------------------- direct protocol

// Every field of the sweep's geometry is the same in every thread (it was built from the plan, or copied from
// LDS): into scalar registers with all of it.
__device__ __forceinline__ void uniformGeom(SweepGeom& g) {
  g.count = (int64_t)uniform64((uint64_t)g.count);
  g.loop = (int64_t)uniform64((uint64_t)g.loop);
  g.chunkElems = (int64_t)uniform64((uint64_t)g.chunkElems);
  g.lastReal = (int64_t)uniform64((uint64_t)g.lastReal);
  g.L = (int64_t)uniform64((uint64_t)g.L);
  g.T = (int64_t)uniform64((uint64_t)g.T);
  g.instBase = uniform64(g.instBase);
  g.ctr = uniform64(g.ctr);
  g.n = __builtin_amdgcn_readfirstlane(g.n);
  g.C = __builtin_amdgcn_readfirstlane(g.C);
  g.ch = __builtin_amdgcn_readfirstlane(g.ch);
  g.es = __builtin_amdgcn_readfirstlane(g.es);
  g.me = __builtin_amdgcn_readfirstlane(g.me);
  g.dtype = __builtin_amdgcn_readfirstlane(g.dtype);
  g.op = __builtin_amdgcn_readfirstlane(g.op);
  g.nd = __builtin_amdgcn_readfirstlane(g.nd);
  g.tn = __builtin_amdgcn_readfirstlane(g.tn);
  g.tme = __builtin_amdgcn_readfirstlane(g.tme);
  g.scaleKind = __builtin_amdgcn_readfirstlane(g.scaleKind);
  g.scaleBits = uniform64(g.scaleBits);
#pragma unroll
  for (int t = 0; t < kMaxDirectRanks; t++) {
    g.src[t] = uniform64(g.src[t]);
    g.dst[t] = uniform64(g.dst[t]);
  }
}

// Wave 0, after the wait for the peers' publications: lanes 0..n-1 hold the peers' send words, lanes
// 32..32+n-1 their receive words.  Every lane builds the whole geometry of the sweep in registers.
__device__ __forceinline__ void layOutSweep(SweepGeom& g, const CollPlan& P, int ch, uint64_t inst, uint64_t word) {
  const int kind = P.kind, root = P.root, n = P.nRanks, me = P.rank, C = P.nChannels, es = P.elemSize;
  const int64_t L = P.loopsPerInstance;
  const bool owned = (kind == kAllReduce || kind == kReduce || kind == kBroadcast);
  const bool folds = (kind == kAllReduce || kind == kReduce || kind == kReduceScatter);
  const bool toAll = (kind == kAllReduce || kind == kBroadcast || kind == kAllGather);
  const int first = ((kind == kReduce) ? root : me) + 1;  // rank the fold starts with (before wrapping)
  const uint64_t srcOff = (kind == kReduceScatter) ? (uint64_t)me * (uint64_t)P.count * (uint64_t)es : 0;
  const uint64_t dstOff = (kind == kAllGather) ? (uint64_t)me * (uint64_t)P.count * (uint64_t)es : 0;
  g.n = folds ? n : 1;
  g.nd = toAll ? n : 1;
#pragma unroll
  for (int t = 0; t < kMaxDirectRanks; t++) {
    int sr = folds ? first + t : (kind == kBroadcast ? root : me);
    if (sr >= n) sr -= n;
    if (sr >= n) sr = 0;  // (t >= n: the entry is not used)
    int dr = toAll ? t : (kind == kReduce ? root : me);
    if (dr >= n) dr = 0;
    const uint64_t sp = readLane64(word, sr) & kPtrMask, dp = readLane64(word, 32 + dr) & kPtrMask;
    g.src[t] = (t < g.n) ? sp + srcOff : 0;
    g.dst[t] = (t < g.nd) ? dp + dstOff : 0;
  }
  g.tn = owned ? n : 1;
  g.tme = owned ? me : 0;
  g.count = P.count;
  g.loop = (int64_t)C * g.tn * P.chunkElems;
  g.chunkElems = P.chunkElems;
  g.lastReal = P.lastChunkElems;
  g.L = L;
  g.T = L * C;
  g.instBase = inst * (uint64_t)(L * C);
  g.ctr = (uint64_t)(uintptr_t)P.tileCtr;
  g.C = C;
  g.ch = ch;
  g.es = es;
  g.me = me;
  g.dtype = P.dtype;
  g.op = P.op;
  g.scaleKind = folds ? P.scaleKind : (int)kScaleNone;
  g.scaleBits = P.scaleBits;
  g.pad1 = 0;
}

// Collectives in which the virtual ranks, whose buffers share one HBM, read each
// other's send buffers and write each other's receive buffers in place.
//   publish   my buffers for this instance (normally done when the submission was
//             ingested); wait until every peer has published (its receive buffer
//             may be written from then on);
//   sweep     my share of the work, tile by tile: fold the sources in the ring's
//             order for those elements and store the result into the destinations;
//             release; p1[me] = loops done;
//   finally   wait until every peer's p1 covers the instance: everything that had
//             to land in my receive buffer has, and nobody reads my send buffer any
//             more, so the completion may be posted.
// What "my share", sources and destinations are (n ranks, me, root; chunks as in
// ring_schedule.h: loop l, channel slot c, chunk j starts at l * loop + (c * n + j) * real):
//   all-reduce      the chunks owned by me;  in[me+1], ..., in[me] (the order in which the ring
//                   accumulates a chunk that ends at its owner)  ->  every receive buffer
//   reduce          the chunks owned by me;  in[root+1], ..., in[root]  ->  the root's receive buffer
//   broadcast       the chunks owned by me;  the root's send buffer  ->  every receive buffer
//   reduce-scatter  all of block me of the send buffers;  in[me+1], ..., in[me]  ->  my receive buffer
//   all-gather      all of my send buffer  ->  block me of every receive buffer
// Every input element is read once and every output element written once, against
// the FIFO ring's staging of every slice through HBM at every step.
// Two waits per instance whatever its size; each is a WaitDesc and can preempt.
// dyn.step is the phase (0 = sweep, 2 = only the final wait is left),
// dyn.gridOffset the sweep's position (see sweepTiles), dyn.slice whether the
// instance is published.
//
// Small collectives (the low-latency path): when the whole share of this rank is one tile of at most
// kSoloMaxBytes, wave 0 runs the instance alone (`solo`): waits, sweep, release and the final wait follow each
// other inside one wave, with every decision in registers and not one workgroup barrier in between, while the
// other waves go straight to the barrier that ends the visit.  The steps, the memory ordering and the saved
// state are the same as for the whole workgroup; only who takes part differs.
// `solo`: the collective was marked at launch as one that wave 0 runs alone (soloCollective); only wave 0 is here then.
__device__ __forceinline__ int runDirect(const DaemonArgs& A, WgShared& sh, int ch, int tid, const bool solo) {
  const CollPlan& P = sh.plan;
  const int lane = tid & 63, wave = DFCCL_UNIFORM(tid >> 6);
  const int n = DFCCL_UNIFORM(P.nRanks), C = DFCCL_UNIFORM(P.nChannels), me = DFCCL_UNIFORM(P.rank);
  const int64_t L = DFCCL_UNIFORM(P.loopsPerInstance);
  const int64_t forceEvery = A.knobs.forceQuitEvery;
  const int nthr = solo ? 64 : kWgThreads;   // threads that take part
  const int mtid = solo ? lane : tid;

  const uint64_t inst = DFCCL_UNIFORM(sh.dyn.instance);
  const uint64_t base = inst * (uint64_t)L;
  const uint64_t sendbuff = DFCCL_UNIFORM(sh.dyn.sendbuff), recvbuff = DFCCL_UNIFORM(sh.dyn.recvbuff);
  const int published = DFCCL_UNIFORM(sh.dyn.slice);
  // (a wave on its own keeps the sweep's geometry in registers)
  const int peersLoaded = solo ? 0 : DFCCL_UNIFORM(sh.peersLoaded);
  const int pubStride = C * (int)sizeof(PeerPub), ctrStride = C * 8;
  PeerPub* const pubs = DFCCL_UNIFORM(P.pubs);
  uint64_t* const p1 = DFCCL_UNIFORM(P.p1);
  const int scaleKind = DFCCL_UNIFORM(P.scaleKind);
  PeerPub* myPub = &pubs[(size_t)me * C + ch];
  const int64_t l0 = DFCCL_UNIFORM(sh.dyn.gridOffset);
  const int phase = DFCCL_UNIFORM(sh.dyn.step);
  int64_t threshold = DFCCL_UNIFORM(sh.threshold);  // the visit's spin budget (every thread keeps the same copy)
  int64_t slicesSinceLoad = 0;                      // tiles this visit has moved
  // With other collectives queued a wait is only a look: switching is cheap here (contexts are small and
  // nothing is held while parked), and the workgroup is better off moving the next collective's data.
  const int64_t cap = (DFCCL_UNIFORM(sh.numActive) > 1 && forceEvery == 0) ? kSoftWaitSpins : 0;
  // every thread has taken its copy of the position before thread 0 changes it
  if (solo) {
    DFCCL_WAVE_LDS_SYNC();
  } else {
    __syncthreads();
  }

  if (!published && tid == 0) {
    publishBuffers(myPub, sendbuff, recvbuff, inst, sh.plan.scalePtr, sh.plan.elemSize);
    sh.dyn.slice = 1;
  }

  if (phase == 0) {
    SweepGeom g;
    uint64_t scaleV = 0;  // pre-multiplied sums: lane t holds the scalar of the rank whose input is source t of the fold
    if (!peersLoaded) {
      bool ok = true;
      if (wave == 0) {
        // lanes 0..n-1 watch the peers' send words, lanes 32..32+n-1 their receive words
        const WaitDesc w0 = waitFor(&pubs[ch].send, pubTag(inst) >> 48, pubStride, n | kWaitTagged);
        const WaitDesc w1 = waitFor(&pubs[ch].recv, pubTag(inst) >> 48, pubStride, n | kWaitTagged);
        const WaitResult r = waitDescs(A, sh, lane, w0, w1, true, threshold, slicesSinceLoad, cap);
        ok = r.ok;
        if (ok) {
          // a pre-multiplied sum scales every rank's input by that rank's own scalar, found next to its
          // pointers (written before them: the wait's acquire has made it visible)
          if (scaleKind == kScalePre) {
            uint64_t scaleWord = 0;
            if (lane < n) scaleWord = __hip_atomic_load(G(&pubs[(size_t)lane * C + ch].scale), __ATOMIC_RELAXED, DFCCL_AGENT);
            // source t of the fold is rank first + t (layOutSweep)
            int sr = ((P.kind == kReduce) ? P.root : me) + 1 + (lane & (kMaxDirectRanks - 1));
            if (sr >= n) sr -= n;
            if (sr >= n) sr = 0;
            scaleV = __shfl(scaleWord, sr);
            if (!solo && lane < kMaxDirectRanks) sh.sweepScale[lane] = scaleV;
          }
          layOutSweep(g, P, ch, inst, r.word);
          if (tid == 0) trace(A, sh, kTrLaidOut, 0);
          if (!solo && lane == 0) {
            sh.sweep = g;  // for the other waves, and for a later visit that finds the context still resident
            sh.peersLoaded = 1;
          }
        }
      }
      if (!solo) {
        __syncthreads();
        if (wave != 0) ok = DFCCL_UNIFORM(sh.waitOk) != 0;
      }
      if (!ok) return kRunPreempted;  // position unchanged
    }
    if (!solo) {
      g = sh.sweep;
      if (scaleKind == kScalePre) scaleV = sh.sweepScale[lane & (kMaxDirectRanks - 1)];
    }
    uniformGeom(g);

    if (tid == 0) trace(A, sh, kTrMoveBegin, 0);
    int64_t pos = l0, tilesDone = 0;
    bool finished = false;
    if (forceEvery > 0) {
      // test hook: one tile at a time, with a preemption point before each
      while (!finished) {
        __syncthreads();  // (the previous tile's ticket has been read by everybody before it is handed out again)
        if (slicesSinceLoad >= forceEvery) {
          if (tid == 0) {
            sh.stats.forcedQuits++;
            sh.dyn.gridOffset = pos;
            sh.dyn.step = 0;
            sh.dyn.wait[0] = noWait();
            sh.dyn.wait[1] = noWait();
          }
          return kRunPreempted;
        }
        sweepFoldAny(g, scaleV, sh.ticket, pos, 1, mtid, nthr, tilesDone, finished);
        slicesSinceLoad += tilesDone;
        if (tid == 0 && tilesDone > 0) {
          sh.progressed = 1;
          sh.stats.slicesMoved += (uint64_t)tilesDone;
        }
      }
    } else {
      sweepFoldAny(g, scaleV, sh.ticket, pos, INT64_MAX, mtid, nthr, tilesDone, finished);
      if (tid == 0) {
        trace(A, sh, kTrFolded, 0);
        sh.progressed = 1;
        sh.stats.slicesMoved += (uint64_t)tilesDone;
      }
    }
    // Released to the system here, while the peers are still busy, so that the completion need not wait for it.
    // Whole workgroup: the barrier orders every thread's stores before thread 0's fence.  Wave 0 alone: every
    // lane's stores are covered by the fence the wave executes together.
    if (solo) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    } else {
      __syncthreads();
    }
    if (tid == 0) {
      trace(A, sh, kTrMoveEnd, 0);
      if (!solo) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
      sh.released = 1;
      __hip_atomic_store(G(&p1[(size_t)me * C + ch]), base + (uint64_t)L, __ATOMIC_RELAXED, DFCCL_AGENT);
      trace(A, sh, kTrPosted, 1);
    }
  }

  // every chunk of my receive buffer is written, and nobody reads my send buffer any more
  if (phase != 0 && tid == 0) sh.released = 1;  // resumed here: the sweep's release was done before it was parked
  {
    const WaitDesc w0 = waitFor(&p1[ch], base + (uint64_t)L, ctrStride, n);
    bool ok = true;
    if (wave == 0) ok = waitDescs(A, sh, lane, w0, noWait(), true, threshold, slicesSinceLoad, cap).ok;
    if (!solo) {
      __syncthreads();
      if (wave != 0) ok = DFCCL_UNIFORM(sh.waitOk) != 0;
    }
    if (!ok) {
      if (tid == 0) {
        sh.dyn.gridOffset = 0;
        sh.dyn.step = 2;
      }
      return kRunPreempted;
    }
  }
  if (tid == 0) {
    sh.dyn.instance = inst + 1;
    sh.dyn.slice = 0;
  }
  return kRunDone;
}

__device__ __forceinline__ int runColl(const DaemonArgs& A, WgShared& sh, int ch, int tid, const bool solo) {
  if (solo || DFCCL_UNIFORM(sh.plan.proto) == kProtoDirect) return runDirect(A, sh, ch, tid, solo);
  return runFifo(A, sh, ch, tid);
}

// Whether wave 0 runs a collective alone (decided once per launch, from the plan): a direct collective whose whole
// share of this rank is one tile of at most kSoloMaxBytes, and no forced preemption points asked for.
__device__ __forceinline__ bool soloCollective(const DFCCL_GLOBAL CollPlan* pl, int64_t forceQuitEvery) {
  return pl->proto == kProtoDirect && pl->nChannels == 1 && pl->loopsPerInstance == 1 && forceQuitEvery == 0 &&
         pl->lastChunkElems * pl->elemSize <= kSoloMaxBytes;
}

// One thread: the resident collective has finished an instance.  Resets its position for the next instance
// (link counters and the instance number persist), posts the completion and stores the context.
// (manipulateCQ7ResetDoneColl, enqueue_ofccl_dev.cu:773-920.)
__device__ __forceinline__ void completeColl(const DaemonArgs& A, const RankDev& R, WgShared& sh, int ch, uint32_t coll) {
  sh.dyn.gridOffset = 0;
  sh.dyn.step = 0;
  sh.dyn.tryCnt = 0;
  sh.dyn.active = 0;
  if (sh.plan.proto == kProtoFifo) sh.dyn.slice = 0;
  sh.dyn.wait[0] = noWait();
  sh.dyn.wait[1] = noWait();
  sh.peersLoaded = 0;
  // results are released to the system (unless the protocol has done so already), then the last channel to
  // finish posts the entry
  if (!sh.released) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
  bool last = true;
  if (sh.plan.nChannels > 1) {
    // (with the results released already there is nothing left to write back: acquire is enough, and spares
    // the completion a walk through the L2)
    const uint64_t old = sh.released
                             ? __hip_atomic_fetch_add(G(sh.plan.doneCounter), 1ull, __ATOMIC_ACQUIRE, DFCCL_AGENT)
                             : __hip_atomic_fetch_add(G(sh.plan.doneCounter), 1ull, __ATOMIC_ACQ_REL, DFCCL_AGENT);
    last = ((old + 1) % (uint64_t)sh.plan.nChannels == 0);
  }
  if (last) {
    // a rank with a single channel has a single poster, which keeps the ticket itself
    const uint64_t t = (R.nChannels == 1) ? sh.cqNext++
                                          : __hip_atomic_fetch_add(G(R.cqTicket), 1ull, __ATOMIC_RELAXED, DFCCL_AGENT);
    const uint64_t cqe = cqeEncode((unsigned)ch, (unsigned)(t + 1), (unsigned)sh.plan.collId);
    if (sh.released) {
      __hip_atomic_store(G(&R.cq[t & (kCqRing - 1)]), cqe, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    } else {
      __hip_atomic_store(G(&R.cq[t & (kCqRing - 1)]), cqe, __ATOMIC_RELEASE, DFCCL_SYSTEM);
    }
    sh.stats.cqesWritten++;
    trace(A, sh, kTrCqePosted, coll);
  }
  storeStruct(&R.dyn[(size_t)ch * R.nColls + coll], sh.dyn);
}

// One thread, at the start of a visit: make the collective's context resident and set the visit's spin budget.
__device__ __forceinline__ void beginVisit(const DaemonArgs& A, const RankDev& R, WgShared& sh, int ch, uint32_t coll,
                                           int qi) {
  const Knobs& K = A.knobs;
  if (sh.loadedColl != (int32_t)coll) {
    loadStruct(sh.plan, &R.plans[coll]);
    loadStruct(sh.dyn, &R.dyn[(size_t)ch * R.nColls + coll]);
    sh.loadedColl = (int32_t)coll;
    sh.peersLoaded = 0;
    sh.stats.ctxLoads++;
  }
  sh.dyn.tryCnt++;
  // spin budget of this visit: BASE * min(tries, NUM_TRY); the queue head is given NUM_TRY times more
  const int64_t tries = sh.dyn.tryCnt < K.numTryTaskqHead ? sh.dyn.tryCnt : K.numTryTaskqHead;
  int64_t thr = K.baseCtxSwitchThreshold * tries;
  if (qi == 0) thr *= K.numTryTaskqHead;
  sh.threshold = thr < 1 ? 1 : thr;
  sh.waitOk = 1;
  sh.progressed = 0;
  sh.released = 0;
  sh.dyn.wait[0] = noWait();
  sh.dyn.wait[1] = noWait();
  trace(A, sh, kTrVisitBegin, coll);
}

// One thread, at the end of a visit: post the completion, or save the context.
__device__ __forceinline__ void endVisit(const DaemonArgs& A, const RankDev& R, WgShared& sh, int ch, uint32_t coll, int qi,
                                         int status) {
  if (sh.progressed) sh.progressedRound = 1;
  if (status == kRunDone) {
    sh.taskq[qi] = (uint16_t)kInvalidTask;
    completeColl(A, R, sh, ch, coll);
  } else {
    // preempted: save the context (saveExcutingCollCtx, enqueue_ofccl_dev.cu:664-677)
    storeStruct(&R.dyn[(size_t)ch * R.nColls + coll], sh.dyn);
    sh.stats.ctxSaves++;
  }
  trace(A, sh, kTrVisitEnd, (uint32_t)status);
}

// Visit one collective of the task queue: make its context resident, run it,
// then post the completion or save the context.
// `solo` (from the round's readySolo bitmap, the same in every thread): wave 0 does all of that by itself, its
// lane 0 in the part of thread 0, without a workgroup barrier from the context to the completion entry; the
// other waves touch nothing and wait at the barrier that ends the visit.
__device__ __forceinline__ void visit(const DaemonArgs& A, const RankDev& R, WgShared& sh, int ch, int tid, int wave, int qi,
                                      const bool solo) {
  const int lane = tid & 63;
  const bool first = solo ? (wave == 0 && lane == 0) : (tid == 0);  // the thread that does the bookkeeping
  uint32_t coll = 0;
  if (solo) {
    if (wave == 0) {
      if (first) {
        coll = sh.taskq[qi];
        beginVisit(A, R, sh, ch, coll, qi);
      }
      DFCCL_WAVE_LDS_SYNC();  // (the context lane 0 has put into LDS is what the other lanes read next)
    }
  } else {
    coll = DFCCL_UNIFORM((uint32_t)sh.taskq[qi]);
    if (first) beginVisit(A, R, sh, ch, coll, qi);
    __syncthreads();
  }
  int status = kRunDone;
  if (!solo || wave == 0) {  // (one call for both cases: the movers are inlined into it)
    if (first) trace(A, sh, kTrRunEntry, 0);
    status = runColl(A, sh, ch, tid, solo);
    if (first) trace(A, sh, kTrRunReturned, (uint32_t)status);
  }
  if (solo) {
    if (wave == 0) {
      DFCCL_WAVE_LDS_SYNC();
      if (first) endVisit(A, R, sh, ch, coll, qi, status);
    }
    __syncthreads();
  } else {
    __syncthreads();
    if (first) endVisit(A, R, sh, ch, coll, qi, status);
    __syncthreads();
  }
}

extern "C" __global__ __launch_bounds__(kWgThreads) void DFCCL_DAEMON_KERNEL(const DaemonArgs* __restrict__ argsPtr) {
  DFCCL_WG_SHARED(WgShared, sh);
  const DaemonArgs& A = *argsPtr;
  const int tid0 = threadIdx.x, wave = DFCCL_UNIFORM(tid0 >> 6);
  // Workgroups go to the XCDs round robin.  The channels of a rank are rotated by its slot, so that the
  // leaders (channel 0), which talk to the host, do not all sit on one XCD.
  const int slot = (int)blockIdx.x / A.channelsPerRank;
  const int ch = ((int)blockIdx.x % A.channelsPerRank + A.channelsPerRank - slot % A.channelsPerRank) % A.channelsPerRank;
  if (slot >= A.nSlots) return;
  const RankDev& R = A.ranks[slot];
  if (!R.active || ch >= R.nChannels) return;
  const Knobs& K = A.knobs;
  const uint64_t startTick = wall_clock64();

  // ---- restore the state a previous launch saved (blockInit, enqueue_ofccl_dev.cu:203-479)
  DFCCL_GLOBAL WgSaved& S = *G(&R.saved[ch]);
  Wave0Regs st;  // (see Wave0Regs: only wave 0's copy is ever used)
  st.frontier = DFCCL_WAVE_UNIFORM(S.frontier);
  st.hostFrontier = DFCCL_WAVE_UNIFORM(S.hostFrontier);
  st.publishedHead = ~0ull;
  st.idle = 0;
  st.round = 0;
  st.statsReqSeen = 0;
  st.numActive = 0;
  st.ingested = 0;
  st.allFresh = 0;
  st.rankBusy = 0;
  st.finalQuit = 0;
  st.numReady = 0;
  if (tid0 == 0) {
    sh.numActive = S.numActive;
    sh.numReady = 0;
    sh.exitKind = kExitNone;
    sh.progressedRound = 0;
    sh.loadedColl = -1;
    sh.peersLoaded = 0;
    sh.wgIndex = (uint32_t)(slot * A.channelsPerRank + ch);
    sh.traceCount = 0;
    sh.cqNext = S.cqNext;
    trace(A, sh, kTrLaunch, A.epoch);
    const DFCCL_GLOBAL WgStats* hs = G(&R.stats[ch]);
    sh.stats.sqesRead = hs->sqesRead;
    sh.stats.cqesWritten = hs->cqesWritten;
    sh.stats.ctxSaves = hs->ctxSaves;
    sh.stats.ctxLoads = hs->ctxLoads;
    sh.stats.voluntaryQuits = hs->voluntaryQuits;
    sh.stats.forcedQuits = hs->forcedQuits;
    sh.stats.slicesMoved = hs->slicesMoved;
    sh.stats.spins = hs->spins;
    sh.statsEpoch = 0;
  }
  __syncthreads();
  for (int i = tid0; i < sh.numActive; i += kWgThreads) sh.taskq[i] = S.taskq[i];
  for (int i = tid0; i < R.nColls; i += kWgThreads) {
    const DFCCL_GLOBAL CollPlan* pl = G(&R.plans[i]);
    sh.collChannels[i] = (uint8_t)((uint8_t)pl->nChannels | (soloCollective(pl, K.forceQuitEvery) ? kCollSolo : (uint8_t)0));
  }
  __syncthreads();

  for (;;) {
    // (this round's copy of the thread number: see DFCCL_FRESH_PER_ROUND)
    int tid = tid0;
    DFCCL_FRESH_PER_ROUND(tid);
    const int lane = tid & 63;
    // ---- ingest phase (wave 0; the scheduler's own state is in `st`, the same in every lane)
    if (wave == 0) {
      st.numActive = DFCCL_WAVE_UNIFORM(sh.numActive);  // (thread 0 compacts the queue at the end of a run phase)
      if (ch == 0) {
        pollHost(A, R, sh, st, lane);
      } else {
        ingestMirror(A, R, sh, st, ch, lane);
      }
      scanReady(R, sh, st, ch, lane);
      if (lane == 0 && st.ingested > 0) {
        trace(A, sh, kTrScanDone, 0);
      }
      // The round's decisions.  The host's requests and the lifetime limit are looked at every 8th round, and only
      // every 64th while submissions keep arriving: nobody waits on them, and a new submission does not wait for
      // them either.
      uint32_t abortFlag = 0, quitFlag = 0, expired = 0;
      const uint32_t round = st.round++;
      if ((round & 7u) == 0 && (st.ingested == 0 || (round & 63u) == 0)) {
        abortFlag = DFCCL_WAVE_UNIFORM(__hip_atomic_load(G(&A.devFlags[1]), __ATOMIC_RELAXED, DFCCL_AGENT));
        quitFlag = DFCCL_WAVE_UNIFORM(__hip_atomic_load(G(&A.devFlags[0]), __ATOMIC_RELAXED, DFCCL_AGENT));
        const uint32_t statsReq = DFCCL_WAVE_UNIFORM(__hip_atomic_load(G(&A.devFlags[2]), __ATOMIC_RELAXED, DFCCL_AGENT));
        if (lane == 0 && statsReq != sh.statsEpoch) {
          // the host wants the counters
          sh.statsEpoch = statsReq;
          flushStats(R, sh, ch, statsReq);
        }
        // (not in the first round of a launch: a lifetime shorter than the start-up would otherwise end every
        // launch before its first visit, and nothing would ever move)
        expired = DFCCL_WAVE_UNIFORM((uint32_t)(K.maxLifetimeTicks > 0 && round != 0 &&
                                                (int64_t)(wall_clock64() - startTick) > K.maxLifetimeTicks));
      }
      const int32_t progressedRound = DFCCL_WAVE_UNIFORM(sh.progressedRound);  // (set by thread 0 during the visits)
      DFCCL_WAVE_LDS_SYNC();  // (every lane has read it before lane 0 clears it)
      if (st.ingested > 0 || progressedRound) {
        st.idle = 0;
      } else {
        st.idle++;
      }
      if (lane == 0 && st.numActive > 0 && st.idle > 0 && (st.idle & (kStuckReportRounds - 1)) == 0) {
        reportStuck(R, sh, ch);
      }
      int exitKind = kExitNone;
      bool takeDaemonAlong = false;
      if (abortFlag) {
        exitKind = kExitAbort;
      } else if (st.finalQuit) {
        exitKind = kExitFinal;
      } else if (quitFlag || expired) {
        exitKind = kExitVoluntary;
      } else if (st.idle >= K.tolerantUnprogressedCnt) {
        // Idle for long: leave, and take the whole daemon along (every workgroup saves its state and leaves at
        // its next look at this flag).  The kernel can only be launched again once all of it has ended, and a
        // submission for a rank whose workgroups have left is not seen by anybody until then: a daemon that
        // stays half resident because other ranks are busy would starve that rank.
        exitKind = kExitVoluntary;
        takeDaemonAlong = true;
      }
      if (DFCCL_TEST_NEVER_LEAVES()) exitKind = kExitNone;
      if (lane == 0) {
        if (exitKind != kExitNone) {
          sh.exitKind = exitKind;
          if (takeDaemonAlong) __hip_atomic_store(G(&A.devFlags[0]), 1u, __ATOMIC_RELAXED, DFCCL_AGENT);
        }
        if (progressedRound) sh.progressedRound = 0;
      }
      if (st.numReady == 0 && st.ingested == 0) {
        // nothing can move: the leader's next poll is a PCIe round trip anyway, the others back off a little
        if (ch != 0) {
          __builtin_amdgcn_s_sleep(20);
        } else if (st.rankBusy) {
          __builtin_amdgcn_s_sleep(100);
        }
      }
      // A run phase follows: the scheduler's registers wait in LDS meanwhile (a dozen values that would
      // otherwise be live, and set aside lane by lane, across all of the data movement).
      if (st.numReady > 0 && exitKind == kExitNone && lane == 0) sh.w0 = st;
    }
    __syncthreads();
    // Every thread takes this round's decisions into registers, and only then may wave 0 go on to the next
    // round and overwrite them (without the second barrier a wave that is late reading numReady could see the
    // next round's value, enter the run phase alone and leave the workgroup's barriers out of step for good).
    const int roundExit = DFCCL_UNIFORM(sh.exitKind);
    const int nq = DFCCL_UNIFORM(sh.numActive);
    const int numReady = DFCCL_UNIFORM(sh.numReady);
    __syncthreads();
    if (roundExit != kExitNone) break;
    if (tid == 0 && numReady > 0) trace(A, sh, kTrRoundDecided, (uint32_t)numReady);

    // ---- run phase: visit the collectives that can move, in arrival order
    // (traverseTaskQ, enqueue_ofccl_dev.cu:922-1016)
    if (numReady > 0) {
      for (int wd = 0; wd * 64 < nq; wd++) {
        uint64_t m = DFCCL_UNIFORM(sh.ready[wd]);
        const uint64_t ms = DFCCL_UNIFORM(sh.readySolo[wd]);
        while (m) {
          const int b = (int)__builtin_ctzll(m);
          m &= m - 1;
          visit(A, R, sh, ch, tid, wave, wd * 64 + b, ((ms >> b) & 1ull) != 0);
        }
      }
      // drop finished collectives from the task queue, keeping arrival order
      if (tid == 0) {
        int w = 0;
        for (int i = 0; i < nq; i++) {
          const uint16_t c = sh.taskq[i];
          if (c != (uint16_t)kInvalidTask) sh.taskq[w++] = c;
        }
        sh.numActive = w;
      }
      __syncthreads();
      // (the other waves' copies, which nobody uses, are given new values too, so that no wave has to keep the old
      // ones across the run phase; they do not read LDS for it: wave 0 may write there again before they get here)
      if (wave == 0) {
        st.frontier = DFCCL_UNIFORM(sh.w0.frontier);
        st.hostFrontier = DFCCL_UNIFORM(sh.w0.hostFrontier);
        st.publishedHead = DFCCL_UNIFORM(sh.w0.publishedHead);
        st.idle = DFCCL_UNIFORM(sh.w0.idle);
        st.round = DFCCL_UNIFORM(sh.w0.round);
        st.statsReqSeen = DFCCL_UNIFORM(sh.w0.statsReqSeen);
        st.numActive = DFCCL_UNIFORM(sh.w0.numActive);
        st.ingested = DFCCL_UNIFORM(sh.w0.ingested);
        st.allFresh = DFCCL_UNIFORM(sh.w0.allFresh);
        st.rankBusy = DFCCL_UNIFORM(sh.w0.rankBusy);
        st.finalQuit = DFCCL_UNIFORM(sh.w0.finalQuit);
        st.numReady = DFCCL_UNIFORM(sh.w0.numReady);
      } else {
        st.frontier = st.hostFrontier = st.publishedHead = 0;
        st.idle = 0;
        st.round = st.statsReqSeen = 0;
        st.numActive = st.ingested = st.allFresh = st.rankBusy = st.finalQuit = st.numReady = 0;
      }
    }
  }

  // ---- leave
  const int exitKind = DFCCL_UNIFORM(sh.exitKind);
  if (exitKind == kExitVoluntary) {
    for (int i = tid0; i < sh.numActive; i += kWgThreads) S.taskq[i] = sh.taskq[i];
    if (tid0 == 0) {
      S.frontier = st.frontier;
      S.hostFrontier = st.hostFrontier;
      S.numActive = sh.numActive;
      S.cqNext = sh.cqNext;
      sh.stats.voluntaryQuits++;
    }
  }
  __syncthreads();
  if (tid0 == 0) {
    trace(A, sh, kTrExit, (uint32_t)exitKind);
    if (A.trace != nullptr)  // the last record slot of the workgroup holds how many records it wrote
      G(A.trace)[((size_t)sh.wgIndex * kTraceRecords + (kTraceRecords - 1)) * 2 + 1] = sh.traceCount;
    flushStats(R, sh, ch, sh.statsEpoch);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    __hip_atomic_store(G(&R.wgExit[ch]), (A.epoch << 4) | (uint32_t)exitKind, __ATOMIC_RELEASE, DFCCL_SYSTEM);
  }
}

}  // namespace dfccl

// Host-side launcher used by the runtime (kept here so that the kernel symbol
// and its launch shape live in one translation unit).
extern "C" hipError_t DFCCL_DAEMON_LAUNCH(const dfccl::DaemonArgs* devArgs, int nSlots, int channelsPerRank,
                                          hipStream_t stream) {
  const unsigned grid = (unsigned)(nSlots * channelsPerRank);
  if (grid == 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dfccl::DFCCL_DAEMON_KERNEL, dim3(grid), dim3(dfccl::kWgThreads), 0, stream, devArgs);
  return hipGetLastError();
}

// Workgroups of the daemon kernel one CU keeps resident.
extern "C" hipError_t DFCCL_DAEMON_OCCUPANCY(int* perCu) {
  return hipOccupancyMaxActiveBlocksPerMultiprocessor(perCu, dfccl::DFCCL_DAEMON_KERNEL, dfccl::kWgThreads, 0);
}
