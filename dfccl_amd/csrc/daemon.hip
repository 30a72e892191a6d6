// The persistent daemon kernel of the DFCCL data path for gfx950.
//
// One launch serves every virtual rank of a device: workgroup (slot, channel)
// is channel `channel` of the rank context in slot `slot`.  Each workgroup runs
// the scheduler of the reference's daemonKernel
// (src/collectives_ofccl/device/enqueue_ofccl_dev.cu:1026-1483) on its own:
//
//   poll submissions -> append to the task queue -> visit every active
//   collective: load its context, run ring steps slice by slice until it is
//   done or a bounded wait expires, save the context (preemption) or post the
//   completion -> repeat; leave after a long idle period, or when told to.
//
// Differences that come from the hardware rather than from the algorithm:
//  * only the rank's leader workgroup (channel 0) reads the host-coherent
//    submission ring; one wave fetches up to 15 entries per poll (four lanes
//    per entry, each word validated by its own tag) and mirrors them into an
//    HBM ring the other channels read, so PCIe sees one poller per rank;
//  * waits are done by wave 0 with a ballot over the two flag lanes (receive
//    ready, send ready); the vote also carries the quit decision;
//  * completions go to a host-coherent ring with a device-side ticket, no
//    compare-and-swap over PCIe;
//  * the collective's plan and resumable position live in LDS while it runs.
#include <hip/hip_runtime.h>

#include "dfccl_common.h"
#include "reduce_copy_wg.h"

namespace dfccl {

constexpr int kDaemonUnroll = 1;  // see reduce_copy.hip: shallow unrolling keeps DRAM accesses ordered
enum RunStatus : int { kRunDone = 0, kRunPreempted = 1 };

struct WgShared {
  // scheduler state
  uint64_t frontier;       // next submission ticket this workgroup reads from the mirror ring
  uint64_t hostFrontier;   // leader: next ticket to fetch from the host ring (== mirror tail)
  uint64_t publishedHead;  // leader: last value written to the host's head word
  int64_t idle;            // consecutive rounds without work or progress
  int32_t numActive;
  int32_t finalQuit;
  int32_t exitKind;
  int32_t ingested;
  int32_t progressedRound;
  // collective being run
  int32_t waitOk;
  int32_t progressed;
  int32_t recvSuccess;
  int64_t threshold;
  int64_t slicesSinceLoad;
  CollPlan plan;
  DynCtx dyn;
  WgStats stats;
  uint16_t taskq[kMaxColls];
};

#define DFCCL_AGENT __HIP_MEMORY_SCOPE_AGENT
#define DFCCL_SYSTEM __HIP_MEMORY_SCOPE_SYSTEM

__device__ __forceinline__ uint64_t waveMin64(uint64_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    uint64_t other = __shfl_xor(v, o);
    v = other < v ? other : v;
  }
  return v;
}

// Writes the workgroup's counters to host-coherent memory (thread 0).
__device__ __forceinline__ void flushStats(const RankDev& R, const WgShared& sh, int ch) {
  WgStats* out = &R.stats[ch];
  __hip_atomic_store(&out->sqesRead, sh.stats.sqesRead, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->cqesWritten, sh.stats.cqesWritten, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->ctxSaves, sh.stats.ctxSaves, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->ctxLoads, sh.stats.ctxLoads, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->voluntaryQuits, sh.stats.voluntaryQuits, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->forcedQuits, sh.stats.forcedQuits, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->slicesMoved, sh.stats.slicesMoved, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  __hip_atomic_store(&out->spins, sh.stats.spins, __ATOMIC_RELAXED, DFCCL_SYSTEM);
}

// Leader, wave 0: fetch submissions from the host ring into the HBM mirror and
// pick up the host's control word.  (Role of sqRead, enqueue_ofccl_dev.cu:85-173.)
__device__ __forceinline__ void pollHost(const DaemonArgs& A, const RankDev& R, WgShared& sh, int lane) {
  const uint64_t base = sh.hostFrontier;
  uint64_t w = 0;
  bool valid = false;
  if (lane < kSqesPerPoll * kSqeWords) {
    const uint64_t ticket = base + (uint64_t)(lane >> 2);
    const uint64_t* p = R.sq + ((ticket & (kSqRing - 1)) * kSqeWords + (lane & 3));
    w = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    valid = (w & ~kPtrMask) == sqeTag(ticket);
  }
  uint32_t ctrl = 0;
  if (lane == 60) ctrl = __hip_atomic_load(R.ctrl, __ATOMIC_RELAXED, DFCCL_SYSTEM);
  ctrl = __shfl(ctrl, 60);
  if (ctrl != 0 && lane == 0) {
    if (ctrl & kCtrlQuitRequest) __hip_atomic_store(&A.devFlags[0], 1u, __ATOMIC_RELAXED, DFCCL_AGENT);
    if (ctrl & kCtrlAbort) __hip_atomic_store(&A.devFlags[1], 1u, __ATOMIC_RELAXED, DFCCL_AGENT);
  }
  const uint64_t vm = __ballot(valid);
  int n = 0;
  while (n < kSqesPerPoll && ((vm >> (4 * n)) & 0xfull) == 0xfull) n++;
  if (n > 0) {
    const int first = lane & ~3;
    const uint64_t w1 = __shfl(w, first + 1);
    const uint64_t w2 = __shfl(w, first + 2);
    if ((lane & 3) == 0 && (lane >> 2) < n) {
      const uint64_t ticket = base + (uint64_t)(lane >> 2);
      DevSqe* e = &R.mirror[ticket & (kSqRing - 1)];
      e->sendbuff = w & kPtrMask;
      e->recvbuff = w1 & kPtrMask;
      e->coll = (uint32_t)(w2 & 0xffffffffull);
      e->flags = (uint32_t)((w2 >> 32) & 0xffffull);
      e->ticket = ticket;
    }
    // every lane's entry is written before lane 0 publishes the new tail
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    if (lane == 0) {
      __hip_atomic_store(R.mirrorTail, base + (uint64_t)n, __ATOMIC_RELEASE, DFCCL_AGENT);
      sh.hostFrontier = base + (uint64_t)n;
    }
  }
  // the host may reuse entries every workgroup of the rank has consumed
  uint64_t f = ~0ull;
  if (lane < R.nChannels) f = __hip_atomic_load(&R.wgFrontier[lane], __ATOMIC_RELAXED, DFCCL_AGENT);
  f = waveMin64(f);
  if (lane == 0 && f != sh.publishedHead) {
    __hip_atomic_store(R.sqHead, f, __ATOMIC_RELAXED, DFCCL_SYSTEM);
    sh.publishedHead = f;
  }
}

// Wave 0 of every workgroup: take new entries from the mirror ring, one lane per
// entry, and append the collectives this channel takes part in to the task queue.
// (Role of checkSQ7TidyTaskQ, enqueue_ofccl_dev.cu:491-627.)
__device__ __forceinline__ void ingest(const RankDev& R, WgShared& sh, int ch, int lane) {
  const uint64_t f = sh.frontier;
  const uint64_t tail = __hip_atomic_load(R.mirrorTail, __ATOMIC_ACQUIRE, DFCCL_AGENT);
  const int avail = (int)((tail - f) < 64 ? (tail - f) : 64);
  if (avail <= 0) {
    if (lane == 0) sh.ingested = 0;
    return;
  }
  // buffers named by the new entries may have been written by the host, a copy
  // engine or another kernel before the submission
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
  DevSqe e;
  e.sendbuff = e.recvbuff = 0;
  e.coll = 0;
  e.flags = 0;
  bool isQuit = false, mine = false;
  if (lane < avail) {
    e = R.mirror[(f + (uint64_t)lane) & (kSqRing - 1)];
    isQuit = (e.flags & kSqeFlagQuit) != 0;
    if (!isQuit && e.coll < (uint32_t)R.nColls) mine = ch < R.plans[e.coll].nChannels;
  }
  const uint64_t qm = __ballot(isQuit);
  const int q = qm ? (int)__builtin_ctzll(qm) : 64;
  const int take = avail < q ? avail : q;
  const uint64_t mm = __ballot(mine && lane < take);
  const int pos = __builtin_popcountll(mm & ((1ull << lane) - 1ull));
  const int base = sh.numActive;
  if (mine && lane < take && base + pos < kMaxColls) {
    DynCtx* d = &R.dyn[(size_t)ch * R.nColls + e.coll];
    d->sendbuff = e.sendbuff;
    d->recvbuff = e.recvbuff;
    d->active = 1;
    sh.taskq[base + pos] = (uint16_t)e.coll;
  }
  if (lane == 0) {
    const int added = __builtin_popcountll(mm);
    sh.numActive = base + added;
    const int consumed = take + (q < avail ? 1 : 0);
    sh.frontier = f + (uint64_t)consumed;
    if (q < avail) sh.finalQuit = 1;
    sh.ingested = consumed;
    sh.stats.sqesRead += (uint64_t)consumed;
    __hip_atomic_store(&R.wgFrontier[ch], f + (uint64_t)consumed, __ATOMIC_RELAXED, DFCCL_AGENT);
  }
}

// Wave 0: wait until the receive slot is filled and / or a send slot is free.
// Lane 0 watches the receive link's tail, lane 1 the send link's head; the
// ballot decides for the whole wave.  The wait is bounded: when the budget is
// spent the collective is preempted.  (Role of waitPeer,
// src/collectives_ofccl/device/ofccl_prims_simple.h:90-198.)
__device__ __forceinline__ void waitPeer(const DaemonArgs& A, WgShared& sh, int ch, int lane, bool recv, bool send,
                                         uint64_t recvStep, uint64_t sendStep) {
  const CollPlan& P = sh.plan;
  bool ok;
  int64_t spins = 0;
  const int64_t forceEvery = A.knobs.forceQuitEvery;
  if (forceEvery > 0 && sh.slicesSinceLoad >= forceEvery) {
    ok = false;
    if (lane == 0) sh.stats.forcedQuits++;
  } else {
    const uint64_t* p = nullptr;
    if (lane == 0 && recv) p = &P.recvFlags[ch].tail;
    if (lane == 1 && send) p = &P.sendFlags[ch].head;
    bool ready = (p == nullptr);
    const int64_t threshold = sh.threshold;
    for (;;) {
      if (!ready) {
        const uint64_t v = __hip_atomic_load(p, __ATOMIC_RELAXED, DFCCL_AGENT);
        ready = (lane == 0) ? (v >= recvStep + 1) : (v + (uint64_t)P.fifoSlots >= sendStep + 1);
      }
      if (__ballot(!ready) == 0) { ok = true; break; }
      if (++spins >= threshold) { ok = false; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    if (ok) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  if (lane == 0) {
    sh.waitOk = ok ? 1 : 0;
    sh.stats.spins += (uint64_t)spins;
    if (ok && recv) {
      sh.recvSuccess = 1;
      const int64_t t = A.knobs.recvSuccessFactor * spins;
      if (t > sh.threshold) sh.threshold = t;
    }
  }
}

template <int DT, int OP>
__device__ __forceinline__ void moveReduce(const void* s0, const void* s1, void* d0, void* d1, size_t nbytes, int tid) {
  const void* s[2] = {s0, s1};
  if (d1 != nullptr) {
    void* d[2] = {d0, d1};
    reduceCopyWG<DT, OP, 2, 2, kDaemonUnroll, false>(s, d, nbytes, tid, kWgThreads);
  } else {
    void* d[1] = {d0};
    reduceCopyWG<DT, OP, 2, 1, kDaemonUnroll, false>(s, d, nbytes, tid, kWgThreads);
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

// One slice: 1 or 2 sources into 1 or 2 destinations (d1 may be null).
__device__ __forceinline__ void moveSlice(int dtype, int op, const void* s0, const void* s1, void* d0, void* d1,
                                          size_t nbytes, int tid) {
  if (s1 == nullptr) {
    const void* s[1] = {s0};
    if (d1 != nullptr) {
      void* d[2] = {d0, d1};
      reduceCopyWG<kI8, kSum, 1, 2, kDaemonUnroll, false>(s, d, nbytes, tid, kWgThreads);
    } else {
      void* d[1] = {d0};
      reduceCopyWG<kI8, kSum, 1, 1, kDaemonUnroll, false>(s, d, nbytes, tid, kWgThreads);
    }
    return;
  }
  switch (dtype) {
    case kF32: moveReduceOp<kF32>(op, s0, s1, d0, d1, nbytes, tid); break;
    case kBF16: moveReduceOp<kBF16>(op, s0, s1, d0, d1, nbytes, tid); break;
    case kF16: moveReduceOp<kF16>(op, s0, s1, d0, d1, nbytes, tid); break;
    case kI32: moveReduceOp<kI32>(op, s0, s1, d0, d1, nbytes, tid); break;
    default: moveReduceOp<kI8>(op, s0, s1, d0, d1, nbytes, tid); break;
  }
}

// Runs the loaded collective from its saved position until it is done or a wait
// expires.  Every thread takes the same path: all decisions come from LDS after
// a barrier.  (Role of the resumable runRing bodies and genericOp; see
// ring_schedule.h for the per-step roles.)
__device__ __forceinline__ int runColl(const DaemonArgs& A, WgShared& sh, int ch, int tid) {
  const CollPlan& P = sh.plan;
  const int lane = tid & 63, wave = tid >> 6;
  const int kind = P.kind, n = P.nRanks, C = P.nChannels, es = P.elemSize;
  const int64_t count = P.count;
  const int64_t loop = loopElems(kind, n, C, P.chunkElems);
  const int nsteps = stepsPerLoop(kind, n);
  const char* sendbuff = (const char*)sh.dyn.sendbuff;
  char* recvbuff = (char*)sh.dyn.recvbuff;
  char* sendFifo = P.sendFifo + (int64_t)ch * P.fifoChanStride;
  const char* recvFifo = P.recvFifo + (int64_t)ch * P.fifoChanStride;
  int inPlace;
  if (kind == kAllGather) inPlace = (sendbuff == recvbuff + (int64_t)P.rank * count * es);
  else inPlace = (sendbuff == recvbuff);

  int64_t grid = sh.dyn.gridOffset;
  int step0 = sh.dyn.step, slice0 = sh.dyn.slice;
  uint64_t sendStep = sh.dyn.sendStep, recvStep = sh.dyn.recvStep;

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
          if (wave == 0) waitPeer(A, sh, ch, lane, d.recv != 0, d.send != 0, recvStep, sendStep);
          __syncthreads();
          if (!sh.waitOk) {
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
        if (d.useIn) { s0 = sendbuff + (d.inOff + off) * es; s1 = fifoIn; }
        else s0 = fifoIn;
        if (d.useOut) { d0 = recvbuff + (d.outOff + off) * es; d1 = fifoOut; }
        else d0 = fifoOut;
        if (s0 != nullptr && d0 != nullptr) moveSlice(P.dtype, P.op, s0, s1, d0, d1, (size_t)(len * es), tid);
        if (d.recv || d.send) {
          __syncthreads();  // every thread's loads and stores of this slice are done
          if (tid == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            if (d.send) __hip_atomic_store(&P.sendFlags[ch].tail, sendStep + 1, __ATOMIC_RELAXED, DFCCL_AGENT);
            if (d.recv) __hip_atomic_store(&P.recvFlags[ch].head, recvStep + 1, __ATOMIC_RELAXED, DFCCL_AGENT);
            sh.progressed = 1;
            sh.slicesSinceLoad++;
            sh.stats.slicesMoved++;
          }
          sendStep += d.send ? 1 : 0;
          recvStep += d.recv ? 1 : 0;
        } else if (tid == 0) {
          sh.progressed = 1;
          sh.stats.slicesMoved++;
        }
      }
    }
  }
  if (tid == 0) {
    sh.dyn.sendStep = sendStep;
    sh.dyn.recvStep = recvStep;
  }
  return kRunDone;
}

extern "C" __global__ __launch_bounds__(kWgThreads) void dfcclDaemonKernel(const DaemonArgs* __restrict__ argsPtr) {
  __shared__ WgShared sh;
  const DaemonArgs& A = *argsPtr;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = (int)blockIdx.x / A.channelsPerRank;
  const int ch = (int)blockIdx.x % A.channelsPerRank;
  if (slot >= A.nSlots) return;
  const RankDev& R = A.ranks[slot];
  if (!R.active || ch >= R.nChannels) return;
  const Knobs& K = A.knobs;
  const uint64_t startTick = wall_clock64();

  // ---- restore the state a previous launch saved (blockInit, enqueue_ofccl_dev.cu:203-479)
  WgSaved& S = R.saved[ch];
  if (tid == 0) {
    sh.frontier = S.frontier;
    sh.hostFrontier = S.hostFrontier;
    sh.publishedHead = ~0ull;
    sh.numActive = S.numActive;
    sh.finalQuit = 0;
    sh.exitKind = kExitNone;
    sh.idle = 0;
    sh.ingested = 0;
    sh.progressedRound = 0;
    const WgStats* hs = &R.stats[ch];
    sh.stats.sqesRead = hs->sqesRead;
    sh.stats.cqesWritten = hs->cqesWritten;
    sh.stats.ctxSaves = hs->ctxSaves;
    sh.stats.ctxLoads = hs->ctxLoads;
    sh.stats.voluntaryQuits = hs->voluntaryQuits;
    sh.stats.forcedQuits = hs->forcedQuits;
    sh.stats.slicesMoved = hs->slicesMoved;
    sh.stats.spins = hs->spins;
  }
  __syncthreads();
  for (int i = tid; i < sh.numActive; i += kWgThreads) sh.taskq[i] = S.taskq[i];
  __syncthreads();

  for (;;) {
    // ---- ingest phase (wave 0)
    if (wave == 0) {
      if (ch == 0) pollHost(A, R, sh, lane);
      ingest(R, sh, ch, lane);
      if (lane == 0) {
        const uint32_t abortFlag = __hip_atomic_load(&A.devFlags[1], __ATOMIC_RELAXED, DFCCL_AGENT);
        const uint32_t quitFlag = __hip_atomic_load(&A.devFlags[0], __ATOMIC_RELAXED, DFCCL_AGENT);
        const bool expired = K.maxLifetimeTicks > 0 && (int64_t)(wall_clock64() - startTick) > K.maxLifetimeTicks;
        if (sh.ingested > 0 || sh.progressedRound) sh.idle = 0;
        else sh.idle++;
        if (abortFlag) sh.exitKind = kExitAbort;
        else if (sh.finalQuit) sh.exitKind = kExitFinal;
        else if (quitFlag || expired) sh.exitKind = kExitVoluntary;
        else if (sh.idle >= K.tolerantUnprogressedCnt) sh.exitKind = kExitVoluntary;
        sh.progressedRound = 0;
      }
      if (sh.numActive == 0 && sh.ingested == 0) {
        // nothing to do: the leader's next poll is a PCIe round trip anyway, the others back off a little
        if (ch == 0) __builtin_amdgcn_s_sleep(2);
        else __builtin_amdgcn_s_sleep(20);
      }
    }
    __syncthreads();
    if (sh.exitKind != kExitNone) break;

    // ---- run phase: visit every active collective once (traverseTaskQ, enqueue_ofccl_dev.cu:922-1016)
    const int nq = sh.numActive;
    for (int qi = 0; qi < nq; qi++) {
      const uint32_t coll = sh.taskq[qi];
      DynCtx* dynG = &R.dyn[(size_t)ch * R.nColls + coll];
      if (tid == 0) {
        sh.plan = R.plans[coll];
        sh.dyn = *dynG;
        sh.dyn.tryCnt++;
        // spin budget of this visit: BASE * min(tries, NUM_TRY), the queue head is given NUM_TRY times more
        const int64_t tries = sh.dyn.tryCnt < K.numTryTaskqHead ? sh.dyn.tryCnt : K.numTryTaskqHead;
        int64_t thr = K.baseCtxSwitchThreshold * tries;
        if (qi == 0) thr *= K.numTryTaskqHead;
        sh.threshold = thr < 1 ? 1 : thr;
        sh.waitOk = 1;
        sh.progressed = 0;
        sh.recvSuccess = 0;
        sh.slicesSinceLoad = 0;
        sh.stats.ctxLoads++;
      }
      __syncthreads();
      const int status = runColl(A, sh, ch, tid);
      __syncthreads();
      if (tid == 0) {
        if (sh.progressed) sh.progressedRound = 1;
        if (status == kRunDone) {
          // reset the position for the next instance; the link counters persist
          dynG->gridOffset = 0;
          dynG->step = 0;
          dynG->slice = 0;
          dynG->tryCnt = 0;
          dynG->active = 0;
          dynG->sendStep = sh.dyn.sendStep;
          dynG->recvStep = sh.dyn.recvStep;
          sh.taskq[qi] = (uint16_t)kInvalidTask;
          // completion (manipulateCQ7ResetDoneColl, enqueue_ofccl_dev.cu:773-920): the
          // last channel to finish posts the entry; results are released to the system first
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
          const uint64_t old = __hip_atomic_fetch_add(sh.plan.doneCounter, 1ull, __ATOMIC_ACQ_REL, DFCCL_AGENT);
          if ((old + 1) % (uint64_t)sh.plan.nChannels == 0) {
            const uint64_t t = __hip_atomic_fetch_add(R.cqTicket, 1ull, __ATOMIC_RELAXED, DFCCL_AGENT);
            sh.stats.cqesWritten++;
            flushStats(R, sh, ch);
            __hip_atomic_store(&R.cq[t & (kCqRing - 1)],
                               cqeEncode((unsigned)ch, (unsigned)(t + 1), (unsigned)sh.plan.collId), __ATOMIC_RELEASE,
                               DFCCL_SYSTEM);
          } else {
            flushStats(R, sh, ch);
          }
        } else {
          // preempted: save the context (saveExcutingCollCtx, enqueue_ofccl_dev.cu:664-677)
          dynG->gridOffset = sh.dyn.gridOffset;
          dynG->step = sh.dyn.step;
          dynG->slice = sh.dyn.slice;
          dynG->sendStep = sh.dyn.sendStep;
          dynG->recvStep = sh.dyn.recvStep;
          dynG->tryCnt = sh.dyn.tryCnt;
          sh.stats.ctxSaves++;
        }
      }
      __syncthreads();
    }
    // ---- drop finished collectives from the task queue, keeping arrival order
    if (tid == 0 && nq > 0) {
      int w = 0;
      const int total = sh.numActive;
      for (int i = 0; i < total; i++) {
        const uint16_t c = sh.taskq[i];
        if (c != (uint16_t)kInvalidTask) sh.taskq[w++] = c;
      }
      sh.numActive = w;
    }
    __syncthreads();
  }

  // ---- leave
  const int exitKind = sh.exitKind;
  if (exitKind == kExitVoluntary) {
    for (int i = tid; i < sh.numActive; i += kWgThreads) S.taskq[i] = sh.taskq[i];
    if (tid == 0) {
      S.frontier = sh.frontier;
      S.hostFrontier = sh.hostFrontier;
      S.numActive = sh.numActive;
      sh.stats.voluntaryQuits++;
    }
  }
  __syncthreads();
  if (tid == 0) {
    flushStats(R, sh, ch);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    __hip_atomic_store(&R.wgExit[ch], (A.epoch << 4) | (uint32_t)exitKind, __ATOMIC_RELEASE, DFCCL_SYSTEM);
  }
}

}  // namespace dfccl

// Host-side launcher used by the runtime (kept here so that the kernel symbol
// and its launch shape live in one translation unit).
extern "C" hipError_t dfcclLaunchDaemon(const dfccl::DaemonArgs* devArgs, int nSlots, int channelsPerRank,
                                        hipStream_t stream) {
  const unsigned grid = (unsigned)(nSlots * channelsPerRank);
  if (grid == 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dfccl::dfcclDaemonKernel, dim3(grid), dim3(dfccl::kWgThreads), 0, stream, devArgs);
  return hipGetLastError();
}
