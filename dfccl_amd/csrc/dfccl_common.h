// Data structures shared by the host runtime and the daemon kernel.
//
// Where each one lives:
//   host-coherent (fine-grained, hipHostMalloc): submission ring, its head,
//     completion ring, control word, per-workgroup exit flags and counters;
//   HBM: mirror of the submission ring, per-collective plans, per-(workgroup,
//     collective) contexts, FIFO slots and their head/tail flags, saved
//     workgroup state.
// They take the place of the reference's SQE/SQ/CQE/CQ, StaticCollCtx,
// DynamicCollCtx, BlkStatus and ncclConnInfo (src/include/collectives_ofccl.h:
// 129-157,171-183,328-355; src/include/devcomm.h:81-97).
#pragma once

#include <stdint.h>

#include "ring_schedule.h"

namespace dfccl {

constexpr int kMaxColls = 2000;      // collIds and collectives per rank context (MAX_LENGTH)
constexpr int kSqCapacity = 2000;    // submissions that may be outstanding per rank (QLen)
constexpr int kSqRing = 2048;        // ring size, a power of two >= kSqCapacity + 1
constexpr int kCqRing = 4096;        // completions can never outnumber kMaxColls in flight
#ifndef DFCCL_WG_THREADS  // (a host build of the kernels for testing may use fewer waves)
#define DFCCL_WG_THREADS 512
#endif
constexpr int kWgThreads = DFCCL_WG_THREADS;  // daemon workgroup: 8 wave64
constexpr int kMaxRankSlots = 16;    // virtual ranks one device daemon serves
constexpr int kMaxChannels = 64;     // workgroups per virtual rank
constexpr int kAlignBytes = 1024;    // chunk rounding unit: one wave's 128-bit access
constexpr int kSqeWords = 4;         // 64-bit words per submission entry
constexpr int kSqesPerPoll = 15;     // entries one wave fetches per poll (lane 60 reads the control word)
constexpr uint64_t kPtrMask = 0x0000ffffffffffffull;  // device pointers fit 48 bits
constexpr uint32_t kInvalidTask = 0xffffu;

// Submission entry in host-coherent memory: four 64-bit words, each tagged in
// its top 16 bits with (ticket + 1) & 0xffff so that a word can be validated on
// its own (the device reads the words of an entry with independent loads).
//   word 0: sendbuff | tag     word 1: recvbuff | tag
//   word 2: collIndex (32) | flags (16) | tag     word 3: tag only
constexpr uint32_t kSqeFlagQuit = 1u;

DFCCL_HD uint64_t sqeTag(uint64_t ticket) { return ((ticket + 1) & 0xffffull) << 48; }

// Control word the host writes, read by each rank's leader workgroup.
constexpr uint32_t kCtrlQuitRequest = 1u;  // save state and leave (the host will relaunch)
constexpr uint32_t kCtrlAbort = 2u;        // leave at once, state is abandoned

// How a workgroup left the kernel (written to its host-coherent exit word as
// epoch << 4 | kind, epoch = launch number).
enum ExitKind : uint32_t { kExitNone = 0, kExitVoluntary = 1, kExitFinal = 2, kExitAbort = 3, kExitUnused = 4 };

// Mirror of one submission in HBM, written by the rank's leader workgroup.
struct alignas(32) DevSqe {
  uint64_t sendbuff;
  uint64_t recvbuff;
  uint32_t coll;   // dense collective index of this rank context
  uint32_t flags;
  uint64_t ticket;
};

// Flow-control words of one FIFO (one link, one channel). tail counts slices the
// sender has published, head slices the receiver has released.
struct alignas(128) ConnFlags {
  uint64_t tail;
  uint64_t pad0[7];
  uint64_t head;
  uint64_t pad1[7];
};

// Direct protocol: what a rank's workgroup publishes when it starts an instance
// of a collective, so that its peers can read its buffers in place (the role of
// the reference's ptrExchange, src/collectives_ofccl/device/ofccl_prims_simple.h:737-869).
// Each word carries the instance it belongs to in its top 16 bits (pubTag), so a peer that polls the word
// gets the pointer with the same load that tells it the instance has started.
// `scale` is the rank's own scalar of a pre-multiplied sum (ncclAvg on float types, PreMulSum): the peer that
// folds this rank's input multiplies it by this rank's scalar, as the rank's own primitives would have.  The
// host writes it at finalize; for a scalar that lives in device memory the workgroup reads it when it announces
// an instance and stores it here before the tagged words (which it then stores with release semantics).
struct alignas(32) PeerPub {
  uint64_t send;       // sendbuff | pubTag(instance)
  uint64_t recv;       // recvbuff | pubTag(instance)
  uint64_t scale;      // one element of the run dtype in the low bytes
  uint64_t pad;
};
DFCCL_HD uint64_t pubTag(uint64_t instance) { return ((instance + 1) & 0xffffull) << 48; }

// A wait condition: all of `count` 64-bit counters at ptr, ptr + stride, ... have
// reached `value`.  Every blocking point of both protocols is expressed as (at
// most) two of these, which lets the scheduler test the readiness of a parked
// collective without loading its context.
// With kWaitTagged set in `count` the words are tagged pointers instead: the condition is that the top 16
// bits of every word have reached `value` in modular (16-bit window) order.
struct WaitDesc {
  uint64_t ptr;
  uint64_t value;
  int32_t stride;  // bytes
  int32_t count;   // 0 = no condition; may carry kWaitTagged
};
constexpr int32_t kWaitTagged = 0x10000;
DFCCL_HD bool waitReached(uint64_t word, uint64_t value, bool tagged) {
  return tagged ? (int16_t)((uint16_t)(word >> 48) - (uint16_t)value) >= 0 : word >= value;
}

enum Proto : int { kProtoFifo = 0, kProtoDirect = 1 };
constexpr int kMaxDirectRanks = 8;           // ranks whose buffers one workgroup folds in a single pass

// Immutable plan of one collective on one rank (HBM, written at finalize).
struct alignas(16) CollPlan {
  int32_t kind, dtype, op, root;
  int32_t nRanks, rank, nChannels, collId;
  int64_t count;        // elements of the run dtype (bytes for all-gather / broadcast)
  int64_t chunkElems;   // nominal chunk
  int64_t alignElems;
  int64_t sliceElems;   // nominal slice = FIFO slot capacity in elements
  int32_t slicesPerChunk, fifoSlots;
  int32_t elemSize, pad;
  int64_t slotBytes;
  int64_t fifoChanStride;  // bytes between two channels' FIFOs of one link
  char* sendFifo;          // link rank -> next, channel 0
  char* recvFifo;          // link prev -> rank, channel 0
  ConnFlags* sendFlags;    // indexed by channel
  ConnFlags* recvFlags;
  uint64_t* doneCounter;   // workgroups that finished an instance, monotonic
  // direct protocol (peers read each other's buffers, no FIFO)
  int32_t proto;
  int32_t scaleKind;       // a Sum with a scale (ncclAvg, PreMulSum): kScaleNone / kScalePre / kScalePost of reduce_ops.h
  uint64_t scaleBits;      // this rank's scalar: one element of dtype in the low bytes, or the divisor
  const void* scalePtr;    // PreMulSum with the scalar in device memory: read whenever an instance starts (else null)
  PeerPub* pubs;           // [nRanks][nChannels]
  uint64_t* p1;            // [nRanks][nChannels] loops whose own chunk is folded and stored everywhere
  int64_t loopsPerInstance;
  int64_t lastChunkElems;  // chunk size of the last loop (every other loop uses the nominal chunk)
  uint64_t* tileCtr;       // direct protocol, several channels: this rank's tile counter (see sweepFoldN)
};

// Resumable position of one collective on one workgroup (HBM). This is the
// context a preemption saves and a resume restores.
struct alignas(128) DynCtx {
  uint64_t sendbuff;
  uint64_t recvbuff;
  int64_t gridOffset;   // FIFO: first element of the loop the workgroup is in; direct: position of the sweep
  int32_t step;         // FIFO: ring step inside the loop; direct: 0 = sweep, 2 = only the final wait is left
  int32_t slice;        // FIFO: slice inside the step's chunk; direct: 1 once the instance is published
  uint64_t sendStep;    // FIFO: slices ever sent on the send link (persists across instances)
  uint64_t recvStep;    // FIFO: slices ever received on the receive link
  uint64_t instance;    // direct: instances completed (persists)
  int32_t tryCnt;       // scheduler visits since the instance started
  int32_t active;
  WaitDesc wait[2];     // what the collective is parked on (count 0: runnable)
  uint64_t pad[2];
};

// Counters of one workgroup, in host-coherent memory.  A workgroup writes them when it leaves the kernel, and
// when the host asks (the host raises the request number in the word after the control word; a workgroup that
// has written its counters for request e stores e in `epoch`).  They are not written after every collective:
// thousands of small writes over PCIe would queue up in front of the completions.
struct alignas(128) WgStats {
  uint64_t sqesRead, cqesWritten, ctxSaves, ctxLoads, voluntaryQuits, forcedQuits, slicesMoved, spins;
  uint64_t epoch;
  // Written by a workgroup that has had collectives queued without any progress for a long time (what the head
  // of its task queue is parked on), for the host to print when it gives up on a daemon:
  //   [0] reports so far  [1] collective index | step << 32 | published << 40 | queue length << 48
  //   [2] instance  [3] first wait: address  [4] value waited for | count << 48  [5] value seen at that address
  //   [6] second wait: address
  uint64_t stuck[7];
};
constexpr int64_t kStuckReportRounds = 1 << 18;  // idle rounds between two such reports

// Scheduler state a workgroup saves when it leaves voluntarily and restores at
// the next launch (HBM).
struct WgSaved {
  uint64_t frontier;      // next mirror-ring ticket to read
  uint64_t hostFrontier;  // leader only: next host-ring ticket to read
  int32_t numActive;
  int32_t finalQuit;
  uint64_t cqNext;        // single-channel ranks: next completion ticket (kept by the one workgroup that posts)
  uint16_t taskq[kMaxColls];
};

// Everything the kernel needs about one virtual rank.
struct RankDev {
  int32_t active;
  int32_t nChannels;   // workgroups this rank uses (<= grid channels)
  int32_t nColls;
  int32_t rank;
  // host-coherent
  uint64_t* sq;        // kSqRing * kSqeWords words
  uint64_t* sqHead;    // written by the leader: every workgroup has consumed tickets < *sqHead
  uint64_t* cq;        // kCqRing entries
  uint32_t* ctrl;      // control word (shared by all ranks of the daemon)
  uint32_t* wgExit;    // [kMaxChannels]
  WgStats* stats;      // [kMaxChannels]
  // HBM
  DevSqe* mirror;      // kSqRing entries
  uint64_t* mirrorTail;
  uint64_t* wgFrontier;  // [kMaxChannels]
  uint64_t* cqTicket;
  CollPlan* plans;     // [nColls]
  DynCtx* dyn;         // [kMaxChannels][nColls]
  WgSaved* saved;      // [kMaxChannels]
};

// Scheduling knobs; names and defaults are the reference's environment
// variables (src/enqueue_ofccl.cc:763,1287-1297).
struct Knobs {
  int64_t baseCtxSwitchThreshold;   // BASE_CTX_SWITCH_THRESHOLD, default 80
  int64_t numTryTaskqHead;          // NUM_TRY_TASKQ_HEAD, default 5
  int64_t recvSuccessFactor;        // RECV_SUCCESS_FACTOR, default 5
  int64_t tolerantUnprogressedCnt;  // TOLERANT_UNPROGRESSED_CNT, default 500000
  int64_t forceQuitEvery;           // DFCCL_FORCE_QUIT_EVERY: preempt after this many slices (0 = off)
  int64_t maxLifetimeTicks;         // DFCCL_DAEMON_MAX_MS in 100 MHz ticks (0 = unlimited)
  int64_t idlePollRounds;           // DFCCL_IDLE_POLL_ROUNDS: 0 switches the pipelined polling of idle leaders off
};

struct DaemonArgs {
  RankDev ranks[kMaxRankSlots];
  Knobs knobs;
  int32_t nSlots;
  int32_t channelsPerRank;
  uint32_t epoch;
  uint32_t pad;
  uint32_t* devFlags;  // HBM: [0] quit request, [1] abort (set by leaders from the control word)
  // optional timeline (DFCCL_TRACE=1): kTraceRecords records of {event | arg << 32, 100 MHz tick} per workgroup,
  // the stamps the reference takes under DEBUG_CLOCK (src/include/collectives_ofccl.h:219-299)
  uint64_t* trace;
};

constexpr int kTraceRecords = 4096;
enum TraceEvent : uint32_t {
  kTrSqeFetched = 1, kTrIngested = 2, kTrVisitBegin = 3, kTrWaitBegin = 4, kTrWaitEnd = 5, kTrMoveBegin = 6,
  kTrMoveEnd = 7, kTrPosted = 8, kTrCqePosted = 9, kTrVisitEnd = 10, kTrScanDone = 11, kTrLaunch = 12, kTrExit = 13,
  // finer stamps inside one scheduler round and one visit (what the time between the events above is spent on)
  kTrRoundDecided = 14,  // the round's decisions are taken, the run phase begins
  kTrRunEntry = 15,      // the visit's first barrier is passed, the collective's code begins
  kTrLaidOut = 16,       // direct protocol: sources and destinations of the sweep are known
  kTrFolded = 17,        // direct protocol: the sweep's loads and stores are issued (before the release)
  kTrRunReturned = 18    // the collective's code has returned to the visit
};

}  // namespace dfccl
