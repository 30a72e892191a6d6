// Host runtime of the DFCCL data path: rank contexts, virtual communicators,
// submission / completion queues, the per-device daemon launcher ("observer")
// and the per-rank completion poller.  Mirrors src/enqueue_ofccl.cc of the
// reference (rank context :751, prepare :773, finalize :1285, sqWrite :616,
// cqRead :697, poller :908, observer :967, destroy :1582) and the shims in
// src/collectives_ofccl/ofccl_*.cc, over the HIP runtime.
//
// One daemon kernel serves all rank contexts of a device (they are virtual
// ranks sharing one GPU), so the daemon object is per device and rank contexts
// attach to one of its slots.
#include <hip/hip_runtime.h>
#include <immintrin.h>
#include <sched.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

#include "../../include/ofccl.h"
#include "avg_scale.h"
#include "dfccl_common.h"

#define DFCCL_API extern "C" __attribute__((visibility("default")))

// daemon.hip is compiled twice: the kernel that normally runs, and one that also writes the timeline stamps
// (launched when DFCCL_TRACE=1)
extern "C" hipError_t dfcclDaemonOccupancy(int* perCu);
extern "C" hipError_t dfcclDaemonOccupancyTraced(int* perCu);
extern "C" hipError_t dfcclLaunchDaemon(const dfccl::DaemonArgs* devArgs, int nSlots, int channelsPerRank,
                                        hipStream_t stream);
extern "C" hipError_t dfcclLaunchDaemonTraced(const dfccl::DaemonArgs* devArgs, int nSlots, int channelsPerRank,
                                              hipStream_t stream);

namespace dfccl {

#define HIPCHECK(call)                                                                                  \
  do {                                                                                                  \
    hipError_t e_ = (call);                                                                             \
    if (e_ != hipSuccess) {                                                                             \
      fprintf(stderr, "dfccl: %s failed: %s (%s:%d)\n", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
      return ncclUnhandledCudaError;                                                                    \
    }                                                                                                   \
  } while (0)

static inline uint64_t nowNs() {
  return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
             std::chrono::steady_clock::now().time_since_epoch()).count();
}

static int64_t envInt(const char* name, int64_t dflt) {
  const char* v = getenv(name);
  if (v == nullptr || *v == 0) return dflt;
  char* end = nullptr;
  long long x = strtoll(v, &end, 10);
  return (end == v) ? dflt : (int64_t)x;
}

static int typeSizeOf(int dt) {
  switch (dt) {
    case ncclInt8: case ncclUint8: return 1;
    case ncclFloat16: case ncclBfloat16: return 2;
    case ncclInt32: case ncclUint32: case ncclFloat32: return 4;
    case ncclInt64: case ncclUint64: case ncclFloat64: return 8;
    default: return 0;
  }
}

// ------------------------------------------------------------------ communicators

struct CommGroup {
  uint64_t id = 0;
  int nRanks = 0;
  int device = 0;
  std::mutex mu;
  int handles = 0;
  // the collective this communicator serves, fixed by the first Prepare
  bool planned = false;
  // a rank context that ran this collective has been destroyed: the counters in the group's device memory no
  // longer match a fresh context's, so the communicator cannot be registered again
  bool retired = false;
  bool capacityUnknown = false;  // the device would not say how many workgroups it keeps resident (planGroup)
  int kind = 0, dtypeUser = 0, op = 0, root = 0;  // op: the element op the kernels apply (Sum for the scaled sums)
  int scaleKind = kScaleNone;                      // ncclAvg / PreMulSum: see Scale in reduce_ops.h
  // every rank's own scalar (a PreMulSum operator is made per rank, and a rank's input is multiplied by that
  // rank's scalar): the bits of one element, or for an operator made with ncclScalarDevice the device address
  // the scalar is read from whenever an instance starts.  Set by each rank's Prepare.
  std::vector<uint64_t> scaleBits, scalePtr;
  size_t countUser = 0;
  // derived plan
  int dtype = 0, elemSize = 1, nChannels = 1, slicesPerChunk = 1, fifoSlots = 1;
  int64_t count = 0, chunkElems = 0, alignElems = 0, sliceElems = 0, slotBytes = 0, chanStride = 0;
  // device memory: [nRanks links][nChannels] FIFOs and flags; link r goes from rank r to rank (r+1)%n
  char* fifo = nullptr;
  ConnFlags* flags = nullptr;
  // direct protocol
  int proto = kProtoFifo;
  int64_t loopsPerInstance = 0, lastChunkElems = 0;
  PeerPub* pubs = nullptr;   // [nRanks][nChannels]
  uint64_t* p1 = nullptr;        // [nRanks][nChannels]
  uint64_t* tileCtrs = nullptr;  // [nRanks] x 128 bytes
};

}  // namespace dfccl

struct ncclComm {
  dfccl::CommGroup* group;
  int rank;
  bool registered;
  // reduction operators made by ncclRedOpCreatePreMulSum: op value - ncclNumOps -> the datatype and the scalar
  // (its bits, or the device address it is to be read from)
  struct UserOp {
    int datatype;
    uint64_t bits;
    uint64_t devPtr;
  };
  std::map<int, UserOp> userOps;
  int nextUserOp = 0;
};

namespace dfccl {

static std::mutex gCommMu;
static std::unordered_map<uint64_t, CommGroup*> gGroups;
static std::atomic<uint64_t> gNextCommId{1};

struct Daemon;
static int deviceWorkgroupSlots(int device);

struct CollReg {
  int collId;
  ncclComm* comm;
};

}  // namespace dfccl

struct ofcclRankCtx {
  int rank = 0;
  int device = 0;
  std::vector<dfccl::CollReg> colls;
  int16_t collIndex[dfccl::kMaxColls];
  bool finalized = false;
  dfccl::Daemon* daemon = nullptr;
  int slot = -1;
  int nChannels = 1;
  dfccl::RankDev dev{};
  uint64_t* doneCounters = nullptr;
  // submission side
  std::mutex sqMu;
  uint64_t sqTail = 0;
  uint64_t sqCapacity = dfccl::kSqCapacity;  // entries that may be outstanding (DFCCL_SQ_CAPACITY lowers it, for tests)
  // completion side
  uint64_t cqRead = 0;
  CallbackFunc callbacks[dfccl::kMaxColls];
  void* cbArgs[dfccl::kMaxColls];
  std::atomic<int> inflight[dfccl::kMaxColls];
  uint64_t submitNs[dfccl::kMaxColls];    // steady-clock time the last instance was queued
  uint64_t completeNs[dfccl::kMaxColls];  // steady-clock time its completion entry was seen by the poller
  std::atomic<uint64_t> submitted{0}, completed{0};
  std::atomic<uint64_t> sqFullSpins{0};  // times a Run found the submission ring full and had to wait
  std::thread poller;
  std::atomic<bool> stopPoller{false};
  std::atomic<bool> pollerAsleep{false};
  std::mutex pollMu;
  std::condition_variable pollCv;
};

namespace dfccl {

// ------------------------------------------------------------------------ daemon

struct Daemon {
  int device = 0;
  hipStream_t stream = nullptr;
  hipEvent_t doneEv = nullptr;
  std::mutex mu;
  std::condition_variable cv;
  ofcclRankCtx* slots[kMaxRankSlots] = {};
  int nActive = 0;
  bool running = false;
  bool shutdown = false;
  bool launchRequested = false;
  std::atomic<bool> failed{false};  // launch failed or the kernel had to be aborted: never launched again
  uint32_t epoch = 0;
  uint64_t launches = 0;
  long capacity = 0;
  uint32_t* ctrl = nullptr;      // host-coherent: [0] control word, [1] request number for the counters
  uint32_t statsEpoch = 0;
  uint32_t* devFlags = nullptr;  // HBM
  DaemonArgs* devArgs = nullptr; // HBM
  DaemonArgs hostArgs{};
  uint64_t* trace = nullptr;     // HBM, only with DFCCL_TRACE=1
  Knobs knobs{};
  std::thread observer;
  std::vector<void*> garbageDev, garbageHost;

  // Workgroups of the daemon kernel the device can hold at once: all of them must be resident, because a
  // workgroup that is not resident cannot answer its peers.
  long residentCapacity() {
    if (capacity > 0) return capacity;
    // every workgroup of the daemon has to be resident at the same time (they wait for each other): the grid
    // may not exceed what the occupancy calculation says fits the GPU (one 512-thread workgroup per CU while
    // the kernel needs more than 128 VGPRs per lane)
    capacity = deviceWorkgroupSlots(device);
    return capacity;
  }

  bool wantLaunch() const {
    if (launchRequested) return true;
    for (int s = 0; s < kMaxRankSlots; s++) {
      const ofcclRankCtx* c = slots[s];
      if (c && c->submitted.load(std::memory_order_acquire) > c->completed.load(std::memory_order_acquire)) return true;
    }
    return false;
  }

  void collectGarbage() {  // only while the kernel is not running: hipFree waits for the device
    for (void* p : garbageDev) (void)hipFree(p);
    for (void* p : garbageHost) (void)hipHostFree(p);
    garbageDev.clear();
    garbageHost.clear();
  }

  void readKnobs() {
    knobs.baseCtxSwitchThreshold = envInt("BASE_CTX_SWITCH_THRESHOLD", 80);
    knobs.numTryTaskqHead = envInt("NUM_TRY_TASKQ_HEAD", 5);
    knobs.recvSuccessFactor = envInt("RECV_SUCCESS_FACTOR", 5);
    knobs.tolerantUnprogressedCnt = envInt("TOLERANT_UNPROGRESSED_CNT", 500000);
    knobs.forceQuitEvery = envInt("DFCCL_FORCE_QUIT_EVERY", 0);
    knobs.maxLifetimeTicks = envInt("DFCCL_DAEMON_MAX_MS", 0) * 100000;  // wall_clock64 runs at 100 MHz
    knobs.idlePollRounds = envInt("DFCCL_IDLE_POLL_ROUNDS", 8);
    if (knobs.numTryTaskqHead < 1) knobs.numTryTaskqHead = 1;
    if (knobs.tolerantUnprogressedCnt < 1) knobs.tolerantUnprogressedCnt = 1;
  }

  // Launches the kernel for the current set of slots. Caller holds mu; the kernel is not running.
  bool launchLocked() {
    int nSlots = 0, chans = 1;
    memset(&hostArgs, 0, sizeof(hostArgs));
    for (int s = 0; s < kMaxRankSlots; s++) {
      if (slots[s] == nullptr) continue;
      hostArgs.ranks[s] = slots[s]->dev;
      hostArgs.ranks[s].active = 1;
      nSlots = s + 1;
      if (slots[s]->nChannels > chans) chans = slots[s]->nChannels;
    }
    if (nSlots == 0) return false;
    // a multiple of 8 channels keeps channel c of every rank on XCD c % 8
    if (chans > 1) chans = (chans + 7) & ~7;
    if (residentCapacity() <= 0) {
      fprintf(stderr, "dfccl: cannot tell how many daemon workgroups device %d keeps resident\n", device);
      return false;
    }
    if ((long)nSlots * chans > residentCapacity()) {
      fprintf(stderr,
              "dfccl: %d rank slots x %d channels do not fit the %ld workgroups the GPU keeps resident; "
              "lower NCCL_MAX_NCHANNELS\n", nSlots, chans, residentCapacity());
      return false;
    }
    epoch++;
    hostArgs.knobs = knobs;
    hostArgs.nSlots = nSlots;
    hostArgs.channelsPerRank = chans;
    hostArgs.epoch = epoch;
    hostArgs.devFlags = devFlags;
    hostArgs.trace = trace;
    __atomic_store_n(ctrl, 0u, __ATOMIC_RELEASE);
    if (hipMemcpy(devArgs, &hostArgs, sizeof(hostArgs), hipMemcpyHostToDevice) != hipSuccess) return false;
    if (hipMemset(devFlags, 0, 64) != hipSuccess) return false;
    if (hipStreamSynchronize(nullptr) != hipSuccess) return false;  // args and flags are in place before the launch
    if ((trace != nullptr ? dfcclLaunchDaemonTraced : dfcclLaunchDaemon)(devArgs, nSlots, chans, stream) != hipSuccess)
      return false;
    if (hipEventRecord(doneEv, stream) != hipSuccess) return false;
    running = true;
    launches++;
    return true;
  }

  // (Re)launches the kernel whenever work is outstanding and it is not running
  // (startKernel7SqObserver, src/enqueue_ofccl.cc:967-985).
  void observerLoop() {
    (void)hipSetDevice(device);
    std::unique_lock<std::mutex> lk(mu);
    for (;;) {
      cv.wait(lk, [&] { return shutdown || (!failed && wantLaunch()); });
      if (shutdown) break;
      launchRequested = false;
      if (!launchLocked()) {
        fprintf(stderr, "dfccl: daemon launch failed on device %d: %s\n", device, hipGetErrorString(hipGetLastError()));
        failed = true;
        cv.notify_all();
        continue;
      }
      cv.notify_all();
      lk.unlock();
      hipError_t e = hipEventSynchronize(doneEv);
      lk.lock();
      running = false;
      if (e != hipSuccess) {
        fprintf(stderr, "dfccl: daemon kernel ended with %s\n", hipGetErrorString(e));
        failed = true;
      }
      collectGarbage();
      cv.notify_all();
    }
  }

  // Asks a running kernel to save its state and leave; returns once it has. Caller holds lk.
  void quiesceLocked(std::unique_lock<std::mutex>& lk) {
    if (!running) return;
    __atomic_store_n(ctrl, kCtrlQuitRequest, __ATOMIC_RELEASE);
    if (!cv.wait_for(lk, std::chrono::seconds(20), [&] { return !running; })) {
      fprintf(stderr, "dfccl: daemon did not leave on request, aborting it\n");
      failed = true;  // the aborted kernel's state is abandoned: no relaunch
      __atomic_store_n(ctrl, kCtrlAbort, __ATOMIC_RELEASE);
      cv.wait_for(lk, std::chrono::milliseconds(abortWaitMs()), [&] { return !running; });
    }
  }
  // how long an aborted kernel is given to leave (DFCCL_ABORT_WAIT_MS is for tests)
  static int64_t abortWaitMs() { return std::max<int64_t>(1, envInt("DFCCL_ABORT_WAIT_MS", 10000)); }
};

// What the host knows about every attached rank, printed before a daemon is aborted (caller holds d->mu).
static void dumpDaemonState(const Daemon* d) {
  fprintf(stderr, "dfccl: daemon on device %d: launch %u, %s\n", d->device, d->epoch, d->running ? "resident" : "not resident");
  for (int s = 0; s < kMaxRankSlots; s++) {
    const ofcclRankCtx* c = d->slots[s];
    if (c == nullptr) continue;
    fprintf(stderr, "dfccl:   slot %d rank %d: %llu submitted, %llu completed, %d channels; exit words (launch:kind)", s,
            c->rank, (unsigned long long)c->submitted.load(), (unsigned long long)c->completed.load(), c->nChannels);
    for (int ch = 0; ch < c->nChannels; ch++) {
      const uint32_t w = __atomic_load_n(&c->dev.wgExit[ch], __ATOMIC_ACQUIRE);
      fprintf(stderr, " %u:%u", w >> 4, w & 0xf);
    }
    fprintf(stderr, "\n");
    for (size_t i = 0; i < c->colls.size(); i++)
      if (c->inflight[c->colls[i].collId].load() != 0)
        fprintf(stderr, "dfccl:     collective %d (index %zu) in flight\n", c->colls[i].collId, i);
    for (int ch = 0; ch < c->nChannels; ch++) {
      const WgStats* st = &c->dev.stats[ch];
      if (__atomic_load_n(&st->stuck[0], __ATOMIC_ACQUIRE) == 0) continue;
      const uint64_t w1 = st->stuck[1], w4 = st->stuck[4];
      fprintf(stderr, "dfccl:     channel %d parked %llu times: queue of %u headed by collective index %u, phase %u, "
              "published %u, instance %llu; waits at %#llx for %llu (x%u), sees %#llx; second wait at %#llx\n", ch,
              (unsigned long long)st->stuck[0], (unsigned)(w1 >> 48), (unsigned)(w1 & 0xffffffffu),
              (unsigned)((w1 >> 32) & 0xff), (unsigned)((w1 >> 40) & 0xff), (unsigned long long)st->stuck[2],
              (unsigned long long)st->stuck[3], (unsigned long long)(w4 & 0xffffffffffffull), (unsigned)(w4 >> 48),
              (unsigned long long)st->stuck[5], (unsigned long long)st->stuck[6]);
    }
  }
}

// The kernel is still resident although it was told to abort (a workgroup that cannot reach the point where it
// looks at the flag).  Nothing of the daemon can be freed while it runs, the observer thread is inside
// hipEventSynchronize and every call that waits for the device would block for good: say what is known and end
// the process.  Caller holds d->mu.
[[noreturn]] static void giveUpOnResidentDaemon(const Daemon* d, const char* where) {
  fprintf(stderr, "dfccl: the daemon kernel on device %d is still resident after an abort request (%s); "
          "ending the process\n", d->device, where);
  dumpDaemonState(d);
  fflush(stderr);
  fflush(stdout);
  _exit(70);
}

static std::mutex gDaemonMu;
static std::map<int, Daemon*> gDaemons;
static bool gAtexitRegistered = false;

static void abortAllDaemonsAtExit() {
  std::lock_guard<std::mutex> g(gDaemonMu);
  for (auto& kv : gDaemons) {
    Daemon* d = kv.second;
    std::unique_lock<std::mutex> lk(d->mu);
    if (d->running) {
      d->failed = true;
      __atomic_store_n(d->ctrl, kCtrlAbort, __ATOMIC_RELEASE);
      d->cv.wait_for(lk, std::chrono::milliseconds(Daemon::abortWaitMs()), [&] { return !d->running; });
      if (d->running) giveUpOnResidentDaemon(d, "process exit");
    }
  }
}

static ncclResult_t getDaemon(int device, Daemon** out) {
  std::lock_guard<std::mutex> g(gDaemonMu);
  auto it = gDaemons.find(device);
  if (it != gDaemons.end()) {
    *out = it->second;
    return ncclSuccess;
  }
  Daemon* d = new Daemon();
  d->device = device;
  HIPCHECK(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking));
  HIPCHECK(hipEventCreateWithFlags(&d->doneEv, hipEventBlockingSync | hipEventDisableTiming));
  HIPCHECK(hipHostMalloc((void**)&d->ctrl, 64, hipHostMallocCoherent | hipHostMallocMapped));
  memset(d->ctrl, 0, 64);
  HIPCHECK(hipMalloc((void**)&d->devFlags, 64));
  HIPCHECK(hipMemset(d->devFlags, 0, 64));
  HIPCHECK(hipMalloc((void**)&d->devArgs, sizeof(DaemonArgs)));
  if (envInt("DFCCL_TRACE", 0) != 0) {
    const size_t bytes = (size_t)kMaxRankSlots * kMaxChannels * kTraceRecords * 16;
    HIPCHECK(hipMalloc((void**)&d->trace, bytes));
    HIPCHECK(hipMemset(d->trace, 0, bytes));
  }
  d->readKnobs();
  d->observer = std::thread([d] { d->observerLoop(); });
  gDaemons[device] = d;
  if (!gAtexitRegistered) {
    atexit(abortAllDaemonsAtExit);
    gAtexitRegistered = true;
  }
  *out = d;
  return ncclSuccess;
}

// Called with no rank attached any more: stops the observer and frees the daemon.
static void destroyDaemon(Daemon* d) {
  {
    std::lock_guard<std::mutex> g(gDaemonMu);
    gDaemons.erase(d->device);
  }
  {
    std::unique_lock<std::mutex> lk(d->mu);
    if (d->running) {
      // every rank has left; whatever is still resident only has to notice
      if (!d->cv.wait_for(lk, std::chrono::seconds(10), [&] { return !d->running; })) {
        d->failed = true;
        __atomic_store_n(d->ctrl, kCtrlAbort, __ATOMIC_RELEASE);
        d->cv.wait_for(lk, std::chrono::milliseconds(Daemon::abortWaitMs()), [&] { return !d->running; });
        if (d->running) giveUpOnResidentDaemon(d, "freeing the daemon");
      }
    }
    d->shutdown = true;
    d->cv.notify_all();
  }
  if (d->observer.joinable()) d->observer.join();
  if (d->trace != nullptr) {
    // dump the timeline of the last launch: [workgroup][record]{event | arg << 32, tick}
    const char* path = getenv("DFCCL_TRACE_FILE");
    const size_t bytes = (size_t)kMaxRankSlots * kMaxChannels * kTraceRecords * 16;
    std::vector<char> host(bytes);
    if (hipMemcpy(host.data(), d->trace, bytes, hipMemcpyDeviceToHost) == hipSuccess) {
      FILE* f = fopen(path && *path ? path : "dfccl_trace.bin", "wb");
      if (f) {
        fwrite(host.data(), 1, bytes, f);
        fclose(f);
      }
    }
    (void)hipFree(d->trace);
  }
  d->collectGarbage();
  (void)hipFree(d->devArgs);
  (void)hipFree(d->devFlags);
  (void)hipHostFree(d->ctrl);
  (void)hipEventDestroy(d->doneEv);
  (void)hipStreamDestroy(d->stream);
  delete d;
}

// ------------------------------------------------------------------------ planning

// Fixes the chunk geometry of the collective a communicator serves
// (ofcclComputeColl / ofcclGetAlgoInfo, src/enqueue_ofccl.cc:85-283: ring, one
// protocol, channel count shrunk for small messages).
// Rank contexts alive per device: the workgroups of all of them have to fit the GPU together.
static std::atomic<int> gLiveRankCtxs[64];

// Workgroups of the daemon kernel `device` keeps resident at once (compute units x workgroups per unit), asked of
// the runtime once per device.  0 if the runtime cannot say: the callers then refuse to plan or to launch (a grid
// that is not resident as a whole makes every collective park until the idle exit).
static int deviceWorkgroupSlots(int device) {
  static std::mutex mu;
  static std::map<int, int> known;
  std::lock_guard<std::mutex> lk(mu);
  auto it = known.find(device);
  if (it != known.end()) return it->second;
  int cus = 0, perCu = 0, current = -1;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) return 0;
  // the occupancy query answers for the current device
  if (hipGetDevice(&current) != hipSuccess) return 0;
  if (current != device && hipSetDevice(device) != hipSuccess) return 0;
  hipError_t e = dfcclDaemonOccupancy(&perCu);
  if (e == hipSuccess && envInt("DFCCL_TRACE", 0) != 0) {  // the traced kernel will run: it has to fit as well
    int traced = 0;
    e = dfcclDaemonOccupancyTraced(&traced);
    perCu = std::min(perCu, traced);
  }
  if (current != device) (void)hipSetDevice(current);
  if (e != hipSuccess || perCu < 1) return 0;
  // One workgroup per compute unit is the design point, whatever the occupancy calculation would allow beyond
  // that: the workgroups of a rank share its work tile by tile, and a second workgroup per unit only halves what
  // each of them has in flight.  (What the calculation allows beyond one is headroom for residency.)
  known[device] = cus;
  return cus;
}

static void planGroup(CommGroup* g) {
  const int es = typeSizeOf(g->dtypeUser);
  int64_t nBytes = (int64_t)g->countUser * es;
  if (g->kind == kAllGather || g->kind == kBroadcast) {  // run as bytes (src/misc/argcheck.cc:53-57)
    g->dtype = ncclInt8;
    g->elemSize = 1;
    g->count = nBytes;
  } else {
    g->dtype = g->dtypeUser;
    g->elemSize = es;
    g->count = (int64_t)g->countUser;
  }
  if (g->kind == kAllGather || g->kind == kReduceScatter) nBytes *= g->nRanks;
  // protocol: virtual ranks read and write each other's buffers in place unless told otherwise (or too many)
  const char* proto = getenv("DFCCL_PROTO");
  const bool wantFifo = proto != nullptr && strcmp(proto, "fifo") == 0;
  g->proto = (!wantFifo && g->nRanks >= 2 && g->nRanks <= kMaxDirectRanks) ? kProtoDirect : kProtoFifo;
  // index space of the direct sweep: reduce and broadcast split the message among the ranks chunk by chunk as
  // all-reduce does; reduce-scatter and all-gather give every rank a block of its own
  const int geomKind = (g->proto == kProtoDirect) ? directGeomKind(g->kind) : g->kind;
  int64_t buff = envInt("NCCL_BUFFSIZE", 1 << 20);
  if (buff < (64 << 10)) buff = 64 << 10;
  buff = (buff / (8 * kAlignBytes)) * (8 * kAlignBytes);
  const int64_t stepBytes = buff / 8;  // NCCL_STEPS = 8
  int64_t chunkBytes, sliceBytes;
  if (g->proto == kProtoDirect) {
    // no FIFO: the chunk is only the interleaving grain of the sweeps (small grains keep all workgroups
    // inside one compact address window per buffer).  8 KiB up to 256 MiB per rank, 32 KiB from there on
    // (measured with 8 ranks: at 64 MiB 8 KiB tiles are 10 % faster than 32 KiB ones, at 256 MiB 15 % slower).
    const int64_t tileDefault = (nBytes >= ((int64_t)256 << 20)) ? (32 << 10) : (8 << 10);
    chunkBytes = roundUp64(std::max<int64_t>(envInt("DFCCL_DIRECT_CHUNK_BYTES", tileDefault), kAlignBytes), kAlignBytes);
    sliceBytes = chunkBytes;
    g->slicesPerChunk = 1;
    g->fifoSlots = 1;
  } else if (g->kind == kReduce || g->kind == kBroadcast) {  // CHUNKSTEPS = SLICESTEPS = 1
    chunkBytes = stepBytes;
    sliceBytes = stepBytes;
    g->slicesPerChunk = 1;
    g->fifoSlots = 8;
  } else {  // CHUNKSTEPS 4, SLICESTEPS 2: NCCL_STEPS / SLICESTEPS = 4 slices of a link in flight
    chunkBytes = stepBytes * 4;
    sliceBytes = stepBytes * 2;
    g->slicesPerChunk = 2;
    // (DFCCL_FIFO_SLOTS: more slots than the reference's four give neighbours more slack, at that much more memory)
    g->fifoSlots = (int)std::min<int64_t>(16, std::max<int64_t>(2, envInt("DFCCL_FIFO_SLOTS", 4)));
  }
  // Default: share the workgroups the GPU keeps resident (one per CU) among the ranks that will run together,
  // which is the larger of this communicator's size and the rank contexts created on the device so far, and
  // leave a few of them out (DFCCL_RESIDENCY_HEADROOM, 8): every workgroup of the daemon has to be resident,
  // so a grid that needs every last CU would leave one workgroup waiting for a CU that another kernel's
  // workgroup holds.  The launch rounds a rank's workgroups up to whole sets of 8 (one per XCD; the surplus
  // ones leave at once), and that rounded grid has to fit as well.
  int sharers = g->nRanks;
  if (g->device >= 0 && g->device < 64) sharers = std::max(sharers, gLiveRankCtxs[g->device].load());
  sharers = std::max(1, sharers);
  const int capacity = deviceWorkgroupSlots(g->device);
  g->capacityUnknown = capacity <= 0;
  if (g->capacityUnknown) {
    fprintf(stderr, "dfccl: cannot tell how many daemon workgroups device %d keeps resident; not planning\n", g->device);
    return;
  }
  const int headroom = (int)std::min<int64_t>(std::max<int64_t>(0, envInt("DFCCL_RESIDENCY_HEADROOM", 8)), capacity / 2);
  int share = std::max(1, (capacity - headroom) / sharers);
  while (share > 1 && sharers * ((share + 7) & ~7) > capacity) share--;
  int maxCh = (int)envInt("NCCL_MAX_NCHANNELS", share);
  if (maxCh < 1) maxCh = 1;
  if (maxCh > kMaxChannels) maxCh = kMaxChannels;
  const int64_t perChannel = envInt("DFCCL_BYTES_PER_CHANNEL", (int64_t)kWgThreads * 64);
  g->nChannels = planChannels(nBytes, maxCh, perChannel < 1 ? 1 : perChannel);
  g->chunkElems = chunkBytes / g->elemSize;
  g->alignElems = kAlignBytes / g->elemSize;
  g->sliceElems = sliceBytes / g->elemSize;
  // a slot only has to hold the largest slice this collective will ever move
  const int64_t real0 = realChunkElems(geomKind, g->nRanks, g->nChannels, g->chunkElems, g->alignElems,
                                       g->count > 0 ? g->count : 1, 0);
  const int64_t maxSlice = sliceElemsFor(real0, g->slicesPerChunk, g->sliceElems);
  g->slotBytes = roundUp64(maxSlice * g->elemSize, kAlignBytes);
  g->chanStride = g->slotBytes * g->fifoSlots;
  const int64_t loop = loopElems(geomKind, g->nRanks, g->nChannels, g->chunkElems);
  g->loopsPerInstance = g->count > 0 ? divUp64(g->count, loop) : 0;
  g->lastChunkElems = g->count > 0 ? realChunkElems(geomKind, g->nRanks, g->nChannels, g->chunkElems, g->alignElems,
                                                    g->count, (g->loopsPerInstance - 1) * loop)
                                   : 0;
}

static ncclResult_t allocGroupLocked(CommGroup* g) {
  if (g->flags != nullptr) return ncclSuccess;
  const size_t links = (size_t)g->nRanks * g->nChannels;
  HIPCHECK(hipMalloc((void**)&g->flags, links * sizeof(ConnFlags)));
  HIPCHECK(hipMemset(g->flags, 0, links * sizeof(ConnFlags)));
  if (g->proto == kProtoFifo) {
    HIPCHECK(hipMalloc((void**)&g->fifo, links * (size_t)g->chanStride));
  } else {
    HIPCHECK(hipMalloc((void**)&g->pubs, links * sizeof(PeerPub)));
    HIPCHECK(hipMemset(g->pubs, 0, links * sizeof(PeerPub)));
    HIPCHECK(hipMalloc((void**)&g->p1, links * 8));
    HIPCHECK(hipMemset(g->p1, 0, links * 8));
    HIPCHECK(hipMalloc((void**)&g->tileCtrs, (size_t)g->nRanks * 128));
    HIPCHECK(hipMemset(g->tileCtrs, 0, (size_t)g->nRanks * 128));
  }
  // the daemon runs on a stream that does not synchronise with the null stream: the clears must have landed
  // before it can look at this memory
  HIPCHECK(hipStreamSynchronize(nullptr));
  return ncclSuccess;
}

static ncclResult_t prepareColl(int kind, size_t count, int dtype, int op, int root, ncclComm_t comm, int collId,
                                ofcclRankCtx_t ctx) {
  if (ctx == nullptr || comm == nullptr) return ncclInvalidArgument;
  if (ctx->finalized) return ncclInvalidUsage;
  if (collId < 0 || collId >= kMaxColls || (int)ctx->colls.size() >= kMaxColls) return ncclInvalidUsage;
  if (ctx->collIndex[collId] >= 0) return ncclInvalidUsage;
  CommGroup* g = comm->group;
  if (root < 0 || root >= g->nRanks) return ncclInvalidArgument;
  if (dtype < 0 || dtype >= ncclNumTypes) return ncclInvalidArgument;
  const bool reduces = (kind == kAllReduce || kind == kReduceScatter || kind == kReduce);
  if (op < 0) return ncclInvalidArgument;
  if (comm->registered) return ncclInvalidUsage;  // one communicator per collective
  if (comm->rank != ctx->rank) return ncclInvalidArgument;
  // What the op becomes on the device (hostToDevRedOp, src/enqueue.cc:1305-1371): the four element ops as they
  // are; ncclAvg a Sum that divides the result by nRanks (integer types) or multiplies every input by 1/nRanks
  // first (float types); an operator made by ncclRedOpCreatePreMulSum a Sum of inputs times its scalar.
  int devOp = reduces ? op : (int)ncclSum;
  Scale scale;
  scale.kind = kScaleNone;
  scale.bits = 0;
  uint64_t scalePtr = 0;
  if (reduces && op == ncclAvg) {
    devOp = ncclSum;
    scale = dfcclAvgScale(dtype, g->nRanks);
  } else if (reduces && op >= ncclNumOps) {
    auto it = comm->userOps.find(op - (int)ncclNumOps);
    if (it == comm->userOps.end()) return ncclInvalidArgument;
    if (it->second.datatype != dtype) return ncclInvalidArgument;  // made for another datatype (enqueue.cc:1361-1365)
    devOp = ncclSum;
    scale.kind = kScalePre;
    scale.bits = it->second.bits;
    scalePtr = it->second.devPtr;
  } else if (op >= ncclNumOps) {
    return ncclInvalidArgument;
  }
  {
    std::lock_guard<std::mutex> lk(g->mu);
    if (g->device != ctx->device) return ncclInvalidUsage;
    if (g->retired) return ncclInvalidUsage;  // create a new communicator for a new rank context
    if (!g->planned) {
      g->kind = kind;
      g->dtypeUser = dtype;
      g->op = devOp;
      g->scaleKind = scale.kind;
      g->scaleBits.assign((size_t)g->nRanks, 0);
      g->scalePtr.assign((size_t)g->nRanks, 0);
      g->root = root;
      g->countUser = count;
      planGroup(g);
      if (g->capacityUnknown) return ncclUnhandledCudaError;  // (planned stays false: the next Prepare tries again)
      g->planned = true;
    } else if (g->kind != kind || g->dtypeUser != dtype || g->countUser != count || g->root != root ||
               (reduces && (g->op != devOp || g->scaleKind != scale.kind))) {
      // the ranks of a communicator must describe the same collective (every rank may bring its own scalar to a
      // PreMulSum, as in the reference, where each rank scales the input it reads itself)
      return ncclInvalidArgument;
    }
    g->scaleBits[(size_t)comm->rank] = scale.bits;
    g->scalePtr[(size_t)comm->rank] = scalePtr;
  }
  comm->registered = true;
  ctx->collIndex[collId] = (int16_t)ctx->colls.size();
  ctx->colls.push_back(CollReg{collId, comm});
  return ncclSuccess;
}

// ----------------------------------------------------------------------- poller

// Consumes the completion ring in ticket order and fires the callbacks
// (startPoller / cqRead, src/enqueue_ofccl.cc:908-965,697-739).
static void pollerLoop(ofcclRankCtx* c) {
  uint64_t emptySpins = 0, waitingSince = 0;
  while (!c->stopPoller.load(std::memory_order_acquire)) {
    const uint64_t v = __atomic_load_n(&c->dev.cq[c->cqRead & (kCqRing - 1)], __ATOMIC_ACQUIRE);
    if (v != ~0ull && cqeCnt(v) == (unsigned)((c->cqRead + 1) & 0xffffffu)) {
      const uint64_t tSeen = nowNs();
      const int collId = (int)cqeCollId(v);
      c->cqRead++;
      emptySpins = 0;
      waitingSince = 0;
      if (collId >= 0 && collId < kMaxColls) {
        CallbackFunc cb = c->callbacks[collId];
        void* args = c->cbArgs[collId];
        c->completeNs[collId] = tSeen;
        c->completed.fetch_add(1, std::memory_order_acq_rel);
        c->inflight[collId].store(0, std::memory_order_release);
        if (cb) (void)cb(collId, args);
      }
      continue;
    }
    if (c->submitted.load(std::memory_order_acquire) == c->completed.load(std::memory_order_acquire)) {
      // nothing outstanding: sleep at once. (Spinning on here was measured: it gains nothing for a caller that
      // submits again right away, and with as many rank contexts as cores it starves the submitting threads.)
      std::unique_lock<std::mutex> lk(c->pollMu);
      c->pollerAsleep.store(true);  // sequentially consistent, as is the submitter's increment: one sees the other
      c->pollCv.wait_for(lk, std::chrono::milliseconds(2), [&] {
        return c->stopPoller.load() || c->submitted.load() != c->completed.load();
      });
      c->pollerAsleep.store(false);
      emptySpins = 0;
      waitingSince = 0;
    } else if ((++emptySpins & 1023u) == 0) {
      // work is outstanding: keep spinning (giving the CPU away here costs a scheduler slice when it is least
      // affordable); only a completion that has not come for milliseconds is waited for at a lower rate
      const uint64_t now = nowNs();
      if (waitingSince == 0) waitingSince = now;
      else if (now - waitingSince > 5000000ull) usleep(50);
    } else {
      _mm_pause();
    }
  }
}

// --------------------------------------------------------------------- submission

// Writes one entry to the host-coherent ring (sqWrite, src/enqueue_ofccl.cc:616-656).
// Returns -1 if the ring is full.  `stampNs`, if given, receives the steady-clock time just before the entry
// becomes visible to the device (so a completion can never be stamped earlier than its submission).
static int sqWrite(ofcclRankCtx* c, uint64_t sendbuff, uint64_t recvbuff, uint32_t coll, uint32_t flags,
                   uint64_t* stampNs = nullptr) {
  std::lock_guard<std::mutex> lk(c->sqMu);
  const uint64_t head = __atomic_load_n(c->dev.sqHead, __ATOMIC_ACQUIRE);
  if (c->sqTail - head >= c->sqCapacity) return -1;
  const uint64_t t = c->sqTail;
  if (stampNs) *stampNs = nowNs();
  uint64_t* w = c->dev.sq + (t & (kSqRing - 1)) * kSqeWords;
  const uint64_t tag = sqeTag(t);
  __atomic_store_n(&w[0], (sendbuff & kPtrMask) | tag, __ATOMIC_RELEASE);
  __atomic_store_n(&w[1], (recvbuff & kPtrMask) | tag, __ATOMIC_RELEASE);
  __atomic_store_n(&w[2], (uint64_t)coll | ((uint64_t)(flags & 0xffffu) << 32) | tag, __ATOMIC_RELEASE);
  __atomic_store_n(&w[3], tag, __ATOMIC_RELEASE);
  c->sqTail = t + 1;
  return 0;
}

static ncclResult_t runColl(const void* sendbuff, void* recvbuff, int collId, CallbackFunc cb, void* cbArgs,
                            ofcclRankCtx_t c) {
  if (c == nullptr || !c->finalized) return ncclInvalidUsage;
  if (c->daemon->failed) return ncclSystemError;  // the daemon could not be launched, or had to be aborted
  if (collId < 0 || collId >= kMaxColls || c->collIndex[collId] < 0) return ncclInvalidArgument;
  if (((uint64_t)(uintptr_t)sendbuff & ~kPtrMask) || ((uint64_t)(uintptr_t)recvbuff & ~kPtrMask))
    return ncclInvalidArgument;
  Daemon* d = c->daemon;
  // one instance per collId in flight: a second Run waits for the first (for ever only if the daemon is lost)
  int expected = 0;
  while (!c->inflight[collId].compare_exchange_weak(expected, 1, std::memory_order_acq_rel)) {
    expected = 0;
    if (d->failed.load(std::memory_order_acquire)) return ncclSystemError;
    sched_yield();
  }
  c->callbacks[collId] = cb;
  c->cbArgs[collId] = cbArgs;
  c->submitted.fetch_add(1);
  // a full ring back-pressures the caller (CpuSqFull, src/enqueue_ofccl.h:51-54; the spin of
  // src/collectives_ofccl/ofccl_all_reduce.cc:29-33)
  while (sqWrite(c, (uint64_t)(uintptr_t)sendbuff, (uint64_t)(uintptr_t)recvbuff, (uint32_t)c->collIndex[collId], 0,
                 &c->submitNs[collId]) == -1) {
    if (d->failed.load(std::memory_order_acquire)) {
      c->submitted.fetch_sub(1);
      c->inflight[collId].store(0, std::memory_order_release);
      return ncclSystemError;
    }
    c->sqFullSpins.fetch_add(1, std::memory_order_relaxed);
    sched_yield();
  }
  {
    // wake the observer if the kernel is not resident (cheap check first)
    std::unique_lock<std::mutex> lk(d->mu, std::try_to_lock);
    if (!lk.owns_lock() || !d->running) {
      if (!lk.owns_lock()) lk.lock();
      d->cv.notify_all();
    }
  }
  if (c->pollerAsleep.load()) {
    // taking the mutex orders this notification after the poller's test of the predicate
    { std::lock_guard<std::mutex> lk(c->pollMu); }
    c->pollCv.notify_one();
  }
  return ncclSuccess;
}

}  // namespace dfccl

using namespace dfccl;

// ================================================================ communicator API

DFCCL_API ncclResult_t ncclGetUniqueId(ncclUniqueId* uniqueId) {
  if (uniqueId == nullptr) return ncclInvalidArgument;
  memset(uniqueId, 0, sizeof(*uniqueId));
  const uint64_t id = gNextCommId.fetch_add(1);
  const uint64_t magic = 0x4446434c56434f4dull;  // "DFCLVCOM"
  const uint64_t pid = (uint64_t)getpid();
  memcpy(uniqueId->internal, &magic, 8);
  memcpy(uniqueId->internal + 8, &id, 8);
  memcpy(uniqueId->internal + 16, &pid, 8);
  return ncclSuccess;
}

DFCCL_API ncclResult_t ncclCommInitRank(ncclComm_t* comm, int nranks, ncclUniqueId commId, int rank) {
  if (comm == nullptr) return ncclInvalidArgument;
  if (nranks < 1 || rank < 0 || rank >= nranks) return ncclInvalidArgument;
  uint64_t magic, id, pid;
  memcpy(&magic, commId.internal, 8);
  memcpy(&id, commId.internal + 8, 8);
  memcpy(&pid, commId.internal + 16, 8);
  if (magic != 0x4446434c56434f4dull || pid != (uint64_t)getpid()) return ncclInvalidArgument;
  int device = 0;
  HIPCHECK(hipGetDevice(&device));
  std::lock_guard<std::mutex> lk(gCommMu);
  CommGroup* g;
  auto it = gGroups.find(id);
  if (it == gGroups.end()) {
    g = new CommGroup();
    g->id = id;
    g->nRanks = nranks;
    g->device = device;
    gGroups[id] = g;
  } else {
    g = it->second;
    if (g->nRanks != nranks || g->device != device) return ncclInvalidArgument;
  }
  g->handles++;
  ncclComm* c = new ncclComm();
  c->group = g;
  c->rank = rank;
  c->registered = false;
  *comm = c;
  return ncclSuccess;
}

DFCCL_API ncclResult_t ncclCommDestroy(ncclComm_t comm) {
  if (comm == nullptr) return ncclSuccess;
  CommGroup* g = comm->group;
  bool last;
  {
    std::lock_guard<std::mutex> lk(gCommMu);
    last = (--g->handles == 0);
    if (last) gGroups.erase(g->id);
  }
  delete comm;
  if (last) {
    // freeing device memory waits for the device, which a resident daemon would
    // block for good: hand the memory to the daemon, it frees it between launches
    Daemon* d = nullptr;
    {
      std::lock_guard<std::mutex> g2(gDaemonMu);
      auto it = gDaemons.find(g->device);
      if (it != gDaemons.end()) d = it->second;
    }
    if (d != nullptr) {
      std::lock_guard<std::mutex> lk(d->mu);
      if (d->running) {
        for (void* p : {(void*)g->fifo, (void*)g->flags, (void*)g->pubs, (void*)g->p1, (void*)g->tileCtrs})
          if (p) d->garbageDev.push_back(p);
        g->fifo = nullptr; g->flags = nullptr; g->pubs = nullptr; g->p1 = nullptr; g->tileCtrs = nullptr;
      }
    }
    for (void* p : {(void*)g->fifo, (void*)g->flags, (void*)g->pubs, (void*)g->p1, (void*)g->tileCtrs})
      if (p) (void)hipFree(p);
    delete g;
  }
  return ncclSuccess;
}

DFCCL_API ncclResult_t ncclCommCount(const ncclComm_t comm, int* count) {
  if (comm == nullptr || count == nullptr) return ncclInvalidArgument;
  *count = comm->group->nRanks;
  return ncclSuccess;
}

DFCCL_API ncclResult_t ncclCommUserRank(const ncclComm_t comm, int* rank) {
  if (comm == nullptr || rank == nullptr) return ncclInvalidArgument;
  *rank = comm->rank;
  return ncclSuccess;
}

// A reduction operator that multiplies every input by *scalar before summing (src/nccl.h.in:148-180,
// src/enqueue.cc:1443-1490).  ncclScalarHostImmediate: the scalar is read now.  ncclScalarDevice: `scalar` is a
// device address, kept as it is (enqueue.cc:1470-1472) and dereferenced on the device whenever an instance of a
// collective prepared with the operator starts (the reference dereferences it when the kernel starts on the
// work element, src/collectives/device/common.h:117-136); the memory has to stay valid, and hold an element of
// `datatype` at its natural alignment, for as long as the collective is registered.
DFCCL_API ncclResult_t ncclRedOpCreatePreMulSum(ncclRedOp_t* op, void* scalar, ncclDataType_t datatype,
                                                ncclScalarResidence_t residence, ncclComm_t comm) {
  if (op == nullptr || scalar == nullptr || comm == nullptr) return ncclInvalidArgument;
  const int es = typeSizeOf((int)datatype);
  if (es == 0) return ncclInvalidArgument;
  if (residence != ncclScalarHostImmediate && residence != ncclScalarDevice) return ncclInvalidArgument;
  uint64_t bits = 0, devPtr = 0;
  if (residence == ncclScalarHostImmediate) {
    memcpy(&bits, scalar, (size_t)es);
  } else {
    devPtr = (uint64_t)(uintptr_t)scalar;
    if ((devPtr & ~kPtrMask) != 0 || devPtr % (uint64_t)es != 0) return ncclInvalidArgument;
  }
  const int ix = comm->nextUserOp++;
  comm->userOps[ix] = ncclComm::UserOp{(int)datatype, bits, devPtr};
  *op = (ncclRedOp_t)((int)ncclNumOps + ix);
  return ncclSuccess;
}

DFCCL_API ncclResult_t ncclRedOpDestroy(ncclRedOp_t op, ncclComm_t comm) {
  if (comm == nullptr) return ncclInvalidArgument;
  if ((int)op < (int)ncclNumOps) return ncclInvalidArgument;  // built-in operators cannot be destroyed
  if (comm->userOps.erase((int)op - (int)ncclNumOps) == 0) return ncclInvalidArgument;
  return ncclSuccess;
}

DFCCL_API const char* ncclGetErrorString(ncclResult_t result) {
  switch (result) {
    case ncclSuccess: return "no error";
    case ncclUnhandledCudaError: return "unhandled HIP error";
    case ncclSystemError: return "unhandled system error";
    case ncclInternalError: return "internal error";
    case ncclInvalidArgument: return "invalid argument";
    case ncclInvalidUsage: return "invalid usage";
    default: return "unknown result code";
  }
}

// ================================================================ rank context API

DFCCL_API ncclResult_t ofcclInitRankCtx(ofcclRankCtx_t* rankCtx, int rank) {
  if (rankCtx == nullptr || rank < 0) return ncclInvalidArgument;
  int device = 0;
  HIPCHECK(hipGetDevice(&device));
  ofcclRankCtx* c = new ofcclRankCtx();
  c->rank = rank;
  c->device = device;
  // QLen of the reference (src/include/collectives_ofccl.h:104,110); a smaller queue is only of use to tests of
  // the full-queue path
  c->sqCapacity = (uint64_t)std::min<int64_t>(kSqCapacity, std::max<int64_t>(1, envInt("DFCCL_SQ_CAPACITY", kSqCapacity)));
  for (int i = 0; i < kMaxColls; i++) {
    c->collIndex[i] = -1;
    c->callbacks[i] = nullptr;
    c->cbArgs[i] = nullptr;
    c->inflight[i].store(0);
    c->submitNs[i] = c->completeNs[i] = 0;
  }
  if (device >= 0 && device < 64) gLiveRankCtxs[device].fetch_add(1);
  *rankCtx = c;
  return ncclSuccess;
}

DFCCL_API ncclResult_t ofcclPrepareAllReduce(size_t count, ncclDataType_t datatype, ncclRedOp_t op, ncclComm_t comm,
                                             int collId, ofcclRankCtx_t rankCtx) {
  return prepareColl(kAllReduce, count, (int)datatype, (int)op, 0, comm, collId, rankCtx);
}
DFCCL_API ncclResult_t ofcclPrepareReduceScatter(size_t recvcount, ncclDataType_t datatype, ncclRedOp_t op,
                                                 ncclComm_t comm, int collId, ofcclRankCtx_t rankCtx) {
  return prepareColl(kReduceScatter, recvcount, (int)datatype, (int)op, 0, comm, collId, rankCtx);
}
DFCCL_API ncclResult_t ofcclPrepareAllGather(size_t sendcount, ncclDataType_t datatype, ncclComm_t comm, int collId,
                                             ofcclRankCtx_t rankCtx) {
  return prepareColl(kAllGather, sendcount, (int)datatype, (int)ncclSum, 0, comm, collId, rankCtx);
}
DFCCL_API ncclResult_t ofcclPrepareReduce(size_t count, ncclDataType_t datatype, ncclRedOp_t op, int root,
                                          ncclComm_t comm, int collId, ofcclRankCtx_t rankCtx) {
  return prepareColl(kReduce, count, (int)datatype, (int)op, root, comm, collId, rankCtx);
}
DFCCL_API ncclResult_t ofcclPrepareBroadcast(size_t count, ncclDataType_t datatype, int root, ncclComm_t comm,
                                             int collId, ofcclRankCtx_t rankCtx) {
  return prepareColl(kBroadcast, count, (int)datatype, (int)ncclSum, root, comm, collId, rankCtx);
}
DFCCL_API ncclResult_t ofcclPrepareBcast(size_t count, ncclDataType_t datatype, int root, ncclComm_t comm, int collId,
                                         ofcclRankCtx_t rankCtx) {
  return ofcclPrepareBroadcast(count, datatype, root, comm, collId, rankCtx);
}

DFCCL_API ncclResult_t ofcclFinalizeRankCtx7StartHostThrds(ofcclRankCtx_t c) {
  if (c == nullptr) return ncclInvalidArgument;
  if (c->finalized) return ncclInvalidUsage;
  HIPCHECK(hipSetDevice(c->device));
  Daemon* d = nullptr;
  ncclResult_t r = getDaemon(c->device, &d);
  if (r != ncclSuccess) return r;
  const int nColls = (int)c->colls.size();
  const int nCollsAlloc = nColls > 0 ? nColls : 1;

  // per-collective plans of this rank
  std::vector<CollPlan> plans((size_t)nCollsAlloc);
  memset(plans.data(), 0, plans.size() * sizeof(CollPlan));
  HIPCHECK(hipMalloc((void**)&c->doneCounters, (size_t)nCollsAlloc * sizeof(uint64_t)));
  HIPCHECK(hipMemset(c->doneCounters, 0, (size_t)nCollsAlloc * sizeof(uint64_t)));
  int maxCh = 1;
  for (int i = 0; i < nColls; i++) {
    CommGroup* g = c->colls[i].comm->group;
    {
      std::lock_guard<std::mutex> lk(g->mu);
      r = allocGroupLocked(g);
      if (r != ncclSuccess) return r;
    }
    CollPlan& p = plans[i];
    const int n = g->nRanks, rank = c->rank, prev = (rank + n - 1) % n;
    p.kind = g->kind; p.dtype = g->dtype; p.op = g->op; p.root = g->root;
    p.nRanks = n; p.rank = rank; p.nChannels = g->nChannels; p.collId = c->colls[i].collId;
    p.count = g->count; p.chunkElems = g->chunkElems; p.alignElems = g->alignElems; p.sliceElems = g->sliceElems;
    p.slicesPerChunk = g->slicesPerChunk; p.fifoSlots = g->fifoSlots; p.elemSize = g->elemSize;
    p.slotBytes = g->slotBytes; p.fifoChanStride = g->chanStride;
    p.sendFifo = g->fifo ? g->fifo + (size_t)rank * g->nChannels * g->chanStride : nullptr;
    p.recvFifo = g->fifo ? g->fifo + (size_t)prev * g->nChannels * g->chanStride : nullptr;
    p.proto = g->proto; p.scaleKind = g->scaleKind; p.pubs = g->pubs; p.p1 = g->p1;
    p.scaleBits = g->scaleBits[(size_t)rank];
    p.scalePtr = (const void*)(uintptr_t)g->scalePtr[(size_t)rank];
    if (g->proto == kProtoDirect && g->scaleKind == kScalePre && p.scalePtr == nullptr) {
      // the peers fold this rank's input: they find its scalar next to its buffer pointers.  Only the `scale`
      // word of every channel of this rank's row is written (the tagged words beside it belong to the kernel).
      for (int ch = 0; ch < g->nChannels; ch++)
        HIPCHECK(hipMemcpy(&g->pubs[(size_t)rank * g->nChannels + ch].scale, &p.scaleBits, sizeof(p.scaleBits),
                           hipMemcpyHostToDevice));
    }
    p.loopsPerInstance = g->loopsPerInstance;
    p.lastChunkElems = g->lastChunkElems;
    p.tileCtr = g->tileCtrs ? g->tileCtrs + (size_t)rank * 16 : nullptr;
    p.sendFlags = g->flags + (size_t)rank * g->nChannels;
    p.recvFlags = g->flags + (size_t)prev * g->nChannels;
    p.doneCounter = c->doneCounters + i;
    if (g->nChannels > maxCh) maxCh = g->nChannels;
  }
  c->nChannels = maxCh;

  // queues and per-workgroup state (sqCreate / cqCreate, src/enqueue_ofccl.cc:596-695)
  RankDev& R = c->dev;
  memset(&R, 0, sizeof(R));
  R.nChannels = maxCh;
  R.nColls = nColls;
  R.rank = c->rank;
  const unsigned hostFlags = hipHostMallocCoherent | hipHostMallocMapped;
  HIPCHECK(hipHostMalloc((void**)&R.sq, (size_t)kSqRing * kSqeWords * 8, hostFlags));
  memset(R.sq, 0, (size_t)kSqRing * kSqeWords * 8);
  HIPCHECK(hipHostMalloc((void**)&R.sqHead, 64, hostFlags));
  *R.sqHead = 0;
  HIPCHECK(hipHostMalloc((void**)&R.cq, (size_t)kCqRing * 8, hostFlags));
  memset(R.cq, 0xff, (size_t)kCqRing * 8);
  HIPCHECK(hipHostMalloc((void**)&R.wgExit, (size_t)kMaxChannels * 4, hostFlags));
  memset(R.wgExit, 0, (size_t)kMaxChannels * 4);
  HIPCHECK(hipHostMalloc((void**)&R.stats, (size_t)kMaxChannels * sizeof(WgStats), hostFlags));
  memset(R.stats, 0, (size_t)kMaxChannels * sizeof(WgStats));
  R.ctrl = d->ctrl;
  HIPCHECK(hipMalloc((void**)&R.mirror, (size_t)kSqRing * sizeof(DevSqe)));
  HIPCHECK(hipMemset(R.mirror, 0, (size_t)kSqRing * sizeof(DevSqe)));
  HIPCHECK(hipMalloc((void**)&R.mirrorTail, 64));
  HIPCHECK(hipMemset(R.mirrorTail, 0, 64));
  HIPCHECK(hipMalloc((void**)&R.wgFrontier, (size_t)kMaxChannels * 8));
  HIPCHECK(hipMemset(R.wgFrontier, 0, (size_t)kMaxChannels * 8));
  HIPCHECK(hipMalloc((void**)&R.cqTicket, 64));
  HIPCHECK(hipMemset(R.cqTicket, 0, 64));
  HIPCHECK(hipMalloc((void**)&R.plans, (size_t)nCollsAlloc * sizeof(CollPlan)));
  HIPCHECK(hipMemcpy(R.plans, plans.data(), (size_t)nCollsAlloc * sizeof(CollPlan), hipMemcpyHostToDevice));
  HIPCHECK(hipMalloc((void**)&R.dyn, (size_t)maxCh * nCollsAlloc * sizeof(DynCtx)));
  HIPCHECK(hipMemset(R.dyn, 0, (size_t)maxCh * nCollsAlloc * sizeof(DynCtx)));
  HIPCHECK(hipMalloc((void**)&R.saved, (size_t)maxCh * sizeof(WgSaved)));
  HIPCHECK(hipMemset(R.saved, 0, (size_t)maxCh * sizeof(WgSaved)));
  HIPCHECK(hipStreamSynchronize(nullptr));  // see allocGroupLocked

  // attach to the device daemon; a resident kernel has to leave first so that
  // the next launch covers this rank's workgroups
  {
    std::unique_lock<std::mutex> lk(d->mu);
    int slot = -1;
    for (int s = 0; s < kMaxRankSlots; s++)
      if (d->slots[s] == nullptr) { slot = s; break; }
    if (slot < 0) return ncclInvalidUsage;
    d->readKnobs();
    d->quiesceLocked(lk);
    if (d->running) giveUpOnResidentDaemon(d, "attaching a rank context");
    d->slots[slot] = c;
    d->nActive++;
    c->slot = slot;
    c->daemon = d;
    c->finalized = true;
    d->cv.notify_all();
  }
  c->poller = std::thread([c] { pollerLoop(c); });
  return ncclSuccess;
}

DFCCL_API ncclResult_t ofcclPrepareDone(ofcclRankCtx_t c) {
  ncclResult_t r = ofcclFinalizeRankCtx7StartHostThrds(c);
  if (r != ncclSuccess) return r;
  Daemon* d = c->daemon;
  std::lock_guard<std::mutex> lk(d->mu);
  if (!d->running) {
    d->launchRequested = true;
    d->cv.notify_all();
  }
  return ncclSuccess;
}

DFCCL_API ncclResult_t ofcclDestroy(ofcclRankCtx_t c) {
  if (c == nullptr) return ncclInvalidArgument;
  if (c->finalized) {
    Daemon* d = c->daemon;
    bool quitSent = false;
    bool lastRank = false;
    // (DFCCL_DESTROY_WAIT_MS: how long the rank's workgroups are given to leave; 20 s unless a test says otherwise)
    const auto deadline = std::chrono::steady_clock::now() +
                          std::chrono::milliseconds(std::max<int64_t>(1, envInt("DFCCL_DESTROY_WAIT_MS", 20000)));
    for (;;) {
      std::unique_lock<std::mutex> lk(d->mu);
      bool out = !d->running;
      if (!out) {
        // out of the kernel once every workgroup of the rank has written its exit word in this launch
        out = true;
        for (int ch = 0; ch < c->nChannels; ch++) {
          const uint32_t w = __atomic_load_n(&c->dev.wgExit[ch], __ATOMIC_ACQUIRE);
          if ((w >> 4) != d->epoch || (w & 0xf) == kExitNone) { out = false; break; }
        }
      }
      if (out) {
        d->slots[c->slot] = nullptr;
        d->nActive--;
        lastRank = (d->nActive == 0);
        break;
      }
      if (!quitSent) {
        lk.unlock();
        // the quit entry (src/enqueue_ofccl.cc:1593-1594). It does not count as outstanding work: if the
        // kernel ends before reading it, the rank is simply left out of the next launch.
        while (sqWrite(c, 0, 0, 0, kSqeFlagQuit) == -1) sched_yield();
        quitSent = true;
        continue;
      }
      if (std::chrono::steady_clock::now() > deadline) {
        fprintf(stderr, "dfccl: rank %d did not leave the daemon, aborting the daemon\n", c->rank);
        dumpDaemonState(d);
        // an aborted kernel abandons its scheduler state: it must never be launched again on top of it
        d->failed = true;
        __atomic_store_n(d->ctrl, kCtrlAbort, __ATOMIC_RELEASE);
        d->cv.wait_for(lk, std::chrono::milliseconds(Daemon::abortWaitMs()), [&] { return !d->running; });
        if (d->running) giveUpOnResidentDaemon(d, "destroying a rank context");
        d->slots[c->slot] = nullptr;
        d->nActive--;
        lastRank = (d->nActive == 0);
        break;
      }
      lk.unlock();
      usleep(50);
    }
    c->stopPoller.store(true, std::memory_order_release);
    c->pollCv.notify_all();
    if (c->poller.joinable()) c->poller.join();

    RankDev& R = c->dev;
    void* devPtrs[] = {R.mirror, R.mirrorTail, R.wgFrontier, R.cqTicket, R.plans, R.dyn, R.saved, c->doneCounters};
    void* hostPtrs[] = {R.sq, R.sqHead, R.cq, R.wgExit, R.stats};
    if (lastRank) {
      destroyDaemon(d);
      for (void* p : devPtrs) if (p) (void)hipFree(p);
      for (void* p : hostPtrs) if (p) (void)hipHostFree(p);
    } else {
      std::lock_guard<std::mutex> lk(d->mu);
      if (d->running) {
        for (void* p : devPtrs) if (p) d->garbageDev.push_back(p);
        for (void* p : hostPtrs) if (p) d->garbageHost.push_back(p);
      } else {
        for (void* p : devPtrs) if (p) (void)hipFree(p);
        for (void* p : hostPtrs) if (p) (void)hipHostFree(p);
      }
    }
  }
  for (auto& reg : c->colls) {
    reg.comm->registered = false;
    if (c->finalized) {
      std::lock_guard<std::mutex> lk(reg.comm->group->mu);
      reg.comm->group->retired = true;
    }
  }
  if (c->device >= 0 && c->device < 64) gLiveRankCtxs[c->device].fetch_sub(1);
  delete c;
  return ncclSuccess;
}

// ======================================================================== run API

DFCCL_API ncclResult_t ofcclRunAllReduce(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                                         void* callbackArgs, ofcclRankCtx_t rankCtx) {
  return runColl(sendbuff, recvbuff, collId, callback, callbackArgs, rankCtx);
}
DFCCL_API ncclResult_t ofcclRunReduceScatter(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                                             void* callbackArgs, ofcclRankCtx_t rankCtx) {
  return runColl(sendbuff, recvbuff, collId, callback, callbackArgs, rankCtx);
}
DFCCL_API ncclResult_t ofcclRunAllGather(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                                         void* callbackArgs, ofcclRankCtx_t rankCtx) {
  return runColl(sendbuff, recvbuff, collId, callback, callbackArgs, rankCtx);
}
DFCCL_API ncclResult_t ofcclRunReduce(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                                      void* callbackArgs, ofcclRankCtx_t rankCtx) {
  return runColl(sendbuff, recvbuff, collId, callback, callbackArgs, rankCtx);
}
DFCCL_API ncclResult_t ofcclRunBroadcast(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                                         void* callbackArgs, ofcclRankCtx_t rankCtx) {
  return runColl(sendbuff, recvbuff, collId, callback, callbackArgs, rankCtx);
}
DFCCL_API ncclResult_t ofcclRunBcast(void* buff, int collId, CallbackFunc callback, void* callbackArgs,
                                     ofcclRankCtx_t rankCtx) {
  return runColl(buff, buff, collId, callback, callbackArgs, rankCtx);  // in place (ofccl_broadcast.cc:37-44)
}

// ================================================================== introspection

DFCCL_API ncclResult_t dfcclGetStats(ofcclRankCtx_t c, dfcclStats* out) {
  if (c == nullptr || out == nullptr) return ncclInvalidArgument;
  // the caller says how large its structure is: nothing is written beyond that
  const uint64_t callerBytes = out->structBytes;
  if (callerBytes < 16 || callerBytes > 4096) return ncclInvalidArgument;
  dfcclStats full;
  dfcclStats* const user = out;
  out = &full;
  memset(out, 0, sizeof(*out));
  out->structBytes = std::min<uint64_t>(callerBytes, sizeof(dfcclStats));
  if (!c->finalized) {
    memcpy(user, out, (size_t)out->structBytes);
    return ncclInvalidUsage;
  }
  Daemon* d = c->daemon;
  {
    // A resident daemon writes its counters on request: raise the request number (the word after the control
    // word) and wait, for a bounded time, until every workgroup of this rank has answered. Workgroups in the
    // middle of a long transfer answer late; then the figures are those of their previous answer.
    std::unique_lock<std::mutex> lk(d->mu);
    if (d->running && !d->failed) {
      uint32_t e = ++d->statsEpoch;
      if (e == 0) e = ++d->statsEpoch;
      __atomic_store_n(&d->ctrl[1], e, __ATOMIC_RELEASE);
      lk.unlock();
      // (20 ms is ample on the GPU; DFCCL_STATS_WAIT_MS is for hosts where the daemon runs much slower than that)
      const uint64_t deadline = nowNs() + (uint64_t)envInt("DFCCL_STATS_WAIT_MS", 20) * 1000000ull;
      for (;;) {
        bool all = true;
        for (int ch = 0; ch < c->nChannels && all; ch++)
          all = __atomic_load_n(&c->dev.stats[ch].epoch, __ATOMIC_ACQUIRE) == (uint64_t)e;
        if (all || nowNs() > deadline) break;
        lk.lock();
        const bool gone = !d->running;
        lk.unlock();
        if (gone) break;
        usleep(20);
      }
    }
  }
  for (int ch = 0; ch < c->nChannels; ch++) {
    const WgStats* s = &c->dev.stats[ch];
    out->sqesRead += __atomic_load_n(&s->sqesRead, __ATOMIC_ACQUIRE);
    out->cqesWritten += __atomic_load_n(&s->cqesWritten, __ATOMIC_ACQUIRE);
    out->ctxSaves += __atomic_load_n(&s->ctxSaves, __ATOMIC_ACQUIRE);
    out->ctxLoads += __atomic_load_n(&s->ctxLoads, __ATOMIC_ACQUIRE);
    out->voluntaryQuits += __atomic_load_n(&s->voluntaryQuits, __ATOMIC_ACQUIRE);
    out->forcedQuits += __atomic_load_n(&s->forcedQuits, __ATOMIC_ACQUIRE);
    out->slicesMoved += __atomic_load_n(&s->slicesMoved, __ATOMIC_ACQUIRE);
  }
  out->sqFullWaits = c->sqFullSpins.load(std::memory_order_relaxed);
  {
    std::lock_guard<std::mutex> lk(d->mu);
    out->daemonLaunches = d->launches;
  }
  memcpy(user, out, (size_t)out->structBytes);
  return ncclSuccess;
}

DFCCL_API ncclResult_t dfcclDumpState(ofcclRankCtx_t c) {
  if (c == nullptr || !c->finalized) return ncclInvalidUsage;
  std::lock_guard<std::mutex> lk(c->daemon->mu);
  dumpDaemonState(c->daemon);
  return ncclSuccess;
}

DFCCL_API ncclResult_t dfcclGetCollTiming(ofcclRankCtx_t c, int collId, uint64_t* submitNs, uint64_t* completeNs) {
  if (c == nullptr || collId < 0 || collId >= kMaxColls || c->collIndex[collId] < 0) return ncclInvalidArgument;
  if (submitNs) *submitNs = c->submitNs[collId];
  if (completeNs) *completeNs = c->completeNs[collId];
  return ncclSuccess;
}

DFCCL_API ncclResult_t dfcclGetCollGeometry(ofcclRankCtx_t c, int collId, dfcclCollGeometry* geom) {
  if (c == nullptr || geom == nullptr) return ncclInvalidArgument;
  if (collId < 0 || collId >= kMaxColls || c->collIndex[collId] < 0) return ncclInvalidArgument;
  const CommGroup* g = c->colls[(size_t)c->collIndex[collId]].comm->group;
  geom->nRanks = g->nRanks;
  geom->nChannels = g->nChannels;
  geom->chunkElems = g->chunkElems;
  geom->alignElems = g->alignElems;
  geom->sliceElems = g->sliceElems;
  geom->slicesPerChunk = g->slicesPerChunk;
  geom->fifoSlots = g->fifoSlots;
  geom->protocol = g->proto;
  return ncclSuccess;
}
