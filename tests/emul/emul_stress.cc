// Scenarios for the host emulation of the daemon kernel (see hip/hip_runtime.h here), through the public C ABI.
// Each scenario runs collectives between virtual ranks, checks every result against a host loop, and ends with an
// orderly teardown; a workgroup out of step, a run that stops moving, a bad address (AddressSanitizer build) or a
// data race in LDS (ThreadSanitizer build) ends the process with a report.
//
//   emul_stress repeat <ranks> <count> <reps> <colls>   the same small fp32 Sum all-reduces over and over, one
//        after the other, every rank submitted in turn from this thread (the shape of the GPU test
//        test_small_all_reduce_repeated_and_fallbacks); knobs come from the environment
//   emul_stress mixed <ranks> <reps>    all five collectives side by side, int32, ranks submit in different orders
//   emul_stress relaunch <ranks>        idle exit and relaunch, with and without a collective parked
//   emul_stress reuse <ranks>           rank contexts destroyed and created again: old communicators are refused
//   emul_stress fuzz <seed> <rounds>    random collectives, element types, ops, ranks and submission orders
//   emul_stress backpressure <ranks> <colls> <rounds> <callback sleep us>   two submitting threads per rank push
//        every collective `rounds` times as fast as the queue takes them (DFCCL_SQ_CAPACITY makes it small), the
//        last rank starting late; every submission must get exactly one callback
//   emul_stress tworings <ranks>        one ring stays busy while the other's workgroups leave for idleness; the
//        idle ring's next submission must still get through (the whole daemon leaves and is launched again)
//   emul_stress stuck <ranks>           (with EMUL_NEVER_LEAVE=1) the daemon never leaves: Destroy must end the
//        process with a report instead of blocking for good
#include <hip/hip_runtime.h>
#include <ofccl.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <string>
#include <thread>
#include <vector>

#define CHECK(call)                                                                   \
  do {                                                                                \
    ncclResult_t r_ = (call);                                                         \
    if (r_ != ncclSuccess) {                                                          \
      fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #call, ncclGetErrorString(r_)); \
      exit(2);                                                                        \
    }                                                                                 \
  } while (0)

extern "C" void emulDumpThreads();

struct Ring {
  int n = 0;
  std::vector<ofcclRankCtx_t> ctxs;
  std::vector<std::vector<ncclComm_t>> comms;  // per collective
  std::vector<std::atomic<int>> done;          // completions per (rank, collective)
  int ncolls = 0;
  explicit Ring(int n_) : n(n_), ctxs((size_t)n_) {
    for (int r = 0; r < n; r++) CHECK(ofcclInitRankCtx(&ctxs[r], r));
  }
  std::vector<ncclComm_t>& newComms() {
    ncclUniqueId id;
    CHECK(ncclGetUniqueId(&id));
    std::vector<ncclComm_t> c((size_t)n);
    for (int r = 0; r < n; r++) CHECK(ncclCommInitRank(&c[r], n, id, r));
    comms.push_back(c);
    ncolls++;
    return comms.back();
  }
  void finalize() {
    done = std::vector<std::atomic<int>>((size_t)n * ncolls);
    for (auto& d : done) d.store(0);
    for (int r = 0; r < n; r++) CHECK(ofcclFinalizeRankCtx7StartHostThrds(ctxs[r]));
  }
  std::atomic<int>& flag(int r, int cid) { return done[(size_t)r * ncolls + cid]; }
  static int cb(int, void* arg) {
    ((std::atomic<int>*)arg)->fetch_add(1);
    return 0;
  }
  void waitAll(const std::vector<int>& want, double timeoutS, const char* what) {
    const auto t0 = std::chrono::steady_clock::now();
    for (;;) {
      bool all = true;
      for (int r = 0; r < n; r++)
        for (int c = 0; c < ncolls; c++) all = all && flag(r, c).load() >= want[(size_t)r * ncolls + c];
      if (all) return;
      if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > timeoutS) {
        fprintf(stderr, "emul_stress: %s: not complete after %.0f s\n", what, timeoutS);
        for (int r = 0; r < n; r++)
          for (int c = 0; c < ncolls; c++)
            if (flag(r, c).load() < want[(size_t)r * ncolls + c])
              fprintf(stderr, "  rank %d collective %d: %d of %d\n", r, c, flag(r, c).load(), want[(size_t)r * ncolls + c]);
        dfcclDumpState(ctxs[0]);
        emulDumpThreads();
        exit(3);
      }
      usleep(1000);
    }
  }
  void destroy() {
    for (int r = 0; r < n; r++) CHECK(ofcclDestroy(ctxs[r]));
    for (auto& c : comms)
      for (int r = 0; r < n; r++) CHECK(ncclCommDestroy(c[r]));
  }
};

static std::vector<void*> gBuffers;  // everything devAlloc handed out since the last freeBuffers()
template <typename T>
static T* devAlloc(size_t count) {
  void* p = nullptr;
  if (hipMalloc(&p, count * sizeof(T) + 16) != hipSuccess) exit(4);
  gBuffers.push_back(p);
  return (T*)p;
}
static std::vector<char*> gExactBuffers;
// Host memory of exactly `bytes` bytes (16-byte aligned), standing in for device memory: AddressSanitizer then
// reports the first byte a kernel touches past the end, which hipMalloc's rounding would hide.
static char* exactAlloc(size_t bytes) {
  char* p = new char[bytes ? bytes : 1];
  gExactBuffers.push_back(p);
  return p;
}
static void freeBuffers() {
  for (void* p : gBuffers) hipFree(p);
  gBuffers.clear();
  for (char* p : gExactBuffers) delete[] p;
  gExactBuffers.clear();
}

static uint16_t bf16Of(int v) {  // small integers are exact in bfloat16
  const float f = (float)v;
  return (uint16_t)(__builtin_bit_cast(uint32_t, f) >> 16);
}

// Collective 0 is an fp32 Sum of `count` elements; a second one, if asked for, a bf16 Max of 3 * count.  With two
// the order is 0, 0, 1, 0, 0, 1, ...: the context that is resident in the workgroup changes now and then, and
// every second run of collective 0 finds its context resident.
static int scenarioRepeat(int n, int count, int reps, int ncolls) {
  Ring ring(n);
  if (ncolls > 2) ncolls = 2;
  for (int c = 0; c < ncolls; c++) {
    auto& comms = ring.newComms();
    for (int r = 0; r < n; r++) {
      if (c == 0) CHECK(ofcclPrepareAllReduce((size_t)count, ncclFloat32, ncclSum, comms[r], c, ring.ctxs[r]));
      else CHECK(ofcclPrepareAllReduce((size_t)count * 3, ncclBfloat16, ncclMax, comms[r], c, ring.ctxs[r]));
    }
  }
  ring.finalize();
  std::vector<float*> send((size_t)n), recv((size_t)n);
  std::vector<uint16_t*> sendB((size_t)n), recvB((size_t)n);
  for (int r = 0; r < n; r++) {
    send[r] = devAlloc<float>((size_t)count);
    recv[r] = devAlloc<float>((size_t)count);
    sendB[r] = devAlloc<uint16_t>((size_t)count * 3);
    recvB[r] = devAlloc<uint16_t>((size_t)count * 3);
  }
  std::vector<int> want((size_t)n * ncolls, 0);
  for (int rep = 0; rep < reps; rep++) {
    const int cid = ncolls == 2 ? rep % 3 / 2 : 0;
    auto valB = [&](int r, int i) { return (i * 5 + r * 37 + rep * 3) % 200 - 100; };
    for (int r = 0; r < n; r++) {
      for (int i = 0; i < count; i++) {
        send[r][i] = (float)((i * 7 + r * 13 + rep) % 64);  // small integers: the sum is exact in any order
        recv[r][i] = -1.0f;
      }
      for (int i = 0; i < count * 3; i++) {
        sendB[r][i] = bf16Of(valB(r, i));
        recvB[r][i] = 0x7fc0;
      }
    }
    for (int r = 0; r < n; r++) {
      want[(size_t)r * ncolls + cid]++;
      if (cid == 0) CHECK(ofcclRunAllReduce(send[r], recv[r], cid, Ring::cb, &ring.flag(r, cid), ring.ctxs[r]));
      else CHECK(ofcclRunAllReduce(sendB[r], recvB[r], cid, Ring::cb, &ring.flag(r, cid), ring.ctxs[r]));
    }
    ring.waitAll(want, 120.0, "repeat");
    for (int r = 0; r < n; r++) {
      if (cid == 0) {
        for (int i = 0; i < count; i++) {
          float s = 0;
          for (int q = 0; q < n; q++) s += (float)((i * 7 + q * 13 + rep) % 64);
          if (recv[r][i] != s) {
            fprintf(stderr, "emul_stress: repeat: rep %d rank %d element %d: %g, expected %g\n", rep, r, i, recv[r][i], s);
            return 1;
          }
        }
      } else {
        for (int i = 0; i < count * 3; i++) {
          int m = valB(0, i);
          for (int q = 1; q < n; q++) m = valB(q, i) > m ? valB(q, i) : m;
          if (recvB[r][i] != bf16Of(m)) {
            fprintf(stderr, "emul_stress: repeat: rep %d rank %d bf16 element %d: %04x, expected %04x\n", rep, r, i,
                    recvB[r][i], bf16Of(m));
            return 1;
          }
        }
      }
    }
  }
  dfcclStats st;
  st.structBytes = sizeof(st);
  uint64_t saves = 0, cqes = 0;
  for (int r = 0; r < n; r++) {
    CHECK(dfcclGetStats(ring.ctxs[r], &st));
    saves += st.ctxSaves;
    cqes += st.cqesWritten;
  }
  ring.destroy();
  freeBuffers();
  printf("repeat: %d ranks x %d reps of %d elements ok, %llu completions, %llu context saves\n", n, reps, count,
         (unsigned long long)cqes, (unsigned long long)saves);
  return 0;
}

// all five collectives, int32 Sum, every rank submits them in its own order, `reps` times
static int scenarioMixed(int n, int reps) {
  const int count = 3000, root = n - 1;
  Ring ring(n);
  const char* names[5] = {"all_reduce", "reduce_scatter", "all_gather", "reduce", "broadcast"};
  for (int c = 0; c < 5; c++) {
    auto& comms = ring.newComms();
    for (int r = 0; r < n; r++) {
      switch (c) {
        case 0: CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, comms[r], c, ring.ctxs[r])); break;
        case 1: CHECK(ofcclPrepareReduceScatter(count, ncclInt32, ncclSum, comms[r], c, ring.ctxs[r])); break;
        case 2: CHECK(ofcclPrepareAllGather(count, ncclInt32, comms[r], c, ring.ctxs[r])); break;
        case 3: CHECK(ofcclPrepareReduce(count, ncclInt32, ncclSum, root, comms[r], c, ring.ctxs[r])); break;
        default: CHECK(ofcclPrepareBroadcast(count, ncclInt32, root, comms[r], c, ring.ctxs[r])); break;
      }
    }
  }
  ring.finalize();
  auto sendLen = [&](int c) { return c == 1 ? count * n : count; };
  auto recvLen = [&](int c) { return c == 2 ? count * n : count; };
  std::vector<std::vector<int32_t*>> send(5), recv(5);
  for (int c = 0; c < 5; c++)
    for (int r = 0; r < n; r++) {
      send[c].push_back(devAlloc<int32_t>((size_t)sendLen(c)));
      recv[c].push_back(devAlloc<int32_t>((size_t)recvLen(c)));
    }
  auto val = [](int c, int r, int i, int rep) { return (int32_t)(i * 31 + r * 1009 + c * 77 + rep); };
  std::vector<int> want((size_t)n * 5, 0);
  for (int rep = 0; rep < reps; rep++) {
    for (int c = 0; c < 5; c++)
      for (int r = 0; r < n; r++) {
        for (int i = 0; i < sendLen(c); i++) send[c][r][i] = val(c, r, i, rep);
        for (int i = 0; i < recvLen(c); i++) recv[c][r][i] = -7;
      }
    for (int k = 0; k < 5; k++)
      for (int r = 0; r < n; r++) {
        const int c = (k * (r % 2 ? 3 : 1) + r) % 5;  // every rank in its own order
        want[(size_t)r * 5 + c]++;
        auto* f = &ring.flag(r, c);
        switch (c) {
          case 0: CHECK(ofcclRunAllReduce(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
          case 1: CHECK(ofcclRunReduceScatter(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
          case 2: CHECK(ofcclRunAllGather(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
          case 3: CHECK(ofcclRunReduce(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
          default: CHECK(ofcclRunBroadcast(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
        }
      }
    ring.waitAll(want, 180.0, "mixed");
    for (int c = 0; c < 5; c++)
      for (int r = 0; r < n; r++) {
        if (c == 3 && r != root) continue;
        for (int i = 0; i < recvLen(c); i++) {
          int32_t e = 0;
          if (c == 0 || c == 3) for (int q = 0; q < n; q++) e += val(c, q, i, rep);
          else if (c == 1) for (int q = 0; q < n; q++) e += val(c, q, r * count + i, rep);
          else if (c == 2) e = val(c, i / count, i % count, rep);
          else e = val(c, root, i, rep);
          if (recv[c][r][i] != e) {
            fprintf(stderr, "emul_stress: mixed: rep %d %s rank %d element %d: %d, expected %d\n", rep, names[c], r, i,
                    recv[c][r][i], e);
            return 1;
          }
        }
      }
  }
  ring.destroy();
  freeBuffers();
  printf("mixed: %d ranks x %d reps of the five collectives ok\n", n, reps);
  return 0;
}

// idle exit and relaunch: one collective, a pause long enough for the daemon to leave, the collective again; then
// one rank submits and the others only after the daemon has left with the collective parked
static int scenarioRelaunch(int n) {
  const int count = 5000;
  Ring ring(n);
  auto& comms = ring.newComms();
  for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, comms[r], 0, ring.ctxs[r]));
  ring.finalize();
  std::vector<int32_t*> send, recv;
  for (int r = 0; r < n; r++) {
    send.push_back(devAlloc<int32_t>(count));
    recv.push_back(devAlloc<int32_t>(count));
  }
  std::vector<int> want((size_t)n, 0);
  for (int round = 0; round < 3; round++) {
    for (int r = 0; r < n; r++)
      for (int i = 0; i < count; i++) {
        send[r][i] = i + r * 100 + round;
        recv[r][i] = -1;
      }
    for (int r = 0; r < n; r++) {
      want[r]++;
      CHECK(ofcclRunAllReduce(send[r], recv[r], 0, Ring::cb, &ring.flag(r, 0), ring.ctxs[r]));
      if (round == 2 && r == 0) sleep(3);  // the others come after rank 0's workgroup has given up and left
    }
    ring.waitAll(want, 180.0, "relaunch");
    for (int r = 0; r < n; r++)
      for (int i = 0; i < count; i++) {
        int32_t e = 0;
        for (int q = 0; q < n; q++) e += i + q * 100 + round;
        if (recv[r][i] != e) {
          fprintf(stderr, "emul_stress: relaunch: round %d rank %d element %d: %d, expected %d\n", round, r, i, recv[r][i], e);
          return 1;
        }
      }
    if (round == 0) sleep(3);  // idle: every workgroup leaves
  }
  dfcclStats st;
  st.structBytes = sizeof(st);
  CHECK(dfcclGetStats(ring.ctxs[0], &st));
  ring.destroy();
  freeBuffers();
  printf("relaunch: ok, %llu daemon launches, %llu voluntary exits of rank 0\n", (unsigned long long)st.daemonLaunches,
         (unsigned long long)st.voluntaryQuits);
  return st.daemonLaunches >= 2 ? 0 : 1;
}

// A communicator whose collective has run cannot be registered with a new rank context (its device-side counters
// would not match the fresh context's); a new communicator can, while the daemon of the first ring is still around.
static int scenarioReuse(int n) {
  const int count = 4000;
  Ring ring(n);
  auto comms = ring.newComms();
  for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, comms[r], 0, ring.ctxs[r]));
  ring.finalize();
  std::vector<int32_t*> send, recv;
  for (int r = 0; r < n; r++) {
    send.push_back(devAlloc<int32_t>(count));
    recv.push_back(devAlloc<int32_t>(count));
    for (int i = 0; i < count; i++) send[r][i] = i + r;
  }
  std::vector<int> want((size_t)n, 1);
  for (int r = 0; r < n; r++) CHECK(ofcclRunAllReduce(send[r], recv[r], 0, Ring::cb, &ring.flag(r, 0), ring.ctxs[r]));
  ring.waitAll(want, 120.0, "reuse");
  for (int r = 0; r < n; r++) CHECK(ofcclDestroy(ring.ctxs[r]));
  // second generation of contexts
  Ring ring2(n);
  for (int r = 0; r < n; r++) {
    const ncclResult_t res = ofcclPrepareAllReduce(count, ncclInt32, ncclSum, comms[r], 0, ring2.ctxs[r]);
    if (res != ncclInvalidUsage) {
      fprintf(stderr, "emul_stress: reuse: registering a used communicator returned %d\n", (int)res);
      return 1;
    }
  }
  auto& fresh = ring2.newComms();
  for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, fresh[r], 0, ring2.ctxs[r]));
  ring2.finalize();
  for (int r = 0; r < n; r++)
    for (int i = 0; i < count; i++) recv[r][i] = -1;
  for (int r = 0; r < n; r++) CHECK(ofcclRunAllReduce(send[r], recv[r], 0, Ring::cb, &ring2.flag(r, 0), ring2.ctxs[r]));
  ring2.waitAll(want, 120.0, "reuse, second generation");
  for (int r = 0; r < n; r++)
    for (int i = 0; i < count; i++) {
      int32_t e = 0;
      for (int q = 0; q < n; q++) e += i + q;
      if (recv[r][i] != e) {
        fprintf(stderr, "emul_stress: reuse: rank %d element %d: %d, expected %d\n", r, i, recv[r][i], e);
        return 1;
      }
    }
  ring2.destroy();
  freeBuffers();
  for (int r = 0; r < n; r++) CHECK(ncclCommDestroy(comms[r]));
  printf("reuse: ok\n");
  return 0;
}

// One small non-negative integer as an element of any ncclDataType_t (exact in every type up to 2048).
static int elemSize(int dt) {
  switch (dt) {
    case ncclInt8: case ncclUint8: return 1;
    case ncclFloat16: case ncclBfloat16: return 2;
    case ncclInt32: case ncclUint32: case ncclFloat32: return 4;
    default: return 8;
  }
}
static void putElem(void* base, size_t i, int dt, int v) {
  char* p = (char*)base + i * (size_t)elemSize(dt);
  switch (dt) {
    case ncclInt8: case ncclUint8: { uint8_t x = (uint8_t)v; memcpy(p, &x, 1); break; }
    case ncclInt32: case ncclUint32: { int32_t x = v; memcpy(p, &x, 4); break; }
    case ncclInt64: case ncclUint64: { int64_t x = v; memcpy(p, &x, 8); break; }
    case ncclFloat16: { _Float16 x = (_Float16)v; memcpy(p, &x, 2); break; }
    case ncclBfloat16: { uint16_t x = bf16Of(v); memcpy(p, &x, 2); break; }
    case ncclFloat32: { float x = (float)v; memcpy(p, &x, 4); break; }
    default: { double x = (double)v; memcpy(p, &x, 8); break; }
  }
}
static bool elemIs(const void* base, size_t i, int dt, int v) {
  char want[8], got[8];
  putElem(want, 0, dt, v);
  memcpy(got, (const char*)base + i * (size_t)elemSize(dt), (size_t)elemSize(dt));
  return memcmp(want, got, (size_t)elemSize(dt)) == 0;
}

// Random collectives (kind, count, root, element type, op), every rank submits them in its own random order,
// several rounds.  Inputs are small non-negative integers, so that Sum, Max and the integer Avg have exact
// results in every element type and any result can be checked with integer arithmetic.  The knobs come from the
// environment.
static int scenarioFuzz(uint64_t seed, int rounds) {
  uint64_t x = seed * 0x9e3779b97f4a7c15ull + 12345;
  auto rnd = [&](uint64_t m) {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return (x >> 11) % m;
  };
  const int n = 2 + (int)rnd(5), ncolls = 1 + (int)rnd(7);
  // op: ncclSum / ncclMax / ncclMin / ncclAvg, or kPreMul: every rank makes its own PreMulSum operator with the
  // scalar (rank % 3) + 1, read from host memory when the operator is made or (premulDevice) from memory the
  // daemon dereferences whenever an instance starts
  constexpr int kPreMul = 100;
  struct Coll { int kind, count, root, dt, op, premulDevice; };
  auto scalarOf = [](int r) { return (r % 3) + 1; };
  std::vector<Coll> colls;
  Ring ring(n);
  for (int c = 0; c < ncolls; c++) {
    Coll k;
    k.kind = (int)rnd(5);
    const int shape = (int)rnd(4);
    k.count = shape == 0 ? 1 + (int)rnd(16) : shape == 1 ? 1 + (int)rnd(3000) : shape == 2 ? 256 * (1 + (int)rnd(40)) : 1 + (int)rnd(60000);
    k.root = (int)rnd((uint64_t)n);
    k.dt = (int)rnd(10);
    const bool isFloat = k.dt == ncclFloat16 || k.dt == ncclFloat32 || k.dt == ncclFloat64 || k.dt == ncclBfloat16;
    const int pick = (int)rnd(4);
    k.op = pick == 0 ? (int)ncclSum : pick == 1 ? (int)ncclMax : pick == 2 ? (isFloat ? (int)ncclMin : (int)ncclAvg) : kPreMul;
    k.premulDevice = (int)rnd(2);
    colls.push_back(k);
    auto& comms = ring.newComms();
    const ncclDataType_t dt = (ncclDataType_t)k.dt;
    for (int r = 0; r < n; r++) {
      ncclRedOp_t op = (ncclRedOp_t)k.op;
      if (k.op == kPreMul) {
        // one element of the type holding the rank's scalar (the buffer lives as long as the run: the daemon reads
        // it at every instance when the operator was made with ncclScalarDevice)
        char* scalar = exactAlloc((size_t)elemSize(k.dt));
        putElem(scalar, 0, k.dt, scalarOf(r));
        CHECK(ncclRedOpCreatePreMulSum(&op, scalar, dt, k.premulDevice ? ncclScalarDevice : ncclScalarHostImmediate, comms[r]));
      }
      switch (k.kind) {
        case 0: CHECK(ofcclPrepareAllReduce(k.count, dt, op, comms[r], c, ring.ctxs[r])); break;
        case 1: CHECK(ofcclPrepareReduceScatter(k.count, dt, op, comms[r], c, ring.ctxs[r])); break;
        case 2: CHECK(ofcclPrepareAllGather(k.count, dt, comms[r], c, ring.ctxs[r])); break;
        case 3: CHECK(ofcclPrepareReduce(k.count, dt, op, k.root, comms[r], c, ring.ctxs[r])); break;
        default: CHECK(ofcclPrepareBroadcast(k.count, dt, k.root, comms[r], c, ring.ctxs[r])); break;
      }
    }
  }
  ring.finalize();
  auto sendLen = [&](int c) { return colls[c].kind == 1 ? colls[c].count * n : colls[c].count; };
  auto recvLen = [&](int c) { return colls[c].kind == 2 ? colls[c].count * n : colls[c].count; };
  std::vector<std::vector<char*>> send((size_t)ncolls), recv((size_t)ncolls);
  for (int c = 0; c < ncolls; c++)
    for (int r = 0; r < n; r++) {
      // (exactly as long as the collective needs: an access past the end is AddressSanitizer's to report)
      send[c].push_back(exactAlloc((size_t)sendLen(c) * elemSize(colls[c].dt)));
      recv[c].push_back(exactAlloc((size_t)recvLen(c) * elemSize(colls[c].dt)));
    }
  auto val = [](int c, int r, int i, int rep) { return (i * 31 + r * 5 + c * 7 + rep * 3) % 4; };
  auto reduce = [&](int c, int i, int rep) {  // the reduction of element i over the ranks
    int acc = 0, mx = 0, mn = 1 << 30, scaled = 0;
    for (int q = 0; q < n; q++) {
      const int v = val(c, q, i, rep);
      acc += v;
      scaled += v * scalarOf(q);  // (at most 6 ranks x 3 x 3: exact in every element type)
      mx = v > mx ? v : mx;
      mn = v < mn ? v : mn;
    }
    switch (colls[c].op) {
      case kPreMul: return scaled;
      case ncclSum: return acc;
      case ncclMax: return mx;
      case ncclMin: return mn;
      default: return acc / n;  // ncclAvg of an integer type
    }
  };
  std::vector<int> want((size_t)n * ncolls, 0);
  for (int rep = 0; rep < rounds; rep++) {
    for (int c = 0; c < ncolls; c++)
      for (int r = 0; r < n; r++) {
        for (int i = 0; i < sendLen(c); i++) putElem(send[c][r], (size_t)i, colls[c].dt, val(c, r, i, rep));
        memset(recv[c][r], 0x5a, (size_t)recvLen(c) * elemSize(colls[c].dt));
      }
    // per-rank random order; ranks are interleaved at random as well
    std::vector<std::vector<int>> order((size_t)n);
    for (int r = 0; r < n; r++) {
      for (int c = 0; c < ncolls; c++) order[r].push_back(c);
      for (int i = ncolls - 1; i > 0; i--) std::swap(order[r][i], order[r][rnd((uint64_t)i + 1)]);
    }
    std::vector<int> next((size_t)n, 0);
    for (int left = n * ncolls; left > 0;) {
      const int r = (int)rnd((uint64_t)n);
      if (next[r] >= ncolls) continue;
      const int c = order[r][next[r]++];
      left--;
      want[(size_t)r * ncolls + c]++;
      auto* f = &ring.flag(r, c);
      switch (colls[c].kind) {
        case 0: CHECK(ofcclRunAllReduce(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
        case 1: CHECK(ofcclRunReduceScatter(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
        case 2: CHECK(ofcclRunAllGather(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
        case 3: CHECK(ofcclRunReduce(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
        default: CHECK(ofcclRunBroadcast(send[c][r], recv[c][r], c, Ring::cb, f, ring.ctxs[r])); break;
      }
      if (rnd(4) == 0) usleep((useconds_t)rnd(3000));
    }
    ring.waitAll(want, 240.0, "fuzz");
    for (int c = 0; c < ncolls; c++)
      for (int r = 0; r < n; r++) {
        const int kind = colls[c].kind, count = colls[c].count, root = colls[c].root;
        if (kind == 3 && r != root) continue;
        for (int i = 0; i < recvLen(c); i++) {
          int e;
          if (kind == 0 || kind == 3) e = reduce(c, i, rep);
          else if (kind == 1) e = reduce(c, r * count + i, rep);
          else if (kind == 2) e = val(c, i / count, i % count, rep);
          else e = val(c, root, i, rep);
          if (!elemIs(recv[c][r], (size_t)i, colls[c].dt, e)) {
            fprintf(stderr, "emul_stress: fuzz seed %llu: round %d collective %d (kind %d, type %d, op %d, count %d, root %d) "
                    "rank %d of %d element %d: expected %d\n", (unsigned long long)seed, rep, c, kind, colls[c].dt,
                    colls[c].op, count, root, r, n, i, e);
            return 1;
          }
        }
      }
  }
  ring.destroy();
  freeBuffers();
  printf("fuzz: seed %llu: %d ranks, %d collectives, %d rounds ok\n", (unsigned long long)seed, n, ncolls, rounds);
  return 0;
}

// Back-pressure of the queues: `colls` small all-reduces, every rank has two threads that submit all of them
// `rounds` times (a collective again as soon as its previous instance has called back), the last rank starts
// 200 ms late so that the others pile up parked collectives, and the callback sleeps for `cbSleepUs` on the
// poller thread.  Checks: every submission got exactly one callback, results are right, and (when the queue was
// made small) the full-queue path was taken.
static int scenarioBackpressure(int n, int ncolls, int rounds, int cbSleepUs) {
  const int count = 600;
  Ring ring(n);
  for (int c = 0; c < ncolls; c++) {
    auto& comms = ring.newComms();
    for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, comms[r], c, ring.ctxs[r]));
  }
  ring.finalize();
  struct CbArg { std::atomic<int> calls{0}; int sleepUs = 0; };
  std::vector<CbArg> args((size_t)n * ncolls);
  for (auto& a : args) a.sleepUs = cbSleepUs;
  auto cb = +[](int, void* p) {
    CbArg* a = (CbArg*)p;
    if (a->sleepUs > 0) usleep((useconds_t)a->sleepUs);
    a->calls.fetch_add(1);
    return 0;
  };
  std::vector<std::vector<int32_t*>> send((size_t)ncolls), recv((size_t)ncolls);
  for (int c = 0; c < ncolls; c++)
    for (int r = 0; r < n; r++) {
      send[c].push_back(devAlloc<int32_t>(count));
      recv[c].push_back(devAlloc<int32_t>(count));
      for (int i = 0; i < count; i++) {
        send[c][r][i] = i + 3 * r + 7 * c;
        recv[c][r][i] = -1;
      }
    }
  std::atomic<int> failures{0};
  std::vector<std::thread> threads;
  for (int r = 0; r < n; r++)
    for (int half = 0; half < 2; half++)
      threads.emplace_back([&, r, half] {
        if (r == n - 1) usleep(200000);
        for (int round = 0; round < rounds; round++)
          for (int c = half; c < ncolls; c += 2) {
            CbArg& a = args[(size_t)r * ncolls + c];
            // (a second Run of a collective waits for the first inside the library; the test adds no wait of its own)
            const ncclResult_t res = ofcclRunAllReduce(send[c][r], recv[c][r], c, cb, &a, ring.ctxs[r]);
            if (res != ncclSuccess) failures.fetch_add(1);
          }
      });
  for (auto& t : threads) t.join();
  const auto t0 = std::chrono::steady_clock::now();
  for (;;) {
    bool all = true;
    for (auto& a : args) all = all && a.calls.load() >= rounds;
    if (all) break;
    if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 240.0) {
      fprintf(stderr, "emul_stress: backpressure: callbacks missing after 240 s\n");
      dfcclDumpState(ring.ctxs[0]);
      emulDumpThreads();
      return 3;
    }
    usleep(1000);
  }
  usleep(50000);  // a callback too many would show up now
  for (auto& a : args)
    if (a.calls.load() != rounds) {
      fprintf(stderr, "emul_stress: backpressure: %d callbacks for %d submissions\n", a.calls.load(), rounds);
      return 1;
    }
  for (int c = 0; c < ncolls; c++)
    for (int r = 0; r < n; r++)
      for (int i = 0; i < count; i++) {
        int32_t e = 0;
        for (int q = 0; q < n; q++) e += i + 3 * q + 7 * c;
        if (recv[c][r][i] != e) {
          fprintf(stderr, "emul_stress: backpressure: collective %d rank %d element %d: %d, expected %d\n", c, r, i, recv[c][r][i], e);
          return 1;
        }
      }
  uint64_t fullWaits = 0, cqes = 0;
  dfcclStats st;
  st.structBytes = sizeof(st);
  for (int r = 0; r < n; r++) {
    CHECK(dfcclGetStats(ring.ctxs[r], &st));
    fullWaits += st.sqFullWaits;
    cqes += st.cqesWritten;
  }
  ring.destroy();
  freeBuffers();
  if (failures.load() != 0 || cqes != (uint64_t)n * ncolls * rounds) {
    fprintf(stderr, "emul_stress: backpressure: %d failed submissions, %llu completions\n", failures.load(), (unsigned long long)cqes);
    return 1;
  }
  const char* cap = getenv("DFCCL_SQ_CAPACITY");
  if (cap != nullptr && atoi(cap) < ncolls / 2 && fullWaits == 0) {
    fprintf(stderr, "emul_stress: backpressure: the queue of %s entries was never found full\n", cap);
    return 1;
  }
  printf("backpressure: %d ranks x %d collectives x %d rounds ok, %llu completions, queue found full %llu times\n", n,
         ncolls, rounds, (unsigned long long)cqes, (unsigned long long)fullWaits);
  return 0;
}

// Two rings on one daemon.  Ring A keeps running small all-reduces; ring B stays silent until its workgroups have
// left for idleness (TOLERANT_UNPROGRESSED_CNT is small), then submits.  B's submission is only seen after a new
// launch, which needs A's workgroups to leave too although they are busy.
static int scenarioTwoRings(int n) {
  const int count = 500;
  Ring a(n), b(n);
  auto& ca = a.newComms();
  for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, ca[r], 0, a.ctxs[r]));
  auto& cb = b.newComms();
  for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, cb[r], 0, b.ctxs[r]));
  a.finalize();
  b.finalize();
  std::vector<int32_t*> sa, ra, sb, rb;
  for (int r = 0; r < n; r++) {
    sa.push_back(devAlloc<int32_t>(count));
    ra.push_back(devAlloc<int32_t>(count));
    sb.push_back(devAlloc<int32_t>(count));
    rb.push_back(devAlloc<int32_t>(count));
    for (int i = 0; i < count; i++) {
      sa[r][i] = i + r;
      sb[r][i] = 5 * i - r;
    }
  }
  std::atomic<bool> stop{false};
  std::atomic<int> repsA{0};
  std::thread busy([&] {
    std::vector<int> want((size_t)n, 0);
    while (!stop.load()) {
      for (int r = 0; r < n; r++) {
        want[r]++;
        CHECK(ofcclRunAllReduce(sa[r], ra[r], 0, Ring::cb, &a.flag(r, 0), a.ctxs[r]));
      }
      a.waitAll(want, 180.0, "two rings, the busy ring");
      repsA.fetch_add(1);
    }
  });
  sleep(4);  // ring B's workgroups have seen nothing for long and have left
  std::vector<int> wantB((size_t)n, 1);
  for (int r = 0; r < n; r++) CHECK(ofcclRunAllReduce(sb[r], rb[r], 0, Ring::cb, &b.flag(r, 0), b.ctxs[r]));
  b.waitAll(wantB, 120.0, "two rings, the ring that had gone idle");
  stop.store(true);
  busy.join();
  for (int r = 0; r < n; r++)
    for (int i = 0; i < count; i++) {
      int32_t eb = 0, ea = 0;
      for (int q = 0; q < n; q++) {
        eb += 5 * i - q;
        ea += i + q;
      }
      if (rb[r][i] != eb || ra[r][i] != ea) {
        fprintf(stderr, "emul_stress: tworings: rank %d element %d: %d / %d, expected %d / %d\n", r, i, ra[r][i], rb[r][i], ea, eb);
        return 1;
      }
    }
  dfcclStats st;
  st.structBytes = sizeof(st);
  CHECK(dfcclGetStats(b.ctxs[0], &st));
  a.destroy();
  b.destroy();
  freeBuffers();
  printf("tworings: ok, %d collectives of the busy ring, %llu daemon launches\n", repsA.load(), (unsigned long long)st.daemonLaunches);
  return st.daemonLaunches >= 2 ? 0 : 1;
}

// With EMUL_NEVER_LEAVE=1 no workgroup ever leaves the kernel.  One collective runs, then Destroy: after its wait
// (DFCCL_DESTROY_WAIT_MS) and the abort's (DFCCL_ABORT_WAIT_MS) the library has to report and end the process
// with status 70; returning from Destroy, or blocking for good, is the failure.
static int scenarioStuck(int n) {
  const int count = 1000;
  Ring ring(n);
  auto& comms = ring.newComms();
  for (int r = 0; r < n; r++) CHECK(ofcclPrepareAllReduce(count, ncclInt32, ncclSum, comms[r], 0, ring.ctxs[r]));
  ring.finalize();
  std::vector<int32_t*> send, recv;
  for (int r = 0; r < n; r++) {
    send.push_back(devAlloc<int32_t>(count));
    recv.push_back(devAlloc<int32_t>(count));
    for (int i = 0; i < count; i++) send[r][i] = i;
  }
  std::vector<int> want((size_t)n, 1);
  for (int r = 0; r < n; r++) CHECK(ofcclRunAllReduce(send[r], recv[r], 0, Ring::cb, &ring.flag(r, 0), ring.ctxs[r]));
  ring.waitAll(want, 120.0, "stuck");
  printf("stuck: collective done, destroying\n");
  ofcclDestroy(ring.ctxs[0]);
  printf("stuck: ofcclDestroy returned although the daemon cannot have left\n");
  return 1;
}

int main(int argc, char** argv) {
  setvbuf(stdout, nullptr, _IOLBF, 0);
  setenv("DFCCL_STATS_WAIT_MS", "5000", 0);  // emulated workgroups answer a request for their counters slowly
  const std::string mode = argc > 1 ? argv[1] : "";
  if (mode == "repeat" && argc == 6) return scenarioRepeat(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]));
  if (mode == "mixed" && argc == 4) return scenarioMixed(atoi(argv[2]), atoi(argv[3]));
  if (mode == "relaunch" && argc == 3) return scenarioRelaunch(atoi(argv[2]));
  if (mode == "reuse" && argc == 3) return scenarioReuse(atoi(argv[2]));
  if (mode == "fuzz" && argc == 4) return scenarioFuzz(strtoull(argv[2], nullptr, 10), atoi(argv[3]));
  if (mode == "backpressure" && argc == 6) return scenarioBackpressure(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]));
  if (mode == "tworings" && argc == 3) return scenarioTwoRings(atoi(argv[2]));
  if (mode == "stuck" && argc == 3) return scenarioStuck(atoi(argv[2]));
  fprintf(stderr, "usage: emul_stress repeat <ranks> <count> <reps> <colls> | mixed <ranks> <reps> | relaunch <ranks> | reuse <ranks> | fuzz <seed> <rounds>\n");
  return 64;
}
