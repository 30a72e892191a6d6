// Native driver for the timing workloads of the DFCCL data path.  It uses only
// the public C ABI (include/ofccl.h) plus HIP for buffers, with one host thread
// per virtual rank, the way one process per rank would drive the reference.
//
//   dfccl_bench latency   --ranks 4 --bytes 4096 --iters 2000
//   dfccl_bench disorder  --ranks 4 --colls 256 --min-bytes 4096 --max-bytes 4194304
//   dfccl_bench allreduce --ranks 8 --bytes 67108864 --dtype bf16 --iters 10
//   dfccl_bench buckets   --ranks 4 --colls 40 --elems 25000000 --dtype int32
//   dfccl_bench collective --kind reduce_scatter|all_gather|reduce|broadcast --ranks 8 --bytes 67108864 --dtype bf16
//
// Every mode prints one JSON object on stdout.  Inputs are small integers
// (rank + 1) so that every reduction is exact in every dtype and the outputs can
// be verified element by element on the host.
#include <hip/hip_runtime.h>

#include <signal.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../../include/ofccl.h"

#define CK(x)                                                                          \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      exit(1);                                                                         \
    }                                                                                  \
  } while (0)
#define NK(x)                                                                          \
  do {                                                                                 \
    ncclResult_t r_ = (x);                                                             \
    if (r_ != ncclSuccess) {                                                           \
      fprintf(stderr, "dfccl error %s at %s:%d\n", ncclGetErrorString(r_), __FILE__, __LINE__); \
      exit(1);                                                                         \
    }                                                                                  \
  } while (0)

static uint64_t nowNs() {
  return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
             std::chrono::steady_clock::now().time_since_epoch()).count();
}

struct Args {
  std::string mode;
  int ranks = 4, colls = 256, iters = 1000, warmup = 50;
  size_t bytes = 4096, minBytes = 4096, maxBytes = 4 << 20, elems = 25000000;
  std::string dtype = "fp16", kind = "reduce_scatter";
  uint64_t seed = 3;
  int timeoutS = 20;
};

static int dtypeCode(const std::string& s) {
  if (s == "fp16") return ncclFloat16;
  if (s == "bf16") return ncclBfloat16;
  if (s == "fp32") return ncclFloat32;
  if (s == "int32") return ncclInt32;
  if (s == "int8") return ncclInt8;
  fprintf(stderr, "unknown dtype %s\n", s.c_str());
  exit(1);
}
static int dtypeSize(int dt) { return dt == ncclInt8 ? 1 : (dt == ncclFloat16 || dt == ncclBfloat16) ? 2 : 4; }

// bit pattern of the small integer v in dtype dt
static uint32_t encodeValue(int dt, int v) {
  if (dt == ncclInt32) return (uint32_t)v;
  if (dt == ncclInt8) return (uint32_t)(uint8_t)v;
  float f = (float)v;
  uint32_t u;
  memcpy(&u, &f, 4);
  if (dt == ncclFloat32) return u;
  if (dt == ncclBfloat16) return u >> 16;  // small integers are exact in bf16
  // fp16 of a small positive integer
  if (v == 0) return 0;
  int e = (int)((u >> 23) & 0xff) - 127 + 15;
  return (uint32_t)((e << 10) | ((u >> 13) & 0x3ff));
}

static void fillBuffer(void* p, size_t elems, int dt, int v) {
  const uint32_t bits = encodeValue(dt, v);
  const int es = dtypeSize(dt);
  if (es == 4) CK(hipMemsetD32((hipDeviceptr_t)p, (int)bits, elems));
  else if (es == 2) CK(hipMemsetD16((hipDeviceptr_t)p, (unsigned short)bits, elems));
  else CK(hipMemsetD8((hipDeviceptr_t)p, (unsigned char)bits, elems));
}

// every element of the device buffer equals v?  (checks the whole buffer)
static bool verifyBuffer(const void* p, size_t elems, int dt, int v, std::vector<char>& scratch) {
  const int es = dtypeSize(dt);
  scratch.resize(elems * es);
  CK(hipMemcpy(scratch.data(), p, elems * es, hipMemcpyDeviceToHost));
  const uint32_t bits = encodeValue(dt, v);
  if (es == 4) { const uint32_t* q = (const uint32_t*)scratch.data(); for (size_t i = 0; i < elems; i++) if (q[i] != bits) return false; }
  else if (es == 2) { const uint16_t* q = (const uint16_t*)scratch.data(); for (size_t i = 0; i < elems; i++) if (q[i] != (uint16_t)bits) return false; }
  else { const uint8_t* q = (const uint8_t*)scratch.data(); for (size_t i = 0; i < elems; i++) if (q[i] != (uint8_t)bits) return false; }
  return true;
}

struct Flag {
  std::atomic<int> done{0};
  char pad[60];
};
static int onDone(int, void* arg) {
  ((Flag*)arg)->done.store(1, std::memory_order_release);
  return 0;
}

// Set when a rank has given up waiting (or the process was told to stop): every wait in the driver ends then, so
// that the run is torn down in order (a driver that is killed while the daemon kernel is resident leaves the GPU
// with a kernel nobody will ever stop).
static std::atomic<int> gGiveUp{0};

struct SpinBarrier {
  std::atomic<int> count{0};
  std::atomic<int> gen{0};
  int n;
  explicit SpinBarrier(int n_) : n(n_) {}
  void wait() {
    const int g = gen.load(std::memory_order_acquire);
    if (count.fetch_add(1, std::memory_order_acq_rel) == n - 1) {
      count.store(0, std::memory_order_release);
      gen.fetch_add(1, std::memory_order_acq_rel);
    } else {
      while (gen.load(std::memory_order_acquire) == g && !gGiveUp.load(std::memory_order_acquire)) __builtin_ia32_pause();
    }
  }
};

static double pct(std::vector<double>& v, double p) {
  if (v.empty()) return 0;
  std::sort(v.begin(), v.end());
  size_t i = (size_t)(p * (v.size() - 1) + 0.5);
  return v[i];
}

static bool waitFlag(Flag& f, int timeoutS) {
  const uint64_t deadline = nowNs() + (uint64_t)timeoutS * 1000000000ull;
  uint64_t spins = 0;
  while (!f.done.load(std::memory_order_acquire)) {
    __builtin_ia32_pause();
    if ((++spins & 0xfff) == 0 && (gGiveUp.load(std::memory_order_acquire) || nowNs() > deadline)) {
      gGiveUp.store(1, std::memory_order_release);
      return false;
    }
  }
  return true;
}

struct World {
  int n;
  std::vector<ofcclRankCtx_t> ctx;
  std::vector<std::vector<ncclComm_t>> comms;  // [coll][rank]
  explicit World(int n_) : n(n_), ctx(n_) {
    for (int r = 0; r < n; r++) NK(ofcclInitRankCtx(&ctx[r], r));
  }
  void prepareAllReduce(int collId, size_t count, int dt) {
    ncclUniqueId id;
    NK(ncclGetUniqueId(&id));
    std::vector<ncclComm_t> c(n);
    for (int r = 0; r < n; r++) {
      NK(ncclCommInitRank(&c[r], n, id, r));
      NK(ofcclPrepareAllReduce(count, (ncclDataType_t)dt, ncclSum, c[r], collId, ctx[r]));
    }
    comms.push_back(c);
  }
  // kind: 1 reduce-scatter, 2 all-gather, 3 reduce, 4 broadcast (count as the respective Prepare call takes it)
  void prepareKind(int kind, int collId, size_t count, int dt, int root) {
    ncclUniqueId id;
    NK(ncclGetUniqueId(&id));
    std::vector<ncclComm_t> c(n);
    for (int r = 0; r < n; r++) {
      NK(ncclCommInitRank(&c[r], n, id, r));
      const ncclDataType_t t = (ncclDataType_t)dt;
      if (kind == 1) NK(ofcclPrepareReduceScatter(count, t, ncclSum, c[r], collId, ctx[r]));
      else if (kind == 2) NK(ofcclPrepareAllGather(count, t, c[r], collId, ctx[r]));
      else if (kind == 3) NK(ofcclPrepareReduce(count, t, ncclSum, root, c[r], collId, ctx[r]));
      else NK(ofcclPrepareBroadcast(count, t, root, c[r], collId, ctx[r]));
    }
    comms.push_back(c);
  }
  void finalize() {
    for (int r = 0; r < n; r++) NK(ofcclFinalizeRankCtx7StartHostThrds(ctx[r]));
  }
  dfcclStats stats() {
    dfcclStats t{};
    for (int r = 0; r < n; r++) {
      dfcclStats s{};
      s.structBytes = sizeof(s);
      NK(dfcclGetStats(ctx[r], &s));
      t.sqesRead += s.sqesRead; t.cqesWritten += s.cqesWritten; t.ctxSaves += s.ctxSaves; t.ctxLoads += s.ctxLoads;
      t.voluntaryQuits += s.voluntaryQuits; t.forcedQuits += s.forcedQuits; t.slicesMoved += s.slicesMoved;
      t.sqFullWaits += s.sqFullWaits;
      t.daemonLaunches = std::max(t.daemonLaunches, s.daemonLaunches);
    }
    return t;
  }
  // what the daemon has done so far, rank by rank (printed when a run is given up)
  void report() {
    (void)dfcclDumpState(ctx[0]);
    for (int r = 0; r < n; r++) {
      dfcclStats s{};
      s.structBytes = sizeof(s);
      if (dfcclGetStats(ctx[r], &s) != ncclSuccess) continue;
      fprintf(stderr, "rank %d: sqes read %llu, cqes written %llu, ctx saves %llu, loads %llu, slices moved %llu, "
              "voluntary quits %llu, launches %llu\n", r, (unsigned long long)s.sqesRead,
              (unsigned long long)s.cqesWritten, (unsigned long long)s.ctxSaves, (unsigned long long)s.ctxLoads,
              (unsigned long long)s.slicesMoved, (unsigned long long)s.voluntaryQuits,
              (unsigned long long)s.daemonLaunches);
    }
  }
  void destroy() {
    for (int r = 0; r < n; r++) NK(ofcclDestroy(ctx[r]));
    for (auto& c : comms)
      for (auto h : c) NK(ncclCommDestroy(h));
  }
};

// ---- latency: one small all-reduce, all ranks submit together, repeated --------------------------
static int runLatency(const Args& a) {
  const int n = a.ranks, dt = dtypeCode(a.dtype), es = dtypeSize(dt);
  const size_t count = a.bytes / es;
  World w(n);
  w.prepareAllReduce(0, count, dt);
  w.finalize();
  std::vector<void*> send(n), recv(n);
  for (int r = 0; r < n; r++) {
    CK(hipMalloc(&send[r], a.bytes));
    CK(hipMalloc(&recv[r], a.bytes));
    fillBuffer(send[r], count, dt, r + 1);
    fillBuffer(recv[r], count, dt, 0);
  }
  CK(hipStreamSynchronize(nullptr));
  const int total = a.iters + a.warmup;
  std::vector<std::vector<double>> lat(n);
  std::vector<Flag> flags(n);
  SpinBarrier bar(n);
  std::atomic<int> failed{0};
  std::vector<std::thread> th;
  for (int r = 0; r < n; r++) {
    th.emplace_back([&, r] {
      CK(hipSetDevice(0));
      for (int it = 0; it < total && !failed.load() && !gGiveUp.load(); it++) {
        flags[r].done.store(0, std::memory_order_release);
        bar.wait();
        NK(ofcclRunAllReduce(send[r], recv[r], 0, onDone, &flags[r], w.ctx[r]));
        if (!waitFlag(flags[r], a.timeoutS)) { failed.store(1); fprintf(stderr, "rank %d timed out at iter %d\n", r, it); break; }
        uint64_t s, c;
        NK(dfcclGetCollTiming(w.ctx[r], 0, &s, &c));
        if (it >= a.warmup) lat[r].push_back((double)(c - s) / 1000.0);
      }
    });
  }
  for (auto& t : th) t.join();
  std::vector<char> scratch;
  bool ok = !failed.load() && !gGiveUp.load();
  if (!ok) w.report();
  for (int r = 0; r < n && ok; r++) ok = verifyBuffer(recv[r], count, dt, n * (n + 1) / 2, scratch);
  std::vector<double> all;
  for (auto& v : lat) all.insert(all.end(), v.begin(), v.end());
  dfcclStats st = w.stats();
  w.destroy();
  printf("{\"mode\": \"latency\", \"ranks\": %d, \"bytes\": %zu, \"dtype\": \"%s\", \"iters\": %d, \"correct\": %s, "
         "\"p50_us\": %.2f, \"p90_us\": %.2f, \"p99_us\": %.2f, \"min_us\": %.2f, \"max_us\": %.2f, "
         "\"ctx_saves\": %llu, \"daemon_launches\": %llu}\n",
         n, a.bytes, a.dtype.c_str(), a.iters, ok ? "true" : "false", pct(all, 0.5), pct(all, 0.9), pct(all, 0.99),
         all.empty() ? 0.0 : all.front(), all.empty() ? 0.0 : all.back(), (unsigned long long)st.ctxSaves,
         (unsigned long long)st.daemonLaunches);
  return ok ? 0 : 1;
}

// ---- disorder: many registered all-reduces, every rank submits them in its own random order ------
static uint64_t splitmix(uint64_t& s) {
  uint64_t z = (s += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

static int runDisorder(const Args& a) {
  const int n = a.ranks, nc = a.colls, dt = dtypeCode(a.dtype), es = dtypeSize(dt);
  uint64_t s = a.seed;
  std::vector<size_t> bytes(nc);
  for (int c = 0; c < nc; c++) {
    const double u = (double)(splitmix(s) >> 11) / (double)(1ull << 53);
    double b = std::exp(std::log((double)a.minBytes) + u * (std::log((double)a.maxBytes) - std::log((double)a.minBytes)));
    bytes[c] = std::max<size_t>(16, ((size_t)b / 16) * 16);
  }
  bytes[0] = a.minBytes;  // make sure the smallest bucket is populated
  World w(n);
  for (int c = 0; c < nc; c++) w.prepareAllReduce(c, bytes[c] / es, dt);
  w.finalize();
  std::vector<std::vector<void*>> send(nc, std::vector<void*>(n)), recv(nc, std::vector<void*>(n));
  for (int c = 0; c < nc; c++)
    for (int r = 0; r < n; r++) {
      CK(hipMalloc(&send[c][r], bytes[c]));
      CK(hipMalloc(&recv[c][r], bytes[c]));
      fillBuffer(send[c][r], bytes[c] / es, dt, r + 1);
      fillBuffer(recv[c][r], bytes[c] / es, dt, 0);
    }
  CK(hipStreamSynchronize(nullptr));
  std::vector<std::vector<int>> order(n, std::vector<int>(nc));
  for (int r = 0; r < n; r++) {
    uint64_t sr = 30 + r;
    for (int c = 0; c < nc; c++) order[r][c] = c;
    for (int c = nc - 1; c > 0; c--) std::swap(order[r][c], order[r][splitmix(sr) % (uint64_t)(c + 1)]);
  }
  std::vector<Flag> flags((size_t)n * nc);
  SpinBarrier bar(n);
  std::atomic<int> failed{0};
  std::vector<std::thread> th;
  const uint64_t t0 = nowNs();
  std::atomic<uint64_t> tEnd{0};
  for (int r = 0; r < n; r++) {
    th.emplace_back([&, r] {
      CK(hipSetDevice(0));
      bar.wait();
      for (int i = 0; i < nc; i++) {
        const int c = order[r][i];
        NK(ofcclRunAllReduce(send[c][r], recv[c][r], c, onDone, &flags[(size_t)r * nc + c], w.ctx[r]));
      }
      for (int c = 0; c < nc; c++)
        if (!waitFlag(flags[(size_t)r * nc + c], a.timeoutS)) { failed.store(1); fprintf(stderr, "rank %d coll %d timed out (deadlock?)\n", r, c); return; }
      uint64_t t = nowNs(), prev = tEnd.load();
      while (prev < t && !tEnd.compare_exchange_weak(prev, t)) {}
    });
  }
  for (auto& t : th) t.join();
  bool ok = !failed.load() && !gGiveUp.load();
  if (!ok) w.report();
  std::vector<double> all, small;
  for (int r = 0; r < n && ok; r++)
    for (int c = 0; c < nc; c++) {
      uint64_t sN, cN;
      NK(dfcclGetCollTiming(w.ctx[r], c, &sN, &cN));
      const double us = (double)(cN - sN) / 1000.0;
      all.push_back(us);
      if (bytes[c] <= 2 * a.minBytes) small.push_back(us);
    }
  std::vector<char> scratch;
  for (int c = 0; c < nc && ok; c++)
    for (int r = 0; r < n && ok; r++) ok = verifyBuffer(recv[c][r], bytes[c] / es, dt, n * (n + 1) / 2, scratch);
  dfcclStats st = w.stats();
  w.destroy();
  size_t totalBytes = 0;
  for (auto b : bytes) totalBytes += b;
  printf("{\"mode\": \"disorder\", \"ranks\": %d, \"colls\": %d, \"dtype\": \"%s\", \"min_bytes\": %zu, \"max_bytes\": %zu, "
         "\"total_bytes_per_rank\": %zu, \"deadlocks\": %d, \"correct\": %s, \"wall_ms\": %.3f, "
         "\"p50_us\": %.1f, \"p90_us\": %.1f, \"p99_us\": %.1f, \"small_bucket_count\": %zu, \"small_bucket_p50_us\": %.1f, "
         "\"preemptions_ctx_saves\": %llu, \"ctx_loads\": %llu, \"cqes\": %llu, \"sq_full_waits\": %llu}\n",
         n, nc, a.dtype.c_str(), a.minBytes, a.maxBytes, totalBytes, failed.load(), ok ? "true" : "false",
         (double)(tEnd.load() - t0) / 1e6, pct(all, 0.5), pct(all, 0.9), pct(all, 0.99), small.size(), pct(small, 0.5),
         (unsigned long long)st.ctxSaves, (unsigned long long)st.ctxLoads, (unsigned long long)st.cqesWritten,
         (unsigned long long)st.sqFullWaits);
  return ok ? 0 : 1;
}

// ---- allreduce / buckets: throughput of large all-reduces ------------------------------------------
static int runBuckets(const Args& a, bool single) {
  const int n = a.ranks, dt = dtypeCode(a.dtype), es = dtypeSize(dt);
  const int nc = single ? 1 : a.colls;
  const size_t count = single ? a.bytes / es : a.elems;
  const size_t bytes = count * es;
  World w(n);
  for (int c = 0; c < nc; c++) w.prepareAllReduce(c, count, dt);
  w.finalize();
  dfcclCollGeometry geom{};
  NK(dfcclGetCollGeometry(w.ctx[0], 0, &geom));
  std::vector<std::vector<void*>> send(nc, std::vector<void*>(n)), recv(nc, std::vector<void*>(n));
  for (int c = 0; c < nc; c++)
    for (int r = 0; r < n; r++) {
      CK(hipMalloc(&send[c][r], bytes));
      CK(hipMalloc(&recv[c][r], bytes));
      fillBuffer(send[c][r], count, dt, r + 1);
      fillBuffer(recv[c][r], count, dt, 0);
    }
  CK(hipStreamSynchronize(nullptr));
  std::vector<Flag> flags((size_t)n * nc);
  SpinBarrier bar(n);
  std::atomic<int> failed{0};
  const int total = a.iters + (single ? 2 : 1);
  std::vector<double> ms;
  std::vector<uint64_t> tStart(total), tStop(total);
  std::vector<std::atomic<uint64_t>> endNs(total);
  for (auto& e : endNs) e.store(0);
  std::vector<double> lastSubmit(n, 0), lastComplete(n, 0), lastSeen(n, 0);
  std::vector<std::thread> th;
  for (int r = 0; r < n; r++) {
    th.emplace_back([&, r] {
      CK(hipSetDevice(0));
      for (int it = 0; it < total && !failed.load() && !gGiveUp.load(); it++) {
        for (int c = 0; c < nc; c++) flags[(size_t)r * nc + c].done.store(0);
        bar.wait();
        if (r == 0) tStart[it] = nowNs();
        for (int c = 0; c < nc; c++)
          NK(ofcclRunAllReduce(send[c][r], recv[c][r], c, onDone, &flags[(size_t)r * nc + c], w.ctx[r]));
        for (int c = 0; c < nc; c++)
          if (!waitFlag(flags[(size_t)r * nc + c], a.timeoutS)) { failed.store(1); fprintf(stderr, "rank %d coll %d timed out\n", r, c); return; }
        uint64_t t = nowNs(), prev = endNs[it].load();
        while (prev < t && !endNs[it].compare_exchange_weak(prev, t)) {}
        if (it == total - 1) {
          uint64_t sN = 0, cN = 0;
          NK(dfcclGetCollTiming(w.ctx[r], nc - 1, &sN, &cN));
          lastSubmit[r] = (double)(sN - tStart[it]) / 1000.0;
          lastComplete[r] = (double)(cN - tStart[it]) / 1000.0;
          lastSeen[r] = (double)(t - tStart[it]) / 1000.0;
        }
        bar.wait();
      }
    });
  }
  for (auto& t : th) t.join();
  bool ok = !failed.load() && !gGiveUp.load();
  if (!ok) w.report();
  for (int it = (single ? 2 : 1); it < total && ok; it++) ms.push_back((double)(endNs[it].load() - tStart[it]) / 1e6);
  std::vector<char> scratch;
  for (int c = 0; c < nc && ok; c += std::max(1, nc / 4))
    for (int r = 0; r < n && ok; r++) ok = verifyBuffer(recv[c][r], count, dt, n * (n + 1) / 2, scratch);
  dfcclStats st = w.stats();
  w.destroy();
  const double best = ms.empty() ? 0 : *std::min_element(ms.begin(), ms.end());
  const double med = pct(ms, 0.5);
  if (getenv("DFCCL_BENCH_VERBOSE")) {
    fprintf(stderr, "iterations (ms):");
    for (int it = (single ? 2 : 1); it < total; it++) fprintf(stderr, " %.3f", (double)(endNs[it].load() - tStart[it]) / 1e6);
    fprintf(stderr, "\n");
    // last iteration, microseconds after rank 0's start stamp: last entry written, last completion seen by the
    // poller, waiting thread released
    for (int r = 0; r < n; r++)
      fprintf(stderr, "rank %d: submitted %.1f  completion seen %.1f  thread released %.1f (iteration %.1f)\n", r,
              lastSubmit[r], lastComplete[r], lastSeen[r], ms.empty() ? 0.0 : ms.back() * 1000.0);
  }
  // bytes the schedule moves, all ranks together: the FIFO ring reads and writes every staged slice
  // ((6n-4)/n * N per rank), the direct protocol reads every input once and writes every output once (2 N)
  const double perRank = geom.protocol == 1 ? 2.0 : (6.0 * n - 4.0) / n;
  const double sched = perRank * (double)bytes * n * nc;
  printf("{\"mode\": \"%s\", \"ranks\": %d, \"colls\": %d, \"dtype\": \"%s\", \"bytes_per_rank_per_coll\": %zu, "
         "\"protocol\": \"%s\", \"channels\": %d, \"chunk_bytes\": %lld, \"iters\": %d, \"correct\": %s, \"best_ms\": %.4f, "
         "\"median_ms\": %.4f, \"algbw_GBps\": %.1f, \"busbw_GBps\": %.1f, \"moved_GBps\": %.1f, \"ctx_saves\": %llu}\n",
         single ? "allreduce" : "buckets", n, nc, a.dtype.c_str(), bytes, geom.protocol == 1 ? "direct" : "fifo",
         geom.nChannels,
         (long long)geom.chunkElems * es, a.iters, ok ? "true" : "false", best, med,
         best > 0 ? (double)bytes * nc / (best * 1e-3) / 1e9 : 0, best > 0 ? (double)bytes * nc / (best * 1e-3) / 1e9 * 2 * (n - 1) / n : 0,
         best > 0 ? sched / (best * 1e-3) / 1e9 : 0, (unsigned long long)st.ctxSaves);
  return ok ? 0 : 1;
}

// ---- collective: one large reduce-scatter / all-gather / reduce / broadcast ----------------------
static int runCollective(const Args& a) {
  const int n = a.ranks, dt = dtypeCode(a.dtype), es = dtypeSize(dt), root = 0;
  const int kind = a.kind == "reduce_scatter" ? 1 : a.kind == "all_gather" ? 2 : a.kind == "reduce" ? 3 : a.kind == "broadcast" ? 4 : 0;
  if (kind == 0) { fprintf(stderr, "unknown --kind %s\n", a.kind.c_str()); return 2; }
  const size_t count = a.bytes / es;
  const size_t sendElems = kind == 1 ? count * n : count, recvElems = kind == 2 ? count * n : count;
  World w(n);
  w.prepareKind(kind, 0, count, dt, root);
  w.finalize();
  dfcclCollGeometry geom{};
  NK(dfcclGetCollGeometry(w.ctx[0], 0, &geom));
  std::vector<void*> send(n), recv(n);
  for (int r = 0; r < n; r++) {
    CK(hipMalloc(&send[r], sendElems * es));
    CK(hipMalloc(&recv[r], recvElems * es));
    fillBuffer(send[r], sendElems, dt, r + 1);
    fillBuffer(recv[r], recvElems, dt, 0);
  }
  CK(hipStreamSynchronize(nullptr));
  std::vector<Flag> flags(n);
  SpinBarrier bar(n);
  std::atomic<int> failed{0};
  const int total = a.iters + 2;
  std::vector<uint64_t> tStart(total);
  std::vector<std::atomic<uint64_t>> endNs(total);
  for (auto& e : endNs) e.store(0);
  std::vector<std::thread> th;
  for (int r = 0; r < n; r++) {
    th.emplace_back([&, r] {
      CK(hipSetDevice(0));
      for (int it = 0; it < total && !failed.load() && !gGiveUp.load(); it++) {
        flags[r].done.store(0);
        bar.wait();
        if (r == 0) tStart[it] = nowNs();
        if (kind == 1) NK(ofcclRunReduceScatter(send[r], recv[r], 0, onDone, &flags[r], w.ctx[r]));
        else if (kind == 2) NK(ofcclRunAllGather(send[r], recv[r], 0, onDone, &flags[r], w.ctx[r]));
        else if (kind == 3) NK(ofcclRunReduce(send[r], recv[r], 0, onDone, &flags[r], w.ctx[r]));
        else NK(ofcclRunBroadcast(send[r], recv[r], 0, onDone, &flags[r], w.ctx[r]));
        if (!waitFlag(flags[r], a.timeoutS)) { failed.store(1); fprintf(stderr, "rank %d timed out\n", r); return; }
        uint64_t t = nowNs(), prev = endNs[it].load();
        while (prev < t && !endNs[it].compare_exchange_weak(prev, t)) {}
        bar.wait();
      }
    });
  }
  for (auto& t : th) t.join();
  bool ok = !failed.load() && !gGiveUp.load();
  if (!ok) w.report();
  std::vector<double> ms;
  for (int it = 2; it < total && ok; it++) ms.push_back((double)(endNs[it].load() - tStart[it]) / 1e6);
  std::vector<char> scratch;
  const int sum = n * (n + 1) / 2;
  for (int r = 0; r < n && ok; r++) {
    if (kind == 1) ok = verifyBuffer(recv[r], count, dt, sum, scratch);
    else if (kind == 2) { for (int b = 0; b < n && ok; b++) ok = verifyBuffer((char*)recv[r] + (size_t)b * count * es, count, dt, b + 1, scratch); }
    else if (kind == 3) { if (r == root) ok = verifyBuffer(recv[r], count, dt, sum, scratch); }
    else ok = verifyBuffer(recv[r], count, dt, root + 1, scratch);
  }
  w.destroy();
  const double best = ms.empty() ? 0 : *std::min_element(ms.begin(), ms.end());
  // HBM bytes the direct protocol moves, all ranks together (every input element read once, every output written once)
  const double B = (double)count * es;
  const double moved = kind == 1 ? 1.0 * n * n * B + n * B : kind == 2 ? n * B + 1.0 * n * n * B : kind == 3 ? n * B + B : B + n * B;
  printf("{\"mode\": \"collective\", \"kind\": \"%s\", \"ranks\": %d, \"dtype\": \"%s\", \"count_bytes\": %zu, \"protocol\": \"%s\", "
         "\"channels\": %d, \"iters\": %d, \"correct\": %s, \"best_ms\": %.4f, \"median_ms\": %.4f, \"direct_traffic_GBps\": %.1f}\n",
         a.kind.c_str(), n, a.dtype.c_str(), count * es, geom.protocol == 1 ? "direct" : "fifo", geom.nChannels, a.iters,
         ok ? "true" : "false", best, pct(ms, 0.5), best > 0 ? moved / (best * 1e-3) / 1e9 : 0);
  return ok ? 0 : 1;
}

static void onSignal(int sig) {
  // end the waits; the modes then tear the rank contexts down, which stops the daemon kernel
  gGiveUp.store(1, std::memory_order_release);
  (void)sig;
}

int main(int argc, char** argv) {
  signal(SIGTERM, onSignal);
  signal(SIGINT, onSignal);
  if (argc < 2) {
    fprintf(stderr, "usage: dfccl_bench latency|disorder|allreduce|buckets|collective [options]\n");
    return 2;
  }
  Args a;
  a.mode = argv[1];
  for (int i = 2; i + 1 < argc; i += 2) {
    std::string k = argv[i], v = argv[i + 1];
    if (k == "--ranks") a.ranks = atoi(v.c_str());
    else if (k == "--colls") a.colls = atoi(v.c_str());
    else if (k == "--iters") a.iters = atoi(v.c_str());
    else if (k == "--warmup") a.warmup = atoi(v.c_str());
    else if (k == "--bytes") a.bytes = strtoull(v.c_str(), nullptr, 10);
    else if (k == "--min-bytes") a.minBytes = strtoull(v.c_str(), nullptr, 10);
    else if (k == "--max-bytes") a.maxBytes = strtoull(v.c_str(), nullptr, 10);
    else if (k == "--elems") a.elems = strtoull(v.c_str(), nullptr, 10);
    else if (k == "--dtype") a.dtype = v;
    else if (k == "--kind") a.kind = v;
    else if (k == "--seed") a.seed = strtoull(v.c_str(), nullptr, 10);
    else if (k == "--timeout") a.timeoutS = atoi(v.c_str());
    else { fprintf(stderr, "unknown option %s\n", k.c_str()); return 2; }
  }
  CK(hipSetDevice(0));
  if (a.mode == "latency") return runLatency(a);
  if (a.mode == "disorder") return runDisorder(a);
  if (a.mode == "allreduce") return runBuckets(a, true);
  if (a.mode == "buckets") return runBuckets(a, false);
  if (a.mode == "collective") return runCollective(a);
  fprintf(stderr, "unknown mode %s\n", a.mode.c_str());
  return 2;
}
