// Host emulation of the HIP runtime calls and of kernel launches (see hip/hip_runtime.h in this directory):
// test infrastructure.
#include <hip/hip_runtime.h>

#include <errno.h>
#include <unistd.h>

#include <condition_variable>
#include <thread>

namespace emul {

thread_local ThreadCtx tls;
std::atomic<uint64_t> gProgress{0};

struct Job {
  unsigned grid = 0, block = 0;
  std::function<void()> body;
  std::vector<std::unique_ptr<Workgroup>> wgs;
  std::vector<pthread_t> threads;
  std::mutex mu;
  std::atomic<bool> joined{false};
  void join() {
    std::lock_guard<std::mutex> lk(mu);
    if (joined) return;
    for (pthread_t t : threads) pthread_join(t, nullptr);
    joined = true;
  }
};

struct Stream {
  std::mutex mu;
  std::shared_ptr<Job> last;
};
struct Event {
  std::mutex mu;
  std::shared_ptr<Job> job;
};

// (never destroyed: the watchdog thread may still be looking at them when the process ends)
static std::mutex& gJobsMu = *new std::mutex();
static std::vector<std::shared_ptr<Job>>& gJobs = *new std::vector<std::shared_ptr<Job>>();  // every launch
static Stream& gNullStream = *new Stream();

int gJitterPerMille = getenv("EMUL_JITTER") ? atoi(getenv("EMUL_JITTER")) : 0;
bool gNeverLeave = getenv("EMUL_NEVER_LEAVE") && atoi(getenv("EMUL_NEVER_LEAVE")) != 0;
void jitterSleep() {
  static thread_local uint64_t rng = 0x9e3779b97f4a7c15ull ^ ((uint64_t)tls.bIdx.x << 32) ^ tls.tIdx.x ^ (uint64_t)time(nullptr) << 16;
  rng ^= rng << 13;
  rng ^= rng >> 7;
  rng ^= rng << 17;
  // whole waves are delayed together more often than single lanes: that is what the GPU does
  if ((int)(rng % 1000u) < gJitterPerMille) usleep((useconds_t)(rng >> 40) % 300u);
}

void barrierMismatch(int tid, int line, int line0) {
  fprintf(stderr,
          "emul: WORKGROUP OUT OF STEP: block %u thread %d is at the __syncthreads() of line %d, thread 0 at the one of "
          "line %d\n",
          tls.bIdx.x, tid, line, line0);
  fflush(stderr);
  abort();
}

void notUniform(int line, uint64_t mine, uint64_t first) {
  fprintf(stderr,
          "emul: NOT UNIFORM: block %u thread %u holds %#llx at the DFCCL_UNIFORM of line %d, lane 0 of its wave holds "
          "%#llx\n",
          tls.bIdx.x, tls.tIdx.x, (unsigned long long)mine, line, (unsigned long long)first);
  fflush(stderr);
  abort();
}

void* wgSharedMem(size_t bytes) {
  Workgroup* wg = tls.wg;
  if (bytes > sizeof(wg->lds)) {
    fprintf(stderr, "emul: %zu bytes of LDS asked for\n", bytes);
    abort();
  }
  return wg->lds;
}

struct ThreadArg {
  Job* job;
  unsigned b, t;
};

static void* threadMain(void* p) {
  ThreadArg* a = (ThreadArg*)p;
  Job* job = a->job;
  tls.tIdx = Dim3(a->t);
  tls.bIdx = Dim3(a->b);
  tls.bDim = Dim3(job->block);
  tls.gDim = Dim3(job->grid);
  tls.wg = job->wgs[a->b].get();
  tls.barriers = 0;
  const unsigned t = a->t;
  delete a;
  job->body();
  tls.wg->where[t].store(-1, std::memory_order_relaxed);
  return nullptr;
}

void launch(Stream* s, unsigned grid, unsigned block, std::function<void()> body) {
  if (s == nullptr) s = &gNullStream;
  std::shared_ptr<Job> prev;
  {
    std::lock_guard<std::mutex> lk(s->mu);
    prev = s->last;
  }
  if (prev) prev->join();  // launches of one stream run one after the other
  if (block % kWaveSize != 0) {
    fprintf(stderr, "emul: block size %u is not a multiple of the wave size\n", block);
    abort();
  }
  auto job = std::make_shared<Job>();
  job->grid = grid;
  job->block = block;
  job->body = std::move(body);
  for (unsigned b = 0; b < grid; b++) {
    auto wg = std::make_unique<Workgroup>();
    wg->nThreads = (int)block;
    pthread_barrier_init(&wg->bar, nullptr, block);
    wg->waves = std::vector<Wave>(block / kWaveSize);
    for (Wave& w : wg->waves) pthread_barrier_init(&w.bar, nullptr, kWaveSize);
    wg->lines[0].assign(block, 0);
    wg->lines[1].assign(block, 0);
    wg->where = std::vector<std::atomic<int>>(block);
    for (auto& w : wg->where) w.store(0);
    memset(wg->lds, 0xA5, sizeof(wg->lds));  // LDS is not cleared between launches on the GPU either
    job->wgs.push_back(std::move(wg));
  }
  pthread_attr_t attr;
  pthread_attr_init(&attr);
  pthread_attr_setstacksize(&attr, 1 << 20);
  for (unsigned b = 0; b < grid; b++)
    for (unsigned t = 0; t < block; t++) {
      pthread_t th;
      ThreadArg* a = new ThreadArg{job.get(), b, t};
      const int rc = pthread_create(&th, &attr, threadMain, a);
      if (rc != 0) {
        fprintf(stderr, "emul: pthread_create failed (%d) after %zu threads\n", rc, job->threads.size());
        abort();
      }
      job->threads.push_back(th);
    }
  pthread_attr_destroy(&attr);
  {
    std::lock_guard<std::mutex> lk(s->mu);
    s->last = job;
  }
  std::lock_guard<std::mutex> lk(gJobsMu);
  gJobs.push_back(job);
}

// Where every thread of every launch that has not ended is (for a run that has stopped moving).
void dumpThreads(FILE* f) {
  std::lock_guard<std::mutex> lk(gJobsMu);
  for (size_t j = 0; j < gJobs.size(); j++) {
    Job& job = *gJobs[j];
    for (unsigned b = 0; b < job.grid; b++) {
      Workgroup& wg = *job.wgs[b];
      int first = wg.where[0].load();
      bool allGone = true;
      for (int t = 0; t < wg.nThreads; t++) allGone = allGone && wg.where[t].load() == -1;
      if (allGone) continue;
      fprintf(f, "emul: launch %zu block %u:", j, b);
      int runStart = 0;
      for (int t = 1; t <= wg.nThreads; t++) {
        const int w = t < wg.nThreads ? wg.where[t].load() : INT32_MIN;
        if (w != first) {
          fprintf(f, " [%d..%d]=%d", runStart, t - 1, first);
          runStart = t;
          first = w;
        }
      }
      fprintf(f, "   (>0: waiting at the barrier of that line, 0 running, -1 returned, < -1: in the cross-lane operation of that line)\n");
    }
  }
  fflush(f);
}

static void watchdogMain() {
  const char* env = getenv("EMUL_WATCHDOG_S");
  const int limit = env ? atoi(env) : 60;
  uint64_t last = gProgress.load();
  int quiet = 0;
  for (;;) {
    sleep(1);
    const uint64_t now = gProgress.load();
    bool running = false;
    {
      std::lock_guard<std::mutex> lk(gJobsMu);
      for (auto& j : gJobs) running = running || !j->joined;
    }
    if (now != last || !running) {
      last = now;
      quiet = 0;
      continue;
    }
    if (++quiet >= limit) {
      fprintf(stderr, "emul: no barrier or cross-lane operation completed for %d s\n", limit);
      dumpThreads(stderr);
      abort();
    }
  }
}

static void startWatchdog() {
  static std::once_flag once;
  std::call_once(once, [] { std::thread(watchdogMain).detach(); });
}

}  // namespace emul

extern "C" void emulDumpThreads() { emul::dumpThreads(stderr); }
// for callers outside C++ (the Python tests): wait for the kernels launched on the null stream
extern "C" void emulNullStreamSynchronize() { (void)hipStreamSynchronize(nullptr); }

static size_t roundUp(size_t n, size_t a) { return (n + a - 1) / a * a; }

hipError_t hipMalloc(void** p, size_t bytes) {
  emul::startWatchdog();
  void* m = aligned_alloc(256, roundUp(bytes ? bytes : 1, 256));
  if (m == nullptr) return hipErrorOutOfMemory;
  memset(m, 0xCD, bytes);  // hipMalloc does not clear
  *p = m;
  return hipSuccess;
}
hipError_t hipFree(void* p) {
  free(p);
  return hipSuccess;
}
hipError_t hipHostMalloc(void** p, size_t bytes, unsigned) { return hipMalloc(p, bytes); }
hipError_t hipHostFree(void* p) { return hipFree(p); }
hipError_t hipMemset(void* p, int value, size_t bytes) {
  memset(p, value, bytes);
  return hipSuccess;
}
hipError_t hipMemsetD8(hipDeviceptr_t p, unsigned char value, size_t count) {
  memset(p, value, count);
  return hipSuccess;
}
hipError_t hipMemsetD16(hipDeviceptr_t p, unsigned short value, size_t count) {
  for (size_t i = 0; i < count; i++) ((unsigned short*)p)[i] = value;
  return hipSuccess;
}
hipError_t hipMemsetD32(hipDeviceptr_t p, int value, size_t count) {
  for (size_t i = 0; i < count; i++) ((int*)p)[i] = value;
  return hipSuccess;
}
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind) {
  memcpy(dst, src, bytes);
  return hipSuccess;
}
hipError_t hipSetDevice(int device) { return device == 0 ? hipSuccess : hipErrorInvalidValue; }
hipError_t hipGetDevice(int* device) {
  *device = 0;
  return hipSuccess;
}
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) {
  *value = 256;
  return hipSuccess;
}
hipError_t hipGetLastError() { return hipSuccess; }
const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "emulated error"; }
hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) {
  *s = new emul::Stream();
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t s) {
  if (s == nullptr) s = &emul::gNullStream;
  std::shared_ptr<emul::Job> j;
  {
    std::lock_guard<std::mutex> lk(s->mu);
    j = s->last;
  }
  if (j) j->join();
  return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t s) {
  hipStreamSynchronize(s);
  delete s;
  return hipSuccess;
}
hipError_t hipDeviceSynchronize() {
  std::vector<std::shared_ptr<emul::Job>> jobs;
  {
    std::lock_guard<std::mutex> lk(emul::gJobsMu);
    jobs = emul::gJobs;
  }
  for (auto& j : jobs) j->join();
  return hipSuccess;
}
hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) {
  *e = new emul::Event();
  return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t e) {
  delete e;
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s) {
  if (s == nullptr) s = &emul::gNullStream;
  std::shared_ptr<emul::Job> j;
  {
    std::lock_guard<std::mutex> lk(s->mu);
    j = s->last;
  }
  std::lock_guard<std::mutex> lk(e->mu);
  e->job = j;
  return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t e) {
  std::shared_ptr<emul::Job> j;
  {
    std::lock_guard<std::mutex> lk(e->mu);
    j = e->job;
  }
  if (j) j->join();
  return hipSuccess;
}
