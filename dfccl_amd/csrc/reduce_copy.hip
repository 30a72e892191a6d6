// One-shot launch of the reduce-copy primitive (dfcclReduceCopy in ofccl.h).
// The data-moving code is reduceCopyWG, the same function the daemon kernel
// calls per slice; here a grid of workgroups walks the buffer chunk by chunk.
// Algorithmic traffic: (nsrcs + 1) * count * sizeof(T) bytes, HBM-bound.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "../../include/ofccl.h"
#include "reduce_copy_wg.h"

namespace dfccl {

constexpr int kRcThreads = 512;
// Launch shape from a sweep on MI355X at 256 MiB per buffer: one 128-bit load per source in flight per thread
// and 16 KiB chunks walked by 2 workgroups per CU keep all CUs inside one compact, forward-moving address window
// (6.8 TB/s); deeper unrolling or larger per-workgroup chunks lose 5-15 %.
constexpr int kRcUnroll = 1;
constexpr int kRcMaxSrcsPerLaunch = 4;

struct RcArgs {
  const void* srcs[kRcMaxSrcsPerLaunch];
  void* dst;
  size_t nbytes;
  size_t chunkBytes;
};

template <int DT, int OP, int K>
__global__ __launch_bounds__(kRcThreads) void reduceCopyKernel(RcArgs a) {
  const size_t nchunks = (a.nbytes + a.chunkBytes - 1) / a.chunkBytes;
  for (size_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const size_t off = c * a.chunkBytes;
    const size_t len = (a.nbytes - off < a.chunkBytes) ? a.nbytes - off : a.chunkBytes;
    const void* s[K];
#pragma unroll
    for (int k = 0; k < K; k++) s[k] = (const char*)a.srcs[k] + off;
    void* d[1] = {(char*)a.dst + off};
    reduceCopyWG<DT, OP, K, 1, kRcUnroll, true>(s, d, len, threadIdx.x, kRcThreads);
  }
}

typedef void (*RcKernel)(RcArgs);

template <int DT, int OP>
static RcKernel pickK(int k) {
  switch (k) {
    case 2: return reduceCopyKernel<DT, OP, 2>;
    case 3: return reduceCopyKernel<DT, OP, 3>;
    case 4: return reduceCopyKernel<DT, OP, 4>;
    default: return nullptr;
  }
}

template <int DT>
static RcKernel pickOp(int op, int k) {
  switch (op) {
    case kSum: return pickK<DT, kSum>(k);
    case kProd: return pickK<DT, kProd>(k);
    case kMax: return pickK<DT, kMax>(k);
    case kMin: return pickK<DT, kMin>(k);
    default: return nullptr;
  }
}

static RcKernel pickKernel(int dt, int op, int k) {
  if (k == 1) return reduceCopyKernel<kI8, kSum, 1>;  // a copy does not look at the elements
  switch (dt) {
    case kI8: return pickOp<kI8>(op, k);
    case kI32: return pickOp<kI32>(op, k);
    case kF16: return pickOp<kF16>(op, k);
    case kF32: return pickOp<kF32>(op, k);
    case kBF16: return pickOp<kBF16>(op, k);
    default: return nullptr;
  }
}

static int envInt(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}

}  // namespace dfccl

using namespace dfccl;

extern "C" __attribute__((visibility("default"))) ncclResult_t dfcclReduceCopy(const void* const* srcs, int nsrcs,
                                                                                void* dst, size_t count,
                                                                                ncclDataType_t datatype, ncclRedOp_t op,
                                                                                size_t chunkBytes, void* stream) {
  const int es = typeSize((int)datatype);
  if (es == 0) return ncclInvalidArgument;
  if ((int)op < 0 || (int)op > (int)ncclMin) return ncclInvalidArgument;
  if (srcs == nullptr || nsrcs < 1 || nsrcs > 8) return ncclInvalidArgument;
  if (count == 0) return ncclSuccess;
  if (dst == nullptr) return ncclInvalidArgument;
  for (int i = 0; i < nsrcs; i++)
    if (srcs[i] == nullptr) return ncclInvalidArgument;
  if (chunkBytes == 0) chunkBytes = (size_t)envInt("DFCCL_RC_CHUNK_BYTES", 16 << 10);
  chunkBytes = (chunkBytes + 1023) & ~(size_t)1023;  // keeps every chunk 16-byte aligned relative to the base

  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return ncclUnhandledCudaError;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return ncclUnhandledCudaError;
  const int wgsPerCu = std::max(1, envInt("DFCCL_RC_WGS_PER_CU", 2));

  const size_t nbytes = count * (size_t)es;
  const size_t nchunks = (nbytes + chunkBytes - 1) / chunkBytes;
  const unsigned grid = (unsigned)std::min<size_t>(nchunks, (size_t)cus * wgsPerCu);

  // Up to four sources per launch; further sources are folded into dst in
  // place, which keeps the left-to-right order of the fold.
  int done = 0;
  while (done < nsrcs) {
    RcArgs a{};
    int k = 0;
    if (done > 0) a.srcs[k++] = dst;
    while (k < kRcMaxSrcsPerLaunch && done < nsrcs) a.srcs[k++] = srcs[done++];
    a.dst = dst;
    a.nbytes = nbytes;
    a.chunkBytes = chunkBytes;
    RcKernel fn = pickKernel((int)datatype, (int)op, k);
    if (fn == nullptr) return ncclInvalidArgument;
    hipLaunchKernelGGL(fn, dim3(grid), dim3(kRcThreads), 0, (hipStream_t)stream, a);
    if (hipGetLastError() != hipSuccess) return ncclUnhandledCudaError;
  }
  return ncclSuccess;
}
