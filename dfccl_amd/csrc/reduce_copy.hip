// One-shot launch of the reduce-copy primitive (dfcclReduceCopy in ofccl.h).
// The data-moving code is reduceCopyWG, the same function the daemon kernel
// calls per slice; here a grid of workgroups walks the buffer chunk by chunk.
// Algorithmic traffic: (nsrcs + 1) * count * sizeof(T) bytes, HBM-bound.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "../../include/ofccl.h"
#include "avg_scale.h"
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
  ScaleUse su;  // only read by the scaled kernels
};

template <int DT, int OP, int K, bool SC>
__global__ __launch_bounds__(kRcThreads) void reduceCopyKernel(RcArgs a) {
  const size_t nchunks = (a.nbytes + a.chunkBytes - 1) / a.chunkBytes;
  for (size_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const size_t off = c * a.chunkBytes;
    const size_t len = (a.nbytes - off < a.chunkBytes) ? a.nbytes - off : a.chunkBytes;
    const void* s[K];
#pragma unroll
    for (int k = 0; k < K; k++) s[k] = (const char*)a.srcs[k] + off;
    void* d[1] = {(char*)a.dst + off};
    if constexpr (SC) reduceCopyWG<DT, OP, K, 1, kRcUnroll, true, true>(s, d, len, threadIdx.x, kRcThreads, a.su);
    else reduceCopyWG<DT, OP, K, 1, kRcUnroll, true>(s, d, len, threadIdx.x, kRcThreads);
  }
}

typedef void (*RcKernel)(RcArgs);

template <int DT, int OP, bool SC>
static RcKernel pickK(int k) {
  switch (k) {
    case 1: return SC ? reduceCopyKernel<DT, OP, 1, SC> : nullptr;  // (an unscaled single source is the plain copy)
    case 2: return reduceCopyKernel<DT, OP, 2, SC>;
    case 3: return reduceCopyKernel<DT, OP, 3, SC>;
    case 4: return reduceCopyKernel<DT, OP, 4, SC>;
    default: return nullptr;
  }
}

template <int DT>
static RcKernel pickOp(int op, int k, bool scaled) {
  if (scaled) return pickK<DT, kSum, true>(k);
  switch (op) {
    case kSum: return pickK<DT, kSum, false>(k);
    case kProd: return pickK<DT, kProd, false>(k);
    case kMax: return pickK<DT, kMax, false>(k);
    case kMin: return pickK<DT, kMin, false>(k);
    default: return nullptr;
  }
}

static RcKernel pickKernel(int dt, int op, int k, bool scaled) {
  if (k == 1 && !scaled) return reduceCopyKernel<kI8, kSum, 1, false>;  // a copy does not look at the elements
  switch (dt) {
    case kI8: return pickOp<kI8>(op, k, scaled);
    case kU8: return pickOp<kU8>(op, k, scaled);
    case kI32: return pickOp<kI32>(op, k, scaled);
    case kU32: return pickOp<kU32>(op, k, scaled);
    case kI64: return pickOp<kI64>(op, k, scaled);
    case kU64: return pickOp<kU64>(op, k, scaled);
    case kF16: return pickOp<kF16>(op, k, scaled);
    case kF32: return pickOp<kF32>(op, k, scaled);
    case kF64: return pickOp<kF64>(op, k, scaled);
    case kBF16: return pickOp<kBF16>(op, k, scaled);
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
  if ((int)op < 0 || (int)op > (int)ncclAvg) return ncclInvalidArgument;
  if (srcs == nullptr || nsrcs < 1 || nsrcs > 8) return ncclInvalidArgument;
  if (count == 0) return ncclSuccess;
  if (dst == nullptr) return ncclInvalidArgument;
  for (int i = 0; i < nsrcs; i++)
    if (srcs[i] == nullptr) return ncclInvalidArgument;
  if (chunkBytes == 0) chunkBytes = (size_t)envInt("DFCCL_RC_CHUNK_BYTES", 16 << 10);
  chunkBytes = (chunkBytes + 1023) & ~(size_t)1023;  // keeps every chunk 16-byte aligned relative to the base
  // ncclAvg over the nsrcs sources: what hostToDevRedOp (src/enqueue.cc:1326-1357) makes of it for a group of nsrcs
  Scale scale = dfcclAvgScale((int)datatype, nsrcs);
  if (op != ncclAvg) scale.kind = kScaleNone;
  const int baseOp = (op == ncclAvg) ? (int)kSum : (int)op;

  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return ncclUnhandledCudaError;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return ncclUnhandledCudaError;
  const int wgsPerCu = std::max(1, envInt("DFCCL_RC_WGS_PER_CU", 2));

  const size_t nbytes = count * (size_t)es;
  const size_t nchunks = (nbytes + chunkBytes - 1) / chunkBytes;
  size_t maxWgs = (size_t)cus * wgsPerCu;
  const int capWgs = envInt("DFCCL_RC_MAX_WGS", 0);  // (a cap on the grid, for hosts that run the kernel on few threads)
  if (capWgs > 0) maxWgs = std::min<size_t>(maxWgs, (size_t)capWgs);
  const unsigned grid = (unsigned)std::min<size_t>(nchunks, maxWgs);

  // Up to four sources per launch; further sources are folded into dst in
  // place, which keeps the left-to-right order of the fold.  A scaled sum multiplies the sources it reads from
  // the caller (not the running value in dst) and divides in the launch that finishes the sum.
  int done = 0;
  while (done < nsrcs) {
    RcArgs a{};
    a.su = noScale();
    int k = 0;
    if (done > 0) a.srcs[k++] = dst;
    const int firstUser = k;
    while (k < kRcMaxSrcsPerLaunch && done < nsrcs) a.srcs[k++] = srcs[done++];
    a.dst = dst;
    a.nbytes = nbytes;
    a.chunkBytes = chunkBytes;
    const bool scaled = scale.kind != kScaleNone;
    if (scaled) {
      a.su.scale = scale;
      a.su.preMask = ((1u << k) - 1u) & ~((1u << firstUser) - 1u);
      a.su.post = (done == nsrcs);
    }
    RcKernel fn = pickKernel((int)datatype, baseOp, k, scaled);
    if (fn == nullptr) return ncclInvalidArgument;
    hipLaunchKernelGGL(fn, dim3(grid), dim3(kRcThreads), 0, (hipStream_t)stream, a);
    if (hipGetLastError() != hipSuccess) return ncclUnhandledCudaError;
  }
  return ncclSuccess;
}
