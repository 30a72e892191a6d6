// Workgroup-level reduce-copy for gfx950: NS sources folded left to right into
// ND destinations (the role of ReduceOrCopyMulti in the reference,
// src/include/common_kernel.h:629-690).  When every pointer is 16-byte aligned
// the bulk moves as 128-bit loads and stores: per iteration the workgroup takes
// U rows of nthr*16 bytes, each row one contiguous, fully coalesced access of
// the whole workgroup (measured on MI355X: keeping the workgroup's accesses in
// one compact window is worth ~15 % of HBM bandwidth over per-wave strips);
// what is left goes pack by pack and finally element by element.  Misaligned
// operands take the element path for everything.
#pragma once

#include "reduce_ops.h"

namespace dfccl {

// All operands of the data path are in global memory (HBM or host-coherent), never LDS or scratch: saying so
// turns what would be flat_load / flat_store (pointers that come out of context structures have no known
// address space) into global_load / global_store, which do not also occupy the LDS path.
template <bool NT>
__device__ __forceinline__ u32x4 loadPack(const void* base, size_t pack) {
  const DFCCL_GLOBAL u32x4* p = (const DFCCL_GLOBAL u32x4*)base + pack;
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT>
__device__ __forceinline__ void storePack(void* base, size_t pack, u32x4 v) {
  DFCCL_GLOBAL u32x4* p = (DFCCL_GLOBAL u32x4*)base + pack;
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

template <int DT, int OP, int NS, int ND, int U, bool NT>
__device__ __forceinline__ void reduceCopyWG(const void* const (&srcs)[NS], void* const (&dsts)[ND], size_t nbytes,
                                             int tid, int nthr) {
  constexpr int ES = typeSize(DT);
  uintptr_t align = 0;
#pragma unroll
  for (int s = 0; s < NS; s++) align |= (uintptr_t)srcs[s];
#pragma unroll
  for (int d = 0; d < ND; d++) align |= (uintptr_t)dsts[d];

  size_t doneBytes = 0;
  if ((align & 15u) == 0) {
    const size_t npacks = nbytes >> 4;
    const size_t tile = (size_t)nthr * U;  // packs the workgroup moves per iteration
    const size_t ntiles = npacks / tile;
    for (size_t t = 0; t < ntiles; t++) {
      // load u of every thread is one contiguous nthr*16-byte row: at any instant the
      // workgroup's accesses cover a compact address window
      const size_t base = t * tile + tid;
      u32x4 v[NS][U];
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
        for (int s = 0; s < NS; s++) v[s][u] = loadPack<NT>(srcs[s], base + (size_t)u * nthr);
#pragma unroll
      for (int u = 0; u < U; u++) {
        u32x4 acc = v[0][u];
#pragma unroll
        for (int s = 1; s < NS; s++) acc = packOp<DT, OP>(acc, v[s][u]);
#pragma unroll
        for (int d = 0; d < ND; d++) storePack<NT>(dsts[d], base + (size_t)u * nthr, acc);
      }
    }
    for (size_t i = ntiles * tile + tid; i < npacks; i += nthr) {
      u32x4 acc = loadPack<NT>(srcs[0], i);
#pragma unroll
      for (int s = 1; s < NS; s++) acc = packOp<DT, OP>(acc, loadPack<NT>(srcs[s], i));
#pragma unroll
      for (int d = 0; d < ND; d++) storePack<NT>(dsts[d], i, acc);
    }
    doneBytes = npacks << 4;
  }
  const size_t first = doneBytes / ES, nelem = nbytes / ES;
  for (size_t i = first + tid; i < nelem; i += nthr) {
    uint32_t acc = loadElem<ES>(srcs[0], i);
#pragma unroll
    for (int s = 1; s < NS; s++) acc = wordOp<DT, OP>(acc, loadElem<ES>(srcs[s], i));
#pragma unroll
    for (int d = 0; d < ND; d++) storeElem<ES>(dsts[d], i, acc);
  }
}

}  // namespace dfccl
