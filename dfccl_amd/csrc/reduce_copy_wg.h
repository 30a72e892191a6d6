// Workgroup-level reduce-copy for gfx950: NS sources folded left to right into
// ND destinations (the role of ReduceOrCopyMulti in the reference,
// src/include/common_kernel.h:629-690).  When every pointer is 16-byte aligned
// the bulk moves as 128-bit loads and stores, one wave covering U contiguous
// 1 KiB rows per iteration so that each global_load_dwordx4 of a wave is one
// fully coalesced kilobyte; what is left goes pack by pack and finally element
// by element.  Misaligned operands take the element path for everything.
#pragma once

#include "reduce_ops.h"

namespace dfccl {

template <bool NT>
__device__ __forceinline__ u32x4 loadPack(const void* base, size_t pack) {
  const u32x4* p = (const u32x4*)base + pack;
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT>
__device__ __forceinline__ void storePack(void* base, size_t pack, u32x4 v) {
  u32x4* p = (u32x4*)base + pack;
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
    const int lane = tid & 63, wave = tid >> 6, nwaves = nthr >> 6;
    constexpr size_t kTile = 64 * U;  // packs one wave moves per iteration
    const size_t ntiles = npacks / kTile;
    for (size_t t = wave; t < ntiles; t += nwaves) {
      const size_t base = t * kTile + lane;
      u32x4 v[NS][U];
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
        for (int s = 0; s < NS; s++) v[s][u] = loadPack<NT>(srcs[s], base + u * 64);
#pragma unroll
      for (int u = 0; u < U; u++) {
        u32x4 acc = v[0][u];
#pragma unroll
        for (int s = 1; s < NS; s++) acc = packOp<DT, OP>(acc, v[s][u]);
#pragma unroll
        for (int d = 0; d < ND; d++) storePack<NT>(dsts[d], base + u * 64, acc);
      }
    }
    for (size_t i = ntiles * kTile + tid; i < npacks; i += nthr) {
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
