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

// Scaling of a Sum (see Scale in reduce_ops.h): the sources whose bit is set in `preMask` are user inputs and are
// multiplied by the scalar as they are read (kScalePre); `post` says that this call produces the final value,
// which an integer average divides by the group size (kScalePost).  Only the Sum instantiations look at it.
struct ScaleUse {
  Scale scale;
  uint32_t preMask;
  bool post;
};
__host__ __device__ __forceinline__ ScaleUse noScale() {
  ScaleUse u;
  u.scale.kind = kScaleNone;
  u.scale.bits = 0;
  u.preMask = 0;
  u.post = false;
  return u;
}

// SC = false compiles the scaling away altogether (the plain ops' code is what it is without it).
// NT: non-temporal loads (every byte is read once); NTS: non-temporal stores, by default like the loads.
template <int DT, int OP, int NS, int ND, int U, bool NT, bool SC = false, bool NTS = NT>
__device__ __forceinline__ void reduceCopyWG(const void* const (&srcs)[NS], void* const (&dsts)[ND], size_t nbytes,
                                             int tid, int nthr, const ScaleUse su = noScale()) {
  constexpr int ES = typeSize(DT);
  uintptr_t align = 0;
#pragma unroll
  for (int s = 0; s < NS; s++) align |= (uintptr_t)srcs[s];
#pragma unroll
  for (int d = 0; d < ND; d++) align |= (uintptr_t)dsts[d];
  // (uniform over the workgroup; constant false unless this is a scaled sum)
  const bool pre = SC && OP == kSum && su.scale.kind == kScalePre && su.preMask != 0;
  const bool post = SC && OP == kSum && !isFloatType(DT) && su.scale.kind == kScalePost && su.post;
  const u32x4 factor = splatScalar<DT>(su.scale.bits);
  const int divisor = (int)su.scale.bits;

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
      if (pre) {
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
          for (int s = 0; s < NS; s++)
            if ((su.preMask >> s) & 1u) v[s][u] = packOp<DT, kProd>(v[s][u], factor);
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        u32x4 acc = v[0][u];
#pragma unroll
        for (int s = 1; s < NS; s++) acc = packOp<DT, OP>(acc, v[s][u]);
        if (post) acc = packPostDiv<DT>(acc, divisor);
#pragma unroll
        for (int d = 0; d < ND; d++) storePack<NTS>(dsts[d], base + (size_t)u * nthr, acc);
      }
    }
    for (size_t i = ntiles * tile + tid; i < npacks; i += nthr) {
      u32x4 acc = loadPack<NT>(srcs[0], i);
      if (pre && (su.preMask & 1u)) acc = packOp<DT, kProd>(acc, factor);
#pragma unroll
      for (int s = 1; s < NS; s++) {
        u32x4 v = loadPack<NT>(srcs[s], i);
        if (pre && ((su.preMask >> s) & 1u)) v = packOp<DT, kProd>(v, factor);
        acc = packOp<DT, OP>(acc, v);
      }
      if (post) acc = packPostDiv<DT>(acc, divisor);
#pragma unroll
      for (int d = 0; d < ND; d++) storePack<NTS>(dsts[d], i, acc);
    }
    doneBytes = npacks << 4;
  }
  const size_t first = doneBytes / ES, nelem = nbytes / ES;
  for (size_t i = first + tid; i < nelem; i += nthr) {
    uint64_t acc = loadElem<ES>(srcs[0], i);
    if (pre && (su.preMask & 1u)) acc = elemPreMul<DT>(acc, su.scale.bits);
#pragma unroll
    for (int s = 1; s < NS; s++) {
      uint64_t v = loadElem<ES>(srcs[s], i);
      if (pre && ((su.preMask >> s) & 1u)) v = elemPreMul<DT>(v, su.scale.bits);
      acc = elemOp<DT, OP>(acc, v);
    }
    if (post) acc = elemPostDiv<DT>(acc, divisor);
#pragma unroll
    for (int d = 0; d < ND; d++) storeElem<ES>(dsts[d], i, acc);
  }
}

}  // namespace dfccl
