// Chunk geometry and per-step roles of the ring collectives, shared by the
// host planner and the daemon kernel (plain inline functions, no HIP types).
// The formulas restate the reference's resumable runRing bodies:
//   all-reduce      src/collectives_ofccl/device/ofccl_all_reduce.h:44-188
//   reduce-scatter  src/collectives_ofccl/device/ofccl_reduce_scatter.h:31-89
//   all-gather      src/collectives_ofccl/device/ofccl_all_gather.h:44-138
//   reduce          src/collectives_ofccl/device/ofccl_reduce.h:44-106
//   broadcast       src/collectives_ofccl/device/ofccl_broadcast.h:33-69
//   slice sizing    src/collectives_ofccl/device/ofccl_prims_simple.h:231-235
// The ring is 0 -> 1 -> ... -> n-1 -> 0, so a rank's ring index is its rank and
// ringRanks[i] of rank r is (r + i) % n.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define DFCCL_HD __host__ __device__ inline
#else
#define DFCCL_HD inline
#endif

namespace dfccl {

enum CollKind : int { kAllReduce = 0, kReduceScatter = 1, kAllGather = 2, kReduce = 3, kBroadcast = 4, kNumKinds = 5 };

DFCCL_HD int64_t divUp64(int64_t a, int64_t b) { return (a + b - 1) / b; }
DFCCL_HD int64_t roundUp64(int64_t a, int64_t b) { return divUp64(a, b) * b; }
DFCCL_HD int64_t min64(int64_t a, int64_t b) { return a < b ? a : b; }
DFCCL_HD int64_t max64(int64_t a, int64_t b) { return a > b ? a : b; }

// Ring steps one loop iteration takes on every rank.
DFCCL_HD int stepsPerLoop(int kind, int n) {
  if (n == 1) return 1;
  switch (kind) {
    case kAllReduce: return 2 * n - 1;
    case kReduceScatter: return n;
    case kAllGather: return n;
    default: return 1;  // reduce and broadcast are chains: one primitive per rank and loop
  }
}

// Elements one loop iteration covers across all channels (nominal chunk).
DFCCL_HD int64_t loopElems(int kind, int n, int nChannels, int64_t chunkElems) {
  return (kind == kAllReduce ? (int64_t)nChannels * n : (int64_t)nChannels) * chunkElems;
}

// Chunk size actually used by the loop that starts at gridOffset: the nominal
// chunk, or an even split of what is left, rounded up to alignElems.
DFCCL_HD int64_t realChunkElems(int kind, int n, int nChannels, int64_t chunkElems, int64_t alignElems, int64_t count,
                                int64_t gridOffset) {
  const int64_t divisor = (kind == kAllReduce) ? (int64_t)nChannels * n : (int64_t)nChannels;
  return roundUp64(min64(chunkElems, divUp64(count - gridOffset, divisor)), alignElems);
}

// Elements per slice of a chunk of nelem elements (one slice fills one FIFO slot).
DFCCL_HD int64_t sliceElemsFor(int64_t nelem, int slicesPerChunk, int64_t nominalSliceElems) {
  return max64(divUp64(nelem, 16 * (int64_t)slicesPerChunk) * 16, nominalSliceElems / 32);
}

// What one rank does in one ring step: which operands take part and where the
// user-buffer operands start (element offsets into sendbuff / recvbuff).
struct StepDesc {
  int recv;      // take a slice from the previous rank's FIFO
  int send;      // put the result into the FIFO towards the next rank
  int useIn;     // read the user's send buffer at inOff
  int useOut;    // write the user's receive buffer at outOff
  int post;      // this step produces the final value of a reduction (the reference's postOp = true)
  int64_t inOff;
  int64_t outOff;
  int64_t nelem; // may be <= 0: nothing to do for this rank/step (both ends agree)
};

// `real` is realChunkElems() of this loop, `bid` the channel, `inPlace` whether
// the step-0 copy of all-gather / broadcast can be skipped (src == dst).
DFCCL_HD StepDesc describeStep(int kind, int n, int rank, int root, int nChannels, int bid, int64_t count,
                               int64_t gridOffset, int64_t real, int step, int inPlace) {
  StepDesc d;
  d.recv = d.send = d.useIn = d.useOut = d.post = 0;
  d.inOff = d.outOff = 0;
  d.nelem = 0;
  (void)nChannels;
  if (n == 1) {  // a one-rank communicator only copies
    const int64_t off = gridOffset + (kind == kAllReduce ? (int64_t)bid * real : (int64_t)bid * real);
    d.useIn = 1;
    d.useOut = inPlace ? 0 : 1;
    d.inOff = d.outOff = off;
    d.nelem = min64(real, count - off);
    return d;
  }
  if (kind == kAllReduce) {
    int chunk;
    if (step == 0) { chunk = (rank + n - 1) % n; d.useIn = 1; d.send = 1; }
    else if (step <= n - 2) { chunk = (rank + n - (step + 1)) % n; d.recv = 1; d.useIn = 1; d.send = 1; }
    else if (step == n - 1) { chunk = rank; d.recv = 1; d.useIn = 1; d.useOut = 1; d.send = 1; d.post = 1; }
    else if (step <= 2 * n - 3) { chunk = (rank + n - (step - n + 1)) % n; d.recv = 1; d.useOut = 1; d.send = 1; }
    else { chunk = (rank + 1) % n; d.recv = 1; d.useOut = 1; }
    const int64_t off = gridOffset + (int64_t)bid * n * real + (int64_t)chunk * real;
    d.inOff = d.outOff = off;
    d.nelem = min64(real, count - off);
    return d;
  }
  const int64_t chunkOff = gridOffset + (int64_t)bid * real;
  d.nelem = min64(real, count - chunkOff);
  if (kind == kReduceScatter) {
    int dest;
    if (step == 0) { dest = (rank + n - 1) % n; d.useIn = 1; d.send = 1; }
    else if (step <= n - 2) { dest = (rank + n - (step + 1)) % n; d.recv = 1; d.useIn = 1; d.send = 1; }
    else { dest = rank; d.recv = 1; d.useIn = 1; d.useOut = 1; d.post = 1; }
    d.inOff = chunkOff + (int64_t)dest * count;
    d.outOff = chunkOff;
  } else if (kind == kAllGather) {
    int dest;
    if (step == 0) { dest = rank; d.useIn = 1; d.send = 1; d.useOut = inPlace ? 0 : 1; }
    else if (step <= n - 2) { dest = (rank + n - step) % n; d.recv = 1; d.useOut = 1; d.send = 1; }
    else { dest = (rank + 1) % n; d.recv = 1; d.useOut = 1; }
    d.inOff = chunkOff;
    d.outOff = chunkOff + (int64_t)dest * count;
  } else if (kind == kReduce) {
    d.inOff = d.outOff = chunkOff;
    if ((rank + n - 1) % n == root) { d.useIn = 1; d.send = 1; }
    else if (rank == root) { d.recv = 1; d.useIn = 1; d.useOut = 1; d.post = 1; }
    else { d.recv = 1; d.useIn = 1; d.send = 1; }
  } else {  // broadcast
    d.inOff = d.outOff = chunkOff;
    if (rank == root) { d.useIn = 1; d.send = 1; d.useOut = inPlace ? 0 : 1; }
    else if ((rank + 1) % n == root) { d.recv = 1; d.useOut = 1; }
    else { d.recv = 1; d.useOut = 1; d.send = 1; }
  }
  return d;
}

// ---- direct protocol (virtual ranks read and write each other's buffers in place) -------------------
//
// Host-side statement of the roles and the tile geometry (used by the planner and by the CPU tests, which run
// every rank's share through it and compare with the oracle); the daemon kernel evaluates the same expressions
// in place (runDirect, sweepFoldN).
//
// Every rank does a share of the collective: it folds `nSrc` send buffers (in the order in which the ring would
// have accumulated those elements) and stores the result into `nDst` receive buffers.  The share is a set of
// tiles: the index space [0, count) is cut into loops of nChannels * tn chunks, and tile t of a rank is chunk
// number tme of channel slot t % nChannels in loop t / nChannels.
//   all-reduce      tn = n, tme = me (the chunks the ring would finish at me);  in[me+1], ..., in[me] -> all
//   reduce          tn = n, tme = me;  in[root+1], ..., in[root] -> the root's receive buffer
//   broadcast       tn = n, tme = me;  the root's send buffer -> all
//   reduce-scatter  tn = 1 (block me of every send buffer is all mine);  in[me+1], ..., in[me] -> mine
//   all-gather      tn = 1;  my send buffer -> block me of all
struct DirectRole {
  int nSrc, nDst;
  int firstSrc;       // rank of source 0; source t is rank (firstSrc + t) % n
  int onlyDst;        // rank of the single destination, -1: destination k is rank k
  int tn, tme;
  int64_t srcOff;     // elements added to every source / destination pointer
  int64_t dstOff;
};

DFCCL_HD DirectRole directRole(int kind, int n, int me, int root, int64_t count) {
  DirectRole r;
  const bool folds = (kind == kAllReduce || kind == kReduce || kind == kReduceScatter);
  const bool toAll = (kind == kAllReduce || kind == kBroadcast || kind == kAllGather);
  const bool owned = (kind == kAllReduce || kind == kReduce || kind == kBroadcast);
  r.nSrc = folds ? n : 1;
  r.nDst = toAll ? n : 1;
  r.firstSrc = folds ? ((kind == kReduce ? root : me) + 1) % n : (kind == kBroadcast ? root : me);
  r.onlyDst = toAll ? -1 : (kind == kReduce ? root : me);
  r.tn = owned ? n : 1;
  r.tme = owned ? me : 0;
  r.srcOff = (kind == kReduceScatter) ? (int64_t)me * count : 0;
  r.dstOff = (kind == kAllGather) ? (int64_t)me * count : 0;
  return r;
}

// Geometry kind whose loop / chunk arithmetic (loopElems, realChunkElems) the direct protocol uses for `kind`:
// a loop of all-reduce holds nChannels * n chunks, a loop of the others nChannels.
DFCCL_HD int directGeomKind(int kind) { return (kind == kReduce || kind == kBroadcast) ? (int)kAllReduce : kind; }

// Tile t of a rank: offset and length in elements (length <= 0: nothing there).  lastReal is the chunk size of
// the last loop (realChunkElems at its start), every other loop uses the nominal chunk.
DFCCL_HD void directTile(int64_t tile, int nChannels, int64_t loops, int64_t chunkElems, int64_t lastReal, int tn,
                         int tme, int64_t count, int64_t* off, int64_t* nelem) {
  // (tile numbers fit 32 bits: 64-bit divisions are long instruction sequences on the GPU)
  const int64_t l = (int64_t)((uint32_t)tile / (uint32_t)nChannels), slot = (int64_t)((uint32_t)tile % (uint32_t)nChannels);
  const int64_t real = (l == loops - 1) ? lastReal : chunkElems;
  const int64_t o = l * ((int64_t)nChannels * tn * chunkElems) + (slot * tn + tme) * real;
  *off = o;
  *nelem = (count - o < real) ? count - o : real;
}

// Channels (workgroups per rank) for a collective of nBytes: as many as allowed,
// shrunk until each gets at least bytesPerChannel (the thread-count shrink rule
// of src/enqueue_ofccl.cc:133-137 with a fixed workgroup size).
DFCCL_HD int planChannels(int64_t nBytes, int maxChannels, int64_t bytesPerChannel) {
  int nc = maxChannels < 1 ? 1 : maxChannels;
  while (nc > 1 && nBytes < (int64_t)nc * bytesPerChannel) nc--;
  return nc;
}

// Completion-queue entry: channel<<56 | (sequence & 0xFFFFFF)<<32 | collId
// (bit layout of src/include/collectives_ofccl.h:11-19).
DFCCL_HD uint64_t cqeEncode(unsigned blk, unsigned cnt, unsigned collId) {
  return ((uint64_t)(blk & 0xffu) << 56) | ((uint64_t)(cnt & 0xffffffu) << 32) | (uint64_t)collId;
}
DFCCL_HD unsigned cqeBlk(uint64_t v) { return (unsigned)(v >> 56); }
DFCCL_HD unsigned cqeCnt(uint64_t v) { return (unsigned)((v >> 32) & 0xffffffu); }
DFCCL_HD unsigned cqeCollId(uint64_t v) { return (unsigned)(v & 0xffffffffu); }

}  // namespace dfccl
