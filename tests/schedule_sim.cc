// Host-side interpreter of the ring schedule the daemon kernel executes
// (dfccl_amd/csrc/ring_schedule.h): every virtual rank is a resumable state
// machine (loop, step, slice) that blocks on the same head / tail counters and
// uses the same FIFO slot indexing as the device code.  Element arithmetic is
// the oracle's.  Test infrastructure: lets the CPU suite check the schedule,
// the slice sizing and the flow control against the oracle without a GPU.
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <utility>
#include <vector>

#include "../dfccl_amd/csrc/ring_schedule.h"
#include "../oracle/dfccl_oracle.h"

using namespace dfccl;

namespace {
struct Link {            // FIFO from rank r to rank (r+1)%n, one per channel
  std::vector<char> data;
  uint64_t tail = 0, head = 0;
};
struct RankState {
  int64_t grid = 0;
  int step = 0, slice = 0;
  uint64_t sendStep = 0, recvStep = 0;
  bool done = false;
};
}  // namespace

extern "C" int sim_collective(int kind, int dtype, int op, int n, int nChannels, int64_t chunkElems,
                              int64_t alignElems, int64_t sliceElems, int slicesPerChunk, int fifoSlots,
                              int64_t count, int root, const void* const* send, void* const* recv,
                              int64_t* maxSliceSeen) {
  const int es = (kind == kAllGather || kind == kBroadcast) ? 1 : orc_type_size(dtype);
  if (kind == kAllGather || kind == kBroadcast) { count *= orc_type_size(dtype); dtype = ORC_I8; }
  // ncclAvg: a Sum whose user inputs are multiplied by 1/n as a step reads them (float types), or whose final
  // value is divided by n in the step the schedule marks `post` (integer types)
  int how = 0;
  uint64_t scalar = 0;
  if (op == ORC_AVG) {
    op = ORC_SUM;
    if (n > 1) {
      scalar = orc_avg_scalar(dtype, n);
      how = (dtype == ORC_F16 || dtype == ORC_BF16 || dtype == ORC_F32 || dtype == ORC_F64) ? 1 : 2;
    }
  }
  const int64_t real0 = realChunkElems(kind, n, nChannels, chunkElems, alignElems, count > 0 ? count : 1, 0);
  const int64_t slotElems = sliceElemsFor(real0, slicesPerChunk, sliceElems);
  *maxSliceSeen = 0;
  for (int ch = 0; ch < nChannels; ch++) {
    std::vector<Link> links(n);
    for (auto& l : links) l.data.resize((size_t)slotElems * es * fifoSlots);
    std::vector<RankState> st(n);
    const int64_t loop = loopElems(kind, n, nChannels, chunkElems);
    const int nsteps = stepsPerLoop(kind, n);
    int remaining = n;
    for (auto& s : st) if (count <= 0) { s.done = true; remaining--; }
    long guard = 0;
    while (remaining > 0) {
      bool any = false;
      for (int r = 0; r < n; r++) {
        RankState& s = st[r];
        if (s.done) continue;
        // run rank r until it blocks (this is one "visit" of the scheduler)
        for (;;) {
          if (s.grid >= count) { s.done = true; remaining--; break; }
          const int64_t real = realChunkElems(kind, n, nChannels, chunkElems, alignElems, count, s.grid);
          const char* sb = (const char*)send[r];
          char* rb = (char*)recv[r];
          int inPlace = (kind == kAllGather) ? (sb == rb + (int64_t)r * count * es) : (sb == rb);
          StepDesc d = describeStep(kind, n, r, root, nChannels, ch, count, s.grid, real, s.step, inPlace);
          bool advanceStep = false;
          if (d.nelem <= 0) advanceStep = true;
          else {
            const int64_t sl = sliceElemsFor(d.nelem, slicesPerChunk, sliceElems);
            if (sl > *maxSliceSeen) *maxSliceSeen = sl;
            if (sl > slotElems) return -2;  // a slice would not fit its FIFO slot
            const int64_t off = (int64_t)s.slice * sl;
            if (off >= d.nelem) advanceStep = true;
            else {
              const int64_t len = (d.nelem - off < sl) ? d.nelem - off : sl;
              Link& in = links[(r + n - 1) % n];
              Link& out = links[r];
              if (d.recv && in.tail < s.recvStep + 1) break;                          // wait for data
              if (d.send && out.head + (uint64_t)fifoSlots < s.sendStep + 1) break;    // wait for space
              const char* fifoIn = d.recv ? in.data.data() + (s.recvStep % fifoSlots) * slotElems * es : nullptr;
              char* fifoOut = d.send ? out.data.data() + (s.sendStep % fifoSlots) * slotElems * es : nullptr;
              const char* s0; const char* s1 = nullptr; char* d0; char* d1 = nullptr;
              if (d.useIn) { s0 = sb + (d.inOff + off) * es; s1 = fifoIn; } else s0 = fifoIn;
              if (d.useOut) { d0 = rb + (d.outOff + off) * es; d1 = fifoOut; } else d0 = fifoOut;
              if (s0 && d0) {
                std::vector<char> tmp((size_t)len * es), in0;
                if (how == 1 && d.useIn) {  // source 0 is the user's input: scaled as it enters
                  in0.assign(s0, s0 + (size_t)len * es);
                  orc_scale_apply(dtype, 1, scalar, in0.data(), (size_t)len);
                  s0 = in0.data();
                }
                if (s1) { const void* srcs[2] = {s0, s1}; orc_reduce_copy(dtype, op, 2, srcs, tmp.data(), (size_t)len); }
                else memcpy(tmp.data(), s0, (size_t)len * es);
                if (how == 2 && d.post) orc_scale_apply(dtype, 2, scalar, tmp.data(), (size_t)len);
                memcpy(d0, tmp.data(), (size_t)len * es);
                if (d1) memcpy(d1, tmp.data(), (size_t)len * es);
              }
              if (d.send) { s.sendStep++; out.tail = s.sendStep; }
              if (d.recv) { s.recvStep++; in.head = s.recvStep; }
              s.slice++;
              any = true;
              continue;
            }
          }
          if (advanceStep) {
            s.slice = 0;
            if (++s.step >= nsteps) { s.step = 0; s.grid += loop; }
            any = true;
          }
        }
      }
      if (!any && remaining > 0) return -1;  // deadlock: nobody can move
      if (++guard > 100000000L) return -3;
    }
  }
  return 0;
}

extern "C" int sim_plan_channels(int64_t nBytes, int maxChannels, int64_t bytesPerChannel) {
  return planChannels(nBytes, maxChannels, bytesPerChannel);
}
extern "C" uint64_t sim_cqe_encode(unsigned blk, unsigned cnt, unsigned coll) { return cqeEncode(blk, cnt, coll); }
extern "C" void sim_cqe_decode(uint64_t v, unsigned* blk, unsigned* cnt, unsigned* coll) {
  *blk = cqeBlk(v); *cnt = cqeCnt(v); *coll = cqeCollId(v);
}

// The direct protocol on the host: every rank's share is processed tile by tile, in the order given by
// `order` (a permutation seed: tiles may be taken by any workgroup at any time on the device), with the roles
// and the tile geometry of ring_schedule.h and the oracle's element arithmetic.  Returns the number of elements
// written, or -1 if a destination element was written twice.
extern "C" int64_t sim_direct(int kind, int dtype, int op, int n, int nChannels, int64_t chunkElems, int64_t alignElems,
                              int64_t count, int root, const void* const* send, void* const* recv, uint64_t order) {
  int es = orc_type_size(dtype);
  if (kind == kAllGather || kind == kBroadcast) { count *= es; dtype = ORC_I8; es = 1; }
  const int gk = directGeomKind(kind);
  const int64_t loop = loopElems(gk, n, nChannels, chunkElems);
  const int64_t loops = count > 0 ? (count + loop - 1) / loop : 0;
  const int64_t lastReal = count > 0 ? realChunkElems(gk, n, nChannels, chunkElems, alignElems, count, (loops - 1) * loop) : 0;
  const int64_t tiles = loops * nChannels;
  int64_t written = 0;
  // snapshot of the inputs: in place runs read what the instance started with only where the device does too
  // (each element is read by the one thread that writes it), so reading the live buffers is the faithful model
  std::vector<std::pair<int, int64_t>> work;  // (rank, tile)
  for (int r = 0; r < n; r++)
    for (int64_t t = 0; t < tiles; t++) work.push_back({r, t});
  uint64_t s = order * 0x9E3779B97F4A7C15ull + 1;
  for (size_t i = work.size(); i > 1; i--) {  // Fisher-Yates with splitmix steps
    s += 0x9E3779B97F4A7C15ull;
    uint64_t z = s; z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; z ^= z >> 31;
    std::swap(work[i - 1], work[(size_t)(z % i)]);
  }
  std::vector<char> tmp;
  for (auto& w : work) {
    const int me = w.first;
    const DirectRole role = directRole(kind, n, me, root, count);
    int64_t off, nelem;
    directTile(w.second, nChannels, loops, chunkElems, lastReal, role.tn, role.tme, count, &off, &nelem);
    if (nelem <= 0) continue;
    std::vector<const void*> srcs(role.nSrc);
    for (int t = 0; t < role.nSrc; t++)
      srcs[t] = (const char*)send[(role.firstSrc + t) % n] + (role.srcOff + off) * es;
    tmp.resize((size_t)nelem * es);
    orc_reduce_copy(dtype, op, role.nSrc, srcs.data(), tmp.data(), (size_t)nelem);
    for (int k = 0; k < role.nDst; k++) {
      const int dr = role.onlyDst < 0 ? k : role.onlyDst;
      memcpy((char*)recv[dr] + (role.dstOff + off) * es, tmp.data(), (size_t)nelem * es);
      written += nelem;
    }
  }
  return written;
}
