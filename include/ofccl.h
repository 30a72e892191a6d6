/*
 * ofccl.h - C ABI of the MI355X DFCCL data path.
 *
 * The entry points, their argument order and their error behaviour are the
 * ones the reference declares for its "ofccl" path in src/nccl.h.in; each
 * declaration below cites the line it replaces.  Everything is plain C:
 * opaque handles, raw device pointers, sizes and enums.  Ranks are virtual:
 * all of a communicator's ranks live in one process and one GPU's HBM.
 *
 * Lifecycle (same as the reference, src/enqueue_ofccl.cc:751-1662):
 *   ofcclInitRankCtx -> ofcclPrepare* (one communicator per collId)
 *   -> ofcclFinalizeRankCtx7StartHostThrds -> ofcclRun*(..., callback) ...
 *   -> ofcclDestroy.
 * Completion is reported only through the callback, which runs on the rank
 * context's poller thread.
 */
#ifndef DFCCL_OFCCL_H_
#define DFCCL_OFCCL_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- types shared with the NCCL API (src/nccl.h.in:30-48,113-146) -------- */

typedef struct ncclComm* ncclComm_t;           /* nccl.h.in:30, opaque */
typedef struct ofcclRankCtx* ofcclRankCtx_t;   /* nccl.h.in:32, opaque */
typedef int (*CallbackFunc)(int collId, void* args); /* nccl.h.in:36 */

#define NCCL_UNIQUE_ID_BYTES 128
typedef struct { char internal[NCCL_UNIQUE_ID_BYTES]; } ncclUniqueId; /* nccl.h.in:38-39 */

typedef enum { /* nccl.h.in:42-48 */
  ncclSuccess = 0,
  ncclUnhandledCudaError = 1, /* here: an unhandled HIP error */
  ncclSystemError = 2,
  ncclInternalError = 3,
  ncclInvalidArgument = 4,
  ncclInvalidUsage = 5,
  ncclNumResults = 6
} ncclResult_t;

typedef enum { /* nccl.h.in:113-128 */
  ncclSum = 0,
  ncclProd = 1,
  ncclMax = 2,
  ncclMin = 3,
  ncclAvg = 4,
  ncclNumOps = 5, /* operators made by ncclRedOpCreatePreMulSum have values from here on */
  ncclMaxRedOp = 0x7fffffff
} ncclRedOp_t;

typedef enum { /* nccl.h.in:131-146 */
  ncclInt8 = 0, ncclChar = 0,
  ncclUint8 = 1,
  ncclInt32 = 2, ncclInt = 2,
  ncclUint32 = 3,
  ncclInt64 = 4,
  ncclUint64 = 5,
  ncclFloat16 = 6, ncclHalf = 6,
  ncclFloat32 = 7, ncclFloat = 7,
  ncclFloat64 = 8, ncclDouble = 8,
  ncclBfloat16 = 9,
  ncclNumTypes = 10
} ncclDataType_t;

/* ---- virtual communicators ------------------------------------------------
 * Stand-ins for the stock communicator calls the reference's callers use
 * before ofcclPrepare* (src/nccl.h.in:60-108; src/init.cc:94,1077).  The
 * bootstrap, topology search and transports behind the stock versions are
 * replaced by HBM-resident FIFOs between the virtual ranks of one GPU, so
 * ncclCommInitRank never blocks: ranks that present the same unique id join
 * the same ring 0 -> 1 -> ... -> nranks-1 -> 0 on the current HIP device.
 * As in the reference (src/enqueue_ofccl.cc:807-811) a communicator serves
 * exactly one collId. */
ncclResult_t ncclGetUniqueId(ncclUniqueId* uniqueId);                                      /* nccl.h.in:60 */
ncclResult_t ncclCommInitRank(ncclComm_t* comm, int nranks, ncclUniqueId commId, int rank); /* nccl.h.in:69 */
ncclResult_t ncclCommDestroy(ncclComm_t comm);                                             /* nccl.h.in:83 */
ncclResult_t ncclCommCount(const ncclComm_t comm, int* count);                             /* nccl.h.in:100 */
ncclResult_t ncclCommUserRank(const ncclComm_t comm, int* rank);                           /* nccl.h.in:108 */
const char* ncclGetErrorString(ncclResult_t result);                                       /* nccl.h.in:92 */

/* ---- reduction operators with a scalar (nccl.h.in:148-180) ----------------
 * ncclRedOpCreatePreMulSum makes an operator that multiplies every input by
 * *scalar (one element of `datatype`) before summing, for collectives prepared
 * on `comm` with that datatype (src/enqueue.cc:1443-1490; device semantics
 * src/include/reduce_kernel.h:503-668: one rounded multiply in the element type).
 * Every rank makes its own operator and may give its own scalar: rank r's
 * input enters the sum multiplied by rank r's scalar.  With
 * ncclScalarHostImmediate the scalar is read when the operator is created;
 * with ncclScalarDevice `scalar` is a device address (aligned to the element
 * size) that is dereferenced on the device whenever an instance of a
 * collective prepared with the operator starts, so the memory has to stay
 * valid while the collective is registered, and a new value takes effect with
 * the next ofcclRun* (src/collectives/device/common.h:117-136 dereferences it
 * when the kernel starts on the work element).
 * ncclAvg needs none of this: Prepare turns it into a sum that is divided by
 * the number of ranks afterwards (integer types, C++ integer division) or
 * whose inputs are multiplied by 1/nranks first (float types), as
 * src/enqueue.cc:1326-1357 does. */
typedef enum { ncclScalarDevice = 0, ncclScalarHostImmediate = 1 } ncclScalarResidence_t; /* nccl.h.in:148-156 */
ncclResult_t ncclRedOpCreatePreMulSum(ncclRedOp_t* op, void* scalar, ncclDataType_t datatype,
                                      ncclScalarResidence_t residence, ncclComm_t comm);   /* nccl.h.in:169 */
ncclResult_t ncclRedOpDestroy(ncclRedOp_t op, ncclComm_t comm);                            /* nccl.h.in:179 */

/* ---- rank context ---------------------------------------------------------*/

/* Allocates a rank context for virtual rank `rank` on the current HIP device.
 * Replaces ofcclInitRankCtx, nccl.h.in:202 (src/enqueue_ofccl.cc:751). */
ncclResult_t ofcclInitRankCtx(ofcclRankCtx_t* rankCtx, int rank);

/* Plans every prepared collective, creates the submission / completion queues
 * and starts the poller thread; the daemon kernel starts with the first
 * submission.  Replaces nccl.h.in:213 (src/enqueue_ofccl.cc:1285). */
ncclResult_t ofcclFinalizeRankCtx7StartHostThrds(ofcclRankCtx_t rankCtx);

/* Finalize plus an immediate daemon launch. Replaces nccl.h.in:223
 * (src/enqueue_ofccl.cc:1561). */
ncclResult_t ofcclPrepareDone(ofcclRankCtx_t rankCtx);

/* Submits a quit entry, waits for this rank's workgroups to leave the daemon,
 * joins the poller and frees the context.  Replaces nccl.h.in:234
 * (src/enqueue_ofccl.cc:1582). */
ncclResult_t ofcclDestroy(ofcclRankCtx_t rankCtx);

/* ---- prepare: register one collective under collId ------------------------
 * Validation follows src/enqueue_ofccl.cc:779-813 and src/misc/argcheck.cc:36-71:
 * collId in [0, 2000), at most 2000 collectives per context, a communicator
 * may be registered once (and not again after a rank context that ran its
 * collective has been destroyed: create a new communicator), root / dtype / op in range.  Buffers are given at
 * Run time.  Unlike the reference (which drops `op` and always sums,
 * src/enqueue_ofccl.cc:211-215) the op is honoured: Sum / Prod / Max / Min / Avg and operators made by
 * ncclRedOpCreatePreMulSum, on every ncclDataType_t. */
ncclResult_t ofcclPrepareReduce(size_t count, ncclDataType_t datatype, ncclRedOp_t op, int root, ncclComm_t comm,
                                int collId, ofcclRankCtx_t rankCtx);                       /* nccl.h.in:253 */
ncclResult_t ofcclPrepareBcast(size_t count, ncclDataType_t datatype, int root, ncclComm_t comm, int collId,
                               ofcclRankCtx_t rankCtx);                                    /* nccl.h.in:273 */
ncclResult_t ofcclPrepareBroadcast(size_t count, ncclDataType_t datatype, int root, ncclComm_t comm, int collId,
                                   ofcclRankCtx_t rankCtx);                                /* nccl.h.in:293 */
ncclResult_t ofcclPrepareAllReduce(size_t count, ncclDataType_t datatype, ncclRedOp_t op, ncclComm_t comm,
                                   int collId, ofcclRankCtx_t rankCtx);                    /* nccl.h.in:318 */
ncclResult_t ofcclPrepareReduceScatter(size_t recvcount, ncclDataType_t datatype, ncclRedOp_t op, ncclComm_t comm,
                                       int collId, ofcclRankCtx_t rankCtx);                /* nccl.h.in:353 */
ncclResult_t ofcclPrepareAllGather(size_t sendcount, ncclDataType_t datatype, ncclComm_t comm, int collId,
                                   ofcclRankCtx_t rankCtx);                                /* nccl.h.in:374 */

/* ---- run: submit one instance of a prepared collective --------------------
 * Builds a submission-queue entry and spins while the queue is full
 * (src/collectives_ofccl/ofccl_all_reduce.cc:18-34).  Returns ncclSuccess once
 * the entry is queued.  Unlike the reference, which always returns ncclSuccess
 * (ofccl_all_reduce.cc:29-33), a Run returns ncclSystemError when the daemon
 * kernel could not be launched or had to be aborted (also out of the wait for a
 * full queue or for an earlier instance): no callback will come for that call.
 * ncclInvalidUsage / ncclInvalidArgument report a context that is not
 * finalized, an unknown collId or a pointer that is not a device address.
 * sendbuff / recvbuff are device pointers that must stay valid until
 * `callback(collId, callbackArgs)` has been called on the poller thread.  At
 * most one instance per collId may be in flight; a second Run for the same
 * collId waits for the first. */
ncclResult_t ofcclRunReduce(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                            void* callbackArgs, ofcclRankCtx_t rankCtx);                   /* nccl.h.in:256 */
ncclResult_t ofcclRunBcast(void* buff, int collId, CallbackFunc callback, void* callbackArgs,
                           ofcclRankCtx_t rankCtx);                                        /* nccl.h.in:276 */
ncclResult_t ofcclRunBroadcast(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                               void* callbackArgs, ofcclRankCtx_t rankCtx);                /* nccl.h.in:296 */
ncclResult_t ofcclRunAllReduce(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                               void* callbackArgs, ofcclRankCtx_t rankCtx);                /* nccl.h.in:332 */
ncclResult_t ofcclRunReduceScatter(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                                   void* callbackArgs, ofcclRankCtx_t rankCtx);            /* nccl.h.in:356 */
ncclResult_t ofcclRunAllGather(const void* sendbuff, void* recvbuff, int collId, CallbackFunc callback,
                               void* callbackArgs, ofcclRankCtx_t rankCtx);                /* nccl.h.in:377 */

/* ---- the reduce-copy primitive as a one-shot launch -----------------------
 * dst[i] = op(...op(srcs[0][i], srcs[1][i])..., srcs[nsrcs-1][i]) for count
 * elements, sources folded left to right as ReduceCopy128bMulti does
 * (src/include/common_kernel.h:557-622,629-690).  The same device code moves
 * the data inside the daemon kernel; this entry point exposes it for the
 * semantics check against a host loop and for the bandwidth measurement.
 * Every ncclDataType_t; op is Sum, Prod, Max, Min or Avg (the average over
 * the nsrcs sources: integer sums divided by nsrcs afterwards, float inputs
 * multiplied by 1/nsrcs first, as ncclAvg over nsrcs ranks would be).
 * srcs is a host array of nsrcs (1..8) device pointers; more than four
 * sources take several launches that fold into dst.  chunkBytes is the
 * grain handed to one workgroup at a time (0 = default); stream is a
 * hipStream_t (NULL = the null stream).  Asynchronous; allocates nothing. */
ncclResult_t dfcclReduceCopy(const void* const* srcs, int nsrcs, void* dst, size_t count, ncclDataType_t datatype,
                             ncclRedOp_t op, size_t chunkBytes, void* stream);

/* ---- introspection (reference: counters printed at final quit,
 * src/include/collectives_ofccl.h:173-179, enqueue_ofccl_dev.cu:1148) ------ */

typedef struct {
  uint64_t structBytes;     /* in: sizeof(dfcclStats) as the caller knows it; the library writes no more than that */
  uint64_t sqesRead;        /* submissions taken from the queue              */
  uint64_t cqesWritten;     /* completions posted                            */
  uint64_t ctxSaves;        /* preemptions: contexts saved to HBM            */
  uint64_t ctxLoads;        /* contexts (re)loaded                           */
  uint64_t voluntaryQuits;  /* workgroup exits after a long idle period      */
  uint64_t daemonLaunches;  /* daemon kernel launches on this device         */
  uint64_t forcedQuits;     /* preemptions raised by DFCCL_FORCE_QUIT_EVERY  */
  uint64_t slicesMoved;     /* reduce-copy / copy slices executed            */
  uint64_t sqFullWaits;     /* times a Run found the submission queue full and had to wait (host side) */
} dfcclStats;

/* Sums the counters over this rank's workgroups. Valid after Finalize; exact
 * once the rank is idle.  Set stats->structBytes = sizeof(dfcclStats) before
 * the call: counters added to the end of the structure by a later version of
 * the library are then not written past the caller's copy
 * (ncclInvalidArgument if it is smaller than the first counter's end). */
ncclResult_t dfcclGetStats(ofcclRankCtx_t rankCtx, dfcclStats* stats);

/* Host steady-clock times (ns) of collId's last instance on this rank: when its
 * submission-queue entry was written and when the poller saw its completion
 * entry, i.e. the SQE->CQE interval without the callback's own cost (the
 * reference measures the same interval with its DEBUG_CLOCK_IO probe,
 * src/include/collectives_ofccl.h:50-54). Read it from the callback or later. */
ncclResult_t dfcclGetCollTiming(ofcclRankCtx_t rankCtx, int collId, uint64_t* submitNs, uint64_t* completeNs);

/* Chunk geometry the library planned for collId (needed to reproduce the
 * ring's accumulation order on the host). Valid after Finalize. */
typedef struct {
  int nRanks;
  int nChannels;
  int64_t chunkElems;  /* nominal chunk, elements of the run dtype */
  int64_t alignElems;  /* rounding unit of the per-loop chunk size */
  int64_t sliceElems;  /* nominal slice (one FIFO slot)            */
  int slicesPerChunk;
  int fifoSlots;
  int protocol;        /* 0: FIFO ring, 1: direct (peers read each other's buffers) */
} dfcclCollGeometry;
ncclResult_t dfcclGetCollGeometry(ofcclRankCtx_t rankCtx, int collId, dfcclCollGeometry* geom);

/* Prints to stderr what the host knows about the daemon this rank context is attached to: per rank the entries
 * submitted and completed, how every workgroup left the last launch, the collectives in flight, and what a
 * workgroup that has made no progress for a long time is parked on. (The reference prints comparable state under
 * its DEBUG_* switches, src/collectives_ofccl/device/enqueue_ofccl_dev.cu:1290-1483.) */
ncclResult_t dfcclDumpState(ofcclRankCtx_t rankCtx);

#ifdef __cplusplus
}
#endif
#endif
