/*
 * CPU oracle for the DFCCL single-GPU data path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the reference algorithm, used as the checker
 * in tests, in the smoke test and as the timed CPU baseline.  The shipped
 * library never links, loads or calls anything in this directory.
 *
 * What each function follows in the reference (paths relative to the reference
 * tree):
 *   element ops          src/include/reduce_kernel.h:23-53 (generic Sum/Prod/Max/Min, also for uint8 / uint32 /
 *                        int64 / uint64), :456-469 (fp64 Max/Min = fmax/fmin),
 *                        :485-704 (SumPostDiv, PreMulSum) with src/enqueue.cc:1305-1371 (what ncclAvg becomes),
 *                        :66-134 (int8 Sum/Prod wrap), :146-218 (int8 Max/Min signed),
 *                        :244-440 (fp16 / bf16: one correctly rounded op per step),
 *                        :442-455 (fp32 Max/Min = fmaxf/fminf)
 *   reduce-copy          src/include/common_kernel.h:557-622 (vals = fn(vals, vals2),
 *                        sources folded left to right)
 *   all-reduce ring      src/collectives_ofccl/device/ofccl_all_reduce.h:44-188
 *   reduce-scatter ring  src/collectives_ofccl/device/ofccl_reduce_scatter.h:31-89
 *   all-gather ring      src/collectives_ofccl/device/ofccl_all_gather.h:44-138
 *   reduce chain         src/collectives_ofccl/device/ofccl_reduce.h:44-106
 *   broadcast chain      src/collectives_ofccl/device/ofccl_broadcast.h:33-69
 *   count -> bytes       src/misc/argcheck.cc:53-57 (all-gather / broadcast run as int8)
 *   CQ slot encoding     src/include/collectives_ofccl.h:11-19
 *   SQ full / empty      src/include/enqueue_ofccl.h:51-54, enqueue_ofccl_dev.h:27-30
 *
 * Parity status: the reference holds no golden vectors for this path and cannot
 * be compiled here (CUDA + PTX), so every function below is pinned by
 * independent checks in tests/ (numpy float16 and torch bfloat16 arithmetic for
 * the soft-float code, two's-complement closed forms for the integer ops, a
 * per-element closed form of the ring order for the schedules, permutation
 * identities for the copy collectives).  Not pinned by anything but a live run
 * of the reference, and therefore judged by invariants only: which collectives
 * get preempted and the order of completions.  Max/Min with NaN operands
 * follow fmaxf / fminf (the operand that is a number wins) and are pinned
 * against float64 extremes over the non-NaN operands.  Which of +0 and -0
 * Max/Min return is "parity unpinned" (not fixed by fmax / fmin); test inputs
 * avoid mixing the two zeros.
 */
#ifndef DFCCL_ORACLE_H_
#define DFCCL_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype / op codes are the reference's ncclDataType_t / ncclRedOp_t values
 * (src/nccl.h.in:113-146). */
enum { ORC_I8 = 0, ORC_U8 = 1, ORC_I32 = 2, ORC_U32 = 3, ORC_I64 = 4, ORC_U64 = 5, ORC_F16 = 6, ORC_F32 = 7,
       ORC_F64 = 8, ORC_BF16 = 9 };
/* ORC_AVG is ncclAvg: a sum divided by the group size afterwards (integer types) or with every input multiplied
 * by 1 / size first (float types).  ORC_PREMULSUM is the device op behind ncclRedOpCreatePreMulSum: a sum of
 * inputs multiplied by a caller's scalar (the `_x` functions take its bits). */
enum { ORC_SUM = 0, ORC_PROD = 1, ORC_MAX = 2, ORC_MIN = 3, ORC_AVG = 4, ORC_PREMULSUM = 5 };

/* Chunk geometry of a ring collective. chunk_elems is the nominal chunk
 * (stepSize*CHUNKSTEPS/sizeof(T) in the reference), align_elems the rounding
 * unit of the per-loop real chunk size. */
typedef struct {
  int n_ranks;
  int n_channels;
  int64_t chunk_elems;
  int64_t align_elems;
} orc_geom;

int orc_type_size(int dtype);

/* soft-float conversions (round to nearest even) */
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);

/* One application of op on two elements stored at a and b, result to out. */
void orc_apply(int dtype, int op, const void* a, const void* b, void* out);

/* dst[i] = op(...op(op(src0[i], src1[i]), src2[i])..., src{k-1}[i]), rounded to
 * the storage type after every op. k >= 1 (k == 1 is a copy). */
int orc_reduce_copy(int dtype, int op, int k, const void* const* srcs, void* dst, size_t n);
/* ... with a scalar for ORC_PREMULSUM (the bits of one element, in the low bytes).  For ORC_AVG the group is
 * the k sources. */
int orc_reduce_copy_x(int dtype, int op, uint64_t scalar, int k, const void* const* srcs, void* dst, size_t n);
/* The scalar ncclAvg turns into for a group of n: n itself for integer types, 1/n rounded to the element type
 * for float types (bits in the low bytes). */
uint64_t orc_avg_scalar(int dtype, int n);
/* The two halves of a scaled sum on their own, in place: how = 1 multiplies every element by the scalar (one
 * element's bits), how = 2 divides every element of an integer type by (int)scalar as SumPostDiv does. */
void orc_scale_apply(int dtype, int how, uint64_t scalar, void* buf, size_t n);
/* Same result, element range split statically over nthreads host threads. */
int orc_reduce_copy_mt(int dtype, int op, int k, const void* const* srcs, void* dst, size_t n, int nthreads);

/* Real chunk size of one loop iteration (all-reduce divides by nChannels*nRanks,
 * the others by nChannels). */
int64_t orc_real_chunk(int64_t chunk_elems, int64_t remaining, int64_t divisor, int64_t align_elems);

/* Ring collectives over n virtual ranks, ring order 0 -> 1 -> ... -> n-1 -> 0.
 * send[r] / recv[r] are rank r's buffers. Returns 0 on success. */
int orc_all_reduce(int dtype, int op, const orc_geom* g, int64_t count, const void* const* send, void* const* recv);
int orc_reduce_scatter(int dtype, int op, const orc_geom* g, int64_t recvcount, const void* const* send,
                       void* const* recv);
int orc_all_gather(int dtype, const orc_geom* g, int64_t sendcount, const void* const* send, void* const* recv);
int orc_reduce(int dtype, int op, const orc_geom* g, int64_t count, int root, const void* const* send,
               void* const* recv);
int orc_broadcast(int dtype, const orc_geom* g, int64_t count, int root, const void* const* send, void* const* recv);

/* The reducing collectives with a scalar for ORC_PREMULSUM. */
int orc_all_reduce_x(int dtype, int op, uint64_t scalar, const orc_geom* g, int64_t count, const void* const* send,
                     void* const* recv);
int orc_reduce_scatter_x(int dtype, int op, uint64_t scalar, const orc_geom* g, int64_t recvcount,
                         const void* const* send, void* const* recv);
int orc_reduce_x(int dtype, int op, uint64_t scalar, const orc_geom* g, int64_t count, int root,
                 const void* const* send, void* const* recv);
/* ... and with one scalar per rank (scalars[r] is rank r's): every rank makes its own PreMulSum operator
 * (src/enqueue.cc:1443-1475) and the multiplication is applied to a rank's input by that rank's own primitives
 * (preOp on the user-input source, src/collectives_ofccl/device/ofccl_prims_simple.h:405-411), so rank r's input
 * enters the sum multiplied by rank r's scalar.  At most ORC_MAX_RANKS ranks. */
#define ORC_MAX_RANKS 64
int orc_all_reduce_xr(int dtype, int op, const uint64_t* scalars, const orc_geom* g, int64_t count,
                      const void* const* send, void* const* recv);
int orc_reduce_scatter_xr(int dtype, int op, const uint64_t* scalars, const orc_geom* g, int64_t recvcount,
                          const void* const* send, void* const* recv);
int orc_reduce_xr(int dtype, int op, const uint64_t* scalars, const orc_geom* g, int64_t count, int root,
                  const void* const* send, void* const* recv);

/* Ring position that owns element i of an all-reduce (does the last reduction
 * and so fixes the accumulation order). Closed form, independent of the
 * simulation above. */
int orc_all_reduce_owner(const orc_geom* g, int64_t count, int64_t i);

/* Completion-queue slot value: blockIdx<<56 | (cnt & 0xFFFFFF)<<32 | collId. */
uint64_t orc_cqe_encode(unsigned blk, unsigned cnt, unsigned coll_id);
void orc_cqe_decode(uint64_t v, unsigned* blk, unsigned* cnt, unsigned* coll_id);

/* Sequential model of the submission ring: length entries, one kept empty. */
int orc_sq_full(uint64_t head, uint64_t tail, uint64_t length);
int orc_sq_empty(uint64_t frontier, uint64_t tail);

#ifdef __cplusplus
}
#endif
#endif
