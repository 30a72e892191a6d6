/* CPU oracle for the DFCCL data path. Test infrastructure only; see dfccl_oracle.h
 * for the reference lines every function follows and how each one is pinned. */
#include "dfccl_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

int orc_type_size(int dtype) {
  switch (dtype) {
    case ORC_I8: case ORC_U8: return 1;
    case ORC_I32: case ORC_U32: case ORC_F32: return 4;
    case ORC_I64: case ORC_U64: case ORC_F64: return 8;
    case ORC_F16: case ORC_BF16: return 2;
    default: return 0;
  }
}

static int is_float_type(int dtype) { return dtype == ORC_F16 || dtype == ORC_BF16 || dtype == ORC_F32 || dtype == ORC_F64; }

/* ---------------------------------------------------------------- soft float */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t orc_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb; /* round to nearest, ties to even */
  return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t orc_f32_to_f16(float f) {
  uint32_t u = f2u(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t absu = u & 0x7fffffffu;
  if (absu >= 0x7f800000u) { /* inf / nan */
    if (absu > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absu >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absu >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absu < 0x38800000u) { /* below the smallest normal half 2^-14: subnormal result */
    if (absu < 0x33000000u) { /* < 2^-25: rounds to zero (2^-25 itself ties to even = 0) */
      return (uint16_t)sign;
    }
    /* value = mant * 2^(e-150); half subnormal unit is 2^-24 */
    uint32_t e = absu >> 23;
    uint32_t mant = (absu & 0x007fffffu) | 0x00800000u;
    uint32_t shift = 126u - e; /* in [14, 24]: result = mant >> shift in units of 2^-24 */
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  /* normal: rebias exponent 127 -> 15, round 13 dropped bits to nearest even */
  uint32_t v = absu - 0x38000000u;
  uint32_t lsb = (v >> 13) & 1u;
  v += 0x0fffu + lsb;
  return (uint16_t)(sign | (v >> 13));
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0) {
    if (m == 0) return u2f(sign);
    /* subnormal: m * 2^-24 */
    float v = (float)m * 5.9604644775390625e-08f;
    return u2f(f2u(v) | sign);
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* ------------------------------------------------------------- element ops */

static inline float op_f32(int op, float a, float b) {
  switch (op) {
    case ORC_SUM: return a + b;
    case ORC_PROD: return a * b;
    case ORC_MAX: return fmaxf(a, b);
    default: return fminf(a, b);
  }
}
static inline int32_t op_i32(int op, int32_t a, int32_t b) {
  switch (op) {
    case ORC_SUM: return (int32_t)((uint32_t)a + (uint32_t)b);
    case ORC_PROD: return (int32_t)((uint32_t)a * (uint32_t)b);
    case ORC_MAX: return (a < b) ? b : a;
    default: return (a < b) ? a : b;
  }
}
static inline int8_t op_i8(int op, int8_t a, int8_t b) {
  switch (op) {
    case ORC_SUM: return (int8_t)(uint8_t)((uint8_t)a + (uint8_t)b);
    case ORC_PROD: return (int8_t)(uint8_t)((unsigned)(uint8_t)a * (unsigned)(uint8_t)b);
    case ORC_MAX: return (a > b) ? a : b;
    default: return (a < b) ? a : b;
  }
}
/* the generic functors of src/include/reduce_kernel.h:23-53 on the remaining integer types (unsigned arithmetic
 * wraps; Max = (x<y)?y:x, Min = (x<y)?x:y) and fmax / fmin for double (:456-469) */
static inline uint8_t op_u8(int op, uint8_t a, uint8_t b) {
  switch (op) {
    case ORC_SUM: return (uint8_t)(a + b);
    case ORC_PROD: return (uint8_t)((unsigned)a * (unsigned)b);
    case ORC_MAX: return (a > b) ? a : b;
    default: return (a < b) ? a : b;
  }
}
static inline uint32_t op_u32(int op, uint32_t a, uint32_t b) {
  switch (op) {
    case ORC_SUM: return a + b;
    case ORC_PROD: return a * b;
    case ORC_MAX: return (a < b) ? b : a;
    default: return (a < b) ? a : b;
  }
}
static inline int64_t op_i64(int op, int64_t a, int64_t b) {
  switch (op) {
    case ORC_SUM: return (int64_t)((uint64_t)a + (uint64_t)b);
    case ORC_PROD: return (int64_t)((uint64_t)a * (uint64_t)b);
    case ORC_MAX: return (a < b) ? b : a;
    default: return (a < b) ? a : b;
  }
}
static inline uint64_t op_u64(int op, uint64_t a, uint64_t b) {
  switch (op) {
    case ORC_SUM: return a + b;
    case ORC_PROD: return a * b;
    case ORC_MAX: return (a < b) ? b : a;
    default: return (a < b) ? a : b;
  }
}
static inline double op_f64(int op, double a, double b) {
  switch (op) {
    case ORC_SUM: return a + b;
    case ORC_PROD: return a * b;
    case ORC_MAX: return fmax(a, b);
    default: return fmin(a, b);
  }
}
static inline uint16_t op_f16(int op, uint16_t a, uint16_t b) {
  return orc_f32_to_f16(op_f32(op, orc_f16_to_f32(a), orc_f16_to_f32(b)));
}
static inline uint16_t op_bf16(int op, uint16_t a, uint16_t b) {
  return orc_f32_to_bf16(op_f32(op, orc_bf16_to_f32(a), orc_bf16_to_f32(b)));
}

void orc_apply(int dtype, int op, const void* a, const void* b, void* out) {
  switch (dtype) {
    case ORC_I8: *(int8_t*)out = op_i8(op, *(const int8_t*)a, *(const int8_t*)b); break;
    case ORC_I32: *(int32_t*)out = op_i32(op, *(const int32_t*)a, *(const int32_t*)b); break;
    case ORC_F16: *(uint16_t*)out = op_f16(op, *(const uint16_t*)a, *(const uint16_t*)b); break;
    case ORC_F32: *(float*)out = op_f32(op, *(const float*)a, *(const float*)b); break;
    case ORC_BF16: *(uint16_t*)out = op_bf16(op, *(const uint16_t*)a, *(const uint16_t*)b); break;
    case ORC_U8: *(uint8_t*)out = op_u8(op, *(const uint8_t*)a, *(const uint8_t*)b); break;
    case ORC_U32: *(uint32_t*)out = op_u32(op, *(const uint32_t*)a, *(const uint32_t*)b); break;
    case ORC_I64: *(int64_t*)out = op_i64(op, *(const int64_t*)a, *(const int64_t*)b); break;
    case ORC_U64: *(uint64_t*)out = op_u64(op, *(const uint64_t*)a, *(const uint64_t*)b); break;
    case ORC_F64: *(double*)out = op_f64(op, *(const double*)a, *(const double*)b); break;
    default: break;
  }
}

/* out[i] = op(a[i], b[i]) over a contiguous range; out may alias a or b. */
#define RANGE_LOOP(T, FN)                                         \
  do {                                                            \
    const T* pa = (const T*)a; const T* pb = (const T*)b; T* po = (T*)out; \
    switch (op) {                                                 \
      case ORC_SUM: for (size_t i = 0; i < n; i++) po[i] = FN(ORC_SUM, pa[i], pb[i]); break;   \
      case ORC_PROD: for (size_t i = 0; i < n; i++) po[i] = FN(ORC_PROD, pa[i], pb[i]); break; \
      case ORC_MAX: for (size_t i = 0; i < n; i++) po[i] = FN(ORC_MAX, pa[i], pb[i]); break;   \
      default: for (size_t i = 0; i < n; i++) po[i] = FN(ORC_MIN, pa[i], pb[i]); break;        \
    }                                                             \
  } while (0)

static void apply_range(int dtype, int op, const void* a, const void* b, void* out, size_t n) {
  switch (dtype) {
    case ORC_I8: RANGE_LOOP(int8_t, op_i8); break;
    case ORC_I32: RANGE_LOOP(int32_t, op_i32); break;
    case ORC_F16: RANGE_LOOP(uint16_t, op_f16); break;
    case ORC_F32: RANGE_LOOP(float, op_f32); break;
    case ORC_BF16: RANGE_LOOP(uint16_t, op_bf16); break;
    case ORC_U8: RANGE_LOOP(uint8_t, op_u8); break;
    case ORC_U32: RANGE_LOOP(uint32_t, op_u32); break;
    case ORC_I64: RANGE_LOOP(int64_t, op_i64); break;
    case ORC_U64: RANGE_LOOP(uint64_t, op_u64); break;
    case ORC_F64: RANGE_LOOP(double, op_f64); break;
    default: break;
  }
}

/* ------------------------------------------------- scaled sums (ncclAvg, PreMulSum)
 *
 * The reference turns ncclAvg into a device op with a scalar (hostToDevRedOp, src/enqueue.cc:1305-1371):
 * integer types -> SumPostDiv with n = nRanks, float types -> PreMulSum with the scalar 1/nRanks converted
 * to the element type.  PreMulSum multiplies every rank's input by the scalar as it enters the reduction
 * (preOp on the user-input source, src/collectives_ofccl/device/ofccl_prims_simple.h:405-411,
 * src/include/common_kernel.h:506-538), one correctly rounded multiply in the element type
 * (src/include/reduce_kernel.h:503-668); SumPostDiv divides the finished sum, T(x / n) with C++ integer
 * division (:491-501), at the step that writes the final value (postOp = true:
 * ofccl_all_reduce.h:132, ofccl_reduce_scatter.h:84, ofccl_reduce.h:78). */

typedef struct {
  int base;      /* ORC_SUM..ORC_MIN: the op applied between elements */
  int pre;       /* multiply every input by a scalar (bits of one element) first */
  int post;      /* divide the final value by (int)scalar */
  uint64_t scalar;
  /* PreMulSum with one scalar per rank: every rank makes its own operator, and the multiplication is applied
   * to a rank's input where that rank reads it (preOp on the user-input source of the rank's own primitives,
   * src/collectives_ofccl/device/ofccl_prims_simple.h:405-411), so input r is scaled by rank r's scalar.
   * NULL: `scalar` serves every rank. */
  const uint64_t* per_rank;
} orc_xop;

uint64_t orc_avg_scalar(int dtype, int n) {
  uint64_t bits = 0;
  if (!is_float_type(dtype)) return (uint64_t)n;
  if (dtype == ORC_F64) { double d = 1.0 / n; memcpy(&bits, &d, 8); }
  else {
    float f = (float)(1.0 / n);
    if (dtype == ORC_F32) { uint32_t u = f2u(f); bits = u; }
    else if (dtype == ORC_F16) bits = orc_f32_to_f16(f);
    else bits = orc_f32_to_bf16(f);
  }
  return bits;
}

/* resolves a public op code (+ scalar for ORC_PREMULSUM, group size for ORC_AVG); returns 0 if valid */
static int resolve_op(int dtype, int op, uint64_t scalar, int n, orc_xop* x) {
  x->base = op; x->pre = 0; x->post = 0; x->scalar = 0; x->per_rank = NULL;
  if (op >= ORC_SUM && op <= ORC_MIN) return 0;
  x->base = ORC_SUM;
  if (op == ORC_AVG) {
    x->scalar = orc_avg_scalar(dtype, n);
    if (is_float_type(dtype)) x->pre = 1; else x->post = 1;
    return 0;
  }
  if (op == ORC_PREMULSUM) { x->pre = 1; x->scalar = scalar; return 0; }
  return -1;
}

/* out[i] = in[i] * scalar, one multiply in the element type */
static void premul_range(int dtype, uint64_t scalar, const void* in, void* out, size_t n) {
  const size_t s = (size_t)orc_type_size(dtype);
  char k[8];
  memcpy(k, &scalar, 8);  /* little endian: the low bytes hold the element */
  for (size_t i = 0; i < n; i++) orc_apply(dtype, ORC_PROD, (const char*)in + i * s, k, (char*)out + i * s);
}

/* x[i] = T(x[i] / n), the integer division of C++ after the usual arithmetic conversions with `int n` */
static void postdiv_range(int dtype, uint64_t scalar, void* x, size_t n) {
  const int d = (int)scalar;
  switch (dtype) {
    case ORC_I8: { int8_t* p = x; for (size_t i = 0; i < n; i++) p[i] = (int8_t)((int)p[i] / d); break; }
    case ORC_U8: { uint8_t* p = x; for (size_t i = 0; i < n; i++) p[i] = (uint8_t)((int)p[i] / d); break; }
    case ORC_I32: { int32_t* p = x; for (size_t i = 0; i < n; i++) p[i] = p[i] / d; break; }
    case ORC_U32: { uint32_t* p = x; for (size_t i = 0; i < n; i++) p[i] = p[i] / (uint32_t)d; break; }
    case ORC_I64: { int64_t* p = x; for (size_t i = 0; i < n; i++) p[i] = p[i] / (int64_t)d; break; }
    case ORC_U64: { uint64_t* p = x; for (size_t i = 0; i < n; i++) p[i] = p[i] / (uint64_t)(int64_t)d; break; }
    default: break;
  }
}

void orc_scale_apply(int dtype, int how, uint64_t scalar, void* buf, size_t n) {
  if (how == 1) premul_range(dtype, scalar, buf, buf, n);
  else if (how == 2) postdiv_range(dtype, scalar, buf, n);
}

/* rank r's input as it enters the reduction: the buffer itself, or a copy in tmp scaled by r's scalar */
static const void* entering(int dtype, const orc_xop* x, int r, const void* in, void* tmp, size_t n) {
  if (!x->pre) return in;
  premul_range(dtype, x->per_rank ? x->per_rank[r] : x->scalar, in, tmp, n);
  return tmp;
}

/* the same resolution with one scalar per rank for ORC_PREMULSUM (scalars may be NULL for every other op) */
static int resolve_op_r(int dtype, int op, const uint64_t* scalars, int n, orc_xop* x) {
  if (op == ORC_PREMULSUM && scalars == NULL) return -1;
  if (resolve_op(dtype, op, 0, n, x) != 0) return -1;
  if (op == ORC_PREMULSUM) x->per_rank = scalars;
  return 0;
}

/* ------------------------------------------------------------- reduce-copy */

static void reduce_copy_range(int dtype, const orc_xop* x, int k, const void* const* srcs, void* dst, size_t begin,
                              size_t n) {
  size_t s = (size_t)orc_type_size(dtype);
  char* d = (char*)dst + begin * s;
  if (k == 1 && !x->pre && !x->post) {
    memmove(d, (const char*)srcs[0] + begin * s, n * s);
    return;
  }
  /* fold left to right; the first op reads src0 and src1, later ones the running value.  Every source is a
   * user input here, so a pre-multiplication applies to each of them. */
  void* tmp = x->pre ? malloc(n * s + 1) : NULL;
  void* tmp0 = x->pre ? malloc(n * s + 1) : NULL;
  const void* first = entering(dtype, x, 0, (const char*)srcs[0] + begin * s, tmp0, n);
  if (k == 1) memmove(d, first, n * s);
  else apply_range(dtype, x->base, first, entering(dtype, x, 1, (const char*)srcs[1] + begin * s, tmp, n), d, n);
  for (int j = 2; j < k; j++)
    apply_range(dtype, x->base, d, entering(dtype, x, j, (const char*)srcs[j] + begin * s, tmp, n), d, n);
  if (x->post) postdiv_range(dtype, x->scalar, d, n);
  free(tmp);
  free(tmp0);
}

int orc_reduce_copy_x(int dtype, int op, uint64_t scalar, int k, const void* const* srcs, void* dst, size_t n) {
  orc_xop x;
  if (orc_type_size(dtype) == 0 || k < 1 || resolve_op(dtype, op, scalar, k, &x) != 0) return -1;
  reduce_copy_range(dtype, &x, k, srcs, dst, 0, n);
  return 0;
}

int orc_reduce_copy(int dtype, int op, int k, const void* const* srcs, void* dst, size_t n) {
  return orc_reduce_copy_x(dtype, op, 0, k, srcs, dst, n);
}

typedef struct {
  int dtype, k;
  orc_xop x;
  const void* const* srcs;
  void* dst;
  size_t begin, n;
} rc_job;

static void* rc_thread(void* p) {
  rc_job* j = (rc_job*)p;
  reduce_copy_range(j->dtype, &j->x, j->k, j->srcs, j->dst, j->begin, j->n);
  return NULL;
}

int orc_reduce_copy_mt(int dtype, int op, int k, const void* const* srcs, void* dst, size_t n, int nthreads) {
  orc_xop x;
  if (orc_type_size(dtype) == 0 || k < 1 || resolve_op(dtype, op, 0, k, &x) != 0) return -1;
  if (nthreads <= 1) return orc_reduce_copy(dtype, op, k, srcs, dst, n);
  if (nthreads > 256) nthreads = 256;
  pthread_t th[256];
  rc_job jobs[256];
  size_t per = (n + (size_t)nthreads - 1) / (size_t)nthreads;
  per = (per + 63) & ~(size_t)63;
  int started = 0;
  for (int t = 0; t < nthreads; t++) {
    size_t b = (size_t)t * per;
    if (b >= n) break;
    size_t len = (n - b < per) ? n - b : per;
    jobs[t] = (rc_job){dtype, k, x, srcs, dst, b, len};
    if (pthread_create(&th[t], NULL, rc_thread, &jobs[t]) != 0) {
      rc_thread(&jobs[t]);
      th[t] = 0;
      started = t + 1;
      continue;
    }
    started = t + 1;
  }
  for (int t = 0; t < started; t++)
    if (th[t]) pthread_join(th[t], NULL);
  return 0;
}

/* ------------------------------------------------------------ ring schedule */

static inline int64_t div_up(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t round_up(int64_t a, int64_t b) { return div_up(a, b) * b; }
static inline int64_t min64(int64_t a, int64_t b) { return a < b ? a : b; }

int64_t orc_real_chunk(int64_t chunk_elems, int64_t remaining, int64_t divisor, int64_t align_elems) {
  int64_t r = min64(chunk_elems, div_up(remaining, divisor));
  return round_up(r, align_elems);
}

static int geom_ok(const orc_geom* g) {
  return g && g->n_ranks >= 1 && g->n_channels >= 1 && g->chunk_elems >= 1 && g->align_elems >= 1;
}

/* A message in flight on the link rank -> next rank: the data of one chunk. */
typedef struct {
  char* data;
  int64_t nelem;
} orc_msg;

static void local_copy(int dtype, const void* src, void* dst, int64_t n) {
  if (n > 0 && src != dst) memmove(dst, src, (size_t)n * (size_t)orc_type_size(dtype));
}

int orc_all_reduce(int dtype, int op, const orc_geom* g, int64_t count, const void* const* send, void* const* recv) {
  return orc_all_reduce_x(dtype, op, 0, g, count, send, recv);
}

int orc_all_reduce_x(int dtype, int op, uint64_t scalar, const orc_geom* g, int64_t count, const void* const* send,
                     void* const* recv) {
  uint64_t same[ORC_MAX_RANKS];
  if (!geom_ok(g) || g->n_ranks > ORC_MAX_RANKS) return -1;
  for (int r = 0; r < g->n_ranks; r++) same[r] = scalar;
  return orc_all_reduce_xr(dtype, op, same, g, count, send, recv);
}

int orc_all_reduce_xr(int dtype, int op, const uint64_t* scalars, const orc_geom* g, int64_t count,
                      const void* const* send, void* const* recv) {
  orc_xop x;
  if (!geom_ok(g) || orc_type_size(dtype) == 0 || resolve_op_r(dtype, op, scalars, g->n_ranks, &x) != 0) return -1;
  const int n = g->n_ranks;
  const size_t s = (size_t)orc_type_size(dtype);
  if (n == 1) { /* one rank: a copy, with the scaling a sum of one term still gets */
    const void* src[1] = {send[0]};
    reduce_copy_range(dtype, &x, 1, src, recv[0], 0, (size_t)count);
    return 0;
  }
  op = x.base;
  char* tmp = malloc((size_t)round_up(g->chunk_elems, g->align_elems) * s + 1);
  const int64_t loop_size = (int64_t)g->n_channels * n * g->chunk_elems;
  const int64_t max_chunk = round_up(g->chunk_elems, g->align_elems);
  orc_msg* cur = calloc((size_t)n, sizeof(orc_msg));
  orc_msg* prv = calloc((size_t)n, sizeof(orc_msg));
  for (int r = 0; r < n; r++) {
    cur[r].data = malloc((size_t)max_chunk * s);
    prv[r].data = malloc((size_t)max_chunk * s);
  }
  for (int bid = 0; bid < g->n_channels; bid++) {
    for (int64_t grid = 0; grid < count; grid += loop_size) {
      const int64_t real = orc_real_chunk(g->chunk_elems, count - grid, (int64_t)g->n_channels * n, g->align_elems);
      for (int step = 0; step < 2 * n - 1; step++) {
        for (int r = 0; r < n; r++) {
          const int prev = (r + n - 1) % n;
          int chunk;
          if (step == 0) chunk = (r + n - 1) % n;
          else if (step <= n - 2) chunk = (r + n - (step + 1)) % n;
          else if (step == n - 1) chunk = r;
          else if (step <= 2 * n - 3) chunk = (r + n - (step - n + 1)) % n;
          else chunk = (r + 1) % n;
          const int64_t off = grid + (int64_t)bid * n * real + (int64_t)chunk * real;
          int64_t nelem = min64(real, count - off);
          if (nelem < 0) nelem = 0;
          const char* in = (const char*)send[r] + (size_t)off * s;
          char* out = (char*)recv[r] + (size_t)off * s;
          if (step <= n - 1) in = entering(dtype, &x, r, in, tmp, (size_t)nelem); /* the steps that read the user's input */
          if (step == 0) { /* send */
            memcpy(cur[r].data, in, (size_t)nelem * s);
          } else if (step <= n - 2) { /* recvReduceSend */
            apply_range(dtype, op, in, prv[prev].data, cur[r].data, (size_t)nelem);
          } else if (step == n - 1) { /* recvReduceCopySend, postOp = true */
            apply_range(dtype, op, in, prv[prev].data, cur[r].data, (size_t)nelem);
            if (x.post) postdiv_range(dtype, x.scalar, cur[r].data, (size_t)nelem);
            memcpy(out, cur[r].data, (size_t)nelem * s);
          } else if (step <= 2 * n - 3) { /* recvCopySend */
            memcpy(cur[r].data, prv[prev].data, (size_t)nelem * s);
            memcpy(out, cur[r].data, (size_t)nelem * s);
          } else { /* recv */
            memcpy(out, prv[prev].data, (size_t)nelem * s);
          }
          cur[r].nelem = nelem;
        }
        orc_msg* t = cur; cur = prv; prv = t;
      }
    }
  }
  for (int r = 0; r < n; r++) { free(cur[r].data); free(prv[r].data); }
  free(cur); free(prv); free(tmp);
  return 0;
}

int orc_all_reduce_owner(const orc_geom* g, int64_t count, int64_t i) {
  const int n = g->n_ranks;
  const int64_t loop_size = (int64_t)g->n_channels * n * g->chunk_elems;
  const int64_t l = i / loop_size;
  const int64_t grid = l * loop_size;
  const int64_t real = orc_real_chunk(g->chunk_elems, count - grid, (int64_t)g->n_channels * n, g->align_elems);
  const int64_t rel = i - grid;
  const int64_t bid = rel / (n * real);
  return (int)((rel - bid * n * real) / real);
}

int orc_reduce_scatter(int dtype, int op, const orc_geom* g, int64_t recvcount, const void* const* send,
                       void* const* recv) {
  return orc_reduce_scatter_x(dtype, op, 0, g, recvcount, send, recv);
}

int orc_reduce_scatter_x(int dtype, int op, uint64_t scalar, const orc_geom* g, int64_t recvcount,
                         const void* const* send, void* const* recv) {
  uint64_t same[ORC_MAX_RANKS];
  if (!geom_ok(g) || g->n_ranks > ORC_MAX_RANKS) return -1;
  for (int r = 0; r < g->n_ranks; r++) same[r] = scalar;
  return orc_reduce_scatter_xr(dtype, op, same, g, recvcount, send, recv);
}

int orc_reduce_scatter_xr(int dtype, int op, const uint64_t* scalars, const orc_geom* g, int64_t recvcount,
                          const void* const* send, void* const* recv) {
  orc_xop x;
  if (!geom_ok(g) || orc_type_size(dtype) == 0 || resolve_op_r(dtype, op, scalars, g->n_ranks, &x) != 0) return -1;
  const int n = g->n_ranks;
  const size_t s = (size_t)orc_type_size(dtype);
  if (n == 1) {
    const void* src[1] = {send[0]};
    reduce_copy_range(dtype, &x, 1, src, recv[0], 0, (size_t)recvcount);
    return 0;
  }
  op = x.base;
  char* tmp = malloc((size_t)round_up(g->chunk_elems, g->align_elems) * s + 1);
  const int64_t loop_size = (int64_t)g->n_channels * g->chunk_elems;
  const int64_t max_chunk = round_up(g->chunk_elems, g->align_elems);
  orc_msg* cur = calloc((size_t)n, sizeof(orc_msg));
  orc_msg* prv = calloc((size_t)n, sizeof(orc_msg));
  for (int r = 0; r < n; r++) {
    cur[r].data = malloc((size_t)max_chunk * s);
    prv[r].data = malloc((size_t)max_chunk * s);
  }
  for (int bid = 0; bid < g->n_channels; bid++) {
    for (int64_t grid = 0; grid < recvcount; grid += loop_size) {
      const int64_t real = orc_real_chunk(g->chunk_elems, recvcount - grid, g->n_channels, g->align_elems);
      const int64_t chunk_off = grid + (int64_t)bid * real;
      int64_t nelem = min64(real, recvcount - chunk_off);
      if (nelem < 0) nelem = 0;
      for (int step = 0; step < n; step++) {
        for (int r = 0; r < n; r++) {
          const int prev = (r + n - 1) % n;
          /* ringRanks[i] of rank r is (r + i) % n */
          int dest;
          if (step == 0) dest = (r + n - 1) % n;
          else if (step <= n - 2) dest = (r + n - (step + 1)) % n;
          else dest = r;
          const int64_t off = chunk_off + (int64_t)dest * recvcount;
          const char* in = entering(dtype, &x, r, (const char*)send[r] + (size_t)off * s, tmp, (size_t)nelem);
          if (step == 0) {
            memcpy(cur[r].data, in, (size_t)nelem * s);
          } else if (step <= n - 2) {
            apply_range(dtype, op, in, prv[prev].data, cur[r].data, (size_t)nelem);
          } else {
            /* stage through the message buffer so an in-place recv buffer is safe; postOp = true */
            apply_range(dtype, op, in, prv[prev].data, cur[r].data, (size_t)nelem);
            if (x.post) postdiv_range(dtype, x.scalar, cur[r].data, (size_t)nelem);
            memcpy((char*)recv[r] + (size_t)chunk_off * s, cur[r].data, (size_t)nelem * s);
          }
        }
        orc_msg* t = cur; cur = prv; prv = t;
      }
    }
  }
  for (int r = 0; r < n; r++) { free(cur[r].data); free(prv[r].data); }
  free(cur); free(prv); free(tmp);
  return 0;
}

int orc_all_gather(int dtype, const orc_geom* g, int64_t sendcount, const void* const* send, void* const* recv) {
  if (!geom_ok(g) || orc_type_size(dtype) == 0) return -1;
  /* the reference runs all-gather on bytes: count *= sizeof(T), dtype = int8 */
  const int n = g->n_ranks;
  const int64_t size = sendcount * orc_type_size(dtype);
  if (n == 1) { local_copy(ORC_I8, send[0], recv[0], size); return 0; }
  const int64_t loop_size = (int64_t)g->n_channels * g->chunk_elems;
  const int64_t max_chunk = round_up(g->chunk_elems, g->align_elems);
  orc_msg* cur = calloc((size_t)n, sizeof(orc_msg));
  orc_msg* prv = calloc((size_t)n, sizeof(orc_msg));
  for (int r = 0; r < n; r++) {
    cur[r].data = malloc((size_t)max_chunk);
    prv[r].data = malloc((size_t)max_chunk);
  }
  for (int bid = 0; bid < g->n_channels; bid++) {
    for (int64_t grid = 0; grid < size; grid += loop_size) {
      const int64_t real = orc_real_chunk(g->chunk_elems, size - grid, g->n_channels, g->align_elems);
      const int64_t chunk_off = grid + (int64_t)bid * real;
      int64_t nelem = min64(real, size - chunk_off);
      if (nelem < 0) nelem = 0;
      for (int step = 0; step < n; step++) {
        for (int r = 0; r < n; r++) {
          const int prev = (r + n - 1) % n;
          int dest;
          if (step == 0) dest = r;
          else if (step <= n - 2) dest = (r + n - step) % n;
          else dest = (r + 1) % n;
          const int64_t off = chunk_off + (int64_t)dest * size;
          char* out = (char*)recv[r] + off;
          if (step == 0) {
            const char* in = (const char*)send[r] + chunk_off;
            memcpy(cur[r].data, in, (size_t)nelem);
            if (in != out) memmove(out, in, (size_t)nelem);
          } else if (step <= n - 2) {
            memcpy(cur[r].data, prv[prev].data, (size_t)nelem);
            memcpy(out, cur[r].data, (size_t)nelem);
          } else {
            memcpy(out, prv[prev].data, (size_t)nelem);
          }
        }
        orc_msg* t = cur; cur = prv; prv = t;
      }
    }
  }
  for (int r = 0; r < n; r++) { free(cur[r].data); free(prv[r].data); }
  free(cur); free(prv);
  return 0;
}

int orc_reduce(int dtype, int op, const orc_geom* g, int64_t count, int root, const void* const* send,
               void* const* recv) {
  return orc_reduce_x(dtype, op, 0, g, count, root, send, recv);
}

int orc_reduce_x(int dtype, int op, uint64_t scalar, const orc_geom* g, int64_t count, int root,
                 const void* const* send, void* const* recv) {
  uint64_t same[ORC_MAX_RANKS];
  if (!geom_ok(g) || g->n_ranks > ORC_MAX_RANKS) return -1;
  for (int r = 0; r < g->n_ranks; r++) same[r] = scalar;
  return orc_reduce_xr(dtype, op, same, g, count, root, send, recv);
}

int orc_reduce_xr(int dtype, int op, const uint64_t* scalars, const orc_geom* g, int64_t count, int root,
                  const void* const* send, void* const* recv) {
  orc_xop x;
  if (!geom_ok(g) || orc_type_size(dtype) == 0 || resolve_op_r(dtype, op, scalars, g->n_ranks, &x) != 0) return -1;
  const int n = g->n_ranks;
  if (root < 0 || root >= n) return -1;
  const size_t s = (size_t)orc_type_size(dtype);
  if (n == 1) {
    const void* src[1] = {send[0]};
    reduce_copy_range(dtype, &x, 1, src, recv[0], 0, (size_t)count);
    return 0;
  }
  op = x.base;
  char* tmp = malloc((size_t)round_up(g->chunk_elems, g->align_elems) * s + 1);
  const int64_t loop_size = (int64_t)g->n_channels * g->chunk_elems;
  const int64_t max_chunk = round_up(g->chunk_elems, g->align_elems);
  char* msg = malloc((size_t)max_chunk * s);
  for (int bid = 0; bid < g->n_channels; bid++) {
    for (int64_t grid = 0; grid < count; grid += loop_size) {
      const int64_t real = orc_real_chunk(g->chunk_elems, count - grid, g->n_channels, g->align_elems);
      const int64_t off = grid + (int64_t)bid * real;
      int64_t nelem = min64(real, count - off);
      if (nelem < 0) nelem = 0;
      /* the chain starts at the rank whose predecessor is the root and ends at the root */
      for (int k = 1; k <= n; k++) {
        const int r = (root + k) % n;
        const char* in = entering(dtype, &x, r, (const char*)send[r] + (size_t)off * s, tmp, (size_t)nelem);
        if (k == 1) {
          memcpy(msg, in, (size_t)nelem * s); /* send */
        } else if (k < n) {
          apply_range(dtype, op, in, msg, msg, (size_t)nelem); /* recvReduceSend */
        } else {
          apply_range(dtype, op, in, msg, msg, (size_t)nelem); /* recvReduceCopy, postOp = true */
          if (x.post) postdiv_range(dtype, x.scalar, msg, (size_t)nelem);
          memcpy((char*)recv[r] + (size_t)off * s, msg, (size_t)nelem * s);
        }
      }
    }
  }
  free(msg);
  free(tmp);
  return 0;
}

int orc_broadcast(int dtype, const orc_geom* g, int64_t count, int root, const void* const* send, void* const* recv) {
  if (!geom_ok(g) || orc_type_size(dtype) == 0) return -1;
  const int n = g->n_ranks;
  if (root < 0 || root >= n) return -1;
  const int64_t size = count * orc_type_size(dtype);
  if (n == 1) { local_copy(ORC_I8, send[0], recv[0], size); return 0; }
  const int64_t loop_size = (int64_t)g->n_channels * g->chunk_elems;
  for (int bid = 0; bid < g->n_channels; bid++) {
    for (int64_t grid = 0; grid < size; grid += loop_size) {
      const int64_t real = orc_real_chunk(g->chunk_elems, size - grid, g->n_channels, g->align_elems);
      const int64_t off = grid + (int64_t)bid * real;
      int64_t nelem = min64(real, size - off);
      if (nelem <= 0) continue;
      const char* src = (const char*)send[root] + off;
      for (int k = 0; k < n; k++) {
        const int r = (root + k) % n;
        char* out = (char*)recv[r] + off;
        if (out != src) memmove(out, src, (size_t)nelem);
      }
    }
  }
  return 0;
}

/* ------------------------------------------------------------------ queues */

uint64_t orc_cqe_encode(unsigned blk, unsigned cnt, unsigned coll_id) {
  return ((uint64_t)(blk & 0xffu) << 56) | ((uint64_t)(cnt & 0xffffffu) << 32) | (uint64_t)coll_id;
}

void orc_cqe_decode(uint64_t v, unsigned* blk, unsigned* cnt, unsigned* coll_id) {
  if (blk) *blk = (unsigned)(v >> 56);
  if (cnt) *cnt = (unsigned)((v >> 32) & 0xffffffu);
  if (coll_id) *coll_id = (unsigned)(v & 0xffffffffu);
}

int orc_sq_full(uint64_t head, uint64_t tail, uint64_t length) { return tail + 1 - head == length; }
int orc_sq_empty(uint64_t frontier, uint64_t tail) { return frontier == tail; }
