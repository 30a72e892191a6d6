// Element arithmetic of the reduce-copy path for gfx950, expressed on 32-bit
// words: one word holds 1 (fp32 / int32 / uint32), 2 (fp16 / bf16) or 4 (int8 /
// uint8) elements, two words hold one 64-bit element (int64 / uint64 / fp64), and
// a 128-bit pack is four words.  Semantics follow the reference's
// src/include/reduce_kernel.h: integers wrap mod 2^bits (:23-36,66-134), Max / Min
// compare in the element's signedness (:39-53,146-218), fp16 / bf16 are one
// correctly rounded (nearest-even) operation per step in the storage type
// (:244-440), fp32 / fp64 Max/Min are fmaxf / fminf / fmax / fmin (:442-469).
// Scaled sums (:485-704): PreMulSum multiplies an input by a scalar as it enters
// the reduction, SumPostDiv divides the finished integer sum by the group size.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dfccl {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Values of ncclDataType_t, and the four element ops of ncclRedOp_t (ncclAvg is a Sum with a scale, see Scale).
enum : int { kI8 = 0, kU8 = 1, kI32 = 2, kU32 = 3, kI64 = 4, kU64 = 5, kF16 = 6, kF32 = 7, kF64 = 8, kBF16 = 9 };
enum : int { kSum = 0, kProd = 1, kMax = 2, kMin = 3 };

__host__ __device__ constexpr int typeSize(int dt) {
  return (dt == kI8 || dt == kU8) ? 1
         : (dt == kI32 || dt == kU32 || dt == kF32) ? 4
         : (dt == kF16 || dt == kBF16) ? 2
         : (dt == kI64 || dt == kU64 || dt == kF64) ? 8 : 0;
}
__host__ __device__ constexpr bool isFloatType(int dt) { return dt == kF16 || dt == kBF16 || dt == kF32 || dt == kF64; }

template <int OP>
__device__ __forceinline__ float opF32(float a, float b) {
  if constexpr (OP == kSum) return a + b;
  else if constexpr (OP == kProd) return a * b;
  else if constexpr (OP == kMax) return __builtin_fmaxf(a, b);
  else return __builtin_fminf(a, b);
}

// One op on a 32-bit word of elements (types of at most 4 bytes).
template <int DT, int OP>
__device__ __forceinline__ uint32_t wordOp(uint32_t a, uint32_t b) {
  static_assert(typeSize(DT) <= 4, "64-bit elements go through dwordOp");
  if constexpr (DT == kF32) {
    return __float_as_uint(opF32<OP>(__uint_as_float(a), __uint_as_float(b)));
  } else if constexpr (DT == kI32 || DT == kU32) {
    if constexpr (OP == kSum) return a + b;
    else if constexpr (OP == kProd) return a * b;
    else if constexpr (DT == kI32 && OP == kMax) return (uint32_t)(((int32_t)a < (int32_t)b) ? (int32_t)b : (int32_t)a);
    else if constexpr (DT == kI32) return (uint32_t)(((int32_t)a < (int32_t)b) ? (int32_t)a : (int32_t)b);
    else if constexpr (OP == kMax) return (a < b) ? b : a;
    else return (a < b) ? a : b;
  } else if constexpr (DT == kF16) {
    f16x2 x = __builtin_bit_cast(f16x2, a), y = __builtin_bit_cast(f16x2, b), r;
    if constexpr (OP == kSum) r = x + y;
    else if constexpr (OP == kProd) r = x * y;
    else if constexpr (OP == kMax) r = __builtin_elementwise_max(x, y);
    else r = __builtin_elementwise_min(x, y);
    return __builtin_bit_cast(uint32_t, r);
  } else if constexpr (DT == kBF16) {
    // widen (exact), operate in fp32, round both results to bfloat16 (nearest even) with one v_cvt_pk_bf16_f32
    float alo = __uint_as_float(a << 16), ahi = __uint_as_float(a & 0xffff0000u);
    float blo = __uint_as_float(b << 16), bhi = __uint_as_float(b & 0xffff0000u);
    f32x2 r;
    r.x = opF32<OP>(alo, blo);
    r.y = opF32<OP>(ahi, bhi);
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(r, bf16x2));
  } else {  // int8 / uint8, four per word
    if constexpr (OP == kSum) {
      // add even and odd bytes separately so that carries cannot cross a byte
      uint32_t r0 = (a & 0x00ff00ffu) + (b & 0x00ff00ffu);
      uint32_t r1 = (a & 0xff00ff00u) + (b & 0xff00ff00u);
      return (r0 & 0x00ff00ffu) | (r1 & 0xff00ff00u);
    } else if constexpr (OP == kProd) {
      uint32_t r = 0;
#pragma unroll
      for (int k = 0; k < 4; k++) r |= ((((a >> (8 * k)) & 0xffu) * ((b >> (8 * k)) & 0xffu)) & 0xffu) << (8 * k);
      return r;
    } else if constexpr (DT == kI8) {
      // signed compare per byte: move each byte to the top of a 16-bit lane,
      // where a signed 16-bit compare orders exactly as the signed byte does
      i16x2 ahi = __builtin_bit_cast(i16x2, a & 0xff00ff00u), bhi = __builtin_bit_cast(i16x2, b & 0xff00ff00u);
      i16x2 alo = __builtin_bit_cast(i16x2, (a << 8) & 0xff00ff00u), blo = __builtin_bit_cast(i16x2, (b << 8) & 0xff00ff00u);
      i16x2 rhi, rlo;
      if constexpr (OP == kMax) {
        rhi = __builtin_elementwise_max(ahi, bhi);
        rlo = __builtin_elementwise_max(alo, blo);
      } else {
        rhi = __builtin_elementwise_min(ahi, bhi);
        rlo = __builtin_elementwise_min(alo, blo);
      }
      return (__builtin_bit_cast(uint32_t, rhi) & 0xff00ff00u) | ((__builtin_bit_cast(uint32_t, rlo) >> 8) & 0x00ff00ffu);
    } else {
      // unsigned compare per byte: even and odd bytes as the low bytes of 16-bit lanes
      u16x2 ae = __builtin_bit_cast(u16x2, a & 0x00ff00ffu), be = __builtin_bit_cast(u16x2, b & 0x00ff00ffu);
      u16x2 ao = __builtin_bit_cast(u16x2, (a >> 8) & 0x00ff00ffu), bo = __builtin_bit_cast(u16x2, (b >> 8) & 0x00ff00ffu);
      u16x2 re, ro;
      if constexpr (OP == kMax) {
        re = __builtin_elementwise_max(ae, be);
        ro = __builtin_elementwise_max(ao, bo);
      } else {
        re = __builtin_elementwise_min(ae, be);
        ro = __builtin_elementwise_min(ao, bo);
      }
      return __builtin_bit_cast(uint32_t, re) | (__builtin_bit_cast(uint32_t, ro) << 8);
    }
  }
}

// One op on a 64-bit element.
template <int DT, int OP>
__device__ __forceinline__ uint64_t dwordOp(uint64_t a, uint64_t b) {
  static_assert(typeSize(DT) == 8, "64-bit elements only");
  if constexpr (DT == kF64) {
    const double x = __builtin_bit_cast(double, a), y = __builtin_bit_cast(double, b);
    double r;
    if constexpr (OP == kSum) r = x + y;
    else if constexpr (OP == kProd) r = x * y;
    else if constexpr (OP == kMax) r = __builtin_fmax(x, y);
    else r = __builtin_fmin(x, y);
    return __builtin_bit_cast(uint64_t, r);
  } else {
    if constexpr (OP == kSum) return a + b;
    else if constexpr (OP == kProd) return a * b;
    else if constexpr (DT == kI64 && OP == kMax) return (uint64_t)(((int64_t)a < (int64_t)b) ? (int64_t)b : (int64_t)a);
    else if constexpr (DT == kI64) return (uint64_t)(((int64_t)a < (int64_t)b) ? (int64_t)a : (int64_t)b);
    else if constexpr (OP == kMax) return (a < b) ? b : a;
    else return (a < b) ? a : b;
  }
}

template <int DT, int OP>
__device__ __forceinline__ u32x4 packOp(u32x4 a, u32x4 b) {
  u32x4 r;
  if constexpr (typeSize(DT) == 8) {
    const uint64_t lo = dwordOp<DT, OP>((uint64_t)a.x | ((uint64_t)a.y << 32), (uint64_t)b.x | ((uint64_t)b.y << 32));
    const uint64_t hi = dwordOp<DT, OP>((uint64_t)a.z | ((uint64_t)a.w << 32), (uint64_t)b.z | ((uint64_t)b.w << 32));
    r.x = (uint32_t)lo;
    r.y = (uint32_t)(lo >> 32);
    r.z = (uint32_t)hi;
    r.w = (uint32_t)(hi >> 32);
  } else {
    r.x = wordOp<DT, OP>(a.x, b.x);
    r.y = wordOp<DT, OP>(a.y, b.y);
    r.z = wordOp<DT, OP>(a.z, b.z);
    r.w = wordOp<DT, OP>(a.w, b.w);
  }
  return r;
}

// ---- scaled sums --------------------------------------------------------------------------------------------
// What ncclAvg (and a PreMulSum op) adds to a Sum: `kind` kScalePre multiplies every user input by the scalar
// in `bits` (one element of the type, in the low bytes) as it enters the reduction, one rounded multiply in
// the element type, i.e. exactly the Prod op with a constant; kScalePost divides the finished sum of an integer
// type by (int)bits, T(x / n) with C++'s truncating division after the usual conversions
// (src/include/reduce_kernel.h:491-520; src/enqueue.cc:1326-1357 for what ncclAvg becomes per type).
enum : int { kScaleNone = 0, kScalePre = 1, kScalePost = 2 };
struct Scale {
  int kind;
  uint64_t bits;
};

// the scalar repeated over a pack, so that the pre-multiplication is packOp<DT, kProd> with it
template <int DT>
__device__ __forceinline__ u32x4 splatScalar(uint64_t bits) {
  u32x4 r;
  if constexpr (typeSize(DT) == 8) {
    r.x = r.z = (uint32_t)bits;
    r.y = r.w = (uint32_t)(bits >> 32);
  } else {
    uint32_t w = (uint32_t)bits;
    if constexpr (typeSize(DT) == 2) w = (w & 0xffffu) | (w << 16);
    if constexpr (typeSize(DT) == 1) w = (w & 0xffu) * 0x01010101u;
    r.x = r.y = r.z = r.w = w;
  }
  return r;
}

// T(x / n) on every element of a word / a 64-bit element (integer types only; n > 0)
template <int DT>
__device__ __forceinline__ uint32_t wordPostDiv(uint32_t a, int n) {
  if constexpr (DT == kI32) return (uint32_t)((int32_t)a / n);
  else if constexpr (DT == kU32) return a / (uint32_t)n;
  else if constexpr (DT == kI8) {
    uint32_t r = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) r |= ((uint32_t)((int32_t)(int8_t)(a >> (8 * k)) / n) & 0xffu) << (8 * k);
    return r;
  } else if constexpr (DT == kU8) {
    uint32_t r = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) r |= ((uint32_t)((int32_t)((a >> (8 * k)) & 0xffu) / n) & 0xffu) << (8 * k);
    return r;
  } else {
    return a;  // float types have no post-division (their average is a pre-multiplication)
  }
}
template <int DT>
__device__ __forceinline__ uint64_t dwordPostDiv(uint64_t a, int n) {
  if constexpr (DT == kI64) return (uint64_t)((int64_t)a / (int64_t)n);
  else if constexpr (DT == kU64) return a / (uint64_t)(int64_t)n;
  else return a;
}
template <int DT>
__device__ __forceinline__ u32x4 packPostDiv(u32x4 a, int n) {
  u32x4 r;
  if constexpr (typeSize(DT) == 8) {
    const uint64_t lo = dwordPostDiv<DT>((uint64_t)a.x | ((uint64_t)a.y << 32), n);
    const uint64_t hi = dwordPostDiv<DT>((uint64_t)a.z | ((uint64_t)a.w << 32), n);
    r.x = (uint32_t)lo;
    r.y = (uint32_t)(lo >> 32);
    r.z = (uint32_t)hi;
    r.w = (uint32_t)(hi >> 32);
  } else {
    r.x = wordPostDiv<DT>(a.x, n);
    r.y = wordPostDiv<DT>(a.y, n);
    r.z = wordPostDiv<DT>(a.z, n);
    r.w = wordPostDiv<DT>(a.w, n);
  }
  return r;
}

#ifndef DFCCL_GLOBAL  // (a host build of the kernels for testing defines it empty)
#define DFCCL_GLOBAL __attribute__((address_space(1)))
#endif

// One element held in the low bits of a 64-bit value (upper bits zero). Operands are in global memory.
template <int ES>
__device__ __forceinline__ uint64_t loadElem(const void* p, size_t i) {
  if constexpr (ES == 1) return ((const DFCCL_GLOBAL uint8_t*)p)[i];
  else if constexpr (ES == 2) return ((const DFCCL_GLOBAL uint16_t*)p)[i];
  else if constexpr (ES == 4) return ((const DFCCL_GLOBAL uint32_t*)p)[i];
  else return ((const DFCCL_GLOBAL uint64_t*)p)[i];
}
template <int ES>
__device__ __forceinline__ void storeElem(void* p, size_t i, uint64_t v) {
  if constexpr (ES == 1) ((DFCCL_GLOBAL uint8_t*)p)[i] = (uint8_t)v;
  else if constexpr (ES == 2) ((DFCCL_GLOBAL uint16_t*)p)[i] = (uint16_t)v;
  else if constexpr (ES == 4) ((DFCCL_GLOBAL uint32_t*)p)[i] = (uint32_t)v;
  else ((DFCCL_GLOBAL uint64_t*)p)[i] = v;
}
// the same ops on single elements (the tails of ragged or misaligned buffers)
template <int DT, int OP>
__device__ __forceinline__ uint64_t elemOp(uint64_t a, uint64_t b) {
  if constexpr (typeSize(DT) == 8) return dwordOp<DT, OP>(a, b);
  else return wordOp<DT, OP>((uint32_t)a, (uint32_t)b);
}
template <int DT>
__device__ __forceinline__ uint64_t elemPreMul(uint64_t a, uint64_t bits) {
  if constexpr (typeSize(DT) == 8) return dwordOp<DT, kProd>(a, bits);
  else return wordOp<DT, kProd>((uint32_t)a, (uint32_t)bits);
}
template <int DT>
__device__ __forceinline__ uint64_t elemPostDiv(uint64_t a, int n) {
  if constexpr (typeSize(DT) == 8) return dwordPostDiv<DT>(a, n);
  else return wordPostDiv<DT>((uint32_t)a, n);
}

}  // namespace dfccl
