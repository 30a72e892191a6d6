// Element arithmetic of the reduce-copy path for gfx950, expressed on 32-bit
// words: one word holds 1 (fp32 / int32), 2 (fp16 / bf16) or 4 (int8) elements,
// and a 128-bit pack is four words.  Semantics follow the reference's
// src/include/reduce_kernel.h: integers wrap mod 2^bits (:66-134), int8 Max/Min
// compare signed bytes (:146-218), fp16 / bf16 are one correctly rounded
// (nearest-even) operation per step in the storage type (:244-440), fp32 Max/Min
// are fmaxf / fminf (:442-455).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dfccl {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Values of ncclDataType_t / ncclRedOp_t that this path implements.
enum : int { kI8 = 0, kI32 = 2, kF16 = 6, kF32 = 7, kBF16 = 9 };
enum : int { kSum = 0, kProd = 1, kMax = 2, kMin = 3 };

__host__ __device__ constexpr int typeSize(int dt) {
  return dt == kI8 ? 1 : (dt == kI32 || dt == kF32) ? 4 : (dt == kF16 || dt == kBF16) ? 2 : 0;
}

template <int OP>
__device__ __forceinline__ float opF32(float a, float b) {
  if constexpr (OP == kSum) return a + b;
  else if constexpr (OP == kProd) return a * b;
  else if constexpr (OP == kMax) return __builtin_fmaxf(a, b);
  else return __builtin_fminf(a, b);
}

template <int DT, int OP>
__device__ __forceinline__ uint32_t wordOp(uint32_t a, uint32_t b) {
  if constexpr (DT == kF32) {
    return __float_as_uint(opF32<OP>(__uint_as_float(a), __uint_as_float(b)));
  } else if constexpr (DT == kI32) {
    if constexpr (OP == kSum) return a + b;
    else if constexpr (OP == kProd) return a * b;
    else if constexpr (OP == kMax) return (uint32_t)(((int32_t)a < (int32_t)b) ? (int32_t)b : (int32_t)a);
    else return (uint32_t)(((int32_t)a < (int32_t)b) ? (int32_t)a : (int32_t)b);
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
  } else {  // int8, four per word
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
    } else {
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
    }
  }
}

template <int DT, int OP>
__device__ __forceinline__ u32x4 packOp(u32x4 a, u32x4 b) {
  u32x4 r;
  r.x = wordOp<DT, OP>(a.x, b.x);
  r.y = wordOp<DT, OP>(a.y, b.y);
  r.z = wordOp<DT, OP>(a.z, b.z);
  r.w = wordOp<DT, OP>(a.w, b.w);
  return r;
}

#ifndef DFCCL_GLOBAL  // (a host build of the kernels for testing defines it empty)
#define DFCCL_GLOBAL __attribute__((address_space(1)))
#endif

// One element held in the low bits of a word (upper bits zero). Operands are in global memory.
template <int ES>
__device__ __forceinline__ uint32_t loadElem(const void* p, size_t i) {
  if constexpr (ES == 1) return ((const DFCCL_GLOBAL uint8_t*)p)[i];
  else if constexpr (ES == 2) return ((const DFCCL_GLOBAL uint16_t*)p)[i];
  else return ((const DFCCL_GLOBAL uint32_t*)p)[i];
}
template <int ES>
__device__ __forceinline__ void storeElem(void* p, size_t i, uint32_t v) {
  if constexpr (ES == 1) ((DFCCL_GLOBAL uint8_t*)p)[i] = (uint8_t)v;
  else if constexpr (ES == 2) ((DFCCL_GLOBAL uint16_t*)p)[i] = (uint16_t)v;
  else ((DFCCL_GLOBAL uint32_t*)p)[i] = v;
}

}  // namespace dfccl
