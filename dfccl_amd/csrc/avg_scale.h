// Host side: what ncclAvg becomes for a group of n ranks, following hostToDevRedOp of the reference
// (src/enqueue.cc:1326-1357): integer types sum and divide the result by n afterwards (SumPostDiv, scalar n);
// float types multiply every input by 1/n first (PreMulSum), the scalar being float(1.0 / n) converted to the
// element type with round-to-nearest-even (1.0 / n itself for fp64).
#pragma once

#include <stdint.h>
#include <string.h>

#include "reduce_ops.h"

namespace dfccl {

inline uint16_t hostF32ToBf16Bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);  // nearest, ties to even (1/n is never NaN or infinite)
  return (uint16_t)(u >> 16);
}
inline uint16_t hostF32ToF16Bits(float f) {
  const _Float16 h = (_Float16)f;  // the compiler's conversion rounds to nearest even
  uint16_t b;
  memcpy(&b, &h, 2);
  return b;
}

inline Scale dfcclAvgScale(int dtype, int n) {
  Scale s;
  s.kind = kScaleNone;
  s.bits = 0;
  if (n <= 1) return s;  // the average of one rank's value is the value
  if (!isFloatType(dtype)) {
    s.kind = kScalePost;
    s.bits = (uint64_t)n;
    return s;
  }
  s.kind = kScalePre;
  if (dtype == kF64) {
    const double d = 1.0 / n;
    memcpy(&s.bits, &d, 8);
  } else {
    const float f = (float)(1.0 / n);
    if (dtype == kF32) {
      uint32_t u;
      memcpy(&u, &f, 4);
      s.bits = u;
    } else if (dtype == kF16) {
      s.bits = hostF32ToF16Bits(f);
    } else {
      s.bits = hostF32ToBf16Bits(f);
    }
  }
  return s;
}

}  // namespace dfccl
