// Widening and narrowing between the operands' 16-bit float types and f32, shared by the
// row-wise kernels (the attention prologue and the row norms).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace svodk {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

// Eight 16-bit values of the operands' type, widened exactly.
template <bool F16>
__device__ __forceinline__ void widen(const u32x4 &w, float (&x)[8]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if constexpr (F16) {
      const uint32_t pair = w[i];  // a copy: the cast below wants an object of its own, not a vector's element
      const f32x2 f = __builtin_convertvector(__builtin_bit_cast(f16x2, pair), f32x2);
      x[2 * i] = f[0];
      x[2 * i + 1] = f[1];
    } else {
      x[2 * i] = bf16_lo(w[i]);
      x[2 * i + 1] = bf16_hi(w[i]);
    }
  }
}

// Two f32 values rounded to the operands' type, nearest even, a NaN quieted with its upper payload kept
// (tk/src/interp.rs:37-50).  The bf16 arm is the hardware's packed conversion: over all 2^32 inputs it gives the
// bits of the reference's rule, (bits + 0x7fff + ((bits >> 16) & 1)) >> 16 and (bits | 0x00400000) >> 16 for a NaN,
// in one instruction for two values where that rule takes a dozen.
template <bool F16>
__device__ __forceinline__ uint32_t narrow(float lo, float hi) {
  if constexpr (F16) {
    const f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  } else {
    const f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
  }
}

}  // namespace svodk
