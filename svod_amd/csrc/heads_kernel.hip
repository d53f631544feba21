// The attention prologue for gfx950: a fused [q | k | v] projection row split
// into sequence-major heads, q and k RMS-normalised over the head and rotated.
//
// Follows heads_body (tk/src/kernels/heads.rs:73-124) op for op, in f32:
//   x1, x2 = the head's halves widened to f32
//   q/k:  inv = rsqrt(sum(x1*x1 + x2*x2) * (1/d) + eps);  y = (x * inv) * w
//   rope: y1' = y1*cos - y2*sin ;  y2' = y1*sin + y2*cos   (halves paired)
//   v:    copied bit for bit
// and rounds to bf16 (nearest even) at the store.
//
// The kernel is HBM-bound (every byte is touched once), so the layout of the
// work is chosen for the memory system: a head slot of d elements is shared by
// d/16 lanes, each lane owning 8 consecutive elements of the first half and the
// 8 elements of the second half they rotate with.  Both are single 128-bit
// accesses, consecutive lanes touch consecutive 16-byte chunks, the rotation
// needs no lane exchange, and the sum of squares needs log2(d/16) exchanges.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace svodk {
namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kThreads = 256;

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Round to nearest even, NaN quieted: the rule of tk/src/interp.rs:37-44.
__device__ __forceinline__ uint32_t to_bf16_bits(float x) {
  uint32_t bits = __float_as_uint(x);
  uint32_t rounded = (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
  return (x != x) ? ((bits | 0x00400000u) >> 16) : rounded;
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return to_bf16_bits(lo) | (to_bf16_bits(hi) << 16);
}

__device__ __forceinline__ void widen(const u32x4 &w, float (&x)[8]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    x[2 * i] = bf16_lo(w[i]);
    x[2 * i + 1] = bf16_hi(w[i]);
  }
}

template <int D>
__global__ __launch_bounds__(kThreads) void heads_kernel(const uint16_t *__restrict__ qkv,
                                                         const uint16_t *__restrict__ q_w,
                                                         const uint16_t *__restrict__ k_w,
                                                         const uint16_t *__restrict__ cos_t,
                                                         const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ q,
                                                         uint16_t *__restrict__ k, uint16_t *__restrict__ v,
                                                         int64_t items, int32_t t, int32_t heads, int32_t kv_heads,
                                                         float eps, int32_t rope) {
#pragma clang fp contract(off)
  constexpr int kHalf = D / 2;
  constexpr int kLanes = D / 16;  // lanes sharing one head slot
  const int32_t slots = heads + 2 * kv_heads;
  const int64_t gid = (int64_t)__builtin_amdgcn_workgroup_id_x() * kThreads + __builtin_amdgcn_workitem_id_x();
  const int64_t item = gid / kLanes;  // (row, slot), slots fastest
  const int32_t part = (int32_t)(gid % kLanes);
  // Lanes of a slot always run together (kLanes divides 64 and the item count
  // is rounded up per wave below), so the exchanges see their partners.
  const bool live = item < items;
  const int64_t row = live ? item / slots : 0;
  const int32_t slot = live ? (int32_t)(item % slots) : 0;

  const uint16_t *src = qkv + (row * slots + slot) * D + part * 8;
  u32x4 w1 = {0, 0, 0, 0}, w2 = {0, 0, 0, 0};
  if (live) {
    w1 = *reinterpret_cast<const u32x4 *>(src);
    w2 = *reinterpret_cast<const u32x4 *>(src + kHalf);
  }

  const bool is_q = slot < heads;
  const bool is_k = !is_q && slot < heads + kv_heads;
  const uint16_t *weight = is_q ? q_w : (is_k ? k_w : nullptr);
  const bool rotate = rope != 0 && (is_q || is_k);

  uint16_t *dst;
  if (is_q)
    dst = q + (row * heads + slot) * D;
  else if (is_k)
    dst = k + (row * kv_heads + (slot - heads)) * D;
  else
    dst = v + (row * kv_heads + (slot - heads - kv_heads)) * D;
  dst += part * 8;

  // Slots are uniform across the lanes of a slot, not across the wave: the
  // exchanges below run for every lane, the arithmetic is selected per lane.
  float y1[8], y2[8];
  widen(w1, y1);
  widen(w2, y2);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; i++) sum += y1[i] * y1[i] + y2[i] * y2[i];
#pragma unroll
  for (int m = 1; m < kLanes; m <<= 1) sum += __shfl_xor(sum, m, 64);

  if (weight != nullptr) {
    const float inv = __builtin_amdgcn_rsqf(sum * (1.0f / (float)D) + eps);
    const u32x4 g1 = *reinterpret_cast<const u32x4 *>(weight + part * 8);
    const u32x4 g2 = *reinterpret_cast<const u32x4 *>(weight + kHalf + part * 8);
    float a1[8], a2[8];
    widen(g1, a1);
    widen(g2, a2);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      y1[i] = (y1[i] * inv) * a1[i];
      y2[i] = (y2[i] * inv) * a2[i];
    }
  }
  if (rotate) {
    const int64_t trow = (rope == 2) ? row : row % t;
    const u32x4 cw = *reinterpret_cast<const u32x4 *>(cos_t + trow * kHalf + part * 8);
    const u32x4 sw = *reinterpret_cast<const u32x4 *>(sin_t + trow * kHalf + part * 8);
    float c[8], s[8];
    widen(cw, c);
    widen(sw, s);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float r1 = y1[i] * c[i] - y2[i] * s[i];
      const float r2 = y1[i] * s[i] + y2[i] * c[i];
      y1[i] = r1;
      y2[i] = r2;
    }
  }
  if (!live) return;
  u32x4 o1, o2;
  if (weight != nullptr || rotate) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      o1[i] = pack_bf16(y1[2 * i], y1[2 * i + 1]);
      o2[i] = pack_bf16(y2[2 * i], y2[2 * i + 1]);
    }
  } else {
    o1 = w1;  // untouched slots (v, or q/k with neither norm nor rope) keep their bits
    o2 = w2;
  }
  *reinterpret_cast<u32x4 *>(dst) = o1;
  *reinterpret_cast<u32x4 *>(dst + kHalf) = o2;
}

template <int D>
hipError_t launch(const HeadsArgs &a, hipStream_t stream) {
  constexpr int kLanes = D / 16;
  const int64_t items = a.rows * (a.heads + 2 * a.kv_heads);
  if (items == 0) return hipSuccess;
  const int64_t threads = items * kLanes;
  const int64_t blocks = (threads + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(heads_kernel<D>, dim3((uint32_t)blocks), dim3(kThreads), 0, stream,
                     (const uint16_t *)a.qkv, (const uint16_t *)a.q_w, (const uint16_t *)a.k_w,
                     (const uint16_t *)a.cos, (const uint16_t *)a.sin, (uint16_t *)a.q, (uint16_t *)a.k,
                     (uint16_t *)a.v, items, a.t, a.heads, a.kv_heads, a.eps, a.rope);
  return hipGetLastError();
}

}  // namespace

bool heads_supports(int32_t d) { return d == 16 || d == 32 || d == 64 || d == 128 || d == 256; }

hipError_t launch_heads(const HeadsArgs &a, hipStream_t stream) {
  switch (a.d) {
    case 16: return launch<16>(a, stream);
    case 32: return launch<32>(a, stream);
    case 64: return launch<64>(a, stream);
    case 128: return launch<128>(a, stream);
    case 256: return launch<256>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace svodk
