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

#include "convert.h"
#include "kernels.h"

namespace svodk {
namespace {

constexpr int kThreads = 256;

// Rows and slots come from flat item numbers by division.  The 32-bit form divides with a
// reciprocal from the host (rcp = floor(2^32 / d), 2^32 - 1 for d = 1: the estimate is the
// quotient or one less); the 64-bit form is for tensors past 2^32 lanes.
struct Div32 {
  typedef uint32_t index;
  uint32_t d, rcp;
  __device__ __forceinline__ uint32_t quot(uint32_t n) const {
    const uint32_t q = __umulhi(n, rcp);
    return n - q * d >= d ? q + 1 : q;
  }
};
struct Div64 {
  typedef int64_t index;
  int64_t d;
  uint32_t unused;
  __device__ __forceinline__ int64_t quot(int64_t n) const { return n / d; }
};

// A block owns kItems * kThreads consecutive lanes of the flat (row, slot, part) space, slots
// fastest: thread i takes lanes i, i + kThreads, ...  All loads of a thread are issued before
// any arithmetic.  One item per thread measured fastest on an MI355X (2 and 4 were 5 % and
// 20 % slower: the many small waves keep more of HBM's channels busy than fewer long ones),
// and every byte is touched once, so loads and stores are marked non-temporal.
constexpr int kItems = 1;

// The workgroup's program, for the kernels below to inline.
template <int D, typename Div, bool F16>
__device__ __forceinline__ void heads_body(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ q_w,
                                           const uint16_t *__restrict__ k_w, const uint16_t *__restrict__ cos_t,
                                           const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ q,
                                           uint16_t *__restrict__ k, uint16_t *__restrict__ v, int64_t items,
                                           const Div &by_slots, const Div &by_t, int32_t heads, int32_t kv_heads,
                                           float eps, int32_t rope) {
#pragma clang fp contract(off)
  typedef typename Div::index Index;
  constexpr int kHalf = D / 2;
  constexpr int kLanes = D / 16;  // lanes sharing one head slot
  static_assert(kThreads % kLanes == 0, "a thread keeps its part of the slot across its items");
  const Index slots = (Index)by_slots.d;
  const Index first = (Index)__builtin_amdgcn_workgroup_id_x() * (kThreads * kItems) + __builtin_amdgcn_workitem_id_x();
  const int32_t part = (int32_t)(__builtin_amdgcn_workitem_id_x() % kLanes);

  // Lanes of a slot always run together (kLanes divides 64), so the exchanges see their partners.
  bool live[kItems];
  Index row[kItems];
  int32_t slot[kItems];
  u32x4 w1[kItems], w2[kItems];
#pragma unroll
  for (int u = 0; u < kItems; u++) {
    const Index item = (first + (Index)u * kThreads) / kLanes;  // (row, slot), slots fastest
    live[u] = (int64_t)item < items;
    row[u] = live[u] ? by_slots.quot(item) : 0;
    slot[u] = live[u] ? (int32_t)(item - row[u] * slots) : 0;
    const uint16_t *src = qkv + ((int64_t)row[u] * slots + slot[u]) * D + part * 8;
    w1[u] = w2[u] = u32x4{0, 0, 0, 0};
    if (live[u]) {
      w1[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
      w2[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + kHalf));
    }
  }

#pragma unroll
  for (int u = 0; u < kItems; u++) {
    const bool is_q = slot[u] < heads;
    const bool is_k = !is_q && slot[u] < heads + kv_heads;
    const uint16_t *weight = is_q ? q_w : (is_k ? k_w : nullptr);
    const bool rotate = rope != 0 && (is_q || is_k);

    uint16_t *dst;
    if (is_q)
      dst = q + ((int64_t)row[u] * heads + slot[u]) * D;
    else if (is_k)
      dst = k + ((int64_t)row[u] * kv_heads + (slot[u] - heads)) * D;
    else
      dst = v + ((int64_t)row[u] * kv_heads + (slot[u] - heads - kv_heads)) * D;
    dst += part * 8;

    // Slots are uniform across the lanes of a slot, not across the wave: the
    // exchanges below run for every lane, the arithmetic is selected per lane.
    float y1[8], y2[8];
    widen<F16>(w1[u], y1);
    widen<F16>(w2[u], y2);
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
      widen<F16>(g1, a1);
      widen<F16>(g2, a2);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        y1[i] = (y1[i] * inv) * a1[i];
        y2[i] = (y2[i] * inv) * a2[i];
      }
    }
    if (rotate) {
      const Index trow = (rope == 2) ? row[u] : row[u] - by_t.quot(row[u]) * (Index)by_t.d;
      const u32x4 cw = *reinterpret_cast<const u32x4 *>(cos_t + (int64_t)trow * kHalf + part * 8);
      const u32x4 sw = *reinterpret_cast<const u32x4 *>(sin_t + (int64_t)trow * kHalf + part * 8);
      float c[8], s[8];
      widen<F16>(cw, c);
      widen<F16>(sw, s);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float r1 = y1[i] * c[i] - y2[i] * s[i];
        const float r2 = y1[i] * s[i] + y2[i] * c[i];
        y1[i] = r1;
        y2[i] = r2;
      }
    }
    if (!live[u]) continue;
    u32x4 o1, o2;
    if (weight != nullptr || rotate) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        o1[i] = narrow<F16>(y1[2 * i], y1[2 * i + 1]);
        o2[i] = narrow<F16>(y2[2 * i], y2[2 * i + 1]);
      }
    } else {
      o1 = w1[u];  // untouched slots (v, or q/k with neither norm nor rope) keep their bits
      o2 = w2[u];
    }
    __builtin_nontemporal_store(o1, reinterpret_cast<u32x4 *>(dst));
    __builtin_nontemporal_store(o2, reinterpret_cast<u32x4 *>(dst + kHalf));
  }
}

#if !defined(SVODK_CODE_OBJECT)  // the library's kernel and its launch: not part of a code object build
template <int D, typename Div, bool F16>
__global__ __launch_bounds__(kThreads) void heads_kernel(const uint16_t *__restrict__ qkv,
                                                         const uint16_t *__restrict__ q_w,
                                                         const uint16_t *__restrict__ k_w,
                                                         const uint16_t *__restrict__ cos_t,
                                                         const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ q,
                                                         uint16_t *__restrict__ k, uint16_t *__restrict__ v,
                                                         int64_t items, Div by_slots, Div by_t, int32_t heads,
                                                         int32_t kv_heads, float eps, int32_t rope) {
  heads_body<D, Div, F16>(qkv, q_w, k_w, cos_t, sin_t, q, k, v, items, by_slots, by_t, heads, kv_heads, eps, rope);
}

template <int D, bool F16>
hipError_t launch(const HeadsArgs &a, hipStream_t stream) {
  constexpr int kLanes = D / 16;
  const int64_t slots = a.heads + 2 * a.kv_heads;
  const int64_t items = a.rows * slots;
  if (items == 0) return hipSuccess;
  const int64_t threads = items * kLanes;
  const int64_t per_block = (int64_t)kThreads * kItems;
  const int64_t blocks = (threads + per_block - 1) / per_block;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  const int64_t t = a.t > 0 ? a.t : 1;
  if (blocks * per_block < 0xffffffffLL) {
    auto rcp = [](uint32_t d) { return d == 1 ? 0xffffffffu : (uint32_t)((1ull << 32) / d); };
    const Div32 by_slots = {(uint32_t)slots, rcp((uint32_t)slots)}, by_t = {(uint32_t)t, rcp((uint32_t)t)};
    hipLaunchKernelGGL((heads_kernel<D, Div32, F16>), dim3((uint32_t)blocks), dim3(kThreads), 0, stream,
                       (const uint16_t *)a.qkv, (const uint16_t *)a.q_w, (const uint16_t *)a.k_w,
                       (const uint16_t *)a.cos, (const uint16_t *)a.sin, (uint16_t *)a.q, (uint16_t *)a.k,
                       (uint16_t *)a.v, items, by_slots, by_t, a.heads, a.kv_heads, a.eps, a.rope);
  } else {
    const Div64 by_slots = {slots, 0}, by_t = {t, 0};
    hipLaunchKernelGGL((heads_kernel<D, Div64, F16>), dim3((uint32_t)blocks), dim3(kThreads), 0, stream,
                       (const uint16_t *)a.qkv, (const uint16_t *)a.q_w, (const uint16_t *)a.k_w,
                       (const uint16_t *)a.cos, (const uint16_t *)a.sin, (uint16_t *)a.q, (uint16_t *)a.k,
                       (uint16_t *)a.v, items, by_slots, by_t, a.heads, a.kv_heads, a.eps, a.rope);
  }
  return hipGetLastError();
}

}  // namespace

bool heads_supports(int32_t d) { return d == 16 || d == 32 || d == 64 || d == 128 || d == 256; }

template <bool F16>
static hipError_t launch_any(const HeadsArgs &a, hipStream_t stream) {
  switch (a.d) {
    case 16: return launch<16, F16>(a, stream);
    case 32: return launch<32, F16>(a, stream);
    case 64: return launch<64, F16>(a, stream);
    case 128: return launch<128, F16>(a, stream);
    case 256: return launch<256, F16>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_heads(const HeadsArgs &a, hipStream_t stream) {
  return a.f16 ? launch_any<true>(a, stream) : launch_any<false>(a, stream);
}

}  // namespace svodk

#else  // SVODK_CODE_OBJECT
// The prologue as kernels for a loader that takes a code object and a flat argument record
// (device/src/amd/program.rs:403-414, 655-675; device/src/hcq.rs:1262-1285): buffers first, then
// 4-byte scalars, nothing hidden, no launch geometry from the dispatch packet.
// Parameters: qkv, q_w, k_w (address 0: that norm is off), cos, sin (unread when rope is 0), q, k, v,
// then rows (batch * t), t, heads, kv_heads, eps_bits, rope (0 none, 1 a [t, D/2] table shared by
// the batch, 2 a [rows, D/2] table).  Launch: ceil(rows * (heads + 2 kv_heads) * (D / 16) / 256)
// workgroups of 256 threads; rows * (heads + 2 kv_heads) * (D / 16) < 2^32 - 256 is the caller's check.
template <int D, bool F16>
__device__ __forceinline__ void heads_entry(const uint16_t *qkv, const uint16_t *q_w, const uint16_t *k_w,
                                            const uint16_t *cos_t, const uint16_t *sin_t, uint16_t *q, uint16_t *k,
                                            uint16_t *v, int32_t rows, int32_t t, int32_t heads, int32_t kv_heads,
                                            int32_t eps_bits, int32_t rope) {
  if (rows <= 0 || heads < 0 || kv_heads < 0 || heads + 2 * kv_heads <= 0) return;
  auto rcp = [](uint32_t d) { return d <= 1 ? 0xffffffffu : 0xffffffffu / d; };  // within one of floor(2^32 / d)
  const uint32_t slots = (uint32_t)(heads + 2 * kv_heads), tt = (uint32_t)(t > 0 ? t : 1);
  const Div32 by_slots = {slots, rcp(slots)}, by_t = {tt, rcp(tt)};
  heads_body<D, Div32, F16>(qkv, q_w, k_w, cos_t, sin_t, q, k, v, (int64_t)rows * slots, by_slots, by_t, heads, kv_heads,
                            __builtin_bit_cast(float, eps_bits), rope);
}

#define SVODK_HEADS_ENTRY(NAME, D, F16)                                                                              \
  extern "C" __global__ __launch_bounds__(kThreads) void NAME(                                                        \
      const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ q_w, const uint16_t *__restrict__ k_w,           \
      const uint16_t *__restrict__ cos_t, const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ q,               \
      uint16_t *__restrict__ k, uint16_t *__restrict__ v, int32_t rows, int32_t t, int32_t heads, int32_t kv_heads,   \
      int32_t eps_bits, int32_t rope) {                                                                               \
    heads_entry<D, F16>(qkv, q_w, k_w, cos_t, sin_t, q, k, v, rows, t, heads, kv_heads, eps_bits, rope);              \
  }

SVODK_HEADS_ENTRY(svodk_heads_d16_bf16, 16, false)
SVODK_HEADS_ENTRY(svodk_heads_d32_bf16, 32, false)
SVODK_HEADS_ENTRY(svodk_heads_d64_bf16, 64, false)
SVODK_HEADS_ENTRY(svodk_heads_d128_bf16, 128, false)
SVODK_HEADS_ENTRY(svodk_heads_d256_bf16, 256, false)
SVODK_HEADS_ENTRY(svodk_heads_d16_f16, 16, true)
SVODK_HEADS_ENTRY(svodk_heads_d32_f16, 32, true)
SVODK_HEADS_ENTRY(svodk_heads_d64_f16, 64, true)
SVODK_HEADS_ENTRY(svodk_heads_d128_f16, 128, true)
SVODK_HEADS_ENTRY(svodk_heads_d256_f16, 256, true)
#undef SVODK_HEADS_ENTRY

}  // namespace
}  // namespace svodk
#endif  // SVODK_CODE_OBJECT
