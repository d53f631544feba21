// Row norms for gfx950: LayerNorm and RMSNorm over the last dim, optionally after a residual
// add whose rounded sum is also written out.
//
// Follows norm_body (tk/src/kernels/rows.rs:52-114) op for op, in f32:
//   xs = x widened                       (with a residual: s = T(x + r) stored as `sum`, xs = s widened)
//   Layer: mean = sum(xs) * (1/d);  c = xs - mean        Rms: c = xs
//   var = sum(c * c) * (1/d) + eps;  inv = rsqrt(var);  y = (c * inv) * w  (+ b for a LayerNorm)
// and rounds to the operands' type at the store.
//
// A wave works on a row at a time, as in the reference ("one warp per row"), the row held in registers
// between the passes: a lane owns 8 consecutive elements of every 512-element span (one 128-bit access,
// consecutive lanes consecutive chunks), d / 64 elements in all.  A row is read once and written
// once, so the kernel is priced against HBM bandwidth; the row sums are in-lane adds followed
// by a butterfly over the wave (DPP and the permlane swaps: no trip through LDS), the same order for
// every row.  The library's launch holds as many workgroups as the device takes at once and every wave
// walks its share of the rows, the next row's loads in flight under the current row's arithmetic.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>

#include "convert.h"
#include "kernels.h"

namespace svodk {
namespace {

constexpr int kRowsPerBlock = 4;  // NormCfg { br: 4 }: four waves, a row each
constexpr int kSpan = 512;        // elements one wave-wide 128-bit access covers

// x of the lane a DPP control names.
template <int CTRL>
__device__ __forceinline__ float moved(float x) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), CTRL, 0xf, 0xf, true));
}
// The sum over the wave, in every lane, without a trip through LDS: neighbours, pairs of neighbours, the halves of a
// row of 16 lanes mirrored, the row mirrored (all DPP), then the rows 16 and 32 lanes apart (the permlane swaps).
// The same order for every row.
__device__ __forceinline__ float wave_sum(float x) {
  x += moved<0xB1>(x);   // quad_perm [1,0,3,2]
  x += moved<0x4E>(x);   // quad_perm [2,3,0,1]
  x += moved<0x141>(x);  // row_half_mirror
  x += moved<0x140>(x);  // row_mirror
  const uint32_t u = __float_as_uint(x);
  const auto r16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);
  const uint32_t v = __float_as_uint(x);
  const auto r32 = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return __uint_as_float(r32[0]) + __uint_as_float(r32[1]);
}

__device__ __forceinline__ u32x4 load_once(const u32x4 *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_once(u32x4 *p, const u32x4 &v) { __builtin_nontemporal_store(v, p); }

// SPANS = ceil(d / 512): the 128-bit accesses a lane makes per row and tensor.
// The workgroup's program, for the kernels below to inline: a wave takes rows `first`, `first + stride`, ...; a row's
// loads are in flight while the row before it is normalised and stored, and the weight (and bias) are read once a
// wave, not once a row.  (A wave a row, the reference's form, leaves a wave's start and end, and the weight's 2 d
// bytes from L2, on every row's bill: 25.5 us against 23.3 for a [16384, 2048] RMSNorm.)
template <int SPANS, bool LAYER, bool RESIDUAL, bool BIAS, bool F16>
__device__ __forceinline__ void rows_body(const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual,
                                          const uint16_t *__restrict__ w, const uint16_t *__restrict__ b,
                                          uint16_t *__restrict__ out, uint16_t *__restrict__ sum, int64_t rows, int32_t d,
                                          float inv_d, float eps, int64_t first, int64_t stride) {
  const int lane = threadIdx.x & 63;
  if (first >= rows) return;
  bool live[SPANS];
  u32x4 wp[SPANS], bp[SPANS];
#pragma unroll
  for (int s = 0; s < SPANS; s++) {
    const int at = s * kSpan + lane * 8;
    live[s] = at < d;  // d is a multiple of 256: a row's last span is whole or half
    wp[s] = bp[s] = u32x4{0, 0, 0, 0};
    if (live[s]) {
      wp[s] = *reinterpret_cast<const u32x4 *>(w + at);
      if (LAYER && BIAS) bp[s] = *reinterpret_cast<const u32x4 *>(b + at);
    }
  }
  // A row's x (and residual) as they lie in memory.
  struct Raw {
    u32x4 x[SPANS], r[SPANS];
  };
  auto ask = [&](Raw &raw, int64_t row) {
    const int64_t base = row * d;
#pragma unroll
    for (int s = 0; s < SPANS; s++) {
      const int at = s * kSpan + lane * 8;
      raw.x[s] = raw.r[s] = u32x4{0, 0, 0, 0};
      if (live[s] && row < rows) {
        raw.x[s] = load_once(reinterpret_cast<const u32x4 *>(x + base + at));
        if (RESIDUAL) raw.r[s] = load_once(reinterpret_cast<const u32x4 *>(residual + base + at));
      }
    }
  };
  auto finish = [&](const Raw &raw, int64_t row) {
    const int64_t base = row * d;
    float xs[SPANS][8];
#pragma unroll
    for (int s = 0; s < SPANS; s++) {
      const int at = s * kSpan + lane * 8;
      widen<F16>(raw.x[s], xs[s]);
      if (RESIDUAL && live[s]) {
        float rs[8];
        widen<F16>(raw.r[s], rs);
        // L77-86: the sum is rounded to the operands' type, stored, and read back as f32.
        u32x4 packed;
#pragma unroll
        for (int i = 0; i < 4; i++) packed[i] = narrow<F16>(xs[s][2 * i] + rs[2 * i], xs[s][2 * i + 1] + rs[2 * i + 1]);
        store_once(reinterpret_cast<u32x4 *>(sum + base + at), packed);
        widen<F16>(packed, xs[s]);
      }
    }
    float mean = 0.0f;
    if (LAYER) {
      float acc = 0.0f;
#pragma unroll
      for (int s = 0; s < SPANS; s++) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc += xs[s][i];
      }
      mean = wave_sum(acc) * inv_d;  // L88-91
    }
    float acc = 0.0f;
#pragma unroll
    for (int s = 0; s < SPANS; s++) {
#pragma unroll
      for (int i = 0; i < 8; i++) {
        // A lane past the row's end holds zeros, which must not be centred into -mean.
        const float c = live[s] ? xs[s][i] - mean : 0.0f;
        xs[s][i] = c;
        acc += c * c;
      }
    }
    const float var = wave_sum(acc) * inv_d + eps;
    const float inv = __builtin_amdgcn_rsqf(var);  // v_rsq_f32, as in the attention prologue
#pragma unroll
    for (int s = 0; s < SPANS; s++) {
      const int at = s * kSpan + lane * 8;
      if (!live[s]) continue;
      float ws[8], bs[8];
      widen<F16>(wp[s], ws);
      if (LAYER && BIAS) widen<F16>(bp[s], bs);
      u32x4 packed;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float y0 = (xs[s][2 * i] * inv) * ws[2 * i], y1 = (xs[s][2 * i + 1] * inv) * ws[2 * i + 1];
        if (LAYER && BIAS) {
          y0 += bs[2 * i];
          y1 += bs[2 * i + 1];
        }
        packed[i] = narrow<F16>(y0, y1);
      }
      store_once(reinterpret_cast<u32x4 *>(out + base + at), packed);
    }
  };
  // Two sets of registers take turns: one row is worked on while the next is on its way.
  Raw one, two;
  ask(one, first);
  for (int64_t row = first; row < rows; row += 2 * stride) {
    ask(two, row + stride);
    finish(one, row);
    if (row + stride >= rows) break;
    ask(one, row + 2 * stride);
    finish(two, row + stride);
  }
}

#if !defined(SVODK_CODE_OBJECT)  // the library's kernel and its launch: not part of a code object build
template <int SPANS, bool LAYER, bool RESIDUAL, bool BIAS, bool F16>
__global__ __launch_bounds__(kRowsPerBlock * 64) void rows_kernel(const uint16_t *__restrict__ x,
                                                                   const uint16_t *__restrict__ residual,
                                                                   const uint16_t *__restrict__ w,
                                                                   const uint16_t *__restrict__ b,
                                                                   uint16_t *__restrict__ out, uint16_t *__restrict__ sum,
                                                                   int64_t rows, int32_t d, float inv_d, float eps) {
  rows_body<SPANS, LAYER, RESIDUAL, BIAS, F16>(x, residual, w, b, out, sum, rows, d, inv_d, eps,
                                               (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6),
                                               (int64_t)gridDim.x * kRowsPerBlock);
}

template <int SPANS, bool LAYER, bool RESIDUAL, bool BIAS, bool F16>
hipError_t launch_rows(const NormArgs &a, hipStream_t stream) {
  // The same number of workgroups on every compute unit, at most what this instantiation's registers let a unit
  // hold (asked of the runtime once a device), every wave walking its share of the rows.  The units share the
  // memory's bandwidth, so a launch costs about (rows a wave) x (workgroups a unit, or the count that keeps the
  // memory busy if that is more): the count that makes that least, the larger on a tie (more rows in flight).  A unit with a workgroup more than its neighbours, or a wave
  // with a row more, is what the launch then waits for (683 workgroups for 16384 rows: 50.5 us; 512: 46.5).
  static std::atomic<int> geometry[64];  // (workgroups a unit) << 16 | units
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  int known = device >= 0 && device < 64 ? geometry[device].load(std::memory_order_acquire) : 0;
  if (known == 0) {
    int per_unit = 0, units = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, rows_kernel<SPANS, LAYER, RESIDUAL, BIAS, F16>,
                                                     kRowsPerBlock * 64, 0);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
    if (e != hipSuccess) return e;
    known = std::min(std::max(1, per_unit), 255) << 16 | std::min(std::max(1, units), 0xffff);
    if (device >= 0 && device < 64) geometry[device].store(known, std::memory_order_release);
  }
  const int64_t per_unit = known >> 16, units = known & 0xffff;
  const int64_t all = (a.rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (all == 0) return hipSuccess;
  int64_t blocks = all;
  if (all > units) {
    // Below about 64 KiB of loads in flight a unit the memory system is not kept busy and a row takes as long
    // whatever the count: fewer workgroups than that buy nothing (a wave asks for a row ahead: a KiB a span and tensor).
    constexpr int64_t kInFlight = 64 * 1024, kOfAWorkgroup = kRowsPerBlock * SPANS * (RESIDUAL ? 2 : 1) * 1024;
    const int64_t enough = std::min(per_unit, (kInFlight + kOfAWorkgroup - 1) / kOfAWorkgroup);
    int64_t best = 0;
    for (int64_t m = per_unit; m >= 1; m--) {
      const int64_t cost = (all + units * m - 1) / (units * m) * std::max(m, enough);
      if (best == 0 || cost < best) best = cost, blocks = units * m;
    }
  }
  hipLaunchKernelGGL((rows_kernel<SPANS, LAYER, RESIDUAL, BIAS, F16>), dim3((uint32_t)blocks), dim3(kRowsPerBlock * 64), 0,
                     stream, (const uint16_t *)a.x, (const uint16_t *)a.residual, (const uint16_t *)a.w,
                     (const uint16_t *)a.b, (uint16_t *)a.out, (uint16_t *)a.sum, a.rows, a.d,
                     (float)(1.0 / (double)a.d), (float)a.eps);
  return hipGetLastError();
}

template <int SPANS, bool F16>
hipError_t launch_kind(const NormArgs &a, hipStream_t stream) {
  const bool res = a.residual != nullptr, bias = a.b != nullptr;
  if (a.layer) {
    if (res) return bias ? launch_rows<SPANS, true, true, true, F16>(a, stream) : launch_rows<SPANS, true, true, false, F16>(a, stream);
    return bias ? launch_rows<SPANS, true, false, true, F16>(a, stream) : launch_rows<SPANS, true, false, false, F16>(a, stream);
  }
  return res ? launch_rows<SPANS, false, true, false, F16>(a, stream) : launch_rows<SPANS, false, false, false, F16>(a, stream);
}

template <bool F16>
hipError_t launch_spans(const NormArgs &a, hipStream_t stream) {
  switch ((a.d + kSpan - 1) / kSpan) {
    case 1: return launch_kind<1, F16>(a, stream);
    case 2: return launch_kind<2, F16>(a, stream);
    case 3: return launch_kind<3, F16>(a, stream);
    case 4: return launch_kind<4, F16>(a, stream);
    case 5: return launch_kind<5, F16>(a, stream);
    case 6: return launch_kind<6, F16>(a, stream);
    case 7: return launch_kind<7, F16>(a, stream);
    case 8: return launch_kind<8, F16>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool norm_supports(int64_t d) { return d >= 256 && d <= 4096 && d % 256 == 0; }

hipError_t launch_norm(const NormArgs &a, hipStream_t stream) {
  if (!norm_supports(a.d)) return hipErrorInvalidValue;
  return a.f16 ? launch_spans<true>(a, stream) : launch_spans<false>(a, stream);
}

}  // namespace svodk

#else  // SVODK_CODE_OBJECT
// The row norms as kernels for a loader that takes a code object and a flat argument record
// (device/src/amd/program.rs:403-414, 655-675; device/src/hcq.rs:1262-1285): buffers first, then
// 4-byte scalars, nothing hidden.  A kernel covers the row lengths up to the one in its name
// (d a multiple of 256).  Parameters, in the reference kernels' order (tk/src/kernels/rows.rs:41-50):
//   rms_norm        x, w, out                    rows, d, eps_bits
//   add_rms_norm    x, residual, w, out, sum     rows, d, eps_bits
//   layer_norm      x, w, b, out                 rows, d, eps_bits
//   add_layer_norm  x, residual, w, b, out, sum  rows, d, eps_bits
// Launch: ceil(rows / 4) workgroups of 256 threads.
// A wave a row here (a kernel without the dispatch packet cannot ask how many workgroups walk beside it): the row of
// this wave, and a stride past any row count.
#define SVODK_ROW_OF_WAVE \
  (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6), (int64_t)1 << 40
#define SVODK_ROWS_ENTRIES(DMAX, TYPE, F16)                                                                           \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_rms_norm_d##DMAX##_##TYPE(                    \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ w, uint16_t *__restrict__ out, int32_t rows,         \
      int32_t d, int32_t eps_bits) {                                                                                   \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, false, false, false, F16>(x, nullptr, w, nullptr, out, nullptr, rows, d, 1.0f / (float)d,  \
                                                      __builtin_bit_cast(float, eps_bits), SVODK_ROW_OF_WAVE);                            \
  }                                                                                                                    \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_add_rms_norm_d##DMAX##_##TYPE(                \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual, const uint16_t *__restrict__ w,           \
      uint16_t *__restrict__ out, uint16_t *__restrict__ sum, int32_t rows, int32_t d, int32_t eps_bits) {             \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, false, true, false, F16>(x, residual, w, nullptr, out, sum, rows, d, 1.0f / (float)d,      \
                                                     __builtin_bit_cast(float, eps_bits), SVODK_ROW_OF_WAVE);                             \
  }                                                                                                                    \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_layer_norm_d##DMAX##_##TYPE(                  \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ w, const uint16_t *__restrict__ b,                  \
      uint16_t *__restrict__ out, int32_t rows, int32_t d, int32_t eps_bits) {                                         \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, true, false, true, F16>(x, nullptr, w, b, out, nullptr, rows, d, 1.0f / (float)d,          \
                                                    __builtin_bit_cast(float, eps_bits), SVODK_ROW_OF_WAVE);                              \
  }                                                                                                                    \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_add_layer_norm_d##DMAX##_##TYPE(              \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual, const uint16_t *__restrict__ w,           \
      const uint16_t *__restrict__ b, uint16_t *__restrict__ out, uint16_t *__restrict__ sum, int32_t rows, int32_t d, \
      int32_t eps_bits) {                                                                                              \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, true, true, true, F16>(x, residual, w, b, out, sum, rows, d, 1.0f / (float)d,              \
                                                   __builtin_bit_cast(float, eps_bits), SVODK_ROW_OF_WAVE);                               \
  }

SVODK_ROWS_ENTRIES(1024, bf16, false)
SVODK_ROWS_ENTRIES(2048, bf16, false)
SVODK_ROWS_ENTRIES(4096, bf16, false)
SVODK_ROWS_ENTRIES(1024, f16, true)
SVODK_ROWS_ENTRIES(2048, f16, true)
SVODK_ROWS_ENTRIES(4096, f16, true)
#undef SVODK_ROWS_ENTRIES

}  // namespace
}  // namespace svodk
#endif  // SVODK_CODE_OBJECT
