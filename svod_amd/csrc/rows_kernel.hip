// Row norms for gfx950: LayerNorm and RMSNorm over the last dim, optionally after a residual
// add whose rounded sum is also written out.
//
// Follows norm_body (tk/src/kernels/rows.rs:52-114) op for op, in f32:
//   xs = x widened                       (with a residual: s = T(x + r) stored as `sum`, xs = s widened)
//   Layer: mean = sum(xs) * (1/d);  c = xs - mean        Rms: c = xs
//   var = sum(c * c) * (1/d) + eps;  inv = rsqrt(var);  y = (c * inv) * w  (+ b for a LayerNorm)
// and rounds to the operands' type at the store.
//
// One wave per row, as in the reference ("one warp per row"), the row held in registers between
// the passes: a lane owns 8 consecutive elements of every 512-element span (one 128-bit access,
// consecutive lanes consecutive chunks), d / 64 elements in all.  A row is read once and written
// once, so the kernel is priced against HBM bandwidth; the row sums are in-lane adds followed
// by an xor butterfly over the wave, the same order for every row.
#include <hip/hip_runtime.h>

#include "convert.h"
#include "kernels.h"

namespace svodk {
namespace {

constexpr int kRowsPerBlock = 4;  // NormCfg { br: 4 }: four waves, a row each
constexpr int kSpan = 512;        // elements one wave-wide 128-bit access covers

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}

__device__ __forceinline__ u32x4 load_once(const u32x4 *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_once(u32x4 *p, const u32x4 &v) { __builtin_nontemporal_store(v, p); }

// SPANS = ceil(d / 512): the 128-bit accesses a lane makes per row and tensor.
// The workgroup's program, for the kernels below to inline.
template <int SPANS, bool LAYER, bool RESIDUAL, bool BIAS, bool F16>
__device__ __forceinline__ void rows_body(const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual,
                                          const uint16_t *__restrict__ w, const uint16_t *__restrict__ b,
                                          uint16_t *__restrict__ out, uint16_t *__restrict__ sum, int64_t rows, int32_t d,
                                          float inv_d, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t base = row * d;
  float xs[SPANS][8];
  bool live[SPANS];
#pragma unroll
  for (int s = 0; s < SPANS; s++) {
    const int at = s * kSpan + lane * 8;
    live[s] = at < d;  // d is a multiple of 256: a row's last span is whole or half
#pragma unroll
    for (int i = 0; i < 8; i++) xs[s][i] = 0.0f;
    if (live[s]) {
      widen<F16>(load_once(reinterpret_cast<const u32x4 *>(x + base + at)), xs[s]);
      if (RESIDUAL) {
        float rs[8];
        widen<F16>(load_once(reinterpret_cast<const u32x4 *>(residual + base + at)), rs);
        // L77-86: the sum is rounded to the operands' type, stored, and read back as f32.
        u32x4 packed;
#pragma unroll
        for (int i = 0; i < 4; i++) packed[i] = narrow<F16>(xs[s][2 * i] + rs[2 * i], xs[s][2 * i + 1] + rs[2 * i + 1]);
        store_once(reinterpret_cast<u32x4 *>(sum + base + at), packed);
        widen<F16>(packed, xs[s]);
      }
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
    widen<F16>(*reinterpret_cast<const u32x4 *>(w + at), ws);
    if (LAYER && BIAS) widen<F16>(*reinterpret_cast<const u32x4 *>(b + at), bs);
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
}

#if !defined(SVODK_CODE_OBJECT)  // the library's kernel and its launch: not part of a code object build
template <int SPANS, bool LAYER, bool RESIDUAL, bool BIAS, bool F16>
__global__ __launch_bounds__(kRowsPerBlock * 64) void rows_kernel(const uint16_t *__restrict__ x,
                                                                   const uint16_t *__restrict__ residual,
                                                                   const uint16_t *__restrict__ w,
                                                                   const uint16_t *__restrict__ b,
                                                                   uint16_t *__restrict__ out, uint16_t *__restrict__ sum,
                                                                   int64_t rows, int32_t d, float inv_d, float eps) {
  rows_body<SPANS, LAYER, RESIDUAL, BIAS, F16>(x, residual, w, b, out, sum, rows, d, inv_d, eps);
}

template <int SPANS, bool LAYER, bool RESIDUAL, bool BIAS, bool F16>
hipError_t launch_rows(const NormArgs &a, hipStream_t stream) {
  const int64_t blocks = (a.rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks == 0) return hipSuccess;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
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
#define SVODK_ROWS_ENTRIES(DMAX, TYPE, F16)                                                                           \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_rms_norm_d##DMAX##_##TYPE(                    \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ w, uint16_t *__restrict__ out, int32_t rows,         \
      int32_t d, int32_t eps_bits) {                                                                                   \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, false, false, false, F16>(x, nullptr, w, nullptr, out, nullptr, rows, d, 1.0f / (float)d,  \
                                                      __builtin_bit_cast(float, eps_bits));                            \
  }                                                                                                                    \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_add_rms_norm_d##DMAX##_##TYPE(                \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual, const uint16_t *__restrict__ w,           \
      uint16_t *__restrict__ out, uint16_t *__restrict__ sum, int32_t rows, int32_t d, int32_t eps_bits) {             \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, false, true, false, F16>(x, residual, w, nullptr, out, sum, rows, d, 1.0f / (float)d,      \
                                                     __builtin_bit_cast(float, eps_bits));                             \
  }                                                                                                                    \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_layer_norm_d##DMAX##_##TYPE(                  \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ w, const uint16_t *__restrict__ b,                  \
      uint16_t *__restrict__ out, int32_t rows, int32_t d, int32_t eps_bits) {                                         \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, true, false, true, F16>(x, nullptr, w, b, out, nullptr, rows, d, 1.0f / (float)d,          \
                                                    __builtin_bit_cast(float, eps_bits));                              \
  }                                                                                                                    \
  extern "C" __global__ __launch_bounds__(kRowsPerBlock * 64) void svodk_add_layer_norm_d##DMAX##_##TYPE(              \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual, const uint16_t *__restrict__ w,           \
      const uint16_t *__restrict__ b, uint16_t *__restrict__ out, uint16_t *__restrict__ sum, int32_t rows, int32_t d, \
      int32_t eps_bits) {                                                                                              \
    if (d <= 0 || d > DMAX) return;                                                                                    \
    rows_body<DMAX / kSpan, true, true, true, F16>(x, residual, w, b, out, sum, rows, d, 1.0f / (float)d,              \
                                                   __builtin_bit_cast(float, eps_bits));                               \
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
