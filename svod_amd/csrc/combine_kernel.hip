// combine_splits for gfx950: the partial online-softmax states the attention kernel's key
// splits leave are merged into the output (tk/src/kernels/attention.rs:948-1014):
//   m = max_s m_s ;  w_s = 2^(m_s - m) ;  l = sum_s l_s w_s ;  o = sum_s o_s w_s
//   out = o / (l == 0 ? 1 : l), a row no key reached coming out as zeros (L971-980).
// Sums run in split order, one op at a time in f32, as the reference's tile program does.
//
// The kernel is HBM-bound (every partial is read once): a row of d floats is shared by d/4
// lanes, each reading one 128-bit chunk per split and writing 8 bytes of bf16.
#include <hip/hip_runtime.h>

#include <atomic>

#include "kernels.h"

#if !defined(SVODK_CODE_OBJECT)
// The partial states of a split call whose caller cannot lend a workspace because it cannot allocate
// one (code under graph capture, a serving loop with a fixed memory plan): kSplitScratchBytes of
// device memory that every GPU the library runs on holds until the process ends.  In host code the
// array's name is a stand-in, not a device address: each device's copy has its own address, which
// split_scratch() looks up once with that device current and keeps; kernels take that pointer as an
// argument.
static __device__ __align__(256) unsigned char scratch[svodk::kSplitScratchBytes];
#endif

namespace svodk {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

constexpr int kThreads = 256;

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

// Round to nearest even into the output's type.
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 f = {lo, hi};
  if constexpr (F16)
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  else
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// The workgroup's program, for the kernels below to inline.
template <int D, bool F16>
__device__ __forceinline__ void combine_body(const float *__restrict__ o_part, const float *__restrict__ m_part,
                                             const float *__restrict__ l_part, uint16_t *__restrict__ o, int64_t rows,
                                             int32_t splits) {
#pragma clang fp contract(off)
  constexpr int kLanes = D / 4;  // lanes sharing a row
  const int64_t gid = (int64_t)__builtin_amdgcn_workgroup_id_x() * kThreads + __builtin_amdgcn_workitem_id_x();
  const int64_t row = gid / kLanes;
  const int part = (int)(gid % kLanes);
  if (row >= rows) return;
  float m = m_part[row];
  for (int s = 1; s < splits; s++) m = __builtin_fmaxf(m, m_part[(int64_t)s * rows + row]);
  float l = 0.0f;
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int s = 0; s < splits; s++) {
    const int64_t at = (int64_t)s * rows + row;
    const float w = __builtin_amdgcn_exp2f(m_part[at] - m);
    const float lw = l_part[at] * w;
    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(o_part + at * D) + part);
    const f32x4 ow = x * w;
    l = s == 0 ? lw : l + lw;
    acc = s == 0 ? ow : acc + ow;
  }
  const float ll = l == 0.0f ? 1.0f : l;
  u32x2 out;
  out[0] = pack2<F16>(acc[0] / ll, acc[1] / ll);
  out[1] = pack2<F16>(acc[2] / ll, acc[3] / ll);
  *(reinterpret_cast<u32x2 *>(o + row * D) + part) = out;
}

#if !defined(SVODK_CODE_OBJECT)  // the library's kernel and its launch: not part of a code object build
template <int D, bool F16>
__global__ __launch_bounds__(kThreads) void combine_kernel(const float *__restrict__ o_part,
                                                           const float *__restrict__ m_part,
                                                           const float *__restrict__ l_part, uint16_t *__restrict__ o,
                                                           int64_t rows, int32_t splits) {
  combine_body<D, F16>(o_part, m_part, l_part, o, rows, splits);
}

template <int D, bool F16>
hipError_t launch(const CombineArgs &a, hipStream_t stream) {
  const int64_t threads = a.rows * (D / 4);
  if (threads == 0) return hipSuccess;
  const int64_t blocks = (threads + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((combine_kernel<D, F16>), dim3((uint32_t)blocks), dim3(kThreads), 0, stream, a.o_part, a.m_part,
                     a.l_part, (uint16_t *)a.o, a.rows, a.splits);
  return hipGetLastError();
}

std::atomic<void *> g_scratch_at[64];  // `scratch` by device ordinal; devices past 63 ask every time

}  // namespace

hipError_t split_scratch(void **ptr, int64_t *bytes) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  void *at = device >= 0 && device < 64 ? g_scratch_at[device].load(std::memory_order_acquire) : nullptr;
  if (at == nullptr) {
    e = hipGetSymbolAddress(&at, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (at == nullptr) return hipErrorInvalidSymbol;
    if (device >= 0 && device < 64) g_scratch_at[device].store(at, std::memory_order_release);
  }
  *ptr = at;
  *bytes = kSplitScratchBytes;
  return hipSuccess;
}

hipError_t launch_combine(const CombineArgs &a, hipStream_t stream) {
  if (a.splits < 1) return hipErrorInvalidValue;
  switch (a.d) {
    case 32: return a.f16 ? launch<32, true>(a, stream) : launch<32, false>(a, stream);
    case 48: return a.f16 ? launch<48, true>(a, stream) : launch<48, false>(a, stream);
    case 64: return a.f16 ? launch<64, true>(a, stream) : launch<64, false>(a, stream);
    case 128: return a.f16 ? launch<128, true>(a, stream) : launch<128, false>(a, stream);
    case 256: return a.f16 ? launch<256, true>(a, stream) : launch<256, false>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace svodk

#else  // SVODK_CODE_OBJECT
// The merge as kernels for a loader that takes a code object and a flat argument record
// (device/src/amd/program.rs:403-414, 655-675; device/src/hcq.rs:1262-1285): o_part [splits, rows, D],
// m_part and l_part [splits, rows] (f32, what a split attention kernel wrote), o [rows, D], then rows
// (batch * t * heads) and splits.  Launch: ceil(rows * (D / 4) / 256) workgroups of 256 threads.
#define SVODK_COMBINE_ENTRY(NAME, D, F16)                                                                             \
  extern "C" __global__ __launch_bounds__(kThreads) void NAME(const float *__restrict__ o_part,                       \
                                                              const float *__restrict__ m_part,                       \
                                                              const float *__restrict__ l_part,                       \
                                                              uint16_t *__restrict__ o, int32_t rows, int32_t splits) { \
    if (splits >= 1) combine_body<D, F16>(o_part, m_part, l_part, o, rows, splits);                                   \
  }
SVODK_COMBINE_ENTRY(svodk_combine_d32_bf16, 32, false)
SVODK_COMBINE_ENTRY(svodk_combine_d48_bf16, 48, false)
SVODK_COMBINE_ENTRY(svodk_combine_d64_bf16, 64, false)
SVODK_COMBINE_ENTRY(svodk_combine_d128_bf16, 128, false)
SVODK_COMBINE_ENTRY(svodk_combine_d256_bf16, 256, false)
SVODK_COMBINE_ENTRY(svodk_combine_d32_f16, 32, true)
SVODK_COMBINE_ENTRY(svodk_combine_d48_f16, 48, true)
SVODK_COMBINE_ENTRY(svodk_combine_d64_f16, 64, true)
SVODK_COMBINE_ENTRY(svodk_combine_d128_f16, 128, true)
SVODK_COMBINE_ENTRY(svodk_combine_d256_f16, 256, true)
#undef SVODK_COMBINE_ENTRY

}  // namespace
}  // namespace svodk
#endif  // SVODK_CODE_OBJECT
