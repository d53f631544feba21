// Cost probe: the attention step as an instruction mix with live data (the counterpart of the `step`
// probe of tk/src/probe.rs at the scale of a whole key block): MFMAs fed from LDS (a 1 KiB fragment per
// read, as the K rows by ds_read_b128 and the transposed V rows by ds_read_b64_tr_b16), the softmax's
// VALU work beside them, random bf16 operands (so the matrix pipe draws what it draws on real data).
// R = query row blocks (of 32) a wave owns: each LDS fragment feeds R MFMAs.  Wall-clock per MFMA per SIMD
// in nominal 2.4 GHz cycles, chip-wide TFLOP/s, and the clock held (s_memtime / s_memrealtime).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#include <cstdlib>
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
#define LDS_PTR(T) __attribute__((address_space(3))) T *
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s line %d\n", hipGetErrorString(e), __LINE__); return 1;}}while(0)
constexpr int ITERS = 600;

__device__ __forceinline__ void unit(float (&x)[16], int i, float y) {
  // two scores -> two probabilities: 2 fma, 2 exp, 2 add, 1 cvt, 1 max3
  float a = __builtin_fmaf(x[i & 15], y, -y), b = __builtin_fmaf(x[(i + 1) & 15], y, -y);
  a = __builtin_amdgcn_exp2f(a); b = __builtin_amdgcn_exp2f(b);
  x[(i + 2) & 15] += a; x[(i + 3) & 15] += b;
  typedef __attribute__((ext_vector_type(2))) float f2; typedef __attribute__((ext_vector_type(2))) __bf16 b2;
  f2 f = {a, b}; b2 h = __builtin_convertvector(f, b2);
  x[(i + 4) & 15] = __builtin_bit_cast(float, h);
  x[(i + 5) & 15] = __builtin_fmaxf(__builtin_fmaxf(x[(i + 5) & 15], a), b);
  asm volatile("" : "+v"(x[(i + 2) & 15]), "+v"(x[(i + 3) & 15]), "+v"(x[(i + 4) & 15]), "+v"(x[(i + 5) & 15]));
}

// MODE 0: operands in registers (no LDS); 1: K-side reads (ds_read_b128); 2: half K-side, half V-side (tr reads)
// R: MFMAs per fragment; VALU: softmax units per 2*R MFMAs... (one unit per two MFMAs, the D=128 ratio)
template <int MODE, int R, bool VALU, int EVERY = 2>
__global__ __launch_bounds__(256) void k(float* out, uint64_t* clk, const uint32_t* rnd) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 12288; i += 256) ((uint32_t*)lds)[i] = rnd[i];  // 48 KiB of random bf16 pairs
  __syncthreads();
  const uint8_t* a128 = lds + lane * 16;
  const uint8_t* a64 = lds + lane * 8;
  f32x16 acc[4 * R];
  for (int j = 0; j < 4 * R; j++) for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
  u32x4 b[R];
  for (int r = 0; r < R; r++) for (int i = 0; i < 4; i++) b[r][i] = rnd[(tid * 4 + i + 1024 * r) & 16383];
  float x[16]; for (int i = 0; i < 16; i++) x[i] = __uint_as_float(rnd[(tid + i * 256) & 16383] & 0x3fffffff);
  float y = 0.37f; asm volatile("" : "+v"(y));
  auto frag = [&](int s) -> u32x4 {
    if (MODE == 0) return b[0];
    if (MODE == 1 || (s & 1) == 0) return *reinterpret_cast<const u32x4*>(a128 + (s % 47) * 1024);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(a64 + (s % 47) * 1024));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(a64 + (s % 47) * 1024 + 512));
    return __builtin_bit_cast(u32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  constexpr int PD = 4;
  u32x4 ring[PD];
#pragma unroll
  for (int p = 0; p < PD; p++) ring[p] = frag(p);
  uint64_t t0 = 0, r0 = 0;
  if (blockIdx.x == 0 && tid == 0) asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t0), "=s"(r0));
  for (int it = 0; it < ITERS; it++) {
#pragma unroll
    for (int j = 0; j < 32; j++) {  // 32 fragments a step
#pragma unroll
      for (int r = 0; r < R; r++)
        acc[(j & 3) * R + r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ring[j % PD]), __builtin_bit_cast(bf16x8, b[r]), acc[(j & 3) * R + r], 0, 0, 0);
      if (MODE != 0) ring[j % PD] = frag(j + PD + it);
      if (VALU) {
#pragma unroll
        for (int r = 0; r < R; r++) if (j % EVERY == 0) unit(x, j * 6 + r * 3, y);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (blockIdx.x == 0 && tid == 0) {
    uint64_t t1, r1;
    asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t1), "=s"(r1));
    clk[0] = t1 - t0; clk[1] = r1 - r0;
  }
  float s = 0; for (int i = 0; i < 16; i++) s += x[i];
  for (int j = 0; j < 4 * R; j++) for (int i = 0; i < 16; i++) s += acc[j][i];
  for (int p = 0; p < PD; p++) s += __uint_as_float(ring[p][0]);
  out[blockIdx.x * 256 + tid] = s;
}
template <int MODE, int R, bool VALU, int EVERY = 2> int run(const char* name, float* d, uint64_t* clk, const uint32_t* rnd) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  printf("%-52s", name);
  CK(hipFuncSetAttribute((const void*)k<MODE, R, VALU, EVERY>, hipFuncAttributeMaxDynamicSharedMemorySize, 49152));
  for (int bpc : {1, 2, 3}) {
    if (bpc == 3 && R > 1) continue;
    int blocks = 256 * bpc;
    k<MODE, R, VALU, EVERY><<<blocks, 256, 49152>>>(d, clk, rnd); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    for (int rep = 0; rep < 3; rep++) k<MODE, R, VALU, EVERY><<<blocks, 256, 49152>>>(d, clk, rnd);
    CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); ms /= 3;
    uint64_t h[2]; CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
    double mf = (double)bpc * ITERS * 32 * R;
    double cyc = ms * 1e-3 * 2.4e9 / mf;
    printf(" | %dw/SIMD %6.1f cyc/MFMA = %4.0f TFLOP/s @ %4.2f GHz", bpc, cyc, 2500.0 * 32.0 / cyc, (double)h[0] / (double)h[1] * 0.1);
  }
  printf("\n"); fflush(stdout); return 0;
}
int main() {
  float* d; CK(hipMalloc(&d, 256 * 3 * 256 * 4));
  uint64_t* clk; CK(hipMalloc(&clk, 16));
  uint32_t* h = (uint32_t*)malloc(65536); srand(1);
  for (int i = 0; i < 16384; i++) {  // two bf16 in [-1, 1) with random mantissas
    auto one = [] { uint32_t sign = rand() & 1, e = 120 + rand() % 7, m = rand() & 0x7f; return (sign << 15) | (e << 7) | m; };
    h[i] = one() | one() << 16;
  }
  uint32_t* rnd; CK(hipMalloc(&rnd, 65536)); CK(hipMemcpy(rnd, h, 65536, hipMemcpyHostToDevice));
  printf("MFMA 32x32x16 bf16 with random operands; a fragment = 1 KiB per wave from LDS; cycles are nominal 2.4 GHz, TFLOP/s chip-wide\n");
  run<0, 1, false>("registers only, no VALU", d, clk, rnd);
  run<0, 1, true>("registers only + softmax (D=128 ratio)", d, clk, rnd);
  run<1, 1, false>("b128 fragment per MFMA, no VALU", d, clk, rnd);
  run<2, 1, false>("b128 / tr_b64 alternating per MFMA, no VALU", d, clk, rnd);
  run<2, 1, true>("b128/tr fragment per MFMA + softmax  [32-row wave]", d, clk, rnd);
  run<1, 1, true>("b128 fragment per MFMA + softmax (if V lay transposed)", d, clk, rnd);
  run<2, 1, true, 1>("b128/tr fragment per MFMA + softmax at the D=64 ratio", d, clk, rnd);
  run<0, 1, true, 1>("registers only + softmax at the D=64 ratio", d, clk, rnd);
  run<2, 2, false>("fragment per 2 MFMAs, no VALU", d, clk, rnd);
  run<2, 2, true>("fragment per 2 MFMAs + softmax      [64-row wave]", d, clk, rnd);
  run<2, 2, true, 1>("fragment per 2 MFMAs + softmax at the D=64 ratio", d, clk, rnd);
  return 0;
}
