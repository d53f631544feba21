// Cost probe: what the matrix pipe and the VALU of a gfx950 SIMD do side by side, with operands in
// registers (the counterpart of the `step` and `score` probes of tk/src/probe.rs, which time a matrix
// step and a softmax element on the device before the planner prices a config).  Every figure is
// wall-clock (HIP events) over a launch that fills the chip, expressed as nominal 2.4 GHz cycles per
// MFMA slot per SIMD; the shader clock actually held is read from s_memtime against s_memrealtime
// (100 MHz) inside the kernel.  Operands are constants: the matrix pipe at its lowest power.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s line %d\n", hipGetErrorString(e), __LINE__); return 1;}}while(0)
constexpr int ITERS = 2000;

#define MFMA_V(acc) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
#define MFMA_A(acc) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
#define FMA(i) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(x[(i) & 15]) : "v"(y));
#define ADD(i) asm volatile("v_add_f32 %0, %0, %1" : "+v"(x[(i) & 15]) : "v"(y));
#define EXP(i) asm volatile("v_exp_f32 %0, %0" : "+v"(x[(i) & 15]));
#define CVT(i) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %1" : "+v"(x[(i) & 15]) : "v"(y));
#define MAX3(i) asm volatile("v_max3_f32 %0, %0, %1, %1" : "+v"(x[(i) & 15]) : "v"(y));

// One "unit" of softmax VALU work for 2 scores: 2 fma, 2 exp, 2 add, 1 cvt, 1 max3 (the D=64 step has
// 16 of these per 16 MFMAs; the D=128 step 16 per 32 MFMAs).
#define UNIT(i) FMA(i) FMA(i + 1) EXP(i) EXP(i + 1) ADD(i + 2) ADD(i + 3) CVT(i + 4) MAX3(i + 5)

// MODE: 0 mfma only; 1 mfma + NV fma each; 2 mfma + NV exp each; 3 mfma + one softmax unit each (D=64 mix);
//       4 mfma + one unit per two (D=128 mix); 5 VALU only: the units of mode 3 without the MFMAs;
//       6 wave-specialised: even waves of a SIMD run MFMA only, odd waves the units only (needs 2 waves/SIMD per WG)
// AG: accumulators in AGPRs.
template <int MODE, int NV, bool AG>
__global__ __launch_bounds__(512) void k(float* out, uint64_t* clk, float seed) {
  f32x16 acc[4];
  for (int j = 0; j < 4; j++) for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
  u32x4 a, b;
  for (int i = 0; i < 4; i++) { a[i] = 0x3c003c00; b[i] = 0x3c003c00; }
  float x[16]; for (int i = 0; i < 16; i++) x[i] = seed + i * 0.01f + threadIdx.x * 1e-5f;
  float y = 0.999f;
  asm volatile("" : "+v"(y));
  const int wave = threadIdx.x >> 6;
  const bool matrix_wave = MODE != 6 || (wave < 4);
  uint64_t t0 = 0, r0 = 0;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t0), "=s"(r0));
  }
  for (int it = 0; it < ITERS; it++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      if (MODE != 5 && matrix_wave) {
        if (AG) { MFMA_A(acc[j & 3]) } else { MFMA_V(acc[j & 3]) }
      }
      if (MODE == 1) {
#pragma unroll
        for (int v = 0; v < NV; v++) { FMA(j * NV + v) }
      }
      if (MODE == 2) {
#pragma unroll
        for (int v = 0; v < NV; v++) { EXP(j * NV + v) }
      }
      if (MODE == 3 || MODE == 5 || (MODE == 6 && !matrix_wave)) { UNIT(j * 6) }
      if (MODE == 4 && (j & 1)) { UNIT(j * 6) }
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    uint64_t t1, r1;
    asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t1), "=s"(r1));
    clk[0] = t1 - t0;
    clk[1] = r1 - r0;
  }
  float s = 0; for (int i = 0; i < 16; i++) s += x[i];
  for (int j = 0; j < 4; j++) for (int i = 0; i < 16; i++) s += acc[j][i];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}
template <int MODE, int NV, bool AG> int run(const char* name, float* d, uint64_t* clk) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  printf("%-44s", name);
  const int threads = MODE == 6 ? 512 : 256;
  for (int bpc : {1, 2, 3}) {
    if (MODE == 6 && bpc == 3) continue;
    int blocks = 256 * bpc;
    k<MODE, NV, AG><<<blocks, threads>>>(d, clk, 0.5f); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); k<MODE, NV, AG><<<blocks, threads>>>(d, clk, 0.5f); CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    uint64_t h[2]; CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
    double per = (double)bpc * ITERS * 16;  // MFMA slots per SIMD
    double cyc = ms * 1e-3 * 2.4e9 / per;
    printf(" | %dw/SIMD %6.1f cyc/slot %4.2f GHz", (MODE == 6 ? 2 : 1) * bpc, cyc, (double)h[0] / (double)h[1] * 0.1);
  }
  printf("\n"); fflush(stdout); return 0;
}
int main() {
  float* d; CK(hipMalloc(&d, 256 * 3 * 512 * 4));
  uint64_t* clk; CK(hipMalloc(&clk, 16));
  printf("a slot = one v_mfma_f32_32x32x16_bf16 (32 cycles of the matrix pipe) and what is issued with it; cycles are nominal 2.4 GHz\n");
  run<0, 0, false>("mfma only, acc in VGPR", d, clk);
  run<0, 0, true>("mfma only, acc in AGPR", d, clk);
  run<1, 2, false>("mfma + 2 fma, VGPR", d, clk);
  run<1, 4, false>("mfma + 4 fma, VGPR", d, clk);
  run<1, 8, false>("mfma + 8 fma, VGPR", d, clk);
  run<1, 12, false>("mfma + 12 fma, VGPR", d, clk);
  run<1, 4, true>("mfma + 4 fma, AGPR", d, clk);
  run<1, 8, true>("mfma + 8 fma, AGPR", d, clk);
  run<1, 12, true>("mfma + 12 fma, AGPR", d, clk);
  run<2, 1, false>("mfma + 1 exp, VGPR", d, clk);
  run<2, 2, false>("mfma + 2 exp, VGPR", d, clk);
  run<2, 3, false>("mfma + 3 exp, VGPR", d, clk);
  run<2, 2, true>("mfma + 2 exp, AGPR", d, clk);
  run<2, 3, true>("mfma + 3 exp, AGPR", d, clk);
  run<5, 0, false>("softmax unit only (no mfma)", d, clk);
  run<3, 0, false>("mfma + unit (D=64 mix), VGPR", d, clk);
  run<3, 0, true>("mfma + unit (D=64 mix), AGPR", d, clk);
  run<4, 0, false>("mfma + unit/2 (D=128 mix), VGPR", d, clk);
  run<4, 0, true>("mfma + unit/2 (D=128 mix), AGPR", d, clk);
  run<6, 0, false>("specialised waves: mfma | unit, VGPR", d, clk);
  run<6, 0, true>("specialised waves: mfma | unit, AGPR", d, clk);
  return 0;
}
