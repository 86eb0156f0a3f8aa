// Issue rate of the vector instructions the attention kernels spend their non-MFMA time on, with one
// to four waves per SIMD: how many shader cycles a SIMD needs per wave instruction.  Each wave runs a
// loop of eight independent instructions of one kind; the shader clock is sampled meanwhile, so the
// result is in cycles, not only in nanoseconds.
//
// usage: valu_rate_probe [seconds per case, default 0.3]
#include "common.hpp"

constexpr int kIters = 20000, kUnroll = 8;

enum Kind { FMA, ADD, MUL, EXP, CVT_BF16, DOT2_BF16, MAX3, PERMLANE_SWAP, KINDS };
static const char *kNames[KINDS] = {"v_fma_f32", "v_add_f32", "v_mul_f32", "v_exp_f32", "v_cvt_pk_bf16_f32",
                                    "v_dot2_f32_bf16", "v_max3_f32", "v_permlane32_swap_b32"};

template <int KIND>
__global__ __launch_bounds__(256) void rate_kernel(float *out, float seed) {
  float x[kUnroll], acc[kUnroll];
  for (int i = 0; i < kUnroll; i++) {
    x[i] = seed + threadIdx.x * 1e-6f + i;
    acc[i] = 0.f;
  }
  for (int it = 0; it < kIters; it++) {
#pragma unroll
    for (int i = 0; i < kUnroll; i++) {
      if (KIND == FMA) asm volatile("v_fma_f32 %0, %1, %1, %0" : "+v"(acc[i]) : "v"(x[i]));
      if (KIND == ADD) asm volatile("v_add_f32 %0, %1, %0" : "+v"(acc[i]) : "v"(x[i]));
      if (KIND == MUL) asm volatile("v_mul_f32 %0, %1, %1" : "=v"(acc[i]) : "v"(x[i]));
      if (KIND == EXP) asm volatile("v_exp_f32 %0, %1" : "=v"(acc[i]) : "v"(x[i]));
      if (KIND == CVT_BF16) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %1" : "=v"(acc[i]) : "v"(x[i]));
      if (KIND == DOT2_BF16) asm volatile("v_dot2_f32_bf16 %0, %1, %1, %0" : "+v"(acc[i]) : "v"(x[i]));
      if (KIND == MAX3) asm volatile("v_max3_f32 %0, %1, %1, %0" : "+v"(acc[i]) : "v"(x[i]));
      if (KIND == PERMLANE_SWAP) asm volatile("v_permlane32_swap_b32 %0, %1" : "+v"(acc[i]), "+v"(x[i]));
    }
  }
  float s = 0.f;
  for (int i = 0; i < kUnroll; i++) s += acc[i] + x[i];
  if (s == 12345.678f) out[threadIdx.x] = s;  // never true: keeps the loop alive
}

template <int KIND>
void run(int waves_per_simd, double seconds, float *out) {
  const dim3 grid(256 * waves_per_simd), block(256);  // 4 waves per workgroup, one per SIMD
  hipEvent_t a, b;
  HIP_CHECK(hipEventCreate(&a));
  HIP_CHECK(hipEventCreate(&b));
  for (int w = 0; w < 3; w++) hipLaunchKernelGGL(rate_kernel<KIND>, grid, block, 0, 0, out, 1.0f);
  HIP_CHECK(hipDeviceSynchronize());
  SysfsSampler sampler;
  sampler.start();
  HIP_CHECK(hipEventRecord(a));
  int launches = 0;
  float ms = 0.f;
  do {
    for (int w = 0; w < 20; w++) hipLaunchKernelGGL(rate_kernel<KIND>, grid, block, 0, 0, out, 1.0f);
    launches += 20;
    HIP_CHECK(hipEventRecord(b));
    HIP_CHECK(hipEventSynchronize(b));
    HIP_CHECK(hipEventElapsedTime(&ms, a, b));
  } while (ms < seconds * 1e3);
  sampler.finish();
  const double mhz = SysfsSampler::mean(sampler.sclk);
  const double instr_per_simd = (double)launches * kIters * kUnroll * waves_per_simd;
  const double ns = ms * 1e6 / instr_per_simd;
  printf("%-24s %d wave(s)/SIMD: %6.2f ns per wave instruction per SIMD, sclk %5.0f MHz -> %5.2f cycles\n",
         kNames[KIND], waves_per_simd, ns, mhz, ns * mhz * 1e-3);
  fflush(stdout);
  HIP_CHECK(hipEventDestroy(a));
  HIP_CHECK(hipEventDestroy(b));
}

int main(int argc, char **argv) {
  const double seconds = argc > 1 ? atof(argv[1]) : 0.3;
  float *out;
  HIP_CHECK(hipMalloc(&out, 4096));
  for (int w = 1; w <= 4; w++) {
    run<FMA>(w, seconds, out);
    run<ADD>(w, seconds, out);
    run<MUL>(w, seconds, out);
    run<EXP>(w, seconds, out);
    run<CVT_BF16>(w, seconds, out);
    run<DOT2_BF16>(w, seconds, out);
    run<MAX3>(w, seconds, out);
    run<PERMLANE_SWAP>(w, seconds, out);
  }
  HIP_CHECK(hipFree(out));
  return 0;
}
