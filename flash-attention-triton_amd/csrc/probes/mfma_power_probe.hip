// Probe: what a loop of nothing but v_mfma_f32_32x32x16_bf16 sustains on MI355X, on constant
// operands and on random ones, with the shader clock and board power sampled meanwhile.
// It prices the "dense bf16 peak" the attention kernels are measured against: the published
// 2.5 PFLOP/s assumes 2.4 GHz, which the 1400 W board limit does not allow on random data.
//
//   usage: mfma_power_probe [seconds per case, default 4]
#include <chrono>
#include <random>

#include "common.hpp"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_loop(const unsigned short *operands, float *out, int iters) {
  bf16x8 a[4], b[4];
  for (int m = 0; m < 4; m++)
    for (int j = 0; j < 8; j++) {
      const unsigned short ua = operands[((threadIdx.x * 4 + m) * 16 + j) % 65536];
      const unsigned short ub = operands[((threadIdx.x * 4 + m) * 16 + 8 + j) % 65536];
      a[m][j] = __builtin_bit_cast(__bf16, ua);
      b[m][j] = __builtin_bit_cast(__bf16, ub);
    }
  f32x16 c[4];
  for (int m = 0; m < 4; m++)
    for (int i = 0; i < 16; i++) c[m][i] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int m = 0; m < 4; m++) c[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m], b[m], c[m], 0, 0, 0);
  }
  float s = 0.f;
  for (int m = 0; m < 4; m++)
    for (int i = 0; i < 16; i++) s += c[m][i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

static void run_case(const char *label, const unsigned short *dev_operands, float *out, double seconds,
                     int waves_per_simd) {
  const int iters = 20000;  // 80000 MFMAs per wave per launch
  const int grid = 256 * waves_per_simd;
  const double flops_per_launch = (double)grid * 4 * iters * 4 * 32768.0;
  for (int i = 0; i < 3; i++) hipLaunchKernelGGL(mfma_loop, dim3(grid), dim3(256), 0, 0, dev_operands, out, iters);
  HIP_CHECK(hipDeviceSynchronize());
  SysfsSampler sampler;
  sampler.start();
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  const auto t0 = std::chrono::steady_clock::now();
  int launches = 0;
  HIP_CHECK(hipEventRecord(e0));
  while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds) {
    for (int i = 0; i < 4; i++) hipLaunchKernelGGL(mfma_loop, dim3(grid), dim3(256), 0, 0, dev_operands, out, iters);
    launches += 4;
    HIP_CHECK(hipDeviceSynchronize());
  }
  HIP_CHECK(hipEventRecord(e1));
  HIP_CHECK(hipEventSynchronize(e1));
  sampler.finish();
  float ms;
  HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  const double tflops = flops_per_launch * launches / (ms * 1e-3) / 1e12;
  const double mhz = SysfsSampler::mean(sampler.sclk), watts = SysfsSampler::mean(sampler.power);
  printf("%-28s %d wave(s)/SIMD: %7.1f TFLOP/s  sclk %6.0f MHz  power %6.0f W  (%.1f %% of 256 CU x 4096 FLOP/clk at that clock)\n",
         label, waves_per_simd, tflops, mhz, watts, mhz > 0 ? 100.0 * tflops / (256 * 4096.0 * mhz * 1e-6) : -1.0);
}

int main(int argc, char **argv) {
  const double seconds = argc > 1 ? atof(argv[1]) : 4.0;
  std::vector<unsigned short> constant(65536, 0x3f80), random_bits(65536);  // 1.0 in bf16
  std::mt19937 rng(42);
  std::normal_distribution<float> normal(0.f, 1.f);
  for (auto &u : random_bits) {
    const float x = normal(rng);
    unsigned bits;
    memcpy(&bits, &x, 4);
    u = (unsigned short)(bits >> 16);
  }
  unsigned short *dev;
  float *out;
  HIP_CHECK(hipMalloc(&dev, 65536 * 2));
  HIP_CHECK(hipMalloc(&out, 1024 * 256 * 4));
  for (int waves = 1; waves <= 2; waves++) {
    HIP_CHECK(hipMemcpy(dev, constant.data(), 65536 * 2, hipMemcpyHostToDevice));
    run_case("constant operands (1.0)", dev, out, seconds, waves);
    HIP_CHECK(hipMemcpy(dev, random_bits.data(), 65536 * 2, hipMemcpyHostToDevice));
    run_case("random operands N(0,1)", dev, out, seconds, waves);
  }
  return 0;
}
