// Probe: what the dQ accumulation of a key-tile-parallel (sequence-parallel) backward costs on
// MI355X when it is done with fp32 global atomic adds, the formulation of the reference's
// non-deterministic mode (src/flash_attention_triton/_triton_kernels_v2.py:336-339, 466-494).
//
// The probe issues exactly the atomic traffic such a backward would issue for the headline
// problem (B*H = 64 heads, N = 4096, D = 128, key tiles of 128 rows, query blocks of 32 rows) and
// nothing else: one workgroup of 4 waves per (head, key tile); for every 32-row query block at
// or below its diagonal it adds a 32 x 128 fp32 block into dQ, wave w owning columns 32w..32w+31,
// each atomic instruction covering two 128-byte row segments.  Heads are mapped to XCDs like the
// library's kernels map them (`group` heads at a time, group/8 per XCD), so that with group = 8
// one head's 2 MiB of fp32 dQ is the only dQ an XCD's 4 MiB L2 sees at a time.
//
//   usage: dq_atomics_probe
#include "common.hpp"

constexpr int N = 4096, D = 128, TILES = N / 128;

template <int HEAD_GROUP>
__global__ __launch_bounds__(256, 1) void atomics_only(float *dq) {
  const int per_group = HEAD_GROUP * TILES;
  const int g = blockIdx.x / per_group, r = blockIdx.x % per_group;
  const int bh = g * HEAD_GROUP + r % HEAD_GROUP, kt = r / HEAD_GROUP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 31, h = lane >> 5;
  float *base = dq + (size_t)bh * N * D + 32 * wave + c;
  for (int qb = kt * 4; qb < N / 32; qb++) {
    float *rowp = base + (size_t)(qb * 32 + 4 * h) * D;
#pragma unroll
    for (int i = 0; i < 16; i++)
      __builtin_amdgcn_global_atomic_fadd_f32(
          (__attribute__((address_space(1))) float *)(rowp + (size_t)(8 * (i / 4) + i % 4) * D), 1.0f);
  }
}

template <int HEAD_GROUP>
static double time_us(float *dq, int heads) {
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  for (int i = 0; i < 3; i++) hipLaunchKernelGGL(atomics_only<HEAD_GROUP>, dim3(heads * TILES), dim3(256), 0, 0, dq);
  HIP_CHECK(hipEventRecord(e0));
  for (int i = 0; i < 10; i++) hipLaunchKernelGGL(atomics_only<HEAD_GROUP>, dim3(heads * TILES), dim3(256), 0, 0, dq);
  HIP_CHECK(hipEventRecord(e1));
  HIP_CHECK(hipEventSynchronize(e1));
  float ms;
  HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  return ms / 10 * 1000;
}

int main() {
  const int heads = 64;
  float *dq;
  HIP_CHECK(hipMalloc(&dq, (size_t)heads * N * D * 4));
  HIP_CHECK(hipMemset(dq, 0, (size_t)heads * N * D * 4));
  // (key tile, query block) pairs per head: sum over tiles kt of (128 - 4 kt) blocks.
  double pairs = 0;
  for (int kt = 0; kt < TILES; kt++) pairs += N / 32 - 4 * kt;
  const double gigabytes = heads * pairs * 32 * 128 * 4 / 1e9;
  printf("fp32 atomic-add payload of one backward at B*H=64, N=4096, D=128, 128-row key tiles: %.2f GB\n", gigabytes);
  const double t64 = time_us<64>(dq, heads), t16 = time_us<16>(dq, heads), t8 = time_us<8>(dq, heads);
  printf("heads per XCD at a time = 8: %7.0f us (%.2f TB/s)\n", t64, gigabytes / t64 * 1e3);
  printf("heads per XCD at a time = 2: %7.0f us (%.2f TB/s)\n", t16, gigabytes / t16 * 1e3);
  printf("heads per XCD at a time = 1: %7.0f us (%.2f TB/s)\n", t8, gigabytes / t8 * 1e3);
  float last[1];
  HIP_CHECK(hipMemcpy(last, dq + (size_t)(N - 1) * D, 4, hipMemcpyDeviceToHost));
  printf("check: dq[head 0][last row][0] = %.0f adds (39 launches x 32 key tiles = 1248)\n", last[0]);
  return 0;
}
