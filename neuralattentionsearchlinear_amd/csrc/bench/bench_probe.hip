// Benchmark aid, NOT part of libnatsl.so or of the C ABI in include/natsl.h: built into csrc/libnatsl_bench.so, which only
// bench.py loads.  A dense bf16 matrix-core loop that reports how fast the shader clock ran while it executed.
//
// Roofline fractions are quoted against the published peak, which assumes the 2.4 GHz boost clock; under a
// sustained matrix load the clock settles lower.  This kernel runs `iters` rounds of four independent
// v_mfma_f32_32x32x16_bf16 per wave on every workgroup and records, per workgroup, the shader-clock cycles and the
// ticks of the constant 100 MHz real-time counter it took, so that a benchmark can print the clock under load and the
// matrix rate a pure MFMA loop reaches on the same box right after its timed steps.
#include "../natsl_device.h"

namespace natsl {

__global__ __launch_bounds__(256) void mfma_clock_probe_kernel(unsigned long long* out, int iters) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(float)((threadIdx.x + i) & 7);
    b[i] = (__bf16)(float)(i + 1);
  }
  f32x16 acc[4];
#pragma unroll
  for (int n = 0; n < 4; ++n)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[n][r] = 0.f;
  __syncthreads();
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int n = 0; n < 4; ++n) acc[n] = mfma32(a, b, acc[n]);
  }
  float s = 0.f;
#pragma unroll
  for (int n = 0; n < 4; ++n) s += acc[n][0];
  // the sum keeps the loop alive; it is never negative, so nothing but the counters is written
  __syncthreads();
  const unsigned long long c1 = clock64(), w1 = wall_clock64();
  if (threadIdx.x == 0) {
    out[2 * blockIdx.x] = (c1 - c0) + (s < 0.f ? 1ull : 0ull);
    out[2 * blockIdx.x + 1] = w1 - w0;
  }
}

}  // namespace natsl

using namespace natsl;

// out[2i] = shader-clock cycles, out[2i+1] = ticks of the constant 100 MHz counter that workgroup i's loop took
// (iters * 4 * 32768 FLOPs per wave, 4 waves per workgroup).  Returns 0, or -1 for a bad argument / refused launch.
extern "C" int natsl_bench_mfma_clock_probe(unsigned long long* out, int n_workgroups, int iters, void* stream) {
  if (!out || n_workgroups <= 0 || iters <= 0) return -1;
  hipLaunchKernelGGL(mfma_clock_probe_kernel, dim3((unsigned)n_workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), out, iters);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}
