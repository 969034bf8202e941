// Measurement probe: the rate the matrix cores sustain when nothing else runs.
//
// Every CU gets one workgroup of 8 waves (2 per SIMD) whose lanes keep a 2x4 grid of 32x32
// accumulator tiles and issue MFMAs back to back from operands held in registers: no LDS,
// no memory, no barrier. With all-zero operands the result is the clock-limited peak; with
// random operand bits the sustained clock drops under the board's power limit, so the rate
// is the ceiling any real GEMM on this part works under. The kernel also reads the shader
// clock counter and the 100 MHz wall counter to report the clock it actually ran at.
#include "common.hpp"

namespace crl {

namespace {

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

template <int IN_DT>
__global__ void __launch_bounds__(512) mfma_probe_kernel(float* sink, long* clocks, int iters, int random_bits) {
  i32x8_t w[2], x[4];
  // fp8: clear bit 3 of every byte so no byte is the e4m3 NaN pattern; 16-bit: clear the top
  // exponent bit so no element is Inf/NaN.
  const unsigned keep = IN_DT == DT_FP8 ? 0xf7f7f7f7u : 0xbfffbfffu;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 8; ++i) w[t][i] = random_bits ? (int)(probe_hash(threadIdx.x * 64 + t * 8 + i + 1) & keep) : 0;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 8; ++i) x[t][i] = random_bits ? (int)(probe_hash(threadIdx.x * 64 + 32 + t * 8 + i + 1) & keep) : 0;
  f32x16_t acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;
  const long c0 = clock64(), t0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        if constexpr (IN_DT == DT_FP8) {
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w[a], x[b], acc[a][b], 0, 0, 0, 0, 0, 0);
        } else {
          const i32x4_t wl = {w[a][0], w[a][1], w[a][2], w[a][3]}, xl = {x[b][0], x[b][1], x[b][2], x[b][3]};
          if constexpr (IN_DT == DT_BF16)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wl), __builtin_bit_cast(bf16x8_t, xl), acc[a][b], 0, 0, 0);
          else
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, wl), __builtin_bit_cast(f16x8_t, xl), acc[a][b], 0, 0, 0);
        }
      }
  }
  const long c1 = clock64(), t1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) s += acc[a][b][i];
  sink[blockIdx.x * 512 + threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) { clocks[0] = c1 - c0; clocks[1] = t1 - t0; }
}

}  // namespace

hipError_t run_mfma_probe(int dtype, int random_bits, int iters, double* tflops, double* ghz, hipStream_t st) {
  int dev = 0, ncu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  float* sink = nullptr;
  long* clocks = nullptr;
  e = hipMalloc((void**)&sink, (size_t)ncu * 512 * sizeof(float));
  if (e != hipSuccess) return e;
  e = hipMalloc((void**)&clocks, 2 * sizeof(long));
  if (e != hipSuccess) { (void)hipFree(sink); return e; }
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  auto launch = [&](int n) {
    if (dtype == DT_FP8) hipLaunchKernelGGL((mfma_probe_kernel<DT_FP8>), dim3(ncu), dim3(512), 0, st, sink, clocks, n, random_bits);
    else if (dtype == DT_F16) hipLaunchKernelGGL((mfma_probe_kernel<DT_F16>), dim3(ncu), dim3(512), 0, st, sink, clocks, n, random_bits);
    else hipLaunchKernelGGL((mfma_probe_kernel<DT_BF16>), dim3(ncu), dim3(512), 0, st, sink, clocks, n, random_bits);
  };
  launch(iters / 4 + 1);  // warm-up, also lets the clock settle under load
  (void)hipEventRecord(e0, st);
  launch(iters);
  (void)hipEventRecord(e1, st);
  e = hipStreamSynchronize(st);
  if (e == hipSuccess) e = hipGetLastError();
  float ms = 0.f;
  long h[2] = {0, 1};
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  if (e == hipSuccess) e = hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  (void)hipFree(clocks);
  if (e != hipSuccess) return e;
  const double flop_per_mfma = 2.0 * 32 * 32 * (dtype == DT_FP8 ? 64 : 16);
  *tflops = (double)ncu * 8 * iters * 8 * flop_per_mfma / (ms * 1e-3) / 1e12;
  *ghz = h[1] > 0 ? (double)h[0] / (double)h[1] * 0.1 : 0.0;  // wall counter ticks at 100 MHz
  return hipSuccess;
}

}  // namespace crl
