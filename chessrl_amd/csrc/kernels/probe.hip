// Measurement probe: the rate the matrix cores sustain when nothing else runs.
//
// Every CU gets one workgroup of 8 waves (2 per SIMD) whose lanes keep a 2x4 grid of 32x32
// accumulator tiles and issue MFMAs back to back from operands held in registers: no LDS,
// no memory, no barrier. With all-zero operands the result is the clock-limited peak; with
// random operand bits the sustained clock drops under the board's power limit, so the rate
// is the ceiling any real GEMM on this part works under. The kernel also reads the shader
// clock counter and the 100 MHz wall counter to report the clock it actually ran at.
#include "common.hpp"
#include "gemm_tile.hpp"

#include <cstring>

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

// Second probe: can the memory-bound kernels of a pass run BESIDE its products on disjoint sets of CUs?
// Two streams with CU masks (the first `gemm_cus` mask bits / the rest; mask bits go round the XCDs, so both sets are
// spread evenly over them) run the e4m3 product of one trunk linear (M x 1024 x 1024, bf16 output) and the trunk
// LayerNorm (M rows of 1024, bf16 in, e4m3 out), each alone on all CUs, alone on its share, and side by side with launch
// counts chosen so that both streams are busy for about the same time.
//   out[0] product, all CUs (us)        out[1] product on its share     out[2] product beside the norm
//   out[3] norm, all CUs (us)           out[4] norm on its share        out[5] norm beside the product
//   out[6] side by side: wall time of both streams (ms)
//   out[7] the same launches back to back on all CUs (ms, from out[0] and out[3])
namespace {
__global__ void probe_fill_kernel(uint32_t* p, long n, uint32_t keep, uint32_t set) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    p[i] = (probe_hash((unsigned)i * 2654435761u + 17u) & keep) | set;
}
}  // namespace

hipError_t run_cu_split_probe(int gemm_cus, int tile, int rows, int iters, double* out) {
  // gemm_cus == 256: no masks, two plain streams that share every CU
  if (gemm_cus < 8 || (gemm_cus > 248 && gemm_cus != 256) || rows < 256 || rows % 256 || iters < 1) return hipErrorInvalidValue;
  const int N = 1024, K = 1024;
  hipError_t e = hipSuccess;
  uint8_t *A = nullptr, *W = nullptr, *X8 = nullptr;
  uint16_t *C = nullptr, *X = nullptr;
  float *g = nullptr, *b = nullptr;
  hipStream_t sAll = nullptr, sG = nullptr, sH = nullptr;
  hipEvent_t ev[4] = {};
#define PROBE_TRY(call) do { e = (call); if (e != hipSuccess) goto done; } while (0)
  {
    uint32_t mg[8] = {}, mh[8] = {};
    for (int i = 0; i < 256; ++i) (i < gemm_cus ? mg : mh)[i / 32] |= 1u << (i % 32);
    PROBE_TRY(hipStreamCreateWithFlags(&sAll, hipStreamNonBlocking));
    if (gemm_cus == 256) {
      PROBE_TRY(hipStreamCreateWithFlags(&sG, hipStreamNonBlocking));
      PROBE_TRY(hipStreamCreateWithFlags(&sH, hipStreamNonBlocking));
    } else {
      PROBE_TRY(hipExtStreamCreateWithCUMask(&sG, 8, mg));
      PROBE_TRY(hipExtStreamCreateWithCUMask(&sH, 8, mh));
    }
    for (auto& v : ev) PROBE_TRY(hipEventCreate(&v));
    PROBE_TRY(hipMalloc((void**)&A, (size_t)rows * K));
    PROBE_TRY(hipMalloc((void**)&W, (size_t)N * K));
    PROBE_TRY(hipMalloc((void**)&C, (size_t)rows * N * 2));
    PROBE_TRY(hipMalloc((void**)&X, (size_t)rows * N * 2));
    PROBE_TRY(hipMalloc((void**)&X8, (size_t)rows * N));
    PROBE_TRY(hipMalloc((void**)&g, N * sizeof(float)));
    PROBE_TRY(hipMalloc((void**)&b, N * sizeof(float)));
    // e4m3 operands with random sign and mantissa, exponents below the NaN pattern; bf16 rows of magnitude ~1
    hipLaunchKernelGGL(probe_fill_kernel, dim3(1024), dim3(256), 0, sAll, (uint32_t*)A, (long)rows * K / 4, 0xb7b7b7b7u, 0u);
    hipLaunchKernelGGL(probe_fill_kernel, dim3(256), dim3(256), 0, sAll, (uint32_t*)W, (long)N * K / 4, 0xb7b7b7b7u, 0u);
    hipLaunchKernelGGL(probe_fill_kernel, dim3(1024), dim3(256), 0, sAll, (uint32_t*)X, (long)rows * N / 2, 0x80ff80ffu, 0x3f003f00u);
    PROBE_TRY(launch_fill_f32(g, 1.f, N, sAll));
    PROBE_TRY(launch_fill_f32(b, 0.f, N, sAll));
    PROBE_TRY(hipStreamSynchronize(sAll));
    GemmArgs ga;
    std::memset(&ga, 0, sizeof(ga));
    ga.A = A; ga.lda = K; ga.W = W; ga.ldw = K; ga.C = C; ga.ldc = N; ga.M = rows; ga.N = N; ga.K = K; ga.nsplit = N;
    ga.descale = 1e-3f; ga.alpha = 1.f; ga.out_scale = 1.f;
    LayerNormArgs la;
    std::memset(&la, 0, sizeof(la));
    la.x = X; la.ldx = N; la.in_dtype = DT_BF16; la.gamma = g; la.beta = b; la.out_fp8 = X8; la.fp8_scale = 16.f; la.ldo = N;
    la.rows = rows; la.C = N; la.eps = 1e-5f; la.out_dtype = DT_BF16;
    auto gemm = [&](hipStream_t s) { return launch_gemm(ga, DT_FP8, DT_BF16, tile, s); };
    auto norm = [&](hipStream_t s) { return launch_layernorm(la, s); };
    auto time_alone = [&](hipStream_t s, int n, bool is_gemm, double* us) -> hipError_t {
      hipError_t te = hipSuccess;
      for (int i = 0; i < 3 && te == hipSuccess; ++i) te = is_gemm ? gemm(s) : norm(s);
      if (te == hipSuccess) te = hipEventRecord(ev[0], s);
      for (int i = 0; i < n && te == hipSuccess; ++i) te = is_gemm ? gemm(s) : norm(s);
      if (te == hipSuccess) te = hipEventRecord(ev[1], s);
      if (te == hipSuccess) te = hipStreamSynchronize(s);
      float ms = 0.f;
      if (te == hipSuccess) te = hipEventElapsedTime(&ms, ev[0], ev[1]);
      *us = ms * 1e3 / n;
      return te;
    };
    PROBE_TRY(time_alone(sAll, iters, true, &out[0]));
    PROBE_TRY(time_alone(sG, iters, true, &out[1]));
    PROBE_TRY(time_alone(sAll, 2 * iters, false, &out[3]));
    PROBE_TRY(time_alone(sH, 2 * iters, false, &out[4]));
    // side by side: `iters` products on their share, norms on theirs for about as long, issued interleaved
    const int nl = (int)(iters * out[1] / out[4]) + 1;
    PROBE_TRY(hipDeviceSynchronize());
    PROBE_TRY(hipEventRecord(ev[0], sG));
    PROBE_TRY(hipEventRecord(ev[2], sH));
    for (int i = 0, il = 0; i < iters; ++i) {
      PROBE_TRY(gemm(sG));
      for (; il < (long)(i + 1) * nl / iters; ++il) PROBE_TRY(norm(sH));
    }
    PROBE_TRY(hipEventRecord(ev[1], sG));
    PROBE_TRY(hipEventRecord(ev[3], sH));
    PROBE_TRY(hipDeviceSynchronize());
    float mg_ms = 0.f, ml_ms = 0.f;
    PROBE_TRY(hipEventElapsedTime(&mg_ms, ev[0], ev[1]));
    PROBE_TRY(hipEventElapsedTime(&ml_ms, ev[2], ev[3]));
    out[2] = mg_ms * 1e3 / iters;
    out[5] = ml_ms * 1e3 / nl;
    out[6] = mg_ms > ml_ms ? mg_ms : ml_ms;
    out[7] = (iters * out[0] + nl * out[3]) * 1e-3;
  }
done:
#undef PROBE_TRY
  (void)hipDeviceSynchronize();
  for (auto& v : ev) if (v) (void)hipEventDestroy(v);
  if (sAll) (void)hipStreamDestroy(sAll);
  if (sG) (void)hipStreamDestroy(sG);
  if (sH) (void)hipStreamDestroy(sH);
  (void)hipFree(A); (void)hipFree(W); (void)hipFree(C); (void)hipFree(X); (void)hipFree(X8); (void)hipFree(g); (void)hipFree(b);
  return e;
}

}  // namespace crl
