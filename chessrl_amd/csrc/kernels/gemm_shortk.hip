// Instances of the GEMM for K = 256 e4m3 operands whose workgroups keep their A rows in registers and walk N
// (gemm_shortk_kernel.hpp), in a translation unit of their own.
#include "gemm_shortk_kernel.hpp"

namespace crl {

// What the kernel takes: a bare scaled product into one 16-bit output too large to stay in the caches, K = 256 e4m3
// elements, M in whole blocks of 256 rows, N in whole steps of 128 columns, 16-byte aligned rows; the blocked output
// layout needs ldc == N.
bool gemm_shortk_can(const GemmArgs& a, int in_dt, int out_dt) {
  if (in_dt != DT_FP8 || (out_dt != DT_BF16 && out_dt != DT_F16)) return false;
  if (a.K != 256 || a.N % ShortKCfg::BN != 0 || a.M <= 0 || a.M % ShortKCfg::BM != 0) return false;
  if ((long)a.M * a.N * 2 <= (64L << 20)) return false;   // (its stores bypass the caches; smaller products are faster through the tiled kernels)
  if (a.bias || a.res || a.amax || a.act != ACT_NONE || a.alpha != 1.f || a.nsplit < a.N || a.ln_out || a.res_stats || a.k_slices > 1) return false;
  if (a.lda % 16 != 0 || a.ldw % 16 != 0 || a.ldc % 8 != 0 || (a.c_blocked && a.ldc != a.N)) return false;
  if ((reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.W) | reinterpret_cast<uintptr_t>(a.C)) & 15) return false;
  return (long)a.N * a.ldw < (1L << 31) && (long)ShortKCfg::BM * a.ldc * 2 < (1L << 31);
}

hipError_t launch_gemm_shortk(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st) {
  if (!gemm_shortk_can(a, in_dt, out_dt)) return hipErrorInvalidValue;
  return out_dt == DT_BF16 ? launch_shortk<DT_BF16>(a, st) : launch_shortk<DT_F16>(a, st);
}

}  // namespace crl
