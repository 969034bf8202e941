// Instances of the eight-wave 256x256 GEMM with address arithmetic kept out of its main loop (gemm_dmaf_kernel.hpp), in
// a translation unit of their own.
#include "gemm_dmaf_kernel.hpp"

namespace crl {

// false: no instance for this combination (the caller falls back to gemm_dma_kernel.hpp).
bool gemm_dmaf_has(int in_dt, int out_dt, bool res_norm) {
  if (res_norm) return in_dt == DT_FP8 && out_dt == DT_BF16;
  if (in_dt == DT_FP8) return out_dt == DT_BF16 || out_dt == DT_F16 || out_dt == DT_FP8;
  return in_dt == out_dt && (in_dt == DT_BF16 || in_dt == DT_F16);
}

hipError_t launch_gemm_dmaf(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st) {
  if (a.res_stats) {
    if (in_dt != DT_FP8 || out_dt != DT_BF16 || !a.res || a.res_dtype != DT_BF16 || !a.res_gamma || a.res_rows > 0 || a.alpha == 0.f || (a.M & 1))
      return hipErrorInvalidValue;
    return dmaf_lean_ok(a) ? launch_dmaf<DT_FP8, DT_BF16, 2, true>(a, st) : launch_dmaf<DT_FP8, DT_BF16, 2>(a, st);
  }
  // (whole tiles in M, aligned rows, a bf16 residual or none, no maximum: the instances without the epilogue's guards)
  const bool lean = dmaf_lean_ok(a);
  if (in_dt == DT_FP8) {
    switch (out_dt) {
      case DT_BF16: return lean ? launch_dmaf<DT_FP8, DT_BF16, 0, true>(a, st) : launch_dmaf<DT_FP8, DT_BF16, 0>(a, st);
      case DT_F16: return launch_dmaf<DT_FP8, DT_F16, 0>(a, st);
      case DT_FP8: return lean ? launch_dmaf<DT_FP8, DT_FP8, 0, true>(a, st) : launch_dmaf<DT_FP8, DT_FP8, 0>(a, st);
    }
  }
  if (in_dt == DT_BF16 && out_dt == DT_BF16) return lean ? launch_dmaf<DT_BF16, DT_BF16, 0, true>(a, st) : launch_dmaf<DT_BF16, DT_BF16, 0>(a, st);
  if (in_dt == DT_F16 && out_dt == DT_F16) return launch_dmaf<DT_F16, DT_F16, 0>(a, st);
  return hipErrorInvalidValue;
}

}  // namespace crl
