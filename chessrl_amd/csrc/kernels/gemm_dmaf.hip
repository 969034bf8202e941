// Instances of the eight-wave 256x256 GEMM with address arithmetic kept out of its main loop (gemm_dmaf_kernel.hpp), in
// a translation unit of their own.
#include "gemm_dmaf_kernel.hpp"

namespace crl {

// false: no instance for this combination (the caller falls back to gemm_dma_kernel.hpp).
bool gemm_dmaf_has(int in_dt, int out_dt, bool res_norm) {
  if (res_norm) return in_dt == DT_FP8 && out_dt == DT_BF16;
  if (in_dt == DT_FP8) return out_dt == DT_BF16 || out_dt == DT_F16 || out_dt == DT_FP8;
  if (in_dt == DT_BF16 && out_dt == DT_F32) return true;   // (an fp32 residual stream, fp32 logits)
  return in_dt == out_dt && (in_dt == DT_BF16 || in_dt == DT_F16);
}

hipError_t launch_gemm_dmaf(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st) {
  if (a.res_stats) {
    if (in_dt != DT_FP8 || out_dt != DT_BF16 || !a.res || a.res_dtype != DT_BF16 || !a.res_gamma || a.res_rows > 0 || a.alpha == 0.f || (a.M & 1))
      return hipErrorInvalidValue;
    switch (dmaf_lean_level(a, out_dt, true)) {
      case 2: return launch_dmaf<DT_FP8, DT_BF16, 2, 2>(a, st);
      case 1: return launch_dmaf<DT_FP8, DT_BF16, 2, 1>(a, st);
    }
    return launch_dmaf<DT_FP8, DT_BF16, 2>(a, st);
  }
  // (whole tiles in M, aligned rows, a bf16 residual or none, no maximum: the instances without the epilogue's guards)
  const int lean = dmaf_lean_level(a, out_dt, false);
  if (in_dt == DT_FP8) {
    switch (out_dt) {
      case DT_BF16:
        if (lean == 2 && dmaf_xtra_ok(a)) return launch_dmaf<DT_FP8, DT_BF16, 0, 2, 1>(a, st);
        return lean == 2 ? launch_dmaf<DT_FP8, DT_BF16, 0, 2>(a, st) : lean == 1 ? launch_dmaf<DT_FP8, DT_BF16, 0, 1>(a, st) : launch_dmaf<DT_FP8, DT_BF16, 0>(a, st);
      case DT_F16: return launch_dmaf<DT_FP8, DT_F16, 0>(a, st);
      case DT_FP8: return lean == 2 ? launch_dmaf<DT_FP8, DT_FP8, 0, 2>(a, st) : lean == 1 ? launch_dmaf<DT_FP8, DT_FP8, 0, 1>(a, st) : launch_dmaf<DT_FP8, DT_FP8, 0>(a, st);
    }
  }
  if (in_dt == DT_BF16 && out_dt == DT_BF16) return lean == 2 ? launch_dmaf<DT_BF16, DT_BF16, 0, 2>(a, st) : lean == 1 ? launch_dmaf<DT_BF16, DT_BF16, 0, 1>(a, st) : launch_dmaf<DT_BF16, DT_BF16, 0>(a, st);
  if (in_dt == DT_F16 && out_dt == DT_F16) return launch_dmaf<DT_F16, DT_F16, 0>(a, st);
  if (in_dt == DT_BF16 && out_dt == DT_F32) return launch_dmaf<DT_BF16, DT_F32, 0>(a, st);
  return hipErrorInvalidValue;
}

}  // namespace crl
