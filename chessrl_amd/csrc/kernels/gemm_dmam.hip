// Instances of the 128x128 and 64x64 GEMMs fed by direct-to-LDS loads through a ring of stages (gemm_dmam_kernel.hpp), in a
// translation unit of their own.
#include "gemm_dmam_kernel.hpp"

namespace crl {

// false: no instance for this combination (the caller keeps the register-staged kernel).
bool gemm_dmam_has(int in_dt, int out_dt) {
  if (in_dt == DT_FP8) return out_dt == DT_BF16 || out_dt == DT_F16 || out_dt == DT_FP8;
  if (in_dt == DT_BF16 && out_dt == DT_F32) return true;   // (an fp32 residual stream, fp32 logits)
  return in_dt == out_dt && (in_dt == DT_BF16 || in_dt == DT_F16);
}

template <typename S>
static hipError_t launch_small(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st) {
  if (in_dt == DT_FP8) {
    switch (out_dt) {
      case DT_BF16: return launch_dmam<DT_FP8, DT_BF16, 0, S>(a, st);
      case DT_F16: return launch_dmam<DT_FP8, DT_F16, 0, S>(a, st);
      case DT_FP8: return launch_dmam<DT_FP8, DT_FP8, 0, S>(a, st);
    }
  }
  if (in_dt == DT_BF16 && out_dt == DT_BF16) return launch_dmam<DT_BF16, DT_BF16, 0, S>(a, st);
  if (in_dt == DT_F16 && out_dt == DT_F16) return launch_dmam<DT_F16, DT_F16, 0, S>(a, st);
  if (in_dt == DT_BF16 && out_dt == DT_F32) return launch_dmam<DT_BF16, DT_F32, 0, S>(a, st);
  return hipErrorInvalidValue;
}

// tile_size: 128 (four stages), 64 (eight) or 32 (sixteen).
hipError_t launch_gemm_dmam(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st, int tile_size) {
  if (tile_size == 64) return launch_small<DmamCfgT<64>>(a, in_dt, out_dt, st);
  if (tile_size == 32) return launch_small<DmamCfgT<32>>(a, in_dt, out_dt, st);
  // (whole tiles in M, aligned rows, a bf16 residual or none, no maximum: the instances without the epilogue's guards)
  const bool lean = a.M % DmamCfg::BM == 0 && a.vec_ok && a.N % 8 == 0 && a.nsplit % 8 == 0 && !a.amax && a.res_rows == 0 && !a.ln_out &&
                    (!a.res || a.res_dtype == DT_BF16);
  if (lean && in_dt == DT_FP8 && out_dt == DT_BF16) return launch_dmam<DT_FP8, DT_BF16, 1>(a, st);
  if (lean && in_dt == DT_FP8 && out_dt == DT_FP8) return launch_dmam<DT_FP8, DT_FP8, 1>(a, st);
  if (lean && in_dt == DT_BF16 && out_dt == DT_BF16) return launch_dmam<DT_BF16, DT_BF16, 1>(a, st);
  if (in_dt == DT_FP8) {
    switch (out_dt) {
      case DT_BF16: return launch_dmam<DT_FP8, DT_BF16>(a, st);
      case DT_F16: return launch_dmam<DT_FP8, DT_F16>(a, st);
      case DT_FP8: return launch_dmam<DT_FP8, DT_FP8>(a, st);
    }
  }
  if (in_dt == DT_BF16 && out_dt == DT_BF16) return launch_dmam<DT_BF16, DT_BF16>(a, st);
  if (in_dt == DT_F16 && out_dt == DT_F16) return launch_dmam<DT_F16, DT_F16>(a, st);
  if (in_dt == DT_BF16 && out_dt == DT_F32) return launch_dmam<DT_BF16, DT_F32>(a, st);
  return hipErrorInvalidValue;
}

}  // namespace crl
