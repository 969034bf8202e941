// Launches of the 256x256 direct-to-LDS GEMM (gemm_dma_kernel.hpp), all instances but the residual-normalising one.
#include "gemm_dma_kernel.hpp"

namespace crl {

hipError_t launch_gemm_dma(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st) {
  if (a.res_stats) {
    // The residual-normalising epilogue exists for the case that uses it: e4m3 operands, bf16 output and residual.
    if (in_dt != DT_FP8 || out_dt != DT_BF16 || !a.res || a.res_dtype != DT_BF16 || !a.res_gamma || a.res_rows > 0 || a.alpha == 0.f || (a.M & 1))
      return hipErrorInvalidValue;
    return launch_gemm_dma_resnorm(a, st);
  }
#define DMA_OUT(IN)                                                        \
  switch (out_dt) {                                                        \
    case DT_F32: return launch_dma<DmaCfg2, IN, DT_F32>(a, st);            \
    case DT_BF16: return launch_dma<DmaCfg2, IN, DT_BF16>(a, st);          \
    case DT_F16: return launch_dma<DmaCfg2, IN, DT_F16>(a, st);            \
    case DT_FP8: return launch_dma<DmaCfg2, IN, DT_FP8>(a, st);            \
  }                                                                        \
  return hipErrorInvalidValue
  if (in_dt == DT_BF16) { DMA_OUT(DT_BF16); }
  if (in_dt == DT_F16) { DMA_OUT(DT_F16); }
  if (in_dt == DT_FP8) { DMA_OUT(DT_FP8); }
#undef DMA_OUT
  return hipErrorInvalidValue;
}

}  // namespace crl
