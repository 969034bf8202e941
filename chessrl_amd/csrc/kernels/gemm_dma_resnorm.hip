// The residual-normalising instance of the 256x256 GEMM (e4m3 operands, bf16 output and residual), in a translation
// unit of its own so that the other instances stay where they were measured.
#include "gemm_dma_kernel.hpp"

namespace crl {

hipError_t launch_gemm_dma_resnorm(const GemmArgs& a, hipStream_t st) { return launch_dma<DmaCfg2, DT_FP8, DT_BF16, 2>(a, st); }

}  // namespace crl
