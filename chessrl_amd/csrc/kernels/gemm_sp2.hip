// Instances of the four-wave software-pipelined 256x256 e4m3 GEMM fed in 128-byte slabs (gemm_sp2_kernel.hpp), in a
// translation unit of their own.
#include "gemm_sp2_kernel.hpp"

namespace crl {

hipError_t launch_gemm_sp2(const GemmArgs& a, int out_dt, hipStream_t st) {
  if (a.res_stats) {
    if (out_dt != DT_BF16 || !a.res || a.res_dtype != DT_BF16 || !a.res_gamma || a.res_rows > 0 || a.alpha == 0.f || (a.M & 1))
      return hipErrorInvalidValue;
    return launch_sp2<DT_BF16, 2>(a, st);
  }
  switch (out_dt) {
    case DT_BF16: return launch_sp2<DT_BF16, 0>(a, st);
    case DT_F16: return launch_sp2<DT_F16, 0>(a, st);
    case DT_FP8: return launch_sp2<DT_FP8, 0>(a, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace crl
