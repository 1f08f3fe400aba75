// One pair of operand formats of the FP8 GEMM kernels (compiled four times: -DMSAMP_XF=5|6 -DMSAMP_YF=5|6).
#include "gemm_kernels.cuh"

namespace msamp {
template int run_gemm_pair<MSAMP_XF, MSAMP_YF>(const GemmCall&);
}    // namespace msamp
