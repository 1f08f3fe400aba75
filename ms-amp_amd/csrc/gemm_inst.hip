// One pair of operand formats of the FP8 GEMM kernels (compiled four times: -DMSAMP_XF=5|6 -DMSAMP_YF=5|6), and once more
// per pair with -DMSAMP_GEMM_SPLIT_UNIT for the split-wait instantiations alone, so that the eight units compile side by side.
#include "gemm_kernels.cuh"

namespace msamp {
#ifdef MSAMP_GEMM_SPLIT_UNIT
template int run_gemm_split<MSAMP_XF, MSAMP_YF>(MSAMP_SPLIT_ARGS);
#else
template int run_gemm_pair<MSAMP_XF, MSAMP_YF>(const GemmCall&);
#endif
}    // namespace msamp
