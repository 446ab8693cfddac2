// One translation unit per variant of the NVFP4 GEMM (compiled with -DSVDQ_VARIANT=4: plain epilogue,
// 5: with the next-layer / norm + rotary / SiLU epilogue) so that they build in parallel.
#include "gemm_kernel.h"

namespace svdq {

#if SVDQ_VARIANT == 4
int launch_gemm_fp4_v4(const GemmParams &p, int nwg, hipStream_t stream) { return launch_gemm_variant<false>(p, nwg, stream); }
#else
int launch_gemm_fp4_v5(const GemmParams &p, int nwg, hipStream_t stream) { return launch_gemm_variant<true>(p, nwg, stream); }
#endif

}  // namespace svdq
