// One translation unit per variant of the INT4 GEMM (compiled with -DSVDQ_VARIANT=0: plain epilogue,
// 1: with the next-layer / norm + rotary / SiLU epilogue) so that they build in parallel.
#include "gemm6_kernel.h"

namespace svdq {
namespace g6 {

#if SVDQ_VARIANT == 0
int launch_plain(const Params &p, int nwg, hipStream_t stream) { return launch_gemm6<false>(p, nwg, stream); }
#else
int launch_next(const Params &p, int nwg, hipStream_t stream) { return launch_gemm6<true>(p, nwg, stream); }
#endif

}  // namespace g6
}  // namespace svdq
