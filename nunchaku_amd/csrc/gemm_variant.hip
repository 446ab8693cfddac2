// One translation unit per GEMM variant: compiled with -DSVDQ_VARIANT=0..5 so that the six kernels
// build in parallel.  Variant = 2 * kind + next, kind 0: INT4 signed activations, 1: INT4 unsigned
// activations, 2: NVFP4.
#include "gemm_kernel.h"

namespace svdq {

#define SVDQ_KIND (SVDQ_VARIANT / 2)
#define SVDQ_NEXT (SVDQ_VARIANT % 2 == 1)

#if SVDQ_KIND == 0
#define SVDQ_LAUNCH_NAME launch_gemm_int4
#elif SVDQ_KIND == 1
#define SVDQ_LAUNCH_NAME launch_gemm_int4u
#else
#define SVDQ_LAUNCH_NAME launch_gemm_fp4
#endif
#define SVDQ_CAT2(a, b) a##b
#define SVDQ_CAT(a, b) SVDQ_CAT2(a, b)

int SVDQ_CAT(SVDQ_LAUNCH_NAME, SVDQ_CAT(_v, SVDQ_VARIANT))(const GemmParams &p, int nwg, hipStream_t stream) {
    return launch_gemm_variant<SVDQ_KIND == 1, SVDQ_KIND == 2, SVDQ_NEXT>(p, nwg, stream);
}

}  // namespace svdq
