// Instantiations of the global -> LDS grouped GEMM kernel (gmm_direct.h) for bf16 operands: the 256-row tile, on 8
// wavefronts whose two wavefronts per SIMD alternate between a memory phase and a matrix phase.
#include "gmm_direct.h"

namespace dmoe {

int launch_direct_bf16_256(const GmmArgs &args, bool trans_b, bool swiglu, hipStream_t stream) {
    return launch_direct_tile<256, 8, 2, 0, 1>(args, trans_b, swiglu, stream);
}

}  // namespace dmoe
