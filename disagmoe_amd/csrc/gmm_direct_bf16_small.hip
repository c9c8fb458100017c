// Instantiations of the global -> LDS grouped GEMM kernel (gmm_direct.h) for bf16 operands: the 64- and 128-row tiles
// (a translation unit of their own so that the library builds in parallel).
#include "gmm_direct.h"

namespace dmoe {

int launch_direct_bf16_small(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream) {
    if (tile_rows == 64) return launch_direct_tile<64, 4, 1, 2>(args, trans_b, swiglu, stream);   // 4 + 2 copying wavefronts
    return launch_direct_tile<128, 4, 2>(args, trans_b, swiglu, stream);
}

}  // namespace dmoe
