// Instantiations of the global -> LDS grouped GEMM kernel (gmm_direct.h) for fp8 e4m3 operands.
#include "gmm_direct.h"

namespace dmoe {

// Preconditions: e4m3 operands, K-contiguous on both sides, K % 64 == 0, N % 8 == 0, K * N < 2^32.
int launch_direct_fp8(const GmmArgs &args, int tile_rows, bool swiglu, hipStream_t stream) {
    if (tile_rows == 64) return swiglu ? launch_direct_one<64, 4, 1, true, true, true>(args, stream) : launch_direct_one<64, 4, 1, true, false, true>(args, stream);
    // 256-row tiles: on 4 wavefronts they would need 256 accumulator + 96 operand registers per lane plus addressing;
    // on 8 wavefronts a wavefront holds 128 + 48
    // whole k-steps of 128: the tile that copies whole 128-byte lines (gmm_tile256_fp8.h)
    if (tile_rows == 256 && args.K % 128 == 0) return launch_tile256_fp8(args, swiglu, stream);
    if (tile_rows == 256) return swiglu ? launch_direct_one<256, 8, 2, true, true, true>(args, stream) : launch_direct_one<256, 8, 2, true, false, true>(args, stream);
    return swiglu ? launch_direct_one<128, 4, 2, true, true, true>(args, stream) : launch_direct_one<128, 4, 2, true, false, true>(args, stream);
}

}  // namespace dmoe
