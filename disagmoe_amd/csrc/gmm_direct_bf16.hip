// Instantiations of the global -> LDS grouped GEMM kernel (gmm_direct.h) for bf16 operands: the 256-row tiles.
#include "gmm_direct.h"

namespace dmoe {

int launch_direct_bf16_small(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream);

// Preconditions (checked by the caller): bf16, K % 32 == 0, N % 8 == 0, K * N * 2 < 2^32.
// tile_rows: 256 (8 wavefronts), 128 (4 wavefronts) or 64 (4 computing + 2 copying wavefronts); 260 = 256 rows on 4
// wavefronts (comparison).
int launch_direct_bf16(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream) {
    if (tile_rows == 64 || tile_rows == 128) return launch_direct_bf16_small(args, tile_rows, trans_b, swiglu, stream);
    if (tile_rows == 260) return launch_direct_tile<256, 4, 2>(args, trans_b, swiglu, stream);   // 256 rows on 4 wavefronts
    return launch_direct_tile<256, 8, 2>(args, trans_b, swiglu, stream);
}

}  // namespace dmoe
