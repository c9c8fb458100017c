// Dispatch of the global -> LDS grouped GEMM kernel (gmm_direct.h) for bf16 operands by tile rows; the instantiations
// live in translation units of their own so that the library builds in parallel.
#include "gmm_common.h"

namespace dmoe {

int launch_direct_bf16_small(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream);
int launch_direct_bf16_256(const GmmArgs &args, bool trans_b, bool swiglu, hipStream_t stream);

// Preconditions (checked by the caller): bf16, K % 32 == 0, N % 8 == 0, K * N * 2 < 2^32.
// tile_rows: 256 (gmm_tile256.h), 128 (4 wavefronts) or 64 (4 computing + 2 copying wavefronts) (gmm_direct.h).
int launch_direct_bf16(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream) {
    if (tile_rows == 64 || tile_rows == 128) return launch_direct_bf16_small(args, tile_rows, trans_b, swiglu, stream);
    return launch_direct_bf16_256(args, trans_b, swiglu, stream);
}

}  // namespace dmoe
