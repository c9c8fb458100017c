// Instantiations of the 256 x 256 bf16 tile kernel (gmm_tile256.h).
#include "gmm_tile256.h"

namespace dmoe {

int launch_direct_bf16_256(const GmmArgs &args, bool trans_b, bool swiglu, hipStream_t stream) {
    if (trans_b) return swiglu ? launch_tile256_one<true, true>(args, stream) : launch_tile256_one<true, false>(args, stream);
    return swiglu ? launch_tile256_one<false, true>(args, stream) : launch_tile256_one<false, false>(args, stream);
}

// The gate-up projection on rows fetched through args.a_rows ([K, N] weights, fused SiLU * up).
int launch_tile256_rows(const GmmArgs &args, hipStream_t stream) { return launch_tile256_one<false, true, true>(args, stream); }

}  // namespace dmoe
