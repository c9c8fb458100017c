// Instantiations of the 256 x 256 bf16 tile kernel on 4 wavefronts of 128 x 128 (gmm_wave128.h).
#include "gmm_wave128.h"

namespace dmoe {

// Preconditions: bf16, weights [E, K, N], K % 32 == 0, N % 8 == 0, K * N * 2 < 2^32.
int launch_wave128(const GmmArgs &args, bool swiglu, hipStream_t stream) {
    return swiglu ? launch_wave128_one<true>(args, stream) : launch_wave128_one<false>(args, stream);
}

}  // namespace dmoe
