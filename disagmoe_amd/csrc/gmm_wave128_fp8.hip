// Instantiations of the 256 x 256 fp8 tile kernel on 4 wavefronts of 128 x 128 (gmm_wave128_fp8.h).
#include "gmm_wave128_fp8.h"

namespace dmoe {

// Preconditions: e4m3 operands, K-contiguous on both sides, K % 128 == 0, N % 8 == 0, K * N < 2^32.
int launch_wave128_fp8(const GmmArgs &args, bool swiglu, hipStream_t stream) {
    return swiglu ? launch_wave128_fp8_one<true>(args, stream) : launch_wave128_fp8_one<false>(args, stream);
}

}  // namespace dmoe
