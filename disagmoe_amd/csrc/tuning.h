// Hook of the library's own tests and benchmarks; not part of the public ABI (include/dmoe.h), no counterpart in
// the reference.  Forces the grouped GEMM's kernel and tile shape, process-wide and unsynchronised: 0 = choose from
// the rows per expert (default); 1 = register-staged 256x256 tile on 4 wavefronts; 2 = 64x256; 3 = 128x256;
// 4 = register-staged 256x256 tile on 8 wavefronts; 5, 6, 7 = the global -> LDS kernels with tiles of 64, 128, 256
// rows whatever the rows per expert.
#pragma once

extern "C" int dmoe_gmm_tune(int variant);
