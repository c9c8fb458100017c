// Hook of the library's own tests and benchmarks; not part of the public ABI (include/dmoe.h), no counterpart in
// the reference.  Forces the grouped GEMM's kernel and tile shape, process-wide and unsynchronised: 0 = choose from
// the rows per expert (default); 1 = register-staged 256x256 tile on 4 wavefronts; 2 = 64x256; 3 = 128x256;
// 4 = register-staged 256x256 tile on 8 wavefronts; 5, 6, 7 = the global -> LDS kernels with tiles of 64, 128, 256
// rows whatever the rows per expert; 8 = 256-row tiles on 4 wavefronts of 128 x 128 (bf16, [K, N] weights; 7 elsewhere).
#pragma once

extern "C" int dmoe_gmm_tune(int variant);

// What a launch with these shapes would run: kernel, tile rows, grid and (with the batch sizes in host memory) the
// split of the last round, as the library itself derives them; for the benchmark's labels and the tests' expectations.
// launch_has_sizes: the launch is given the host sizes as well (host_batch_sizes of dmoe_gmm*) and decides with them.
extern "C" int dmoe_gmm_plan(const int64_t *host_batch_sizes, int launch_has_sizes, int64_t rows, int E, int64_t K, int64_t N,
                             int trans_b, int swiglu, int dtype, size_t workspace_bytes, int64_t *out);
