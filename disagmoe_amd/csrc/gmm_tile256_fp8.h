// fp8 (e4m3) grouped GEMM, the 256 x 256 tile on 8 wavefronts with v_mfma_f32_16x16x128_f8f6f4.
//
// Two measurements shape it.  Under MFMA load the chip is power-limited, and a loop of nothing but MFMAs on random fp8
// operands sustains about 4.0 PFLOP/s with the 16x16x128 form against 3.6 with 32x32x64.  And a global -> LDS copy
// instruction whose 64 lanes fetch 8 whole 128-byte lines costs the memory path visibly less than one that fetches 16
// half lines (a main loop of MFMAs, operand reads and the copies of a 4 x 8 patch of tiles per XCD, no other work:
// 2.63 - 2.70 PFLOP/s against 2.11 - 2.17), so a row of a tile is 128 bytes in LDS and every copy brings whole lines.
//
//   * operands are e4m3 bytes, K-contiguous on both sides; scales per row of a and per column of b are applied in the
//     epilogue;
//   * a k-step is 128 k: 32 KiB of A + 32 KiB of B in LDS (rows of 128 bytes), two k-steps resident; an MFMA contracts
//     the 128 k of a row, lane l holding row l % 16 and the 16-byte chunks g and g + 4 of it (g = l / 16; which k a
//     lane multiplies does not matter as long as both operands agree);
//   * chunk c of row r sits at c ^ swizzle(r), swizzle(r) = 4 * bit 1 of r + 2 * bit 2 of r: a probe that timed this
//     read (row = lane % 16 at 128-byte pitch, chunk = lane / 16) for all XOR-linear swizzles found it among those free
//     of bank conflicts (4 cycles per ds_read_b128);
//   * a k-step is two half steps (row fragments 0 - 3, then 4 - 7, 16 MFMAs each), and the two wavefronts of a SIMD
//     alternate between the memory phase and the matrix phase of a half step, one phase apart;
//   * a copy goes out as soon as its place in LDS has been read: the B tile and the A rows of row fragments 0 - 3 of
//     k-step t + 2 in the second memory phase of k-step t, the A rows of row fragments 4 - 7 in the first memory phase
//     of k-step t + 1, so every copy is in flight for a k-step and a half with two buffers (against all of k-step
//     t + 1 in the first memory phase of k-step t: gate-up + 5 %, down + 9 % on the 8x22B shapes).
#pragma once
#include "gmm_tile256.h"

namespace dmoe {

template <bool SWIGLU>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gmm_tile256_fp8_kernel(const GmmArgs p) {
    constexpr int kDM = 256, NW = 8, WN = 4;
    constexpr int TM = 128, TN = 64;
    constexpr int FM = TM / 16, FN = TN / 16;
    constexpr int FNO = SWIGLU ? FN / 2 : FN;
    constexpr int kStepK = 128;                          // k (= bytes per row) of a k-step
    constexpr int kBufA = kDM * kStepK, kBufB = kDN * kStepK;
    constexpr int kBuf = kBufA + kBufB;                  // 64 KiB
    constexpr int kBufs = 2;
    constexpr int CA = kDM / (8 * NW), CB = kDN / (8 * NW);   // copies (8 rows of 128 B each) per wavefront per k-step
    constexpr int kBlock = NW * 1024;
    constexpr int BNO = SWIGLU ? kDN / 2 : kDN;
    static_assert(CA == 4 && CB == 4, "copies per k-step");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int s_tile_start[kMaxGroups + 1];
    __shared__ int s_row_start[kMaxGroups + 1];
    __shared__ long long s_item;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int E = p.E;

    build_work_list<kDM>(p, s_tile_start, s_row_start);
    __syncthreads();

    const int n_out = SWIGLU ? p.N / 2 : p.N;
    const int n_tiles = (n_out + BNO - 1) / BNO;
    const int T_all = p.K / kStepK;                      // k-steps of a whole tile
    const int G = gridDim.x;
    constexpr long long kPieceBytes = (long long)kDM * kDN * sizeof(float);
    // a k-step takes the time of two 32-k stages of the bf16 tile, the unit plan_work's estimates are made in
    const WorkPlan plan = plan_work((long long)s_tile_start[E] * n_tiles, G, 2 * T_all,
                                    p.arrive != nullptr ? p.partial_bytes / kPieceBytes : 0, kWsArriveCount / NW);
    const long long total = plan.items;
    const uint32_t pitch = (uint32_t)p.K;
    const uint32_t smem_addr = lds_addr(smem);
    const int streams = (G % kXcds == 0) ? kXcds : 1;

    auto swizzle = [](int row) { return (((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1); };
    // copies: a 1 KiB block is 8 rows of 128 B; lane l fills row l / 8, physical chunk l % 8 of it, which holds the
    // logical chunk (l % 8) ^ swizzle(row).  Block number i * NW + wave: its rows are 8 (wave & 1) + l / 8 modulo 16.
    const int kc_row = lane >> 3;
    const int kc_chunk = (lane & 7) ^ swizzle((wave & 1) * 8 + kc_row);

    // operand reads: lane l, row l % 16, chunks g and g + 4 (g = l / 16): the second sits 64 bytes from the first
    const int l16 = lane & 15, g16 = lane >> 4;
    const int rd = (g16 ^ swizzle(l16)) << 4;
    const int fa_base = (wm * TM + l16) * kStepK + rd;
    // B fragment j of this wavefront: one base register, the fragments at constant distances
    const int fb_base = kBufA + ((SWIGLU ? wn * (TN / 2) : wn * TN) + l16) * kStepK + rd;
    auto fb_dist = [](int j) {   // bytes from fragment 0 to fragment j
        return (SWIGLU ? ((j < FN / 2) ? j * 16 : kDN / 2 + (j - FN / 2) * 16) : j * 16) * kStepK;
    };

    int e = 0, row0 = 0, rows_e = 0, n0 = 0;
    int t_lo = 0, T = 0;                                 // k-steps [t_lo, t_lo + T) of the tile
    int part = -1, split_tile = 0;
    uint64_t a_base = 0, b_exp = 0;
    uint32_t a_off[CA], b_off[CB];

    auto b_col = [&](int slot) {
        const int rh = (SWIGLU && slot >= kDN / 2) ? slot - kDN / 2 : slot;
        const int base = (SWIGLU && slot >= kDN / 2) ? n_out + n0 : n0;
        return base + (rh < n_out - n0 ? rh : 0);          // slots past the end read a valid column (never stored)
    };
    auto open_tile = [&](long long q) {
        const WorkItem it = decode_item<kDM>(q, G, plan, T_all, n_tiles, E, s_tile_start, s_row_start);
        e = it.tile.e; row0 = it.tile.row0; rows_e = it.tile.rows_e; n0 = it.tile.nt * BNO;
        t_lo = it.s_lo; T = it.s_cnt;
        part = it.piece; split_tile = it.split_tile;
        a_base = to_scalar((uint64_t)(uintptr_t)p.a + (uint64_t)row0 * pitch + (uint64_t)t_lo * kStepK);
        b_exp = to_scalar((uint64_t)(uintptr_t)p.b + (uint64_t)e * p.K * p.N + (uint64_t)t_lo * kStepK);
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            int r = (i * NW + wave) * 8 + kc_row;
            if (r >= rows_e) r = rows_e - 1;               // clamp: loaded, never stored
            a_off[i] = (uint32_t)r * pitch + kc_chunk * 16;
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) b_off[i] = (uint32_t)b_col((i * NW + wave) * 8 + kc_row) * pitch + kc_chunk * 16;
    };
    // The copies of k-step t of the item, in two groups by when their place in LDS is free.  The B tile and the A rows
    // of row fragments 0 - 3 of either half of the tile (this wavefront's blocks 0 and 2) are read in the first memory
    // phase of a k-step, the A rows of row fragments 4 - 7 (blocks 1 and 3) in the second.
    auto issue_early = [&](int t) {
        const uint32_t lds = smem_addr + (t % kBufs) * kBuf + wave * 1024;
        const uint64_t k_off = (uint64_t)t * kStepK;
        static_for<0, CB>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            copy_g2lds_16<kBufA + i * kBlock>(b_off[i], b_exp + k_off, lds);
        });
        copy_g2lds_16<0 * kBlock>(a_off[0], a_base + k_off, lds);
        copy_g2lds_16<2 * kBlock>(a_off[2], a_base + k_off, lds);
    };
    auto issue_late = [&](int t) {
        const uint32_t lds = smem_addr + (t % kBufs) * kBuf + wave * 1024;
        const uint64_t k_off = (uint64_t)t * kStepK;
        copy_g2lds_16<1 * kBlock>(a_off[1], a_base + k_off, lds);
        copy_g2lds_16<3 * kBlock>(a_off[3], a_base + k_off, lds);
    };
    constexpr int kEarly = CB + 2, kLate = 2;
    auto issue_prologue = [&]() {
        issue_early(0);
        issue_late(0);
        if (T > 1) { issue_early(1); issue_late(1); }
    };

    i32x8 fa[FM / 2], fb[FN];
    auto read32 = [&](const char *base, int off, int dist) {   // off: from the start of the buffer; dist: a multiple of 128
        base += dist;
        const u32x4 x0 = *(const u32x4 *)(base + off);
        const u32x4 x1 = *(const u32x4 *)(base + (off ^ 64));      // the lane's second chunk sits 4 chunks away
        return i32x8{(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
    };

    unsigned int draw = 0;
    const bool drawer = tid == 0;
    if (drawer) draw = sched_draw(p.sched, streams);       // always one draw ahead: its round trip hides behind a tile
    long long q = blockIdx.x;                              // the first item needs no draw (see sched_item)
    if (q < total) {
        open_tile(q);
        issue_prologue();
    }

    // Ticks of the 100 MHz clock that a k-step of this workgroup's full tiles takes (0: none finished yet).  A tile with
    // fewer than 256 rows skips the MFMAs of its empty row fragments; left to itself it walks K faster than the tiles
    // beside it that share its weight tile, ends early, and from then on its workgroup draws every tile ahead of its
    // neighbours: the compute units of an XCD fall out of step for the rest of the launch and what they share in
    // principle no longer meets in the 4 MB of their L2 (measured on 8 experts of 4031 .. 4143 rows, K = 6144: tiles
    // start within 2 us of each other inside an XCD until the first short tiles, 26 us apart behind them and 113 us at
    // the end; the launch fetches 6 times its operands).  So a short tile holds the pace of a full one: the first
    // wavefront waits at the end of every k-step until a full tile would be there (the others wait at the barrier; a
    // wait on a clock, so it always ends).  With that the tiles of an XCD start within 4.4 us of each other to the end
    // of the launch and it fetches 10.0 GB instead of 17.9 GB at the same speed (2736 - 2777 against 2749 - 2774
    // TFLOP/s in alternating runs).  Only in the fused launch: the plain product of the same rows (K = 16384, N = 6144)
    // fetches 5.7 GB instead of 7.9 GB that way but runs 1.5 % slower, the idle time of its short tiles being worth
    // more than the traffic.
    long long full_step_ticks = 0;
    while (q < total) {
        const int cur_row0 = row0, cur_rows_e = rows_e, cur_n0 = n0, cur_e = e;
        const int cur_part = part, cur_split_tile = split_tile;
        int nfr = ((rows_e < kDM ? rows_e : kDM) - wm * TM + 15) / 16;
        nfr = __builtin_amdgcn_readfirstlane(nfr < 0 ? 0 : (nfr > FM ? FM : nfr));

        auto run_tile = [&](auto guard_tag) {
            constexpr bool kGuard = decltype(guard_tag)::value;
            f32x4 acc[FM][FN];
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

            // the early group of k-step 0 has landed (its late group and k-step 1 may be in flight)
            if (T > 1) DMOE_WAIT_VMCNT(kLate + kEarly + kLate); else DMOE_WAIT_VMCNT(kLate);
            __syncthreads();
            const bool short_tile = cur_rows_e < kDM;
            const bool pace = SWIGLU && short_tile && full_step_ticks > 0 && wave == 0;
            const long long t_begin = (long long)wall_clock64();
            // Phases of k-step t, for the early half of the wavefronts (the late half one phase later): memory a (the B
            // fragments, row fragments 0 - 3), matrix a, memory b (row fragments 4 - 7), matrix b.  What memory a reads is
            // free once the late half has left its memory a, so memory b of k-step t issues the early group of k-step
            // t + 2 into it, and memory a of k-step t + 1 the late group of k-step t + 2 (the prologue stands in for the
            // first ones): a copy is in flight for a k-step and a half.  A wavefront's copies complete in the order early(t),
            // late(t), early(t + 1), ...; before the barrier that lets the early half into memory a of k-step t + 1 every
            // wavefront has waited for its early(t + 1), behind which it has issued late(t + 1) and early(t + 2), and
            // before the barrier that lets it into memory b of k-step t for its late(t), behind which early(t + 1) and late(t + 1).
            auto landed_early = [&](int t) {   // early(t + 1), at the end of k-step t
                if (t + 2 < T) DMOE_WAIT_VMCNT(kLate + kEarly); else DMOE_WAIT_VMCNT(kLate);
            };
            auto landed_late = [&](int t) {    // late(t), in the middle of k-step t
                if (t + 1 < T) DMOE_WAIT_VMCNT(kEarly + kLate); else DMOE_WAIT_VMCNT(0);
            };
            auto half_step = [&](int t, auto h_tag, bool next) {
                constexpr int h = decltype(h_tag)::value;
                const char *base = smem + (t % kBufs) * kBuf;
                if (h == 0) {
#pragma unroll
                    for (int j = 0; j < FN; ++j) fb[j] = read32(base, fb_base, fb_dist(j));
                }
#pragma unroll
                for (int i = 0; i < FM / 2; ++i) fa[i] = read32(base, fa_base, (h * (FM / 2) + i) * (16 * kStepK));
                if (h == 0 && t >= 1 && next) issue_late(t + 1);
                if (h == 1 && t + 2 < T) issue_early(t + 2);
                if (wm == 1) {
                    if (h == 0) landed_late(t);
                    else if (next) landed_early(t);
                }
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_setprio(1);
                static_for<0, FM / 2>([&](auto i_tag) {
                    constexpr int i = h * (FM / 2) + decltype(i_tag)::value;
                    if (kGuard && i >= nfr) return;        // wave-uniform
                    // (j back and forth, so that every MFMA shares an operand with the one before it: less energy)
#pragma unroll
                    for (int jj = 0; jj < FN; ++jj) {
                        const int j = (i & 1) ? FN - 1 - jj : jj;
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[decltype(i_tag)::value], acc[i][j],
                                                                                     0, 0, 0, 0, 0, 0);
                    }
                });
                __builtin_amdgcn_s_setprio(0);
                if (wm == 0) {
                    if (h == 0) landed_late(t);
                    else if (next) landed_early(t);
                }
                if (h == 1 && pace) {
                    const long long due = t_begin + (long long)(t + 1) * full_step_ticks;
                    while ((long long)wall_clock64() < due) __builtin_amdgcn_s_sleep(2);
                }
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            };
            if (wm == 1) __syncthreads();                  // the late half
            for (int t = 0; t < T; ++t) {
                half_step(t, std::integral_constant<int, 0>{}, t + 1 < T);
                half_step(t, std::integral_constant<int, 1>{}, t + 1 < T);
            }
            if (wm == 0) __syncthreads();
            if (!short_tile && wave == 0) {
                // (the fastest full tile so far: a tile that was held up by something else must not set the pace)
                const long long ticks = ((long long)wall_clock64() - t_begin) / T;
                if (full_step_ticks == 0 || ticks < full_step_ticks) full_step_ticks = ticks;
            }

            // a piece of a split tile: its sums go to the workspace, and the piece that arrives last adds all of them up
            if (cur_part >= 0 &&
                !meet_pieces<NW>(acc, p, plan.split, cur_split_tile, cur_part, wave, lane, kGuard ? nfr : FM))
                return;

            // ---- epilogue: scales, (SiLU * up), 32 rows at a time through LDS, out by rows (see gmm_tile256.h) ----
            constexpr int RB = FNO * 32;
            constexpr int CPR = RB / 16;
            constexpr int RPI = 64 / CPR;
            char *stg = smem + (T % kBufs) * kBuf + wave * 4096;   // the buffer that the last k-step did not use
            auto swz = [](int row) { return CPR == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3); };
            const int col0 = cur_n0 + (SWIGLU ? wn * (TN / 2) : wn * TN);
            // the column scales of this lane's 4 columns of every fragment (columns outside the tile read a valid one)
            float4 sb[FNO][SWIGLU ? 2 : 1];
#pragma unroll
            for (int j = 0; j < FNO; ++j) {
                const int col = col0 + j * 16 + g16 * 4;
                const float *src = p.b_scale + (long long)cur_e * p.N + (col < n_out ? col : cur_n0);
                sb[j][0] = *(const float4 *)src;
                if (SWIGLU) sb[j][SWIGLU ? 1 : 0] = *(const float4 *)(src + n_out);
            }
#pragma unroll
            for (int i2 = 0; i2 < FM / 2; ++i2) {
                if (kGuard && i2 * 2 >= nfr) break;
#pragma unroll
                for (int ii = 0; ii < 2; ++ii) {
                    const int i = i2 * 2 + ii;
                    const int row = ii * 16 + l16;
                    const int r = wm * TM + i * 16 + l16;
                    const float sa = p.a_scale[cur_row0 + (r < cur_rows_e ? r : 0)];
#pragma unroll
                    for (int j = 0; j < FNO; ++j) {
                        const float s0[4] = {sb[j][0].x, sb[j][0].y, sb[j][0].z, sb[j][0].w};
                        const float s1[4] = {sb[j][SWIGLU ? 1 : 0].x, sb[j][SWIGLU ? 1 : 0].y, sb[j][SWIGLU ? 1 : 0].z, sb[j][SWIGLU ? 1 : 0].w};
                        float v[4];
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            const float g = acc[i][j][x] * (sa * s0[x]);
                            v[x] = SWIGLU ? silu_mul(g, acc[i][j + FN / 2][x] * (sa * s1[x])) : g;
                        }
                        uint2 pk;
                        pk.x = pack_bf16x2(v[0], v[1]);
                        pk.y = pack_bf16x2(v[2], v[3]);
                        const int cb = j * 32 + g16 * 8;
                        *(uint2 *)(stg + row * RB + (((cb >> 4) ^ swz(row)) << 4) + (cb & 8)) = pk;
                    }
                }
#pragma unroll
                for (int t = 0; t < 32 / RPI; ++t) {
                    const int row = t * RPI + lane / CPR, c = lane % CPR;
                    const u32x4 val = *(const u32x4 *)(stg + row * RB + ((c ^ swz(row)) << 4));
                    const int grow = wm * TM + i2 * 32 + row;
                    const int gcol = col0 + c * 8;
                    if (grow >= cur_rows_e || gcol >= n_out) continue;
                    *(u32x4 *)((uint16_t *)p.c + (long long)(cur_row0 + grow) * p.ldc + gcol) = val;
                }
            }
        };
        if (nfr == FM) run_tile(std::false_type{});
        else run_tile(std::true_type{});

        if (drawer) s_item = sched_item(draw, streams);
        __syncthreads();
        q = s_item;
        if (q < total) {
            if (drawer) draw = sched_draw(p.sched, streams);
            open_tile(q);
            issue_prologue();
        }
    }
    sched_finish(p.sched, drawer, draw, streams, total);
}

template <bool SWIGLU>
static int launch_tile256_fp8_one(const GmmArgs &args, hipStream_t stream) {
    const size_t lds = (size_t)2 * (256 * 128 + 256 * 128);
    auto kern = gmm_tile256_fp8_kernel<SWIGLU>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, 256, SWIGLU, 64, true, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_tile256_fp8_kernel");
    return DMOE_OK;
}

}  // namespace dmoe
