// bf16 grouped GEMM, the 256 x 256 tile on 8 wavefronts with v_mfma_f32_16x16x32_bf16.
//
// The chip is power-limited under MFMA load: a loop of nothing but MFMAs on random bf16 operands sustains about
// 2.05 PFLOP/s with the 16x16x32 form and about 1.75 with 32x32x16 (8 wavefronts per CU, 256 CUs), so this tile uses the
// former: a wavefront owns 128 x 64 of the tile as 8 x 4 accumulators of 16 x 16.
//
//   * A and B tiles go global -> LDS directly (global_load_lds_dwordx4, 1 KiB per wavefront instruction); K in stages
//     of 32 (64 bytes per row), 4 stages of 32 KiB in LDS, a copy is issued 3 stages before its data is read;
//   * LDS images: K-contiguous rows of 64 B with the 16-byte chunk c of row r at c ^ kc_swizzle(r), read with
//     ds_read_b128 (lane l: row l % 16, the 8 k of chunk l / 16: one read is a whole 16 x 32 operand).  A probe that
//     timed this read for all 256 XOR-linear swizzles of the row found it free of bank conflicts (4 cycles per
//     instruction) exactly for those that flip chunk bit 1 by row bit 2 or 3 but not both alike, and 2-way conflicted
//     with the ((r >> 2) & 3) that serves the 32 x 32 fragments of gmm_direct.h.  B in the [K, N] layout is kept
//     [k][256 n] (512-byte rows of 32 chunks) with chunk ^ kn_swizzle(k), read with two ds_read_b64_tr_b16 per operand:
//     32 lanes of such a read address 4 k-rows of two k-groups (k, k + 8) x 16 columns, and the swizzle spreads those 8
//     rows x 32 bytes over all banks;
//   * the two wavefronts of a SIMD (w and w + 4) alternate between a memory phase (the 12 or 16 operand reads of a
//     stage into the one register set, the wavefront's 4 copies, the waits) and a matrix phase (the stage's 32 MFMAs,
//     nothing else), one phase apart, handed over by workgroup barriers: while one issues MFMAs the other issues
//     everything else;
//   * the MFMAs take the B fragment as first operand, so a lane holds 4 consecutive columns of one row; the epilogue
//     (SiLU(gate) * up on the fp32 accumulators in the fused form) stages 32 rows at a time through LDS and stores whole
//     rows of the result.
#pragma once
#include "gmm_direct.h"

namespace dmoe {

// GATHER: row r of the product is row p.a_rows[r] of a (the tokens, in their own order): the permute that sorts the
// routed rows by expert needs no launch and no copy of the rows.  A tile's row numbers are fetched and waited for before
// the epilogue of the tile before it, when nothing else of the wavefront is in flight: behind the epilogue the same
// wait would also be one for the epilogue's stores.
template <bool TRANS_B, bool SWIGLU, bool GATHER = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gmm_tile256_kernel(const GmmArgs p) {
    constexpr int kDM = 256, NW = 8, WN = 4;
    constexpr int TM = 128, TN = 64;
    constexpr int FM = TM / 16, FN = TN / 16;            // 8 x 4 accumulators of 16 x 16
    constexpr int FNO = SWIGLU ? FN / 2 : FN;            // column fragments of the result
    constexpr int CA = kDM / (16 * NW);                  // A copies (16 rows each) per wavefront per stage
    constexpr int CB = 16 / NW;                          // B copies (1 KiB of the 16 KiB each)
    constexpr int kLoads = CA + CB;
    constexpr int kBlock = NW * 1024;
    constexpr int kStageA = kDM * kDK * 2;
    constexpr int kStage = kStageA + kStageB;
    constexpr int kStages = 4;
    constexpr int BNO = SWIGLU ? kDN / 2 : kDN;
    static_assert(CA == 2 && CB == 2 && (kStages - 1) * kLoads <= 63, "copies per stage");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int s_tile_start[kMaxGroups + 1];
    __shared__ int s_row_start[kMaxGroups + 1];
    __shared__ long long s_item;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;            // wm also numbers the half that runs a phase behind
    const int E = p.E;

    build_work_list<kDM>(p, s_tile_start, s_row_start);
    __syncthreads();

    const int n_out = SWIGLU ? p.N / 2 : p.N;
    const int n_tiles = (n_out + BNO - 1) / BNO;
    const int S_all = p.K / kDK;
    const int G = gridDim.x;
    constexpr long long kPieceBytes = (long long)kDM * kDN * sizeof(float);
    const WorkPlan plan = plan_work((long long)s_tile_start[E] * n_tiles, G, S_all,
                                    p.arrive != nullptr ? p.partial_bytes / kPieceBytes : 0, kWsArriveCount / NW);
    const long long total = plan.items;
    // A launch whose m-tiles are less than half full on average (a decode-sized batch) streams weights, and what its loop
    // does besides is what the stream has to overlap with: its short tiles read only the row fragments that hold a valid
    // row and run every stage as one phase of all wavefronts (one barrier) instead of two alternating ones.  Elsewhere
    // short tiles keep the schedule of the full tiles they share operands with.
    const bool lean = 2ll * s_row_start[E] < (long long)s_tile_start[E] * kDM;
    const uint32_t pitch = (uint32_t)p.K * 2;
    const uint32_t smem_addr = lds_addr(smem);
    const int streams = (G % kXcds == 0) ? kXcds : 1;

    // ---- per-lane constants of the global -> LDS copies (see gmm_direct.h) ----
    auto kc_swizzle = [](int row) { return ((row >> 2) & 1) << 1; };
    const int kc_row = lane >> 2;                          // a 1 KiB block is 16 rows of 64 B: lane l fills row l / 4,
    const int kc_chunk = (lane & 3) ^ kc_swizzle(kc_row);  // physical chunk l % 4, with this logical chunk
    auto kn_swizzle = [](int k) { return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1); };
    const int kn_k = 2 * wave + (lane >> 5);               // block i adds 16: the swizzle stays
    const int kn_chunk = (lane & 31) ^ kn_swizzle(kn_k);

    // ---- per-lane constants of the operand reads ----
    const int l16 = lane & 15, g16 = lane >> 4;            // row / column inside a fragment, k-group (8 k each)
    const int kc_read = (g16 ^ kc_swizzle(l16)) << 4;       // rows 16 apart share the swizzle
    const int fa_base = (wm * TM + l16) * 64 + kc_read;
    int fb_off[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int slot0 = SWIGLU ? ((j < FN / 2) ? wn * (TN / 2) + j * 16 : kDN / 2 + wn * (TN / 2) + (j - FN / 2) * 16)
                                 : wn * TN + j * 16;
        if constexpr (TRANS_B) {
            fb_off[j] = (slot0 + l16) * 64 + kc_read;
        } else {
            // the 16 lanes of a k-group address 4 k-rows x 16 columns, a lane 4 columns of one k-row; the transposing
            // read hands lane l16 the 4 k of column slot0 + l16.  k-rows g16 * 8 + (l16 >> 2) (and 4 further on).
            const int col = slot0 + 4 * (l16 & 3);
            const int krow = g16 * 8 + (l16 >> 2);
            const int chunk = (col >> 3) ^ kn_swizzle(krow);   // k-row krow + 4 has the same swizzle
            fb_off[j] = krow * 512 + chunk * 16 + (col & 7) * 2;
        }
    }

    // ---- state of the item whose copies are being issued ----
    int e = 0, row0 = 0, rows_e = 0, n0 = 0;
    int s_lo = 0, S = 0, pre = 0;
    int part = -1, split_tile = 0;
    uint64_t a_base = 0, b_exp = 0;
    uint32_t a_off[CA], b_off[CB];
    int a_tok[GATHER ? CA : 1];                            // GATHER: source rows of this lane's A rows
    // the expert of the item has a single m-tile: its weights pass through this workgroup once and through no other, so
    // their copies take the non-temporal policy (wave-uniform)
    bool b_once = false;

    auto b_col = [&](int slot) {
        const int rh = (SWIGLU && slot >= kDN / 2) ? slot - kDN / 2 : slot;
        const int base = (SWIGLU && slot >= kDN / 2) ? n_out + n0 : n0;
        return base + (rh < n_out - n0 ? rh : 0);          // slots past the end read a valid column (never stored)
    };
    auto locate = [&](long long q) { return decode_item<kDM>(q, G, plan, S_all, n_tiles, E, s_tile_start, s_row_start); };
    // GATHER: asks for the row numbers of this lane's A rows of item `it`
    auto fetch_rows = [&](const WorkItem &it) {
        if constexpr (GATHER) {
#pragma unroll
            for (int i = 0; i < CA; ++i) {
                int r = (i * NW + wave) * 16 + kc_row;
                if (r >= it.tile.rows_e) r = it.tile.rows_e - 1;
                a_tok[i] = p.a_rows[it.tile.row0 + r];
            }
        }
    };
    auto open_item = [&](const WorkItem &it) {
        e = it.tile.e; row0 = it.tile.row0; rows_e = it.tile.rows_e; n0 = it.tile.nt * BNO;
        b_once = __builtin_amdgcn_readfirstlane(s_tile_start[e + 1] - s_tile_start[e]) == 1;
        s_lo = it.s_lo; S = it.s_cnt;
        part = it.piece; split_tile = it.split_tile;
        pre = S < kStages ? S : kStages;
        a_base = to_scalar((uint64_t)(uintptr_t)p.a + (GATHER ? 0 : (uint64_t)row0 * pitch) + (uint64_t)s_lo * 64);
        b_exp = to_scalar((uint64_t)(uintptr_t)p.b + (uint64_t)e * p.K * p.N * 2 +
                          (uint64_t)s_lo * (TRANS_B ? 64 : (uint64_t)kDK * p.N * 2));
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            int r = (i * NW + wave) * 16 + kc_row;
            if (r >= rows_e) r = rows_e - 1;               // clamp: loaded, never stored
            if constexpr (!GATHER) a_off[i] = (uint32_t)r * pitch + kc_chunk * 16;   // (GATHER: see aim_rows)
        }
        if constexpr (TRANS_B) {
#pragma unroll
            for (int i = 0; i < CB; ++i) b_off[i] = (uint32_t)b_col((i * NW + wave) * 16 + kc_row) * pitch + kc_chunk * 16;
        } else {
#pragma unroll
            for (int i = 0; i < CB; ++i)
                b_off[i] = (uint32_t)(i * 2 * NW + kn_k) * (uint32_t)p.N * 2 + (uint32_t)b_col(kn_chunk * 8) * 2;
        }
    };
    auto open_tile = [&](long long q) {
        const WorkItem it = locate(q);
        fetch_rows(it);
        open_item(it);
    };
    // the kLoads copies of this wavefront for stage s of the item: its CA blocks of A, then its CB blocks of B
    auto issue_copies = [&](int s) {
        const uint32_t lds = smem_addr + (s % kStages) * kStage + wave * 1024;
        // (GATHER: the compiler loses track of these wave-uniform addresses being uniform where the next item is
        // located from inside the tile's code; to_scalar costs nothing where it has not)
        const uint64_t a_stage = GATHER ? to_scalar(a_base + (uint64_t)s * 64) : a_base + (uint64_t)s * 64;
        static_for<0, CA>([&](auto c_tag) {
            constexpr int c = decltype(c_tag)::value;
            copy_g2lds_16<c * kBlock>(a_off[c], a_stage, lds);
        });
        const uint64_t b_stage = b_exp + (TRANS_B ? (uint64_t)s * 64 : (uint64_t)s * kDK * p.N * 2);
        const uint64_t base = GATHER ? to_scalar(b_stage) : b_stage;
        if (b_once) {   // one branch per stage
            static_for<0, CB>([&](auto i_tag) {
                constexpr int i = decltype(i_tag)::value;
                copy_g2lds_16_nt<kStageA + i * kBlock>(b_off[i], base, lds);
            });
        } else {
            static_for<0, CB>([&](auto i_tag) {
                constexpr int i = decltype(i_tag)::value;
                copy_g2lds_16<kStageA + i * kBlock>(b_off[i], base, lds);
            });
        }
    };
    // GATHER: the row numbers that fetch_rows asked for, as offsets of this lane's copies
    uint32_t a_off_next[GATHER ? CA : 1];
    auto aim_rows = [&]() {
        if constexpr (GATHER) {
#pragma unroll
            for (int i = 0; i < CA; ++i) {
                int tok = a_tok[i];
                tok = tok < 0 ? 0 : (tok >= (int)p.a_src_rows ? (int)p.a_src_rows - 1 : tok);   // never outside a
                a_off_next[i] = (uint32_t)tok * pitch + kc_chunk * 16;
            }
        }
    };
    auto take_rows = [&]() {
        if constexpr (GATHER) {
#pragma unroll
            for (int i = 0; i < CA; ++i) a_off[i] = a_off_next[i];
        }
    };
    auto issue_prologue = [&]() {
        for (int s = 0; s < pre; ++s) issue_copies(s);
    };
    auto wait_ahead = [&](int n) {   // at most n stages of this wavefront's copies outstanding
        if (n >= 3) DMOE_WAIT_VMCNT(3 * kLoads);
        else if (n == 2) DMOE_WAIT_VMCNT(2 * kLoads);
        else if (n == 1) DMOE_WAIT_VMCNT(kLoads);
        else DMOE_WAIT_VMCNT(0);
    };

    bf16x8 fa[FM], fb[FN];
    // `lim`: row fragments to read (wave-uniform; FM for a full tile); a wavefront without a valid row reads nothing.
    // In the guarded build `lim` is a run-time value, so every fragment sits behind a scalar branch and the reads have
    // completed before the phase's barrier; in the build of full tiles it is the constant FM and the reads are waited for
    // behind the barrier, next to the first MFMA.  Deliberately so: a short tile's stage is then a little slower than a
    // full tile's instead of much faster, its workgroup keeps pace with the m-tiles it shares operand tiles with, and
    // those still meet in L2 (measured on 8 experts of ~1024 rows, K = 4096: half the bytes from beyond L2, 1.5 - 2.5 %
    // more throughput than with short tiles that run ahead).
    auto load_operands = [&](int s, int lim) {
        const char *tA = smem + (s % kStages) * kStage;
        const char *tB = tA + kStageA;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if (i >= lim) break;
            const u32x4 x = *(const u32x4 *)(tA + fa_base + i * (16 * 64));
            __builtin_memcpy(&fa[i], &x, 16);
        }
        if (lim <= 0) return;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            if constexpr (TRANS_B) {
                const u32x4 x = *(const u32x4 *)(tB + fb_off[j]);
                __builtin_memcpy(&fb[j], &x, 16);
            } else {
                const char *src = tB + fb_off[j];
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)DMOE_LDS_PTR(src));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)DMOE_LDS_PTR(src + 4 * 512));
                const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                __builtin_memcpy(&fb[j], &v, 16);
            }
        }
    };

    // ---- first work item ----
    unsigned int draw = 0;
    const bool drawer = tid == 0;
    if (drawer) draw = sched_draw(p.sched, streams);       // always one draw ahead: its round trip hides behind a tile
    long long q = blockIdx.x;                              // the first item needs no draw (see sched_item)
    if (q < total) {
        open_tile(q);
        aim_rows();
        take_rows();
        issue_prologue();
    }

    while (q < total) {
        WorkItem next_item{};                              // GATHER: the next item, located before this one's epilogue
        const int cur_row0 = row0, cur_rows_e = rows_e, cur_n0 = n0;
        const int cur_part = part, cur_split_tile = split_tile, cur_S = S;
        // 16-row fragments of this wavefront that hold at least one valid row (a short last tile skips the rest)
        int nfr = ((rows_e < kDM ? rows_e : kDM) - wm * TM + 15) / 16;
        nfr = __builtin_amdgcn_readfirstlane(nfr < 0 ? 0 : (nfr > FM ? FM : nfr));

        auto run_tile = [&](auto guard_tag) {
            constexpr bool kGuard = decltype(guard_tag)::value;
            // Alternating phases of the two halves of the workgroup, or one phase per stage: the same for every wavefront
            // of the workgroup (they share the barriers), so the one-phase form needs a tile in which every wavefront runs
            // this guarded build: at most 7 row fragments in the upper half, none in the lower.
            const bool kAlt = !(kGuard && lean && cur_rows_e <= (FM - 1) * 16);
            f32x4 acc[FM][FN];
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

            // stage 0 has landed (the other stages of the prologue and stores of the previous epilogue, issued before
            // them, may still be in flight: waiting for fewer is only stricter)
            wait_ahead(pre - 1);
            __syncthreads();
            // The slot of stage s - 1 is free once every wavefront has read that stage, i.e. behind the barrier that
            // closes the memory phase of the late half; from then on (memory phases of stage s) it is refilled with
            // stage s + kStages - 1.  Before the barrier that lets the early half read stage s + 1, every wavefront has
            // waited for its own copies of that stage.
            auto stage = [&](int s, auto refill_tag, int ahead, bool next) {
                constexpr bool kRefill = decltype(refill_tag)::value;
                auto landed = [&]() {
                    if constexpr (kRefill) DMOE_WAIT_VMCNT((kStages - 2) * kLoads);
                    else wait_ahead(ahead);
                };
                load_operands(s, kAlt ? FM : nfr);
                if constexpr (kRefill) issue_copies(s + kStages - 1);
                if (kAlt) {
                    // the guarded build has its operands in registers before the barrier (see load_operands)
                    if constexpr (kGuard) __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
                    if (next && wm == 1) landed();
                    __builtin_amdgcn_sched_barrier(0);
                    __syncthreads();
                    __builtin_amdgcn_sched_barrier(0);
                } else {
                    // one phase: the slot refilled above was read by everyone before the barrier that ended the stage before
                    if (next) landed();
                }
                __builtin_amdgcn_s_setprio(1);
                static_for<0, FM>([&](auto i_tag) {
                    constexpr int i = decltype(i_tag)::value;
                    if (kGuard && i >= nfr) return;        // wave-uniform
                    // (j back and forth: one operand of every MFMA is the one the MFMA before it had, which the chip's
                    // power limit pays back as clock: 2.7 % on a loop of MFMAs alone, 0.7 % here)
#pragma unroll
                    for (int jj = 0; jj < FN; ++jj) {
                        const int j = (i & 1) ? FN - 1 - jj : jj;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
                    }
                });
                __builtin_amdgcn_s_setprio(0);
                if (kAlt && next && wm == 0) landed();
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            };
            if (kAlt && wm == 1) __syncthreads();          // the late half
            int s = 0;
            stage(0, std::false_type{}, (S - 2 < kStages - 2 ? S - 2 : kStages - 2), S > 1);
            for (s = 1; s + kStages - 1 < S; ++s) stage(s, std::true_type{}, 0, true);
            for (; s < S; ++s) {
                const int left = S - 1 - s;
                stage(s, std::false_type{}, left - 1 < kStages - 2 ? left - 1 : kStages - 2, left > 0);
            }
            if (kAlt && wm == 0) __syncthreads();

            if constexpr (GATHER) {
                // the next work item now, so that its row numbers travel while this tile's results are written
                if (drawer) s_item = sched_item(draw, streams);
                __syncthreads();
                q = (long long)to_scalar((uint64_t)s_item);
                if (q < total) {
                    if (drawer) draw = sched_draw(p.sched, streams);
                    next_item = locate(q);
                    fetch_rows(next_item);
                    aim_rows();
                }
            }
            // a piece of a split tile: its sums go to the workspace, and the piece that arrives last adds all of them up
            if (cur_part >= 0 &&
                !meet_pieces<NW>(acc, p, plan.split, cur_split_tile, cur_part, wave, lane, kGuard ? nfr : FM))
                return;

            // ---- epilogue ----
            // Lane l holds, of fragment (i, j), row i * 16 + l % 16 and the 4 columns j * 16 + (l / 16) * 4 ...: 8 bytes
            // of the result.  32 rows at a time they go through LDS (the stage buffer that is free after the last stage,
            // 4 KiB private to the wavefront, no barrier) and leave by rows of the result, 16 bytes per lane: a store
            // instruction writes 8 whole rows of 128 bytes, or 16 rows of 64 bytes in the fused form.  The 16-byte chunk c
            // of row r sits at c ^ ((r >> 1) & 7) (128-byte rows) or c ^ ((r >> 2) & 3) (64-byte rows): neither the 8-byte
            // writes of 32 lanes nor the 16-byte reads of 16 lanes meet in a bank.
            constexpr int RB = FNO * 32;                   // bytes per staged row
            constexpr int CPR = RB / 16;                   // lanes that write a row out
            constexpr int RPI = 64 / CPR;                  // rows per store instruction
            char *stg = smem + (cur_S % kStages) * kStage + wave * 4096;
            auto swz = [](int row) { return CPR == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3); };
            const int col0 = cur_n0 + (SWIGLU ? wn * (TN / 2) : wn * TN);
#pragma unroll
            for (int i2 = 0; i2 < FM / 2; ++i2) {
                if (kGuard && i2 * 2 >= nfr) break;        // wave-uniform: no valid row from here on
#pragma unroll
                for (int ii = 0; ii < 2; ++ii) {
                    const int i = i2 * 2 + ii;
                    const int row = ii * 16 + l16;
#pragma unroll
                    for (int j = 0; j < FNO; ++j) {
                        float v[4];
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            v[x] = SWIGLU ? silu_mul(acc[i][j][x], acc[i][j + FN / 2][x]) : acc[i][j][x];
                        uint2 pk;
                        pk.x = pack_bf16x2(v[0], v[1]);
                        pk.y = pack_bf16x2(v[2], v[3]);
                        const int cb = j * 32 + g16 * 8;   // byte of the row where this lane's 4 columns start
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

        // ---- next work item and its first copies (the stores above are older than them) ----
        if constexpr (GATHER) {
            __syncthreads();   // the last stage has been read by everyone and the staged rows have been read back
            if (q < total) {
                open_item(next_item);
                take_rows();
                issue_prologue();
            }
        } else {
            if (drawer) s_item = sched_item(draw, streams);
            __syncthreads();   // also: the last stage has been read by everyone and the staged rows have been read back
            q = s_item;
            if (q < total) {
                if (drawer) draw = sched_draw(p.sched, streams);
                open_tile(q);
                issue_prologue();
            }
        }
    }
    sched_finish(p.sched, drawer, draw, streams, total);
}

template <bool TRANS_B, bool SWIGLU, bool GATHER = false>
static int launch_tile256_one(const GmmArgs &args, hipStream_t stream) {
    const size_t lds = (size_t)4 * (256 * kDK * 2 + kStageB);
    auto kern = gmm_tile256_kernel<TRANS_B, SWIGLU, GATHER>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, 256, SWIGLU, kDK, true, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_tile256_kernel");
    return DMOE_OK;
}

}  // namespace dmoe
