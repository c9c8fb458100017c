// bf16 grouped GEMM, the 256 x 256 tile on 4 wavefronts of 128 x 128 with v_mfma_f32_16x16x32_bf16.
//
// The chip is power-limited under MFMA load, and what the loop does besides the MFMAs is paid for in clock.  A wavefront
// that owns 128 x 128 of the tile reads 8 + 8 operand fragments from LDS for its 64 MFMAs of a stage, one of 128 x 64
// reads 8 + 4 for 32: a third fewer LDS bytes per MFMA, and half the barriers.  The price is one wavefront per SIMD (its
// 256 accumulator registers are the upper half of the register file), so the operand reads, the global -> LDS copies
// and the MFMAs of a stage share one instruction stream: every other instruction is issued in the shadow of an MFMA, at
// most one or two behind each.
//
//   * weights in the [K, N] layout; LDS images, swizzles, copies and epilogue as in gmm_tile256.h: 4 stages of 32 KiB,
//     K in stages of 32;
//   * a stage is 8 rows of 8 MFMAs (row fragment i against the 8 column fragments) on one of two register sets; the
//     16 operand fragments of stage s + 1 are read into the other set while stage s is multiplied, so an LDS buffer
//     is free again a whole stage before its stage is multiplied: the registers are a fifth buffer;
//   * ONE barrier per stage, in front of its MFMA 16.  Before it a wavefront has waited for its own copies of stage
//     s + 1; behind it everybody's are there and everybody has read stage s (during stage s - 1), so the copies of
//     stage s + 4 go into that buffer, one every 4 MFMAs, and the reads of stage s + 1 begin: a copy is in flight for
//     2.5 to 3 stages, and an operand read is at least 16 MFMAs old when the next barrier waits for it.
#pragma once
#include "gmm_direct.h"

namespace dmoe {

template <bool SWIGLU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gmm_wave128_kernel(const GmmArgs p) {
    constexpr int kDM = 256, NW = 4;
    constexpr int TM = 128, TN = 128;
    constexpr int FM = TM / 16, FN = TN / 16;            // 8 x 8 accumulators of 16 x 16
    constexpr int FNO = SWIGLU ? FN / 2 : FN;            // column fragments of the result
    constexpr int CA = 4, CB = 4;                        // copies (1 KiB) of A and of B per wavefront per stage
    constexpr int kLoads = CA + CB;
    constexpr int kStageA = kDM * kDK * 2;
    constexpr int kStage = kStageA + kStageB;
    constexpr int kStages = 4;
    constexpr int kAhead = kStages;                      // stages copied ahead of the one being multiplied (its own
                                                         // operands are in registers)
    constexpr int BNO = SWIGLU ? kDN / 2 : kDN;
    constexpr int kBarrierSlot = 16;                     // the stage's barrier stands in front of this MFMA
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int s_tile_start[kMaxGroups + 1];
    __shared__ int s_row_start[kMaxGroups + 1];
    __shared__ long long s_item;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
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
    const uint32_t pitch = (uint32_t)p.K * 2;
    const uint32_t smem_addr = lds_addr(smem);
    const int streams = (G % kXcds == 0) ? kXcds : 1;

    // ---- per-lane constants of the global -> LDS copies ----
    // A: a 1 KiB block is 16 rows of 64 B, lane l fills row l / 4, physical chunk l % 4; block i of this wavefront
    // holds rows 64 wave + 16 i ... of the tile.  B: a block is 2 k-rows of 512 B, lane l fills k-row l / 32, physical
    // chunk l % 32; block i of this wavefront holds k-rows 8 wave + 2 i, + 1 of the stage.
    auto kc_swizzle = [](int row) { return ((row >> 2) & 1) << 1; };
    const int kc_row = lane >> 2;
    const int kc_chunk = (lane & 3) ^ kc_swizzle(kc_row);
    auto kn_swizzle = [](int k) { return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1); };

    // ---- state of the item whose copies are being issued ----
    int e = 0, row0 = 0, rows_e = 0, n0 = 0;
    int s_lo = 0, S = 0;
    int part = -1, split_tile = 0;
    uint64_t a_base = 0, b_exp = 0;
    uint32_t a_off[CA], b_off[CB];

    auto b_col = [&](int slot) {
        const int rh = (SWIGLU && slot >= kDN / 2) ? slot - kDN / 2 : slot;
        const int base = (SWIGLU && slot >= kDN / 2) ? n_out + n0 : n0;
        return base + (rh < n_out - n0 ? rh : 0);          // slots past the end read a valid column (never stored)
    };
    auto open_tile = [&](long long q) {
        const WorkItem it = decode_item<kDM>(q, G, plan, S_all, n_tiles, E, s_tile_start, s_row_start);
        e = it.tile.e; row0 = it.tile.row0; rows_e = it.tile.rows_e; n0 = it.tile.nt * BNO;
        s_lo = it.s_lo; S = it.s_cnt;
        part = it.piece; split_tile = it.split_tile;
        a_base = to_scalar((uint64_t)(uintptr_t)p.a + (uint64_t)row0 * pitch + (uint64_t)s_lo * 64);
        b_exp = to_scalar((uint64_t)(uintptr_t)p.b + (uint64_t)e * p.K * p.N * 2 + (uint64_t)s_lo * ((uint64_t)kDK * p.N * 2));
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            int r = (wave * CA + i) * 16 + kc_row;
            if (r >= rows_e) r = rows_e - 1;               // clamp: loaded, never stored
            a_off[i] = (uint32_t)r * pitch + kc_chunk * 16;
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int k = wave * 8 + 2 * i + (lane >> 5);
            const int chunk = (lane & 31) ^ kn_swizzle(k);
            b_off[i] = (uint32_t)k * (uint32_t)p.N * 2 + (uint32_t)b_col(chunk * 8) * 2;
        }
    };
    // Copy c (0 .. 7: 4 blocks of A, 4 of B) of this wavefront for a stage whose operand rows start at a_ptr / b_ptr
    // (wave-uniform), into LDS buffer kBuf.  In two halves, so that an MFMA can stand between the write of M0 and the
    // load that reads it (the wait state the hardware asks for) and no gap between two MFMAs holds more than two
    // other instructions.
    const uint32_t lds_wave = smem_addr + wave * 4096;
    auto copy_aim = [&](auto buf_tag, auto c_tag) {
        constexpr int c = decltype(c_tag)::value, kBuf = decltype(buf_tag)::value;
        constexpr int imm = kBuf * kStage + (c < CA ? c * 1024 : kStageA + (c - CA) * 1024);
        const uint32_t base = lds_wave;                    // (an asm operand cannot name a captured variable)
        asm volatile("s_add_u32 m0, %0, %1" :: "s"(base), "n"(imm) : "m0", "scc");
    };
    auto copy_fire = [&](uint64_t a_ptr, uint64_t b_ptr, auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
        uint32_t off;
        if constexpr (c < CA) off = a_off[c]; else off = b_off[c - CA];
        const uint64_t ptr = c < CA ? a_ptr : b_ptr;
        asm volatile("global_load_lds_dwordx4 %0, %1" :: "v"(off), "s"(ptr) : "memory");
    };
    // stage u of the item, or its last one if there is no such stage (a copy that nobody reads, into a buffer that
    // nobody needs: the loop then has no branch and every stage issues the same number of copies)
    auto a_stage_ptr = [&](int u) { return a_base + (uint64_t)(u < S ? u : S - 1) * 64; };
    auto b_stage_ptr = [&](int u) { return b_exp + (uint64_t)(u < S ? u : S - 1) * ((uint64_t)kDK * p.N * 2); };
    auto issue_prologue = [&]() {
        static_for<0, kStages>([&](auto b_tag) {
            const uint64_t a_ptr = a_stage_ptr(decltype(b_tag)::value), b_ptr = b_stage_ptr(decltype(b_tag)::value);
            static_for<0, kLoads>([&](auto c) {
                copy_aim(b_tag, c);
                asm volatile("s_nop 0");
                copy_fire(a_ptr, b_ptr, c);
            });
        });
    };

    // ---- first work item ----
    unsigned int draw = 0;
    const bool drawer = tid == 0;
    if (drawer) draw = sched_draw(p.sched, streams);       // always one draw ahead: its round trip hides behind a tile
    long long q = blockIdx.x;                              // the first item needs no draw (see sched_item)
    if (q < total) {
        open_tile(q);
        issue_prologue();
    }

    while (q < total) {
        const int cur_row0 = row0, cur_rows_e = rows_e, cur_n0 = n0;
        const int cur_part = part, cur_split_tile = split_tile;
        // 16-row fragments of this wavefront that hold at least one valid row (a short last tile skips the rest)
        int nfr = ((rows_e < kDM ? rows_e : kDM) - wm * TM + 15) / 16;
        nfr = __builtin_amdgcn_readfirstlane(nfr < 0 ? 0 : (nfr > FM ? FM : nfr));

        auto run_tile = [&](auto guard_tag) {
            constexpr bool kGuard = decltype(guard_tag)::value;
            // ---- per-lane addresses of the operand reads (see gmm_tile256.h), worked out per tile: registers that live
            // from the top of the kernel across the epilogue would be spilled, and a reload inside the loop makes the
            // compiler wait for every copy in flight ----
            const int l16 = lane & 15, g16 = lane >> 4;
            // address registers for buffers 0, 1 and for 2, 3 (an LDS instruction's offset field reaches 64 KiB), the
            // rest is the instruction's constant
            int fa_addr[2], fb_addr[2][FN];
            {
                const int fa_base = (wm * TM + l16) * 64 + ((g16 ^ kc_swizzle(l16)) << 4);
                fa_addr[0] = fa_base; fa_addr[1] = fa_base + 2 * kStage;
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    // SWIGLU: the wavefront's 128 columns are 64 gate columns and the 64 up columns of the same outputs
                    const int slot0 = SWIGLU ? ((j < FN / 2) ? wn * (TN / 2) + j * 16 : kDN / 2 + wn * (TN / 2) + (j - FN / 2) * 16)
                                             : wn * TN + j * 16;
                    const int col = slot0 + 4 * (l16 & 3);
                    const int krow = g16 * 8 + (l16 >> 2);
                    const int chunk = (col >> 3) ^ kn_swizzle(krow);   // k-row krow + 4 has the same swizzle
                    fb_addr[0][j] = kStageA + krow * 512 + chunk * 16 + (col & 7) * 2;
                    fb_addr[1][j] = fb_addr[0][j] + 2 * kStage;
                }
            }
            bf16x8 fa[2][FM], fb[2][FN];
            auto read_a = [&](auto buf_tag, int i) {       // row fragment i of the stage in buffer kBuf
                constexpr int kBuf = decltype(buf_tag)::value;
                const u32x4 x = *(const u32x4 *)(smem + fa_addr[kBuf >> 1] + ((kBuf & 1) * kStage + i * (16 * 64)));
                bf16x8 v;
                __builtin_memcpy(&v, &x, 16);
                return v;
            };
            auto read_b = [&](auto buf_tag, int j) {       // column fragment j of the stage in buffer kBuf
                constexpr int kBuf = decltype(buf_tag)::value;
                const char *src = smem + fb_addr[kBuf >> 1][j] + (kBuf & 1) * kStage;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)DMOE_LDS_PTR(src));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)DMOE_LDS_PTR(src + 4 * 512));
                const s16x8 v8 = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                bf16x8 v;
                __builtin_memcpy(&v, &v8, 16);
                return v;
            };
            f32x4 acc[FM][FN];
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

            // stage 0 has landed (the other three of the prologue may be in flight; stores of the previous epilogue are
            // older than all of them: waiting for fewer is only stricter)
            DMOE_WAIT_VMCNT(3 * kLoads);
            __syncthreads();
#pragma unroll
            for (int j = 0; j < FN; ++j) fb[0][j] = read_b(std::integral_constant<int, 0>{}, j);
#pragma unroll
            for (int i = 0; i < FM; ++i) fa[0][i] = read_a(std::integral_constant<int, 0>{}, i);

            // Stage s, whose operands are in register set kBuf % 2 and came from LDS buffer kBuf.  No branch: the reads
            // of the next stage's operands, the barrier and the 8 copies of stage s + 4 are unconditional (see
            // a_stage_ptr), so every stage is the same instruction stream and leaves the same number of copies in
            // flight.
            auto stage = [&](int s, auto buf_tag) {
                constexpr int kBuf = decltype(buf_tag)::value, P = kBuf & 1;
                constexpr auto next_tag = std::integral_constant<int, (kBuf + 1) % kStages>{};
                const uint64_t a_ptr = a_stage_ptr(s + kAhead), b_ptr = b_stage_ptr(s + kAhead);
                static_for<0, FM * FN>([&](auto t_tag) {
                    constexpr int t = decltype(t_tag)::value;
                    constexpr int i = t / FN, j = t % FN;
                    if constexpr (t == kBarrierSlot) {
                        // The operand reads of this stage were issued 16 and more MFMAs ago, so waiting for them here
                        // (the barrier's own wait) costs nothing.  Stage s + 1 has landed; s + 2, s + 3 may be in flight.
                        DMOE_WAIT_VMCNT(2 * kLoads);
                        __builtin_amdgcn_sched_barrier(0);
                        __syncthreads();
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if (!kGuard || i < nfr)                // wave-uniform
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[P][j], fa[P][i], acc[i][j], 0, 0, 0);
                    // behind the barrier: the B fragments of stage s + 1 (first needed by MFMAs 0 - 7 of that stage), then
                    // its A fragments (row i by MFMA 8 i)
                    if constexpr (t > kBarrierSlot && t < 48 && t % 4 == 1) fb[P ^ 1][(t - 17) / 4] = read_b(next_tag, (t - 17) / 4);
                    if constexpr (t >= 48 && t % 2 == 0) {
                        if (!kGuard || (t - 48) / 2 < nfr) fa[P ^ 1][(t - 48) / 2] = read_a(next_tag, (t - 48) / 2);
                    }
                    // copy c into the buffer that this stage's operands came from: M0 behind MFMA 18 + 4 c, the load behind
                    // the next one
                    if constexpr (t >= 18 && t < 50 && t % 4 == 2) copy_aim(buf_tag, std::integral_constant<int, (t - 18) / 4>{});
                    if constexpr (t >= 18 && t < 50 && t % 4 == 3) copy_fire(a_ptr, b_ptr, std::integral_constant<int, (t - 18) / 4>{});
                    __builtin_amdgcn_sched_barrier(0);
                });
            };
            for (int s = 0; s < S; s += kStages) {
                stage(s, std::integral_constant<int, 0>{});
                if (s + 1 < S) stage(s + 1, std::integral_constant<int, 1>{});
                if (s + 2 < S) stage(s + 2, std::integral_constant<int, 2>{});
                if (s + 3 < S) stage(s + 3, std::integral_constant<int, 3>{});
            }
            DMOE_WAIT_VMCNT(0);                            // the copies that nobody reads
            __syncthreads();                               // the last stage has been read by everyone: its buffers may be reused

            // a piece of a split tile: its sums go to the workspace, and the piece that arrives last adds all of them up
            if (cur_part >= 0 && !meet_pieces<NW>(acc, p, plan.split, cur_split_tile, cur_part, wave, lane, kGuard ? nfr : FM))
                return;

            // ---- epilogue (see gmm_tile256.h) ----
            // 32 rows at a time through LDS (8 KiB, or 4 in the fused form, private to the wavefront, no barrier), out by
            // rows of the result: a store instruction writes 4 whole rows of 256 bytes (8 rows of 128 in the fused form).
            // The 16-byte chunk c of staged row r sits at c ^ (r & 15) (256-byte rows: a row spans all banks, and the
            // 16 rows that the lanes of an 8-byte write share a column with land in 16 different chunks) or at
            // c ^ ((r >> 1) & 7) (128-byte rows).
            constexpr int RB = FNO * 32;                   // bytes per staged row
            constexpr int CPR = RB / 16;                   // lanes that write a row out
            constexpr int RPI = 64 / CPR;                  // rows per store instruction
            char *stg = smem + wave * (32 * RB);
            auto swz = [](int row) { return CPR == 16 ? (row & 15) : ((row >> 1) & 7); };
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
        if (drawer) s_item = sched_item(draw, streams);
        __syncthreads();   // also: the staged rows have been read back
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
static int launch_wave128_one(const GmmArgs &args, hipStream_t stream) {
    const size_t lds = (size_t)4 * (256 * kDK * 2 + kStageB);
    auto kern = gmm_wave128_kernel<SWIGLU>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, 256, SWIGLU, kDK, true, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_wave128_kernel");
    return DMOE_OK;
}

}  // namespace dmoe
