// bf16 (and fp8 e4m3) grouped GEMM on the CDNA4 data path: tiles of 256, 128 or 64 rows by 256 columns.
//
//   * A and B tiles go global -> LDS directly (global_load_lds_dwordx4: each lane
//     fetches 16 bytes, the wavefront fills 1 KiB of LDS), no staging registers,
//     no LDS store instructions;
//   * K is cut in stages of 32; 4 stages of 32 KiB (256-row tile), 5 of 24 KiB (128) or 6 of 20 KiB (64) live
//     in LDS, so a copy is issued 3 to 5 stages before its data is needed (small tiles stream weights from
//     HBM and need the depth);
//   * the LDS images are permuted on the way in (the lane picks WHICH 16 bytes of
//     the row it fetches) so that the operand reads are bank-conflict free:
//       - K-contiguous operands ([rows][32 k] = 64 B rows): chunk ^ ((row >> 2) & 3),
//         read with ds_read_b128;
//       - B in the [K, N] layout is kept [k][256 n] (512 B rows): chunk ^ ((k & 3) << 2),
//         read with ds_read_b64_tr_b16, which transposes 4 k x 16 n inside 16 lanes
//         and hands every lane 4 consecutive k of its column - the MFMA B operand;
//   * 8 wavefronts (two per SIMD) on the 256-row tile, each with 128x64 of it; 4 wavefronts on the smaller tiles
//     (64x128 of a 128-row tile, 64x64 of a 64-row tile); 32x32 v_mfma_f32_32x32x16_bf16 accumulators; operands are
//     double buffered in registers one k-step ahead; one workgroup barrier per stage.
#pragma once
#include "gmm_common.h"

namespace dmoe {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
#define DMOE_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

// One wavefront copies 64 x 16 bytes from global memory to 1 KiB of LDS.  Lane l reads at base + off (wave-uniform
// 64-bit base in scalar registers, 32-bit unsigned lane offset) and its bytes land at lds + kLdsImm + 16 l (wave-uniform
// byte address, goes through M0).  Three instructions; written as asm so that the compiler does not serialise later
// LDS reads behind every outstanding copy: completion is tracked by hand with vmcnt (the copies complete in issue order).
template <int kLdsImm>
__device__ __forceinline__ void copy_g2lds_16(uint32_t off, uint64_t base, uint32_t lds) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(off), "s"(base), "s"(lds), "n"(kLdsImm) : "memory", "m0", "scc");
}
// The same copy with the non-temporal policy: for bytes that nobody will ask the caches for again (weights that a
// single tile streams through once); a copy probe reads 6.9 - 7.0 TB/s from HBM this way against 6.2 with the default
// policy.
template <int kLdsImm>
__device__ __forceinline__ void copy_g2lds_16_nt(uint32_t off, uint64_t base, uint32_t lds) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :: "v"(off), "s"(base), "s"(lds), "n"(kLdsImm) : "memory", "m0", "scc");
}
// a wave-uniform 64-bit value held in a VGPR pair, moved to scalar registers
__device__ __forceinline__ uint64_t to_scalar(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint32_t lds_addr(const void *p) { return (uint32_t)(uintptr_t)DMOE_LDS_PTR(p); }

// f(integral_constant<int, I>) for I = LO .. HI-1, unrolled at compile time
template <int LO, int HI, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (LO < HI) {
        f(std::integral_constant<int, LO>{});
        static_for<LO + 1, HI>(f);
    }
}
// n copies spread evenly over the MFMA slots first .. slots-1 of a k-step: the copies behind MFMA t are
// copy_slot(t) .. copy_slot(t + 1) - 1
constexpr int copy_slot(int t, int n, int first, int slots) { return t < first ? 0 : (t - first) * n / (slots - first); }
// fp8 (all copies of a stage go out in one k-step): MFMA slot behind which copy j of n goes out for the wavefront
// with number `phase`.  The copies of one wavefront are slots / n apart and the four wavefronts start one slot
// after each other, so that they do not queue up at the texture path behind the same MFMA.
constexpr int copy_slot_of(int j, int n, int slots, int phase) { return (j * (slots / n > 0 ? slots / n : 1) + phase) % slots; }

constexpr int kDN = 256;                   // tile columns
constexpr int kDK = 32;                    // k per stage
constexpr int kStageB = kDN * kDK * 2;     // 16 KiB of B per stage

// s_waitcnt with only vmcnt set (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
#define DMOE_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (15 << 8) | (((n) >> 4) << 14))

// FP8: operands are e4m3 bytes, K-contiguous on both sides (TRANS_B), a stage holds 64 k = one
// v_mfma_f32_32x32x64_f8f6f4 k-step, and per-row / per-column scales are applied in the epilogue.
// NW wavefronts (4: one per SIMD; 8: two per SIMD, each with half the accumulators, so that one can issue MFMAs
// while the other issues its reads and copies), WM of them along the rows.
// NP = 0: every wavefront copies its share of a stage and computes.  NP = 2: wavefronts NW and NW + 1 only copy
// (and draw the work items), the first NW only compute: a copy that waits for room in the memory pipeline then holds
// up no MFMA, which is what small tiles on weights streamed from HBM need.
template <int kDM, int NW, int WM, bool TRANS_B, bool SWIGLU, bool FP8, int NP = 0>
__global__ __launch_bounds__((NW + NP) * 64) __attribute__((amdgpu_waves_per_eu((NW + NP + 3) / 4, (NW + NP + 3) / 4)))
void gmm_direct_kernel(const GmmArgs p) {
    constexpr int kStageK = FP8 ? 64 : kDK;               // k per stage: 64 bytes per row either way
    static_assert(!FP8 || TRANS_B, "fp8 operands are K-contiguous");
    constexpr int WN = NW / WM;                          // wavefronts along N
    constexpr int TM = kDM / WM, TN = kDN / WN;          // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;            // 32x32 accumulators per wavefront
    constexpr int NM = FM * FN;                          // MFMAs per k-step
    constexpr int NR = FM + FN;                          // operand reads per k-step (a B read = 2 transposing reads)
    constexpr int NC = NP ? NP : NW;                     // wavefronts that copy
    constexpr int CA = kDM / (16 * NC);                  // A copies (16 rows each) per copying wavefront per stage
    constexpr int CB = 16 / NC;                          // B copies (1 KiB of the 16 KiB each)
    constexpr int kLoads = CA + CB;                      // copies per copying wavefront per stage
    constexpr int kBlock = NC * 1024;                    // LDS bytes filled by one copy of every copying wavefront
    constexpr int kStageA = kDM * kDK * 2;
    constexpr int kStage = kStageA + kStageB;
    constexpr int kStages = kDM == 256 ? 4 : (kDM == 128 ? 5 : 6);
    constexpr int BNO = SWIGLU ? kDN / 2 : kDN;
    static_assert(kDM == 64 || kDM == 128 || kDM == 256, "tile rows");
    static_assert((NW == 4 || NW == 8) && WM * WN == NW && CA >= 1 && FM >= 1 && FN >= 2 && NR <= NM, "wave layout");
    static_assert(NP == 0 || (NP == 2 && NW == 4 && !FP8), "copying wavefronts: two, beside four computing ones");
    static_assert((kStages - 1) * kLoads <= 63, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int s_tile_start[kMaxGroups + 1];
    __shared__ int s_row_start[kMaxGroups + 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // kept in a scalar register: what derives from it stays wave-uniform
    const int wm = wave / WN, wn = wave % WN;
    const int cw = NP ? wave - NW : wave;                      // number among the copying wavefronts (< 0: does not copy)
    const int E = p.E;

    build_work_list<kDM>(p, s_tile_start, s_row_start);
    __syncthreads();

    const int n_out = SWIGLU ? p.N / 2 : p.N;
    const int n_tiles = (n_out + BNO - 1) / BNO;
    const int S_all = p.K / kStageK;               // stages of a whole tile (whole stages only)
    const int G = gridDim.x;
    // tiles of the last, partly filled round are cut along K (plan_work) when the launch has a workspace for their sums
    constexpr long long kPieceBytes = (long long)kDM * kDN * sizeof(float);
    const WorkPlan plan = plan_work((long long)s_tile_start[E] * n_tiles, G, S_all,
                                    p.arrive != nullptr ? p.partial_bytes / kPieceBytes : 0, kWsArriveCount / NW);
    const long long total = plan.items;
    const uint32_t pitch = (uint32_t)p.K * (FP8 ? 1 : 2);   // bytes per row of a (and of b when K-contiguous)
    const uint32_t smem_addr = lds_addr(smem);

    // ---- per-lane constants of the global -> LDS copies ----
    // K-contiguous image: a 1 KiB block is 16 rows of 64 B; lane l fills row l/4, physical chunk l%4
    const int kc_row = lane >> 2;
    const int kc_chunk = (lane & 3) ^ ((lane >> 4) & 3);      // logical chunk stored there
    // [k][n] image: a 1 KiB block is 2 k-rows of 512 B; lane l fills k-row l/32, physical chunk l%32
    const int kn_k = 2 * cw + (lane >> 5);                    // k inside the stage, block i adds 2 NC i
    const int kn_chunk = (lane & 31) ^ ((kn_k & 3) << 2);     // logical chunk (8 columns) stored there

    // ---- per-lane constants of the operand reads ----
    const int l31 = lane & 31, kgrp = lane >> 5;
    const int fa_base = (wm * TM + l31) * 64;
    const int f_sw = (l31 >> 2) & 3;
    const int g16 = lane >> 4, i16 = lane & 15;

    __shared__ long long s_item;
    const int streams = (G % kXcds == 0) ? kXcds : 1;

    // ---- state of the tile whose copies are being issued (set by open_tile) ----
    int e = 0, row0 = 0, rows_e = 0, n0 = 0;
    int s_lo = 0, S = 0, pre = 0;        // its stages [s_lo, s_lo + S); pre = the first of them, copied ahead of its first MFMA
    int part = -1, split_tile = 0;       // piece of a split tile (-1: a whole tile) and the tile's number among those
    uint64_t a_base = 0, b_exp = 0;      // wave-uniform bases of the tile's rows of a and of the expert's weights
    uint32_t a_off[CA], b_off[CB];        // per-lane byte offsets of this wavefront's copies from those bases

    // tile column slot (0..255) -> column of b; slots past the end read the first column (never stored)
    auto b_col = [&](int slot) {
        const int rh = (SWIGLU && slot >= kDN / 2) ? slot - kDN / 2 : slot;
        const int nb = n0;
        const int base = (SWIGLU && slot >= kDN / 2) ? n_out + nb : nb;
        return base + (rh < n_out - n0 ? rh : 0);
    };
    auto locate_tile = [&](long long q) {
        const WorkItem it = decode_item<kDM>(q, G, plan, S_all, n_tiles, E, s_tile_start, s_row_start);
        e = it.tile.e; row0 = it.tile.row0; rows_e = it.tile.rows_e; n0 = it.tile.nt * BNO;
        s_lo = it.s_lo; S = it.s_cnt; pre = S < kStages ? S : kStages;
        part = it.piece; split_tile = it.split_tile;
    };
    auto open_tile = [&](long long q) {
        locate_tile(q);
        // stage s of the item is stage s_lo + s of the tile
        a_base = to_scalar((uint64_t)(uintptr_t)p.a + (uint64_t)row0 * pitch + (uint64_t)s_lo * 64);
        b_exp = to_scalar((uint64_t)(uintptr_t)p.b + (uint64_t)e * p.K * p.N * (FP8 ? 1 : 2) +
                          (uint64_t)s_lo * (TRANS_B ? 64 : (uint64_t)kDK * p.N * 2));
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            int r = (i * NC + cw) * 16 + kc_row;
            if (r >= rows_e) r = rows_e - 1;                   // clamp: loaded, never stored
            a_off[i] = (uint32_t)r * pitch + kc_chunk * 16;
        }
        if constexpr (TRANS_B) {
#pragma unroll
            for (int i = 0; i < CB; ++i) b_off[i] = (uint32_t)b_col((i * NC + cw) * 16 + kc_row) * pitch + kc_chunk * 16;
        } else {
            // block i of this wavefront holds k-rows 2 NC i + kn_k of the stage
#pragma unroll
            for (int i = 0; i < CB; ++i)
                b_off[i] = (uint32_t)(i * 2 * NC + kn_k) * (uint32_t)p.N * 2 + (uint32_t)b_col(kn_chunk * 8) * 2;
        }
    };

    // copy number c (0 .. kLoads-1) of this wavefront for stage s: first its CA blocks of A, then its CB blocks of B
    auto issue_copy = [&](int s, auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
        const uint32_t lds = smem_addr + (s % kStages) * kStage + cw * 1024;
        if constexpr (c < CA) {
            copy_g2lds_16<c * kBlock>(a_off[c], a_base + (uint64_t)s * 64, lds);
        } else {
            constexpr int i = c - CA;
            if constexpr (TRANS_B) copy_g2lds_16<kStageA + i * kBlock>(b_off[i], b_exp + (uint64_t)s * 64, lds);
            else copy_g2lds_16<kStageA + i * kBlock>(b_off[i], b_exp + (uint64_t)s * kDK * p.N * 2, lds);
        }
    };
    auto issue_prologue = [&]() {
        for (int s = 0; s < pre; ++s) {
            static_for<0, kLoads>([&](auto c) { issue_copy(s, c); });
        }
    };

    // B operand rows / columns of this wavefront: fragment j covers 32 tile columns
    int fb_off[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int slot0 = SWIGLU ? ((j < FN / 2) ? wn * (TN / 2) + j * 32 : kDN / 2 + wn * (TN / 2) + (j - FN / 2) * 32)
                                 : wn * TN + j * 32;
        if constexpr (TRANS_B) {
            fb_off[j] = (slot0 + l31) * 64;
        } else {
            const int col = slot0 + (g16 & 1) * 16 + 4 * (i16 & 3);          // tile column of this lane's 4 values
            const int chunk = (col >> 3) ^ (((i16 >> 2) & 3) << 2);
            fb_off[j] = ((kgrp * 8) + (i16 >> 2)) * 512 + chunk * 16 + (col & 7) * 2;
        }
    }

    typedef typename std::conditional<FP8, i32x8, bf16x8>::type frag_t;
    // fp8 on 8 wavefronts keeps a single register set for both operands: every fragment is re-read right behind its
    // last MFMA of the stage, and the other wavefront of the SIMD covers the wait for the last of those reads
    constexpr bool kOneSet = FP8 && NW == 8;
    frag_t fa[FP8 ? 1 : 2][FM], fb[kOneSet ? 1 : 2][FN];
    // operand read number r (0 .. NR-1) of k-step ks of stage s into register set `slot`: first the FM A fragments,
    // then the FN B fragments
    auto load_frag = [&](int s, int ks, int slot, int r) {
        const char *tA = smem + (s % kStages) * kStage;
        const char *tB = tA + kStageA;
        const int c0 = ((ks * 2 + kgrp) ^ f_sw) << 4;
        if constexpr (FP8) {
            // a lane holds 32 consecutive k of its row: chunks 2*kgrp and 2*kgrp + 1 of the 64-byte row
            const int d0 = ((kgrp * 2) ^ f_sw) << 4, d1 = ((kgrp * 2 + 1) ^ f_sw) << 4;
            const char *src = r < FM ? tA + fa_base + r * 2048 : tB + fb_off[r - FM];
            const u32x4 x0 = *(const u32x4 *)(src + d0);
            const u32x4 x1 = *(const u32x4 *)(src + d1);
            const i32x8 v = {(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
            if (r < FM) __builtin_memcpy(&fa[slot][r], &v, 32);
            else __builtin_memcpy(&fb[slot][r - FM], &v, 32);
        } else if (r < FM) {
            const u32x4 x = *(const u32x4 *)(tA + fa_base + r * 2048 + c0);
            __builtin_memcpy(&fa[slot][r], &x, 16);
        } else {
            const int j = r - FM;
            if constexpr (TRANS_B) {
                const u32x4 x = *(const u32x4 *)(tB + fb_off[j] + c0);
                __builtin_memcpy(&fb[slot][j], &x, 16);
            } else {
                const char *src = tB + fb_off[j] + ks * (16 * 512);
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)DMOE_LDS_PTR(src));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)DMOE_LDS_PTR(src + 4 * 512));
                const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                __builtin_memcpy(&fb[slot][j], &v, 16);
            }
        }
    };

    // wait until at most n * kLoads of this wavefront's copies are outstanding (n known only at run time)
    auto wait_ahead = [&](int n) {
        if (n >= 5) DMOE_WAIT_VMCNT(5 * kLoads > 63 ? 63 : 5 * kLoads);
        else if (n == 4) DMOE_WAIT_VMCNT(4 * kLoads > 63 ? 63 : 4 * kLoads);
        else if (n == 3) DMOE_WAIT_VMCNT(3 * kLoads);
        else if (n == 2) DMOE_WAIT_VMCNT(2 * kLoads);
        else if (n == 1) DMOE_WAIT_VMCNT(kLoads);
        else DMOE_WAIT_VMCNT(0);
    };

    // ---- first work item ----
    unsigned int draw = 0;
    const bool drawer = tid == (NP ? NW * 64 : 0);
    if (drawer) draw = sched_draw(p.sched, streams);   // always one draw ahead: its round trip hides behind a tile
    long long q = blockIdx.x;                          // the first item needs no draw (see sched_item)
    if (q < total) {
        if (NP == 0 || cw >= 0) {
            open_tile(q);
            issue_prologue();
        } else {
            locate_tile(q);
        }
    }

    if constexpr (NP > 0) {
        if (cw >= 0) {
            // ---- a copying wavefront: the same barriers as the computing ones, tile by tile ----
            while (q < total) {
                wait_ahead(pre - 1);
                __syncthreads();                   // stage 0 has landed
                for (int s = 0; s + 1 < S; ++s) {
                    const int left = S - 1 - s;    // stages after s; s + 1 has to land, the ones behind it may be in flight
                    wait_ahead(left - 1 < kStages - 2 ? left - 1 : kStages - 2);
                    __syncthreads();               // hand-over: stage s + 1 is there, stage s has been read
                    if (s + kStages < S) static_for<0, kLoads>([&](auto c) { issue_copy(s + kStages, c); });
                }
                if (drawer) s_item = sched_item(draw, streams);
                __syncthreads();                   // the last stage has been read: all of the LDS may be refilled
                q = s_item;
                if (q < total) {
                    if (drawer) draw = sched_draw(p.sched, streams);
                    open_tile(q);
                    issue_prologue();
                }
            }
            sched_finish(p.sched, drawer, draw, streams, total);
            return;
        }
    }

    while (q < total) {
        // results of this tile go here after the next tile's copies have been issued
        const int cur_row0 = row0, cur_rows_e = rows_e, cur_n0 = n0, cur_e = e;
        const int cur_part = part, cur_split_tile = split_tile;
        // row fragments of this wavefront that hold at least one valid row (a short last tile skips the rest)
        int nfr = ((rows_e < kDM ? rows_e : kDM) - wm * TM + 31) / 32;
        nfr = __builtin_amdgcn_readfirstlane(nfr < 0 ? 0 : (nfr > FM ? FM : nfr));

        // The tile from its first MFMA to its last store, in two builds: without any branch around the MFMAs (every
        // row fragment of this wavefront holds rows: all but the last tile of an expert) and with one per MFMA.
        // Wavefronts of one workgroup may take different builds; both execute the same copies and barriers.
        auto run_tile = [&](auto guard_tag, auto phase_tag) {
        constexpr bool kGuard = decltype(guard_tag)::value;
        f32x16 acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int x = 0; x < 16; ++x) acc[i][j][x] = 0.f;
        auto mfma_one = [&](int slot, int t) {
            const int i = t / FN, j = t % FN;
            if (kGuard && i >= nfr) return;   // wave-uniform: a scalar branch around the MFMA
            if constexpr (!FP8)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
        };
        auto mfma_one_fp8 = [&](int bslot, int t) {
            const int i = t / FN, j = t % FN;
            if (kGuard && i >= nfr) return;
            if constexpr (FP8)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[bslot][j], fa[0][i], acc[i][j], 0, 0, 0, 0, 0, 0);
        };

        // stage 0 of this tile has landed (its other prologue stages, and stores of the previous tile's
        // epilogue that were issued after them, may still be in flight: waiting for fewer is only stricter)
        if constexpr (NP == 0) wait_ahead(pre - 1);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < NR; ++r) load_frag(0, 0, 0, r);

        // One stage = 2 k-steps of NM MFMAs.  A wavefront issues in order and an MFMA occupies the matrix pipe
        // for 32 cycles, so the LDS reads and global -> LDS copies are slotted one per MFMA: they are issued in
        // the shadow of the MFMA before them and the pipe never waits for the issue port.
        //   k-step 0: MFMAs on register set 0; the NR operand reads of k-step 1 go to set 1.
        //   hand-over: this wavefront's share of stage s+1 has landed (vmcnt), barrier (everybody's has, and
        //              every read of stage s is complete).
        //   k-step 1: MFMAs on set 1; the NR operand reads of stage s+1 go to set 0; the copies that refill the LDS
        //              stage just drained with stage s + kStages are spread over this k-step and the next one.
        // kSteady: the copies of s+1 .. s+kStages-1 are in flight; otherwise `ahead` stages after s+1 are.
        // FP8: a stage is a single k-step, so the hand-over comes first and the register sets alternate by stage:
        // MFMAs of stage s run on set s % 2 while stage s+1 is read into the other set.
        // copies c with slot_lo(t) <= c < slot_lo(t + 1) go out behind MFMA t: n copies spread evenly over the NM slots
        // (the texture path moves one 1 KiB copy per 16 cycles for the whole CU; bunched copies back up into the
        // issue queues of all four wavefronts)
        auto run_stage = [&](int s, auto steady_tag, int ahead, bool next, bool deferred, auto odd_tag) {
            constexpr bool kSteady = decltype(steady_tag)::value;
            constexpr int kCur = FP8 ? (!kOneSet && decltype(odd_tag)::value ? 1 : 0) : 1;   // set used by the MFMAs after the hand-over
            constexpr int kFirst = FP8 ? kLoads : kLoads / 2;   // copies of stage s + kStages issued in this stage
            constexpr int kLate = kLoads - kFirst;              // ... and behind the MFMAs of k-step 0 of the next stage
            // bf16: copies go behind the MFMAs that have no operand read if those slots suffice
            constexpr int kSlot0 = FP8 ? 0 : (NM - NR >= kLate ? NR : 0);
            if constexpr (!FP8) {
                static_for<0, NM>([&](auto t_tag) {
                    constexpr int t = decltype(t_tag)::value;
                    mfma_one(0, t);
                    if (t < NR) load_frag(s, 1, 1, t);
                    if (NP == 0 && deferred) {
                        static_for<copy_slot(t, kLate, kSlot0, NM), copy_slot(t + 1, kLate, kSlot0, NM)>(
                            [&](auto c) { issue_copy(s - 1 + kStages, std::integral_constant<int, kFirst + decltype(c)::value>{}); });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
            if (kSteady || next) {
                if constexpr (NP > 0) {}   // the copying wavefronts wait for the data
                else if constexpr (kSteady) DMOE_WAIT_VMCNT((kStages - 2) * kLoads);
                else wait_ahead(ahead);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            static_for<0, NM>([&](auto t_tag) {
                constexpr int t = decltype(t_tag)::value;
                if constexpr (FP8) {
                    // 8 registers per operand: A fragments live in one register set and are re-read for stage s+1
                    // right behind their last MFMA of this stage; B fragments alternate between two sets.
                    mfma_one_fp8(kCur, t);
                    if (kSteady || next) {
                        if constexpr (kOneSet) {
                            if (t >= NM - FN) load_frag(s + 1, 0, 0, FM + t - (NM - FN));   // B fragment j, last used by MFMA t
                        } else {
                            if (t < FN) load_frag(s + 1, 0, kCur ^ 1, FM + t);
                        }
                        if ((t % FN) == FN - 1) load_frag(s + 1, 0, 0, t / FN);
                    }
                } else {
                    mfma_one(kCur, t);
                    if ((kSteady || next) && t < NR) load_frag(s + 1, 0, kCur ^ 1, t);
                }
                if constexpr (kSteady && NP == 0) {
                    if constexpr (FP8) {
                        static_for<0, kFirst>([&](auto c) {
                            if constexpr (copy_slot_of(decltype(c)::value, kFirst, NM, decltype(phase_tag)::value) == t)
                                issue_copy(s + kStages, c);
                        });
                    } else {
                        static_for<copy_slot(t, kFirst, kSlot0, NM), copy_slot(t + 1, kFirst, kSlot0, NM)>(
                            [&](auto c) { issue_copy(s + kStages, c); });
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        auto step = [&](int s, auto steady_tag, int ahead, bool next, bool deferred) {
            if (FP8 && !kOneSet && (s & 1)) run_stage(s, steady_tag, ahead, next, deferred, std::true_type{});
            else run_stage(s, steady_tag, ahead, next, deferred, std::false_type{});
        };
        int s = 0;
        if constexpr (FP8 && !kOneSet) {
            // even and odd stages as one straight-line loop body: the accumulators stay where they are
            for (; s + 1 + kStages < S; s += 2) {
                run_stage(s, std::true_type{}, 0, true, false, std::false_type{});
                run_stage(s + 1, std::true_type{}, 0, true, false, std::true_type{});
            }
        }
        // bf16: the second half of a stage's copies goes out one stage later, behind the MFMAs of k-step 0; the first
        // stage after the steady ones still owes the late copies of the last steady stage
        for (; s + kStages < S; ++s) step(s, std::true_type{}, 0, true, !FP8 && s > 0);
        for (; s < S; ++s) {
            const int left = S - 1 - s;                           // stages after this one
            step(s, std::false_type{}, left - 1 < kStages - 2 ? left - 1 : kStages - 2, left > 0,
                 !FP8 && s > 0 && s + kStages == S);
        }

        if constexpr (NP > 0) {
            __syncthreads();   // every wavefront has read its last fragments: the copying wavefronts may refill the LDS
            q = s_item;        // the next work item, written by them before the barrier
        }

        auto epilogue = [&]() {
            // ---- epilogue of the finished tile ----
            // The MFMAs take the B fragment as their first operand, so an accumulator holds the tile transposed:
            // lane l owns output row l % 32 of its fragment and, in element x, column (x/4)*8 + (l/32)*4 + x%4:
            // of every group of 8 columns the lower half of the wavefront holds the first 4, the upper half the last 4.
            // Two groups at a time, the halves trade (v_permlane32_swap) what the other needs to own 8 consecutive
            // columns: the lower half those of the first group, the upper half those of the second.  One 16-byte store
            // per lane, 32 bytes per row and instruction; a row is valid or not for both lanes that share it.
            constexpr int FNO = SWIGLU ? FN / 2 : FN;
            const int col0 = cur_n0 + (SWIGLU ? wn * (TN / 2) : wn * TN);
            // fp8 on 8 wavefronts: every scale this lane needs is fetched up front, all loads in flight together.  Rows
            // and columns outside the tile read a valid neighbour; their results are never stored.  (On 4 wavefronts the
            // registers for that are not there: the loads stay inside the loops.)
            constexpr bool kScalesUpFront = FP8 && NW == 8;
            float sa_all[kScalesUpFront ? FM : 1];
            float4 sb_all[kScalesUpFront ? FNO * 4 * (SWIGLU ? 2 : 1) : 1];
            if constexpr (kScalesUpFront) {
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    const int r = wm * TM + i * 32 + l31;
                    sa_all[i] = p.a_scale[cur_row0 + (r < cur_rows_e ? r : 0)];
                }
#pragma unroll
                for (int j = 0; j < FNO; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int col = col0 + kgrp * 4 + j * 32 + g * 8;
                        const float *sb = p.b_scale + (long long)cur_e * p.N + (col < n_out ? col : cur_n0);
                        sb_all[(j * 4 + g) * (SWIGLU ? 2 : 1)] = *(const float4 *)sb;
                        if (SWIGLU) sb_all[(j * 4 + g) * 2 + 1] = *(const float4 *)(sb + n_out);
                    }
            }
            // Beside computing-only kernels the 16-byte pieces then pass through LDS (the stage buffer after the last
            // stage's, private 4 KiB per wavefront, free until the next tile's copies are issued behind the barrier that
            // follows): a block of 32 rows x 64 (or 32) columns goes in by row of the fragment and comes out by row of
            // the result, so that a store instruction writes 8 whole rows of 128 bytes (16 of 64), not 32 pieces of 32.
            // Chunks are placed at chunk ^ (row & 7) (128-byte rows) or chunk ^ ((row >> 1) & 3) (64-byte rows, two to a
            // line of banks): the writes and the reads are free of bank conflicts.
            constexpr bool kViaLds = NP == 0;
            constexpr int CW = FNO >= 2 ? 2 : 1;          // fragments (of 32 columns) staged together
            constexpr int RB = CW * 64;                   // bytes per staged row
            constexpr int CPR = RB / 16;                  // 16-byte chunks per row = lanes that write a row out
            constexpr int RPI = 64 / CPR;                 // rows per store instruction
            char *stg = smem + (S % kStages) * kStage + wave * 4096;
            auto swz = [](int row) { return CPR == 8 ? (row & 7) : ((row >> 1) & 3); };
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const int r = wm * TM + i * 32 + l31;
                const bool row_ok = r < cur_rows_e;
                if (!kViaLds && !row_ok) continue;
                uint16_t *crow = (uint16_t *)p.c + (long long)(cur_row0 + r) * p.ldc + col0;
                float sa = 1.f;
                if constexpr (kScalesUpFront) sa = sa_all[i];
                else if constexpr (FP8) sa = p.a_scale[cur_row0 + (row_ok ? r : 0)];
#pragma unroll
                for (int j = 0; j < FNO; ++j) {
#pragma unroll
                    for (int gp = 0; gp < 4; gp += 2) {
                        uint2 pk[2];
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int g = gp + h;
                            float sb0[4] = {1.f, 1.f, 1.f, 1.f}, sb1[4] = {1.f, 1.f, 1.f, 1.f};
                            if constexpr (kScalesUpFront) {
                                const float4 t0 = sb_all[(j * 4 + g) * (SWIGLU ? 2 : 1)];
                                sb0[0] = t0.x; sb0[1] = t0.y; sb0[2] = t0.z; sb0[3] = t0.w;
                                if (SWIGLU) {
                                    const float4 t1 = sb_all[(j * 4 + g) * 2 + 1];
                                    sb1[0] = t1.x; sb1[1] = t1.y; sb1[2] = t1.z; sb1[3] = t1.w;
                                }
                            } else if constexpr (FP8) {
                                const int col = col0 + kgrp * 4 + j * 32 + g * 8;   // the 4 columns whose values this lane holds
                                if (col < n_out) {   // n_out % 8 == 0: a group of 8 columns is inside or outside as a whole
                                    const float4 t0 = *(const float4 *)(p.b_scale + (long long)cur_e * p.N + col);
                                    sb0[0] = t0.x; sb0[1] = t0.y; sb0[2] = t0.z; sb0[3] = t0.w;
                                    if (SWIGLU) {
                                        const float4 t1 = *(const float4 *)(p.b_scale + (long long)cur_e * p.N + n_out + col);
                                        sb1[0] = t1.x; sb1[1] = t1.y; sb1[2] = t1.z; sb1[3] = t1.w;
                                    }
                                }
                            }
                            float v[4];
#pragma unroll
                            for (int x = 0; x < 4; ++x) {
                                if (SWIGLU) {
                                    const float gate = acc[i][j][g * 4 + x] * (sa * sb0[x]);
                                    v[x] = silu_mul(gate, acc[i][j + FN / 2][g * 4 + x] * (sa * sb1[x]));
                                } else {
                                    v[x] = acc[i][j][g * 4 + x] * (sa * sb0[x]);
                                }
                            }
                            pk[h].x = pack_bf16x2(v[0], v[1]);
                            pk[h].y = pack_bf16x2(v[2], v[3]);
                        }
                        // lower half: [0] = its own part of group gp, [1] = the upper half's; upper half: [0] = the lower
                        // half's part of group gp + 1, [1] = its own
                        const auto lo = __builtin_amdgcn_permlane32_swap(pk[0].x, pk[1].x, false, false);
                        const auto hi = __builtin_amdgcn_permlane32_swap(pk[0].y, pk[1].y, false, false);
                        const u32x4 piece = {lo[0], hi[0], lo[1], hi[1]};
                        if constexpr (kViaLds) {
                            const int cidx = (j % CW) * 4 + gp + kgrp;          // chunk of the staged row this lane holds
                            *(u32x4 *)(stg + l31 * RB + ((cidx ^ swz(l31)) << 4)) = piece;
                            if ((j % CW) == CW - 1 && gp == 2) {
                                // the block is complete: out by rows
#pragma unroll
                                for (int q = 0; q < 32 / RPI; ++q) {
                                    const int row = q * RPI + lane / CPR, c = lane % CPR;
                                    const u32x4 val = *(const u32x4 *)(stg + row * RB + ((c ^ swz(row)) << 4));
                                    const int grow = wm * TM + i * 32 + row;
                                    const int gcol = col0 + (j - (CW - 1)) * 32 + c * 8;
                                    if (grow >= cur_rows_e || gcol >= n_out) continue;
                                    *(u32x4 *)((uint16_t *)p.c + (long long)(cur_row0 + grow) * p.ldc + gcol) = val;
                                }
                            }
                        } else {
                            const int cst = j * 32 + (gp + kgrp) * 8;           // the 8 columns this lane stores
                            if (col0 + cst >= n_out) continue;
                            *(u32x4 *)(crow + cst) = piece;
                        }
                    }
                }
            }
        };
        // a piece of a split tile: its sums go to the workspace, and the piece that arrives last adds all of them up
        if (cur_part < 0 || meet_pieces<NW>(acc, p, plan.split, cur_split_tile, cur_part, wave, lane, FM))
            epilogue();
        };   // run_tile
        // fp8: one instance per wavefront number (the MFMA slots of its copies are compile-time constants)
        auto run_build = [&](auto guard_tag) {
            if constexpr (FP8) {
                if constexpr (NW == 8) {
                    run_tile(guard_tag, std::integral_constant<int, 0>{});   // two wavefronts per SIMD: no staggering needed
                } else {
                    if (wave == 0) run_tile(guard_tag, std::integral_constant<int, 0>{});
                    else if (wave == 1) run_tile(guard_tag, std::integral_constant<int, 1>{});
                    else if (wave == 2) run_tile(guard_tag, std::integral_constant<int, 2>{});
                    else run_tile(guard_tag, std::integral_constant<int, 3>{});
                }
            } else {
                run_tile(guard_tag, std::integral_constant<int, 0>{});
            }
        };
        if (nfr == FM) run_build(std::false_type{});
        else run_build(std::true_type{});

        auto next_item = [&]() {
            // ---- next work item and its first copies ----
            if (drawer) s_item = sched_item(draw, streams);
            __syncthreads();   // also: the last stage has been read by everyone, LDS may be refilled
            q = s_item;
            if (q < total) {
                if (drawer) draw = sched_draw(p.sched, streams);
                open_tile(q);
                issue_prologue();
            }
        };
        // stores first: they are then older than the next tile's copies and never hold up a vmcnt wait of its pipeline
        if constexpr (NP == 0) next_item();
        else if (q < total) locate_tile(q);
    }
    sched_finish(p.sched, drawer, draw, streams, total);
}

template <int kDM, int NW, int WM, bool TRANS_B, bool SWIGLU, bool FP8, int NP = 0>
static int launch_direct_one(const GmmArgs &args, hipStream_t stream) {
    constexpr int kStages = kDM == 256 ? 4 : (kDM == 128 ? 5 : 6);
    const size_t lds = (size_t)kStages * (kDM * kDK * 2 + kStageB);
    auto kern = gmm_direct_kernel<kDM, NW, WM, TRANS_B, SWIGLU, FP8, NP>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, kDM, SWIGLU, FP8 ? 64 : kDK, true, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3((NW + NP) * 64), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_direct_kernel");
    return DMOE_OK;
}

template <int kDM, int NW, int WM, int NP = 0>
static int launch_direct_tile(const GmmArgs &args, bool trans_b, bool swiglu, hipStream_t stream) {
    if (trans_b) return swiglu ? launch_direct_one<kDM, NW, WM, true, true, false, NP>(args, stream) : launch_direct_one<kDM, NW, WM, true, false, false, NP>(args, stream);
    return swiglu ? launch_direct_one<kDM, NW, WM, false, true, false, NP>(args, stream) : launch_direct_one<kDM, NW, WM, false, false, false, NP>(args, stream);
}

}  // namespace dmoe
