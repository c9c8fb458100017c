// bf16 grouped GEMM, the 256 x 256 tile on 4 wavefronts of 128 x 128 with v_mfma_f32_16x16x32_bf16, as ONE software
// pipeline over all the work items of a workgroup.
//
// The chip is power-limited under MFMA load, and what the loop does besides the MFMAs is paid for in clock.  A wavefront
// that owns 128 x 128 of the tile reads 8 + 8 operand fragments from LDS for its 64 MFMAs of a stage, one of 128 x 64
// reads 8 + 4 for 32: a third fewer LDS bytes per MFMA, and half the barriers.  The price is one wavefront per SIMD (its
// 256 accumulator registers are the upper half of the register file), so the operand reads, the global -> LDS copies
// and the MFMAs of a stage share one instruction stream: whatever is not an MFMA has to be issued in the shadow of one,
// at most two instructions behind each, and nothing in the loop may wait.
//
//   * weights in the [K, N] layout; LDS images, swizzles and copies as in gmm_tile256.h: 4 stage buffers of 32 KiB,
//     K in stages of 32;
//   * a stage is 8 rows of 8 MFMAs (row fragment i against the 8 column fragments) on one of two register sets; the
//     16 operand fragments of the next stage are read into the other set while this one is multiplied, so an LDS
//     buffer is free again a whole stage before its stage is multiplied: the registers are a fifth buffer;
//   * ONE barrier per stage, in front of its MFMA 16.  Before it a wavefront has waited for its own copies of the next
//     stage; behind it everybody's are there and everybody has read this stage (during the stage before), so the
//     copies of the stage four on go into this stage's buffer, one every 4 MFMAs, and the reads of the next stage
//     begin: a copy is in flight for 2.5 to 3 stages, and an operand read is at least 16 MFMAs old when the next
//     barrier waits for it;
//   * the copies run four stages ahead of the MFMAs whatever item those stages belong to, so a new tile's first
//     operands are in LDS when the last MFMA of the tile before it has been issued, and no tile starts by waiting for
//     memory.  What separates two tiles is the epilogue alone, which has an LDS staging area of its own (the stage
//     buffers are never free).  Every item is a whole number of rounds of the four buffers (K % 128 == 0, pieces of
//     split tiles cut at multiples of four stages), so every item begins in buffer 0 and the loop over a tile's
//     stages is a plain counted loop;
//   * a short last tile of an expert runs all its MFMAs (rows past the expert's end are clamped copies that are never
//     stored); a wavefront without any valid row runs none.
//
// Needs K % 128 == 0 and K >= 256 (an item is at least 8 stages, so that the copies are never more than one item ahead).
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
    constexpr int kStaging = kStages * kStage;           // 4 KiB per wavefront for the epilogue, behind the stage buffers
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
    const uint32_t b_stride = (uint32_t)kDK * (uint32_t)p.N * 2;   // bytes from a stage of the weights to the next
    const uint32_t smem_addr = lds_addr(smem);
    const int streams = (G % kXcds == 0) ? kXcds : 1;
    const bool drawer = tid == 0;

    long long q = blockIdx.x;                              // the first item needs no draw (see sched_item)
    unsigned int draw = 0;
    if (drawer) draw = sched_draw(p.sched, streams);       // always one draw ahead: its round trip hides behind a tile
    if (q >= total) {
        sched_finish(p.sched, drawer, draw, streams, total);
        return;
    }

    // ---- per-lane constants of the global -> LDS copies ----
    // A: a 1 KiB block is 16 rows of 64 B, lane l fills row l / 4, physical chunk l % 4; block i of this wavefront
    // holds rows 64 wave + 16 i ... of the tile.  B: a block is 2 k-rows of 512 B, lane l fills k-row l / 32, physical
    // chunk l % 32; block i of this wavefront holds k-rows 8 wave + 2 i, + 1 of the stage.
    auto kc_swizzle = [](int row) { return ((row >> 2) & 1) << 1; };
    auto kn_swizzle = [](int k) { return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1); };

    // An item as the MFMAs and the epilogue see it.
    struct Item {
        int row0, rows_e, n0, S, part, split_tile;
    };

    // ---- the copies' item: they run kStages stages ahead of the MFMAs ----
    // What the copies need of an item: where its stages begin, and the per-lane offsets of this wavefront's blocks.
    struct CopyItem {
        Item item;
        uint64_t a_ptr, b_ptr;                             // its first stage: rows of a, rows of the expert's weights
        uint32_t a_off[CA], b_off[CB];
    };
    CopyItem cp{};                                         // the item whose stages are being copied
    CopyItem pend{};                                       // the item after it, decoded ahead of time (see take_next)
    bool pend_valid = false;
    int cp_left = 0;                                       // stages of cp that have not been issued
    uint64_t a_cp = 0, b_cp = 0;                           // the next stage to copy
    uint32_t a_adv = 64, b_adv = b_stride;                 // what a stage adds to them (0 past the last item)

    auto decode_copies = [&](long long item, CopyItem &c) {
        const WorkItem it = decode_item<kDM, kStages>(item, G, plan, S_all, n_tiles, E, s_tile_start, s_row_start);
        // (wave-uniform values that come out of LDS tables: into scalar registers, so that what is decided on them in
        // the loop is a scalar branch and no vector register has to be kept, or spilled, for it)
        auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
        c.item.row0 = uni(it.tile.row0); c.item.rows_e = uni(it.tile.rows_e); c.item.n0 = uni(it.tile.nt * BNO);
        c.item.S = uni(it.s_cnt); c.item.part = uni(it.piece); c.item.split_tile = uni(it.split_tile);
        c.a_ptr = to_scalar((uint64_t)(uintptr_t)p.a + (uint64_t)c.item.row0 * pitch + (uint64_t)it.s_lo * 64);
        c.b_ptr = to_scalar((uint64_t)(uintptr_t)p.b + (uint64_t)it.tile.e * p.K * p.N * 2 + (uint64_t)it.s_lo * b_stride);
        const int kc_row = lane >> 2;
        const int kc_chunk = (lane & 3) ^ kc_swizzle(kc_row);
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            int r = (wave * CA + i) * 16 + kc_row;
            if (r >= c.item.rows_e) r = c.item.rows_e - 1; // clamp: loaded, never stored
            c.a_off[i] = (uint32_t)r * pitch + kc_chunk * 16;
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int k = wave * 8 + 2 * i + (lane >> 5);
            const int slot = ((lane & 31) ^ kn_swizzle(k)) * 8;
            // tile column slot (0 .. 255) -> column of b; slots past the end read a valid column (never stored)
            const int rh = (SWIGLU && slot >= kDN / 2) ? slot - kDN / 2 : slot;
            const int base = (SWIGLU && slot >= kDN / 2) ? n_out + c.item.n0 : c.item.n0;
            c.b_off[i] = (uint32_t)k * (uint32_t)p.N * 2 + (uint32_t)(base + (rh < n_out - c.item.n0 ? rh : 0)) * 2;
        }
    };
    // The item after the copies' one, decoded where registers are free and nothing is in the way (at the start, and
    // behind every epilogue): the drawer's number goes round through LDS, and the loop later only swaps it in.
    auto take_next = [&]() {
        if (drawer) s_item = sched_item(draw, streams);
        __syncthreads();
        q = to_scalar((uint64_t)s_item);
        pend_valid = q < total;
        if (pend_valid) {
            if (drawer) draw = sched_draw(p.sched, streams);
            decode_copies(q, pend);
        }
    };
    // Copy c (0 .. 7: 4 blocks of A, 4 of B) of this wavefront for the copies' next stage into LDS buffer kBuf.  In two
    // halves, so that an MFMA can stand between the write of M0 and the load that reads it (the wait state the
    // hardware asks for) and no gap between two MFMAs holds more than two other instructions.
    const uint32_t lds_wave = smem_addr + wave * 4096;
    auto copy_aim = [&](auto buf_tag, auto c_tag) {
        constexpr int c = decltype(c_tag)::value, kBuf = decltype(buf_tag)::value;
        constexpr int imm = kBuf * kStage + (c < CA ? c * 1024 : kStageA + (c - CA) * 1024);
        const uint32_t base = lds_wave;                    // (an asm operand cannot name a captured variable)
        asm volatile("s_add_u32 m0, %0, %1" :: "s"(base), "n"(imm) : "m0", "scc");
    };
    auto copy_fire = [&](auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
        uint32_t off;
        if constexpr (c < CA) off = cp.a_off[c]; else off = cp.b_off[c - CA];
        const uint64_t ptr = c < CA ? a_cp : b_cp;
        asm volatile("global_load_lds_dwordx4 %0, %1" :: "v"(off), "s"(ptr) : "memory");
    };
    // The copies' item has been issued to its last stage: on to the next one, which take_next has prepared.  Past the
    // last item the copies repeat the last stage, which nobody reads: the loop keeps one shape, and every stage leaves
    // the same number of copies in flight.
    bool cp_switch = false;                                // (wave-uniform) the next stage's copies belong to a new item
    bool have_next = false;                                // the copies have begun an item that the MFMAs have not
    auto next_copies = [&]() {
        if (pend_valid) {
            cp = pend;
            a_cp = cp.a_ptr; b_cp = cp.b_ptr;
            cp_left = cp.item.S;
            have_next = true;
            pend_valid = false;
        } else {
            a_cp -= a_adv; b_cp -= b_adv;                  // back to the last stage, and stay there
            a_adv = 0; b_adv = 0;
            cp_left = 1 << 30;
        }
        cp_switch = false;
    };

    // ---- first item: its first kStages stages ----
    decode_copies(q, cp);
    a_cp = cp.a_ptr; b_cp = cp.b_ptr;
    cp_left = cp.item.S;
    Item cur = cp.item;                                    // the item being multiplied
    static_for<0, kStages>([&](auto b_tag) {
        static_for<0, kLoads>([&](auto c) {
            copy_aim(b_tag, c);
            asm volatile("s_nop 0");
            copy_fire(c);
        });
        a_cp += a_adv; b_cp += b_adv;
    });
    cp_left -= kStages;                                    // (from here on counted round by round, in buffer 3)

    // ---- per-lane addresses of the operand reads (see gmm_tile256.h) ----
    const int l16 = lane & 15, g16 = lane >> 4;
    // address registers for buffers 0, 1 and for 2, 3 (an LDS instruction's offset field reaches 64 KiB), the rest is
    // the instruction's constant
    int fa_addr[2], fb_addr[2][FN];
    // (worked out anew behind every epilogue rather than kept across it: the epilogue needs the registers, and a
    // register that is spilled around it is reloaded inside the loop, where the compiler then waits for every copy in
    // flight)
    auto set_read_addresses = [&]() {
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
    };
    set_read_addresses();
    bf16x8 fa[2][FM], fb[2][FN];
    auto read_a = [&](auto buf_tag, int i) {               // row fragment i of the stage in buffer kBuf
        constexpr int kBuf = decltype(buf_tag)::value;
        const u32x4 x = *(const u32x4 *)(smem + fa_addr[kBuf >> 1] + ((kBuf & 1) * kStage + i * (16 * 64)));
        bf16x8 v;
        __builtin_memcpy(&v, &x, 16);
        return v;
    };
    auto read_b = [&](auto buf_tag, int j) {               // column fragment j of the stage in buffer kBuf
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

    take_next();
    // the first stage has landed (the other three may be in flight): its operands into register set 0
    DMOE_WAIT_VMCNT(3 * kLoads);
    __syncthreads();
    // all operands of the stage in buffer kBuf into register set kBuf % 2
    auto read_stage = [&](auto buf_tag) {
        constexpr int P = decltype(buf_tag)::value & 1;
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[P][j] = read_b(buf_tag, j);
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[P][i] = read_a(buf_tag, i);
    };
    read_stage(std::integral_constant<int, 0>{});

    // One stage of the pipeline: the MFMAs of the stage whose operands are in register set kBuf % 2 (they came from
    // LDS buffer kBuf), the reads of the next stage's operands from buffer kBuf + 1, the copies of the stage kStages on
    // into buffer kBuf.  `live`: this wavefront has rows in the current item (else it runs no MFMA).
    auto stage_as = [&](auto buf_tag, auto live_tag) {
        constexpr int kBuf = decltype(buf_tag)::value, P = kBuf & 1;
        constexpr bool kLive = decltype(live_tag)::value;
        constexpr auto next_tag = std::integral_constant<int, (kBuf + 1) % kStages>{};
        static_for<0, FM * FN>([&](auto t_tag) {
            constexpr int t = decltype(t_tag)::value;
            constexpr int i = t / FN, j = t % FN;
            if constexpr (t == kBarrierSlot) {
                // The operand reads of this stage were issued 16 and more MFMAs ago, so waiting for them here (the
                // barrier's own wait) costs nothing.  The next stage has landed; the two behind it may be in flight.
                DMOE_WAIT_VMCNT(2 * kLoads);
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                // (an item's last stage is copied while the MFMAs are 5 stages from its end, in buffer 3: the copies move
                // on behind the next barrier, which is buffer 0's)
                if constexpr (kBuf == 0) {
                    if (cp_switch) next_copies();
                }
            }
            // (as asm with the accumulator tied to the upper half of the register file: left to itself the compiler keeps
            // part of the accumulators in the lower half around the epilogue and moves them to and fro in the loop)
            if constexpr (kLive)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fb[P][j]), "v"(fa[P][i]));
            // behind the barrier: the B fragments of the next stage (first needed by its MFMAs 0 - 7), then its A
            // fragments (row i by MFMA 8 i)
            if constexpr (t > kBarrierSlot && t < 48 && t % 4 == 1) fb[P ^ 1][(t - 17) / 4] = read_b(next_tag, (t - 17) / 4);
            if constexpr (t >= 48 && t % 2 == 0) fa[P ^ 1][(t - 48) / 2] = read_a(next_tag, (t - 48) / 2);
            // copy c into the buffer that this stage's operands came from: M0 behind MFMA 18 + 4 c, the load behind the
            // next one
            if constexpr (t >= 18 && t < 50 && t % 4 == 2) copy_aim(buf_tag, std::integral_constant<int, (t - 18) / 4>{});
            if constexpr (t >= 18 && t < 50 && t % 4 == 3) copy_fire(std::integral_constant<int, (t - 18) / 4>{});
            // the copies' next stage; when that was the item's last, the copies move on behind the next barrier
            if constexpr (t == 51) a_cp += a_adv;
            if constexpr (t == 53) b_cp += b_adv;
            if constexpr (t == 55 && kBuf == kStages - 1) {
                if ((cp_left -= kStages) == 0) {             // a scalar branch, taken once per item
                    cp_switch = true;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    auto stage = [&](auto buf_tag, bool) { stage_as(buf_tag, std::true_type{}); };

    // Finishes the current item: a piece of a split tile meets the others, and whoever holds the tile's sums writes the
    // result (see gmm_tile256.h); the accumulators are zero afterwards.
    auto finish_item = [&]() {
        // a piece of a split tile: its sums go to the workspace, and the piece that arrives last adds all of them up
        // (row fragments of this wavefront without a valid row stay out of it: the same ones in every piece of a tile)
        int nfr = (cur.rows_e - wm * TM + 15) / 16;
        nfr = nfr < 0 ? 0 : (nfr > FM ? FM : nfr);
        const bool write = cur.part < 0 || meet_pieces<NW>(acc, p, plan.split, cur.split_tile, cur.part, wave, lane, nfr);
        // ---- epilogue ----
        // Lane l holds, of fragment (i, j), row i * 16 + l % 16 and the 4 columns j * 16 + (l / 16) * 4 ...: 8 bytes of
        // the result.  kRP rows at a time they pass through 4 KiB of LDS private to the wavefront (no barrier) and
        // leave by rows of the result, 16 bytes per lane: a store instruction writes 4 whole rows of 256 bytes (8 rows
        // of 128 in the fused form).  The 16-byte chunk c of staged row r sits at c ^ (r & 15) (256-byte rows: a row
        // spans all banks, and the 16 rows that the lanes of an 8-byte write share a column with land in 16 different
        // chunks) or at c ^ ((r >> 1) & 7) (128-byte rows).
        constexpr int RB = FNO * 32;                       // bytes per staged row
        constexpr int kRP = 4096 / RB;                     // rows per pass: 32 in the fused form, else 16
        constexpr int CPR = RB / 16;                       // lanes that write a row out
        constexpr int RPI = 64 / CPR;                      // rows per store instruction
        char *stg = smem + kStaging + wave * 4096;
        auto swz = [](int row) { return CPR == 16 ? (row & 15) : ((row >> 1) & 7); };
        const int col0 = cur.n0 + (SWIGLU ? wn * (TN / 2) : wn * TN);
        const int rows_w = cur.rows_e - wm * TM;           // valid rows of this wavefront's part of the tile (may be <= 0)
#pragma unroll
        for (int pass = 0; pass < TM / kRP; ++pass) {
            if (write && pass * kRP < rows_w) {            // wave-uniform
#pragma unroll
                for (int ii = 0; ii < kRP / 16; ++ii) {
                    const int i = pass * (kRP / 16) + ii;
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
                for (int t = 0; t < kRP / RPI; ++t) {
                    const int row = t * RPI + lane / CPR, c = lane % CPR;
                    const u32x4 val = *(const u32x4 *)(stg + row * RB + ((c ^ swz(row)) << 4));
                    const int grow = pass * kRP + row;
                    const int gcol = col0 + c * 8;
                    if (grow >= rows_w || gcol >= n_out) continue;
                    *(u32x4 *)((uint16_t *)p.c + (long long)(cur.row0 + wm * TM + grow) * p.ldc + gcol) = val;
                }
            }
#pragma unroll
            for (int ii = 0; ii < kRP / 16; ++ii)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[pass * (kRP / 16) + ii][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };

    // ---- the pipeline: item after item, each a whole number of rounds of the four buffers ----
    for (;;) {
        const bool live = cur.rows_e > wm * TM;
        for (int s = 0; s < cur.S; s += kStages) {
            stage(std::integral_constant<int, 0>{}, live);
            stage(std::integral_constant<int, 1>{}, live);
            stage(std::integral_constant<int, 2>{}, live);
            stage(std::integral_constant<int, 3>{}, live);
        }
        // (the compiler does not know how long the MFMAs above take: the last of them has long left the pipe before the
        // first accumulator is read, 16 cycles after its issue; these wait states make sure of it)
        asm volatile("s_nop 15\n\ts_nop 15");
        finish_item();
        if (!have_next) break;
        cur = cp.item;
        have_next = false;
        take_next();                                       // (behind the epilogue, which has outlasted every copy in flight)
        // The next item's first operands were read during the last stage, but they are not kept across the epilogue
        // (see set_read_addresses): once more from their buffer, which is refilled behind the next barrier.
        set_read_addresses();
        read_stage(std::integral_constant<int, 0>{});
    }
    DMOE_WAIT_VMCNT(0);                                    // the copies that nobody reads
    sched_finish(p.sched, drawer, draw, streams, total);
}

template <bool SWIGLU>
static int launch_wave128_one(const GmmArgs &args, hipStream_t stream) {
    const size_t lds = (size_t)4 * (256 * kDK * 2 + kStageB) + 4 * 4096;
    auto kern = gmm_wave128_kernel<SWIGLU>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, 256, SWIGLU, kDK, true, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_wave128_kernel");
    return DMOE_OK;
}

}  // namespace dmoe
