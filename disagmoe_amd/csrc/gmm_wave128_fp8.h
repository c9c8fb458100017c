// fp8 (e4m3) grouped GEMM, the 256 x 256 tile on 4 wavefronts of 128 x 128 with v_mfma_f32_16x16x128_f8f6f4, operands
// staged through registers on their way to LDS.  Kept beside gmm_tile256_fp8.h as a measured alternative (tuning hook
// 8): it reads a third fewer operand bytes from LDS per MFMA, and its k-steps take as long (1.29 us against 1.30 us at
// 32768 x 32768 x K on 8 experts, where the chip runs this tile's MFMAs at 1.9 GHz for 77 % of the loop's cycles and
// the other tile's at 1.6 GHz for 85 %), while a tile's start and epilogue on one wavefront per SIMD cost 18.7 us
// against 7.4 us: 12 % slower at K = 6144, so no launch takes it by default.
//
// A k-step of this tile is 64 KiB of operands (256 rows and 256 columns of 128 bytes), so LDS holds two of them and a
// copy that goes global -> LDS directly is in flight for one k-step and a half at best (gmm_tile256_fp8.h).  Here a
// wavefront owns 128 x 128 of the tile, which leaves it half of its 512 registers beside the accumulators: all 8 + 8
// operand fragments of a k-step stay in registers (each is read from LDS ONCE per k-step) and a k-step of the lane's
// share of the global loads (16 x 16 bytes) is in flight in registers on top of the k-step that sits in LDS ahead.
//
//   * operands e4m3 bytes, K-contiguous on both sides, scales applied in the epilogue; rows of 128 bytes in LDS, read as
//     in gmm_tile256_fp8.h (lane l: row l % 16, the 16-byte chunks l / 16 and l / 16 + 4), with a swizzle of its own
//     that keeps a lane's two chunks 64 bytes apart (one address register per operand);
//   * one wavefront per SIMD, so everything shares one instruction stream: a k-step is 64 MFMAs of 32 cycles, and the
//     16 LDS writes, 16 global loads and 32 operand reads of a lane are placed one or two behind an MFMA each;
//   * the 8 x 8 MFMAs of a k-step run as four quadrants of 4 x 4 fragments, (rows, columns) = (lo, lo) (lo, hi) (hi, hi)
//     (hi, lo) in even k-steps and (lo, hi) (lo, lo) (hi, lo) (hi, hi) in odd ones.  So four fragments are done with
//     after the second quadrant (rows lo), four after the third (the columns the NEXT k-step starts with) and eight at
//     the end, and the next k-step's fragments are read into them four per quadrant: an even load on LDS instead of
//     16 KiB per wavefront within the last eight MFMAs;
//   * pieces: behind MFMA 1 + 4 m the lane writes B piece m of k-step s + 1 to the other buffer, behind MFMA 35 + 4 m
//     A piece m of k-step s + 2 to this one, and loads the piece 16 on into the registers just freed.  The barrier
//     stands in front of MFMA 33: every read of this k-step's buffer has been issued by then (the last behind MFMA 27)
//     and k-step s + 1 is complete in the other one;
//   * more pieces in flight do not help: a ring of 24 (a k-step and a half, a period of six k-steps in the code) ran
//     1.39 us per k-step against 1.33 with 16 on the same box;
//   * the MFMAs are written as asm with the accumulators tied to the upper half of the register file; the operand
//     loads are buffer loads (rows past an expert's end and columns past N read as zeros without touching memory) and
//     all memory operations are ones the compiler counts (no hand-counted waits in this kernel).
#pragma once
#include "gmm_direct.h"

namespace dmoe {

template <bool SWIGLU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gmm_wave128_fp8_kernel(const GmmArgs p) {
    constexpr int kDM = 256, NW = 4;
    constexpr int TM = 128, TN = 128;
    constexpr int FM = TM / 16, FN = TN / 16;            // 8 x 8 accumulators of 16 x 16
    constexpr int FNO = SWIGLU ? FN / 2 : FN;            // column fragments of the result
    constexpr int kStepK = 128;                          // k (= bytes per row) of a k-step
    constexpr int kBufA = kDM * kStepK, kBuf = kBufA + kDN * kStepK;   // 32 KiB of A, 64 KiB per k-step
    constexpr int kPieces = kDM * kStepK / 16 / 256;     // 16-byte pieces of A (and of B) per lane per k-step: 8
    constexpr int kStaging = 2 * kBuf;                   // 4 KiB per wavefront for the epilogue, behind the two buffers
    constexpr int BNO = SWIGLU ? kDN / 2 : kDN;
    constexpr int kBarrierSlot = 33;
    constexpr int kFlight = 16;                          // pieces of a lane in flight in registers: one k-step
    static_assert(kPieces == 8, "pieces per lane");
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
    const int T_all = p.K / kStepK;                      // k-steps of a whole tile
    const int G = gridDim.x;
    constexpr long long kPieceBytes = (long long)kDM * kDN * sizeof(float);
    // a k-step takes the time of two 32-k stages of the bf16 tile, the unit plan_work's estimates are made in
    const WorkPlan plan = plan_work((long long)s_tile_start[E] * n_tiles, G, 2 * T_all,
                                    p.arrive != nullptr ? p.partial_bytes / kPieceBytes : 0, kWsArriveCount / NW);
    const long long total = plan.items;
    const uint32_t pitch = (uint32_t)p.K;
    const int streams = (G % kXcds == 0) ? kXcds : 1;
    const bool drawer = tid == 0;

    // The LDS image of a k-step: rows of 128 bytes, the 16-byte chunk c of row r at c ^ swizzle(r).  The swizzle moves a
    // chunk inside its half of the row only (rows 2 and 4 apart in different chunks, which is what keeps the 8 lanes of a
    // cycle of ds_read_b128 on different banks), so a lane's two chunks g and g + 4 sit exactly 64 bytes apart and one
    // address register serves both.
    auto swizzle = [](int row) { return ((row >> 1) & 1) | (((row >> 2) & 1) << 1); };
    // ---- a lane's share of a k-step: piece i of A is the 16-byte chunk tid % 8 of tile row tid / 8 + 32 i, piece i of B
    // the same of column slot tid / 8 + 32 i; a wavefront's load instruction fetches 8 whole lines of 128 bytes ----
    const int pc_row = tid >> 3, pc_chunk = tid & 7;
    // where they go in a buffer: rows 32 apart share the swizzle, so piece i sits 4 KiB behind piece i - 1
    const int w_addr = pc_row * kStepK + ((pc_chunk ^ swizzle(pc_row)) << 4);
    // ---- operand reads: lane l, row l % 16, chunks g and g + 4 (g = l / 16) ----
    const int l16 = lane & 15, g16 = lane >> 4;
    const int rd = (g16 ^ swizzle(l16)) << 4;
    // LDS: [A of buffer 0][A of buffer 1][B of buffer 0][B of buffer 1], 32 KiB each, so that one address register per
    // operand reaches both buffers with an instruction's 64 KiB of offset: four registers in all (reads of A and of B,
    // writes of A and of B pieces).
    constexpr int kBufStride = kBufA;                    // from an operand's buffer 0 to its buffer 1
    constexpr int kRegionB = 2 * kBufA;                  // where the B buffers start
    const char *fa_at = smem + (wm * TM + l16) * kStepK + rd;
    const char *fb_at = smem + kRegionB + ((SWIGLU ? wn * (TN / 2) : wn * TN) + l16) * kStepK + rd;
    char *wa_at = smem + w_addr, *wb_at = smem + kRegionB + w_addr;
    auto fb_dist = [](int j) {   // bytes from fragment 0 to fragment j
        return (SWIGLU ? ((j < FN / 2) ? j * 16 : kDN / 2 + (j - FN / 2) * 16) : j * 16) * kStepK;
    };
    auto read32 = [](const char *at, int dist) {          // a lane's 32 bytes of a fragment
        const u32x4 x0 = *(const u32x4 *)(at + dist);
        const u32x4 x1 = *(const u32x4 *)(at + dist + 64);
        return i32x8{(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
    };

    // ---- state of the item ----
    int e = 0, row0 = 0, rows_e = 0, n0 = 0;
    int t_lo = 0, T = 0;                                 // k-steps [t_lo, t_lo + T) of the tile
    int part = -1, split_tile = 0;
    // Where a lane's pieces come from: buffer loads.  The item's rows of a (from its first k-step on) are one buffer and
    // the expert's columns of b from the tile's first one on another; a piece's address is the lane's offset in the first
    // piece (ONE register for both operands) plus a wave-uniform distance (k-step, 32 rows per piece, the up half), added
    // right in front of the load.  Rows past the expert's last one and columns past N lie outside the buffers: such
    // loads touch no memory and give zeros, which end in results that are never stored.
    __amdgpu_buffer_rsrc_t a_buf, b_buf;
    const uint32_t lane_off = (uint32_t)pc_row * pitch + pc_chunk * 16;
    const uint32_t pitch32 = pitch * 32u;
    constexpr int kBufferWord3 = 0x00020000;             // raw buffer of bytes (no format, no stride, range checked)

    auto open_tile = [&](long long q) {
        const WorkItem it = decode_item<kDM>(q, G, plan, T_all, n_tiles, E, s_tile_start, s_row_start);
        // (the same in every lane, and said so: addresses made of them then sit in scalar registers)
        e = __builtin_amdgcn_readfirstlane(it.tile.e);
        row0 = __builtin_amdgcn_readfirstlane(it.tile.row0);
        rows_e = __builtin_amdgcn_readfirstlane(it.tile.rows_e);
        n0 = __builtin_amdgcn_readfirstlane(it.tile.nt * BNO);
        t_lo = __builtin_amdgcn_readfirstlane(it.s_lo);
        T = __builtin_amdgcn_readfirstlane(it.s_cnt);
        part = __builtin_amdgcn_readfirstlane(it.piece);
        split_tile = __builtin_amdgcn_readfirstlane(it.split_tile);
        const uint32_t k_lo = (uint32_t)t_lo * kStepK;
        const int rows_t = rows_e < kDM ? rows_e : kDM;    // valid rows of the tile
        const char *a0 = (const char *)p.a + (uint64_t)row0 * pitch + k_lo;
        const char *b0 = (const char *)p.b + ((uint64_t)e * p.N + n0) * p.K + k_lo;
        a_buf = __builtin_amdgcn_make_buffer_rsrc((void *)a0, 0, (uint32_t)rows_t * pitch - k_lo, kBufferWord3);
        b_buf = __builtin_amdgcn_make_buffer_rsrc((void *)b0, 0, (uint32_t)(p.N - n0) * pitch - k_lo, kBufferWord3);
    };
    // piece k (0 .. 7: of A, 8 .. 15: of B) of k-step t of the item, or of its last one if there is no such k-step (a load
    // that nobody uses: the loop then has no branch)
    auto load_piece = [&](int t, int k) {
        const uint32_t step = (uint32_t)(t < T ? t : T - 1) * kStepK;
        constexpr int kHalfPieces = SWIGLU ? kPieces / 2 : kPieces;
        const int i = k < kPieces ? k : (k - kPieces) % kHalfPieces;
        // the wave-uniform part of the offset, kept apart from the lane's (an empty asm: the compiler would otherwise
        // add up lane_off + 32 i pitch for every piece once and hold 16 registers of offsets through the loop)
        uint32_t dist = step + (uint32_t)i * pitch32;
        if (SWIGLU && k - kPieces >= kHalfPieces) dist += (uint32_t)n_out * pitch;
        asm volatile("" : "+s"(dist));
        return __builtin_amdgcn_raw_buffer_load_b128(k < kPieces ? a_buf : b_buf, lane_off + dist, 0, 0);
    };
    auto store_piece = [&](int buf, int k, const u32x4 &v) {
        *(u32x4 *)((k < kPieces ? wa_at : wb_at) + buf * kBufStride + (k % kPieces) * (32 * kStepK)) = v;
    };

    unsigned int draw = 0;
    if (drawer) draw = sched_draw(p.sched, streams);       // always one draw ahead: its round trip hides behind a tile
    long long q = blockIdx.x;                              // the first item needs no draw (see sched_item)

    while (q < total) {
        open_tile(q);
        int nfr = ((rows_e < kDM ? rows_e : kDM) - wm * TM + 15) / 16;
        nfr = __builtin_amdgcn_readfirstlane(nfr < 0 ? 0 : (nfr > FM ? FM : nfr));

        f32x4 acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        // ---- the item's first pieces: k-step 0 and the A pieces of k-step 1 in LDS, the kFlight pieces behind them on
        // their way, the fragments of the first quadrant in registers ----
        u32x4 g[kFlight];                                  // the pieces in flight, a ring: piece n in g[n % kFlight]
#pragma unroll
        for (int n = 0; n < kFlight; ++n) g[n] = load_piece(n / 16, n % 16);
#pragma unroll
        for (int n = 0; n < 24; ++n) {
            store_piece(n / 16, n % 16, g[n % kFlight]);
            g[n % kFlight] = load_piece((n + kFlight) / 16, (n + kFlight) % 16);
            // (in this order: the k-steps below count on kFlight - 1 younger loads behind the piece they wait for)
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        i32x8 fa[FM], fb[FN];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            fa[x] = read32(fa_at, x * (16 * kStepK));
            fb[x] = read32(fb_at, fb_dist(x));
        }

        // K-step s of the item; kPhase fixes the LDS buffer (s % 2), the order of the quadrants and where the ring of
        // pieces stands ((16 s) % kFlight).
        auto kstep = [&](int s, auto phase_tag) {
            constexpr int kPhase = decltype(phase_tag)::value;
            constexpr int kPar = kPhase % 2;
            constexpr int kRing = (16 * kPhase) % kFlight;
            static_for<0, FM * FN>([&](auto t_tag) {
                constexpr int t = decltype(t_tag)::value;
                // quadrants of 4 x 4 fragments: even k-steps (0,0) (0,1) (1,1) (1,0), odd ones (0,1) (0,0) (1,0) (1,1)
                constexpr int qd = t / 16;
                constexpr int qr = (qd >= 2) ? 1 : 0;
                constexpr int qc = kPar == 0 ? ((qd == 1 || qd == 2) ? 1 : 0) : ((qd == 0 || qd == 3) ? 1 : 0);
                constexpr int i = qr * 4 + (t % 16) / 4, j = qc * 4 + t % 4;
                if constexpr (t == kBarrierSlot) {
                    __builtin_amdgcn_sched_barrier(0);
                    __syncthreads();
                    __builtin_amdgcn_sched_barrier(0);
                }
                asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fb[j]), "v"(fa[i]));
                // B, the half this k-step's second quadrant starts with (its registers were in use to the last k-step's end)
                if constexpr (t < 16 && t % 4 == 0) {
                    constexpr int jj = (kPar == 0 ? 4 : 0) + t / 4;
                    fb[jj] = read32(fb_at, kPar * kBufStride + fb_dist(jj));
                }
                // A, rows 4 .. 7 of this k-step
                if constexpr (t >= 15 && t < 31 && t % 4 == 3) {
                    constexpr int ii = 4 + (t - 15) / 4;
                    fa[ii] = read32(fa_at, kPar * kBufStride + ii * (16 * kStepK));
                }
                // A, rows 0 .. 3 of the next k-step (behind the barrier: it is all in LDS then)
                if constexpr (t >= 34 && t < 50 && t % 4 == 2) {
                    constexpr int ii = (t - 34) / 4;
                    fa[ii] = read32(fa_at, (kPar ^ 1) * kBufStride + ii * (16 * kStepK));
                }
                // B, the half the next k-step's first quadrant takes (done with here since slot 47)
                if constexpr (t >= 48 && t % 4 == 0) {
                    constexpr int jj = (kPar == 0 ? 4 : 0) + (t - 48) / 4;
                    fb[jj] = read32(fb_at, (kPar ^ 1) * kBufStride + fb_dist(jj));
                }
                // pieces: B piece m of k-step s + 1 into the other buffer, A piece m of k-step s + 2 into this one (free
                // behind the barrier); each one's registers then take the piece kFlight on
                if constexpr (t < 32 && t % 4 == 1) {
                    constexpr int m = t / 4;
                    store_piece(kPar ^ 1, 8 + m, g[(kRing + 24 + m) % kFlight]);
                    g[(kRing + 24 + m) % kFlight] = load_piece(s + 1 + (8 + m + kFlight) / 16, (8 + m + kFlight) % 16);
                }
                if constexpr (t >= 35 && t % 4 == 3) {
                    constexpr int m = (t - 35) / 4;
                    store_piece(kPar, m, g[(kRing + 32 + m) % kFlight]);
                    g[(kRing + 32 + m) % kFlight] = load_piece(s + 2 + (m + kFlight) / 16, (m + kFlight) % 16);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        // (pairs without a condition between them, the odd one out behind the loop: the compiler counts the loads between
        // a piece's load and its use along every path, and a k-step that may or may not run would make it wait too early)
        int s = 0;
        if constexpr (kFlight % 16 == 0) {
            for (; s + 1 < T; s += 2) {
                kstep(s, std::integral_constant<int, 0>{});
                kstep(s + 1, std::integral_constant<int, 1>{});
            }
            if (s < T) kstep(s, std::integral_constant<int, 0>{});
        } else {
            // (the ring comes round every 3 k-steps, the buffers every 2: six k-steps are one period)
            for (; s + 5 < T; s += 6) {
                kstep(s, std::integral_constant<int, 0>{});
                kstep(s + 1, std::integral_constant<int, 1>{});
                kstep(s + 2, std::integral_constant<int, 2>{});
                kstep(s + 3, std::integral_constant<int, 3>{});
                kstep(s + 4, std::integral_constant<int, 4>{});
                kstep(s + 5, std::integral_constant<int, 5>{});
            }
            if (s < T) kstep(s, std::integral_constant<int, 0>{});
            if (s + 1 < T) kstep(s + 1, std::integral_constant<int, 1>{});
            if (s + 2 < T) kstep(s + 2, std::integral_constant<int, 2>{});
            if (s + 3 < T) kstep(s + 3, std::integral_constant<int, 3>{});
            if (s + 4 < T) kstep(s + 4, std::integral_constant<int, 4>{});
        }
        // (the compiler does not know how long the MFMAs above take: the last of them has left the pipe long before the
        // first accumulator is read, 32 cycles after its issue; these wait states make sure of it)
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15");
        __syncthreads();                                   // every read of the buffers is over: the next item may write them

        // ---- next work item: its number (the epilogue below does not need it, but the draw is back by now) ----
        const int cur_row0 = row0, cur_rows_e = rows_e, cur_n0 = n0, cur_e = e;
        if (drawer) s_item = sched_item(draw, streams);

        // a piece of a split tile: its sums go to the workspace, and the piece that arrives last adds all of them up
        const bool write = part < 0 || meet_pieces<NW>(acc, p, plan.split, split_tile, part, wave, lane, nfr);
        if (write) {
            // ---- epilogue: scales, (SiLU * up), through 4 KiB of LDS private to the wavefront, out by rows ----
            constexpr int RB = FNO * 32;                   // bytes per staged row
            constexpr int kRP = 4096 / RB;                 // rows per pass: 32 in the fused form, else 16
            constexpr int CPR = RB / 16;                   // lanes that write a row out
            constexpr int RPI = 64 / CPR;                  // rows per store instruction
            char *stg = smem + kStaging + wave * 4096;
            auto swz = [](int row) { return CPR == 16 ? (row & 15) : ((row >> 1) & 7); };
            const int col0 = cur_n0 + (SWIGLU ? wn * (TN / 2) : wn * TN);
            const int rows_w = cur_rows_e - wm * TM;       // valid rows of this wavefront's part of the tile (may be <= 0)
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
            for (int pass = 0; pass < TM / kRP; ++pass) {
                if (pass * kRP >= rows_w) break;           // wave-uniform: no valid row from here on
#pragma unroll
                for (int ii = 0; ii < kRP / 16; ++ii) {
                    const int i = pass * (kRP / 16) + ii;
                    const int row = ii * 16 + l16;
                    const int r = i * 16 + l16;
                    const float sa = p.a_scale[cur_row0 + wm * TM + (r < rows_w ? r : 0)];
#pragma unroll
                    for (int j = 0; j < FNO; ++j) {
                        const float s0[4] = {sb[j][0].x, sb[j][0].y, sb[j][0].z, sb[j][0].w};
                        const float s1[4] = {sb[j][SWIGLU ? 1 : 0].x, sb[j][SWIGLU ? 1 : 0].y, sb[j][SWIGLU ? 1 : 0].z, sb[j][SWIGLU ? 1 : 0].w};
                        float v[4];
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            const float gte = acc[i][j][x] * (sa * s0[x]);
                            v[x] = SWIGLU ? silu_mul(gte, acc[i][j + FN / 2][x] * (sa * s1[x])) : gte;
                        }
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
                    *(u32x4 *)((uint16_t *)p.c + (long long)(cur_row0 + wm * TM + grow) * p.ldc + gcol) = val;
                }
            }
        }

        __syncthreads();                                   // s_item is there
        q = s_item;
        if (q < total && drawer) draw = sched_draw(p.sched, streams);
    }
    sched_finish(p.sched, drawer, draw, streams, total);
}

template <bool SWIGLU>
static int launch_wave128_fp8_one(const GmmArgs &args, hipStream_t stream) {
    const size_t lds = (size_t)2 * (256 * 128 + 256 * 128) + 4 * 4096;
    auto kern = gmm_wave128_fp8_kernel<SWIGLU>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, 256, SWIGLU, 64, true, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_wave128_fp8_kernel");
    return DMOE_OK;
}

}  // namespace dmoe
