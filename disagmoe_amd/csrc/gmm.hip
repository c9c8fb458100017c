// Ragged grouped GEMM on CDNA4 matrix cores (bf16 and fp8-e4m3), with an
// optional fused SiLU(gate)*up epilogue for the gate-up projection.
//
// Shape of the kernel
//   * persistent: one workgroup per compute unit walks a list of
//     (expert, m-tile, n-tile) work items that every workgroup derives from
//     batch_sizes on the device (prefix sums kept in LDS), so zero-row experts
//     cost nothing and no host round trip or scratch table is needed;
//   * work items are ordered m-fastest inside an n-tile, and consecutive blocks
//     of items are handed to the workgroups of one XCD (workgroup id % 8), so the
//     m-tiles that share a weight tile run next to each other on one L2;
//   * a K-slice of 128 bytes per row (64 bf16 / 128 fp8) of the A and B tiles is
//     staged global -> registers -> LDS, double buffered; rows are 128 bytes in
//     LDS with the 16-byte chunk index XOR-swizzled by the row so that both the
//     MFMA operand reads and the staging writes spread over the banks;
//   * B in the [E, K, N] layout (N contiguous) is transposed 8x8 in registers on
//     its way into LDS so that both MFMA operands are read K-contiguous;
//   * each wavefront owns a TM x TN sub-tile as FM x FN accumulators of
//     v_mfma_f32_32x32x16_bf16 (v_mfma_f32_32x32x64_f8f6f4 for fp8).
#include <mutex>

#include "gmm_common.h"
#include "tuning.h"

namespace dmoe {

constexpr int kRowBytes = 128;     // bytes of K per tile row in LDS
constexpr int kDK32 = 32;          // k per stage of the global -> LDS bf16 kernels (gmm_direct.h)

// XOR applied to the 16-byte chunk index of a 128-byte LDS row.  Its period is
// 16 rows, so fragment rows 32 apart differ by a constant.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int lds_off(int row, int chunk) { return row * kRowBytes + ((chunk ^ swz(row)) << 4); }

template <int BM, int BN, int WM, int WN, bool TRANS_B, bool SWIGLU, bool FP8>
__global__ __launch_bounds__(WM *WN *kWave) __attribute__((amdgpu_waves_per_eu(WM *WN / 4, WM *WN / 4)))
void gmm_kernel(const GmmArgs p) {
    constexpr int NT = WM * WN * kWave;          // threads
    constexpr int ES = FP8 ? 1 : 2;              // element bytes
    constexpr int BK = kRowBytes / ES;           // elements of K per tile
    constexpr int TM = BM / WM, TN = BN / WN;    // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;    // 32x32 accumulators per wave
    constexpr int KS = FP8 ? 2 : 4;              // MFMA k-steps per tile
    constexpr int CA = BM * 8 / NT;              // 16-byte chunks of A per thread per tile
    constexpr int CB = BN * 8 / NT;
    constexpr int RSTEP = NT / 8;                // row stride between a thread's chunks
    constexpr int BNO = SWIGLU ? BN / 2 : BN;    // output columns per tile
    constexpr int KR = BK * (BN / 8) / NT;       // [E,K,N] layout: k-rows of one 8-column group per thread
    constexpr int KG = BK / KR;                  // such groups along K
    constexpr bool FRAG_DB = (WM * WN == 4);     // one wave per SIMD: double-buffer the MFMA operands
    constexpr int STEP_KS = FP8 ? 1 : 2;         // two waves per SIMD: MFMA k-steps per ping-pong phase
    constexpr int SLOTS = FRAG_DB ? 2 : STEP_KS;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile");
    static_assert(CA >= 1 && CB >= 1 && (BM * 8) % NT == 0 && (BN * 8) % NT == 0, "staging split");
    static_assert(RSTEP % 32 == 0 && (BN / 2) % RSTEP == 0, "staging rows keep their swizzle and their half");
    static_assert(TRANS_B || ((KR == 8 || KR == 4) && CB == KR), "register transpose handles 8x8 or 4x8 blocks");
    static_assert(WM * WN % 4 == 0, "whole waves per SIMD");
    static_assert(!SWIGLU || FN % 2 == 0, "gate and up fragments pair up inside a wave");
    static_assert(!FP8 || TRANS_B, "fp8 operands are K-contiguous");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int s_tile_start[kMaxGroups + 1];  // m-tiles before expert e
    __shared__ int s_row_start[kMaxGroups + 1];   // rows before expert e
    char *sA = smem;                              // [2][BM][128]
    char *sB = smem + 2 * BM * kRowBytes;         // [2][BN][128]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int wm = wave / WN, wn = wave % WN;
    const int E = p.E;

    build_work_list<BM>(p, s_tile_start, s_row_start);
    __syncthreads();

    const int n_out = SWIGLU ? p.N / 2 : p.N;            // output columns
    const int n_tiles = (n_out + BNO - 1) / BNO;
    const int m_tiles = s_tile_start[E];
    const long long total = (long long)m_tiles * n_tiles;
    const int KT = (p.K * ES + kRowBytes - 1) / kRowBytes;
    const int G = gridDim.x;
    const uint32_t a_pitch = (uint32_t)(p.K * ES);       // bytes per row of a (and of b when K-contiguous)

    // per-thread staging coordinates
    const int a_chunk = tid & 7;
    const int a_row0 = tid >> 3;
    const int b_kg = tid % KG;         // [E,K,N] layout: group of KR k-rows ...
    const int b_ng = tid / KG;         //                 ... of 8 columns
    const int st_off = lds_off(a_row0, a_chunk);         // rows RSTEP apart share the swizzle

    // per-lane MFMA operand coordinates: row = base + lane % 32, k-group = lane / 32
    const int l31 = lane & 31;
    const int kgrp = lane >> 5;
    const int fa_off = (wm * TM + l31) * kRowBytes;
    const int fb_off = ((SWIGLU ? wn * (TN / 2) : wn * TN) + l31) * kRowBytes;
    const int fsw = swz(l31);

    __shared__ long long s_item;
    const int streams = (G % kXcds == 0) ? kXcds : 1;
    unsigned int draw = 0;
    if (tid == 0) draw = sched_draw(p.sched, streams);       // always one draw ahead
    bool first = true;                                       // the first item needs no draw (see sched_item)
    for (;;) {
        if (tid == 0) s_item = first ? (long long)blockIdx.x : sched_item(draw, streams);
        __syncthreads();
        const long long q = s_item;
        if (q >= total) break;
        if (tid == 0 && !first) draw = sched_draw(p.sched, streams);   // next item; the round trip hides behind this tile
        first = false;
        const TileCoord tc = decode_tile<BM>(item_order(q, G, total), n_tiles, E, s_tile_start, s_row_start);
        const int e = tc.e, nt = tc.nt, row0 = tc.row0, rows_e = tc.rows_e;
        const int n0 = nt * BNO;                               // first output column

        // ---- staging offsets (bytes from wave-uniform bases) ----
        const char *a_base = p.a + (long long)row0 * a_pitch;
        const char *b_exp = p.b + (long long)e * p.K * p.N * ES;
        const int n0_b = n0;
        // first column of the tile; the swiglu form reads a second run of columns (the up half)
        const char *b_base0, *b_base1;
        if constexpr (TRANS_B) {
            b_base0 = b_exp + (long long)n0_b * a_pitch;
            b_base1 = SWIGLU ? b_exp + (long long)(n_out + n0_b) * a_pitch : b_base0;
        } else {
            b_base0 = b_exp + (long long)n0_b * ES;
            b_base1 = SWIGLU ? b_exp + (long long)(n_out + n0_b) * ES : b_base0;
        }
        const int half_cols = SWIGLU ? n_out - n0 : p.N - n0;  // valid columns from the first column of half 0
        uint32_t a_off[CA];
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            int r = a_row0 + i * RSTEP;
            if (r >= rows_e) r = rows_e - 1;                   // clamp: loaded, never stored
            a_off[i] = (uint32_t)r * a_pitch + a_chunk * 16;
        }
        // columns past the end of b are clamped to column 0 of their half: loaded, never stored
        uint32_t b_off[TRANS_B ? CB : 1];
        if constexpr (TRANS_B) {
#pragma unroll
            for (int i = 0; i < CB; ++i) {
                const int r = a_row0 + i * RSTEP;              // row of the B tile = output column slot
                const int rh = (SWIGLU && r >= BN / 2) ? r - BN / 2 : r;  // column from its base
                b_off[i] = (uint32_t)(rh < half_cols ? rh : 0) * a_pitch + a_chunk * 16;
            }
        } else {
            const int r = b_ng * 8;                            // first of 8 columns, all in one half
            const int rh = (SWIGLU && r >= BN / 2) ? r - BN / 2 : r;
            b_off[0] = (uint32_t)(rh < half_cols ? rh : 0) * ES;   // N % 8 == 0: the 8 columns are valid together
        }
        const bool b_hi_half = !TRANS_B && SWIGLU && (b_ng * 8 >= BN / 2);

        u32x4 ra[CA], rb[CB];
        // kTail: the tile reaches past K; bytes past the end of a row are read as zero
        auto load_global = [&](int kt, auto tail_tag) {
            constexpr bool kTail = decltype(tail_tag)::value;
            const bool k_ok = !kTail || (kt * kRowBytes + a_chunk * 16 < p.K * ES);
            const char *ak = a_base + (long long)kt * kRowBytes;
#pragma unroll
            for (int i = 0; i < CA; ++i) {
                if (kTail) ra[i] = u32x4{0, 0, 0, 0};
                if (k_ok) ra[i] = *(const u32x4 *)(ak + a_off[i]);
            }
            if constexpr (TRANS_B) {
#pragma unroll
                for (int i = 0; i < CB; ++i) {
                    const char *bk = ((SWIGLU && i * RSTEP >= BN / 2) ? b_base1 : b_base0) + (long long)kt * kRowBytes;
                    if (kTail) rb[i] = u32x4{0, 0, 0, 0};
                    if (k_ok) rb[i] = *(const u32x4 *)(bk + b_off[i]);
                }
            } else {
                const int k_first = kt * BK + b_kg * KR;
                const char *bk = (b_hi_half ? b_base1 : b_base0) + (long long)k_first * p.N * ES + b_off[0];
#pragma unroll
                for (int j = 0; j < KR; ++j) {
                    if (kTail) rb[j] = u32x4{0, 0, 0, 0};
                    if (!kTail || k_first + j < p.K) rb[j] = *(const u32x4 *)(bk + (long long)j * p.N * ES);
                }
            }
        };
        const int KT_full = (p.K * ES) / kRowBytes;            // tiles that lie inside K entirely
        auto load_tile = [&](int kt) {
            if (kt < KT_full) load_global(kt, std::false_type{});
            else load_global(kt, std::true_type{});
        };
        auto store_lds = [&](int buf) {
            char *dA = sA + buf * BM * kRowBytes + st_off;
            char *dB = sB + buf * BN * kRowBytes;
#pragma unroll
            for (int i = 0; i < CA; ++i) *(u32x4 *)(dA + i * RSTEP * kRowBytes) = ra[i];
            if constexpr (TRANS_B) {
#pragma unroll
                for (int i = 0; i < CB; ++i) *(u32x4 *)(dB + st_off + i * RSTEP * kRowBytes) = rb[i];
            } else if constexpr (KR == 8) {
                // rb[j] holds k = j, columns 0..7 (dword c = columns 2c, 2c+1); column n wants k = 0..7
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    u32x4 even, odd;
#pragma unroll
                    for (int c2 = 0; c2 < 4; ++c2) {
                        const uint32_t x = rb[2 * c2][c], y = rb[2 * c2 + 1][c];
                        even[c2] = (x & 0xffffu) | (y << 16);
                        odd[c2] = (x >> 16) | (y & 0xffff0000u);
                    }
                    *(u32x4 *)(dB + lds_off(b_ng * 8 + 2 * c, b_kg)) = even;
                    *(u32x4 *)(dB + lds_off(b_ng * 8 + 2 * c + 1, b_kg)) = odd;
                }
            } else {
                // 4 k-rows per thread: each column gets half a chunk (8 bytes)
                const int half = (b_kg & 1) * 8;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    uint2 even, odd;
                    const uint32_t x0 = rb[0][c], y0 = rb[1][c], x1 = rb[2][c], y1 = rb[3][c];
                    even.x = (x0 & 0xffffu) | (y0 << 16);
                    even.y = (x1 & 0xffffu) | (y1 << 16);
                    odd.x = (x0 >> 16) | (y0 & 0xffff0000u);
                    odd.y = (x1 >> 16) | (y1 & 0xffff0000u);
                    *(uint2 *)(dB + lds_off(b_ng * 8 + 2 * c, b_kg >> 1) + half) = even;
                    *(uint2 *)(dB + lds_off(b_ng * 8 + 2 * c + 1, b_kg >> 1) + half) = odd;
                }
            }
        };

        typedef typename std::conditional<FP8, i32x8, bf16x8>::type frag_t;
        frag_t fa[SLOTS][FM], fb[SLOTS][FN];
        auto frag_row_b = [&](int j) {  // row offset of B fragment j from fb_off, in rows
            if (SWIGLU) return (j < FN / 2) ? j * 32 : BN / 2 + (j - FN / 2) * 32;
            return j * 32;
        };
        auto load_frags = [&](int buf, int ks, int slot) {
            const char *tA = sA + buf * BM * kRowBytes + fa_off;
            const char *tB = sB + buf * BN * kRowBytes + fb_off;
            if constexpr (FP8) {
                const int c0 = ((ks * 4 + kgrp * 2) ^ fsw) << 4, c1 = ((ks * 4 + kgrp * 2 + 1) ^ fsw) << 4;
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    const u32x4 x0 = *(const u32x4 *)(tA + i * 32 * kRowBytes + c0);
                    const u32x4 x1 = *(const u32x4 *)(tA + i * 32 * kRowBytes + c1);
                    const i32x8 v = {(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
                    fa[slot][i] = v;
                }
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const u32x4 x0 = *(const u32x4 *)(tB + frag_row_b(j) * kRowBytes + c0);
                    const u32x4 x1 = *(const u32x4 *)(tB + frag_row_b(j) * kRowBytes + c1);
                    const i32x8 v = {(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
                    fb[slot][j] = v;
                }
            } else {
                const int c0 = ((ks * 2 + kgrp) ^ fsw) << 4;
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    const u32x4 x = *(const u32x4 *)(tA + i * 32 * kRowBytes + c0);
                    __builtin_memcpy(&fa[slot][i], &x, sizeof(x));
                }
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const u32x4 x = *(const u32x4 *)(tB + frag_row_b(j) * kRowBytes + c0);
                    __builtin_memcpy(&fb[slot][j], &x, sizeof(x));
                }
            }
        };
        // row fragments of this wavefront that hold at least one valid row (a short last tile skips the rest)
        int nfr = ((rows_e < BM ? rows_e : BM) - wm * TM + 31) / 32;
        nfr = nfr < 0 ? 0 : (nfr > FM ? FM : nfr);
        auto mfma_all = [&](f32x16 (&acc)[FM][FN], int slot) {
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                if (i >= nfr) continue;
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    if constexpr (FP8)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[slot][j], fa[slot][i], acc[i][j], 0, 0, 0, 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
                }
            }
        };

        f32x16 acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int x = 0; x < 16; ++x) acc[i][j][x] = 0.f;

        // ---- prologue ----
        load_tile(0);
        store_lds(0);
        if (KT > 1) load_tile(1);
        __syncthreads();
        if constexpr (FRAG_DB) load_frags(0, 0, 0);

        // ---- main loop over K tiles ----
        if constexpr (FRAG_DB) {
            for (int kt = 0; kt < KT; ++kt) {
                const int cur = kt & 1;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int slot = ks & 1;
                    if (ks + 1 < KS) load_frags(cur, ks + 1, slot ^ 1);
                    if (ks == KS - 2) {
                        if (kt + 1 < KT) store_lds(cur ^ 1);
                        if (kt + 2 < KT) load_tile(kt + 2);
                    }
                    if (ks == KS - 1) {
                        __syncthreads();
                        if (kt + 1 < KT) load_frags(cur ^ 1, 0, slot ^ 1);
                    }
                    mfma_all(acc, slot);
                }
            }
        } else {
            // Two waves share a SIMD.  The two halves of the workgroup run half a step apart: while one
            // half issues its LDS/global traffic for a step, the other half issues the MFMAs of its step,
            // and the barriers hand the roles over.  Waves w and w + 4 sit on the same SIMD.
            const int grp = wave >> 2;
            if (grp == 1) __syncthreads();
            for (int kt = 0; kt < KT; ++kt) {
                const int cur = kt & 1;
#pragma unroll
                for (int st = 0; st < KS / STEP_KS; ++st) {
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < STEP_KS; ++u) load_frags(cur, st * STEP_KS + u, u);
                    if (st == 0) {
                        if (kt + 1 < KT) store_lds(cur ^ 1);
                        if (kt + 2 < KT) load_tile(kt + 2);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    __syncthreads();
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_s_setprio(1);
#pragma unroll
                    for (int u = 0; u < STEP_KS; ++u) mfma_all(acc, u);
                    __builtin_amdgcn_s_setprio(0);
                    __builtin_amdgcn_sched_barrier(0);
                    __syncthreads();
                }
            }
            if (grp == 0) __syncthreads();
        }

        // ---- epilogue ----
        // The MFMAs take the B fragment as their first operand, so an accumulator holds the tile transposed:
        // lane l owns output row l % 32 of its fragment and, in element x, column (x/4)*8 + (l/32)*4 + x%4.
        // Four consecutive columns per lane -> one 8-byte store; a row is valid or not per lane.
        constexpr int FNO = SWIGLU ? FN / 2 : FN;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int r = wm * TM + i * 32 + l31;
            if (r >= rows_e) continue;
            const int col_lane = n0 + (SWIGLU ? wn * (TN / 2) : wn * TN) + kgrp * 4;
            uint16_t *crow = (uint16_t *)p.c + (long long)(row0 + r) * p.ldc + col_lane;
            float sa = 1.f;
            if (FP8) sa = p.a_scale[row0 + r];
#pragma unroll
            for (int j = 0; j < FNO; ++j) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int col = col_lane + j * 32 + g * 8;
                    if (col >= n_out) continue;                 // n_out % 8 == 0: four columns at once
                    float sb0[4] = {1.f, 1.f, 1.f, 1.f}, sb1[4] = {1.f, 1.f, 1.f, 1.f};
                    if (FP8) {
                        const float4 t0 = *(const float4 *)(p.b_scale + (long long)e * p.N + col);
                        sb0[0] = t0.x; sb0[1] = t0.y; sb0[2] = t0.z; sb0[3] = t0.w;
                        if (SWIGLU) {
                            const float4 t1 = *(const float4 *)(p.b_scale + (long long)e * p.N + n_out + col);
                            sb1[0] = t1.x; sb1[1] = t1.y; sb1[2] = t1.z; sb1[3] = t1.w;
                        }
                    }
                    float v[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        if (SWIGLU) {
                            const float gate = acc[i][j][g * 4 + x] * (sa * sb0[x]);
                            const float up = acc[i][j + FN / 2][g * 4 + x] * (sa * sb1[x]);
                            v[x] = silu_mul(gate, up);
                        } else {
                            v[x] = acc[i][j][g * 4 + x] * (sa * sb0[x]);
                        }
                    }
                    uint2 packed;
                    packed.x = pack_bf16x2(v[0], v[1]);
                    packed.y = pack_bf16x2(v[2], v[3]);
                    *(uint2 *)(crow + j * 32 + g * 8) = packed;
                }
            }
        }
    }
    sched_finish(p.sched, tid == 0, draw, streams, total);
}

template <int BM, int BN, int WM, int WN, bool TRANS_B, bool SWIGLU, bool FP8>
static int launch_one(const GmmArgs &args, hipStream_t stream) {
    constexpr int NT = WM * WN * kWave;
    static_assert(BN == 256, "launch_grid counts tiles of 256 columns");
    const size_t lds = 2 * (size_t)(BM + BN) * kRowBytes;
    auto kern = gmm_kernel<BM, BN, WM, WN, TRANS_B, SWIGLU, FP8>;
    static unsigned long long configured = 0;   // devices on which the kernel's LDS size has been raised
    DMOE_HIP(raise_dynamic_lds((const void *)kern, (int)lds, &configured));
    const long long grid = launch_grid(args, BM, SWIGLU, 64, false, device_cus());
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), lds, stream, args);
    DMOE_LAUNCH_CHECK("gmm_kernel");
    return DMOE_OK;
}

static int g_variant = 0;  // tuning hook, see dmoe_gmm_tune
thread_local const int64_t *t_host_sizes = nullptr;
namespace {
// the host copy of the sizes for the length of one call
struct HostSizes {
    explicit HostSizes(const int64_t *p) { t_host_sizes = p; }
    ~HostSizes() { t_host_sizes = nullptr; }
};
}  // namespace

// ---- where a launch keeps its counters ----------------------------------------------------------------
// With a state block of the caller: there, the split tiles' arrival counters behind them, and the partial sums in
// the caller's workspace.  Without one: in a slot of the library's own, one per stream per device (launches on one stream do not overlap, launches on
// different streams get different slots); nothing is split then.  A launch that is being recorded into a graph may
// be replayed on any stream at any time, so it must bring its own state block.
constexpr int kOwnSlots = 64;
static __device__ SchedSlot g_own_slots[kOwnSlots];

static int own_slot(hipStream_t stream, SchedSlot **out) {
    struct Entry { int dev; hipStream_t stream; };
    static std::mutex mu;
    static Entry table[64][kOwnSlots];
    static int used[64];
    static SchedSlot *base[64];
    int dev = 0;
    DMOE_HIP(hipGetDevice(&dev));
    DMOE_REQUIRE(dev >= 0 && dev < 64, DMOE_ERR_ARG, "grouped GEMM: device ordinal %d outside [0, 64)", dev);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) (void)hipGetLastError();
    DMOE_REQUIRE(capture == hipStreamCaptureStatusNone, DMOE_ERR_WORKSPACE,
                 "grouped GEMM: a launch recorded into a graph needs a caller-owned state block (DMOE_GMM_STATE_BYTES)");
    std::lock_guard<std::mutex> lock(mu);
    if (base[dev] == nullptr) {
        void *ptr = nullptr;
        DMOE_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_own_slots)));
        base[dev] = (SchedSlot *)ptr;
    }
    int slot = -1;
    for (int i = 0; i < used[dev]; ++i)
        if (table[dev][i].stream == stream) { slot = i; break; }
    if (slot < 0 && used[dev] == kOwnSlots) {
        // every slot has had a stream: take over one whose stream has no work pending (its last launch has returned the
        // counters to zero) or no longer exists
        for (int i = 0; i < kOwnSlots && slot < 0; ++i) {
            const hipError_t busy = hipStreamQuery(table[dev][i].stream);
            if (busy != hipSuccess) (void)hipGetLastError();
            if (busy != hipErrorNotReady) slot = i;
        }
        DMOE_REQUIRE(slot >= 0, DMOE_ERR_WORKSPACE,
                     "grouped GEMM: %d streams on device %d have launches without a state block pending; pass one", kOwnSlots, dev);
        table[dev][slot] = Entry{dev, stream};
    }
    if (slot < 0) {
        slot = used[dev]++;
        table[dev][slot] = Entry{dev, stream};
    }
    *out = base[dev] + slot;
    return DMOE_OK;
}

static int bind_state(GmmArgs &args, void *state, void *workspace, size_t workspace_bytes, hipStream_t stream) {
    args.arrive = nullptr; args.partials = nullptr; args.partial_bytes = 0;
    args.a_rows = nullptr; args.a_src_rows = 0;
    if (state == nullptr) return own_slot(stream, &args.sched);
    DMOE_REQUIRE(((uintptr_t)state & 255) == 0, DMOE_ERR_WORKSPACE, "grouped GEMM: the state block must be 256-byte aligned");
    args.sched = (SchedSlot *)state;
    if (workspace != nullptr && workspace_bytes > 0) {
        DMOE_REQUIRE(((uintptr_t)workspace & 15) == 0, DMOE_ERR_WORKSPACE, "grouped GEMM: the workspace must be 16-byte aligned");
        args.arrive = (unsigned int *)((char *)state + kWsArriveOffset);
        args.partials = (float *)workspace;
        args.partial_bytes = (long long)workspace_bytes;
    }
    return DMOE_OK;
}

// Kernel, tile rows and grid of a launch, from what the host knows (the shapes, not how the rows split over the experts).
// The one place where that is decided: launch_by_rows dispatches on the result and dmoe_gmm_plan reports it.
static GmmLaunch choose_launch(const GmmArgs &args, bool trans_b, bool swiglu, bool fp8) {
    const int cus = device_cus();
    GmmLaunch L{};
    if (g_variant >= 1 && g_variant <= 4) {   // test hook: the register-staged kernel with a fixed tile
        L.kernel = kKernelStaged;
        L.tile_rows = g_variant == 2 ? 64 : (g_variant == 3 ? 128 : 256);
        L.waves = g_variant == 4 ? 8 : 4;
    } else {
        // Tile rows.  Every m-tile streams its 256 columns of the weights through the CU whatever its rows, so fewer,
        // taller tiles move fewer bytes (decode-sized batches: 8 tiles of 256 rows instead of 12 of 64 on a Zipf batch of
        // 512 rows, 10 % off the gate-up launch) and a tile's empty row fragments cost no MFMAs: 256 rows wherever such
        // tiles fill the CUs, and where 128-row tiles would need a second round for what 256-row tiles do in one (a
        // small batch on few experts: 176 half-filled tall tiles instead of 264: 12 % off that launch).  Else the rows
        // per expert on average decide, and a size that would leave more than half of the CUs without a tile is halved
        // (small problems: latency counts).
        // With the sizes on the host the tiles of every height are counted, and the rows per expert are those of the
        // experts that have any (a skewed decode batch: a few experts hold most of the rows); without, estimated.
        long long busy = args.E > 0 ? args.E : 1;
        if (t_host_sizes != nullptr) {
            busy = 0;
            for (int e = 0; e < args.E; ++e) busy += t_host_sizes[e] > 0;
            if (busy < 1) busy = 1;
        }
        const long long avg = args.rows / busy;
        const long long n_tiles = ((swiglu ? args.N / 2 : args.N) + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256);
        const bool exact = t_host_sizes != nullptr;
        const long long est256 = (exact ? m_tiles_of(args, 256) : args.rows / 256 + (args.E + 1) / 2) * n_tiles;
        const long long est128 = (exact ? m_tiles_of(args, 128) : args.rows / 128 + (args.E + 1) / 2) * n_tiles;
        // fp8: the 256-row tile copies whole 128-byte lines (gmm_tile256_fp8.h) and streams weights a third faster than
        // the smaller tiles, which copy half lines (decode-sized batch, K 4096, N 28672: 4.1 against 3.2 TB/s); it is
        // taken wherever its tiles fill half of the CUs (a quarter, where the launch may cut its tiles along a long K
        // to fill the rest)
        const bool may_cut = args.arrive != nullptr && args.K / 64 >= 2 * kMinPieceStagesIdle;
        const bool tall = fp8 ? (args.K % 128 == 0 && est256 * (may_cut ? 4 : 2) >= cus) : (est256 >= cus || est128 > cus);
        int tile_rows = 256;
        if (!tall) {
            tile_rows = avg <= 64 ? 64 : (avg <= 160 ? 128 : 256);
            while (tile_rows > 64 && (exact ? m_tiles_of(args, tile_rows) : args.rows / tile_rows + (args.E + 1) / 2) * n_tiles * 2 < cus)
                tile_rows /= 2;
        }
        if (g_variant >= 5) tile_rows = g_variant == 5 ? 64 : (g_variant == 6 ? 128 : 256);   // test hook: fixed tile rows (7, 8: 256)
        L.tile_rows = tile_rows;
        // global -> LDS kernels: whole stages (32 k of bf16, 64 of fp8), 32-bit offsets inside one expert's weights
        const bool direct = fp8 ? (args.K % 64 == 0 && (long long)args.K * args.N < (1ll << 32))
                                : (args.K % 32 == 0 && (long long)args.K * args.N * 2 < (1ll << 32));
        if (!direct) {
            L.kernel = kKernelStaged;
            L.waves = tile_rows == 256 ? 8 : 4;
        } else if (tile_rows == 256 && !fp8 && !trans_b && args.K >= 256 && args.K % 128 == 0 && g_variant == 8) {
            L.kernel = kKernelWave128; L.waves = 4;
        } else if (tile_rows == 256 && !fp8) {
            L.kernel = kKernelTile256; L.waves = 8;
        } else if (tile_rows == 256 && args.K % 128 == 0 && g_variant == 8) {
            L.kernel = kKernelWave128Fp8; L.waves = 4;
        } else if (tile_rows == 256 && args.K % 128 == 0) {
            L.kernel = kKernelTile256Fp8; L.waves = 8;   // whole k-steps of 128: the tile that copies whole 128-byte lines
        } else {
            // fp8 tiles of 256 rows on 4 wavefronts would need 256 accumulator + 96 operand registers per lane: 8 wavefronts
            L.kernel = kKernelDirect;
            L.waves = tile_rows == 256 ? 8 : (tile_rows == 64 && !fp8 ? 6 : 4);
        }
    }
    L.stage_k = fp8 ? 64 : (L.kernel == kKernelStaged ? 64 : kDK32);
    L.may_cut = L.kernel != kKernelStaged;
    L.grid = launch_grid(args, L.tile_rows, swiglu, L.stage_k, L.may_cut, cus);
    return L;
}

template <bool TRANS_B, bool SWIGLU, bool FP8>
static int launch_by_rows(const GmmArgs &args, hipStream_t stream) {
    const GmmLaunch L = choose_launch(args, TRANS_B, SWIGLU, FP8);
    if (L.kernel == kKernelStaged) {
        if (L.tile_rows == 64) return launch_one<64, 256, 1, 4, TRANS_B, SWIGLU, FP8>(args, stream);
        if (L.tile_rows == 128) return launch_one<128, 256, 1, 4, TRANS_B, SWIGLU, FP8>(args, stream);
        if (L.waves == 4) return launch_one<256, 256, 2, 2, TRANS_B, SWIGLU, FP8>(args, stream);
        return launch_one<256, 256, 2, 4, TRANS_B, SWIGLU, FP8>(args, stream);
    }
    if (L.kernel == kKernelWave128) return launch_wave128(args, SWIGLU, stream);
    if (L.kernel == kKernelWave128Fp8) return launch_wave128_fp8(args, SWIGLU, stream);
    if constexpr (FP8) return launch_direct_fp8(args, L.tile_rows, SWIGLU, stream);
    else return launch_direct_bf16(args, L.tile_rows, TRANS_B, SWIGLU, stream);
}

static int check_shape(const char *who, int64_t rows, int E, int64_t K, int64_t N, int align) {
    DMOE_REQUIRE(rows >= 0 && rows < (1ll << 31), DMOE_ERR_SHAPE, "%s: rows=%lld outside [0, 2^31)", who, (long long)rows);
    DMOE_REQUIRE(E > 0 && E <= kMaxGroups, DMOE_ERR_SHAPE, "%s: E=%d outside [1, %d]", who, E, kMaxGroups);
    DMOE_REQUIRE(K > 0 && K < (1ll << 22) && K % align == 0, DMOE_ERR_SHAPE, "%s: K=%lld must be a positive multiple of %d",
                 who, (long long)K, align);
    DMOE_REQUIRE(N > 0 && N < (1ll << 24) && N % 8 == 0, DMOE_ERR_SHAPE, "%s: N=%lld must be a positive multiple of 8", who,
                 (long long)N);
    return DMOE_OK;
}

static int check_gmm(const char *who, const void *a, const void *b, const void *c, const int64_t *bs, int64_t rows,
                     int E, int64_t K, int64_t N, int align) {
    const int rc = check_shape(who, rows, E, K, N, align);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(bs != nullptr && b != nullptr, DMOE_ERR_ARG, "%s: null pointer", who);
    DMOE_REQUIRE(rows == 0 || (a != nullptr && c != nullptr), DMOE_ERR_ARG, "%s: null pointer", who);
    return DMOE_OK;
}

}  // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_gmm_tune(int variant) {
    DMOE_REQUIRE(variant >= 0 && variant <= 8, DMOE_ERR_ARG, "dmoe_gmm_tune: variant %d outside [0, 8]", variant);
    g_variant = variant;
    return DMOE_OK;
}

// What a launch with these shapes would run (see tuning.h).  out: [0] kernel (GmmKernelId), [1] tile rows, [2] wavefronts
// per workgroup, [3] workgroups, [4] k per stage unit; and, when the sizes are given (host memory), what the kernel
// derives from them on the device: [5] tiles, [6] tiles cut along K, [7] pieces per cut tile, [8] work items; -1 without.
// `launch_has_sizes`: the launch in question is given the host sizes too (host_batch_sizes of dmoe_gmm*), so its tile
// height and grid are decided from them; otherwise the sizes only serve the counts [5] .. [8].
extern "C" int dmoe_gmm_plan(const int64_t *host_batch_sizes, int launch_has_sizes, int64_t rows, int E, int64_t K, int64_t N,
                             int trans_b, int swiglu, int dtype, size_t workspace_bytes, int64_t *out) {
    DMOE_REQUIRE(out != nullptr, DMOE_ERR_ARG, "dmoe_gmm_plan: null output");
    DMOE_REQUIRE(dtype == DMOE_BF16 || dtype == DMOE_FP8_E4M3, DMOE_ERR_DTYPE, "dmoe_gmm_plan: dtype %d", dtype);
    const bool fp8 = dtype == DMOE_FP8_E4M3;
    const int64_t n_cols = swiglu ? 2 * N : N;
    int rc = check_shape("dmoe_gmm_plan", rows, E, K, n_cols, fp8 ? 16 : 8);
    if (rc != DMOE_OK) return rc;
    GmmArgs args{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, rows, E, (int)K, (int)n_cols, (int)N};
    args.arrive = workspace_bytes > 0 ? (unsigned int *)out : nullptr;   // only tested against nullptr
    args.partial_bytes = (long long)workspace_bytes;
    const HostSizes known(launch_has_sizes ? host_batch_sizes : nullptr);
    const GmmLaunch L = choose_launch(args, trans_b != 0 || fp8, swiglu != 0, fp8);
    out[0] = L.kernel; out[1] = L.tile_rows; out[2] = L.waves; out[3] = L.grid; out[4] = L.stage_k;
    out[5] = out[6] = out[7] = out[8] = -1;
    if (host_batch_sizes != nullptr) {
        long long m_tiles = 0, left = rows;
        for (int e = 0; e < E; ++e) {
            long long n = host_batch_sizes[e] < 0 ? 0 : host_batch_sizes[e];
            if (n > left) n = left;
            left -= n;
            m_tiles += (n + L.tile_rows - 1) / L.tile_rows;
        }
        const long long n_tiles = (N + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256);
        WorkPlan w;
        if (L.may_cut) {
            const long long piece_bytes = (long long)L.tile_rows * 256 * sizeof(float);
            // the 256-row fp8 tile counts its length in k-steps of 128 and plans in twice that many stage units
            const int stages = (int)(L.kernel == kKernelTile256Fp8 ? 2 * (K / 128) : K / L.stage_k);
            w = plan_work(m_tiles * n_tiles, (int)L.grid, stages, workspace_bytes > 0 ? (long long)workspace_bytes / piece_bytes : 0,
                          kWsArriveCount / (L.waves == 6 ? 4 : L.waves));
        } else {
            w.tiles = w.whole = w.items = m_tiles * n_tiles; w.rem = 0; w.split = 1;
        }
        out[5] = w.tiles; out[6] = w.rem; out[7] = w.split; out[8] = w.items;
    }
    return DMOE_OK;
}

extern "C" int dmoe_gmm_workspace_bytes(int E, size_t *bytes) {
    DMOE_REQUIRE(bytes != nullptr, DMOE_ERR_ARG, "dmoe_gmm_workspace_bytes: null output");
    DMOE_REQUIRE(E > 0 && E <= kMaxGroups, DMOE_ERR_SHAPE, "dmoe_gmm_workspace_bytes: E=%d outside [1, %d]", E, kMaxGroups);
    // room for the partial sums of two pieces per compute unit (a piece of a 256 x 256 tile is 256 KiB of fp32)
    *bytes = (size_t)2 * (size_t)device_cus() * 256 * 256 * sizeof(float);
    return DMOE_OK;
}

extern "C" int dmoe_gmm(const void *a, const void *b, void *c, const int64_t *batch_sizes, int64_t rows, int E,
                        int64_t K, int64_t N, int trans_b, int dtype, void *state, void *workspace,
                        size_t workspace_bytes, const int64_t *host_batch_sizes, void *stream) {
    const HostSizes known(host_batch_sizes);
    DMOE_REQUIRE(dtype == DMOE_BF16, DMOE_ERR_DTYPE, "dmoe_gmm: dtype %d (bf16 only)", dtype);
    int rc = check_gmm("dmoe_gmm", a, b, c, batch_sizes, rows, E, K, N, 8);
    if (rc != DMOE_OK) return rc;
    if (rows == 0) return DMOE_OK;
    GmmArgs args{(const char *)a, (const char *)b, (char *)c, batch_sizes, nullptr, nullptr, rows, E, (int)K, (int)N, (int)N};
    rc = bind_state(args, state, workspace, workspace_bytes, (hipStream_t)stream);
    if (rc != DMOE_OK) return rc;
    return trans_b ? launch_by_rows<true, false, false>(args, (hipStream_t)stream)
                   : launch_by_rows<false, false, false>(args, (hipStream_t)stream);
}

extern "C" int dmoe_gmm_swiglu(const void *a, const void *b, void *h, const int64_t *batch_sizes, int64_t rows, int E,
                               int64_t K, int64_t I, int trans_b, int dtype, void *state, void *workspace,
                               size_t workspace_bytes, const int64_t *host_batch_sizes, void *stream) {
    const HostSizes known(host_batch_sizes);
    DMOE_REQUIRE(dtype == DMOE_BF16, DMOE_ERR_DTYPE, "dmoe_gmm_swiglu: dtype %d (bf16 only)", dtype);
    int rc = check_gmm("dmoe_gmm_swiglu", a, b, h, batch_sizes, rows, E, K, I, 8);
    if (rc != DMOE_OK) return rc;
    if (rows == 0) return DMOE_OK;
    GmmArgs args{(const char *)a, (const char *)b, (char *)h, batch_sizes, nullptr, nullptr, rows, E, (int)K, (int)(2 * I), (int)I};
    rc = bind_state(args, state, workspace, workspace_bytes, (hipStream_t)stream);
    if (rc != DMOE_OK) return rc;
    return trans_b ? launch_by_rows<true, true, false>(args, (hipStream_t)stream)
                   : launch_by_rows<false, true, false>(args, (hipStream_t)stream);
}

extern "C" int dmoe_gmm_swiglu_rows(const void *x, const int32_t *row_token, int64_t T, const void *b, void *h,
                                    const int64_t *batch_sizes, int64_t rows, int E, int64_t K, int64_t I, int dtype,
                                    void *state, void *workspace, size_t workspace_bytes,
                                    const int64_t *host_batch_sizes, void *stream) {
    const HostSizes known(host_batch_sizes);
    DMOE_REQUIRE(dtype == DMOE_BF16, DMOE_ERR_DTYPE, "dmoe_gmm_swiglu_rows: dtype %d (bf16 only)", dtype);
    int rc = check_gmm("dmoe_gmm_swiglu_rows", x, b, h, batch_sizes, rows, E, K, I, 32);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(T > 0 && T * K * 2 < (1ll << 32), DMOE_ERR_SHAPE,
                 "dmoe_gmm_swiglu_rows: T=%lld rows of K=%lld must be fewer than 4 GiB", (long long)T, (long long)K);
    DMOE_REQUIRE(K * 2 * I * 2 < (1ll << 32), DMOE_ERR_SHAPE,
                 "dmoe_gmm_swiglu_rows: one expert's weights (K=%lld x 2I=%lld) must be fewer than 4 GiB", (long long)K, (long long)(2 * I));
    DMOE_REQUIRE(rows == 0 || row_token != nullptr, DMOE_ERR_ARG, "dmoe_gmm_swiglu_rows: null row_token");
    if (rows == 0) return DMOE_OK;
    GmmArgs args{(const char *)x, (const char *)b, (char *)h, batch_sizes, nullptr, nullptr, rows, E, (int)K, (int)(2 * I), (int)I};
    rc = bind_state(args, state, workspace, workspace_bytes, (hipStream_t)stream);
    if (rc != DMOE_OK) return rc;
    args.a_rows = row_token;
    args.a_src_rows = T;
    return launch_tile256_rows(args, (hipStream_t)stream);
}

extern "C" int dmoe_gmm_fp8(const void *a, const float *a_scale, const void *b, const float *b_scale, void *c,
                            const int64_t *batch_sizes, int64_t rows, int E, int64_t K, int64_t N, void *state,
                            void *workspace, size_t workspace_bytes, const int64_t *host_batch_sizes, void *stream) {
    const HostSizes known(host_batch_sizes);
    int rc = check_gmm("dmoe_gmm_fp8", a, b, c, batch_sizes, rows, E, K, N, 16);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(b_scale != nullptr && (rows == 0 || a_scale != nullptr), DMOE_ERR_ARG, "dmoe_gmm_fp8: null scales");
    if (rows == 0) return DMOE_OK;
    GmmArgs args{(const char *)a, (const char *)b, (char *)c, batch_sizes, a_scale, b_scale, rows, E, (int)K, (int)N, (int)N};
    rc = bind_state(args, state, workspace, workspace_bytes, (hipStream_t)stream);
    if (rc != DMOE_OK) return rc;
    return launch_by_rows<true, false, true>(args, (hipStream_t)stream);
}

extern "C" int dmoe_gmm_fp8_swiglu(const void *a, const float *a_scale, const void *b, const float *b_scale, void *h,
                                   const int64_t *batch_sizes, int64_t rows, int E, int64_t K, int64_t I,
                                   void *state, void *workspace, size_t workspace_bytes,
                                   const int64_t *host_batch_sizes, void *stream) {
    const HostSizes known(host_batch_sizes);
    int rc = check_gmm("dmoe_gmm_fp8_swiglu", a, b, h, batch_sizes, rows, E, K, I, 16);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(b_scale != nullptr && (rows == 0 || a_scale != nullptr), DMOE_ERR_ARG, "dmoe_gmm_fp8_swiglu: null scales");
    if (rows == 0) return DMOE_OK;
    GmmArgs args{(const char *)a, (const char *)b, (char *)h, batch_sizes, a_scale, b_scale, rows, E, (int)K, (int)(2 * I), (int)I};
    rc = bind_state(args, state, workspace, workspace_bytes, (hipStream_t)stream);
    if (rc != DMOE_OK) return rc;
    return launch_by_rows<true, true, true>(args, (hipStream_t)stream);
}
