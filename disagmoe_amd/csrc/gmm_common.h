// Pieces shared by the grouped GEMM kernels: argument block, vector types and the
// device-side work list (expert, m-tile, n-tile) derived from batch_sizes.
#pragma once

#include <type_traits>

#include "common.h"

namespace dmoe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

constexpr int kMaxGroups = 1024;   // experts per call (LDS tables)
constexpr int kXcds = 8;

struct GmmArgs {
    const char *a;
    const char *b;
    char *c;
    const int64_t *batch_sizes;
    const float *a_scale;
    const float *b_scale;
    int64_t rows;   // rows of a / c
    int E;
    int K;          // contraction length (elements)
    int N;          // columns of b per expert (2*I for the swiglu form)
    int ldc;        // columns of c (N, or I for the swiglu form)
    // state of the launch in device memory (the caller's state block and workspace, or the library's own counters)
    struct SchedSlot *sched;      // work counters, zero between launches
    unsigned int *arrive;         // arrival counters of the split tiles, zero between launches (nullptr: no splitting)
    float *partials;              // fp32 partial results of the pieces of split tiles
    long long partial_bytes;      // capacity of `partials`
    // (gmm_tile256_kernel's gathering form) row r of the product is row a_rows[r] of `a`, which has a_src_rows rows
    const int32_t *a_rows;
    long long a_src_rows;
};

// ---- work distribution ---------------------------------------------------------------------------
// Tiles differ in cost (an expert's last m-tile may hold a few rows), so workgroups draw work items from
// counters instead of striding over them.  There is one counter per XCD (workgroup id % 8): XCD x draws
// j = 0, 1, 2, ... and works on item q = 8 j + x, which keeps the items that share operand tiles on one
// L2 (see item_order) exactly as a static stride would, while a slow tile no longer holds up the tiles
// queued behind it.  The counters of a launch live in device memory that is zero when the launch starts
// (the caller's state block, or the library's own slot of the launch's stream); the workgroup that
// makes a counter's last draw clears it again (sched_finish).  Launches that may overlap in time must not share them.
struct SchedSlot {
    unsigned int next[kXcds];
    unsigned int done;
    unsigned int pad[7];
};

// Layout of a caller-owned state block (DMOE_GMM_STATE_BYTES): work counters, then arrival counters of the split tiles.
constexpr size_t kWsArriveOffset = 256;
constexpr int kWsArriveCount = 8 * 1024;                                  // (split tiles) x (wavefronts of a tile)
static_assert(kWsArriveOffset + kWsArriveCount * sizeof(unsigned int) == DMOE_GMM_STATE_BYTES, "state block as dmoe.h states it");

// Next work item of this workgroup (all threads get the same value), or -1 when its stream is exhausted.
// `carry` holds the draw made ahead of time by thread 0 (see sched_draw).
__device__ __forceinline__ unsigned int sched_draw(SchedSlot *slot, int streams) {
    return atomicAdd(&slot->next[streams == 1 ? 0 : (blockIdx.x % kXcds)], 1u);
}
// A workgroup's first item is its own number (no draw, so the first tile does not wait for an atomic's round trip);
// the draws number the items behind those gridDim.x.
__device__ __forceinline__ long long sched_item(unsigned int j, int streams) {
    return streams == 1 ? (long long)j + gridDim.x
                        : ((long long)j + gridDim.x / kXcds) * kXcds + (blockIdx.x % kXcds);
}
// Called once per workgroup when its draw has come back past the end of the work (`draw` is that value, held by the
// workgroup's drawing thread).  Every workgroup makes one draw more than it works on drawn items, so a counter hands
// out exactly (its XCD's drawn items) + (its XCD's workgroups) values in a launch: whoever holds the last of them knows
// that nobody will draw from that counter again and sets it back to zero for the next launch: no count of finished
// workgroups, no atomic to wait for at the end of a launch.
__device__ __forceinline__ void sched_finish(SchedSlot *slot, bool drawer, unsigned int draw, int streams, long long total) {
    if (!drawer) return;
    const int x = streams == 1 ? 0 : (int)(blockIdx.x % kXcds);
    const long long wgs = streams == 1 ? (long long)gridDim.x : (long long)(gridDim.x / kXcds);
    // drawn items of this counter: j >= 0 with sched_item(j) < total
    long long drawn = streams == 1 ? total - wgs : (total - x + kXcds - 1) / kXcds - wgs;
    if (drawn < 0) drawn = 0;
    // cleared with the same kind of operation the counter is advanced with, so that the clear is seen wherever the
    // next launch's draws are performed
    if ((long long)draw == drawn + wgs - 1) atomicExch(&slot->next[x], 0u);
}

// ---- the last, partly filled round of tiles ----------------------------------------------------------
// `tiles` tiles on G workgroups leave the last round with rem = tiles % G tiles: G - rem compute units idle for the
// length of a tile.  Those rem tiles are therefore cut along K into `split` pieces of equal length, drawn like any
// other work item after the whole tiles; rem * split pieces fill ceil(rem * split / G) rounds of 1 / split of a
// tile's length.  A piece leaves its fp32 accumulators in the workspace; the piece of a tile that arrives last adds
// all of them up in the order of the pieces (so the sum does not depend on which one that is) and writes the result.
struct WorkPlan {
    long long tiles;     // (expert, m-tile, n-tile) triples
    long long whole;     // tiles computed in one piece: items [0, whole)
    int rem;             // tiles cut in pieces: items [whole, whole + rem * split), piece-major
    int split;           // pieces per such tile (1: nothing is cut, rem == 0)
    long long items;     // whole + rem * split
};
constexpr int kMaxSplit = 8;
constexpr int kMaxWholeRounds = 3;
constexpr int kMinPieceStagesIdle = 24;   // ... unless the launch has fewer tiles than workgroups: the pieces then run
                                          // on compute units that would have nothing to do
constexpr int kMinPieceStages = 88;   // shorter pieces lose to their own overhead (measured: tiles of 44 and 128 stages
                                      // lose when cut, tiles of 448 stages cut in 4 or 5 gain 7 - 11 %)

__device__ __host__ __forceinline__ WorkPlan plan_work(long long tiles, int G, int stages, long long max_pieces, int max_rem) {
    WorkPlan w;
    w.tiles = tiles; w.whole = tiles; w.rem = 0; w.split = 1; w.items = tiles;
    const long long rem = tiles % G;
    // Launches of many rounds gain nothing (measured: 15.3 rounds of 128 stages): their workgroups are up to a tile
    // apart by the time the last round starts, and the counters balance that as well as pieces would.
    if (rem == 0 || rem > max_rem || tiles / G > kMaxWholeRounds) return w;
    // Time of the remainder in stages.  A work item costs its stages and about 8 more (draw, first copies in flight,
    // drain, epilogue); a piece also writes its sums past the L2 and counts itself in (about 12), and the last piece of
    // a tile reads all of them back (4 + 4 per piece).  The smallest wins, if it saves 8 % of a whole tile.
    int best = 1;
    const long long whole_cost = stages + 8;
    long long best_cost = whole_cost;
    for (int p = 2; p <= kMaxSplit; ++p) {
        if (rem * p > max_pieces || stages / p < (tiles < G ? kMinPieceStagesIdle : kMinPieceStages)) break;
        const long long rounds = (rem * p + G - 1) / G;
        const long long cost = rounds * ((stages + p - 1) / p + 20) + 4 + 4 * p;
        if (cost < best_cost) { best = p; best_cost = cost; }
    }
    // the estimate flatters short pieces (measured: 0.79 of a whole tile's time where it says 0.69), so they have to
    // promise more
    if (best == 1 || best_cost * 100 > (stages / best < kMinPieceStages ? 85 : 92) * whole_cost) return w;
    w.split = best; w.rem = (int)rem; w.whole = tiles - rem; w.items = w.whole + rem * best;
    return w;
}

// Prefix sums of rows and m-tiles over the experts, built by the first wavefront
// into LDS tables of E + 1 entries.  Sizes are clamped so that the running row
// count never passes p.rows.  The caller synchronises the workgroup afterwards.
template <int BM>
__device__ __forceinline__ void build_work_list(const GmmArgs &p, int *s_tile_start, int *s_row_start) {
    const int lane = threadIdx.x & (kWave - 1);
    if (threadIdx.x >= kWave) return;
    const int E = p.E;
    long long row_carry = 0;
    int tile_carry = 0;
    for (int e0 = 0; e0 < E; e0 += kWave) {
        const int e = e0 + lane;
        long long n = (e < E) ? (long long)p.batch_sizes[e] : 0;
        n = n < 0 ? 0 : (n > p.rows ? p.rows : n);
        long long incl = n;
#pragma unroll
        for (int s = 1; s < kWave; s <<= 1) {
            long long up = __shfl_up(incl, s, kWave);
            if (lane >= s) incl += up;
        }
        long long start = row_carry + incl - n;
        if (start > p.rows) start = p.rows;
        long long end = row_carry + incl;
        if (end > p.rows) end = p.rows;
        const int mt = (int)((end - start + BM - 1) / BM);
        int tincl = mt;
#pragma unroll
        for (int s = 1; s < kWave; s <<= 1) {
            int up = __shfl_up(tincl, s, kWave);
            if (lane >= s) tincl += up;
        }
        if (e < E) {
            s_row_start[e] = (int)start;
            s_tile_start[e] = tile_carry + tincl - mt;
        }
        row_carry += __shfl(incl, kWave - 1, kWave);
        tile_carry += __shfl(tincl, kWave - 1, kWave);
    }
    if (lane == 0) {
        s_row_start[E] = (int)(row_carry > p.rows ? p.rows : row_carry);
        s_tile_start[E] = tile_carry;
    }
}

struct TileCoord {
    int e;        // expert
    int nt;       // n-tile
    int row0;     // first row of the tile in a / c
    int rows_e;   // rows of the expert from row0 on (>= 1; the tile holds min(rows_e, BM) of them)
};

// Work item q -> position L in the tile order.  Items are cut in rounds of G (the grid size); inside a round, item q
// belongs to XCD q % 8 and the XCD's items of the round are consecutive positions.
__device__ __forceinline__ long long item_order(long long q, int G, long long total) {
    if (G % kXcds != 0) return q;
    // a round holds cnt = min(G, items left) items; XCD x owns those with q % 8 == x, cnt / 8 of them plus one
    // more on the first cnt % 8 XCDs, and they map onto consecutive positions (a bijection for every cnt, so the
    // last, partly filled round - the only round of a small problem - keeps its operand sharing too)
    const long long base = (q / G) * G;
    const long long left = total - base;
    const int cnt = (int)(left < G ? left : G);
    const int w = (int)(q - base), x = w % kXcds;
    const int per = cnt / kXcds, extra = cnt % kXcds;
    return base + (long long)x * per + (x < extra ? x : extra) + (w / kXcds);
}

// Position L in the tile order -> tile.  Inside an expert the tiles are ordered in bands of 4 m-tiles (a lone fifth,
// ninth, ... m-tile joins the band before it); a band walks the n-tiles with its m-tiles innermost, so a weight tile
// is shared by the band's m-tiles on one L2 and the band's A rows stay there while it sweeps N.
template <int BM>
__device__ __forceinline__ TileCoord decode_tile(long long L, int n_tiles, int E, const int *s_tile_start,
                                                 const int *s_row_start) {
    const int u = (int)(L / n_tiles);
    int lo = 0, hi = E;  // last e with s_tile_start[e] <= u
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_tile_start[mid] <= u) lo = mid; else hi = mid;
    }
    TileCoord t;
    t.e = lo;
    constexpr int kBand = 4;
    const int mt_e = s_tile_start[lo + 1] - s_tile_start[lo];
    int idx = (int)(L - (long long)s_tile_start[lo] * n_tiles);
    int bands = mt_e / kBand;                       // full bands
    const int rest = mt_e - bands * kBand;          // 0..3 m-tiles left over
    int band = idx / (kBand * n_tiles), width = kBand;
    if (rest == 1 && bands > 0) {                   // the lone m-tile rides with the last full band
        if (band >= bands - 1) { band = bands - 1; width = kBand + 1; }
    } else if (band >= bands) {
        band = bands; width = rest;
    }
    idx -= band * kBand * n_tiles;
    t.nt = idx / width;
    const int mi = band * kBand + (idx - t.nt * width);
    t.row0 = s_row_start[lo] + mi * BM;
    t.rows_e = s_row_start[lo + 1] - t.row0;
    return t;
}

// A work item: a tile and the stages [s_lo, s_lo + s_cnt) of it; piece >= 0 numbers the piece of a split tile,
// whose number among the split tiles is `split_tile`.
struct WorkItem {
    TileCoord tile;
    int s_lo, s_cnt;
    int piece;
    int split_tile;
};
// kAlign: the pieces of a split tile begin at multiples of kAlign stages (`stages` is one).
template <int BM, int kAlign = 1>
__device__ __forceinline__ WorkItem decode_item(long long q, int G, const WorkPlan &w, int stages, int n_tiles, int E,
                                                const int *s_tile_start, const int *s_row_start) {
    const long long L = item_order(q, G, w.items);
    WorkItem it;
    long long tile = L;
    it.s_lo = 0; it.s_cnt = stages; it.piece = -1; it.split_tile = 0;
    if (L >= w.whole) {
        const long long r = L - w.whole;            // piece-major: the same piece of consecutive tiles is consecutive
        it.piece = (int)(r / w.rem);
        it.split_tile = (int)(r - (long long)it.piece * w.rem);
        tile = w.whole + it.split_tile;
        it.s_lo = (int)((long long)stages * it.piece / w.split) / kAlign * kAlign;
        it.s_cnt = (int)((long long)stages * (it.piece + 1) / w.split) / kAlign * kAlign - it.s_lo;
    }
    it.tile = decode_tile<BM>(tile, n_tiles, E, s_tile_start, s_row_start);
    return it;
}

// ---- a piece of a split tile meets the others ---------------------------------------------------------
// Every wavefront leaves its accumulators in the workspace, as [fragment][value pair][lane] so that an instruction
// moves 512 bytes, and counts itself in at the counter of its part of the tile.  The wavefront that arrives last there,
// of whichever piece, adds the pieces up in their order (the sum does not depend on who that is) and returns true: it
// goes on to the epilogue.  The partial sums and the counter are written and read with accesses of device scope, which
// go past the XCD's L2 to memory that every XCD sees: no fence has to write back or invalidate a whole L2, whose
// other contents (the operand tiles of the compute units beside this one) stay where they are.
// AccT: a vector of 4 or 16 floats; lim: wave-uniform, the row fragments [lim, FM) hold no valid row and stay out of
// the workspace (every piece of a tile leaves out the same ones).
template <int NW, int FM, int FN, typename AccT>
__device__ __forceinline__ bool meet_pieces(AccT (&acc)[FM][FN], const GmmArgs &p, int split, int split_tile, int part,
                                            int wave, int lane, int lim) {
    constexpr int kPairs = (int)(sizeof(AccT) / 8);
    constexpr size_t kWaveFloats = (size_t)FM * FN * kPairs * 2 * kWave;
    unsigned long long *mine = (unsigned long long *)(p.partials + ((size_t)(split_tile * split + part) * NW + wave) * kWaveFloats);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        if (i >= lim) continue;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int x = 0; x < kPairs; ++x) {
                const unsigned long long v = (unsigned long long)__float_as_uint(acc[i][j][2 * x]) |
                                             ((unsigned long long)__float_as_uint(acc[i][j][2 * x + 1]) << 32);
                __hip_atomic_store(mine + ((i * FN + j) * kPairs + x) * kWave + lane, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
    }
    // the stores have reached memory before the wavefront counts itself in
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));   // vmcnt(0)
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    unsigned int *arrived = p.arrive + split_tile * NW + wave;
    unsigned int before = 0;
    if (lane == 0) before = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = __builtin_amdgcn_readfirstlane(before);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    if (before != (unsigned int)(split - 1)) return false;
    if (lane == 0) __hip_atomic_store(arrived, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // as the next launch expects it
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int x = 0; x < 2 * kPairs; ++x) acc[i][j][x] = 0.f;
    for (int k = 0; k < split; ++k) {
        const unsigned long long *src = (const unsigned long long *)(p.partials + ((size_t)(split_tile * split + k) * NW + wave) * kWaveFloats);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if (i >= lim) continue;
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int x = 0; x < kPairs; ++x) {
                    const unsigned long long v = __hip_atomic_load(src + ((i * FN + j) * kPairs + x) * kWave + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    acc[i][j][2 * x] += __uint_as_float((unsigned int)v);
                    acc[i][j][2 * x + 1] += __uint_as_float((unsigned int)(v >> 32));
                }
        }
    }
    return true;
}

// ---- the launch a problem gets (host) -------------------------------------------------------------------
enum GmmKernelId { kKernelStaged = 0, kKernelDirect = 1, kKernelTile256 = 2, kKernelTile256Fp8 = 3, kKernelWave128 = 4, kKernelWave128Fp8 = 5 };
struct GmmLaunch {
    int kernel;        // GmmKernelId
    int tile_rows;     // rows of a tile (64, 128, 256); a tile has 256 columns of b
    int waves;         // wavefronts of a workgroup
    int stage_k;       // k per unit of plan_work's lengths (bf16: 32; fp8: 64)
    bool may_cut;      // the kernel cuts tiles along K when the launch has a workspace
    long long grid;    // workgroups
};
// The caller's copy of batch_sizes in host memory for the call that this thread is in, or nullptr: the reference keeps
// the sizes on the host wherever it does not run its CUTLASS path (disagmoe/frontend/engine.py:377-380, 690-701).
// With it the host knows the m-tiles of every tile height exactly; without it rows / tile_rows + E bounds them from above.
extern thread_local const int64_t *t_host_sizes;
inline long long m_tiles_of(const GmmArgs &args, int tile_rows) {
    if (t_host_sizes == nullptr) return args.rows / tile_rows + args.E;
    long long tiles = 0, left = args.rows;
    for (int e = 0; e < args.E; ++e) {
        long long n = t_host_sizes[e] < 0 ? 0 : t_host_sizes[e];
        if (n > left) n = left;                         // as the kernels clamp them
        left -= n;
        tiles += (n + tile_rows - 1) / tile_rows;
    }
    return tiles;
}
// Workgroups of a persistent launch: one per compute unit, fewer when the tiles (or, where tiles may be cut along a K
// long enough for two pieces, their pieces) do not fill them; whole rows of XCDs, the tile order is XCD-aware only then.
inline long long launch_grid(const GmmArgs &args, int tile_rows, bool swiglu, int stage_k, bool may_cut, int cus) {
    const int n_out = swiglu ? args.N / 2 : args.N;
    const int bno = swiglu ? 128 : 256;
    const long long n_tiles = (n_out + bno - 1) / bno;
    long long pieces = m_tiles_of(args, tile_rows) * n_tiles;
    if (may_cut && args.arrive != nullptr && args.K / stage_k >= 2 * kMinPieceStagesIdle) pieces *= kMaxSplit;
    long long grid = cus;
    if (pieces < grid) grid = pieces;
    if (grid < 1) grid = 1;
    return (grid + kXcds - 1) / kXcds * kXcds;
}

int launch_direct_bf16(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream);
int launch_direct_fp8(const GmmArgs &args, int tile_rows, bool swiglu, hipStream_t stream);
int launch_tile256_fp8(const GmmArgs &args, bool swiglu, hipStream_t stream);
int launch_wave128(const GmmArgs &args, bool swiglu, hipStream_t stream);
int launch_wave128_fp8(const GmmArgs &args, bool swiglu, hipStream_t stream);
int launch_tile256_rows(const GmmArgs &args, hipStream_t stream);

}  // namespace dmoe
