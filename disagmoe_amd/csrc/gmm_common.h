// Pieces shared by the grouped GEMM kernels: argument block, vector types and the
// device-side work list (expert, m-tile, n-tile) derived from batch_sizes.
#pragma once

#include <type_traits>

#include "common.h"

namespace dmoe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
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
    int sched_slot; // entry of the work-counter ring used by this launch
};

// ---- work distribution ---------------------------------------------------------------------------
// Tiles differ in cost (an expert's last m-tile may hold a few rows), so workgroups draw work items from
// counters instead of striding over them.  There is one counter per XCD (workgroup id % 8): XCD x draws
// j = 0, 1, 2, ... and works on item q = 8 j + x, which keeps the items that share operand tiles on one
// L2 (see decode_tile) exactly as a static stride would, while a slow tile no longer holds up the tiles
// queued behind it.  The counters of a launch live in one entry of a small ring in device memory; the
// last workgroup to finish clears the entry, so no host-side reset or scratch argument is needed.
// Launches that run concurrently must not share an entry: the host hands entries out round-robin.
constexpr int kSchedSlots = 64;
struct SchedSlot {
    unsigned int next[kXcds];
    unsigned int done;
    unsigned int pad[7];
};
static __device__ SchedSlot g_sched[kSchedSlots];

// Next work item of this workgroup (all threads get the same value), or -1 when its stream is exhausted.
// `carry` holds the draw made ahead of time by thread 0 (see sched_draw).
__device__ __forceinline__ unsigned int sched_draw(int slot, int streams) {
    return atomicAdd(&g_sched[slot].next[streams == 1 ? 0 : (blockIdx.x % kXcds)], 1u);
}
__device__ __forceinline__ long long sched_item(unsigned int j, int streams) {
    return streams == 1 ? (long long)j : (long long)j * kXcds + (blockIdx.x % kXcds);
}
// Called once per workgroup after its last draw; the last caller of the launch clears the entry.
__device__ __forceinline__ void sched_finish(int slot) {
    if (threadIdx.x == 0) {
        __threadfence();
        const unsigned int before = atomicAdd(&g_sched[slot].done, 1u);
        if (before == gridDim.x - 1) {
            // cleared with the same kind of operation the counters are advanced with, so that the clear is
            // seen wherever the next launch's draws are performed
#pragma unroll
            for (int i = 0; i < kXcds; ++i) atomicExch(&g_sched[slot].next[i], 0u);
            atomicExch(&g_sched[slot].done, 0u);
            __threadfence();
        }
    }
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

// Work item q -> tile.  Items are cut in rounds of G (the grid size); inside a round, item q belongs to XCD
// q % 8 and the XCD's items of the round are consecutive tiles.  Inside an expert the tiles are ordered in
// bands of 4 m-tiles (a lone fifth, ninth, ... m-tile joins the band before it); a band walks the n-tiles
// with its m-tiles innermost, so a weight tile is shared by the band's m-tiles on one L2 and the band's A
// rows stay there while it sweeps N.
template <int BM>
__device__ __forceinline__ TileCoord decode_tile(long long q, int G, long long total, int n_tiles, int E,
                                                 const int *s_tile_start, const int *s_row_start) {
    long long L = q;
    if (G % kXcds == 0) {
        // a round holds cnt = min(G, items left) items; XCD x owns those with q % 8 == x, cnt / 8 of them plus one
        // more on the first cnt % 8 XCDs, and they map onto consecutive tiles (a bijection for every cnt, so the
        // last, partly filled round - the only round of a small problem - keeps its operand sharing too)
        const long long base = (q / G) * G;
        const long long left = total - base;
        const int cnt = (int)(left < G ? left : G);
        const int w = (int)(q - base), x = w % kXcds;
        const int per = cnt / kXcds, extra = cnt % kXcds;
        L = base + (long long)x * per + (x < extra ? x : extra) + (w / kXcds);
    }
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

int next_sched_slot();
int launch_direct_bf16(const GmmArgs &args, int tile_rows, bool trans_b, bool swiglu, hipStream_t stream);
int launch_direct_fp8(const GmmArgs &args, int tile_rows, bool swiglu, hipStream_t stream);

}  // namespace dmoe
