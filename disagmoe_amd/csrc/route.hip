// Routing: expert ids -> destination rows, per-expert counts and offsets.
//
// Counting sort split in chunks of kChunk rows, one wavefront per chunk, so that
// the order of rows inside an expert is fixed by construction (no atomics decide
// a position):
//   pass 1  per-chunk histogram                         -> scratch[chunk][E]
//   pass 2  every chunk sums the histograms before it (its base rank per
//           expert) and all of them (counts, offsets), then walks its rows 64 at a
//           time; a row's rank inside the 64 is the number of lower lanes with
//           the same id, found with log2(E) wave ballots.
// Up to 12 chunks run both passes in one launch of one workgroup, a wavefront
// per chunk and the histograms in LDS.  When summing the
// histograms would take a wavefront of pass 2 more than two batches of loads, a
// launch between the two turns them into their running sums over the chunks and
// pass 2 reads one row instead of all rows (its work would grow with the square
// of the chunk count).
#include <stdarg.h>
#include <string.h>

#include <mutex>

#include "common.h"

namespace dmoe {

static thread_local char g_err[512] = "";
char *error_buffer() { return g_err; }

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int device_cus() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached[dev] = cus;
    }
    return cached[dev];
}

hipError_t raise_dynamic_lds(const void *kernel, int bytes, unsigned long long *seen) {
    static std::mutex mu;
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    const unsigned long long bit = 1ull << (dev & 63);
    std::lock_guard<std::mutex> lock(mu);
    if (*seen & bit) return hipSuccess;
    err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (err == hipSuccess) *seen |= bit;
    return err;
}

// Scratch of dmoe_route_noalloc: the per-chunk histograms of one routing call.  File scope, one copy per device,
// held until the process ends.  Host code reaches it only through the address hipGetSymbolAddress returns.
constexpr size_t kStaticScratchBytes = 4u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kChunk = 512;       // rows per wavefront
constexpr int kMaxExperts = 4096; // 3 int tables of E entries must fit in LDS
// chunks that one workgroup takes, a wavefront each, when their tables fit in LDS (measured: 6144 rows 13 us against
// 16 us for two launches, 8192 rows 16 us against 15 us)
constexpr int kBlockChunks = 12;
constexpr int kSumBatch = 16;     // histogram rows a lane of pass 2 has in flight
constexpr int kScanWaves = 16;    // wavefronts of a scanning workgroup

// The ids of rows base + i * 64 + lane, i < kChunk / 64, of a chunk: -2 past the end, -1 present but outside
// [0, E).  Every load is issued before the first value is looked at (rows past the end re-read the last row).
template <typename IdT>
__device__ __forceinline__ void load_chunk_ids(const IdT *ids, int64_t base, int lane, int64_t R, int E,
                                               int (&out)[kChunk / kWave]) {
    IdT raw[kChunk / kWave];
    if (R <= 0) {   // no row to re-read (and ids may be null)
#pragma unroll
        for (int i = 0; i < kChunk / kWave; ++i) out[i] = -2;
        return;
    }
#pragma unroll
    for (int i = 0; i < kChunk / kWave; ++i) {
        const int64_t t = base + i * kWave + lane;
        raw[i] = ids[t < R ? t : R - 1];
    }
#pragma unroll
    for (int i = 0; i < kChunk / kWave; ++i) {
        const int64_t t = base + i * kWave + lane;
        const long long v = (long long)raw[i];
        out[i] = t >= R ? -2 : ((v >= 0 && v < E) ? (int)v : -1);
    }
}

template <typename IdT>
__global__ __launch_bounds__(kWave) void route_hist_kernel(const IdT *__restrict__ ids, int64_t R, int E,
                                                          int *__restrict__ chunk_hist) {
    extern __shared__ int cnt[];
    const int lane = threadIdx.x;
    const int64_t base = (int64_t)blockIdx.x * kChunk;
    for (int e = lane; e < E; e += kWave) cnt[e] = 0;
    __syncthreads();
    int my_id[kChunk / kWave];
    load_chunk_ids(ids, base, lane, R, E, my_id);
#pragma unroll
    for (int i = 0; i < kChunk / kWave; ++i)
        if (my_id[i] >= 0) atomicAdd(&cnt[my_id[i]], 1);
    __syncthreads();
    for (int e = lane; e < E; e += kWave) chunk_hist[(int64_t)blockIdx.x * E + e] = cnt[e];
}

// chunk_hist[nchunks][E] -> exclusive running sums over the chunks, in place, and totals[E].  A workgroup owns 64
// experts (lane = expert: rows of the table are read 256 bytes at a time), each of its wavefronts a contiguous range
// of chunks: sum of the range, offsets of the ranges through LDS, then the range again, a batch of loads at a time.
__global__ __launch_bounds__(kScanWaves * kWave) void route_scan_kernel(int *__restrict__ chunk_hist, int nchunks, int E,
                                                                       int *__restrict__ totals) {
    __shared__ int part[kScanWaves][kWave];
    constexpr int kBatch = kSumBatch;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int e = blockIdx.x * kWave + lane;
    const int per = (nchunks + kScanWaves - 1) / kScanWaves;
    const int c_lo = wave * per < nchunks ? wave * per : nchunks;
    const int c_hi = c_lo + per < nchunks ? c_lo + per : nchunks;
    int sum = 0;
    if (e < E) {
        for (int c0 = c_lo; c0 < c_hi; c0 += kBatch) {
            int v[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) v[u] = c0 + u < c_hi ? chunk_hist[(int64_t)(c0 + u) * E + e] : 0;
#pragma unroll
            for (int u = 0; u < kBatch; ++u) sum += v[u];
        }
    }
    part[wave][lane] = sum;
    __syncthreads();
    int run = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kScanWaves; ++w) {
        const int v = part[w][lane];
        if (w < wave) run += v;
        all += v;
    }
    if (e >= E) return;
    if (wave == 0) totals[e] = all;
    for (int c0 = c_lo; c0 < c_hi; c0 += kBatch) {
        int v[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) v[u] = c0 + u < c_hi ? chunk_hist[(int64_t)(c0 + u) * E + e] : 0;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (c0 + u < c_hi) chunk_hist[(int64_t)(c0 + u) * E + e] = run;
            run += v[u];
        }
    }
}

// kMode 0: a workgroup (one wavefront) per chunk, chunk_hist holds the histograms of all chunks; 2: the same, but
// chunk_hist holds the running sums over the chunks (route_scan_kernel) and `totals` the column sums; 1: the whole
// problem in one workgroup, a wavefront per chunk, histograms and their running sums in LDS, no chunk_hist.
template <typename IdT, typename MapT, int kMode>
__global__ __launch_bounds__(kMode == 1 ? kBlockChunks * kWave : kWave) void route_map_kernel(
    const IdT *__restrict__ ids, int64_t R, int E, int nchunks, const int *__restrict__ chunk_hist,
    const int *__restrict__ totals, int order, MapT *__restrict__ mappings, int64_t *__restrict__ batch_sizes,
    int64_t *__restrict__ offsets, int top_k, int32_t *__restrict__ row_token) {
    extern __shared__ int sm[];
    constexpr bool kSingle = kMode == 1;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int chunk = kSingle ? wave : blockIdx.x;
    int *excl = sm;                                    // first destination row of expert e
    int *tot = sm + E;                                 // rows of expert e
    int *run = sm + 2 * E + (kSingle ? wave * E : 0);  // rows of expert e before the current 64 (a table per chunk)
    const int64_t base = (int64_t)chunk * kChunk;

    // this lane's rows of the chunk, all loads in flight before anything waits for one
    constexpr int kPerLane = kChunk / kWave;
    int my_id[kPerLane];
    load_chunk_ids(ids, base, lane, R, E, my_id);

    if (kMode == 2) {
        for (int e = lane; e < E; e += kWave) {
            run[e] = chunk_hist[(int64_t)chunk * E + e];
            tot[e] = totals[e];
        }
    } else if (kSingle) {
        const int nw = blockDim.x / kWave;
        for (int e = lane; e < E; e += kWave) run[e] = 0;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < kPerLane; ++i)
            if (my_id[i] >= 0) atomicAdd(&run[my_id[i]], 1);
        __syncthreads();
        // histogram of chunk w -> rows of the chunks before w, and the column sums
        for (int e = threadIdx.x; e < E; e += blockDim.x) {
            int acc = 0;
            for (int w = 0; w < nw; ++w) {
                const int v = sm[(2 + w) * E + e];
                sm[(2 + w) * E + e] = acc;
                acc += v;
            }
            tot[e] = acc;
        }
    } else {
        // Column sums of chunk_hist[nchunks][E]: all rows (tot) and the rows before this chunk (run).  A lane owns
        // expert e0 + lane % span and every slices-th row from row lane / span on, kBatch loads in flight at a
        // time; the slices are added up across the wavefront.
        constexpr int kBatch = kSumBatch;
        int span = kWave;
        while (span / 2 >= E) span /= 2;   // lanes per slice: the power of two that covers E, at most a wavefront
        const int slices = kWave / span, slice = lane / span, el = lane % span;
        for (int e0 = 0; e0 < E; e0 += span) {
            const int e = e0 + el;
            int before = 0, all = 0;
            if (e < E) {
                for (int c0 = slice; c0 < nchunks; c0 += slices * kBatch) {
                    int v[kBatch];
#pragma unroll
                    for (int u = 0; u < kBatch; ++u) {
                        const int c = c0 + u * slices;
                        v[u] = c < nchunks ? chunk_hist[(int64_t)c * E + e] : 0;
                    }
#pragma unroll
                    for (int u = 0; u < kBatch; ++u) {
                        all += v[u];
                        if (c0 + u * slices < chunk) before += v[u];
                    }
                }
            }
            for (int s = span; s < kWave; s <<= 1) {
                before += __shfl_xor(before, s, kWave);
                all += __shfl_xor(all, s, kWave);
            }
            if (e < E && slice == 0) {
                run[e] = before;
                tot[e] = all;
            }
        }
    }
    __syncthreads();

    // exclusive scan of tot over experts, 64 at a time
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += kWave) {
        int e = e0 + lane;
        int v = (e < E) ? tot[e] : 0;
        int incl = v;
#pragma unroll
        for (int s = 1; s < kWave; s <<= 1) {
            int up = __shfl_up(incl, s, kWave);
            if (lane >= s) incl += up;
        }
        if (e < E && wave == 0) excl[e] = carry + incl - v;
        carry += __shfl(incl, kWave - 1, kWave);
    }
    __syncthreads();

    if (chunk == 0) {
        for (int e = lane; e < E; e += kWave) {
            if (batch_sizes) batch_sizes[e] = tot[e];
            if (offsets) offsets[e] = excl[e];
        }
        if (offsets && lane == 0) offsets[E] = carry;
    }

    int nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));

#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const int64_t t = base + i * kWave + lane;
        const int id = my_id[i];
        const bool ok = id >= 0;
        unsigned long long same = __ballot(ok);
        for (int b = 0; b < nbits; ++b) {
            const bool bit = ok && ((id >> b) & 1);
            const unsigned long long bal = __ballot(bit);
            same &= bit ? bal : ~bal;
        }
        const int lower = __popcll(same & below);
        const int total = __popcll(same);
        const int seen = ok ? run[id] : 0;
        __syncthreads();
        if (ok && lower == 0) run[id] = seen + total;
        __syncthreads();
        if (ok) {
            const int rank = seen + lower;
            const int pos = (order == DMOE_ORDER_REFERENCE) ? excl[id] + tot[id] - 1 - rank : excl[id] + rank;
            mappings[t] = (MapT)pos;
            // the inverse, for a consumer that fetches the rows of a [T, d] tensor by their place in the expert-sorted
            // order instead of having them moved there: destination row -> token
            if (row_token != nullptr) row_token[pos] = (int32_t)((uint32_t)t / (uint32_t)top_k);
        } else if (id == -1) {
            mappings[t] = (MapT)-1;
        }
    }
}

// a few chunks are routed by a single workgroup if its 2 + nchunks tables fit in 64 KiB of LDS
static bool one_workgroup(int64_t nchunks, int E) {
    return nchunks <= 1 || (nchunks <= kBlockChunks && (2 + nchunks) * (int64_t)E * (int64_t)sizeof(int) <= (64 << 10));
}

template <typename IdT, typename MapT>
static int launch_route(const void *ids, int64_t R, int E, int order, void *mappings, int64_t *batch_sizes,
                        int64_t *offsets, void *scratch, int top_k, int32_t *row_token, hipStream_t stream) {
    const int nchunks = (int)((R + kChunk - 1) / kChunk);
    const size_t lds = 3 * (size_t)E * sizeof(int);
    if (one_workgroup(nchunks, E)) {
        const int nw = nchunks < 1 ? 1 : nchunks;
        hipLaunchKernelGGL((route_map_kernel<IdT, MapT, 1>), dim3(1), dim3(nw * kWave), (2 + nw) * (size_t)E * sizeof(int),
                           stream, (const IdT *)ids, R, E, nw, (const int *)nullptr, (const int *)nullptr, order,
                           (MapT *)mappings, batch_sizes, offsets, top_k, row_token);
        DMOE_LAUNCH_CHECK("route_map_kernel");
        return DMOE_OK;
    }
    int *hist = (int *)scratch;
    hipLaunchKernelGGL((route_hist_kernel<IdT>), dim3(nchunks), dim3(kWave), (size_t)E * sizeof(int), stream,
                       (const IdT *)ids, R, E, hist);
    DMOE_LAUNCH_CHECK("route_hist_kernel");
    int span = kWave;   // lanes of pass 2 that share a histogram row (see route_map_kernel)
    while (span / 2 >= E) span /= 2;
    if (nchunks > 2 * kSumBatch * (kWave / span)) {
        int *totals = hist + (size_t)nchunks * E;
        hipLaunchKernelGGL(route_scan_kernel, dim3((E + kWave - 1) / kWave), dim3(kScanWaves * kWave), 0, stream, hist,
                           nchunks, E, totals);
        DMOE_LAUNCH_CHECK("route_scan_kernel");
        hipLaunchKernelGGL((route_map_kernel<IdT, MapT, 2>), dim3(nchunks), dim3(kWave), lds, stream, (const IdT *)ids,
                           R, E, nchunks, (const int *)hist, (const int *)totals, order, (MapT *)mappings, batch_sizes,
                           offsets, top_k, row_token);
    } else {
        hipLaunchKernelGGL((route_map_kernel<IdT, MapT, 0>), dim3(nchunks), dim3(kWave), lds, stream, (const IdT *)ids,
                           R, E, nchunks, (const int *)hist, (const int *)nullptr, order, (MapT *)mappings, batch_sizes,
                           offsets, top_k, row_token);
    }
    DMOE_LAUNCH_CHECK("route_map_kernel");
    return DMOE_OK;
}

}  // namespace dmoe

using namespace dmoe;

extern "C" const char *dmoe_version(void) { return "dmoe-hip gfx950 0.1"; }
extern "C" const char *dmoe_last_error(void) { return error_buffer(); }

extern "C" int dmoe_device_cus(int *cus) {
    DMOE_REQUIRE(cus != nullptr, DMOE_ERR_ARG, "dmoe_device_cus: null output");
    *cus = device_cus();
    return DMOE_OK;
}

extern "C" int dmoe_route_scratch_bytes(int64_t R, int E, size_t *bytes) {
    DMOE_REQUIRE(bytes != nullptr, DMOE_ERR_ARG, "dmoe_route_scratch_bytes: null output");
    DMOE_REQUIRE(R >= 0 && R < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_route: R=%lld outside [0, 2^31)", (long long)R);
    DMOE_REQUIRE(E > 0 && E <= kMaxExperts, DMOE_ERR_SHAPE, "dmoe_route: E=%d outside [1, %d]", E, kMaxExperts);
    const int64_t nchunks = (R + kChunk - 1) / kChunk;
    // a histogram per chunk and, behind them, the column sums of the scanned form
    *bytes = one_workgroup(nchunks, E) ? 0 : (size_t)(nchunks + 1) * (size_t)E * sizeof(int);
    return DMOE_OK;
}

// Device address of the file-scope scratch array on the current device (looked up once per device).
static int static_scratch(void **out) {
    static std::mutex mu;
    static void *ptr_of_device[64];
    int dev = 0;
    DMOE_HIP(hipGetDevice(&dev));
    DMOE_REQUIRE(dev >= 0 && dev < 64, DMOE_ERR_ARG, "dmoe_route_noalloc: device ordinal %d outside [0, 64)", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (ptr_of_device[dev] == nullptr) {
        void *ptr = nullptr;
        DMOE_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(dmoe::scratch)));
        DMOE_REQUIRE(ptr != nullptr, DMOE_ERR_HIP, "dmoe_route_noalloc: no device address for the scratch array");
        ptr_of_device[dev] = ptr;
    }
    *out = ptr_of_device[dev];
    return DMOE_OK;
}

extern "C" int dmoe_route_noalloc_max_bytes(size_t *bytes) {
    DMOE_REQUIRE(bytes != nullptr, DMOE_ERR_ARG, "dmoe_route_noalloc_max_bytes: null output");
    *bytes = kStaticScratchBytes;
    return DMOE_OK;
}

extern "C" int dmoe_route_noalloc(const void *ids, int ids_type, int64_t R, int E, int order, void *mappings,
                                  int map_type, int64_t *batch_sizes, int64_t *offsets, void *stream) {
    size_t need = 0;
    int rc = dmoe_route_scratch_bytes(R, E, &need);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(need <= kStaticScratchBytes, DMOE_ERR_WORKSPACE,
                 "dmoe_route_noalloc: R=%lld rows over E=%d experts need %zu bytes of scratch, the built-in buffer holds %zu "
                 "(use dmoe_route with a caller-owned buffer)", (long long)R, E, need, (size_t)kStaticScratchBytes);
    void *ptr = nullptr;
    rc = static_scratch(&ptr);
    if (rc != DMOE_OK) return rc;
    // every entry of the histograms that a launch reads has been written by the launch before it: nothing to clear
    return dmoe_route(ids, ids_type, R, E, order, mappings, map_type, batch_sizes, offsets, ptr, kStaticScratchBytes, stream);
}

static int route_checked(const char *who, const void *ids, int ids_type, int64_t R, int E, int order, void *mappings,
                         int map_type, int64_t *batch_sizes, int64_t *offsets, void *scratch, size_t scratch_bytes,
                         int top_k, int32_t *row_token, void *stream) {
    size_t need = 0;
    int rc = dmoe_route_scratch_bytes(R, E, &need);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(order == DMOE_ORDER_REFERENCE || order == DMOE_ORDER_STABLE, DMOE_ERR_ARG,
                 "%s: unknown order %d", who, order);
    DMOE_REQUIRE(ids_type == DMOE_I32 || ids_type == DMOE_I64, DMOE_ERR_DTYPE, "%s: ids type %d", who, ids_type);
    DMOE_REQUIRE(map_type == DMOE_I32 || map_type == DMOE_I64, DMOE_ERR_DTYPE, "%s: mapping type %d", who, map_type);
    DMOE_REQUIRE(R == 0 || (ids != nullptr && mappings != nullptr), DMOE_ERR_ARG, "%s: null ids/mappings", who);
    DMOE_REQUIRE(need == 0 || (scratch != nullptr && scratch_bytes >= need), DMOE_ERR_WORKSPACE,
                 "%s: scratch of %zu bytes needed, %zu given", who, need, scratch_bytes);
    DMOE_REQUIRE(top_k >= 1 && R % top_k == 0, DMOE_ERR_SHAPE, "%s: R=%lld is not a multiple of top_k=%d", who, (long long)R,
                 top_k);
    hipStream_t s = (hipStream_t)stream;
    if (ids_type == DMOE_I32) {
        if (map_type == DMOE_I32)
            return launch_route<int32_t, int32_t>(ids, R, E, order, mappings, batch_sizes, offsets, scratch, top_k, row_token, s);
        return launch_route<int32_t, int64_t>(ids, R, E, order, mappings, batch_sizes, offsets, scratch, top_k, row_token, s);
    }
    if (map_type == DMOE_I32)
        return launch_route<int64_t, int32_t>(ids, R, E, order, mappings, batch_sizes, offsets, scratch, top_k, row_token, s);
    return launch_route<int64_t, int64_t>(ids, R, E, order, mappings, batch_sizes, offsets, scratch, top_k, row_token, s);
}

extern "C" int dmoe_route(const void *ids, int ids_type, int64_t R, int E, int order, void *mappings, int map_type,
                          int64_t *batch_sizes, int64_t *offsets, void *scratch, size_t scratch_bytes,
                          void *stream) {
    return route_checked("dmoe_route", ids, ids_type, R, E, order, mappings, map_type, batch_sizes, offsets, scratch,
                         scratch_bytes, 1, nullptr, stream);
}

extern "C" int dmoe_route_sources(const void *ids, int ids_type, int64_t R, int E, int order, void *mappings, int map_type,
                                  int64_t *batch_sizes, int64_t *offsets, int top_k, int32_t *row_token, void *scratch,
                                  size_t scratch_bytes, void *stream) {
    DMOE_REQUIRE(R == 0 || row_token != nullptr, DMOE_ERR_ARG, "dmoe_route_sources: null row_token");
    return route_checked("dmoe_route_sources", ids, ids_type, R, E, order, mappings, map_type, batch_sizes, offsets, scratch,
                         scratch_bytes, top_k, row_token, stream);
}
