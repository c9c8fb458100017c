// Row movement: permute (scatter with top-k duplication), gathers, the
// gate-weighted combine and the per-row fp8 quantiser.  All are HBM-bound: one
// wavefront moves one segment of one row with 16-byte accesses per lane, kVecs
// of them in flight per lane, and reads its row index once.
#include "common.h"

namespace dmoe {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kVecs = 4;                    // 16-byte vectors per lane per segment
constexpr int kSegVecs = kWave * kVecs;     // 256 vectors = 4 KiB per segment
constexpr int kBlock = 256;                 // 4 wavefronts per workgroup

template <typename MapT>
__device__ __forceinline__ int64_t load_map(const MapT *m, int64_t i) { return (int64_t)m[i]; }

__device__ __forceinline__ u32x4 scale_bf16x8(u32x4 v, float s) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float lo = bf16_to_f32((uint16_t)(v[i] & 0xffffu)) * s;
        float hi = bf16_to_f32((uint16_t)(v[i] >> 16)) * s;
        r[i] = pack_bf16x2(lo, hi);
    }
    return r;
}

__device__ __forceinline__ float half_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}
__device__ __forceinline__ uint16_t f32_to_half_bits(float f) {
    const _Float16 v = (_Float16)f;  // round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

__device__ __forceinline__ u32x4 scale_f16x8(u32x4 v, float s) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float lo = half_bits_to_f32((uint16_t)(v[i] & 0xffffu)) * s;
        float hi = half_bits_to_f32((uint16_t)(v[i] >> 16)) * s;
        r[i] = (uint32_t)f32_to_half_bits(lo) | ((uint32_t)f32_to_half_bits(hi) << 16);
    }
    return r;
}

// out[map[i*k + j]] = in[i] (* scale[i*k + j]); one wavefront per (token i, segment).
template <typename MapT, int kScale /*0 none, 1 bf16, 2 fp16*/, bool kStreamed>
__global__ __launch_bounds__(kBlock) void permute_kernel(const u32x4 *__restrict__ in, u32x4 *__restrict__ out,
                                                        const MapT *__restrict__ map, int64_t T, int k, int64_t R,
                                                        int vecs, int nseg, const uint16_t *__restrict__ scale) {
    const int64_t item = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x / kWave);
    if (item >= T * nseg) return;
    const int64_t tok = item / nseg;
    const int seg = (int)(item - tok * nseg);
    const int lane = lane_id();
    const int v0 = seg * kSegVecs + lane;
    u32x4 buf[kVecs];
    const u32x4 *src = in + tok * vecs;
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
        const int v = v0 + u * kWave;
        if (v < vecs) buf[u] = src[v];
    }
    for (int j = 0; j < k; ++j) {
        const int64_t t = tok * k + j;
        const int64_t p = load_map(map, t);
        if (p < 0 || p >= R) continue;
        u32x4 *dst = out + p * vecs;
        float s = 1.f;
        if (kScale == 1) s = bf16_to_f32(scale[t]);
        if (kScale == 2) s = half_bits_to_f32(scale[t]);
#pragma unroll
        for (int u = 0; u < kVecs; ++u) {
            const int v = v0 + u * kWave;
            if (v < vecs) {
                u32x4 x = buf[u];
                if (kScale == 1) x = scale_bf16x8(x, s);
                if (kScale == 2) x = scale_f16x8(x, s);
                // an output larger than the last-level cache is written past it
                if (kStreamed) __builtin_nontemporal_store(x, dst + v);
                else dst[v] = x;
            }
        }
    }
}

// out[t] = in[index[t]] or *(rows[t]); one wavefront per (row t, segment).
template <typename IdxT, bool kPtrs>
__global__ __launch_bounds__(kBlock) void gather_kernel(const u32x4 *__restrict__ in,
                                                       const void *const *__restrict__ rows,
                                                       u32x4 *__restrict__ out, const IdxT *__restrict__ index,
                                                       int64_t N, int64_t n_src, int vecs, int nseg) {
    const int64_t item = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x / kWave);
    if (item >= N * nseg) return;
    const int64_t t = item / nseg;
    const int seg = (int)(item - t * nseg);
    const int lane = lane_id();
    const u32x4 *src = nullptr;
    if (kPtrs) {
        src = (const u32x4 *)rows[t];
    } else {
        const int64_t s = (int64_t)index[t];
        if (s >= 0 && s < n_src) src = in + s * vecs;
    }
    u32x4 *dst = out + t * vecs;
    const int v0 = seg * kSegVecs + lane;
    u32x4 buf[kVecs];
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
        const int v = v0 + u * kWave;
        buf[u] = u32x4{0, 0, 0, 0};
        if (v < vecs && src != nullptr) buf[u] = src[v];
    }
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
        const int v = v0 + u * kWave;
        if (v < vecs) dst[v] = buf[u];
    }
}

template <bool kHalf>
__device__ __forceinline__ float elem_to_f32(uint16_t v) { return kHalf ? half_bits_to_f32(v) : bf16_to_f32(v); }
template <bool kHalf>
__device__ __forceinline__ uint16_t f32_to_elem(float f) { return kHalf ? f32_to_half_bits(f) : f32_to_bf16(f); }

// out[i] = sum_j w[i,j] * y[map[i*k+j]]; one wavefront per (token i, segment).
template <typename MapT, bool kHalf, int kMode, bool kStreamed>
__global__ __launch_bounds__(kBlock) void combine_kernel(const u32x4 *__restrict__ y, const MapT *__restrict__ map,
                                                        const float *__restrict__ w, u32x4 *__restrict__ out,
                                                        int64_t T, int k, int64_t R, int vecs, int nseg) {
    const int64_t item = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x / kWave);
    if (item >= T * nseg) return;
    const int64_t tok = item / nseg;
    const int seg = (int)(item - tok * nseg);
    const int lane = lane_id();
    const int v0 = seg * kSegVecs + lane;
    float acc[kVecs][8];
#pragma unroll
    for (int u = 0; u < kVecs; ++u)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[u][i] = 0.f;
    bool first = true;
    for (int j = 0; j < k; ++j) {
        const int64_t t = tok * k + j;
        const int64_t p = load_map(map, t);
        if (p < 0 || p >= R) continue;
        float g = w[t];
        if (kMode == DMOE_COMBINE_REFERENCE) g = elem_to_f32<kHalf>(f32_to_elem<kHalf>(g));
        const u32x4 *src = y + p * vecs;
        u32x4 buf[kVecs];
#pragma unroll
        for (int u = 0; u < kVecs; ++u) {
            const int v = v0 + u * kWave;
            buf[u] = u32x4{0, 0, 0, 0};
            // every row of y is read once; when y is larger than the last-level cache the loads say so
            if (v < vecs) buf[u] = kStreamed ? __builtin_nontemporal_load(src + v) : src[v];
        }
#pragma unroll
        for (int u = 0; u < kVecs; ++u) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = elem_to_f32<kHalf>((uint16_t)(buf[u][i] & 0xffffu));
                const float hi = elem_to_f32<kHalf>((uint16_t)(buf[u][i] >> 16));
                if (kMode == DMOE_COMBINE_REFERENCE) {
                    // product rounded to the row type, running sum rounded after every add
                    const float plo = elem_to_f32<kHalf>(f32_to_elem<kHalf>(lo * g));
                    const float phi = elem_to_f32<kHalf>(f32_to_elem<kHalf>(hi * g));
                    acc[u][2 * i] = first ? plo : elem_to_f32<kHalf>(f32_to_elem<kHalf>(acc[u][2 * i] + plo));
                    acc[u][2 * i + 1] = first ? phi : elem_to_f32<kHalf>(f32_to_elem<kHalf>(acc[u][2 * i + 1] + phi));
                } else {
                    acc[u][2 * i] = fmaf(g, lo, acc[u][2 * i]);
                    acc[u][2 * i + 1] = fmaf(g, hi, acc[u][2 * i + 1]);
                }
            }
        }
        first = false;
    }
    u32x4 *dst = out + tok * vecs;
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
        const int v = v0 + u * kWave;
        if (v < vecs) {
            u32x4 r;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                r[i] = kHalf ? (uint32_t)f32_to_half_bits(acc[u][2 * i]) | ((uint32_t)f32_to_half_bits(acc[u][2 * i + 1]) << 16)
                             : pack_bf16x2(acc[u][2 * i], acc[u][2 * i + 1]);   // one instruction for the pair
            dst[v] = r;
        }
    }
}

// q[map[i*k + j], :] = fp8(x[i, :] / s[i]) and scales[map[i*k + j]] = s[i] for j < k: the permute and the per-row
// quantisation in one pass (without a mapping: the quantisation alone, q[i, :] and scales[i]).  One workgroup per token;
// the row is read once (kept in registers when it has at most 16384 elements), quantised once and stored k times.
template <typename MapT, bool kHalf, bool kStreamed>
__global__ __launch_bounds__(kBlock) void permute_quant_kernel(const u32x4 *__restrict__ x, uint2 *__restrict__ q,
                                                              float *__restrict__ scales, const MapT *__restrict__ map,
                                                              int k, int64_t R, int vecs) {
    constexpr int kKeep = 8;   // 16-byte vectors per thread held in registers
    __shared__ float wave_max[kBlock / kWave];
    const int64_t tok = blockIdx.x;
    const u32x4 *src = x + tok * vecs;
    const bool keep = vecs <= kKeep * kBlock;
    u32x4 held[kKeep];
    float amax = 0.f;
    auto absmax_of = [&](const u32x4 &b) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            amax = fmaxf(amax, fabsf(elem_to_f32<kHalf>((uint16_t)(b[i] & 0xffffu))));
            amax = fmaxf(amax, fabsf(elem_to_f32<kHalf>((uint16_t)(b[i] >> 16))));
        }
    };
    // register slots a row of this length fills (the same for every thread): the conversions, 17 instructions per
    // element, are what bounds this kernel, and a row of 6144 elements fills 3 of the 8 slots
    const int slots = (vecs + kBlock - 1) / kBlock;
    if (keep) {
#pragma unroll
        for (int u = 0; u < kKeep; ++u) {
            const int v = threadIdx.x + u * kBlock;
            held[u] = u32x4{0, 0, 0, 0};
            if (v < vecs) held[u] = __builtin_nontemporal_load(src + v);
        }
#pragma unroll
        for (int u = 0; u < kKeep; ++u)
            if (u < slots) absmax_of(held[u]);
    } else {
        for (int v = threadIdx.x; v < vecs; v += kBlock) absmax_of(src[v]);
    }
#pragma unroll
    for (int s = kWave / 2; s > 0; s >>= 1) amax = fmaxf(amax, __shfl_xor(amax, s, kWave));
    if (lane_id() == 0) wave_max[threadIdx.x / kWave] = amax;
    __syncthreads();
    amax = wave_max[0];
#pragma unroll
    for (int i = 1; i < kBlock / kWave; ++i) amax = fmaxf(amax, wave_max[i]);
    float s = amax / 448.f;
    if (!(s > 0.f)) s = 1.f;
    auto quantised = [&](const u32x4 &b) {
        uint32_t o[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = __builtin_amdgcn_fmed3f(elem_to_f32<kHalf>((uint16_t)(b[i] & 0xffffu)) / s, -448.f, 448.f);
            const float hi = __builtin_amdgcn_fmed3f(elem_to_f32<kHalf>((uint16_t)(b[i] >> 16)) / s, -448.f, 448.f);
            if (i & 1) o[i / 2] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, (int)o[i / 2], true);
            else o[i / 2] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, (int)o[i / 2], false);
        }
        return make_uint2(o[0], o[1]);
    };
    if (keep) {
        uint2 out[kKeep];
#pragma unroll
        for (int u = 0; u < kKeep; ++u)
            if (u < slots) out[u] = quantised(held[u]);
        for (int j = 0; j < k; ++j) {
            const int64_t p = map ? load_map(map, tok * k + j) : tok;   // no mapping: rows stay where they are
            if (p < 0 || p >= R) continue;
            if (threadIdx.x == 0) scales[p] = s;
            uint2 *dst = q + p * vecs;
#pragma unroll
            for (int u = 0; u < kKeep; ++u) {
                const int v = threadIdx.x + u * kBlock;
                if (v >= vecs) continue;
                if (kStreamed)
                    __builtin_nontemporal_store(((unsigned long long)out[u].y << 32) | out[u].x, (unsigned long long *)(dst + v));
                else dst[v] = out[u];
            }
        }
    } else {
        for (int j = 0; j < k; ++j) {
            const int64_t p = map ? load_map(map, tok * k + j) : tok;   // no mapping: rows stay where they are
            if (p < 0 || p >= R) continue;
            if (threadIdx.x == 0) scales[p] = s;
            uint2 *dst = q + p * vecs;
            for (int v = threadIdx.x; v < vecs; v += kBlock) dst[v] = quantised(src[v]);
        }
    }
}

static int check_rows(const char *who, int64_t d, int dtype, int *vecs) {
    DMOE_REQUIRE(dtype == DMOE_BF16 || dtype == DMOE_FP16 || dtype == DMOE_FP8_E4M3, DMOE_ERR_DTYPE,
                 "%s: unsupported dtype %d", who, dtype);
    const int64_t esize = (dtype == DMOE_FP8_E4M3) ? 1 : 2;
    DMOE_REQUIRE(d > 0 && (d * esize) % 16 == 0, DMOE_ERR_SHAPE, "%s: row of %lld bytes is not a multiple of 16",
                 who, (long long)(d * esize));
    DMOE_REQUIRE(d * esize / 16 < (1ll << 30), DMOE_ERR_SHAPE, "%s: row too long", who);
    *vecs = (int)(d * esize / 16);
    return DMOE_OK;
}

static inline int64_t blocks_for(int64_t items) { return (items + (kBlock / kWave) - 1) / (kBlock / kWave); }

}  // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_permute(const void *in, void *out, const void *mappings, int map_type, int64_t T, int64_t R,
                            int64_t d, int dtype, const void *row_scale, void *stream) {
    int vecs = 0;
    int rc = check_rows("dmoe_permute", d, dtype, &vecs);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(T >= 0 && R >= 0, DMOE_ERR_ARG, "dmoe_permute: negative size");
    if (R == 0) return DMOE_OK;
    DMOE_REQUIRE(T > 0 && R % T == 0, DMOE_ERR_SHAPE, "dmoe_permute: R=%lld is not a multiple of T=%lld", (long long)R,
                 (long long)T);
    DMOE_REQUIRE(R / T <= 1024, DMOE_ERR_SHAPE, "dmoe_permute: top-k %lld too large", (long long)(R / T));
    DMOE_REQUIRE(in && out && mappings, DMOE_ERR_ARG, "dmoe_permute: null pointer");
    DMOE_REQUIRE(map_type == DMOE_I32 || map_type == DMOE_I64, DMOE_ERR_DTYPE, "dmoe_permute: mapping type %d",
                 map_type);
    DMOE_REQUIRE(row_scale == nullptr || dtype != DMOE_FP8_E4M3, DMOE_ERR_DTYPE, "dmoe_permute: no scale for fp8 rows");
    const int k = (int)(R / T);
    const int nseg = (vecs + kSegVecs - 1) / kSegVecs;
    const int64_t nblk = blocks_for(T * nseg);
    DMOE_REQUIRE(nblk < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_permute: too many rows");
    hipStream_t s = (hipStream_t)stream;
    const int sc = row_scale ? (dtype == DMOE_FP16 ? 2 : 1) : 0;
    // measured: non-temporal stores are 34 % faster on 403 MB of routed rows (6.7 TB/s moved), within 3 % on 67 MB and
    // 25 % slower on 201 MB, which the 256 MB Infinity Cache can still hand to the kernel that reads the rows next
    const bool streamed = R * (int64_t)vecs * 16 > (256ll << 20);
#define DMOE_PERMUTE_LAUNCH_ONE(MAPT, SC, ST)                                                                      \
    hipLaunchKernelGGL((permute_kernel<MAPT, SC, ST>), dim3((unsigned)nblk), dim3(kBlock), 0, s, (const u32x4 *)in, \
                       (u32x4 *)out, (const MAPT *)mappings, T, k, R, vecs, nseg, (const uint16_t *)row_scale)
#define DMOE_PERMUTE_LAUNCH(MAPT, SC)                                                                              \
    do {                                                                                                            \
        if (streamed) DMOE_PERMUTE_LAUNCH_ONE(MAPT, SC, true);                                                      \
        else DMOE_PERMUTE_LAUNCH_ONE(MAPT, SC, false);                                                              \
    } while (0)
    if (map_type == DMOE_I64) {
        if (sc == 0) DMOE_PERMUTE_LAUNCH(int64_t, 0);
        else if (sc == 1) DMOE_PERMUTE_LAUNCH(int64_t, 1);
        else DMOE_PERMUTE_LAUNCH(int64_t, 2);
    } else {
        if (sc == 0) DMOE_PERMUTE_LAUNCH(int32_t, 0);
        else if (sc == 1) DMOE_PERMUTE_LAUNCH(int32_t, 1);
        else DMOE_PERMUTE_LAUNCH(int32_t, 2);
    }
#undef DMOE_PERMUTE_LAUNCH_ONE
#undef DMOE_PERMUTE_LAUNCH
    DMOE_LAUNCH_CHECK("permute_kernel");
    return DMOE_OK;
}

extern "C" int dmoe_gather_rows(const void *in, void *out, const void *index, int idx_type, int64_t N, int64_t n_src,
                                int64_t d, int dtype, void *stream) {
    int vecs = 0;
    int rc = check_rows("dmoe_gather_rows", d, dtype, &vecs);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(N >= 0 && n_src >= 0, DMOE_ERR_ARG, "dmoe_gather_rows: negative size");
    if (N == 0) return DMOE_OK;
    DMOE_REQUIRE(out && index && (in || n_src == 0), DMOE_ERR_ARG, "dmoe_gather_rows: null pointer");
    DMOE_REQUIRE(idx_type == DMOE_I32 || idx_type == DMOE_I64, DMOE_ERR_DTYPE, "dmoe_gather_rows: index type %d",
                 idx_type);
    const int nseg = (vecs + kSegVecs - 1) / kSegVecs;
    const int64_t nblk = blocks_for(N * nseg);
    DMOE_REQUIRE(nblk < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_gather_rows: too many rows");
    hipStream_t s = (hipStream_t)stream;
    if (idx_type == DMOE_I64)
        hipLaunchKernelGGL((gather_kernel<int64_t, false>), dim3((unsigned)nblk), dim3(kBlock), 0, s, (const u32x4 *)in,
                           (const void *const *)nullptr, (u32x4 *)out, (const int64_t *)index, N, n_src, vecs, nseg);
    else
        hipLaunchKernelGGL((gather_kernel<int32_t, false>), dim3((unsigned)nblk), dim3(kBlock), 0, s, (const u32x4 *)in,
                           (const void *const *)nullptr, (u32x4 *)out, (const int32_t *)index, N, n_src, vecs, nseg);
    DMOE_LAUNCH_CHECK("gather_kernel");
    return DMOE_OK;
}

extern "C" int dmoe_gather_ptrs(const void *const *src_rows, void *out, int64_t N, int64_t d, int dtype,
                                void *stream) {
    int vecs = 0;
    int rc = check_rows("dmoe_gather_ptrs", d, dtype, &vecs);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(N >= 0, DMOE_ERR_ARG, "dmoe_gather_ptrs: negative size");
    if (N == 0) return DMOE_OK;
    DMOE_REQUIRE(out && src_rows, DMOE_ERR_ARG, "dmoe_gather_ptrs: null pointer");
    const int nseg = (vecs + kSegVecs - 1) / kSegVecs;
    const int64_t nblk = blocks_for(N * nseg);
    DMOE_REQUIRE(nblk < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_gather_ptrs: too many rows");
    hipLaunchKernelGGL((gather_kernel<int64_t, true>), dim3((unsigned)nblk), dim3(kBlock), 0, (hipStream_t)stream,
                       (const u32x4 *)nullptr, src_rows, (u32x4 *)out, (const int64_t *)nullptr, N, (int64_t)0, vecs,
                       nseg);
    DMOE_LAUNCH_CHECK("gather_kernel");
    return DMOE_OK;
}

extern "C" int dmoe_combine(const void *y, const void *mappings, int map_type, const float *weights, void *out,
                            int64_t T, int k, int64_t d, int dtype, int mode, void *stream) {
    int vecs = 0;
    int rc = check_rows("dmoe_combine", d, dtype, &vecs);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(dtype == DMOE_BF16 || dtype == DMOE_FP16, DMOE_ERR_DTYPE, "dmoe_combine: dtype %d", dtype);
    DMOE_REQUIRE(T >= 0 && k > 0 && k <= 1024, DMOE_ERR_ARG, "dmoe_combine: bad T/k");
    DMOE_REQUIRE(mode == DMOE_COMBINE_FP32 || mode == DMOE_COMBINE_REFERENCE, DMOE_ERR_ARG,
                 "dmoe_combine: unknown mode %d", mode);
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(y && mappings && weights && out, DMOE_ERR_ARG, "dmoe_combine: null pointer");
    DMOE_REQUIRE(map_type == DMOE_I32 || map_type == DMOE_I64, DMOE_ERR_DTYPE, "dmoe_combine: mapping type %d",
                 map_type);
    const int64_t R = T * k;
    const int nseg = (vecs + kSegVecs - 1) / kSegVecs;
    const int64_t nblk = blocks_for(T * nseg);
    DMOE_REQUIRE(nblk < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_combine: too many rows");
    hipStream_t s = (hipStream_t)stream;
    // measured: non-temporal loads of y are 20 % faster on 403 MB of rows and 8 % slower on 67 and 201 MB, which the
    // 256 MB Infinity Cache can still hold between the GEMM that wrote them and this kernel
    const bool streamed = R * (int64_t)vecs * 16 > (256ll << 20);
#define DMOE_COMBINE_LAUNCH_ONE(MAPT, HALF, MODE, STREAMED)                                                           \
    hipLaunchKernelGGL((combine_kernel<MAPT, HALF, MODE, STREAMED>), dim3((unsigned)nblk), dim3(kBlock), 0, s,         \
                       (const u32x4 *)y, (const MAPT *)mappings, weights, (u32x4 *)out, T, k, R, vecs, nseg)
#define DMOE_COMBINE_LAUNCH(MAPT, HALF, MODE)                                                                       \
    do {                                                                                                            \
        if (streamed) DMOE_COMBINE_LAUNCH_ONE(MAPT, HALF, MODE, true);                                              \
        else DMOE_COMBINE_LAUNCH_ONE(MAPT, HALF, MODE, false);                                                      \
    } while (0)
    const bool half = dtype == DMOE_FP16;
    if (map_type == DMOE_I64) {
        if (!half && mode == 0) DMOE_COMBINE_LAUNCH(int64_t, false, 0);
        else if (!half) DMOE_COMBINE_LAUNCH(int64_t, false, 1);
        else if (mode == 0) DMOE_COMBINE_LAUNCH(int64_t, true, 0);
        else DMOE_COMBINE_LAUNCH(int64_t, true, 1);
    } else {
        if (!half && mode == 0) DMOE_COMBINE_LAUNCH(int32_t, false, 0);
        else if (!half) DMOE_COMBINE_LAUNCH(int32_t, false, 1);
        else if (mode == 0) DMOE_COMBINE_LAUNCH(int32_t, true, 0);
        else DMOE_COMBINE_LAUNCH(int32_t, true, 1);
    }
#undef DMOE_COMBINE_LAUNCH
#undef DMOE_COMBINE_LAUNCH_ONE
    DMOE_LAUNCH_CHECK("combine_kernel");
    return DMOE_OK;
}

extern "C" int dmoe_quant_rows(const void *x, void *q, float *scales, int64_t rows, int64_t d, int dtype,
                               void *stream) {
    int vecs = 0;
    int rc = check_rows("dmoe_quant_rows", d, dtype, &vecs);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(dtype == DMOE_BF16 || dtype == DMOE_FP16, DMOE_ERR_DTYPE, "dmoe_quant_rows: input dtype %d", dtype);
    DMOE_REQUIRE(rows >= 0 && rows < (1ll << 31), DMOE_ERR_ARG, "dmoe_quant_rows: bad row count");
    if (rows == 0) return DMOE_OK;
    DMOE_REQUIRE(x && q && scales, DMOE_ERR_ARG, "dmoe_quant_rows: null pointer");
    // the fused permute + quantise kernel without a mapping; quantised rows beyond the size of the last-level cache
    // leave with non-temporal stores (537 MB: 5 % faster)
    const bool streamed = rows * (int64_t)vecs * 8 > (256ll << 20);
#define DMOE_QUANT_LAUNCH(HALF, ST)                                                                                    \
    hipLaunchKernelGGL((permute_quant_kernel<int64_t, HALF, ST>), dim3((unsigned)rows), dim3(kBlock), 0,               \
                       (hipStream_t)stream, (const u32x4 *)x, (uint2 *)q, scales, (const int64_t *)nullptr, 1, rows, vecs)
    if (dtype == DMOE_FP16) { if (streamed) DMOE_QUANT_LAUNCH(true, true); else DMOE_QUANT_LAUNCH(true, false); }
    else { if (streamed) DMOE_QUANT_LAUNCH(false, true); else DMOE_QUANT_LAUNCH(false, false); }
#undef DMOE_QUANT_LAUNCH
    DMOE_LAUNCH_CHECK("permute_quant_kernel");
    return DMOE_OK;
}

extern "C" int dmoe_permute_quant(const void *in, void *q, float *scales, const void *mappings, int map_type, int64_t T,
                                  int64_t R, int64_t d, int dtype, void *stream) {
    int vecs = 0;
    int rc = check_rows("dmoe_permute_quant", d, dtype, &vecs);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(dtype == DMOE_BF16 || dtype == DMOE_FP16, DMOE_ERR_DTYPE, "dmoe_permute_quant: dtype %d", dtype);
    DMOE_REQUIRE(T >= 0 && R >= 0 && T < (1ll << 31), DMOE_ERR_ARG, "dmoe_permute_quant: bad T/R");
    DMOE_REQUIRE(T == 0 ? R == 0 : R % T == 0, DMOE_ERR_SHAPE, "dmoe_permute_quant: R=%lld is not a multiple of T=%lld",
                 (long long)R, (long long)T);
    DMOE_REQUIRE(map_type == DMOE_I32 || map_type == DMOE_I64, DMOE_ERR_DTYPE, "dmoe_permute_quant: mapping type %d", map_type);
    if (R == 0) return DMOE_OK;
    DMOE_REQUIRE(in && q && scales && mappings, DMOE_ERR_ARG, "dmoe_permute_quant: null pointer");
    const int k = (int)(R / T);
    hipStream_t s = (hipStream_t)stream;
#define DMOE_PQ_LAUNCH(MAPT, HALF)                                                                                     \
    hipLaunchKernelGGL((permute_quant_kernel<MAPT, HALF, false>), dim3((unsigned)T), dim3(kBlock), 0, s,              \
                       (const u32x4 *)in, (uint2 *)q, scales, (const MAPT *)mappings, k, R, vecs)
    const bool half = dtype == DMOE_FP16;
    if (map_type == DMOE_I64) { if (half) DMOE_PQ_LAUNCH(int64_t, true); else DMOE_PQ_LAUNCH(int64_t, false); }
    else { if (half) DMOE_PQ_LAUNCH(int32_t, true); else DMOE_PQ_LAUNCH(int32_t, false); }
#undef DMOE_PQ_LAUNCH
    DMOE_LAUNCH_CHECK("permute_quant_kernel");
    return DMOE_OK;
}
