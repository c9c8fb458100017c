// Routing producer: softmax over the router logits of a token, its k largest probabilities and
// their expert ids, optionally renormalised to sum 1.
//
// A token is handled by a group of W lanes (W = 8, 16, 32 or 64), 64 / W tokens per wavefront; a lane
// keeps ceil(E / W) logits in registers.  Few tokens: W is the power of two that covers E (64 beyond
// that); many tokens: W = 8 or 16 with up to 16 logits per lane.
// Max, sum and the k arg-max rounds are butterfly reductions inside the group; every lane of the
// group ends up with the same winner, so there is no LDS and no atomics.  Ties go to the lower
// expert id.  The work is one read of the logits: HBM-bound, a few microseconds at serving sizes.
#include "common.h"

namespace dmoe {

constexpr int kTopkMaxK = 32;

template <typename T> __device__ __forceinline__ float logit_to_f32(T v);
template <> __device__ __forceinline__ float logit_to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float logit_to_f32<uint16_t>(uint16_t v) { return bf16_to_f32(v); }
template <> __device__ __forceinline__ float logit_to_f32<_Float16>(_Float16 v) { return (float)v; }

// (value, index) ordered by value descending, index ascending
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

template <typename T, typename IdT, int W, int VPL>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T *__restrict__ logits, int64_t n, int E, int k,
                                                           int renormalize, float *__restrict__ weights,
                                                           IdT *__restrict__ ids) {
    constexpr int kPerWave = kWave / W;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane % W;
    const int64_t token = ((int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave) * kPerWave + lane / W;
    const bool live = token < n;
    const T *row = logits + (live ? token : 0) * (int64_t)E;

    // this lane's logits: experts sub, sub + W, ...
    float v[VPL], pr[VPL];
    unsigned alive = 0;   // bit i: v[i] is an expert not yet taken
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int e = sub + i * W;
        v[i] = (e < E) ? logit_to_f32<T>(row[e]) : -INFINITY;
        if (e < E) alive |= 1u << i;
        m = fmaxf(m, v[i]);
    }
#pragma unroll
    for (int o = W / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, kWave));
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        pr[i] = ((alive >> i) & 1u) ? __expf(v[i] - m) : 0.f;   // unnormalised probability
        s += pr[i];
    }
#pragma unroll
    for (int o = W / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
    const float inv_s = 1.f / s;

    // k rounds of arg-max over the logits (exp is monotone: the order of the probabilities, without their rounding);
    // lane j of the group keeps winners j, j + W, ... for the coalesced store
    float wv[(kTopkMaxK + W - 1) / W];
    int wi[(kTopkMaxK + W - 1) / W];
    float chosen = 0.f;
    for (int j = 0; j < k; ++j) {
        float bv = -INFINITY, bp = 0.f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
            if (((alive >> i) & 1u) && better(v[i], sub + i * W, bv, bi)) { bv = v[i]; bi = sub + i * W; bp = pr[i]; }
#pragma unroll
        for (int o = W / 2; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, kWave);
            const float op = __shfl_xor(bp, o, kWave);
            const int oi = __shfl_xor(bi, o, kWave);
            if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; bp = op; }
        }
        bp *= inv_s;                                        // softmax value of the winner
        chosen += bp;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
            if (sub + i * W == bi) alive &= ~(1u << i);     // taken
#pragma unroll
        for (int q = 0; q < (kTopkMaxK + W - 1) / W; ++q)
            if (j == q * W + sub) { wv[q] = bp; wi[q] = bi; }
    }
    const float scale = renormalize ? 1.f / chosen : 1.f;
    if (!live) return;
#pragma unroll
    for (int q = 0; q < (kTopkMaxK + W - 1) / W; ++q) {
        const int j = q * W + sub;
        if (j < k) {
            weights[token * k + j] = wv[q] * scale;
            ids[token * k + j] = (IdT)wi[q];
        }
    }
}

template <typename T, typename IdT, int W, int VPL>
static int launch_topk(const void *logits, int64_t n, int E, int k, int renormalize, float *weights, void *ids,
                       hipStream_t stream) {
    constexpr int kPerBlock = 4 * (kWave / W);
    const int64_t blocks = (n + kPerBlock - 1) / kPerBlock;
    hipLaunchKernelGGL((topk_softmax_kernel<T, IdT, W, VPL>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const T *)logits, n, E, k, renormalize, weights, (IdT *)ids);
    DMOE_LAUNCH_CHECK("topk_softmax_kernel");
    return DMOE_OK;
}

template <typename T, typename IdT>
static int launch_topk_by_width(const void *logits, int64_t n, int E, int k, int renormalize, float *weights,
                                void *ids, hipStream_t stream) {
    // A round of the arg-max costs a lane VPL compares and log2(W) exchanges, and a token W lanes of that: narrow
    // groups do less work in all, wide groups have the shorter chain of dependent instructions.  Few tokens (every
    // wavefront of the wide form resident at once, two per SIMD at most) are latency-bound and take the wide form
    // (512 tokens x 64 experts: 8 against 10 us), many take the narrow one (8192 x 64: 13 against 20 us).
    const bool few = n * (E <= 8 ? 8 : E <= 16 ? 16 : E <= 32 ? 32 : 64) / kWave <= 2048;
    if (E <= 8) return launch_topk<T, IdT, 8, 1>(logits, n, E, k, renormalize, weights, ids, stream);
    if (few) {
        if (E <= 16) return launch_topk<T, IdT, 16, 1>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 32) return launch_topk<T, IdT, 32, 1>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 64) return launch_topk<T, IdT, 64, 1>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 256) return launch_topk<T, IdT, 64, 4>(logits, n, E, k, renormalize, weights, ids, stream);
    } else {
        if (E <= 16) return launch_topk<T, IdT, 8, 2>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 32) return launch_topk<T, IdT, 8, 4>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 64) return launch_topk<T, IdT, 8, 8>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 128) return launch_topk<T, IdT, 16, 8>(logits, n, E, k, renormalize, weights, ids, stream);
        if (E <= 256) return launch_topk<T, IdT, 16, 16>(logits, n, E, k, renormalize, weights, ids, stream);
    }
    return launch_topk<T, IdT, 64, 16>(logits, n, E, k, renormalize, weights, ids, stream);
}

template <typename T>
static int launch_topk_by_ids(const void *logits, int64_t n, int E, int k, int renormalize, float *weights, void *ids,
                              int ids_type, hipStream_t stream) {
    if (ids_type == DMOE_I32)
        return launch_topk_by_width<T, int32_t>(logits, n, E, k, renormalize, weights, ids, stream);
    return launch_topk_by_width<T, int64_t>(logits, n, E, k, renormalize, weights, ids, stream);
}

}  // namespace dmoe

using namespace dmoe;

extern "C" int dmoe_topk_softmax(const void *logits, int logits_dtype, int64_t n, int E, int k, int renormalize,
                                 float *weights, void *ids, int ids_type, void *stream) {
    DMOE_REQUIRE(n >= 0 && n < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_topk_softmax: n=%lld outside [0, 2^31)", (long long)n);
    DMOE_REQUIRE(E >= 1 && E <= 1024, DMOE_ERR_SHAPE, "dmoe_topk_softmax: E=%d outside [1, 1024]", E);
    DMOE_REQUIRE(k >= 1 && k <= E && k <= kTopkMaxK, DMOE_ERR_SHAPE, "dmoe_topk_softmax: k=%d outside [1, min(E, %d)]", k,
                 kTopkMaxK);
    DMOE_REQUIRE(ids_type == DMOE_I32 || ids_type == DMOE_I64, DMOE_ERR_DTYPE, "dmoe_topk_softmax: ids_type=%d", ids_type);
    DMOE_REQUIRE(logits_dtype == DMOE_BF16 || logits_dtype == DMOE_FP16 || logits_dtype == DMOE_FP32, DMOE_ERR_DTYPE,
                 "dmoe_topk_softmax: logits_dtype=%d", logits_dtype);
    if (n == 0) return DMOE_OK;
    DMOE_REQUIRE(logits != nullptr && weights != nullptr && ids != nullptr, DMOE_ERR_ARG, "dmoe_topk_softmax: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (logits_dtype == DMOE_FP32) return launch_topk_by_ids<float>(logits, n, E, k, renormalize, weights, ids, ids_type, s);
    if (logits_dtype == DMOE_BF16) return launch_topk_by_ids<uint16_t>(logits, n, E, k, renormalize, weights, ids, ids_type, s);
    return launch_topk_by_ids<_Float16>(logits, n, E, k, renormalize, weights, ids, ids_type, s);
}
