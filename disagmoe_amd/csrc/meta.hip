// Per-row bookkeeping of the expert worker: the integer lists that travel with a batch (request id, expert id,
// attention DP rank, initial prefill length, top-k weight per row).  Host code like the lists themselves; what it
// produces for the device is a row mapping that dmoe_permute / dmoe_combine take.
#include "common.h"

#include <algorithm>
#include <cstring>
#include <numeric>
#include <vector>

using namespace dmoe;

extern "C" int dmoe_sort_by_prefill_order(const int32_t *req_ids, const int32_t *attn_dp_ranks,
                                          const int32_t *init_prefill_lens, int64_t n, int64_t *mapping) {
    DMOE_REQUIRE(n >= 0 && n < (1ll << 31), DMOE_ERR_SHAPE, "dmoe_sort_by_prefill_order: n=%lld outside [0, 2^31)", (long long)n);
    if (n == 0) return DMOE_OK;
    DMOE_REQUIRE(req_ids && attn_dp_ranks && init_prefill_lens && mapping, DMOE_ERR_ARG, "dmoe_sort_by_prefill_order: null pointer");
    std::vector<int32_t> rank((size_t)n);
    std::iota(rank.begin(), rank.end(), 0);
    // DP rank ascending; inside a rank prefill rows (length != -1) before decode rows; prefill rows by request id.
    // Rows that compare equal (decode rows of one rank, prefill rows of one request) keep their order.
    std::stable_sort(rank.begin(), rank.end(), [&](int32_t i, int32_t j) {
        if (attn_dp_ranks[i] != attn_dp_ranks[j]) return attn_dp_ranks[i] < attn_dp_ranks[j];
        if (init_prefill_lens[i] == -1 || init_prefill_lens[j] == -1) return init_prefill_lens[i] > init_prefill_lens[j];
        return req_ids[i] < req_ids[j];
    });
    for (int64_t i = 0; i < n; ++i) mapping[rank[(size_t)i]] = i;
    return DMOE_OK;
}

extern "C" int dmoe_move_row_infos(const void *values, int elem_bytes, const int64_t *mapping, int64_t n, void *out) {
    DMOE_REQUIRE(n >= 0, DMOE_ERR_SHAPE, "dmoe_move_row_infos: n=%lld", (long long)n);
    DMOE_REQUIRE(elem_bytes == 4 || elem_bytes == 8, DMOE_ERR_DTYPE, "dmoe_move_row_infos: elem_bytes=%d", elem_bytes);
    if (n == 0) return DMOE_OK;
    DMOE_REQUIRE(values && mapping && out && values != out, DMOE_ERR_ARG, "dmoe_move_row_infos: null or aliased pointer");
    for (int64_t i = 0; i < n; ++i) {
        const int64_t j = mapping[i];
        DMOE_REQUIRE(j >= 0 && j < n, DMOE_ERR_ARG, "dmoe_move_row_infos: mapping[%lld]=%lld outside [0, %lld)", (long long)i,
                     (long long)j, (long long)n);
        std::memcpy((char *)out + j * elem_bytes, (const char *)values + i * elem_bytes, (size_t)elem_bytes);
    }
    return DMOE_OK;
}

extern "C" int dmoe_expert_batch_sizes(const int32_t *exp_ids, int64_t n, int n_expert, const int32_t *inner_exp_rank,
                                       int m, int64_t *batches) {
    DMOE_REQUIRE(n >= 0 && n_expert > 0, DMOE_ERR_SHAPE, "dmoe_expert_batch_sizes: n=%lld n_expert=%d", (long long)n, n_expert);
    DMOE_REQUIRE(batches && (n == 0 || exp_ids), DMOE_ERR_ARG, "dmoe_expert_batch_sizes: null pointer");
    std::vector<int64_t> hist((size_t)n_expert, 0);
    for (int64_t i = 0; i < n; ++i) {
        DMOE_REQUIRE(exp_ids[i] >= 0 && exp_ids[i] < n_expert, DMOE_ERR_ARG, "dmoe_expert_batch_sizes: exp_ids[%lld]=%d outside [0, %d)",
                     (long long)i, exp_ids[i], n_expert);
        hist[(size_t)exp_ids[i]] += 1;
    }
    if (inner_exp_rank == nullptr) {
        for (int e = 0; e < n_expert; ++e) batches[e] = hist[(size_t)e];
        return DMOE_OK;
    }
    for (int i = 0; i < m; ++i) {
        DMOE_REQUIRE(inner_exp_rank[i] >= 0 && inner_exp_rank[i] < n_expert, DMOE_ERR_ARG,
                     "dmoe_expert_batch_sizes: inner_exp_rank[%d]=%d outside [0, %d)", i, inner_exp_rank[i], n_expert);
        batches[i] = hist[(size_t)inner_exp_rank[i]];
    }
    return DMOE_OK;
}

extern "C" int dmoe_host_mappings(const int32_t *exp_ids, int64_t n, int n_expert, int64_t *mappings, int64_t *exp_cnt) {
    DMOE_REQUIRE(n >= 0 && n_expert > 0, DMOE_ERR_SHAPE, "dmoe_host_mappings: n=%lld n_expert=%d", (long long)n, n_expert);
    DMOE_REQUIRE(n == 0 || (exp_ids && mappings), DMOE_ERR_ARG, "dmoe_host_mappings: null pointer");
    std::vector<int64_t> cursor((size_t)n_expert, 0);
    for (int64_t i = 0; i < n; ++i) {
        DMOE_REQUIRE(exp_ids[i] >= 0 && exp_ids[i] < n_expert, DMOE_ERR_ARG, "dmoe_host_mappings: exp_ids[%lld]=%d outside [0, %d)",
                     (long long)i, exp_ids[i], n_expert);
        cursor[(size_t)exp_ids[i]] += 1;
    }
    if (exp_cnt)
        for (int e = 0; e < n_expert; ++e) exp_cnt[e] = cursor[(size_t)e];
    for (int e = 1; e < n_expert; ++e) cursor[(size_t)e] += cursor[(size_t)e - 1];   // end of every expert's rows
    // rows of an expert are handed out from its last slot backwards, in the order the rows arrive
    for (int64_t i = 0; i < n; ++i) mappings[i] = --cursor[(size_t)exp_ids[i]];
    return DMOE_OK;
}
