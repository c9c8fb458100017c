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

// ---- wire format of a batch's bookkeeping -------------------------------------------------------------
// The reference sends Metadata between its workers as a cereal BinaryOutputArchive of the fields in the order of
// Metadata::serialize (csrc/include/datatypes.hpp:223-226; csrc/include/utils.hpp:150-174).  cereal (v1.3, a header
// library the reference builds against, not part of its tree) writes, in the byte order of the host: an arithmetic
// value as its bytes; a std::vector of arithmetic values and a std::string as the element count (cereal::size_type,
// 64 bits) followed by the elements' bytes; a struct with a serialize member as its fields one after the other.
// So a blob is   u64 n, u64 shape[n] | u64 n, char dtype[n] | i32 layer_id | u64 n, i32 req_ids[n] | u64 n, i32
// exp_ids[n] | u64 n, i32 attn_dp_ranks[n] | u64 n, i32 init_prefill_lens[n] | u64 n, f32 topk_weights[n].

namespace {

struct Field { const void *data; uint64_t count; size_t elem; };

void fields_of(const dmoe_metadata_view &m, Field (&f)[7]) {
    f[0] = {m.shape, m.n_shape, 8};
    f[1] = {m.dtype, m.n_dtype, 1};
    f[2] = {m.req_ids, m.n_req_ids, 4};
    f[3] = {m.exp_ids, m.n_exp_ids, 4};
    f[4] = {m.attn_dp_ranks, m.n_attn_dp_ranks, 4};
    f[5] = {m.init_prefill_lens, m.n_init_prefill_lens, 4};
    f[6] = {m.topk_weights, m.n_topk_weights, 4};
}

}  // namespace

extern "C" int dmoe_metadata_wire_bytes(const dmoe_metadata_view *m, size_t *bytes) {
    DMOE_REQUIRE(m && bytes, DMOE_ERR_ARG, "dmoe_metadata_wire_bytes: null pointer");
    Field f[7];
    fields_of(*m, f);
    size_t total = 4;   // layer_id
    for (const Field &x : f) {
        DMOE_REQUIRE(x.count < (1ull << 40), DMOE_ERR_SHAPE, "dmoe_metadata_wire_bytes: a list of %llu entries", (unsigned long long)x.count);
        DMOE_REQUIRE(x.count == 0 || x.data, DMOE_ERR_ARG, "dmoe_metadata_wire_bytes: null list with %llu entries", (unsigned long long)x.count);
        total += 8 + (size_t)x.count * x.elem;
    }
    *bytes = total;
    return DMOE_OK;
}

extern "C" int dmoe_metadata_serialize(const dmoe_metadata_view *m, void *out, size_t out_bytes) {
    size_t need = 0;
    int rc = dmoe_metadata_wire_bytes(m, &need);
    if (rc != DMOE_OK) return rc;
    DMOE_REQUIRE(out && out_bytes >= need, DMOE_ERR_WORKSPACE, "dmoe_metadata_serialize: %zu bytes needed, %zu given", need, out_bytes);
    Field f[7];
    fields_of(*m, f);
    char *p = (char *)out;
    auto put_list = [&](const Field &x) {
        std::memcpy(p, &x.count, 8); p += 8;
        if (x.count) std::memcpy(p, x.data, (size_t)x.count * x.elem);
        p += (size_t)x.count * x.elem;
    };
    put_list(f[0]);
    put_list(f[1]);
    std::memcpy(p, &m->layer_id, 4); p += 4;
    for (int i = 2; i < 7; ++i) put_list(f[i]);
    return DMOE_OK;
}

extern "C" int dmoe_metadata_parse(const void *blob, size_t blob_bytes, dmoe_metadata_layout *out) {
    DMOE_REQUIRE(blob && out, DMOE_ERR_ARG, "dmoe_metadata_parse: null pointer");
    const char *base = (const char *)blob;
    size_t pos = 0;
    bool ok = true;
    auto take_list = [&](size_t elem, uint64_t *offset, uint64_t *count) {
        if (!ok || blob_bytes - pos < 8) { ok = false; return; }
        uint64_t n;
        std::memcpy(&n, base + pos, 8);
        pos += 8;
        if (n > (blob_bytes - pos) / elem) { ok = false; return; }
        *offset = pos; *count = n;
        pos += (size_t)n * elem;
    };
    take_list(8, &out->off_shape, &out->n_shape);
    take_list(1, &out->off_dtype, &out->n_dtype);
    if (ok && blob_bytes - pos >= 4) { std::memcpy(&out->layer_id, base + pos, 4); pos += 4; } else ok = false;
    take_list(4, &out->off_req_ids, &out->n_req_ids);
    take_list(4, &out->off_exp_ids, &out->n_exp_ids);
    take_list(4, &out->off_attn_dp_ranks, &out->n_attn_dp_ranks);
    take_list(4, &out->off_init_prefill_lens, &out->n_init_prefill_lens);
    take_list(4, &out->off_topk_weights, &out->n_topk_weights);
    DMOE_REQUIRE(ok, DMOE_ERR_SHAPE, "dmoe_metadata_parse: the blob of %zu bytes ends inside a field (at byte %zu)", blob_bytes, pos);
    DMOE_REQUIRE(pos == blob_bytes, DMOE_ERR_SHAPE, "dmoe_metadata_parse: %zu bytes behind the last field", blob_bytes - pos);
    return DMOE_OK;
}
