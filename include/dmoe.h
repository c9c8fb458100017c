/*
 * dmoe.h -- C ABI of libdmoe_hip.so: the MI355X (gfx950) expert-worker hot path.
 *
 * Routing ids -> expert-sorted row mapping, token permute / gather, ragged
 * grouped GEMM (bf16 and fp8-e4m3, SiLU*mul fused for the gate-up projection)
 * and the gate-weighted combine back to token order.
 *
 * Conventions for every entry point
 *   - all data pointers are DEVICE pointers on the current HIP device unless a
 *     parameter says "host";
 *   - `stream` is a hipStream_t passed as void*; work is only enqueued, no entry
 *     point synchronises the device or allocates device memory;
 *   - the return value is DMOE_OK (0) or a negative DMOE_ERR_* code; nothing
 *     aborts the process (the reference's CUDACHECK prints and exits,
 *     csrc/include/cuda_utils.h:22-41, and its shape checks are C asserts,
 *     csrc/cuda_ops/permute.cu:70,91-98); dmoe_last_error() returns a
 *     thread-local message for the last failure;
 *   - tensors are row-major and contiguous (row stride == row length), as the
 *     reference requires (disagmoe/ops/memory.py:77).
 */
#ifndef DMOE_H_
#define DMOE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DMOE_OK 0
#define DMOE_ERR_ARG (-1)       /* null pointer, negative size, bad enum */
#define DMOE_ERR_SHAPE (-2)     /* shape constraint violated */
#define DMOE_ERR_DTYPE (-3)     /* unsupported element / index type */
#define DMOE_ERR_WORKSPACE (-4) /* scratch buffer missing or too small */
#define DMOE_ERR_HIP (-5)       /* a HIP runtime call failed */

/* element types of row data */
#define DMOE_BF16 0
#define DMOE_FP16 1
#define DMOE_FP8_E4M3 2 /* OCP e4m3fn, max 448 */
#define DMOE_FP32 3     /* router logits only */

/* integer types of ids / mappings: the size in bytes */
#define DMOE_I32 4
#define DMOE_I64 8

/* order of rows inside one expert's range (dmoe_route) */
#define DMOE_ORDER_REFERENCE 0 /* descending t: disagmoe/ops/memory.py:50-52 */
#define DMOE_ORDER_STABLE 1    /* ascending t: disagmoe/ops/memory.py:57-69 with a stable sort */

/* rounding schedule of dmoe_combine */
#define DMOE_COMBINE_FP32 0      /* fp32 accumulate, one rounding */
#define DMOE_COMBINE_REFERENCE 1 /* bf16(w)*y rounded, then left-to-right rounded adds:
                                    disagmoe/frontend/engine.py:726,732,627 */

const char *dmoe_version(void);
const char *dmoe_last_error(void);

/* Number of compute units of the current device (persistent-grid size). */
int dmoe_device_cus(int *cus);

/* ---- routing ------------------------------------------------------------
 * Replaces the host counting sort get_mappings_from_exp_ids
 * (disagmoe/ops/memory.py:34-54), its device variant (:57-69), the merge-side
 * sort Metadata::merge_by_exp_ids (csrc/include/datatypes.hpp:288-337) and the
 * histogram upload Metadata::get_expert_batch_sizes_cuda (:228-247).
 *
 *   ids          [R]   expert id of routed row t (token-major t = i*k + j)
 *   mappings     [R]   destination row of t in the expert-sorted buffer;
 *                      -1 for an id outside [0, E)
 *   batch_sizes  [E]   int64 rows per expert            (may be NULL)
 *   offsets      [E+1] int64 exclusive scan of the above (may be NULL)
 *   scratch            dmoe_route_scratch_bytes(R, E) bytes, contents ignored
 */
int dmoe_route_scratch_bytes(int64_t R, int E, size_t *bytes);
int dmoe_route(const void *ids, int ids_type, int64_t R, int E, int order,
               void *mappings, int map_type, int64_t *batch_sizes, int64_t *offsets,
               void *scratch, size_t scratch_bytes, void *stream);

/* dmoe_route that also writes the inverse of the mapping in tokens: row_token[mappings[t]] = t / top_k, int32 [R]
 * (ids with an expert outside [0, E) leave no entry).  For dmoe_gmm_swiglu_rows, which fetches the rows of the
 * [T, d] activations by their place in the expert-sorted order, so that the duplicating permute of
 * disagmoe/frontend/engine.py:671-680 (permute_tokens_cuda before the FFN) needs no launch of its own.
 * R % top_k == 0. */
int dmoe_route_sources(const void *ids, int ids_type, int64_t R, int E, int order,
                       void *mappings, int map_type, int64_t *batch_sizes, int64_t *offsets,
                       int top_k, int32_t *row_token, void *scratch, size_t scratch_bytes, void *stream);

/* dmoe_route for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in
 * the reference.  Same arguments and results as dmoe_route without the scratch
 * buffer: the per-chunk histograms live in a buffer built into the library, one copy
 * per device, dmoe_route_noalloc_max_bytes() bytes (4 MiB), held until the process
 * ends.  The call allocates nothing and frees nothing.  A problem whose
 * dmoe_route_scratch_bytes(R, E) exceeds that size is refused with
 * DMOE_ERR_WORKSPACE (4 MiB cover e.g. 8.3 M rows over 64 experts, 130 k rows over
 * 4096).  All calls on one device share the buffer: calls that overlap in time on
 * one device (two streams) race; calls on one stream do not. */
int dmoe_route_noalloc_max_bytes(size_t *bytes);
int dmoe_route_noalloc(const void *ids, int ids_type, int64_t R, int E, int order,
                       void *mappings, int map_type, int64_t *batch_sizes, int64_t *offsets,
                       void *stream);

/* ---- routing producer ---------------------------------------------------
 * dmoe_topk_softmax replaces vllm's fused_topk(hidden_states, gating_output,
 * topk, renormalize) as the attention side calls it
 * (disagmoe/models/attention.py:228-231): softmax over the E router logits of
 * a token in fp32, the k largest probabilities and their expert ids, and with
 * renormalize != 0 the k weights divided by their sum.  Ties go to the lower
 * expert id.  The ids feed dmoe_route without visiting the host.
 *
 *   logits   [n, E]  DMOE_FP32, DMOE_BF16 or DMOE_FP16, E <= 1024
 *   weights  [n, k]  fp32, descending
 *   ids      [n, k]  DMOE_I32 (what fused_topk returns) or DMOE_I64, k <= 32
 */
int dmoe_topk_softmax(const void *logits, int logits_dtype, int64_t n, int E, int k, int renormalize,
                      float *weights, void *ids, int ids_type, void *stream);

/* ---- per-row bookkeeping (host arrays, no device work) --------------------
 * The integer lists that travel with a batch on the expert worker: request
 * id, expert id, attention DP rank, initial prefill length per row.
 *
 * dmoe_sort_by_prefill_order replaces Metadata::sort_by_prefill_order
 * (csrc/include/datatypes.hpp:411-433): rows ranked by DP rank, then prefill
 * rows (init_prefill_len != -1) before decode rows, prefill rows by request
 * id; mapping[rank[i]] = i is the return permute of
 * disagmoe/frontend/engine.py:715,734.  The reference leaves rows that compare
 * equal to a non-stable sort; here they keep their order.
 *
 * dmoe_move_row_infos replaces Metadata::permute_token_infos (:377-409) for one
 * list: out[mapping[i]] = values[i], elements of 4 or 8 bytes, out != values.
 *
 * dmoe_expert_batch_sizes replaces Metadata::get_expert_batch_sizes and the
 * selection of the local experts in get_expert_batch_sizes_cuda (:228-247):
 * histogram of exp_ids over n_expert experts; with inner_exp_rank (m entries)
 * batches[i] = hist[inner_exp_rank[i]], without it batches[e] = hist[e].  Any
 * number of experts (the reference's stack buffer holds 8). */
int dmoe_sort_by_prefill_order(const int32_t *req_ids, const int32_t *attn_dp_ranks,
                               const int32_t *init_prefill_lens, int64_t n, int64_t *mapping);
int dmoe_move_row_infos(const void *values, int elem_bytes, const int64_t *mapping, int64_t n, void *out);
int dmoe_expert_batch_sizes(const int32_t *exp_ids, int64_t n, int n_expert, const int32_t *inner_exp_rank, int m,
                            int64_t *batches);
/* The counting sort of Metadata::merge_by_exp_ids (csrc/include/datatypes.hpp:303-324) and of
 * get_mappings_from_exp_ids (disagmoe/ops/memory.py:38-52) on host arrays: mappings[i] = destination row of
 * row i of the concatenated batches, experts ascending, inside an expert the first row that arrives takes the
 * last slot; exp_cnt[n_expert] (may be NULL) = rows per expert.  Any number of experts (the reference's table
 * holds 32).  dmoe_route is the device form of the same rule. */
int dmoe_host_mappings(const int32_t *exp_ids, int64_t n, int n_expert, int64_t *mappings, int64_t *exp_cnt);

/* Wire format of a batch's bookkeeping: the bytes the reference's workers exchange for a Metadata, a cereal
 * BinaryOutputArchive of its fields in the order of Metadata::serialize (csrc/include/datatypes.hpp:223-226, written
 * and read by cerealize / decerealize, csrc/include/utils.hpp:150-174), host byte order:
 *     u64 n, u64 shape[n] | u64 n, char dtype[n] | i32 layer_id | u64 n, i32 req_ids[n] | u64 n, i32 exp_ids[n] |
 *     u64 n, i32 attn_dp_ranks[n] | u64 n, i32 init_prefill_lens[n] | u64 n, f32 topk_weights[n]
 * dmoe_metadata_serialize writes the lists of a view (host pointers) into `out` (dmoe_metadata_wire_bytes bytes);
 * dmoe_metadata_parse checks a blob and reports where each list lies in it (byte offsets: the lists of a blob are
 * not aligned) and how many entries it has.  A blob that ends early or has bytes left over is DMOE_ERR_SHAPE. */
typedef struct dmoe_metadata_view {
    const uint64_t *shape; uint64_t n_shape;
    const char *dtype; uint64_t n_dtype;
    int32_t layer_id;
    const int32_t *req_ids; uint64_t n_req_ids;
    const int32_t *exp_ids; uint64_t n_exp_ids;
    const int32_t *attn_dp_ranks; uint64_t n_attn_dp_ranks;
    const int32_t *init_prefill_lens; uint64_t n_init_prefill_lens;
    const float *topk_weights; uint64_t n_topk_weights;
} dmoe_metadata_view;
typedef struct dmoe_metadata_layout {
    uint64_t off_shape, n_shape;
    uint64_t off_dtype, n_dtype;
    int32_t layer_id;
    uint64_t off_req_ids, n_req_ids;
    uint64_t off_exp_ids, n_exp_ids;
    uint64_t off_attn_dp_ranks, n_attn_dp_ranks;
    uint64_t off_init_prefill_lens, n_init_prefill_lens;
    uint64_t off_topk_weights, n_topk_weights;
} dmoe_metadata_layout;
int dmoe_metadata_wire_bytes(const dmoe_metadata_view *m, size_t *bytes);
int dmoe_metadata_serialize(const dmoe_metadata_view *m, void *out, size_t out_bytes);
int dmoe_metadata_parse(const void *blob, size_t blob_bytes, dmoe_metadata_layout *out);

/* ---- row movement -------------------------------------------------------
 * dmoe_permute replaces permute_tokens_cuda(tokens, mappings, stream)
 * (csrc/include/permute.h:8, csrc/cuda_ops/permute.cu:86-112, bound at
 * csrc/bindings.cpp:173) and the Triton permute (disagmoe/ops/memory.py:72-91):
 *     out[mappings[t], :] = in[t / k, :],  k = R / T,  R % T == 0.
 * Rows whose mapping is outside [0, R) are skipped.  The reference's
 * d % 2048 == 0 limit (permute.cu:70) is relaxed to row_bytes % 16 == 0.
 * `row_scale` (optional, [R], same element type as the rows, NULL for none)
 * multiplies row t before it is stored: the `output * topk_weights` step of
 * disagmoe/frontend/engine.py:731-732 fused into the return permute.
 */
int dmoe_permute(const void *in, void *out, const void *mappings, int map_type,
                 int64_t T, int64_t R, int64_t d, int dtype, const void *row_scale, void *stream);

/* out[t, :] = in[index[t], :] for t in [0, N); rows with an index outside
 * [0, n_src) are zero-filled.  Index form of gather_tokens_cuda
 * (csrc/include/permute.h:10, csrc/cuda_ops/permute.cu:144-152) and of the
 * torch.index_select permute (tests/dp/test_split.py:33). */
int dmoe_gather_rows(const void *in, void *out, const void *index, int idx_type,
                     int64_t N, int64_t n_src, int64_t d, int dtype, void *stream);

/* out[t, :] = *(row*)src_rows[t]: gather_tokens_cuda with the table of raw row
 * pointers ALREADY on the device (the reference uploads it and synchronises
 * per call, permute.cu:147,151).  NULL entries are zero-filled. */
int dmoe_gather_ptrs(const void *const *src_rows, void *out, int64_t N, int64_t d, int dtype,
                     void *stream);

/* Gate-weighted unpermute back to token order:
 *     out[i, :] = sum_j w[i, j] * y[mappings[i*k + j], :]
 * Replaces scale (engine.py:731-732) + return permute (:734) + top-k sum
 * (:624-628).  `weights` is fp32 [T, k].  Rows with a mapping outside [0, R)
 * contribute nothing. */
int dmoe_combine(const void *y, const void *mappings, int map_type, const float *weights,
                 void *out, int64_t T, int k, int64_t d, int dtype, int mode, void *stream);

/* ---- grouped GEMM -------------------------------------------------------
 * dmoe_gmm replaces grouped_gemm.backend.gmm(a, b, batch_sizes, trans_b, c)
 * (third-party; call sites disagmoe/models/experts.py:84,89,92,94 and
 * tests/ops/test_gemm.py:15):
 *     c[o_e:o_e+n_e, :] = a[o_e:o_e+n_e, :] @ (trans_b ? b[e]^T : b[e])
 *   a [rows, K]; b [E, K, N] (or [E, N, K] with trans_b); c [rows, N];
 *   batch_sizes int64 [E] on the DEVICE; rows past sum(batch_sizes) untouched,
 *   sizes are clamped so that no row >= `rows` is ever read or written.
 *   dtype DMOE_BF16: bf16 operands, fp32 accumulate, bf16 result.
 *   K % 8 == 0 and N % 8 == 0 (16-byte rows).
 *
 * dmoe_gmm_swiglu is the gate-up projection of MoEExperts.forward
 * (experts.py:92-93) with the activation fused:
 *     h[r, n] = silu(u[r, n]) * u[r, I + n],  u = a @ b[e],  b [E, K, 2I]
 *   (or [E, 2I, K] with trans_b), h [rows, I]; silu and the product are taken on
 *   the fp32 accumulators, one rounding.
 *
 * `state` and `workspace` replace what the reference obtains from get_arguments()
 * and hands to gmm_with_arguments() (experts.py:69-77): its arguments_ptr and its
 * workspace of workspace_size bytes.
 *   state      device memory of the caller, DMOE_GMM_STATE_BYTES bytes, 256-byte
 *              aligned, zero-filled once before its first use (every launch leaves
 *              it zero-filled again): the launch's work counters.
 *   workspace  device memory of the caller, 16-byte aligned, any contents.  When the
 *              tiles do not fill the compute units a whole number of times, the tiles
 *              of the last round are cut along K and their fp32 partial sums are added
 *              up here in a fixed order (results do not depend on timing).
 *              dmoe_gmm_workspace_bytes() is the size at which no launch is short
 *              of room for that; a smaller one (or NULL) cuts less (or nothing).
 * Launches that may overlap in time must not share a state block or a workspace.
 * state == NULL: counters of the library's own, one set per stream (at most 64
 * streams per device), nothing is cut; refused with DMOE_ERR_WORKSPACE while
 * `stream` is being captured into a graph, whose replays may run beside anything.
 *
 * host_batch_sizes (may be NULL): the caller's copy of batch_sizes in HOST memory,
 * read during the call only.  The reference keeps the sizes on the host wherever
 * it does not run its CUTLASS path (disagmoe/frontend/engine.py:377-380, 690-701:
 * get_expert_batch_sizes for the host, get_expert_batch_sizes_cuda for the device).
 * With them the library counts the tiles of every tile height instead of
 * estimating them from rows / E (tile height and grid of a skewed batch); the
 * kernels still read the sizes on the device, so values that disagree with
 * batch_sizes cost speed, never correctness.
 */
#define DMOE_GMM_STATE_BYTES 33024
int dmoe_gmm_workspace_bytes(int E, size_t *bytes);
int dmoe_gmm(const void *a, const void *b, void *c, const int64_t *batch_sizes,
             int64_t rows, int E, int64_t K, int64_t N, int trans_b, int dtype,
             void *state, void *workspace, size_t workspace_bytes,
             const int64_t *host_batch_sizes, void *stream);
int dmoe_gmm_swiglu(const void *a, const void *b, void *h, const int64_t *batch_sizes,
                    int64_t rows, int E, int64_t K, int64_t I, int trans_b, int dtype,
                    void *state, void *workspace, size_t workspace_bytes,
                    const int64_t *host_batch_sizes, void *stream);

/* dmoe_gmm_swiglu on rows that are fetched where they lie: row r of the product is row row_token[r] of x [T, K]
 * (dmoe_route_sources writes row_token).  The duplicating permute in front of the FFN
 * (disagmoe/frontend/engine.py:671-680, csrc/cuda_ops/permute.cu:86-112) and the gather of
 * TensorBatch::merge (csrc/include/datatypes.hpp:508-549) then need no launch and no copy of the rows.
 * Weights [E, K, 2I]; K % 32 == 0; T * K * 2 and K * 2I * 2 below 4 GiB.  Always runs on tiles of 256 rows:
 * for problems whose rows do not fill such tiles, dmoe_permute + dmoe_gmm_swiglu is the faster pair. */
int dmoe_gmm_swiglu_rows(const void *x, const int32_t *row_token, int64_t T, const void *b, void *h,
                         const int64_t *batch_sizes, int64_t rows, int E, int64_t K, int64_t I, int dtype,
                         void *state, void *workspace, size_t workspace_bytes,
                         const int64_t *host_batch_sizes, void *stream);

/* ---- fp8 (e4m3) path: no counterpart in the reference ---------------------
 * Per-row quantisation: q[r, :] = fp8(x[r, :] / s[r]), s[r] = absmax(x[r, :]) / 448
 * (s = 1 for a zero row).  x is bf16 [rows, d]. */
int dmoe_quant_rows(const void *x, void *q, float *scales, int64_t rows, int64_t d, int dtype,
                    void *stream);

/* dmoe_permute followed by dmoe_quant_rows in one pass: q[mappings[t], :] = fp8(in[t / k, :] / s),
 * scales[mappings[t]] = s = absmax(in[t / k, :]) / 448, k = R / T.  The token row is read once and stored k
 * times as e4m3; the bf16 copy of the routed rows never exists.  Same bits as the two calls. */
int dmoe_permute_quant(const void *in, void *q, float *scales, const void *mappings, int map_type, int64_t T,
                       int64_t R, int64_t d, int dtype, void *stream);

/* fp8 grouped GEMM, operands K-contiguous:
 *   a  fp8 [rows, K] with a_scale fp32 [rows]
 *   b  fp8 [E, N, K] with b_scale fp32 [E, N]     (per output channel)
 *   c  bf16 [rows, N] = (a @ b[e]^T) * a_scale[r] * b_scale[e, n]
 * K % 16 == 0.  The swiglu form takes b [E, 2I, K], b_scale [E, 2I] and writes
 * h bf16 [rows, I] as dmoe_gmm_swiglu does.  `state`, `workspace` and `host_batch_sizes` as for dmoe_gmm. */
int dmoe_gmm_fp8(const void *a, const float *a_scale, const void *b, const float *b_scale, void *c,
                 const int64_t *batch_sizes, int64_t rows, int E, int64_t K, int64_t N,
                 void *state, void *workspace, size_t workspace_bytes,
                 const int64_t *host_batch_sizes, void *stream);
int dmoe_gmm_fp8_swiglu(const void *a, const float *a_scale, const void *b, const float *b_scale,
                        void *h, const int64_t *batch_sizes, int64_t rows, int E, int64_t K,
                        int64_t I, void *state, void *workspace, size_t workspace_bytes,
                        const int64_t *host_batch_sizes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DMOE_H_ */
