/*
 * libminf_hip.so -- C ABI of the MI355X (gfx950) dynamic sparse prefill
 * attention path.  Drop-in boundary for microsoft/MInference's native
 * extension and Triton operators; see each entry point for the reference
 * interface it replaces.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise;
 *   - every function returns an int status: MINF_OK (0) or a negative code
 *     (minf_status_string() gives text); nothing throws, nothing keeps a
 *     "last error";
 *   - no entry point allocates or frees device memory: the caller owns every
 *     buffer, including workspaces whose size the *_workspace_bytes() helpers
 *     report (minf_vs_index_build_static brings its own fixed-size scratch);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     work is only enqueued, never synchronised;
 *   - tensors are described by a base pointer plus ELEMENT strides; the last
 *     (head_dim) stride must be 1 and rows must be 16-byte aligned;
 *   - dtype: MINF_BF16 or MINF_F16 for q/k/v/o.
 */
#ifndef MINF_HIP_H
#define MINF_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MINF_OK 0
#define MINF_ERR_INVALID_ARG (-1)   /* null pointer, negative size, ... */
#define MINF_ERR_UNSUPPORTED (-2)   /* head_dim / block size / dtype not built */
#define MINF_ERR_ALIGNMENT (-3)     /* pointer or stride breaks the 16-byte rule */
#define MINF_ERR_WORKSPACE (-4)     /* workspace too small */
#define MINF_ERR_HIP_BASE (-1000)   /* -1000 - hipError_t of a failed launch */

#define MINF_BF16 0
#define MINF_F16 1

/* Rounding of the two index selectors (pattern estimation, block index).  MINF_ROUND_NONE: fp32
 * arithmetic on the 16-bit inputs.  MINF_ROUND_INPUT_DTYPE: round every intermediate that the
 * reference's torch code holds in the input dtype (bf16/fp16) to that dtype, so that the selected
 * index sets follow the reference's arithmetic and not a more precise one. */
#define MINF_ROUND_NONE 0
#define MINF_ROUND_INPUT_DTYPE 1

/* Library version as major*10000 + minor*100 + patch. */
int minf_version(void);

/* sizeof(minf_qkvo) as this library was compiled.  A caller built against another revision of this
 * header passes a struct of another size and must not call the attention entry points: compare with
 * its own sizeof(minf_qkvo) once at start-up. */
size_t minf_qkvo_size(void);

/* Static text for a status code (pure function, thread-safe). */
const char *minf_status_string(int status);

/*
 * Vertical/slash index conversion.
 * Replaces minference.cuda.convert_vertical_slash_indexes
 *   (reference csrc/kernels.cpp:7-18, csrc/vertical_slash_index.cu:27-167).
 *
 *   seqlens        [batch]                 int32
 *   vertical_idx   [batch, heads, nnz_v]   int32, ascending key positions
 *   slash_idx      [batch, heads, nnz_s]   int32, descending diagonal offsets
 *   block_count    [batch, heads, rows]
 *   block_offset   [batch, heads, rows, nnz_s]
 *   column_count   [batch, heads, rows]
 *   column_index   [batch, heads, rows, nnz_v]      rows = ceil(context/64)
 *
 * Bit-exact with the reference wherever the reference is defined.  With
 * zero_fill != 0 every output element is written (payload, then zeros), which
 * reproduces the reference's torch::zeros allocation (:146-149) in one pass;
 * with zero_fill == 0 only counts and payload are written.  Where the
 * reference reads out of bounds (a row block with no slash offset below its
 * end, :65-67) the row gets zero counts and, if `error_flag` is not NULL,
 * *error_flag is set to 1 (the caller clears it beforehand).
 * Row offsets are 64-bit (the reference's int arithmetic overflows at 2^31
 * elements, :55-59).  Block sizes are fixed at 64x64 like the reference (:135-136).
 */
int minf_vs_index_build(const int32_t *seqlens, const int32_t *vertical_idx,
                        const int32_t *slash_idx, int32_t *block_count,
                        int32_t *block_offset, int32_t *column_count,
                        int32_t *column_index, int batch, int heads, int rows,
                        int nnz_v, int nnz_s, int zero_fill, int32_t *error_flag,
                        void *stream);

/*
 * Same result as minf_vs_index_build, faster: a per-head pass first tabulates the part of the
 * reference's range merge that does not depend on the row block (ranges and blocks of a slash
 * list only move with the row block once no entry is skipped or clipped), then every row block
 * copies its blocks from the table and tests its verticals against a per-head coverage bitmap of
 * the tabulated ranges.
 * workspace: minf_vs_index_workspace_bytes(batch, heads, nnz_s, rows) bytes of device memory,
 * 4-byte aligned, overwritten.  Same reference lines, same bit-exactness and error behaviour.
 */
size_t minf_vs_index_workspace_bytes(int batch, int heads, int nnz_s, int rows);
int minf_vs_index_build_ws(const int32_t *seqlens, const int32_t *vertical_idx,
                           const int32_t *slash_idx, int32_t *block_count,
                           int32_t *block_offset, int32_t *column_count,
                           int32_t *column_index, int batch, int heads, int rows,
                           int nnz_v, int nnz_s, int zero_fill, int32_t *error_flag,
                           void *workspace, size_t workspace_bytes, void *stream);

/*
 * minf_vs_index_build_ws without a workspace argument and without any allocation: the tables and
 * bitmaps live in a device array of MINF_VS_INDEX_STATIC_BYTES that is part of the library image
 * (every GPU the library runs on holds its own copy until the process ends).  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same outputs, bit for
 * bit, as minf_vs_index_build_ws.  Problems whose minf_vs_index_workspace_bytes() exceeds
 * MINF_VS_INDEX_STATIC_BYTES return MINF_ERR_WORKSPACE before anything is enqueued (8 MiB holds
 * 32 heads x 6096 slashes x 524288 tokens).  All calls on one GPU share the one array: calls that
 * overlap in time on the same GPU (different streams or threads) race and must be serialised by
 * the caller.  The device address of the array is looked up once per device, on the first call
 * made with that device current (hipGetDevice + hipGetSymbolAddress): that FIRST call on a device
 * must therefore be made outside stream capture (one warm-up call before capturing is enough; every
 * later call on that device only enqueues kernels).  The array is chosen by the CURRENT device, not
 * by `stream`: the caller must have made the stream's device current, as for any HIP launch.
 */
#define MINF_VS_INDEX_STATIC_BYTES (8u << 20)
int minf_vs_index_build_static(const int32_t *seqlens, const int32_t *vertical_idx,
                               const int32_t *slash_idx, int32_t *block_count,
                               int32_t *block_offset, int32_t *column_count,
                               int32_t *column_index, int batch, int heads, int rows,
                               int nnz_v, int nnz_s, int zero_fill, int32_t *error_flag,
                               void *stream);

/*
 * Sparse flash-attention forward on one shared 64x64 bf16/f16 MFMA tile
 * engine.  Common arguments of the four entry points below:
 *
 *   q [batch, heads_q, n, head_dim], k/v [batch, heads_kv, n, head_dim],
 *   o [batch, heads_q, n, head_dim]: base pointers + element strides
 *   {batch, head, token} (head_dim stride is 1); heads_q % heads_kv == 0 and
 *   query head h reads kv head h / (heads_q / heads_kv) (no repeat_kv copy is
 *   needed; the reference always expands K/V first,
 *   minference/modules/forward.py:128-132).  head_dim must be 64 or 128 (the
 *   reference's kernels accept 16/32/64/128, pit_sparse_flash_attention_v2.py:172;
 *   smaller head dims are zero-padded to 64 by the caller); the A-shape, tri-shape and dense
 *   entry points also take 256, as the reference's streaming kernel does
 *   (minference/ops/streaming_kernel.py:429).
 *   seqlens [batch] int32 may be NULL (= n for every batch).  Rows >= seqlen
 *   are written as zeros (the reference leaves its zeros_like buffer untouched).
 *   sm_scale multiplies q.k before the softmax (reference: head_dim^-0.5).
 *   Every o element of every row < n (of every selected head) is written; nothing else is.
 *   Token strides must be at least head_dim (rows must not overlap).
 */
typedef struct minf_qkvo {
    const void *q, *k, *v;
    void *o;
    int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];   /* batch, head, token */
    int batch, heads_q, heads_kv, n, head_dim, dtype;
    const int32_t *seqlens;
    float sm_scale;
    /* Optional head selection (per-head pattern tables: reference
     * minference/modules/minference_forward.py:621, :657-667 loops over heads and calls one operator
     * per head).  head_list NULL: every query head is processed and index tensors have heads_q
     * heads.  Otherwise head_list is a device array of index_heads distinct query head numbers
     * (ascending order keeps heads that share a kv head together): only these heads are processed
     * (the o rows of all other heads are not touched) and head_list[i] reads its index rows at head
     * position i of index tensors that have index_heads heads.  q, k, v, o are always addressed
     * with the real head number, so a launch per pattern type writes its heads of one shared
     * output in place. */
    const int32_t *head_list;
    int index_heads;
} minf_qkvo;

/*
 * Mixed block-sparse + column-sparse forward over the tensors produced by
 * minf_vs_index_build.  Replaces _triton_mixed_sparse_attention /
 * _triton_mixed_sparse_attn_fwd_kernel
 *   (reference minference/ops/pit_sparse_flash_attention_v2.py:48-192).
 * Row r of row block m attends {c in [off, off+64) for the first
 * block_count[m] offsets : c <= r, c < seqlen} plus the first column_count[m]
 * entries of column_index (no causal test on those, as in the reference).
 * Index tensors are indexed by QUERY head: [batch, heads_q, rows, nnz_*].
 */
int minf_vs_attn_fwd(const minf_qkvo *t, const int32_t *block_count,
                     const int32_t *block_offset, const int32_t *column_count,
                     const int32_t *column_index, int rows, int nnz_s, int nnz_v,
                     void *stream);

/*
 * Block-sparse forward.  Replaces _triton_block_sparse_attention
 *   (reference minference/ops/block_sparse_flash_attention.py:29-148).
 * block_index [batch, heads_q, rows, max_blocks] int32, each row ascending;
 * rows >= ceil(n/64) (the reference builds it on a padded sequence);
 * row block m visits its first min(m+1, max_blocks) entries, element-wise
 * causal (reference :81-96).
 */
int minf_bs_attn_fwd(const minf_qkvo *t, const int32_t *block_index, int rows,
                     int max_blocks, void *stream);

/*
 * A-shape (attention sink + sliding window) forward in one pass.  Replaces
 * streaming_forward's two-stage TritonMultiStageDotProductionAttention
 *   (reference minference/ops/streaming_kernel.py:26-239, 611-646).
 * Row r attends {c : r - n_local < c <= r} plus {c < n_init : c <= r - n_local}.
 */
int minf_ashape_attn_fwd(const minf_qkvo *t, int n_init, int n_local, void *stream);

/*
 * Tri-shape: A-shape for the first n - n_last query rows, dense causal attention for the last
 * n_last rows, in one launch of the same kernel.  Replaces tri_shape_kernel (reference
 * minference/ops/streaming_kernel.py:820-833 and minference/modules/minference_forward.py:444-455),
 * which runs the A-shape op on the truncated sequence, a dense einsum/softmax for the last rows
 * and a torch.cat.  The caller clamps n_last to n - 1 like the reference.
 * sm_scale_last scales q.k of the last n_last rows (0 = t->sm_scale): the reference scales those by
 * head_dim^-0.5 (:826) but the A-shape rows by the power-of-two PADDED head_dim^-0.5 (:575 after
 * :793-797), which differ when head_dim is not a power of two.
 */
int minf_trishape_attn_fwd(const minf_qkvo *t, int n_init, int n_local, int n_last,
                           float sm_scale_last, void *stream);

/*
 * Dense causal forward on the same tile engine (the in-house comparator for
 * the sparse-vs-dense speed-up; the reference uses flash_attn_func,
 * minference/modules/minference_forward.py:666).
 */
int minf_dense_attn_fwd(const minf_qkvo *t, void *stream);

/*
 * Online vertical/slash pattern estimation.  Replaces the torch op chain of
 * vertical_and_slash_kernel (reference
 * minference/modules/minference_forward.py:599-610) and sum_all_diagonal_matrix
 * (:110-116), batched over heads:
 *   P = softmax(q[:, :, -last_q:] . k^T * sm_scale) with the trailing
 *   last_q x last_q corner causally masked (fp32);
 *   vertical[b,h,c] = sum_i P[i,c];  slash[b,h,j] = sum_i P[i, i+j+1-last_q]
 *   (slash[j] is the mass on the diagonal with offset n-1-j);
 *   then vertical[..., :force_vertical] = +inf and slash[..., n-force_slash:] = +inf
 *   (the reference forces 30 and 100; pass 0 to get the raw sums).
 * rounding = MINF_ROUND_INPUT_DTYPE reproduces the reference's rounding points on bf16/fp16 tensors
 * (:602: the einsum result is a tensor of the input dtype, and so is its quotient by sqrt(head_dim);
 * the softmax then runs in fp32, :604): score = round(round(q.k) * sm_scale), both to `dtype`.
 * MINF_ROUND_NONE keeps fp32 (what the reference computes on fp32 tensors).
 * q [batch, heads_q, n, head_dim], k [batch, heads_kv, n, head_dim] (head_dim 64 or 128) as base
 * pointer + element strides {batch, head, token}; last_q <= 64 (clamped to n).
 * vertical, slash: [batch, heads_q, n] fp32, contiguous.
 * workspace: at least minf_vs_estimate_workspace_bytes() bytes, 16-byte aligned.
 */
size_t minf_vs_estimate_workspace_bytes(int batch, int heads_q, int n);
int minf_vs_estimate(const void *q, const void *k, const int64_t *q_stride,
                     const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                     int head_dim, int dtype, float sm_scale, int last_q, int force_vertical,
                     int force_slash, int rounding, float *vertical, float *slash, void *workspace,
                     size_t workspace_bytes, void *stream);

/*
 * minf_vs_estimate for a subset of the query heads (per-head pattern tables: the reference estimates
 * inside its loop over heads, minference/modules/minference_forward.py:657-667, only for the heads
 * whose pattern is vertical_and_slash).  head_list [index_heads] int32 (device): the query heads to
 * score; the scores of head_list[i] are row i of vertical / slash [batch, index_heads, n]; q and k
 * are addressed with the real head numbers.  Workspace:
 * minf_vs_estimate_workspace_bytes(batch, index_heads, n).
 */
int minf_vs_estimate_heads(const void *q, const void *k, const int64_t *q_stride,
                           const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                           int head_dim, int dtype, float sm_scale, int last_q, int force_vertical,
                           int force_slash, int rounding, const int32_t *head_list, int index_heads,
                           float *vertical, float *slash, void *workspace,
                           size_t workspace_bytes, void *stream);

/*
 * Indices of the k largest entries of each fp32 row, written in ASCENDING
 * INDEX order (ties at the k-th value: lowest index first).  Replaces
 * torch.topk(...).indices followed by the sort in the op wrapper (reference
 * minference/modules/minference_forward.py:607,612 and
 * minference/ops/pit_sparse_flash_attention_v2.py:218-219).
 * scores [rows, n] with row_stride elements between rows; out [rows, min(k,n)]
 * with out_stride.  reverse_base < 0: out = index; otherwise out =
 * reverse_base - index (slash: reverse_base = n-1 turns ascending j into
 * descending diagonal offsets, the order the index builder wants).
 * Values are ordered by their bit patterns: -0.0 ranks below +0.0 and denormals are told apart
 * (the scores of this path are sums of probabilities or matrix products, which hold no -0.0);
 * NaN has no defined rank.
 */
int minf_topk_indices(const float *scores, int rows, int n, int64_t row_stride, int k,
                      int32_t *out, int64_t out_stride, int reverse_base, void *stream);

/*
 * minf_topk_indices for block-causal score rows of at most 4096 entries (the block scores of
 * block-sparse attention, reference minference/ops/block_sparse_flash_attention.py:161-166):
 * row r belongs to query block m = r % rows_per_head, entries above the diagonal are -inf by
 * construction and only the first 32 * (m / 32 + 1) entries of a row need to be stored; the rest
 * is never read and counts as -inf.  Same selection and order as minf_topk_indices on the fully
 * stored rows.  n > 4096 returns MINF_ERR_UNSUPPORTED.
 */
int minf_topk_indices_block_causal(const float *scores, int rows, int n, int64_t row_stride, int k,
                                   int32_t *out, int64_t out_stride, int rows_per_head, void *stream);

/*
 * Two selections of minf_topk_indices in one launch (same rows / n / row_stride; separate k,
 * output and reverse_base): the vertical and the slash top-k of a layer
 * (reference minference/modules/minference_forward.py:607 and :612).
 */
int minf_topk_indices_pair(const float *scores_a, int k_a, int32_t *out_a, int64_t out_stride_a,
                           int reverse_base_a, const float *scores_b, int k_b, int32_t *out_b,
                           int64_t out_stride_b, int reverse_base_b, int rows, int n,
                           int64_t row_stride, void *stream);

/*
 * minf_topk_indices_pair with a different k for every row (the per-head vertical_size / slash_size
 * of a pattern table, reference minference_forward.py:621-625): row i keeps k_rows[i] entries
 * (device int32 [rows], clamped to 1..k_max) and the remaining k_max - k_rows[i] output slots are
 * padding.  pad_mode 0: left unwritten; 1: the constant pad_value; 2: the last selected value
 * repeated.  For the index builder both paddings are no-ops of the reference's merge loop
 * (csrc/vertical_slash_index.cu:70-95): a vertical index at or beyond every range end is never
 * emitted (pad verticals with a large constant), and a repeated slash offset neither starts nor
 * extends a range (pad slashes with mode 2), so one index build and one attention launch with the
 * list widths k_max serve heads with different sizes and produce, per head, the tensors of its own
 * sizes (followed by zeros).
 */
int minf_topk_indices_pair_ragged(const float *scores_a, const int32_t *k_rows_a, int k_max_a, int32_t *out_a,
                                  int64_t out_stride_a, int reverse_base_a, int pad_mode_a, int pad_value_a,
                                  const float *scores_b, const int32_t *k_rows_b, int k_max_b, int32_t *out_b,
                                  int64_t out_stride_b, int reverse_base_b, int pad_mode_b, int pad_value_b,
                                  int rows, int n, int64_t row_stride, void *stream);

/*
 * Block index of top-k block-sparse attention: replaces _build_block_index (reference
 * minference/ops/block_sparse_flash_attention.py:151-166) together with the zero padding its
 * caller applies first (:178-180).  Q and K are mean-pooled over 64-token blocks (the token axis
 * padded with 64 - n%64 zero rows, i.e. a whole extra block when n%64 == 0), every (query block,
 * key block) pair is scored with the pooled vectors, key blocks above the diagonal get -inf, and
 * the min(top_k, rows) best key blocks of every query block are written in ascending order (ties:
 * lowest block id first; torch.topk leaves the tie order unspecified).
 * flags: bit 0 (MINF_BS_FORCE_DIAG_FIRST) additionally keeps the diagonal block and block 0 of every
 * query block; bit 1 (MINF_BS_ROUND_INPUT_DTYPE) rounds the pooled means and the pooled dot
 * products to `dtype`, as the reference's torch code does on bf16/fp16 tensors (:159-163: `mean`
 * and `einsum` return tensors of the input dtype); without it the arithmetic is fp32 throughout.
 *   rows = minf_bs_block_index_rows(n) = (n + 64 - n%64) / 64
 *   block_index [batch, heads_q, rows, min(top_k, rows)] int32, contiguous
 *   q [batch, heads_q, n, head_dim], k [batch, heads_kv, n, head_dim] (head_dim 64 or 128): base
 *   pointer + element strides
 *   workspace: minf_bs_block_index_workspace_bytes() bytes, 16-byte aligned
 */
#define MINF_BS_FORCE_DIAG_FIRST 1
#define MINF_BS_ROUND_INPUT_DTYPE 2
int minf_bs_block_index_rows(int n);
size_t minf_bs_block_index_workspace_bytes(int batch, int heads_q, int heads_kv, int n);
int minf_bs_block_index(const void *q, const void *k, const int64_t *q_stride,
                        const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                        int head_dim, int dtype, int top_k, int flags,
                        int32_t *block_index, void *workspace, size_t workspace_bytes,
                        void *stream);

/*
 * minf_bs_block_index for a subset of the query heads (head_list as in minf_vs_estimate_heads):
 * block_index [batch, index_heads, rows, min(top_k, rows)]; workspace
 * minf_bs_block_index_workspace_bytes(batch, index_heads, heads_kv, n).
 */
int minf_bs_block_index_heads(const void *q, const void *k, const int64_t *q_stride,
                              const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                              int head_dim, int dtype, int top_k, int flags,
                              const int32_t *head_list, int index_heads,
                              int32_t *block_index, void *workspace, size_t workspace_bytes,
                              void *stream);

/*
 * Offline pattern search: the share of the exact causal softmax mass that candidate sparse
 * patterns keep, averaged over the query rows >= row_begin.  Replaces the scoring part of
 * search_pattern (reference minference/modules/minference_forward.py:129-227: the stream_llm,
 * vertical_and_slash and block_sparse closures build N x N masks and multiply them into the
 * N x N softmax, :156-161, :166-172, :187-194); here nothing of size N x N is materialised.
 * Up to 8 candidates are scored in one sweep: bit t of every flag byte belongs to candidate t.
 * Element (r, c), c <= r, counts for candidate t iff bit t is set in col_flags[c], in
 * diag_flags[r - c] or in block_flags[r / 32][c / 32].
 *   col_flags, diag_flags [batch*heads_q, flag_pitch] uint8, 4-byte aligned,
 *       flag_pitch % 4 == 0 and flag_pitch >= n rounded up to 64 (padding bytes zero)
 *   block_flags [batch*heads_q, ceil(n/32), block_pitch] uint8 or NULL, block_pitch >= ceil(n/32)
 *   recall [batch*heads_q, 8] fp32: mean over rows r in [row_begin, n) of
 *       sum_{c in candidate} softmax(q.k^T * sm_scale)[r, c]; NaN when n <= row_begin
 *       (the reference's mean of an empty slice); bits nobody set give 0
 *   workspace: minf_pattern_recall_workspace_bytes() bytes, 4-byte aligned
 * Deterministic (fixed summation order).  fp32 softmax on 16-bit q, k (the reference rounds the
 * probabilities to the input dtype before summing them).
 */
size_t minf_pattern_recall_workspace_bytes(int batch, int heads_q, int n);
int minf_pattern_recall(const void *q, const void *k, const int64_t *q_stride,
                        const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                        int head_dim, int dtype, float sm_scale, const uint8_t *col_flags,
                        const uint8_t *diag_flags, int64_t flag_pitch, const uint8_t *block_flags,
                        int64_t block_pitch, int row_begin, float *recall, void *workspace,
                        size_t workspace_bytes, void *stream);

/*
 * Builders of the flag arrays above (reference: the scatter of top-k indices into an N x N mask
 * and the spdiags construction, minference_forward.py:141-155, :166-168, :186-189).
 * minf_flags_set_indices ORs bit `bit` into flags[row, idx[row, i]] for i < k (entries outside
 * [0, limit) are ignored); minf_flags_set_range ORs it into flags[row, begin..end) of every row.
 * flags [rows, flag_pitch] uint8, 4-byte aligned, flag_pitch % 4 == 0; idx [rows, k] int32 with
 * idx_stride elements between rows.
 */
int minf_flags_set_indices(const int32_t *idx, int rows, int k, int64_t idx_stride, int bit,
                           uint8_t *flags, int64_t flag_pitch, int limit, void *stream);
int minf_flags_set_range(int begin, int end, int rows, int bit, uint8_t *flags, int64_t flag_pitch,
                         void *stream);

/*
 * Block index of the block_sparse candidate of the pattern search (reference
 * minference_forward.py:175-186): like minf_bs_block_index with 32-token blocks,
 * rows = ceil(n/32) (zero padding only up to the next multiple of 32) and no forced blocks.
 *   block_index [batch, heads_q, rows, min(top_k, rows)] int32
 */
size_t minf_search_block_index_workspace_bytes(int batch, int heads_q, int heads_kv, int n);
int minf_search_block_index(const void *q, const void *k, const int64_t *q_stride,
                            const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                            int head_dim, int dtype, int top_k, int32_t *block_index,
                            void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MINF_HIP_H */
