/*
 * ORACLE -- TEST INFRASTRUCTURE ONLY.  Never imported, linked or executed by
 * the product path (minference_amd/); only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may use it, and only as the checker.
 *
 * Scalar CPU restatement of MInference's vertical/slash index conversion:
 *   reference kernel   csrc/vertical_slash_index.cu:27-99  (per row block)
 *   reference flush    csrc/vertical_slash_index.cu:21-25  (save_blocks)
 *   reference launcher csrc/vertical_slash_index.cu:101-167 (grid, zero-filled outputs)
 *
 * One call of oracle_vs_index_row() does what one GPU thread of the reference
 * does for one (batch, head, row block).  The two places where the reference
 * reads out of bounds (the initial slash skip with no offset < end_m, :65-67;
 * nnz_v == 0, :63) return -1 here instead; everything the reference defines
 * is reproduced step for step, including the end_m+64 sentinel, the clamp of
 * the column end to 64 and the order in which entries are emitted.
 *
 * Parity pinning: hand-computed known-answer rows, a set-based specification
 * (ranges / columns closed form) and brute-force property checks in
 * tests/test_oracle_index.py.
 */
#include <stdint.h>
#include <string.h>

#define BLK 64

static int imax(int a, int b) { return a > b ? a : b; }

/* csrc/vertical_slash_index.cu:21-25 */
static void flush_range(int32_t *block_offset, int range_start, int range_end,
                        int *block_count) {
    for (int idx = range_start; idx < range_end; idx += BLK)
        block_offset[(*block_count)++] = idx;
}

/* csrc/vertical_slash_index.cu:46-98 for one row block.
 * vertical: ascending [nnz_v]; slash: descending [nnz_s].
 * Outputs for this row: block_offset[nnz_s], column_index[nnz_v], counts.
 * Returns 0, or -1 where the reference would read out of bounds. */
int oracle_vs_index_row(const int32_t *vertical, const int32_t *slash,
                        int nnz_v, int nnz_s, int block_idx_m, int seqlen,
                        int32_t *block_count, int32_t *block_offset,
                        int32_t *column_count, int32_t *column_index) {
    int start_m = block_idx_m * BLK;
    if (start_m >= seqlen) return 0;             /* :49-51 row left untouched */
    int end_m = start_m + BLK;
    if (nnz_v < 1 || nnz_s < 1) return -1;

    int tmp_col_cnt = 0, tmp_blk_cnt = 0;
    int s = 0, v = 0;
    int v_idx = vertical[v++];                   /* :63 */
    int s_idx = slash[s++];                      /* :64 */
    while (s_idx >= end_m) {                     /* :65-67 (bounded here) */
        if (s >= nnz_s) return -1;
        s_idx = slash[s++];
    }
    s_idx = imax(end_m - s_idx, BLK);            /* :68 */
    int range_start = s_idx - BLK, range_end = s_idx;   /* :69 */
    for (;;) {                                   /* :70-95 */
        if (v_idx < range_end) {
            if (v_idx < range_start) column_index[tmp_col_cnt++] = v_idx;
            if (v < nnz_v) v_idx = vertical[v++];
            else v_idx = end_m + BLK;            /* sentinel :78 */
        } else {
            if (s < nnz_s) {
                s_idx = imax(end_m - slash[s++], BLK);
            } else {
                flush_range(block_offset, range_start, range_end, &tmp_blk_cnt);
                break;
            }
            if (s_idx > range_end + BLK) {
                flush_range(block_offset, range_start, range_end, &tmp_blk_cnt);
                range_start = s_idx - BLK;
                range_end = s_idx;
            } else if (s_idx > range_end) {
                range_end += BLK;
            }
        }
    }
    *block_count = tmp_blk_cnt;                  /* :97 */
    *column_count = tmp_col_cnt;                 /* :98 */
    return 0;
}

/* csrc/vertical_slash_index.cu:101-167: all (batch, head, row) triples.
 * Outputs are zero-filled first, as the reference allocates them with
 * torch::zeros (:146-149).  64-bit row offsets (the reference's int offsets
 * overflow once B*H*rows*nnz_s >= 2^31).
 * Returns 0 or the number of rows that hit an out-of-bounds case (negated). */
int oracle_vs_index_build(const int32_t *seqlens, const int32_t *vertical,
                          const int32_t *slash, int32_t *block_count,
                          int32_t *block_offset, int32_t *column_count,
                          int32_t *column_index, int batch, int heads, int rows,
                          int nnz_v, int nnz_s) {
    int64_t nrow = (int64_t)batch * heads * rows;
    memset(block_count, 0, (size_t)nrow * sizeof(int32_t));
    memset(column_count, 0, (size_t)nrow * sizeof(int32_t));
    memset(block_offset, 0, (size_t)nrow * nnz_s * sizeof(int32_t));
    memset(column_index, 0, (size_t)nrow * nnz_v * sizeof(int32_t));
    int bad = 0;
    for (int b = 0; b < batch; b++)
        for (int h = 0; h < heads; h++) {
            const int32_t *vv = vertical + ((int64_t)b * heads + h) * nnz_v;
            const int32_t *ss = slash + ((int64_t)b * heads + h) * nnz_s;
            for (int m = 0; m < rows; m++) {
                int64_t ro = ((int64_t)b * heads + h) * rows + m;
                int rc = oracle_vs_index_row(vv, ss, nnz_v, nnz_s, m, seqlens[b],
                                             block_count + ro, block_offset + ro * nnz_s,
                                             column_count + ro, column_index + ro * nnz_v);
                if (rc) bad++;
            }
        }
    return -bad;
}
