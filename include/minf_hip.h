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
 *     report;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     work is only enqueued, never synchronised;
 *   - tensors are described by a base pointer plus ELEMENT strides; the last
 *     (head_dim) stride must be 1 and rows must be 16-byte aligned;
 *   - dtype: MINF_BF16 or MINF_F16 for q/k/v/o.
 */
#ifndef MINF_HIP_H
#define MINF_HIP_H
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

/* Library version as major*10000 + minor*100 + patch. */
int minf_version(void);

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

#ifdef __cplusplus
}
#endif
#endif /* MINF_HIP_H */
