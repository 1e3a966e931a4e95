// Vertical/slash index conversion for gfx950: one 64-lane wavefront per
// (batch, head, 64-row block).  Produces the same four tensors as the
// reference's one-thread-per-row kernel (csrc/vertical_slash_index.cu:27-99),
// bit for bit, but walks the slash list 64 entries at a time:
//
//   * each valid slash offset o maps to a column end t = max(end_m - o, 64)
//     (ascending in list order);
//   * inside one merged range starting at `a`, the running range end after
//     consuming t is the closed form  e(t) = a + 64*ceil((t - a)/64), so all
//     64 lanes evaluate it at once; a new range starts exactly where
//     t > e(previous t) + 64, found with a ballot, and lanes past the break
//     switch to the new start.  A block [e-64, e) is emitted wherever e
//     changes, at a position given by a wave prefix count;
//   * a vertical index x lands in the output iff, with i the first slash
//     entry whose t exceeds x,  x < a_i  and  x >= e_{i-1}  (it lies in the
//     gap before entry i's range); verticals at or past the last t are never
//     emitted.  Verticals are consumed 64 at a time against the current
//     chunk's (t, a, e) triples kept in LDS.
//
// Writes: payload by prefix-compacted 4-byte stores, zero tails by 16-byte
// stores; all row offsets are 64-bit.
#include "minf_common.h"
#include <limits.h>

#define IDX_WAVES 4

__device__ __forceinline__ void zero_range(int32_t *p, int from, int to, int lane) {
    int n = to - from;
    if (n <= 0) return;
    int32_t *q = p + from;
    int head = (int)(((16u - (unsigned)((uintptr_t)q & 15u)) & 15u) >> 2);
    if (head > n) head = n;
    if (lane < head) q[lane] = 0;
    q += head;
    n -= head;
    int n4 = n >> 2;
    int4 z = make_int4(0, 0, 0, 0);
    for (int i = lane; i < n4; i += MINF_WAVE) reinterpret_cast<int4 *>(q)[i] = z;
    int tail = n & 3;
    if (lane < tail) q[n4 * 4 + lane] = 0;
}

__global__ __launch_bounds__(IDX_WAVES *MINF_WAVE) void vs_index_kernel(
    const int32_t *__restrict__ seqlens, const int32_t *__restrict__ vertical,
    const int32_t *__restrict__ slash, int32_t *__restrict__ block_count,
    int32_t *__restrict__ block_offset, int32_t *__restrict__ column_count,
    int32_t *__restrict__ column_index, int heads, int rows, int nnz_v, int nnz_s,
    int zero_fill, int32_t *error_flag, long long total_rows) {
    __shared__ int lds_t[IDX_WAVES][MINF_WAVE];
    __shared__ int lds_a[IDX_WAVES][MINF_WAVE];
    __shared__ int lds_e[IDX_WAVES][MINF_WAVE];

    const int lane = minf_lane();
    const int wave = (int)(threadIdx.x >> 6);
    const long long ro = (long long)blockIdx.x * IDX_WAVES + wave;   // (b*H + h)*rows + m
    if (ro >= total_rows) return;
    const int m = (int)(ro % rows);
    const long long bh = ro / rows;
    const int b = (int)(bh / heads);

    int32_t *bo_row = block_offset + ro * (long long)nnz_s;
    int32_t *ci_row = column_index + ro * (long long)nnz_v;
    const int32_t *vert = vertical + bh * (long long)nnz_v;
    const int32_t *sl = slash + bh * (long long)nnz_s;

    const int seqlen = seqlens[b];
    const int start_m = m * 64;
    const int end_m = start_m + 64;

    int nb = 0, ncol = 0;
    bool live = start_m < seqlen;

    // first list position whose offset is below end_m (list is descending)
    int s0 = nnz_s;
    if (live) {
        int lo = 0, hi = nnz_s;
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if (sl[mid] >= end_m) lo = mid + 1; else hi = mid;
        }
        s0 = lo;
        if (s0 >= nnz_s) {           // the reference would read past the list here
            live = false;
            if (error_flag && lane == 0) *error_flag = 1;
        }
    }

    if (live) {
        const int n = nnz_s - s0;
        const int nchunks = (n + MINF_WAVE - 1) / MINF_WAVE;
        int vp = 0;
        int carried_e = 0, carried_t = 0, cur_a = 0;
        int ep0 = INT_MIN;           // e of the entry before the chunk's first
        for (int c = 0; c < nchunks; ++c) {
            const int base = s0 + c * MINF_WAVE;
            const int cnt = min(MINF_WAVE, nnz_s - base);
            const bool valid = lane < cnt;
            int t = valid ? max(end_m - sl[base + lane], 64) : 0;
            const int tlast = minf_readlane(t, cnt - 1);
            if (!valid) t = tlast;   // padding lanes repeat the last entry (no-ops)
            if (c == 0) {
                const int t0 = minf_readlane(t, 0);
                cur_a = t0 - 64;
                carried_e = t0 - 64;
                carried_t = t0;
            }
            int a = cur_a;
            int tprev = __shfl_up(t, 1);
            if (lane == 0) tprev = carried_t;
            int start = 0;
            for (;;) {
                int eprev = a + ((((tprev - a) + 63) >> 6) << 6);
                if (lane == 0) eprev = carried_e;
                const bool brk = (lane >= start) && (t > eprev + 64);
                const uint64_t bm = __ballot(brk);
                if (bm == 0) break;
                const int j = __builtin_ctzll(bm);
                const int tj = minf_readlane(t, j);
                if (lane >= j) a = tj - 64;
                start = j + 1;
            }
            const int e = a + ((((t - a) + 63) >> 6) << 6);
            int eprev = __shfl_up(e, 1);
            if (lane == 0) eprev = carried_e;
            const bool changed = valid && (e != eprev);
            const uint64_t cm = __ballot(changed);
            if (changed) bo_row[nb + __builtin_popcountll(cm & minf_lanemask_lt())] = e - 64;
            nb += __builtin_popcountll(cm);

            // verticals below this chunk's last t
            if (vp < nnz_v && vert[vp] < tlast) {
                lds_t[wave][lane] = t;
                lds_a[wave][lane] = a;
                lds_e[wave][lane] = e;
                __builtin_amdgcn_wave_barrier();
                while (vp < nnz_v) {
                    const int x = (vp + lane < nnz_v) ? vert[vp + lane] : INT_MAX;
                    const bool ok = x < tlast;
                    const uint64_t okm = __ballot(ok);
                    const int k = __builtin_popcountll(okm);
                    bool emit = false;
                    if (ok) {
                        int lo = 0, hi = MINF_WAVE - 1;      // first i with t[i] > x (exists)
                        while (lo < hi) {
                            int mid = (lo + hi) >> 1;
                            if (lds_t[wave][mid] > x) hi = mid; else lo = mid + 1;
                        }
                        const int ai = lds_a[wave][lo];
                        const int ep = lo == 0 ? ep0 : lds_e[wave][lo - 1];
                        emit = (x < ai) && (x >= ep);
                    }
                    const uint64_t em = __ballot(emit);
                    if (emit) ci_row[ncol + __builtin_popcountll(em & minf_lanemask_lt())] = x;
                    ncol += __builtin_popcountll(em);
                    vp += k;
                    if (k < MINF_WAVE) break;
                }
                __builtin_amdgcn_wave_barrier();
            }
            carried_e = minf_readlane(e, cnt - 1);
            carried_t = tlast;
            cur_a = minf_readlane(a, cnt - 1);
            ep0 = carried_e;
        }
    }

    if (zero_fill || live) {
        if (lane == 0) {
            block_count[ro] = nb;
            column_count[ro] = ncol;
        }
    }
    if (zero_fill) {
        zero_range(bo_row, nb, nnz_s, lane);
        zero_range(ci_row, ncol, nnz_v, lane);
    }
}

extern "C" int minf_vs_index_build(const int32_t *seqlens, const int32_t *vertical_idx,
                                   const int32_t *slash_idx, int32_t *block_count,
                                   int32_t *block_offset, int32_t *column_count,
                                   int32_t *column_index, int batch, int heads, int rows,
                                   int nnz_v, int nnz_s, int zero_fill, int32_t *error_flag,
                                   void *stream) {
    if (!seqlens || !vertical_idx || !slash_idx || !block_count || !block_offset ||
        !column_count || !column_index)
        return MINF_ERR_INVALID_ARG;
    if (batch < 0 || heads < 0 || rows < 0 || nnz_v < 1 || nnz_s < 1) return MINF_ERR_INVALID_ARG;
    const long long total = (long long)batch * heads * rows;
    if (total == 0) return MINF_OK;
    const long long nblk = (total + IDX_WAVES - 1) / IDX_WAVES;
    if (nblk > 0x7fffffffLL) return MINF_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(vs_index_kernel, dim3((unsigned)nblk), dim3(IDX_WAVES * MINF_WAVE), 0,
                       (hipStream_t)stream, seqlens, vertical_idx, slash_idx, block_count,
                       block_offset, column_count, column_index, heads, rows, nnz_v, nnz_s,
                       zero_fill, error_flag, total);
    return minf_launch_status();
}
