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
#include <atomic>

#define IDX_WAVES 4

// value of the lane below (lane 0 gets 0): one data-parallel-primitive move, where the general
// shuffle goes through the LDS crossbar -- the table pass is one wave walking a chain of chunks and
// pays every cycle of it
__device__ __forceinline__ int lane_above(int x) {
    return __builtin_amdgcn_update_dpp(0, x, 0x138 /* wave_shr:1 */, 0xf, 0xf, true);
}

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

// dst[i] = src[i] + shift for i < n with 16-byte stores: dst is brought to a 16-byte boundary with
// single stores first (src then sits at any 4-byte phase; its 16-byte loads need no alignment)
__device__ __forceinline__ void copy_shifted(int32_t *dst, const int32_t *src, int n, int shift, int lane) {
    if (n <= 0) return;
    int head = (int)(((16u - (unsigned)((uintptr_t)dst & 15u)) & 15u) >> 2);
    if (head > n) head = n;
    if (lane < head) dst[lane] = src[lane] + shift;
    dst += head;
    src += head;
    n -= head;
    const int n4 = n >> 2;
    for (int i = lane; i < n4; i += MINF_WAVE) {
        int4 v;
        __builtin_memcpy(&v, src + 4 * i, 16);
        v.x += shift; v.y += shift; v.z += shift; v.w += shift;
        reinterpret_cast<int4 *>(dst)[i] = v;
    }
    const int tail = n & 3;
    if (lane < tail) dst[n4 * 4 + lane] = src[n4 * 4 + lane] + shift;
}

// Range starts of one chunk of 64 entries.  `t` ascends along the lanes (padding lanes repeat the
// last entry); the state carried in from the previous chunk is the current range start `cur_a`,
// the running range end `carried_e` and the previous entry `carried_t`.  Entry i starts a new
// range iff t_i > e_{i-1} + 64, and t_{i-1} <= e_{i-1} < t_{i-1} + 64, so
//   t_i >  t_{i-1} + 127  is always a start,      (decided for all lanes with one ballot)
//   t_i <= t_{i-1} + 64   never is,
// and only the lanes in between depend on the 64-phase of their range; those are resolved one by
// one in lane order with scalar arithmetic.  Returns this lane's range start; `starts` gets the
// mask of lanes that start a range.
__device__ __forceinline__ int chunk_ranges(int t, int lane, int cur_a, int carried_e, int carried_t,
                                            uint64_t &starts, uint64_t *gaps = nullptr) {
    int tprev = lane_above(t);
    if (lane == 0) tprev = carried_t;
    const bool sure = lane == 0 ? (t > carried_e + 64) : (t > tprev + 127);
    const bool maybe = lane != 0 && !sure && (t > tprev + 64);
    uint64_t sm = __ballot(sure);
    uint64_t mm = __ballot(maybe);
    // entries more than 64 above their predecessor (lane 0: above the last entry of the previous chunk)
    if (gaps) *gaps = ((sm | mm) & ~1ull) | (minf_readlane(t, 0) > carried_t + 64 ? 1ull : 0ull);
    const uint64_t le = minf_lanemask_lt() | (1ull << lane);
    const uint64_t below = sm & le;
    const int j0 = below ? 63 - __builtin_clzll(below) : 0;
    const int tj0 = sm ? __shfl(t, j0) : 0;        // (wave-uniform: no shuffle for a chunk without sure starts)
    int a = below ? tj0 - 64 : cur_a;
    while (mm) {
        const int j = __builtin_ctzll(mm);
        mm &= mm - 1;
        const int ap = minf_readlane(a, j - 1), tp = minf_readlane(t, j - 1), tj = minf_readlane(t, j);
        const int ep = ap + ((((tp - ap) + 63) >> 6) << 6);
        if (tj > ep + 64) {
            const uint64_t later = sm & ~((2ull << j) - 1ull);          // sure starts above lane j
            const int next = later ? __builtin_ctzll(later) : 64;
            if (lane >= j && lane < next) a = tj - 64;
            sm |= 1ull << j;
        }
    }
    starts = sm;
    return a;
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
            uint64_t starts;
            const int a = chunk_ranges(t, lane, cur_a, carried_e, carried_t, starts);
            const int e = a + ((((t - a) + 63) >> 6) << 6);
            int eprev = lane_above(e);
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

// ---------------------------------------------------------------------------------------------
// Translation-invariant fast path.
//
// For an entry that is neither skipped (o >= end_m) nor clipped (end_m - o < 64), t = end_m - o,
// so the whole range logic depends on the row block only through a shift: once a range STARTS at
// list entry g, everything the reference does from g on (ranges, blocks) is the same for every row
// block, moved by end_m.  vs_index_prep_kernel therefore walks each head's slash list ONCE, as a
// virtual row whose end is V = slash[0] + 64 (nothing skipped, nothing clipped), and tabulates
//   cpos[k]   start of the k-th block,                     k < nblocks
//   cpre[i]   index of the first block of the range that starts at entry i, else -1
//   crun[i]   ordinal of that range, else -1
//   run_a[r], run_e[r]   [start, end) of range r
//   cgaps[i]  the number of entries j <= i with t_j > t_{j-1} + 64 ("gap entries": the only entries
//             at which a range can start, for any row block -- skipping and clipping only shrink gaps)
//   glist[j]  the gap entries, ascending, j < ngaps (compacted from cgaps by the bitmap pass): the
//             first gap entry at or after entry x is glist[cgaps[x - 1]]
// all in the virtual row's coordinates (real position = virtual + end_m - V).
// vs_index_fast_kernel then handles a row block as follows: entries from the first valid one are
// processed exactly like vs_index_kernel until a range starts at an entry that also starts a range
// of the table (at once when no entry is skipped or clipped; after a few entries otherwise: chains
// that start at different entries meet at the first gap both see); from there the remaining blocks
// are copied from cpos with a shift (coalesced), and each remaining vertical x is emitted iff it is
// not inside one of the remaining tabulated ranges, is not below the end of the last range of the
// explicit part, and is below the last entry's t - the reference's merge rule restated per element.
// Inside the explicit part, a chunk of 64 entries without any gap above 64 means a dense run of
// diagonals: the entries up to the next entry of glist cannot start a range, so they only extend
// the current one, to a + 64 ceil((t_last - a) / 64), and their blocks are an arithmetic progression
// written at once -- lists whose slashes cluster (the usual case near the diagonal) would otherwise
// walk thousands of entries, 64 at a time, before they meet a tabulated range start.
#define IDX_TAB_HDR 8
// per head: header, seven tables of nnz_s ints, then a coverage bitmap of the virtual row (one bit
// per key position, set inside the tabulated ranges) of bm_words 32-bit words
__host__ __device__ __forceinline__ long long idx_bm_words(int rows) { return ((long long)rows * 64 + 64 + 31) / 32 + 1; }
__host__ __device__ __forceinline__ long long idx_tab_ints(int nnz_s, int rows) {
    return IDX_TAB_HDR + 7ll * nnz_s + idx_bm_words(rows);
}

// The walk of chunks [c_begin, c_end) of one head's list by one wavefront, starting from the state
// (cur_a, carried_e, carried_t) that the entries before chunk c_begin leave behind and from the
// counts (nb, nr, ng) of blocks, ranges and gap entries before it.  WRITE = false only counts.
struct PrepState { int cur_a, carried_e, carried_t; };
template <bool WRITE>
__device__ __forceinline__ void prep_walk(const int32_t *__restrict__ sl, int32_t *__restrict__ hdr, int nnz_s, int V,
                                          int c_begin, int c_end, PrepState &st, int &nb, int &nr, int &ng) {
    const int lane = minf_lane();
    int32_t *cpos = hdr + IDX_TAB_HDR, *cpre = cpos + nnz_s, *crun = cpre + nnz_s;
    int32_t *run_a = crun + nnz_s, *run_e = run_a + nnz_s, *cgaps = run_e + nnz_s;
    int carried_e = st.carried_e, carried_t = st.carried_t, cur_a = st.cur_a;
    // the walk is one chain of chunks; the list entries of the next two chunks are fetched ahead so
    // that no chunk waits for a load
    int o_next = sl[min(c_begin * MINF_WAVE + lane, nnz_s - 1)], o_next2 = sl[min((c_begin + 1) * MINF_WAVE + lane, nnz_s - 1)];
    for (int c = c_begin; c < c_end; ++c) {
        const int base = c * MINF_WAVE;
        const int cnt = min(MINF_WAVE, nnz_s - base);
        const bool valid = lane < cnt;
        const int o_cur = o_next;
        o_next = o_next2;
        o_next2 = sl[min(base + 2 * MINF_WAVE + lane, nnz_s - 1)];
        int t = valid ? max(V - o_cur, 64) : 0;
        const int tlast = minf_readlane(t, cnt - 1);
        if (!valid) t = tlast;
        if (c == 0) {
            const int t0 = minf_readlane(t, 0);
            cur_a = t0 - 64;
            carried_e = t0 - 64;
            carried_t = t0;
        }
        uint64_t starts, gm;
        const int a = chunk_ranges(t, lane, cur_a, carried_e, carried_t, starts, &gm);
        if (WRITE && valid) cgaps[base + lane] = ng + __builtin_popcountll(gm & (minf_lanemask_lt() | (1ull << lane)));
        ng += __builtin_popcountll(gm);             // (padding lanes repeat the last entry: never a gap)
        const bool is_start = valid && (((starts >> lane) & 1ull) || (c == 0 && lane == 0));
        const int e = a + ((((t - a) + 63) >> 6) << 6);
        int eprev = lane_above(e);
        if (lane == 0) eprev = carried_e;
        const bool changed = valid && (e != eprev);
        const uint64_t cm = __ballot(changed), sm = __ballot(is_start);
        if (WRITE) {
            const uint64_t lt = minf_lanemask_lt();
            const int kpos = nb + __builtin_popcountll(cm & lt);
            if (changed) cpos[kpos] = e - 64;
            if (valid) {
                const int r = nr + __builtin_popcountll(sm & lt);
                cpre[base + lane] = is_start ? kpos : -1;
                crun[base + lane] = is_start ? r : -1;
                if (is_start) {
                    run_a[r] = a;
                    if (r > 0) run_e[r - 1] = eprev;
                }
            }
        }
        nb += __builtin_popcountll(cm);
        nr += __builtin_popcountll(sm);
        carried_e = minf_readlane(e, cnt - 1);
        carried_t = tlast;
        cur_a = minf_readlane(a, cnt - 1);
    }
    st.cur_a = cur_a; st.carried_e = carried_e; st.carried_t = carried_t;
}

__device__ __forceinline__ void prep_header(int32_t *hdr, int nnz_s, int rows, int V, const PrepState &st, int nb, int nr, int ng) {
    int32_t *run_e = hdr + IDX_TAB_HDR + 4ll * nnz_s;
    run_e[nr - 1] = st.carried_e;
    hdr[0] = nb;
    hdr[1] = nr;
    hdr[2] = V;
    // the bitmap covers positions [0, 32 * bm_words); a list whose largest offset lies far
    // outside the context does not fit and the row blocks fall back to searching the ranges
    hdr[3] = (long long)V <= 32 * (idx_bm_words(rows) - 1) ? 1 : 0;
    hdr[4] = ng;
}

// The table pass: one workgroup of PREP_WAVES wavefronts per head.  The walk over the list is a chain
// (which range an entry belongs to depends on where the ranges before it started), but an entry more
// than 127 above its predecessor starts a range whatever came before ("sure" start) and only entries
// 65..127 above their predecessor ("maybe") depend on the 64-phase of the current range.  So every
// wavefront takes a contiguous share of the chunks; all of them first mark the sure and maybe entries
// of their chunks (independent work); a wavefront then finds the state at the head of its share by
// going back to the last sure start before it and replaying only the maybe entries in between (none
// inside a dense run, a handful when the offsets are scattered); it walks its share once to count its
// blocks, ranges and gap entries, the counts are summed over the wavefronts before it, and it walks
// the share again to write the tables.  Lists of at most two chunks, or of more chunks than the mark
// arrays hold, are walked by one wavefront alone.
#define PREP_WAVES 16
#define PREP_MAX_CHUNKS 2048
__global__ __launch_bounds__(PREP_WAVES *MINF_WAVE) void vs_index_prep_kernel(const int32_t *__restrict__ slash,
                                                                              int32_t *__restrict__ tables, int nnz_s, int rows) {
    __shared__ uint64_t sure_m[PREP_MAX_CHUNKS], maybe_m[PREP_MAX_CHUNKS];
    __shared__ int cnt_b[PREP_WAVES], cnt_r[PREP_WAVES], cnt_g[PREP_WAVES];
    const int lane = minf_lane();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const long long bh = blockIdx.x;
    const int32_t *sl = slash + bh * (long long)nnz_s;
    int32_t *hdr = tables + bh * idx_tab_ints(nnz_s, rows);
    const int V = sl[0] + 64;
    const int nchunks = (nnz_s + MINF_WAVE - 1) / MINF_WAVE;

    if (nchunks <= 2 || nchunks > PREP_MAX_CHUNKS) {        // (workgroup-uniform)
        if (wave == 0) {
            PrepState st{0, 0, 0};
            int nb = 0, nr = 0, ng = 0;
            prep_walk<true>(sl, hdr, nnz_s, V, 0, nchunks, st, nb, nr, ng);
            if (lane == 0) prep_header(hdr, nnz_s, rows, V, st, nb, nr, ng);
        }
        return;
    }
    const int per = (nchunks + PREP_WAVES - 1) / PREP_WAVES;
    const int c0 = wave * per, c1 = min(c0 + per, nchunks);
    // ---- marks: entry i is a sure start when t_i > t_{i-1} + 127, a maybe when t_i > t_{i-1} + 64
    // (entry 0 starts the first range)
    for (int c = c0; c < c1; ++c) {
        const int i = c * MINF_WAVE + lane;
        const bool valid = i < nnz_s;
        const int t = max(V - sl[min(i, nnz_s - 1)], 64);
        const int tp = max(V - sl[min(max(i - 1, 0), nnz_s - 1)], 64);
        const bool sure = valid && (i == 0 || t > tp + 127);
        const bool maybe = valid && !sure && t > tp + 64;
        const uint64_t sm = __ballot(sure), mm = __ballot(maybe);
        if (lane == 0) { sure_m[c] = sm; maybe_m[c] = mm; }
    }
    __syncthreads();
    // ---- the state at the head of this wavefront's share (wave-uniform scalar work)
    PrepState st{0, 0, 0};
    if (c0 > 0 && c0 < nchunks) {
        int cs = c0 - 1;
        while (cs > 0 && sure_m[cs] == 0) --cs;              // (chunk 0 holds entry 0, a sure start)
        const uint64_t smask = sure_m[cs];
        const int js = cs * MINF_WAVE + (63 - __builtin_clzll(smask));     // the last sure start before the share
        int a = max(V - sl[js], 64) - 64;
        for (int c = cs; c < c0; ++c) {
            uint64_t mm = maybe_m[c];
            if (c == cs) mm &= ~((2ull << (js - cs * MINF_WAVE)) - 1ull);    // maybes above the sure start only
            while (mm) {
                const int j = c * MINF_WAVE + __builtin_ctzll(mm);
                mm &= mm - 1;
                const int tj = max(V - sl[j], 64), tp = max(V - sl[j - 1], 64);
                const int ep = a + ((((tp - a) + 63) >> 6) << 6);
                if (tj > ep + 64) a = tj - 64;
            }
        }
        st.cur_a = a;
        st.carried_t = max(V - sl[c0 * MINF_WAVE - 1], 64);
        st.carried_e = a + ((((st.carried_t - a) + 63) >> 6) << 6);
    }
    // ---- count, sum over the wavefronts before this one, write
    int nb = 0, nr = 0, ng = 0;
    if (c0 < nchunks) {
        PrepState probe = st;
        prep_walk<false>(sl, hdr, nnz_s, V, c0, c1, probe, nb, nr, ng);
    }
    if (lane == 0) { cnt_b[wave] = nb; cnt_r[wave] = nr; cnt_g[wave] = ng; }
    __syncthreads();
    int ob = 0, orr = 0, og = 0, tb = 0, tr = 0, tg = 0;
#pragma unroll
    for (int w = 0; w < PREP_WAVES; ++w) {
        const int b = cnt_b[w], r = cnt_r[w], g = cnt_g[w];
        if (w < wave) { ob += b; orr += r; og += g; }
        tb += b; tr += r; tg += g;
    }
    if (c0 < nchunks) {
        nb = ob; nr = orr; ng = og;
        prep_walk<true>(sl, hdr, nnz_s, V, c0, c1, st, nb, nr, ng);
        if (c1 == nchunks && lane == 0) prep_header(hdr, nnz_s, rows, V, st, tb, tr, tg);
    }
}

// Coverage bitmap of a head's virtual row: bit p of the bitmap is set iff position p lies inside one
// of the tabulated ranges [run_a[r], run_e[r]).  One thread per 32-bit word: a binary search finds
// the first range that ends after the word's first position; ranges are at least 64 long, so at
// most two of them touch a word.
__global__ __launch_bounds__(256) void vs_index_bitmap_kernel(int32_t *__restrict__ tables, int nnz_s, int rows) {
    const long long bh = blockIdx.y;
    int32_t *hdr = tables + bh * idx_tab_ints(nnz_s, rows);
    const int32_t *run_a = hdr + IDX_TAB_HDR + 3ll * nnz_s, *run_e = run_a + nnz_s;
    uint32_t *bm = reinterpret_cast<uint32_t *>(hdr + IDX_TAB_HDR + 7ll * nnz_s);
    const long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (w < nnz_s) {                           // (thread w also serves list entry w: the gap list)
        const int32_t *cgaps = hdr + IDX_TAB_HDR + 5ll * nnz_s;
        int32_t *glist = hdr + IDX_TAB_HDR + 6ll * nnz_s;
        const int c = cgaps[w], cprev = w ? cgaps[w - 1] : 0;
        if (c != cprev) glist[c - 1] = (int)w;
    }
    if (w >= idx_bm_words(rows) || !hdr[3]) return;
    const int nr = hdr[1];
    const long long p0 = 32 * w, p1 = p0 + 32;
    int lo = 0, hi = nr;                       // first range with run_e > p0
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (run_e[mid] > p0) hi = mid; else lo = mid + 1;
    }
    uint32_t bits = 0;
    for (int r = lo; r < nr; ++r) {
        const long long a = run_a[r], e = run_e[r];
        if (a >= p1) break;
        const int from = (int)(max(a, p0) - p0), to = (int)(min(e, p1) - p0);      // [from, to) inside the word
        if (to > from) bits |= (to - from >= 32 ? 0xffffffffu : ((1u << (to - from)) - 1u)) << from;
    }
    bm[w] = bits;
}

// (Two instantiations: the zero-filled form is bound by its stores and measures 3 % faster at 512K
// tokens when the compiler is held to 64 registers; the payload-only form is bound by its chains of
// dependent loads and loses more to the few spills that limit costs than it gains.)
template <bool ZERO_FILL>
__global__ __launch_bounds__(IDX_WAVES *MINF_WAVE, ZERO_FILL ? 8 : 1) void vs_index_fast_kernel(
    const int32_t *__restrict__ seqlens, const int32_t *__restrict__ vertical,
    const int32_t *__restrict__ slash, const int32_t *__restrict__ tables,
    int32_t *__restrict__ block_count, int32_t *__restrict__ block_offset,
    int32_t *__restrict__ column_count, int32_t *__restrict__ column_index, int heads, int rows,
    int nnz_v, int nnz_s, int32_t *error_flag, long long total_rows) {
    constexpr int zero_fill = ZERO_FILL ? 1 : 0;
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
    const int32_t *hdr = tables + bh * idx_tab_ints(nnz_s, rows);
    const int32_t *cpos = hdr + IDX_TAB_HDR, *cpre = cpos + nnz_s, *crun = cpre + nnz_s;
    const int32_t *run_a = crun + nnz_s, *run_e = run_a + nnz_s, *cgaps = run_e + nnz_s, *glist = cgaps + nnz_s;
    const uint32_t *bm = reinterpret_cast<const uint32_t *>(glist + nnz_s);

    const int seqlen = seqlens[b];
    const int start_m = m * 64;
    const int end_m = start_m + 64;
    const uint64_t lt = minf_lanemask_lt();

    int nb = 0, ncol = 0;
    bool live = start_m < seqlen;

    // loads that do not depend on each other, issued together (the kernel is bound by chains of
    // dependent loads, not by bandwidth)
    const int o_first = sl[0], o_last = sl[nnz_s - 1];
    const int tab_blocks = hdr[0], tab_runs = hdr[1], tab_v = hdr[2], bm_ok = hdr[3], ngaps = hdr[4];
    const bool whole_list = o_first <= end_m - 64;      // nothing skipped, nothing clipped

    int s0 = nnz_s;
    if (live) {
        // first entry with an offset below end_m = number of entries >= end_m (descending list):
        // 64 samples one stride apart locate the segment, the lanes then count inside it -- two
        // rounds of independent loads instead of a 13-step chain of dependent ones
        s0 = 0;
        if (!whole_list) {
            const int stride = (nnz_s + MINF_WAVE - 1) / MINF_WAVE;
            const int si = min(lane * stride, nnz_s - 1);
            const bool above = lane * stride < nnz_s && sl[si] >= end_m;
            const int nseg = __builtin_popcountll(__ballot(above));       // samples 0..nseg-1 are >= end_m
            if (nseg > 0) {
                const int seg = (nseg - 1) * stride;                      // entries [0, seg] are >= end_m
                int cnt = 0;
                for (int i0 = 0; i0 < stride; i0 += MINF_WAVE) {        // same trip count in every lane
                    const int idx = seg + i0 + lane;
                    const bool ab = i0 + lane < stride && idx < nnz_s && sl[idx] >= end_m;
                    cnt += __builtin_popcountll(__ballot(ab));
                }
                s0 = seg + cnt;
            }
        }
        if (s0 >= nnz_s) {           // the reference would read past the list here
            live = false;
            if (error_flag && lane == 0) *error_flag = 1;
        }
    }

    if (live) {
        int vp = 0;
        int g = -1;                  // list entry from which the tables apply
        int e_lim = INT_MIN;         // end of the last explicitly built range
        if (whole_list) {
            g = 0;
        } else {
            int carried_e = 0, carried_t = 0, cur_a = 0;
            int ep0 = INT_MIN;
            bool first = true;
            for (int base = s0; base < nnz_s; base += MINF_WAVE) {
                int cnt = min(MINF_WAVE, nnz_s - base);
                const bool full = cnt == MINF_WAVE;
                bool valid = lane < cnt;
                int t = valid ? max(end_m - sl[base + lane], 64) : 0;
                int tlast = minf_readlane(t, cnt - 1);
                if (!valid) t = tlast;
                if (first) {
                    const int t0 = minf_readlane(t, 0);
                    cur_a = t0 - 64;
                    carried_e = t0 - 64;
                    carried_t = t0;
                    first = false;
                }
                uint64_t starts, gm;         // gm: entries of this chunk more than 64 above their predecessor
                int a = chunk_ranges(t, lane, cur_a, carried_e, carried_t, starts, &gm);
                const bool any_gap = gm != 0;
                // the first range start of this chunk that is also a tabulated range start
                const bool tab = ((starts >> lane) & 1ull) && cpre[base + lane] >= 0;
                const uint64_t tm = __ballot(tab);
                const int cut = tm ? __builtin_ctzll(tm) : -1;
                if (cut == 0) {          // nothing of this chunk belongs to the explicit part
                    g = base;
                    e_lim = carried_e;
                    break;
                }
                if (cut > 0) {           // entries [0, cut) only; later lanes repeat entry cut-1
                    cnt = cut;
                    valid = lane < cnt;
                    tlast = minf_readlane(t, cnt - 1);
                    const int alast = minf_readlane(a, cnt - 1);
                    if (!valid) { t = tlast; a = alast; }
                }
                const int e = a + ((((t - a) + 63) >> 6) << 6);
                int eprev = lane_above(e);
                if (lane == 0) eprev = carried_e;
                const bool changed = valid && (e != eprev);
                const uint64_t cm = __ballot(changed);
                if (changed) bo_row[nb + __builtin_popcountll(cm & lt)] = e - 64;
                nb += __builtin_popcountll(cm);

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
                        if (emit) ci_row[ncol + __builtin_popcountll(em & lt)] = x;
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
                if (cut > 0) {
                    g = base + cut;
                    e_lim = carried_e;
                    break;
                }
                // A whole chunk without a gap: a dense run.  No range can start before the next entry of
                // the gap list, so the entries up to there only extend the current range; their blocks
                // are written at once and the walk resumes at that entry.
                const int lo = base + MINF_WAVE;             // first entry not looked at yet
                if (full && !any_gap && lo < nnz_s) {
                    const int pos = __builtin_amdgcn_readfirstlane(cgaps[lo - 1]);   // gap entries below lo
                    const int X = pos < ngaps ? __builtin_amdgcn_readfirstlane(glist[pos]) : nnz_s;      // first one >= lo
                    if (X > lo) {
                        const int t_end = max(end_m - __builtin_amdgcn_readfirstlane(sl[X - 1]), 64);
                        const int e_end = cur_a + ((((t_end - cur_a) + 63) >> 6) << 6);
                        const int nnew = (e_end - carried_e) >> 6;
                        for (int j = lane; j < nnew; j += MINF_WAVE) bo_row[nb + j] = carried_e + 64 * j;
                        nb += nnew;
                        // the verticals below t_end lie inside the current range: none is emitted
                        while (vp < nnz_v) {
                            const int x = (vp + lane < nnz_v) ? vert[vp + lane] : INT_MAX;
                            const int k = __builtin_popcountll(__ballot(x < t_end));
                            vp += k;
                            if (k < MINF_WAVE) break;
                        }
                        carried_e = e_end;
                        carried_t = t_end;
                        ep0 = e_end;
                        base = X - MINF_WAVE;                // (the loop's increment makes it X)
                    }
                }
            }
        }
        if (g >= 0) {
            const int shift = end_m - tab_v;
            const int k0 = g == 0 ? 0 : cpre[g], r0 = g == 0 ? 0 : crun[g];   // entry 0 starts range 0
            const int nblk = tab_blocks - k0, nruns = tab_runs;
            copy_shifted(bo_row + nb, cpos + k0, nblk, shift, lane);
            nb += nblk;
            const int t_end = end_m - o_last;             // t of the last entry (not clipped here)
            const int first_a = run_a[r0];                // start of the first remaining range
            // four batches of 64 verticals per round: their loads and their coverage look-ups are
            // independent, only the ordered emit is sequential
            while (vp < nnz_v) {
                int x[4];
                bool emit[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) x[u] = (vp + u * MINF_WAVE + lane < nnz_v) ? vert[vp + u * MINF_WAVE + lane] : INT_MAX;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    emit[u] = false;
                    if (x[u] < t_end && x[u] >= e_lim) {
                        const int xv = x[u] - shift;
                        if (xv < first_a) {                   // below every remaining range
                            emit[u] = true;
                        } else if (bm_ok) {                   // xv < tab_v: inside the bitmap
                            emit[u] = !((bm[xv >> 5] >> (xv & 31)) & 1u);
                        } else {
                            int lo = r0, hi = nruns;          // first range >= r0 that ends after xv
                            while (lo < hi) {
                                int mid = (lo + hi) >> 1;
                                if (run_e[mid] > xv) hi = mid; else lo = mid + 1;
                            }
                            emit[u] = !(lo < nruns && run_a[lo] <= xv);
                        }
                    }
                }
                bool more = true;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint64_t em = __ballot(emit[u]);
                    if (emit[u]) ci_row[ncol + __builtin_popcountll(em & lt)] = x[u];
                    ncol += __builtin_popcountll(em);
                    more = more && __builtin_popcountll(__ballot(x[u] < t_end)) == MINF_WAVE;
                }
                vp += 4 * MINF_WAVE;
                if (!more) break;                             // verticals ascend: nothing further is below t_end
            }
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


extern "C" size_t minf_vs_index_workspace_bytes(int batch, int heads, int nnz_s, int rows) {
    if (batch <= 0 || heads <= 0 || nnz_s <= 0 || rows < 0) return 0;
    return (size_t)batch * heads * (size_t)idx_tab_ints(nnz_s, rows) * sizeof(int32_t);
}

// launches of the table-driven builder on a workspace that is known to be large enough
static int index_build_tables(const int32_t *seqlens, const int32_t *vertical_idx, const int32_t *slash_idx,
                              int32_t *block_count, int32_t *block_offset, int32_t *column_count,
                              int32_t *column_index, int batch, int heads, int rows, int nnz_v, int nnz_s,
                              int zero_fill, int32_t *error_flag, int32_t *workspace, long long total,
                              hipStream_t stream) {
    const long long nblk = (total + IDX_WAVES - 1) / IDX_WAVES;
    if (nblk > 0x7fffffffLL || (long long)batch * heads > 65535) return MINF_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(vs_index_prep_kernel, dim3((unsigned)(batch * heads)), dim3(PREP_WAVES * MINF_WAVE), 0,
                       stream, slash_idx, workspace, nnz_s, rows);
    int status = minf_launch_status();
    if (status != MINF_OK) return status;
    const long long bm_threads = idx_bm_words(rows) > nnz_s ? idx_bm_words(rows) : (long long)nnz_s;   // words and list entries
    hipLaunchKernelGGL(vs_index_bitmap_kernel, dim3((unsigned)((bm_threads + 255) / 256), (unsigned)(batch * heads)),
                       dim3(256), 0, stream, workspace, nnz_s, rows);
    status = minf_launch_status();
    if (status != MINF_OK) return status;
    // With zero-filled outputs the row-block pass is bound by its stores, and 24 resident waves per CU
    // write faster than 32 (6-9 % at 128K-512K tokens: fewer rows in flight, better DRAM locality); the
    // payload-only form is bound by its chains of dependent loads and wants every wave it can get.
    // Unused dynamic LDS is the occupancy limiter: 3 KB static + 24000 B -> 6 workgroups per CU.
    const unsigned occupancy_lds = zero_fill ? 24000u : 0u;
    if (zero_fill)
        hipLaunchKernelGGL(vs_index_fast_kernel<true>, dim3((unsigned)nblk), dim3(IDX_WAVES * MINF_WAVE), occupancy_lds,
                           stream, seqlens, vertical_idx, slash_idx, (const int32_t *)workspace,
                           block_count, block_offset, column_count, column_index, heads, rows, nnz_v, nnz_s,
                           error_flag, total);
    else
        hipLaunchKernelGGL(vs_index_fast_kernel<false>, dim3((unsigned)nblk), dim3(IDX_WAVES * MINF_WAVE), occupancy_lds,
                           stream, seqlens, vertical_idx, slash_idx, (const int32_t *)workspace,
                           block_count, block_offset, column_count, column_index, heads, rows, nnz_v, nnz_s,
                           error_flag, total);
    return minf_launch_status();
}

extern "C" int minf_vs_index_build_ws(const int32_t *seqlens, const int32_t *vertical_idx,
                                      const int32_t *slash_idx, int32_t *block_count,
                                      int32_t *block_offset, int32_t *column_count,
                                      int32_t *column_index, int batch, int heads, int rows,
                                      int nnz_v, int nnz_s, int zero_fill, int32_t *error_flag,
                                      void *workspace, size_t workspace_bytes, void *stream) {
    if (!seqlens || !vertical_idx || !slash_idx || !block_count || !block_offset ||
        !column_count || !column_index)
        return MINF_ERR_INVALID_ARG;
    if (batch < 0 || heads < 0 || rows < 0 || nnz_v < 1 || nnz_s < 1) return MINF_ERR_INVALID_ARG;
    const long long total = (long long)batch * heads * rows;
    if (total == 0) return MINF_OK;
    if (!workspace || workspace_bytes < minf_vs_index_workspace_bytes(batch, heads, nnz_s, rows) ||
        ((uintptr_t)workspace & 3))
        return MINF_ERR_WORKSPACE;
    return index_build_tables(seqlens, vertical_idx, slash_idx, block_count, block_offset, column_count,
                              column_index, batch, heads, rows, nnz_v, nnz_s, zero_fill, error_flag,
                              (int32_t *)workspace, total, (hipStream_t)stream);
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// The tables and bitmaps of minf_vs_index_build_ws live in this array instead of a caller-owned
// workspace.  Every GPU holds its own copy at its own address; host code only ever uses the address
// hipGetSymbolAddress returned for the current device, never the array's name.  Nothing in it has
// to start at zero: the table pass and the bitmap pass write every word the row-block pass reads.
static __device__ __align__(256) int32_t scratch[MINF_VS_INDEX_STATIC_BYTES / sizeof(int32_t)];

#define IDX_MAX_DEVICES 64
static std::atomic<int32_t *> scratch_ptr[IDX_MAX_DEVICES];

static int scratch_for_current_device(int32_t **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return minf_hip_status(e);
    if (dev < 0 || dev >= IDX_MAX_DEVICES) return MINF_ERR_UNSUPPORTED;
    int32_t *ptr = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // first call on this device; two threads racing here get the same address
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return minf_hip_status(e);
        if (!ptr) return MINF_ERR_HIP_BASE;
        scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return MINF_OK;
}

extern "C" int minf_vs_index_build_static(const int32_t *seqlens, const int32_t *vertical_idx,
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
    // sizes beyond the array are refused before any HIP call
    if (minf_vs_index_workspace_bytes(batch, heads, nnz_s, rows) > (size_t)MINF_VS_INDEX_STATIC_BYTES)
        return MINF_ERR_WORKSPACE;
    int32_t *ws = nullptr;
    const int st = scratch_for_current_device(&ws);
    if (st != MINF_OK) return st;
    return index_build_tables(seqlens, vertical_idx, slash_idx, block_count, block_offset, column_count,
                              column_index, batch, heads, rows, nnz_v, nnz_s, zero_fill, error_flag,
                              ws, total, (hipStream_t)stream);
}
