// Top-k index selection over fp32 score rows for gfx950 (vertical / slash
// candidates: k = 1000 / 6096 of up to ~10^6 entries per head).
//
// Rows longer than 4096 entries, one 1024-thread workgroup per row (shorter rows: one wavefront
// per row, see topk_wave_kernel):
//   1. MSB-first radix select (4 x 8 bits, LDS histogram) finds the exact value
//      T of the k-th largest entry and how many entries equal to T are needed;
//   2. every wavefront counts, over its contiguous slice, entries > T and == T;
//   3. the slices are scanned and the selected indices are written in
//      ASCENDING INDEX order with ballot prefix counts (entries > T always,
//      entries == T lowest index first until k are out).
// Ties are therefore resolved towards the lowest index (torch.topk, which the
// reference uses at minference/modules/minference_forward.py:607,612, leaves the
// tie order unspecified), and the output needs no sort before the index
// builder.  Keys are compared by their bit patterns, so -0.0 ranks just below
// +0.0 instead of tying with it (the score rows of this path hold no
// negative zeros: they are sums of probabilities).  With reverse_base >= 0 the value written is reverse_base - index
// (slash: diagonal offset = N-1-j, so ascending j gives descending offsets).
#include "minf_common.h"
#include <type_traits>

namespace {

constexpr int TK_THREADS = 1024;
constexpr int TK_WAVES = TK_THREADS / 64;
constexpr int TK_DEPTH = 16;          // independent 16-byte loads per thread in the sweeps

__device__ __forceinline__ unsigned order_key(float x) {
    unsigned u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);   // monotone for all finite/inf floats
}

struct TopkProblem {
    const float *scores;
    long long row_stride;
    int k;
    int32_t *out;
    long long out_stride;
    int reverse_base;
    // block-causal score rows (wave kernel only): row r belongs to query block m = r % causal_rows and
    // only its first 32 * (m / 32 + 1) entries are stored; the rest counts as -inf.  0 = plain rows
    int causal_rows;
    // ragged selection: row i keeps k_rows[i] entries (clamped to 1..k) and the rest of its k output
    // slots is padding -- pad_mode 1: the constant pad_value, 2: the last selected value repeated.
    // k_rows == nullptr: every row keeps k entries.
    const int *k_rows;
    int pad_mode, pad_value;
};

// blockIdx.y selects one of two problems over rows of the same length n (vertical and slash
// scores of a layer are selected in one launch so that twice as many CUs are busy)
__global__ __launch_bounds__(TK_THREADS) void topk_kernel(const TopkProblem p0, const TopkProblem p1, int n) {
    const TopkProblem &pr = blockIdx.y == 0 ? p0 : p1;
    const float *__restrict__ scores = pr.scores;
    const long long row_stride = pr.row_stride;
    const int kmax = pr.k;
    const int k = pr.k_rows ? max(1, min(pr.k_rows[blockIdx.x], kmax)) : kmax;
    int32_t *__restrict__ out = pr.out;
    const long long out_stride = pr.out_stride;
    const int reverse_base = pr.reverse_base;
    // 32 copies of the 256-bin histogram, copy = lane % 32 = LDS bank: score rows have few distinct
    // exponents, so most lanes of a wave hit the same bin; with one copy per bank they neither
    // serialise on one address nor conflict on a bank
    __shared__ unsigned hist[256 * 32];
    __shared__ unsigned bins[4];             // bin counts of waves 0..3
    __shared__ unsigned sh_prefix, sh_need;
    __shared__ int sh_last;
    __shared__ int wave_gt[TK_WAVES], wave_eq[TK_WAVES];

    const float *x = scores + (long long)blockIdx.x * row_stride;
    int32_t *o = out + (long long)blockIdx.x * out_stride;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;

    if (k >= n) {                    // everything is selected
        for (int i = tid; i < n; i += TK_THREADS) o[i] = reverse_base >= 0 ? reverse_base - i : i;
        return;
    }

    // ---- 1. radix select --------------------------------------------------
    const int nvec = (((uintptr_t)x & 15) == 0) ? (n >> 2) : 0;
    unsigned prefix = 0;
    unsigned need = (unsigned)k;     // rank (from the top) inside the current prefix bucket
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = tid; i < 256 * 32; i += TK_THREADS) hist[i] = 0;
        __syncthreads();
        // After the first pass the keys that still matter form one bucket [prefix, prefix + width) that
        // lies wholly among the positive or wholly among the negative floats (the sign is part of the
        // first digit), i.e. one range of raw bit patterns: membership is a subtract and an unsigned
        // compare on the raw bits, and only members (few) are turned into keys.
        const unsigned width = shift < 24 ? 1u << (shift + 8) : 0u;
        const unsigned raw_base = (prefix & 0x80000000u) ? (prefix ^ 0x80000000u) : ~(prefix + width - 1u);
        auto sweep = [&](auto first_c) {
            constexpr bool FIRST = decltype(first_c)::value;        // first pass: every entry counts
            auto tally = [&](float xv) {
                if (FIRST || __float_as_uint(xv) - raw_base < width) {
                    const unsigned u = order_key(xv);
                    atomicAdd(&hist[(((u >> shift) & 255u) << 5) + (lane & 31)], 1u);
                }
            };
            // 16-byte loads over the aligned part, TK_DEPTH in flight per thread: one workgroup sweeps a
            // whole row, so its rate is (bytes in flight) / (memory latency) until the CU's load path fills
            int i = tid;
            for (; i + (TK_DEPTH - 1) * TK_THREADS < nvec; i += TK_DEPTH * TK_THREADS) {
                float4 q[TK_DEPTH];
#pragma unroll
                for (int u = 0; u < TK_DEPTH; ++u) q[u] = reinterpret_cast<const float4 *>(x)[i + u * TK_THREADS];
#pragma unroll
                for (int u = 0; u < TK_DEPTH; ++u) { tally(q[u].x); tally(q[u].y); tally(q[u].z); tally(q[u].w); }
            }
            for (; i < nvec; i += TK_THREADS) {
                const float4 q = reinterpret_cast<const float4 *>(x)[i];
                tally(q.x); tally(q.y); tally(q.z); tally(q.w);
            }
            for (int j = nvec * 4 + tid; j < n; j += TK_THREADS) tally(x[j]);
        };
        if (shift == 24) sweep(std::true_type{}); else sweep(std::false_type{});
        __syncthreads();
        // Threads 0..255 fold the 32 copies of one bin each (rotated: one bank per thread), bin 255 - tid,
        // so that an inclusive prefix scan over the threads counts the entries in this bin and above;
        // the bin that takes the running count to `need` is the next digit of the threshold.
        unsigned cnt = 0, incl = 0;
        const int b = 255 - tid;
        if (tid < 256) {
#pragma unroll
            for (int c = 0; c < 32; ++c) cnt += hist[(b << 5) + ((c + b) & 31)];
            incl = cnt;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const unsigned up = __shfl_up(incl, d);
                if (lane >= d) incl += up;
            }
            if (lane == 63) bins[wave] = incl;
        }
        __syncthreads();
        if (tid < 256) {
            for (int wv = 0; wv < wave; ++wv) incl += bins[wv];
            const unsigned excl = incl - cnt;
            if ((excl < need && need <= incl) || (b == 0 && incl < need)) {
                sh_prefix = prefix | ((unsigned)b << shift);
                sh_need = need - excl;
            }
        }
        __syncthreads();
        prefix = sh_prefix;
        need = sh_need;
    }
    const unsigned T = prefix;       // key of the k-th largest; `need` entries equal to T are taken

    // ---- 2. per-wave counts over contiguous slices --------------------------
    const int per_wave = ((n + TK_WAVES * 64 - 1) / (TK_WAVES * 64)) * 64;
    const int begin = wave * per_wave;
    const int end = min(n, begin + per_wave);
    int cgt = 0, ceq = 0;
    const bool vec = nvec > 0;                    // slices start at multiples of 64 elements
    const int vend = vec ? begin + ((max(end - begin, 0)) & ~255) : begin;   // whole 256-element groups
    auto count4 = [&](const float4 &q) {
        const unsigned u0 = order_key(q.x), u1 = order_key(q.y), u2 = order_key(q.z), u3 = order_key(q.w);
        cgt += (u0 > T) + (u1 > T) + (u2 > T) + (u3 > T);
        ceq += (u0 == T) + (u1 == T) + (u2 == T) + (u3 == T);
    };
    {
        int i = begin + 4 * lane;
        for (; i + (TK_DEPTH - 1) * 256 < vend; i += TK_DEPTH * 256) {
            float4 q[TK_DEPTH];
#pragma unroll
            for (int u = 0; u < TK_DEPTH; ++u) q[u] = *reinterpret_cast<const float4 *>(x + i + u * 256);
#pragma unroll
            for (int u = 0; u < TK_DEPTH; ++u) count4(q[u]);
        }
        for (; i < vend; i += 256) count4(*reinterpret_cast<const float4 *>(x + i));
    }
    for (int i = vend + lane; i < end; i += 64) {
        const unsigned u = order_key(x[i]);
        cgt += u > T;
        ceq += u == T;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        cgt += __shfl_xor(cgt, d);
        ceq += __shfl_xor(ceq, d);
    }
    if (lane == 0) { wave_gt[wave] = cgt; wave_eq[wave] = ceq; }
    __syncthreads();
    int gt_before = 0, eq_before = 0;
    for (int wv = 0; wv < wave; ++wv) { gt_before += wave_gt[wv]; eq_before += wave_eq[wv]; }

    // ---- 3. ordered emit ---------------------------------------------------
    int r = (int)need;
    const uint64_t lt = minf_lanemask_lt();
    // When every entry equal to T is taken (r == their number: always so when T occurs once), "selected"
    // is simply key >= T: the loop then runs on the threshold T - 1 with no tie bookkeeping, which
    // halves its ballots.
    int tot_eq = 0;
    for (int wv = 0; wv < TK_WAVES; ++wv) tot_eq += wave_eq[wv];
    const bool all_ties = tot_eq == r && T != 0u;          // (workgroup-uniform)
    const unsigned Te = all_ties ? T - 1u : T;
    if (all_ties) { gt_before += eq_before; eq_before = 0; r = 0; }
    // 256 elements per step: lane l holds indices base + 4l .. 4l+3, so the rank of an element is
    // (selected elements of lower lanes, all four components) + (selected lower components of its lane)
    auto emit4 = [&](const float4 &q, int i0, auto ties_c) {
        constexpr bool TIES = decltype(ties_c)::value;
        const unsigned u[4] = {order_key(q.x), order_key(q.y), order_key(q.z), order_key(q.w)};
        int g_lower = 0, e_lower = 0, g_all = 0, e_all = 0;
        bool gt[4], eq[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            gt[c] = u[c] > Te;
            const uint64_t mg = __ballot(gt[c]);
            g_lower += __builtin_popcountll(mg & lt);
            g_all += __builtin_popcountll(mg);
            eq[c] = false;
            if constexpr (TIES) {
                eq[c] = u[c] == Te;
                const uint64_t me = __ballot(eq[c]);
                e_lower += __builtin_popcountll(me & lt);
                e_all += __builtin_popcountll(me);
            }
        }
        if (TIES || g_all) {                               // (wave-uniform)
            int g_here = gt_before + g_lower, e_here = eq_before + e_lower;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (gt[c] || (eq[c] && e_here < r)) {
                    const int i = i0 + c;
                    const int pos = g_here + min(e_here, r), val = reverse_base >= 0 ? reverse_base - i : i;
                    o[pos] = val;
                    if (pos == k - 1) sh_last = val;
                }
                g_here += gt[c];
                e_here += eq[c];
            }
        }
        gt_before += g_all;
        eq_before += e_all;
    };
    constexpr int EMIT_DEPTH = 8;          // loads of this many steps go out before the first is used
    float4 qn[EMIT_DEPTH];
#pragma unroll
    for (int u = 0; u < EMIT_DEPTH; ++u)
        if (begin + u * 256 < vend) qn[u] = *reinterpret_cast<const float4 *>(x + begin + u * 256 + 4 * lane);
    for (int base0 = begin; base0 < vend; base0 += EMIT_DEPTH * 256) {
        float4 qc[EMIT_DEPTH];
#pragma unroll
        for (int u = 0; u < EMIT_DEPTH; ++u) qc[u] = qn[u];
#pragma unroll
        for (int u = 0; u < EMIT_DEPTH; ++u)
            if (base0 + (EMIT_DEPTH + u) * 256 < vend)
                qn[u] = *reinterpret_cast<const float4 *>(x + base0 + (EMIT_DEPTH + u) * 256 + 4 * lane);
#pragma unroll
        for (int uu = 0; uu < EMIT_DEPTH; ++uu) {
            const int base = base0 + uu * 256;
            if (base >= vend) break;
            if (all_ties) emit4(qc[uu], base + 4 * lane, std::false_type{});
            else emit4(qc[uu], base + 4 * lane, std::true_type{});
        }
    }
    for (int base = vend; base < end; base += 64) {
        const int i = base + lane;
        unsigned u = 0;
        bool gt = false, eq = false;
        if (i < end) { u = order_key(x[i]); gt = u > Te; eq = !all_ties && u == Te; }
        const uint64_t mg = __ballot(gt), me = __ballot(eq);
        const int g_here = gt_before + __builtin_popcountll(mg & lt);
        const int e_here = eq_before + __builtin_popcountll(me & lt);
        const bool take = gt || (eq && e_here < r);
        if (take) {
            const int pos = g_here + min(e_here, r), val = reverse_base >= 0 ? reverse_base - i : i;
            o[pos] = val;
            if (pos == k - 1) sh_last = val;
        }
        gt_before += __builtin_popcountll(mg);
        eq_before += __builtin_popcountll(me);
    }
    if (k < kmax && pr.pad_mode) {                 // (workgroup-uniform)
        __syncthreads();
        const int pad = pr.pad_mode == 2 ? sh_last : pr.pad_value;
        for (int i = k + tid; i < kmax; i += TK_THREADS) o[i] = pad;
    }
}

// Short rows (n <= 64 * ITEMS <= 4096, e.g. the block scores of block-sparse attention): one
// wavefront per row, the row held in registers (lane l owns indices l, l+64, ...).  The k-th
// largest key is found bit by bit: T = the largest value with count(key >= T) >= k, one counting
// pass per bit below the bits all live keys share, stopping as soon as a count hits k exactly
// (no LDS, no barriers); the emit is the same ordered ballot-prefix write as in the wide kernel, so
// both kernels select identical sets.
constexpr int TKW_WAVES = 4;
// (the second launch bound is the number of resident waves per SIMD the register budget must allow:
// the kernel is latency bound, and left alone the 64-item variant took 141 registers = 3 waves)
template <int ITEMS>
__global__ __launch_bounds__(TKW_WAVES * 64, ITEMS >= 64 ? 3 : (ITEMS >= 40 ? 5 : 8)) void topk_wave_kernel(const TopkProblem p0, const TopkProblem p1,
                                                                   int n, int rows) {
    const TopkProblem &pr = blockIdx.y == 0 ? p0 : p1;
    const int lane = (int)threadIdx.x & 63, wave = (int)threadIdx.x >> 6;
    const int row = (int)blockIdx.x * TKW_WAVES + wave;
    if (row >= rows) return;
    const float *__restrict__ x = pr.scores + (long long)row * pr.row_stride;
    int32_t *__restrict__ o = pr.out + (long long)row * pr.out_stride;
    const int kcap = pr.k, reverse_base = pr.reverse_base;
    const int k = pr.k_rows ? max(1, min(pr.k_rows[row], kcap)) : kcap;
    if (k >= n) {
        for (int i = lane; i < n; i += 64) o[i] = reverse_base >= 0 ? reverse_base - i : i;
        return;
    }
    constexpr unsigned KEY_FLOOR = 0x007fffffu;          // order_key(-inf)
    const int stored = pr.causal_rows > 0 ? min(n, 32 * ((row % pr.causal_rows) / 32 + 1)) : n;
    unsigned key[ITEMS];
    constexpr int LGROUP = ITEMS >= 8 ? 8 : ITEMS;
#pragma unroll
    for (int jb = 0; jb < ITEMS; jb += LGROUP) {
        if (jb * 64 < stored) {                        // (wave-uniform: groups past the stored prefix load nothing)
#pragma unroll
            for (int j = jb; j < jb + LGROUP; ++j) {
                const int i = j * 64 + lane;
                // padding sorts below every real score; entries that are not stored are -inf
                key[j] = i < stored ? order_key(x[i]) : (i < n ? KEY_FLOOR : 0u);
            }
        } else {
#pragma unroll
            for (int j = jb; j < jb + LGROUP; ++j) key[j] = j * 64 + lane < n ? KEY_FLOOR : 0u;
        }
    }
    // Rows with a masked (-inf) tail, e.g. block-causal score rows: when at least k entries are above
    // -inf, the threshold is too, and register groups that hold nothing above -inf can be skipped
    // in every pass and in the emit (they add nothing to a count of keys >= cand > key(-inf), and
    // for cand <= key(-inf) the live groups alone already reach k).
    constexpr int GROUP = ITEMS >= 8 ? 8 : ITEMS;
    int nfin = 0, jmax = 0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int c = __builtin_popcountll(__ballot(key[j] > KEY_FLOOR));
        nfin += c;
        if (c) jmax = j + 1;
    }
    const bool with_floor = nfin < k;                // masked / padding entries take part in the selection
    if (with_floor) jmax = ITEMS;
    // Keys that can be the threshold lie between the smallest and the largest live key: the bits
    // those two share are bits of T, the search starts below them.
    unsigned kmax = 0u, kmin = 0xffffffffu;
#pragma unroll
    for (int jb = 0; jb < ITEMS; jb += GROUP) {
        if (jb < jmax) {
#pragma unroll
            for (int j = jb; j < jb + GROUP; ++j) {
                kmax = max(kmax, key[j]);
                kmin = min(kmin, (with_floor || key[j] > KEY_FLOOR) ? key[j] : 0xffffffffu);
            }
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        kmax = max(kmax, (unsigned)__shfl_xor((int)kmax, d));
        kmin = min(kmin, (unsigned)__shfl_xor((int)kmin, d));
    }
    const unsigned diff = kmax ^ kmin;
    const int top_bit = diff ? 31 - __builtin_clz(diff) : -1;            // highest bit in which live keys differ
    unsigned T = top_bit >= 0 ? (top_bit == 31 ? 0u : (kmax >> (top_bit + 1)) << (top_bit + 1)) : kmax;
    // Before the pass of `bit`, the keys that can still decide T are those that agree with T above
    // `bit` (the bucket [T, T + 2^(bit+1))); `above` counts the keys beyond the bucket (exact),
    // `from_t` the keys >= T (exact once T has been raised, an upper bound before).  When at most
    // 64 keys are left in the bucket they are gathered into one register (through LDS) and the
    // remaining passes compare that register only: an early pass costs a compare per held key, and
    // there are about as many late passes as early ones.
    int above = 0, from_t = (jmax + GROUP - 1) / GROUP * GROUP * 64;      // (whole register groups are visited)
    int bit = top_bit;
    for (; bit >= 0 && from_t - above > 64; --bit) {
        const unsigned cand = T | (1u << bit);
        // every lane counts its own keys (compare + add with carry), the lane counts (< 128) are
        // summed through seven ballots of their bits
        int c = 0;
#pragma unroll
        for (int jb = 0; jb < ITEMS; jb += GROUP) {
            if (jb < jmax) {
#pragma unroll
                for (int j = jb; j < jb + GROUP; ++j) c += key[j] >= cand ? 1 : 0;
            }
        }
        int cnt = 0;
#pragma unroll
        for (int b = 0; b < (ITEMS >= 64 ? 7 : (ITEMS >= 32 ? 6 : (ITEMS >= 16 ? 5 : 3))); ++b)
            cnt += __builtin_popcountll(__ballot((c >> b) & 1)) << b;
        if (cnt >= k) { T = cand; from_t = cnt; } else above = cnt;
        if (cnt == k) { bit = -1; break; }           // exactly k keys are >= T: nothing left to decide
    }
    if (bit >= 0) {
        __shared__ unsigned bucket[TKW_WAVES][64];
        const uint64_t lower = minf_lanemask_lt();
        int filled = 0;
#pragma unroll
        for (int jb = 0; jb < ITEMS; jb += GROUP) {
            if (jb < jmax) {
#pragma unroll
                for (int j = jb; j < jb + GROUP; ++j) {
                    const bool in = ((key[j] ^ T) >> bit) >> 1 == 0u;      // agrees with T above `bit`
                    const uint64_t m = __ballot(in);
                    if (in) bucket[wave][filled + __builtin_popcountll(m & lower)] = key[j];
                    filled += __builtin_popcountll(m);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const unsigned mine = lane < filled ? bucket[wave][lane] : 0u;       // 0 lies below every candidate
        // (`above` stays what it was at the gather: the keys beyond the gathered bucket)
        for (; bit >= 0; --bit) {
            const unsigned cand = T | (1u << bit);
            const int cnt = above + __builtin_popcountll(__ballot(mine >= cand));
            if (cnt >= k) T = cand;
            if (cnt == k) break;
        }
    }
    int cgt = 0;
#pragma unroll
    for (int jb = 0; jb < ITEMS; jb += GROUP) {
        if (jb < jmax) {
#pragma unroll
            for (int j = jb; j < jb + GROUP; ++j) cgt += __builtin_popcountll(__ballot(key[j] > T));
        }
    }
    const int r = k - cgt;                           // entries equal to T that are taken, lowest index first
    int gt_before = 0, eq_before = 0;
    int lastv = 0;
    bool has_last = false;
    const uint64_t lt = minf_lanemask_lt();
#pragma unroll
    for (int jb = 0; jb < ITEMS; jb += GROUP) {
        if (jb < jmax) {
#pragma unroll
            for (int j = jb; j < jb + GROUP; ++j) {
                const int i = j * 64 + lane;
                const bool gt = key[j] > T, eq = key[j] == T;
                const uint64_t mg = __ballot(gt), me = __ballot(eq);
                const int e_here = eq_before + __builtin_popcountll(me & lt);
                if (gt || (eq && e_here < r)) {
                    const int pos = gt_before + __builtin_popcountll(mg & lt) + min(e_here, r);
                    const int val = reverse_base >= 0 ? reverse_base - i : i;
                    o[pos] = val;
                    if (pos == k - 1) { lastv = val; has_last = true; }
                }
                gt_before += __builtin_popcountll(mg);
                eq_before += __builtin_popcountll(me);
            }
        }
    }
    if (k < kcap && pr.pad_mode) {                 // (wave-uniform)
        int pad = pr.pad_value;
        if (pr.pad_mode == 2) {
            const uint64_t who = __ballot(has_last);
            pad = who ? minf_readlane(lastv, __builtin_ctzll(who)) : 0;
        }
        for (int i = k + lane; i < kcap; i += 64) o[i] = pad;
    }
}

void launch_topk(const TopkProblem &pa, const TopkProblem &pb, int problems, int rows, int n, hipStream_t st) {
    const dim3 grid_w((unsigned)((rows + TKW_WAVES - 1) / TKW_WAVES), (unsigned)problems);
    if (n <= 64 * 4)
        hipLaunchKernelGGL(topk_wave_kernel<4>, grid_w, dim3(TKW_WAVES * 64), 0, st, pa, pb, n, rows);
    else if (n <= 64 * 16)
        hipLaunchKernelGGL(topk_wave_kernel<16>, grid_w, dim3(TKW_WAVES * 64), 0, st, pa, pb, n, rows);
    else if (n <= 64 * 40)
        hipLaunchKernelGGL(topk_wave_kernel<40>, grid_w, dim3(TKW_WAVES * 64), 0, st, pa, pb, n, rows);
    else if (n <= 64 * 64)
        hipLaunchKernelGGL(topk_wave_kernel<64>, grid_w, dim3(TKW_WAVES * 64), 0, st, pa, pb, n, rows);
    else
        hipLaunchKernelGGL(topk_kernel, dim3((unsigned)rows, (unsigned)problems), dim3(TK_THREADS), 0, st, pa, pb, n);
}

}  // namespace

extern "C" int minf_topk_indices(const float *scores, int rows, int n, int64_t row_stride, int k,
                                 int32_t *out, int64_t out_stride, int reverse_base, void *stream) {
    if (!scores || !out || rows < 0 || n <= 0 || k <= 0) return MINF_ERR_INVALID_ARG;
    if (row_stride < n || out_stride < (k < n ? k : n)) return MINF_ERR_INVALID_ARG;
    if (rows == 0) return MINF_OK;
    TopkProblem p{scores, (long long)row_stride, k, out, (long long)out_stride, reverse_base, 0, nullptr, 0, 0};
    launch_topk(p, p, 1, rows, n, (hipStream_t)stream);
    return minf_launch_status();
}

extern "C" int minf_topk_indices_block_causal(const float *scores, int rows, int n, int64_t row_stride, int k,
                                              int32_t *out, int64_t out_stride, int rows_per_head, void *stream) {
    if (!scores || !out || rows < 0 || n <= 0 || k <= 0 || rows_per_head <= 0) return MINF_ERR_INVALID_ARG;
    if (row_stride < n || out_stride < (k < n ? k : n)) return MINF_ERR_INVALID_ARG;
    if (n > 64 * 64) return MINF_ERR_UNSUPPORTED;      // only the one-wave-per-row kernel knows about stored prefixes
    if (rows == 0) return MINF_OK;
    TopkProblem p{scores, (long long)row_stride, k, out, (long long)out_stride, -1, rows_per_head, nullptr, 0, 0};
    launch_topk(p, p, 1, rows, n, (hipStream_t)stream);
    return minf_launch_status();
}

extern "C" int minf_topk_indices_pair(const float *scores_a, int k_a, int32_t *out_a, int64_t out_stride_a,
                                      int reverse_base_a, const float *scores_b, int k_b, int32_t *out_b,
                                      int64_t out_stride_b, int reverse_base_b, int rows, int n,
                                      int64_t row_stride, void *stream) {
    if (!scores_a || !out_a || !scores_b || !out_b || rows < 0 || n <= 0 || k_a <= 0 || k_b <= 0)
        return MINF_ERR_INVALID_ARG;
    if (row_stride < n || out_stride_a < (k_a < n ? k_a : n) || out_stride_b < (k_b < n ? k_b : n))
        return MINF_ERR_INVALID_ARG;
    if (rows == 0) return MINF_OK;
    TopkProblem pa{scores_a, (long long)row_stride, k_a, out_a, (long long)out_stride_a, reverse_base_a, 0, nullptr, 0, 0};
    TopkProblem pb{scores_b, (long long)row_stride, k_b, out_b, (long long)out_stride_b, reverse_base_b, 0, nullptr, 0, 0};
    launch_topk(pa, pb, 2, rows, n, (hipStream_t)stream);
    return minf_launch_status();
}

extern "C" int minf_topk_indices_pair_ragged(const float *scores_a, const int32_t *k_rows_a, int k_max_a, int32_t *out_a,
                                             int64_t out_stride_a, int reverse_base_a, int pad_mode_a, int pad_value_a,
                                             const float *scores_b, const int32_t *k_rows_b, int k_max_b, int32_t *out_b,
                                             int64_t out_stride_b, int reverse_base_b, int pad_mode_b, int pad_value_b,
                                             int rows, int n, int64_t row_stride, void *stream) {
    if (!scores_a || !out_a || !scores_b || !out_b || !k_rows_a || !k_rows_b || rows < 0 || n <= 0 || k_max_a <= 0 || k_max_b <= 0)
        return MINF_ERR_INVALID_ARG;
    if (pad_mode_a < 0 || pad_mode_a > 2 || pad_mode_b < 0 || pad_mode_b > 2) return MINF_ERR_INVALID_ARG;
    if (k_max_a > n) k_max_a = n;
    if (k_max_b > n) k_max_b = n;
    if (row_stride < n || out_stride_a < k_max_a || out_stride_b < k_max_b) return MINF_ERR_INVALID_ARG;
    if (rows == 0) return MINF_OK;
    TopkProblem pa{scores_a, (long long)row_stride, k_max_a, out_a, (long long)out_stride_a, reverse_base_a, 0, k_rows_a, pad_mode_a, pad_value_a};
    TopkProblem pb{scores_b, (long long)row_stride, k_max_b, out_b, (long long)out_stride_b, reverse_base_b, 0, k_rows_b, pad_mode_b, pad_value_b};
    launch_topk(pa, pb, 2, rows, n, (hipStream_t)stream);
    return minf_launch_status();
}
