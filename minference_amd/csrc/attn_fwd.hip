// Sparse flash-attention forward for gfx950: one 64x64 tile engine, four tile
// sources (vertical-slash block+column lists, block-sparse lists, analytic
// A-shape ranges, dense causal).
//
// Work split: one workgroup of 4 wavefronts per (batch, query head, PAIR of neighbouring 64-row
// blocks); each wavefront owns 32 query rows.  The two row blocks walk their tile lists in lockstep:
// a tile that is on both lists is copied into LDS once for 128 query rows, a tile that only one of
// them visits is copied by that half into buffers of its own while the other half does the same
// with a tile of its list.  For dense causal and A-shape / tri-shape the lists are analytic and
// differ by at most their ends; vertical-slash and block-sparse lists are split into common and
// leftover entries once, in LDS, before the tile loop.  Besides halving the
// copies of shared tiles, the lockstep is what keeps long scattered lists fast: row block m+1's
// list is row block m's shifted by 64 keys, so what one half fetches now the other fetched a step
// ago and finds in L2 (measured +23..38 % on lists of several hundred blocks, +1 % on the
// cache-friendly benchmark layer, against an earlier form of this kernel with one 2-wave workgroup
// per row block).
// Everything is computed in the TRANSPOSED orientation so that softmax statistics are per lane:
//
//   S^T[token][qrow] = K_tile . Q^T      v_mfma_f32_32x32x16 (A = K from LDS, B = Q in VGPRs)
//   O^T[d][qrow]    += V_tile^T . P^T    (A = V^T via ds_read_b64_tr_b16, B = P straight from
//                                          the S^T accumulators, converted to bf16/f16)
//
// In the 32x32 accumulator layout lane l holds column n = l%32 (one query row)
// and rows 8*(r/4) + 4*(l/32) + r%4, so the running max / sum / rescale factor
// of a query row live in lanes l and l^32 and never need a row broadcast, and
// the probabilities of a lane are exactly the B operand of the second MFMA once
// the contraction (token) index is permuted the same way on the V side.
//
// LDS: one K and one V tile per workgroup (two of each for vertical-slash lists: the second pair
// serves row block B in split steps), [64 tokens][128] 16-bit, 256-byte rows whose 16-byte
// chunks are XOR-permuted (K: chunk ^ row%16, V: chunk ^ 4*(row%4)) so that the ds_read_b128 of 32
// K rows and the 4-row transpose reads of V hit distinct banks.  Tiles are copied global -> LDS
// directly (no staging registers, no LDS store instructions); the permutation is applied on the
// global-address side.  Contiguous tiles use buffer_load_dwordx4 ... lds with a scalar descriptor of
// the 64 tile rows, a scalar row offset and one of five loop-invariant per-lane offsets: no vector
// instruction per copy and 8 cycles less issue time per copy than the 64-bit-address form, which
// remains for gathered and clamped rows (global_load_lds_dwordx4).  32-68 KB of LDS and <= 256 registers
// keep two waves per SIMD resident (two 4-wave workgroups per CU).
//
// One iteration of a wave (two workgroup barriers per tile, single buffers):
//   wait own K(it) copies; barrier (all of K(it) visible, everyone done with V(it-1))
//   issue V(it) copy; S^T = K.Q^T with the K fragments read two k-steps ahead of their MFMAs
//   wait own V(it) copies; barrier (all of V(it) visible, everyone done with K(it))
//   issue K(it+1) copy; read all V^T fragments; row max where it is needed; exponentials of keys 0..15
//   O^T += V^T.P^T with the exponentials of key group s+1 (16 keys) placed behind the MFMAs of
//   group s
// The compiler's own schedule read every fragment right before its MFMA (full LDS latency exposed
// sixteen times per tile); the order above is pinned with sched_barrier / sched_group_barrier.
//
// Other choices that measure faster on MI355X:
//  * index entries (block offsets, column counts) are wave-uniform and read through the constant
//    address space, i.e. scalar loads that do not queue behind the vector memory traffic; gathered
//    column ids are fetched one per lane an iteration ahead and distributed with wave shuffles;
//  * the running max is only raised when a tile exceeds it by more than 2^20 (bf16; 2^8 for f16
//    operands, whose probabilities must stay inside the f16 range), so nearly all tiles skip the
//    O^T rescale; for bf16 the row maximum is not even computed in most tiles (see sm_pv_block);
//  * the cross-half max uses v_permlane32_swap, the row sums v_dot2 on the rounded probabilities
//    (the same values the second MFMA consumes);
//  * s_setprio raises the wave while it issues MFMAs;
//  * the epilogue transposes O^T through LDS so each global store is 16 B of one 256-byte row.
#include "minf_common.h"
#include <math.h>
#include <string.h>
#include <type_traits>

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short short4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
// native vectors, not HIP's u32x4_t/u32x2_t structs: arrays of those are not promoted to registers
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2_t;

enum { MODE_VS = 0, MODE_BS = 1, MODE_ASHAPE = 2, MODE_DENSE = 3 };

constexpr int BM = 64;        // query rows per workgroup
constexpr int BN = 64;        // keys per tile
// head_dim (template parameter HD of the kernel): 64, 128 or, for dense / A-shape / tri-shape only, 256
constexpr int NTHREADS = 128; // 2 wavefronts per 64-row block, two row blocks per workgroup
// Scheduling constants (measured on MI355X): K fragments are read QK_AHEAD k-steps ahead of their
// MFMAs; VALU_PER_MFMA softmax instructions are placed behind each of the first twelve PV MFMAs.
constexpr int QK_AHEAD = 2;
constexpr int VALU_PER_MFMA = 6;
#ifndef MAX_PERIOD
#define MAX_PERIOD 8      // (a power of two) the row maximum is recomputed at least every MAX_PERIOD tiles
#endif
#ifndef LAZY_MAX_BF16
#define LAZY_MAX_BF16 20.0f
#endif
constexpr int VALU_MASK = 0x402;             // sched_group_barrier classes: VALU | transcendental

struct AttnParams {
    const char *q, *k, *v;
    char *o;
    long long qs[3], ks[3], vs[3], os[3];   // element strides: batch, head, token
    int batch, hq, hk, n;
    const int *seqlens;
    float scale_log2;
    float scale_log2_dense;  // tri-shape: scale of the rows >= dense_from (the reference scales them by the unpadded head_dim)
    int rows;
    // vertical-slash
    const int *bc, *bo, *cc, *ci;
    int nnz_s, nnz_v;
    // block-sparse
    const int *bidx;
    int max_blocks, bidx_rows;
    // a-shape; query rows >= dense_from attend to every earlier key (tri-shape), INT_MAX = none
    int n_init, n_local, dense_from;
    long long total_wg;
    int descending;          // row blocks are handed out from the last one down
    // optional head selection: head_list[i], i < index_heads, are the query heads to process and i is
    // the head's position in the index tensors (which then have index_heads heads); without a list
    // every head is processed and index_heads = hq
    const int *head_list;
    int index_heads;
};

typedef const __attribute__((address_space(4))) int *cint_ptr;
__device__ __forceinline__ cint_ptr as_const(const int *p) { return (cint_ptr)(unsigned long long)p; }
template <typename T> struct Mma;
template <> struct Mma<__bf16> {
    typedef bf16x8_t vec;
    static __device__ __forceinline__ f32x16_t mfma(vec a, vec b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<_Float16> {
    typedef f16x8_t vec;
    static __device__ __forceinline__ f32x16_t mfma(vec a, vec b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

union Frag {
    u32x4_t u;
    bf16x8_t b;
    f16x8_t h;
    short4_t s4[2];
};

template <typename T> __device__ __forceinline__ typename Mma<T>::vec frag_as(const Frag &f);
template <> __device__ __forceinline__ bf16x8_t frag_as<__bf16>(const Frag &f) { return f.b; }
template <> __device__ __forceinline__ f16x8_t frag_as<_Float16>(const Frag &f) { return f.h; }

template <typename T> __device__ __forceinline__ void cvt8(const float *x, Frag &f);
template <> __device__ __forceinline__ void cvt8<__bf16>(const float *x, Frag &f) {
#pragma unroll
    for (int j = 0; j < 8; ++j) f.b[j] = (__bf16)x[j];
}
template <> __device__ __forceinline__ void cvt8<_Float16>(const float *x, Frag &f) {
#pragma unroll
    for (int j = 0; j < 8; ++j) f.h[j] = (_Float16)x[j];
}

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
template <typename T> __device__ __forceinline__ float pair_sum(const Frag &f, float acc);
template <> __device__ __forceinline__ float pair_sum<__bf16>(const Frag &f, float acc) {
    const bf16x2_t one = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) { bf16x2_t pr = {f.b[2 * j], f.b[2 * j + 1]}; acc = __builtin_amdgcn_fdot2_f32_bf16(pr, one, acc, false); }
    return acc;
}
template <> __device__ __forceinline__ float pair_sum<_Float16>(const Frag &f, float acc) {
    const f16x2_t one = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) { f16x2_t pr = {f.h[2 * j], f.h[2 * j + 1]}; acc = __builtin_amdgcn_fdot2(pr, one, acc, false); }
    return acc;
}
// One tile of keys: either 64 consecutive tokens from `start`, or 64 gathered
// token ids read from `gather` (entries >= nvalid are padding).
struct Tile {
    int start;          // first token (contiguous) / first list position (gathered)
    int gathered;       // 0/1
    int nvalid;         // gathered: number of valid list entries in this tile
    int on_a, on_b;     // paired walks: is the tile on the list of row block A / B
    int split;          // paired list walks: each row block has a tile of its own in this step
};
// (the longest block list the paired kernel splits in LDS is what a K tile holds twice: 2048 entries
// at head_dim 128, 1024 at 64)
constexpr int VS_ONLY_MAX = 512;   // ... and the most entries of one list that the other one lacks

// One workgroup of 4 waves covers the row blocks mA = 2*mp and mB = mA + 1.  It
// walks the union of their two tile lists once, so every K/V tile is copied into LDS once for 128
// query rows; a half skips the tiles that are not on its own list.  For dense causal and A-shape /
// tri-shape the lists are analytic and differ by at most the ends (the three helpers below); for
// block-sparse the two lists are merged on the fly inside the kernel.
template <int MODE>
__device__ __forceinline__ int pair_tile_count(const AttnParams &p, int mA, int mB, int &nblk) {
    if (MODE == MODE_DENSE || mB * BM + BM - 1 >= p.dense_from) {
        nblk = mB + 1;
        return nblk;
    }
    int lo_key = mA * BM - p.n_local + 1;
    int t_lo = lo_key > 0 ? (lo_key >> 6) : 0;
    int sink_tiles = (p.n_init + BN - 1) >> 6;
    nblk = min(sink_tiles, t_lo);
    return nblk + (mB - t_lo + 1);
}
template <int MODE>
__device__ __forceinline__ int pair_tile_start(const AttnParams &p, int mA, int mB, int nblk, int it) {
    if (MODE == MODE_DENSE || mB * BM + BM - 1 >= p.dense_from) return it * BN;
    int lo_key = mA * BM - p.n_local + 1;
    int t_lo = lo_key > 0 ? (lo_key >> 6) : 0;
    return (it < nblk ? it : t_lo + (it - nblk)) * BN;
}
// is the tile that starts at key `start` on the list of row block m ?
template <int MODE>
__device__ __forceinline__ bool tile_on_list(const AttnParams &p, int m, int start) {
    const int ti = start >> 6;
    if (ti > m) return false;
    if (MODE == MODE_DENSE || m * BM + BM - 1 >= p.dense_from) return true;
    int lo_key = m * BM - p.n_local + 1;
    int t_lo = lo_key > 0 ? (lo_key >> 6) : 0;
    return ti >= t_lo || ti < ((p.n_init + BN - 1) >> 6);
}

// LDS of one workgroup (declared by the kernel, see attn_fwd_kernel): separate objects, so that the
// compiler lets reads of one overtake copies into the other.
template <int MODE, int HD> struct AttnLds {
    static constexpr bool VSP = MODE == MODE_VS || MODE == MODE_BS;      // walks of two block lists
    static constexpr int TILE_BYTES = BN * HD * 2;
    static constexpr int NK = (VSP ? 2 : 1) * TILE_BYTES;
    static constexpr int NONLY = VSP ? 2 * VS_ONLY_MAX : 1;
};

// The whole walk of one workgroup.  EVERY_MAX: the row maximum is computed for every tile; otherwise
// only where it is needed (see sm_pv_block), and the function returns true -- for the whole
// workgroup -- when a row sum left the safe range, i.e. when the walk has to be run again with
// EVERY_MAX (the output it wrote is then overwritten).
template <typename T, int MODE, int HD, bool EVERY_MAX>
__device__ __forceinline__ bool attn_walk(const AttnParams &p, char (&lds_k)[AttnLds<MODE, HD>::NK],
                                          char (&lds_v)[AttnLds<MODE, HD>::NK],
                                          int (&vs_only)[AttnLds<MODE, HD>::NONLY], int (&vs_wsum)[4], int &vs_bad,
                                          int &lds_redo) {
    static_assert(HD == 256 || HD == 128 || HD == 64, "head_dim 64, 128 or 256");
    static_assert(HD <= 128 || !(MODE == MODE_VS || MODE == MODE_BS), "the list walks are built for head_dim <= 128");
    constexpr int ROW_BYTES = HD * 2;                       // one token row of K / V / Q / O
    constexpr int KS = HD / 16;                             // k-steps of S^T = K.Q^T
    constexpr int NDB = HD / 32;                            // 32-row blocks of O^T
    constexpr int NCH = ROW_BYTES / 16;                     // 16-byte chunks per row
    constexpr int RPI = 64 / NCH;                           // tile rows one copy instruction fills (64 lanes x 16 B)
    // LDS chunk permutations (conflict-free ds_read_b128 of 32 K rows / transpose reads of 4 V rows):
    // 256-byte rows: K chunk ^ row%16, V chunk ^ 4*(row%4); 128-byte rows (two rows per bank sweep):
    // K chunk ^ (row/2)%8, V chunk ^ 4*((row/2)%2)
    auto swz_k = [](int row) { return HD >= 128 ? (row & 15) : ((row >> 1) & 7); };
    auto swz_v = [](int row) { return HD >= 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); };
    constexpr int NT = 2 * NTHREADS;                        // threads per workgroup
    constexpr int CROWS = 16;                               // tile rows copied by one wave (shared tile)
    // VSP: the paired walk of two block lists -- the vertical-slash block lists, or the block-sparse
    // lists (block numbers, i.e. key starts / 64; no columns)
    constexpr bool VSP = MODE == MODE_VS || MODE == MODE_BS;
    constexpr int LIST_SCALE = MODE == MODE_BS ? BN : 1;     // list entry -> first key of the block
    constexpr int TILE_BYTES = BN * ROW_BYTES;
    constexpr int VS_PAIR_MAX = TILE_BYTES / 8;             // both staged lists fit the second K tile
    // paired list walks (vertical-slash, block-sparse): a second K and V tile (row block B's buffers in the steps in which each
    // row block has a tile of its own); before that, the second K tile stages the two block lists and
    // the second V tile holds their merge
    char *const lds_k1 = lds_k + (VSP ? TILE_BYTES : 0);
    char *const lds_v1 = lds_v + (VSP ? TILE_BYTES : 0);

    // ---- which (batch, head, row block): XCD-aware remap --------------------
    // Consecutive workgroup ids are dealt round-robin to the 8 XCDs; give each
    // XCD one contiguous range of the logical order (batch, kv head, row block,
    // query head inside the GQA group) so that the row blocks and the query
    // heads that share K/V also share an L2.
    // (32-bit arithmetic: the launcher refuses grids beyond 2^31 workgroups, and 64-bit divisions of
    // wave-uniform values cost a thousand scalar instructions per workgroup here)
    const unsigned total_wg = (unsigned)p.total_wg;
    const unsigned per_xcd = (total_wg + 7u) >> 3;
    const unsigned logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total_wg) return false;
    const int group = p.hq / p.hk;
    unsigned rest = logical;
    const int hin = (int)(rest % (unsigned)group); rest /= (unsigned)group;
    // Dense causal work grows with the row block, so the heavy (late) blocks go first.  The sparse
    // modes have near-constant work per row block once the context is long and then measure 1 %
    // faster in ascending order; up to 64K tokens their early row blocks are still growing and the
    // descending order wins for vertical-slash lists (+4 % at 16K, +1.7 % at 32K): the launcher picks.
    const int rows_wg = (p.rows + 1) >> 1;                           // row-block pairs per (batch, head)
    const int mi = (int)(rest % (unsigned)rows_wg); rest /= (unsigned)rows_wg;
    const int mslot = p.descending ? rows_wg - 1 - mi : mi;
    int hkv, b, h, hs;                               // hs: head position in the index tensors
    if (p.head_list) {
        // the selected heads in chunks of `group` consecutive list entries take the place of the kv
        // groups: neighbours in the (ascending) list mostly share a kv head
        const int nch = (p.index_heads + group - 1) / group;
        const int ch = (int)(rest % (unsigned)nch);
        b = (int)(rest / (unsigned)nch);
        hs = ch * group + hin;
        if (hs >= p.index_heads) return false;       // padding of the last chunk (workgroup-uniform)
        h = as_const(p.head_list)[hs];
        hkv = h / group;
    } else {
        hkv = (int)(rest % (unsigned)p.hk);
        b = (int)(rest / (unsigned)p.hk);
        h = hkv * group + hin;
        hs = h;
    }

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave_wg = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keep it in an SGPR
    const int half = wave_wg >> 1;                                   // which row block of the pair
    const int wave = wave_wg & 1;                                    // wave inside the row block
    const int m = 2 * mslot + half;
    const int mA = 2 * mslot, mB = min(mA + 1, p.rows - 1);
    const int l32 = lane & 31;
    const int g = lane >> 5;

    const int seqlen = p.seqlens ? min(p.seqlens[b], p.n) : p.n;
    const int row0 = m * BM;
    const int qrow = row0 + wave * 32 + l32;          // this lane's query row
    char *o_base = p.o + ((long long)b * p.os[0] + (long long)h * p.os[1]) * 2;

    // row block past the sequence: zeros (16 B per lane-step); the other
    // half may still have work, so this half stays for the copies and barriers without tiles
    const bool have_rows = m < p.rows && row0 < seqlen;
    if (!have_rows) {
        if (m < p.rows)
            for (int i = tid & (NTHREADS - 1); i < BM * NCH; i += NTHREADS) {
                int r = row0 + i / NCH;
                if (r < p.n) *reinterpret_cast<u32x4_t *>(o_base + (long long)r * p.os[2] * 2 + (i % NCH) * 16) = u32x4_t{0u, 0u, 0u, 0u};
            }
        if (mA * BM >= seqlen) return false;            // (workgroup-uniform: both halves are past)
    }

    const char *q_base = p.q + ((long long)b * p.qs[0] + (long long)h * p.qs[1]) * 2;
    const char *k_base = p.k + ((long long)b * p.ks[0] + (long long)hkv * p.ks[1]) * 2;
    const char *v_base = p.v + ((long long)b * p.vs[0] + (long long)hkv * p.vs[1]) * 2;
    const long long k_row = p.ks[2] * 2, v_row = p.vs[2] * 2;
    const long long ridx = ((long long)b * p.index_heads + hs) * p.rows + min(m, p.rows - 1);

    constexpr bool every_max = EVERY_MAX;
    // log2-domain scale of this lane's query row: one value per launch, except for the dense rows of a
    // tri-shape launch (the reference scales its A-shape rows by the padded head_dim and its last
    // rows by the unpadded one, streaming_kernel.py:575 against :826)
    float sc_l2 = p.scale_log2;
    if constexpr (MODE == MODE_ASHAPE) sc_l2 = qrow >= p.dense_from ? p.scale_log2_dense : p.scale_log2;
    // ---- Q fragments (B operand of S^T): row qrow, d = 16*ks + 8*g + 0..7 ----
    Frag qf[KS];
    {
        const bool ok = qrow < seqlen;
        const char *qp = q_base + (long long)(ok ? qrow : min(row0, seqlen - 1)) * p.qs[2] * 2 + g * 16;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qf[ks].u = *reinterpret_cast<const u32x4_t *>(qp + ks * 32);
            if (!ok) qf[ks].u = u32x4_t{0u, 0u, 0u, 0u};
        }
    }

    int nblk = 0;
    // Paired list walks (vertical-slash block lists, block-sparse lists scaled to key starts): the
    // block lists of the two row blocks (ascending key starts; vertical-slash lists of
    // neighbouring row blocks are each other's translate by 64 keys wherever no entry is clipped, so
    // runs of blocks share all but their ends) are split ONCE, by all 256 threads, before the tile
    // loop: both lists are staged in LDS, every entry looks itself up in the other list by binary
    // search, and a workgroup prefix sum over the hits places it either in the list of COMMON
    // entries (tiles that both row blocks visit: copied once by four waves, one LDS word per step)
    // or in its row block's list of entries the other one lacks (run ends).  The walk is then
    //   common tiles, both halves computing;
    //   split steps: every half visits its own leftover tiles -- the entries the other list lacks,
    //   then its gathered column tiles -- with the K/V buffers of its own half,
    // i.e. exactly max(tiles of A, tiles of B) steps, never more than the longer list alone.
    // Lists that are too long for LDS or not strictly ascending are not split: each half then walks
    // its whole list in split steps (still in lockstep with its neighbour, which is what keeps the
    // neighbour's tiles in L2 when the lists are long and scattered).
    // where the block lists live: [batch, heads, list_rows, list_w]
    [[maybe_unused]] const int *const list_base = MODE == MODE_BS ? p.bidx : p.bo;
    [[maybe_unused]] const int list_w = MODE == MODE_BS ? p.max_blocks : p.nnz_s;
    [[maybe_unused]] const int list_rows = MODE == MODE_BS ? p.bidx_rows : p.rows;
    [[maybe_unused]] int vs_na = 0, vs_nb = 0, vs_cca = 0, vs_ccb = 0, vs_nc = 0;
    [[maybe_unused]] bool vs_merged = false;
    [[maybe_unused]] long long vs_ra = 0, vs_rb = 0;
    if constexpr (VSP) {
        const bool b_exists = 2 * mslot + 1 < p.rows && (2 * mslot + 1) * BM < seqlen;
        vs_ra = ((long long)b * p.index_heads + hs) * list_rows + mA;
        vs_rb = b_exists ? vs_ra + 1 : vs_ra;
        if constexpr (MODE == MODE_BS) {
            // row block m visits the first min(m + 1, max_blocks) entries of its row; no columns
            vs_na = min(mA + 1, p.max_blocks);
            vs_nb = b_exists ? min(mA + 2, p.max_blocks) : 0;
        } else {
            vs_na = max(0, min(as_const(p.bc)[vs_ra], p.nnz_s));
            vs_cca = max(0, min(as_const(p.cc)[vs_ra], p.nnz_v));
            vs_nb = b_exists ? max(0, min(as_const(p.bc)[vs_rb], p.nnz_s)) : 0;
            vs_ccb = b_exists ? max(0, min(as_const(p.cc)[vs_rb], p.nnz_v)) : 0;
        }
        if (vs_na <= VS_PAIR_MAX && vs_nb <= VS_PAIR_MAX && vs_na > 0 && vs_nb > 0) {
            int *rawA = reinterpret_cast<int *>(lds_k1), *rawB = rawA + VS_PAIR_MAX;
            int *common = reinterpret_cast<int *>(lds_v1);
            const int *ga = list_base + vs_ra * list_w, *gb = list_base + vs_rb * list_w;
            if (tid == 0) vs_bad = 0;
            for (int i = tid; i < vs_na; i += NT) rawA[i] = ga[i] * LIST_SCALE;
            for (int i = tid; i < vs_nb; i += NT) rawB[i] = gb[i] * LIST_SCALE;
            __syncthreads();
            bool bad = false;                              // the look-ups need strictly ascending lists
            for (int i = tid; i + 1 < vs_na; i += NT) bad |= rawA[i + 1] <= rawA[i];
            for (int i = tid; i + 1 < vs_nb; i += NT) bad |= rawB[i + 1] <= rawB[i];
            if (__any(bad) && lane == 0) vs_bad = 1;
            __syncthreads();
            if (!vs_bad) {                                 // (workgroup-uniform)
                const unsigned long long lt = (1ull << lane) - 1ull;
                // entry i of `mine` goes to common[#hits before i] when `other` holds it too (first
                // pass only), else to only[i - #hits before i]; -> number of hits
                auto pass = [&](const int *mine, int nmine, const int *other, int nother, int *only, bool write_common) {
                    int carry = 0;
                    for (int base = 0; base < nmine; base += NT) {        // uniform trip count
                        const int i = base + tid;
                        const bool valid = i < nmine;
                        const int x = valid ? mine[i] : 0;
                        int lo = 0, hi = nother;                           // first entry of `other` >= x
                        while (lo < hi) {
                            const int mid = (lo + hi) >> 1;
                            if (other[mid] < x) lo = mid + 1; else hi = mid;
                        }
                        const bool eq = valid && lo < nother && other[lo] == x;
                        const unsigned long long bal = __ballot(eq);
                        if (lane == 0) vs_wsum[wave_wg] = __builtin_popcountll(bal);
                        __syncthreads();
                        int pre = carry, tot = 0;
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            const int c = vs_wsum[w];
                            pre += w < wave_wg ? c : 0;
                            tot += c;
                        }
                        pre += __builtin_popcountll(bal & lt);
                        if (valid) {
                            if (eq) { if (write_common) common[pre] = x; }
                            else if (i - pre < VS_ONLY_MAX) only[i - pre] = x;
                        }
                        carry += tot;
                        __syncthreads();
                    }
                    return carry;
                };
                vs_nc = pass(rawA, vs_na, rawB, vs_nb, vs_only, true);
                pass(rawB, vs_nb, rawA, vs_na, vs_only + VS_ONLY_MAX, false);
                // (the last barrier of the passes also orders these LDS lists before their readers)
                vs_merged = vs_nc > 0 && vs_na - vs_nc <= VS_ONLY_MAX && vs_nb - vs_nc <= VS_ONLY_MAX;
                if (!vs_merged) vs_nc = 0;
            }
        }
    }
    int ntiles = 0;
    // paired vertical-slash: vs_nc common steps, then the split steps: per half its leftover block
    // entries (from LDS when the lists were split, else its whole list from global memory) and its
    // gathered column tiles.  The barriers are the workgroup's: both halves make max(A, B) split
    // steps and a half without a tile only keeps the barriers.
    [[maybe_unused]] int vs_nb_mine = 0, vs_cc_mine = 0, vs_nt_mine = 0;
    if constexpr (VSP) {
        const int nb_a = vs_na - vs_nc, nb_b = vs_nb - vs_nc;
        const int nt_a = nb_a + ((vs_cca + BN - 1) >> 6), nt_b = nb_b + ((vs_ccb + BN - 1) >> 6);
        vs_nb_mine = half ? nb_b : nb_a;
        vs_cc_mine = half ? vs_ccb : vs_cca;
        vs_nt_mine = have_rows ? (half ? nt_b : nt_a) : 0;
        ntiles = vs_nc + max(nt_a, nt_b);
    }
    else
        ntiles = pair_tile_count<MODE>(p, mA, mB, nblk);
    auto more_tiles = [&](int it) -> bool { return it < ntiles; };   // is there a tile number `it` ?
    // paired vertical-slash: entry it+1 of the common list sits in a scalar when step `it` starts; the
    // LDS read of entry it+2 is issued at the top of step `it` (no tile copy is in flight there: the
    // list shares an LDS object with the V tiles and must not wait for one) and turns into the next
    // scalar at the end of the step, its latency hidden behind the tile's work
    [[maybe_unused]] int vs_entry = 0, vs_pref = 0;
    // this row block's own list in global memory (walked directly when the lists were not split)
    [[maybe_unused]] const cint_ptr sp_list = as_const(list_base) + (((long long)b * p.index_heads + hs) * list_rows + min(m, p.rows - 1)) * list_w;
    auto vs_list = [&](int i) -> int { return reinterpret_cast<const int *>(lds_v1)[min(i, 2 * VS_PAIR_MAX - 1)]; };
    auto tile_of = [&](int it) -> Tile {      // called with it = 0, 1, 2, ... in order
        if constexpr (VSP) {
            Tile t;
            t.gathered = 0;
            t.nvalid = BN;
            if (it < vs_nc) {
                t.split = 0;
                t.on_a = t.on_b = 1;
                t.start = vs_entry;                        // common entry `it`, fetched a step ahead
            } else {
                const int j = it - vs_nc;
                t.split = 1;
                t.on_a = t.on_b = j < vs_nt_mine;          // (this half's own flag)
                t.start = 0;
                if (j < vs_nb_mine) {
                    if (vs_merged) t.start = __builtin_amdgcn_readfirstlane(vs_only[half * VS_ONLY_MAX + j]);
                    else t.start = sp_list[j] * LIST_SCALE;
                } else if (j < vs_nt_mine) {
                    t.gathered = 1;
                    t.start = (j - vs_nb_mine) * BN;
                    t.nvalid = min(BN, vs_cc_mine - t.start);
                }
            }
            return t;
        } else {
            Tile t;
            t.gathered = 0;
            t.nvalid = BN;
            t.on_a = t.on_b = 1;
            t.start = pair_tile_start<MODE>(p, mA, mB, nblk, it);
            return t;
        }
    };

    // ---- global -> LDS copies without a register round trip (global_load_lds_dwordx4): every lane
    // fetches 16 bytes from its own global address and the wave's 64 x 16 B land contiguously in
    // LDS at a wave-uniform base (lane i -> base + 16*i), i.e. one instruction fills 4 tile rows;
    // wave w owns rows 32*w .. 32*w+31 (8 instructions per matrix; 16 rows, 4 instructions when paired).  The 16-byte chunks of a row
    // are permuted for conflict-free reads (K: chunk ^ row%16, V: chunk ^ 4*(row%4)); the
    // permutation is applied on the global side: lane (row, c') loads global chunk c' ^ swz(row).
    // Rows that do not exist (past seqlen, or padding of a gathered tile) are read from a clamped,
    // valid address: their scores are masked to -inf, so their probabilities are exactly 0.
    const int cp_r = lane / NCH;                 // row inside the group of RPI rows one instruction fills
    const int cp_c = lane % NCH;                 // LDS chunk
    // gathered tiles: lane l holds the token id of tile row l (one load per lane, issued an
    // iteration ahead); the copy fetches the ids of its own rows with wave shuffles
    // (per-lane offsets of the buffer-form copies: the K permutation repeats every 16 rows, i.e. every
    // KL copy instructions, the V permutation every 4 rows: every VL instructions)
    constexpr int KL = RPI >= 4 ? 4 : 16 / RPI, VL = RPI >= 4 ? 1 : 4 / RPI;
    int k_lane[KL], v_lane[VL];
#pragma unroll
    for (int jj = 0; jj < KL; ++jj) k_lane[jj] = cp_r * (int)k_row + ((cp_c ^ swz_k(RPI * jj + cp_r)) << 4);
#pragma unroll
    for (int jj = 0; jj < VL; ++jj) v_lane[jj] = cp_r * (int)v_row + ((cp_c ^ swz_v(RPI * jj + cp_r)) << 4);
    auto gather_ids = [&](const Tile &t) -> int {
        if (MODE == MODE_VS && t.gathered) return p.ci[ridx * p.nnz_v + t.start + min(lane, max(t.nvalid, 1) - 1)];
        return 0;
    };
    // rows_c: tile rows copied by one wave (16: the four waves of a pair share the tile, 32: the
    // two waves of a row block copy it); wsel: which part of the tile this wave copies
    auto copy_rows = [&](const Tile &t, const char *base, long long rowstride, auto is_v_c, int idv,
                         char *ldsbuf, auto rows_c, const int wsel) {
        constexpr bool is_v = decltype(is_v_c)::value;
        constexpr int CROWS = decltype(rows_c)::value;
        const bool gathered = MODE == MODE_VS && t.gathered;
        if (!gathered && t.start >= 0 && t.start + BN <= seqlen) {
            // buffer form: descriptor of the 64 tile rows (scalar), one of five per-lane offsets (the V
            // swizzle does not depend on j, the K swizzle only on j % 4) and a scalar row offset
            const char *tb = base + (long long)t.start * rowstride;      // wave-uniform
            const __amdgpu_buffer_rsrc_t srd = __builtin_amdgcn_make_buffer_rsrc((void *)tb, 0, BN * (int)rowstride, 0x00020000);
            // first row offset and step of this wave's part; in the paired vertical-slash kernel (two
            // copy shapes, K and V strides) they are made opaque so that the per-copy offsets are formed
            // with one scalar add each instead of living in two dozen loop-invariant scalar registers
            int soff0 = CROWS * wsel * (int)rowstride, sstep = RPI * (int)rowstride;
            int lds0 = (int)(unsigned)(unsigned long long)(__attribute__((address_space(3))) char *)ldsbuf + CROWS * wsel * ROW_BYTES;
            if constexpr (VSP) asm volatile("" : "+s"(soff0), "+s"(sstep), "+s"(lds0));
#pragma unroll
            for (int j = 0; j < CROWS / RPI; ++j) {
                const int voff = is_v ? v_lane[j & (VL - 1)] : k_lane[j & (KL - 1)];
                __builtin_amdgcn_raw_ptr_buffer_load_lds(srd, (__attribute__((address_space(3))) void *)(unsigned long long)(unsigned)(lds0 + RPI * j * ROW_BYTES),
                                                         16, voff, soff0 + j * sstep, 0, 0);
            }
            return;
        }
        // three straight-line variants (a per-row select would turn into sixteen tiny branches).
        // The two rare ones recompute their per-lane rows and chunks on the spot (the empty asm
        // keeps the compiler from hoisting a dozen loop-invariant registers out of the tile loop).
        int cp_r = lane / NCH, cp_c = lane % NCH;
        asm volatile("" : "+v"(cp_r), "+v"(cp_c));
        if (gathered) {
#pragma unroll
            for (int j = 0; j < CROWS / RPI; ++j) {
                const int r = CROWS * wsel + RPI * j + cp_r;        // tile row
                const int tk = max(0, min(__shfl(idv, r), seqlen - 1));
                const int c = is_v ? (cp_c ^ swz_v(r)) : (cp_c ^ swz_k(r));
                const char *gp = base + tk * rowstride + c * 16;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                                 (__attribute__((address_space(3))) void *)(ldsbuf + (CROWS * wsel + RPI * j) * ROW_BYTES),
                                                 16, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < CROWS / RPI; ++j) {
            const int r = CROWS * wsel + RPI * j + cp_r;
            const int tk = max(0, min(t.start + r, seqlen - 1));
            const int c = is_v ? (cp_c ^ swz_v(r)) : (cp_c ^ swz_k(r));
            const char *gp = base + tk * rowstride + c * 16;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                             (__attribute__((address_space(3))) void *)(ldsbuf + (CROWS * wsel + RPI * j) * ROW_BYTES),
                                             16, 0, 0);
        }
    };
    auto copy_tile = [&](const Tile &t, const char *base, long long rowstride, auto is_v_c, int idv, char *ldsbuf) {
        if constexpr (VSP) {
            if (t.split) {
                if (t.on_a) copy_rows(t, base, rowstride, is_v_c, idv, ldsbuf + half * TILE_BYTES, std::integral_constant<int, 32>{}, wave);
                return;
            }
        }
        copy_rows(t, base, rowstride, is_v_c, idv, ldsbuf, std::integral_constant<int, CROWS>{}, wave_wg);
    };

    // ---- accumulators -------------------------------------------------------
    f32x16_t oacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m_i = -INFINITY;   // running max (log2 domain, scaled)
    int sm_steps = 0;        // tiles this wave has put through the softmax
    int sm_prev_start = -(1 << 30);   // first key of the previous one (wave-uniform)
    bool sm_prev_masked = false;      // ... and whether it was a boundary tile (some rows may have seen none of its keys)
    float l_i = 0.f;         // this lane's share of the running sum

    // LDS read addresses that do not depend on the tile
    // K: row 32*blk + l32, logical chunk 2*ks + g -> physical chunk ^ (row % 16)
    int k_rd_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_rd_off[ks] = l32 * ROW_BYTES + (((2 * ks + g) ^ swz_k(l32)) << 4);
    // V transpose read: row = 16*s + 8*jj + 4*g + rsub (row % 4 == rsub), logical chunk
    // 4*db + vc -> physical 4*(db ^ rsub) + vc
    const int v_rd_rsub = (lane & 15) >> 2;
    const int v_rd_vc = (((lane >> 4) & 1) << 1) + ((lane & 3) >> 1);
    int v_rd_off[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
        v_rd_off[db] = (4 * g + v_rd_rsub) * ROW_BYTES + ((((db << 2) + v_rd_vc) ^ swz_v(v_rd_rsub)) << 4) + ((lane & 1) << 3);

    // ---- S^T = K . Q^T for this wave's 32 query rows; K tile in kbuf.
    auto qk_block = [&](const char *kbuf, f32x16_t &s0, f32x16_t &s1) {
        Frag a0[KS], a1[KS];
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int r = 0; r < 16; ++r) { s0[r] = 0.f; s1[r] = 0.f; }
        // K fragments are fetched QK_AHEAD k-steps before the MFMAs that consume them; the
        // scheduling fences keep the compiler from sinking the reads back to their use
#pragma unroll
        for (int ks = 0; ks < QK_AHEAD; ++ks) {
            a0[ks].u = *reinterpret_cast<const u32x4_t *>(kbuf + k_rd_off[ks]);
            a1[ks].u = *reinterpret_cast<const u32x4_t *>(kbuf + k_rd_off[ks] + 32 * ROW_BYTES);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + QK_AHEAD < KS) {
                a0[ks + QK_AHEAD].u = *reinterpret_cast<const u32x4_t *>(kbuf + k_rd_off[ks + QK_AHEAD]);
                a1[ks + QK_AHEAD].u = *reinterpret_cast<const u32x4_t *>(kbuf + k_rd_off[ks + QK_AHEAD] + 32 * ROW_BYTES);
            }
            s0 = Mma<T>::mfma(frag_as<T>(a0[ks]), frag_as<T>(qf[ks]), s0);
            s1 = Mma<T>::mfma(frag_as<T>(a1[ks]), frag_as<T>(qf[ks]), s1);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
    };

    // ---- mask, V^T fragment reads, online softmax, O^T += V^T . P^T
    auto sm_pv_block = [&](const Tile &cur, const char *vbuf, f32x16_t &s0, f32x16_t &s1) {
        // (head_dim 256: the 64 registers of a whole tile's V^T fragments do not fit next to O^T and Q;
        // that form reads the fragments of one key group at a time, right before their MFMAs)
        constexpr bool VF_AHEAD = HD <= 128;
        Frag vf[VF_AHEAD ? 4 : 1][NDB];
        // element (blk, r) of this lane is tile-local key tk = tkc + 4*g with the compile-time
        // part tkc = 32*blk + 8*(r/4) + r%4.  keep <=> tk <= hi && (tk > wlo || tk < slim).
        bool need_mask;
        const int wrow_lo = row0 + wave * 32, wrow_hi = wrow_lo + 31;
        int hi, wlo = -1, slim = 0;      // per-lane bounds on tkc (4*g already subtracted)
        if (MODE == MODE_VS && cur.gathered) {
            need_mask = cur.nvalid < BN;
            hi = cur.nvalid - 1 - 4 * g;
        } else {
            hi = min(qrow, seqlen - 1) - cur.start - 4 * g;
            if constexpr (MODE == MODE_ASHAPE) {
                const int c_lo = cur.start, c_hi = cur.start + BN - 1;
                const bool causal_ok = c_hi <= wrow_lo && c_hi < seqlen;
                const bool in_window = (wrow_hi - c_lo) < p.n_local;
                const bool in_sink = c_hi < p.n_init;
                const bool all_dense = wrow_lo >= p.dense_from, none_dense = wrow_hi < p.dense_from;
                need_mask = all_dense ? !causal_ok : (none_dense ? !(causal_ok && (in_window || in_sink)) : true);
                wlo = qrow >= p.dense_from ? -(1 << 30) : qrow - cur.start - p.n_local - 4 * g;
                slim = p.n_init - cur.start - 4 * g;
            } else {
                // (a list entry below zero is no key at all: the reference would read out of bounds)
                need_mask = (cur.start + BN - 1 > wrow_lo) || (cur.start + BN > seqlen) || cur.start < 0;
                wlo = -cur.start - 4 * g - 1;
            }
        }
        if (need_mask) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int tkc = 8 * (r >> 2) + (r & 3);
                bool k0 = tkc <= hi, k1 = (tkc + 32) <= hi;
                if constexpr (MODE == MODE_ASHAPE) {
                    k0 = k0 & ((tkc > wlo) | (tkc < slim));
                    k1 = k1 & (((tkc + 32) > wlo) | ((tkc + 32) < slim));
                } else if constexpr (MODE == MODE_VS || MODE == MODE_BS) {
                    k0 = k0 & (tkc > wlo);
                    k1 = k1 & ((tkc + 32) > wlo);
                }
                s0[r] = k0 ? s0[r] : -INFINITY;
                s1[r] = k1 ? s1[r] : -INFINITY;
            }
        }

        {
        // All V^T fragments of the tile are read here, in one scheduling region with the row-max
        // chain: the PV block below is bound by its vector instructions, so every LDS read moved out
        // of it shortens it (+3 % for the 24 reads that used to sit between its MFMAs), and the reads
        // fill the dependency gaps of the max chain (+0.7 % over reading them before the K copy).
        if constexpr (VF_AHEAD) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
                vf[s][db].s4[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) short4_t *)(vbuf + v_rd_off[db] + (16 * s + 8 * jj) * ROW_BYTES));
        }
        }
        // ---- online softmax (exp2 domain) -------------------------------------
        // The reference maximum m_i of a row only has to keep exp2 inside the range of fp32 (bf16 has the
        // same exponent range), so most tiles take it as it is: no row maximum, no rescale factor.  It
        // is recomputed where a row has none yet (first tile, fully masked tiles), every MAX_PERIOD steps,
        // and for every tile of a walk that is run again because a row sum left the safe range (which
        // takes a row whose scores rise by more than a hundred powers of two within MAX_PERIOD tiles).
        float alpha = 1.0f, m_use = m_i;
        // ... and wherever the walk jumps (the first tile of a run of blocks, the first window tile after
        // the sink tiles, every gathered tile): scores move smoothly along a run of neighbouring keys
        // but may differ by any amount across a jump.  A tile after a masked one counts as a jump too:
        // a row that saw none of the masked tile's keys (the window starts a tile later for the last
        // rows of a row block) still carries the maximum from before the jump.
        const bool jump = (MODE == MODE_VS && cur.gathered) || cur.start != sm_prev_start + BN || sm_prev_masked;
        sm_prev_start = cur.start;
        sm_prev_masked = need_mask;
        if (every_max || ((sm_steps++ & (MAX_PERIOD - 1)) == 0) || jump || __any(m_i == -INFINITY)) {
        float mx;
        {
            // four independent chains of three-operand maxima (8 scores each)
            float m4[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                m4[c] = fmaxf(fmaxf(s0[4 * c], s1[4 * c]), s0[4 * c + 1]);
                m4[c] = fmaxf(fmaxf(m4[c], s1[4 * c + 1]), s0[4 * c + 2]);
                m4[c] = fmaxf(fmaxf(m4[c], s1[4 * c + 2]), s0[4 * c + 3]);
                m4[c] = fmaxf(m4[c], s1[4 * c + 3]);
            }
            mx = fmaxf(fmaxf(fmaxf(m4[0], m4[1]), m4[2]), m4[3]);
        }
        { const unsigned u = __float_as_uint(mx); auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false); mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])); }
        const float cand = mx * sc_l2;
        // lazy: raised only when a tile exceeds it by more than LAZY_MAX powers of two (probabilities of
        // f16 operands must stay inside the f16 range: 2^8 leaves room for the row sums)
        constexpr float LAZY_MAX = std::is_same<T, __bf16>::value ? LAZY_MAX_BF16 : 8.0f;
        const bool grow = cand > m_i + LAZY_MAX;
        const float m_new = grow ? cand : m_i;
        m_use = (m_new == -INFINITY) ? 0.f : m_new;
        // `alpha` is the SQUARE ROOT of the rescale factor and is applied twice.  With a maximum that
        // is looked at only now and then, the sums accumulated under the old one may be as large as
        // 2^127 (probabilities far above 1 that have not overflowed), so a factor below 2^-126 does
        // not mean that they are negligible -- and exp2 of such an exponent is flushed to zero.  Half
        // the exponent twice is exact down to 2^-252, beyond which nothing finite is left of them.
        alpha = grow ? __builtin_amdgcn_exp2f(fmaxf(0.5f * (m_i - m_use), -126.0f)) : 1.0f;
        m_i = m_new;
        }
        float psum = 0.f;
        Frag pfr[4];
        // probabilities of key group q (16 keys): registers 8*(q%2) .. +7 of s0 (q < 2) / s1
        auto probs = [&](int q) {
            const f32x16_t &sx = q < 2 ? s0 : s1;
            float pv[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) pv[r] = __builtin_amdgcn_exp2f(fmaf(sx[8 * (q & 1) + r], sc_l2, -m_use));
            cvt8<T>(&pv[0], pfr[q]);
            psum = pair_sum<T>(pfr[q], psum);
        };
        probs(0);
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int i = 0; i < NDB; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[i][r] = (oacc[i][r] * alpha) * alpha;
        }

        __builtin_amdgcn_s_setprio(2);
        // ---- O^T += V^T . P^T; the exponentials of key group q+1 run under the MFMAs of group q ----
        {
            probs(1);
            probs(2);
            probs(3);
            l_i = (l_i * alpha) * alpha + psum;
            if constexpr (VF_AHEAD) {
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int db = 0; db < NDB; ++db)
                    oacc[db] = Mma<T>::mfma(frag_as<T>(vf[s][db]), frag_as<T>(pfr[s]), oacc[db]);
            // the softmax instructions of key groups 1..3 are spread behind the MFMAs of groups 0..2
#pragma unroll
            for (int i = 0; i < 4 * NDB; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (i < 3 * NDB) __builtin_amdgcn_sched_group_barrier(VALU_MASK, VALU_PER_MFMA * 4 / NDB, 0);
            }
            } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj)
                        vf[0][db].s4[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) short4_t *)(vbuf + v_rd_off[db] + (16 * s + 8 * jj) * ROW_BYTES));
#pragma unroll
                for (int db = 0; db < NDB; ++db)
                    oacc[db] = Mma<T>::mfma(frag_as<T>(vf[0][db]), frag_as<T>(pfr[s]), oacc[db]);
            }
            }
        }
        __builtin_amdgcn_s_setprio(0);
    };

    // Single K and V buffers, two barriers per tile:
    //   [own K(it) copies landed] barrier B1 (also: every wave is done with V(it-1))
    //   issue V(it) copy; fetch gathered ids of tile it+1; S^T = K.Q^T
    //   [own V(it) copies landed] barrier B2 (also: every wave is done with K(it))
    //   issue K(it+1) copy; softmax; O^T += V^T.P^T
    Tile cur, nxt;
    int gt_cur = 0, gt_nxt = 0;
    [[maybe_unused]] bool vs_shifted = false;
    bool have_cur = more_tiles(0);
    if (have_cur) {
        if constexpr (VSP) vs_entry = __builtin_amdgcn_readfirstlane(vs_list(0));
        cur = tile_of(0);
        if constexpr (VSP) vs_entry = __builtin_amdgcn_readfirstlane(vs_list(1));
        gt_cur = gather_ids(cur);
        copy_tile(cur, k_base, k_row, std::false_type{}, gt_cur, lds_k);
    }

    // One step of the walk, in three forms (the last two for the paired list walks only):
    // general (kind 0) -- any tile, any successor, every mode;
    // COMMON (kind 1) -- this tile and the next one are both on the list of common entries: shared,
    // contiguous, never gathered;
    // SPLIT (kind 2) -- this step and the next one are both split steps in which each row block
    // visits a block entry of its own, fetched a step ahead: a leftover from the split lists in LDS
    // or, when the lists were not split, an entry of its list in global memory (kind 2).
    // In the two special forms everything that deals with the other cases drops out of the
    // instruction stream (the general form costs about 1.7 times a COMMON step).
    [[maybe_unused]] int sp_entry = 0;
    auto step = [&](const int it, auto kind_c) {
        constexpr int KIND = decltype(kind_c)::value;
        constexpr bool COMMON = KIND == 1, SPLIT = KIND == 2;
        __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0): this wave's part of K(it) is in LDS
        __syncthreads();
        bool have_nxt;
        if constexpr (COMMON) {
            vs_pref = vs_list(it + 2);
            have_nxt = true;
            nxt.gathered = 0; nxt.nvalid = BN; nxt.on_a = nxt.on_b = 1; nxt.split = 0;
            nxt.start = vs_entry;
            gt_nxt = 0;
            cur.gathered = 0; cur.nvalid = BN; cur.on_a = cur.on_b = 1; cur.split = 0;
            copy_rows(cur, v_base, v_row, std::true_type{}, 0, lds_v, std::integral_constant<int, CROWS>{}, wave_wg);
        } else if constexpr (SPLIT) {
            const int j = it - vs_nc;                      // this step's position in the leftover lists
            if (vs_merged) vs_pref = vs_only[half * VS_ONLY_MAX + min(j + 2, VS_ONLY_MAX - 1)];
            else vs_pref = sp_list[min(j + 2, list_w - 1)] * LIST_SCALE;
            have_nxt = true;
            nxt.gathered = 0; nxt.nvalid = BN; nxt.on_a = nxt.on_b = 1; nxt.split = 1;
            nxt.start = sp_entry;
            gt_nxt = 0;
            cur.gathered = 0; cur.nvalid = BN; cur.on_a = cur.on_b = 1; cur.split = 1;
            copy_rows(cur, v_base, v_row, std::true_type{}, 0, lds_v + half * TILE_BYTES, std::integral_constant<int, 32>{}, wave);
        } else if constexpr (VSP) {
            // the merged list shares an LDS object with the V tiles: its entry is read while no copy
            // is in flight, so that the read never waits for one
            vs_pref = vs_list(it + 2);
            have_nxt = more_tiles(it + 1);
            nxt = have_nxt ? tile_of(it + 1) : cur;
            gt_nxt = gather_ids(nxt);
            copy_tile(cur, v_base, v_row, std::true_type{}, gt_cur, lds_v);
            if (cur.split && !vs_shifted) {
                // first split step: row block B reads the second tiles from here on (the LDS read
                // offsets move in place, once)
                vs_shifted = true;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) k_rd_off[ks] += half * TILE_BYTES;
#pragma unroll
                for (int db = 0; db < NDB; ++db) v_rd_off[db] += half * TILE_BYTES;
            }
        } else {
            copy_tile(cur, v_base, v_row, std::true_type{}, gt_cur, lds_v);
            have_nxt = more_tiles(it + 1);
            nxt = have_nxt ? tile_of(it + 1) : cur;
            gt_nxt = gather_ids(nxt);
        }

        // is this tile on the list of this wave's row block ?
        bool active = true;
        if constexpr (COMMON || SPLIT) active = have_rows;
        else if constexpr (VSP) active = have_rows && (half ? cur.on_b : cur.on_a);   // (split steps: on_a == on_b == own flag)
        else active = have_rows && tile_on_list<MODE>(p, m, cur.start);
        f32x16_t s0, s1;
        if (active) qk_block(lds_k, s0, s1);
        __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0): this wave's part of V(it) is in LDS
        __syncthreads();
        if constexpr (COMMON) copy_rows(nxt, k_base, k_row, std::false_type{}, 0, lds_k, std::integral_constant<int, CROWS>{}, wave_wg);
        else if constexpr (SPLIT) copy_rows(nxt, k_base, k_row, std::false_type{}, 0, lds_k + half * TILE_BYTES, std::integral_constant<int, 32>{}, wave);
        else if (have_nxt) copy_tile(nxt, k_base, k_row, std::false_type{}, gt_nxt, lds_k);
        if (active) sm_pv_block(cur, lds_v, s0, s1);
        if constexpr (SPLIT) sp_entry = __builtin_amdgcn_readfirstlane(vs_pref);
        else if constexpr (VSP) vs_entry = __builtin_amdgcn_readfirstlane(vs_pref);
        cur = nxt;
        gt_cur = gt_nxt;
        have_cur = have_nxt;
    };
    int it = 0;
    if constexpr (VSP) {
        // (a first step exists whenever there is a common entry; steps 0 .. vs_nc-2 have a common successor)
        for (; it + 1 < vs_nc; ++it) step(it, std::integral_constant<int, 1>{});
        // block entries of their own that both row blocks still have (leftovers of the split, or the
        // whole lists when they were not split): these steps run in the SPLIT form
        const int nb_both = min(vs_na, vs_nb) - vs_nc;
        if (nb_both >= 3 && have_cur) {
            if (vs_nc > 0) {                               // from the last common tile to the first split step
                step(it, std::integral_constant<int, 0>{});
                ++it;
            }
            // cur is now each row block's entry 0, its K copy is on the way
            if (!vs_shifted) {
                vs_shifted = true;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) k_rd_off[ks] += half * TILE_BYTES;
#pragma unroll
                for (int db = 0; db < NDB; ++db) v_rd_off[db] += half * TILE_BYTES;
            }
            sp_entry = vs_merged ? __builtin_amdgcn_readfirstlane(vs_only[half * VS_ONLY_MAX + 1]) : sp_list[1] * LIST_SCALE;
            for (; it - vs_nc + 1 < nb_both; ++it) step(it, std::integral_constant<int, 2>{});
        }
    }
    for (; have_cur; ++it) step(it, std::integral_constant<int, 0>{});

    // ---- epilogue: O = O^T / l, transposed through LDS so that every global store is 16 bytes
    // of one row and 16 lanes cover a whole 256-byte row ---------------------------------------
    {
        float l_tot = l_i + __shfl_xor(l_i, 32);
        const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        // pitch: 8-byte lane writes spread over all banks (four waves only fit without the pad)
        constexpr int OP = ROW_BYTES;
        // a row sum at 2^100 or beyond (or infinite, or no number at all): some probability may have
        // overflowed.  Compared on the bit pattern: the library is compiled without NaN semantics, which
        // lets the compiler turn !(l < x) into l >= x -- false for the NaN that inf * 0 leaves in a
        // row sum when the maximum is raised after an overflow
        // ... and an accumulator that is infinite or no number: O^T sums twice as many terms per tile
        // as a lane's share of the row sum (and terms scaled by |v|), so it can overflow while the row
        // sum still fits, and a later rescale then hides the size of the sum but not the inf / NaN
        if constexpr (!every_max) {
            unsigned obits = 0;
#pragma unroll
            for (int i = 0; i < NDB; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) obits = max(obits, __float_as_uint(oacc[i][r]) & 0x7fffffffu);
            const bool suspect = (__float_as_uint(l_tot) & 0x7fffffffu) >= __float_as_uint(0x1p100f) || obits >= 0x7f800000u;
            if (__any(suspect) && lane == 0) lds_redo = 1;
        }
        __syncthreads();                                  // K/V tiles no longer needed
        char *ot = (half ? lds_v : lds_k) + wave * 32 * OP;    // 32 rows per wave
        const bool live = qrow < seqlen;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
                union { T e[4]; u32x2_t u; } out4;
#pragma unroll
                for (int e = 0; e < 4; ++e) out4.e[e] = live ? (T)(oacc[db][rq * 4 + e] * inv) : (T)0.f;
                *reinterpret_cast<u32x2_t *>(ot + l32 * OP + (32 * db + 8 * rq + 4 * g) * 2) = out4.u;
            }
        __builtin_amdgcn_wave_barrier();
        // lane -> (row = RPI*i + lane/NCH, chunk = lane%NCH)
#pragma unroll
        for (int i = 0; i < 32 / RPI; ++i) {
            const int r = RPI * i + lane / NCH;
            const int grow = row0 + wave * 32 + r;
            const u32x4_t val = *reinterpret_cast<const u32x4_t *>(ot + r * OP + (lane % NCH) * 16);
            if (grow < p.n && have_rows) *reinterpret_cast<u32x4_t *>(o_base + (long long)grow * p.os[2] * 2 + (lane % NCH) * 16) = val;
        }
    }
    // (the flag was written before the barrier at the head of the epilogue)
    return !every_max && lds_redo != 0;                   // (workgroup-uniform)
}

// (head_dim 256: O^T, Q and the V^T fragments of a wave need more than 256 registers, so that form
// runs one wave per SIMD with the accumulators in the second half of the register file)
template <typename T, int MODE, int HD>
__global__ __launch_bounds__(2 * NTHREADS, HD > 128 ? 1 : 2) void attn_fwd_kernel(const AttnParams p) {
    typedef AttnLds<MODE, HD> L;
    __shared__ __attribute__((aligned(16))) char lds_k[L::NK];
    __shared__ __attribute__((aligned(16))) char lds_v[L::NK];
    __shared__ int vs_only[L::NONLY];        // paired list walks: [row block][entries the other list lacks]
    __shared__ int vs_wsum[4];
    __shared__ int vs_bad;
    __shared__ int lds_redo;
    if (threadIdx.x == 0) lds_redo = 0;      // (ordered before its readers by the barriers of the walk)
    if constexpr (std::is_same<T, __bf16>::value) {
        if (attn_walk<T, MODE, HD, false>(p, lds_k, lds_v, vs_only, vs_wsum, vs_bad, lds_redo)) {
            __syncthreads();                 // everyone has read the flag and is done with LDS
            attn_walk<T, MODE, HD, true>(p, lds_k, lds_v, vs_only, vs_wsum, vs_bad, lds_redo);
        }
    } else {
        // f16 probabilities have no headroom above the lazy threshold: the maximum of every tile
        attn_walk<T, MODE, HD, true>(p, lds_k, lds_v, vs_only, vs_wsum, vs_bad, lds_redo);
    }
}

int check_tensors(const minf_qkvo *t, bool allow_256 = false) {
    if (!t) return MINF_ERR_INVALID_ARG;
    if (t->batch < 0 || t->heads_q <= 0 || t->heads_kv <= 0 || t->n < 0) return MINF_ERR_INVALID_ARG;
    // empty problems (no batch or no tokens) have no storage: nothing to check, nothing is launched
    const bool empty = t->batch == 0 || t->n == 0;
    if (!empty && (!t->q || !t->k || !t->v || !t->o)) return MINF_ERR_INVALID_ARG;
    if (t->heads_q % t->heads_kv != 0) return MINF_ERR_INVALID_ARG;
    if (t->head_list && t->index_heads <= 0) return MINF_ERR_INVALID_ARG;
    if (t->head_dim != 128 && t->head_dim != 64 && !(allow_256 && t->head_dim == 256)) return MINF_ERR_UNSUPPORTED;
    if (t->dtype != MINF_BF16 && t->dtype != MINF_F16) return MINF_ERR_UNSUPPORTED;
    const void *ptrs[4] = {t->q, t->k, t->v, t->o};
    const int64_t *strides[4] = {t->q_stride, t->k_stride, t->v_stride, t->o_stride};
    for (int i = 0; i < 4; ++i) {
        if (((uintptr_t)ptrs[i]) & 15) return MINF_ERR_ALIGNMENT;
        for (int j = 0; j < 3; ++j)
            if (strides[i][j] < 0 || (strides[i][j] & 7)) return MINF_ERR_ALIGNMENT;
        // 64 rows x token stride is formed in 32 bits inside the tile copies
        if (strides[i][2] > (1 << 23)) return MINF_ERR_UNSUPPORTED;
        // rows must not overlap (expanded or interleaved views): the tile copies describe 64 rows of
        // a tile by one buffer descriptor of 64 x token stride bytes
        if (t->n > 1 && strides[i][2] < t->head_dim) return MINF_ERR_UNSUPPORTED;
    }
    return MINF_OK;
}

void fill_params(AttnParams &p, const minf_qkvo *t) {
    p.q = (const char *)t->q; p.k = (const char *)t->k; p.v = (const char *)t->v; p.o = (char *)t->o;
    for (int j = 0; j < 3; ++j) {
        p.qs[j] = t->q_stride[j]; p.ks[j] = t->k_stride[j];
        p.vs[j] = t->v_stride[j]; p.os[j] = t->o_stride[j];
    }
    p.batch = t->batch; p.hq = t->heads_q; p.hk = t->heads_kv; p.n = t->n;
    p.seqlens = t->seqlens;
    p.scale_log2 = t->sm_scale * 1.4426950408889634f;
    p.scale_log2_dense = p.scale_log2;
    p.rows = (t->n + BM - 1) / BM;
    p.bc = p.bo = p.cc = p.ci = nullptr; p.nnz_s = p.nnz_v = 0;
    p.bidx = nullptr; p.max_blocks = 0; p.bidx_rows = 0;
    p.n_init = p.n_local = 0; p.dense_from = 0x7fffffff;
    p.head_list = t->head_list;
    p.index_heads = t->head_list ? t->index_heads : t->heads_q;
    p.total_wg = 0;          // set by the launcher
    p.descending = 0;
}

template <int MODE, int HD> int launch_hd(AttnParams p, int dtype, void *stream) {
    if (p.batch == 0 || p.rows == 0) return MINF_OK;
    // heads of the grid: all of them, or the selected ones rounded up to whole chunks of hq / hk
    const int group = p.hq / p.hk;
    const long long grid_heads = p.head_list ? (long long)((p.index_heads + group - 1) / group) * group : p.hq;
    p.total_wg = (long long)p.batch * grid_heads * ((p.rows + 1) / 2);
    p.descending = MODE == MODE_DENSE || (MODE == MODE_VS && p.rows <= 1024);
    const long long per_xcd = (p.total_wg + 7) >> 3;
    const long long grid = per_xcd * 8;
    if (grid > 0x7fffffffLL) return MINF_ERR_UNSUPPORTED;
    const dim3 block(2 * NTHREADS);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MINF_BF16) hipLaunchKernelGGL((attn_fwd_kernel<__bf16, MODE, HD>), dim3((unsigned)grid), block, 0, st, p);
    else hipLaunchKernelGGL((attn_fwd_kernel<_Float16, MODE, HD>), dim3((unsigned)grid), block, 0, st, p);
    return minf_launch_status();
}

template <int MODE> int launch(const AttnParams &p, const minf_qkvo *t, void *stream) {
    if constexpr (MODE == MODE_ASHAPE || MODE == MODE_DENSE)
        if (t->head_dim == 256) return launch_hd<MODE, 256>(p, t->dtype, stream);
    if (t->head_dim == 256) return MINF_ERR_UNSUPPORTED;
    return t->head_dim == 64 ? launch_hd<MODE, 64>(p, t->dtype, stream) : launch_hd<MODE, 128>(p, t->dtype, stream);
}

}  // namespace

extern "C" int minf_vs_attn_fwd(const minf_qkvo *t, const int32_t *block_count,
                                const int32_t *block_offset, const int32_t *column_count,
                                const int32_t *column_index, int rows, int nnz_s, int nnz_v,
                                void *stream) {
    int st = check_tensors(t);
    if (st) return st;
    if (!block_count || !block_offset || !column_count || !column_index) return MINF_ERR_INVALID_ARG;
    if (nnz_s < 1 || nnz_v < 1) return MINF_ERR_INVALID_ARG;
    AttnParams p;
    fill_params(p, t);
    if (rows != p.rows) return MINF_ERR_INVALID_ARG;
    p.bc = block_count; p.bo = block_offset; p.cc = column_count; p.ci = column_index;
    p.nnz_s = nnz_s; p.nnz_v = nnz_v;
    return launch<MODE_VS>(p, t, stream);
}

extern "C" int minf_bs_attn_fwd(const minf_qkvo *t, const int32_t *block_index, int rows,
                                int max_blocks, void *stream) {
    int st = check_tensors(t);
    if (st) return st;
    if (!block_index || max_blocks < 1) return MINF_ERR_INVALID_ARG;
    AttnParams p;
    fill_params(p, t);
    if (rows < p.rows) return MINF_ERR_INVALID_ARG;
    // block_index may have more rows than ceil(n/64) (the reference pads n first)
    p.bidx = block_index; p.max_blocks = max_blocks; p.bidx_rows = rows;
    return launch<MODE_BS>(p, t, stream);
}

extern "C" int minf_ashape_attn_fwd(const minf_qkvo *t, int n_init, int n_local, void *stream) {
    int st = check_tensors(t, true);
    if (st) return st;
    if (n_init < 0 || n_local < 1) return MINF_ERR_INVALID_ARG;
    AttnParams p;
    fill_params(p, t);
    p.n_init = n_init; p.n_local = n_local;
    return launch<MODE_ASHAPE>(p, t, stream);
}

extern "C" int minf_trishape_attn_fwd(const minf_qkvo *t, int n_init, int n_local, int n_last,
                                      float sm_scale_last, void *stream) {
    int st = check_tensors(t, true);
    if (st) return st;
    uint32_t scale_bits;
    memcpy(&scale_bits, &sm_scale_last, sizeof(scale_bits));          // (negative, infinite or NaN: refused)
    if (n_init < 0 || n_local < 1 || n_last < 0 || (scale_bits >> 31) || (scale_bits & 0x7f800000u) == 0x7f800000u)
        return MINF_ERR_INVALID_ARG;
    AttnParams p;
    fill_params(p, t);
    if (sm_scale_last > 0.f) p.scale_log2_dense = sm_scale_last * 1.4426950408889634f;
    p.n_init = n_init; p.n_local = n_local;
    p.dense_from = n_last < t->n ? t->n - n_last : 0;
    return launch<MODE_ASHAPE>(p, t, stream);
}

extern "C" int minf_dense_attn_fwd(const minf_qkvo *t, void *stream) {
    int st = check_tensors(t, true);
    if (st) return st;
    AttnParams p;
    fill_params(p, t);
    return launch<MODE_DENSE>(p, t, stream);
}
