// Sparse flash-attention forward for gfx950: one 64x64 tile engine, four tile
// sources (vertical-slash block+column lists, block-sparse lists, analytic
// A-shape ranges, dense causal).
//
// Work split: one workgroup (2 wavefronts) per (batch, query head, 64-row
// block); each wavefront owns 32 query rows.  Everything is computed in the
// TRANSPOSED orientation so that softmax statistics are per lane:
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
// LDS: K and V tiles are [64 tokens][128] 16-bit, 256 B per row, no padding;
// 16-byte chunks are XOR-swizzled (K: chunk ^ row%16, V: chunk ^ 4*(row%4)) so
// that ds_read_b128 of 16 rows and the 4-row transpose reads hit distinct banks.
// Global->LDS goes through registers in half tiles (32 keys), prefetched a tile ahead, and the
// main loop is software-pipelined over half tiles: the QK^T MFMAs of half tile h+1 are issued
// next to the softmax VALU work of half tile h (see the schedule above the loop).
#include "minf_common.h"
#include <math.h>
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
constexpr int HD = 128;       // head_dim
constexpr int NTHREADS = 256; // 4 wavefronts: 2 row halves x 2 key halves
constexpr int ROW_BYTES = HD * 2;
// LDS row pitches: +16 B (K) makes ds_read_b128 of 16 consecutive rows hit 64 distinct banks,
// +64 B (V) does the same for the 4-row x 64-byte transpose reads; with plain padding every LDS
// address is one per-lane base plus an immediate offset.
constexpr int K_PITCH = ROW_BYTES + 16;
constexpr int V_PITCH = ROW_BYTES + 64;
constexpr int LDS_K_BYTES = BN * K_PITCH;
constexpr int LDS_V_BYTES = BN * V_PITCH;

struct AttnParams {
    const char *q, *k, *v;
    char *o;
    long long qs[3], ks[3], vs[3], os[3];   // element strides: batch, head, token
    int batch, hq, hk, n;
    const int *seqlens;
    float scale_log2;
    int rows;
    // vertical-slash
    const int *bc, *bo, *cc, *ci;
    int nnz_s, nnz_v;
    // block-sparse
    const int *bidx;
    int max_blocks, bidx_rows;
    // a-shape
    int n_init, n_local;
    long long total_wg;
};

// The index tensors are read-only for the whole launch.  Their wave-uniform entries (counts,
// block offsets, block ids) are read through constant-address-space pointers so that they become
// scalar loads: a vector load whose result is needed at once would make the wave wait for every
// K/V prefetch issued before it.  The gathered column ids stay vector loads (one per lane).
typedef const __attribute__((address_space(4))) int *cint_ptr;
struct IdxPtrs {
    cint_ptr bc, bo, cc, bidx;
    const int *ci;
};
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

// sum of the 8 (rounded) values of a fragment, via the 2-way dot-product instructions
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
template <typename T> __device__ __forceinline__ float pair_sum(const Frag &f);
template <> __device__ __forceinline__ float pair_sum<__bf16>(const Frag &f) {
    const bf16x2_t one = {(__bf16)1.0f, (__bf16)1.0f};
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        bf16x2_t pr = {f.b[2 * j], f.b[2 * j + 1]};
        acc = __builtin_amdgcn_fdot2_f32_bf16(pr, one, acc, false);
    }
    return acc;
}
template <> __device__ __forceinline__ float pair_sum<_Float16>(const Frag &f) {
    const f16x2_t one = {(_Float16)1.0f, (_Float16)1.0f};
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f16x2_t pr = {f.h[2 * j], f.h[2 * j + 1]};
        acc = __builtin_amdgcn_fdot2(pr, one, acc, false);
    }
    return acc;
}

// One tile of keys: either 64 consecutive tokens from `start`, or 64 gathered
// token ids read from `gather` (entries >= nvalid are padding).
struct Tile {
    int start;          // first token (contiguous) / first list position (gathered)
    int gathered;       // 0/1
    int nvalid;         // gathered: number of valid list entries in this tile
};

template <int MODE>
__device__ __forceinline__ int tile_count(const AttnParams &p, const IdxPtrs &ix, long long ridx, int m, int &nblk) {
    if constexpr (MODE == MODE_VS) {
        nblk = ix.bc[ridx];
        return nblk + ((ix.cc[ridx] + BN - 1) >> 6);
    } else if constexpr (MODE == MODE_BS) {
        nblk = min(m + 1, p.max_blocks);
        return nblk;
    } else if constexpr (MODE == MODE_ASHAPE) {
        // window tiles t_lo..m, preceded by the sink tiles that lie before t_lo
        int lo_key = m * BM - p.n_local + 1;
        int t_lo = lo_key > 0 ? (lo_key >> 6) : 0;
        int sink_tiles = (p.n_init + BN - 1) >> 6;
        nblk = min(sink_tiles, t_lo);            // number of leading sink tiles
        return nblk + (m - t_lo + 1);
    } else {
        nblk = m + 1;
        return nblk;
    }
}

template <int MODE>
__device__ __forceinline__ Tile tile_at(const AttnParams &p, const IdxPtrs &ix, long long ridx, int m, int nblk, int it) {
    Tile t;
    t.gathered = 0;
    t.nvalid = BN;
    if constexpr (MODE == MODE_VS) {
        if (it < nblk) {
            t.start = ix.bo[ridx * p.nnz_s + it];
        } else {
            t.gathered = 1;
            t.start = (it - nblk) * BN;
            t.nvalid = min(BN, ix.cc[ridx] - t.start);
        }
    } else if constexpr (MODE == MODE_BS) {
        t.start = ix.bidx[((ridx / p.rows) * p.bidx_rows + m) * p.max_blocks + it] * BN;
    } else if constexpr (MODE == MODE_ASHAPE) {
        int lo_key = m * BM - p.n_local + 1;
        int t_lo = lo_key > 0 ? (lo_key >> 6) : 0;
        t.start = (it < nblk ? it : t_lo + (it - nblk)) * BN;
    } else {
        t.start = it * BN;
    }
    return t;
}

template <typename T, int MODE>
__global__ __launch_bounds__(NTHREADS, 2) void attn_fwd_kernel(const AttnParams p) {
    IdxPtrs ix;
    ix.bc = as_const(p.bc); ix.bo = as_const(p.bo); ix.cc = as_const(p.cc); ix.bidx = as_const(p.bidx);
    ix.ci = p.ci;
    // K tile, V tile, and 1 KB for the (max, sum) pairs of the final merge; the O partials of
    // the merge reuse the K/V space.
    __shared__ __attribute__((aligned(16))) char lds[LDS_K_BYTES + LDS_V_BYTES];
    char *const lds_k = lds;
    char *const lds_v = lds + LDS_K_BYTES;

    // ---- which (batch, head, row block): XCD-aware remap --------------------
    // Consecutive workgroup ids are dealt round-robin to the 8 XCDs; give each
    // XCD one contiguous range of the logical order (batch, kv head, row block,
    // query head inside the GQA group) so that the row blocks and the query
    // heads that share K/V also share an L2.
    const long long per_xcd = (p.total_wg + 7) >> 3;
    const long long logical = (long long)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= p.total_wg) return;
    const int group = p.hq / p.hk;
    long long rest = logical;
    const int hin = (int)(rest % group); rest /= group;
    const int m = p.rows - 1 - (int)(rest % p.rows); rest /= p.rows;   // heavy (late) rows first
    const int hkv = (int)(rest % p.hk);
    const int b = (int)(rest / p.hk);
    const int h = hkv * group + hin;

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int rw = wave & 1;          // which 32 query rows of the block
    const int kw = wave >> 1;         // which 32 keys of every tile
    const int l32 = lane & 31;
    const int g = lane >> 5;

    const int seqlen = p.seqlens ? min(p.seqlens[b], p.n) : p.n;
    const int row0 = m * BM;
    const int qrow = row0 + rw * 32 + l32;          // this lane's query row
    char *o_base = p.o + ((long long)b * p.os[0] + (long long)h * p.os[1]) * 2;

    if (row0 >= seqlen) {
        // row block past the sequence: zeros (16 B per lane-step)
        for (int i = tid; i < BM * 16; i += NTHREADS) {
            int r = row0 + (i >> 4);
            if (r < p.n) *reinterpret_cast<u32x4_t *>(o_base + (long long)r * p.os[2] * 2 + (i & 15) * 16) = u32x4_t{0u, 0u, 0u, 0u};
        }
        return;
    }

    const char *q_base = p.q + ((long long)b * p.qs[0] + (long long)h * p.qs[1]) * 2;
    const char *k_base = p.k + ((long long)b * p.ks[0] + (long long)hkv * p.ks[1]) * 2;
    const char *v_base = p.v + ((long long)b * p.vs[0] + (long long)hkv * p.vs[1]) * 2;
    const long long k_row = p.ks[2] * 2, v_row = p.vs[2] * 2;
    const long long ridx = ((long long)b * p.hq + h) * p.rows + m;

    // ---- Q fragments (B operand of S^T): row qrow, d = 16*ks + 8*g + 0..7 ----
    Frag qf[8];
    {
        const bool ok = qrow < seqlen;
        const char *qp = q_base + (long long)(ok ? qrow : row0) * p.qs[2] * 2 + g * 16;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            qf[ks].u = *reinterpret_cast<const u32x4_t *>(qp + ks * 32);
            if (!ok) qf[ks].u = u32x4_t{0u, 0u, 0u, 0u};
        }
    }

    int nblk = 0;
    const int ntiles = tile_count<MODE>(p, ix, ridx, m, nblk);

    // ---- global -> register -> LDS staging ---------------------------------------
    // A thread covers rows 16*i + tid/16 (i = 0..3) of a tile, 16-byte chunk tid%16.
    // Rows that do not exist (past seqlen, or padding of a gathered tile) are read from a
    // clamped, valid address instead of being zeroed: their scores are always masked to
    // -inf below, so their probabilities are exactly 0 and K/V contents never matter.
    const int ld_r = tid >> 4;       // 0..15
    const int ld_c = tid & 15;       // 16-byte chunk in the row
    u32x4_t kreg[4], vreg[4];        // in flight: next K tile, next V tile

    // byte offset of this thread's first row inside a contiguous tile (rows 16 apart add a
    // wave-uniform 16*pitch, so one 32-bit lane offset serves all four loads)
    const unsigned koff = (unsigned)(ld_r * k_row + ld_c * 16);
    const unsigned voff = (unsigned)(ld_r * v_row + ld_c * 16);
    const bool small_pitch = k_row * 64 < (1ll << 31) && v_row * 64 < (1ll << 31);
    // token ids of this thread's 4 rows of a gathered (column) tile
    auto gather_ids = [&](const Tile &t, int (&tok)[4]) {
        if (MODE == MODE_VS && t.gathered) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                tok[i] = ix.ci[ridx * p.nnz_v + t.start + min(i * 16 + ld_r, t.nvalid - 1)];
        }
    };
    auto load_tile = [&](const Tile &t, const char *base, long long rowstride, const unsigned off,
                         const int (&gtok)[4], u32x4_t (&dst)[4]) {
        const bool gathered = MODE == MODE_VS && t.gathered;
        if (!gathered && small_pitch && t.start >= 0 && t.start + BN <= seqlen) {
            // common case: one wave-uniform base, loop-invariant per-thread offsets
            const char *tb = base + (long long)t.start * rowstride;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                dst[i] = *reinterpret_cast<const u32x4_t *>(tb + (long long)i * 16 * rowstride + off);
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tok = gathered ? gtok[i] : t.start + i * 16 + ld_r;
            const int tk = max(0, min(tok, seqlen - 1));
            dst[i] = *reinterpret_cast<const u32x4_t *>(base + tk * rowstride + ld_c * 16);
        }
    };
    char *const lds_k_st = lds_k + ld_r * K_PITCH + ld_c * 16;
    char *const lds_v_st = lds_v + ld_r * V_PITCH + ld_c * 16;
    auto store_k = [&](const u32x4_t (&src)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<u32x4_t *>(lds_k_st + i * 16 * K_PITCH) = src[i];
        }
    };
    auto store_v = [&](const u32x4_t (&src)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<u32x4_t *>(lds_v_st + i * 16 * V_PITCH) = src[i];
        }
    };

    // ---- accumulators (this wave's share: its 32 rows x its 32 keys of every tile) -----
    f32x16_t oacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m_i = -INFINITY;   // reference max of the row (log2 domain, scaled); lags the true max by <= 8
    float l_i = 0.f;         // this lane's share of the running sum

    // V transpose read: row = T0 + (lane%16)/4, col = 32*db + 16*((lane/16)%2) + 4*(lane%4)
    const int v_rd_rsub = (lane & 15) >> 2;
    const int v_rd_col = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);      // + 32*db
    const int wrow_lo = row0 + rw * 32, wrow_hi = wrow_lo + 31;

    const char *const lds_k_rd = lds_k + (32 * kw + l32) * K_PITCH + g * 16;
    const char *const lds_v_rd = lds_v + (32 * kw + 4 * g + v_rd_rsub) * V_PITCH + v_rd_col * 2;
    // S^T of this wave: keys 32*kw + (0..31) of the tile in LDS x its 32 query rows
    auto qk_tile = [&]() {
        f32x16_t s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            Frag a;
            a.u = *reinterpret_cast<const u32x4_t *>(lds_k_rd + ks * 32);
            s = Mma<T>::mfma(frag_as<T>(a), frag_as<T>(qf[ks]), s);
        }
        return s;
    };

    // does this wave have to mask anything in its keys [32*kw, 32*kw+32) of tile t ?
    auto needs_mask = [&](const Tile &t) {
        if (MODE == MODE_VS && t.gathered) return t.nvalid < 32 * kw + 32;
        const int c_lo = t.start + 32 * kw, c_hi = c_lo + 31;
        if constexpr (MODE == MODE_ASHAPE) {
            const bool causal_ok = c_hi <= wrow_lo && c_hi < seqlen;
            const bool in_window = (wrow_hi - c_lo) < p.n_local;
            const bool in_sink = c_hi < p.n_init;
            return !(causal_ok && (in_window || in_sink));
        }
        return (c_hi > wrow_lo) || (c_hi >= seqlen);
    };

    // online softmax of this wave's 32x32 score block (exp2 domain); s -> probabilities, packed
    // into the B-operand fragments of the two PV k-steps; alpha = factor for the O accumulators.
    // Element r of this lane is tile-local key 32*kw + 4*g + tkc, tkc = 8*(r/4) + r%4.
    // keep <=> tkc <= hi && (tkc > wlo || tkc < slim).
    auto softmax_tile = [&](f32x16_t &s, const Tile &t, auto masked, Frag (&pf)[2], float &alpha, bool &rescale) {
        if constexpr (decltype(masked)::value) {
            int hi, wlo = -1, slim = 0;
            const int sh = 4 * g + 32 * kw;
            if (MODE == MODE_VS && t.gathered) {
                hi = t.nvalid - 1 - sh;
            } else {
                hi = min(qrow, seqlen - 1) - t.start - sh;
                if constexpr (MODE == MODE_ASHAPE) {
                    wlo = qrow - t.start - p.n_local - sh;
                    slim = p.n_init - t.start - sh;
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int tkc = 8 * (r >> 2) + (r & 3);
                bool kp = tkc <= hi;
                if constexpr (MODE == MODE_ASHAPE) kp = kp & ((tkc > wlo) | (tkc < slim));
                s[r] = kp ? s[r] : -INFINITY;
            }
        }
        float mx = fmaxf(s[0], s[1]);
#pragma unroll
        for (int r = 2; r < 16; ++r) mx = fmaxf(mx, s[r]);
        {
            // max over the two lane halves (lanes l and l^32 hold the same query row)
            const unsigned u = __float_as_uint(mx);
            auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
            mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        // lazy reference max: only move it when the row max grew by more than 2^8
        const float cand = mx * p.scale_log2;
        const bool grow = cand > m_i + 8.0f;
        const float m_next = grow ? cand : m_i;
        alpha = grow ? __builtin_amdgcn_exp2f(m_i - m_next) : 1.0f;
        rescale = __any(grow);
        m_i = m_next;
        const float m_sub = (m_next == -INFINITY) ? 0.f : m_next;
        float pr[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) pr[r] = __builtin_amdgcn_exp2f(fmaf(s[r], p.scale_log2, -m_sub));
        cvt8<T>(&pr[0], pf[0]);
        cvt8<T>(&pr[8], pf[1]);
        // row sum of the ROUNDED probabilities (what the PV product really uses)
        l_i = l_i * alpha + pair_sum<T>(pf[0]) + pair_sum<T>(pf[1]);
    };

    auto pv_tile = [&](const Frag (&pf)[2]) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                Frag vf;
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    vf.s4[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) short4_t *)(lds_v_rd + (16 * s2 + 8 * jj) * V_PITCH + db * 64));
                }
                oacc[db] = Mma<T>::mfma(frag_as<T>(vf), frag_as<T>(pf[s2]), oacc[db]);
            }
        }
    };
    auto rescale_o = [&](float alpha) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
    };
    // Ask the scheduler to spread the 8 QK MFMAs of a phase between the softmax VALU work of the
    // same basic block: (1 LDS read, 1 MFMA, 10 VALU) x 8.
    auto interleave_hint = [&]() {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
        }
    };

    // ---- software pipeline over tiles ----------------------------------------------
    // Iteration `it` (t0 = tile it, t1 = it+1, ...; indices clamped to the last tile):
    //   A : S_next = QK(t1) [Kbuf = K(t1)]  ||  softmax(S_cur = scores of t0)
    //   barrier; store K(t2) -> Kbuf; load kreg <- K(t3)
    //   B : O += P.V(t0)   [Vbuf = V(t0)]
    //   barrier; store V(t1) -> Vbuf; load vreg <- V(t2)
    // The QK MFMAs of the next tile share a basic block with the softmax VALU work of the
    // current one; every LDS region is overwritten only after the barrier that follows its
    // last read and read only after the barrier that follows its write.
    if (ntiles > 0) {
        const int last = ntiles - 1;
        Tile t0 = tile_at<MODE>(p, ix, ridx, m, nblk, 0);
        Tile t1 = tile_at<MODE>(p, ix, ridx, m, nblk, min(1, last));
        Tile t2 = tile_at<MODE>(p, ix, ridx, m, nblk, min(2, last));
        Tile t3 = tile_at<MODE>(p, ix, ridx, m, nblk, min(3, last));
        // (global loads are issued in the same order as inside the loop -- gather ids, K, V -- so
        // that the outstanding-load counters the waits are derived from agree on every path)
        Tile t4 = tile_at<MODE>(p, ix, ridx, m, nblk, min(4, last));
        int tokK[4] = {0, 0, 0, 0}, tokV[4] = {0, 0, 0, 0}, tokN[4] = {0, 0, 0, 0};
        gather_ids(t0, tokK);
        load_tile(t0, k_base, k_row, koff, tokK, kreg);
        load_tile(t0, v_base, v_row, voff, tokK, vreg);
        store_k(kreg);
        store_v(vreg);
        gather_ids(t1, tokV);
        load_tile(t1, k_base, k_row, koff, tokV, kreg);
        __syncthreads();
        f32x16_t s_a = qk_tile();
        __syncthreads();
        store_k(kreg);
        gather_ids(t2, tokK);
        gather_ids(t3, tokN);
        load_tile(t2, k_base, k_row, koff, tokK, kreg);
        load_tile(t1, v_base, v_row, voff, tokV, vreg);
#pragma unroll
        for (int i = 0; i < 4; ++i) tokV[i] = tokK[i];
#pragma unroll
        for (int i = 0; i < 4; ++i) tokK[i] = tokN[i];
        __syncthreads();

        // One pipeline step; the score registers ping-pong between two steps (no copies).
        // On entry: Kbuf = K(t1), Vbuf = V(t0), kreg = K(t2) and vreg = V(t1) in flight;
        // tokK / tokV = gathered token ids of t3 / t2 (if those are column tiles).
        auto step = [&](f32x16_t &s_cur, f32x16_t &s_nxt, int it) {
            Frag pf[2];
            float alpha;
            bool rescale;
            gather_ids(t4, tokN);          // needed one step from now: stays older than the K/V loads below
            if (needs_mask(t0)) {
                s_nxt = qk_tile();
                softmax_tile(s_cur, t0, std::true_type{}, pf, alpha, rescale);
                interleave_hint();
            } else {
                s_nxt = qk_tile();
                softmax_tile(s_cur, t0, std::false_type{}, pf, alpha, rescale);
                interleave_hint();
            }
            __syncthreads();
            store_k(kreg);
            load_tile(t3, k_base, k_row, koff, tokK, kreg);
            if (rescale) rescale_o(alpha);
            pv_tile(pf);
            __syncthreads();
            store_v(vreg);
            load_tile(t2, v_base, v_row, voff, tokV, vreg);
            t0 = t1;
            t1 = t2;
            t2 = t3;
            t3 = t4;
            t4 = tile_at<MODE>(p, ix, ridx, m, nblk, min(it + 5, last));
#pragma unroll
            for (int i = 0; i < 4; ++i) tokV[i] = tokK[i];
#pragma unroll
            for (int i = 0; i < 4; ++i) tokK[i] = tokN[i];
        };
        f32x16_t s_b;
        for (int it = 0;;) {
            step(s_a, s_b, it);
            if (++it >= ntiles) break;
            step(s_b, s_a, it);
            if (++it >= ntiles) break;
        }
    }

    // ---- merge the two key halves: waves kw=1 hand (m, l, O) to waves kw=0 through LDS ----
    __syncthreads();
    float *xo = reinterpret_cast<float *>(lds) + rw * (64 * 64);        // [reg 0..63][lane]
    float *xml = reinterpret_cast<float *>(lds + 2 * 64 * 64 * 4) + rw * 128;   // [m|l][lane]
    if (kw == 1) {
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) xo[(db * 16 + r) * 64 + lane] = oacc[db][r];
        xml[lane] = m_i;
        xml[64 + lane] = l_i;
    }
    __syncthreads();
    if (kw == 1) return;
    {
        const float m1 = xml[lane], l1 = xml[64 + lane];
        const float mm = fmaxf(m_i, m1);
        const float mu = (mm == -INFINITY) ? 0.f : mm;
        const float a0 = __builtin_amdgcn_exp2f(m_i - mu), a1 = __builtin_amdgcn_exp2f(m1 - mu);
        l_i = l_i * a0 + l1 * a1;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[db][r] = oacc[db][r] * a0 + xo[(db * 16 + r) * 64 + lane] * a1;
    }

    // ---- epilogue: O = O^T / l, store ------------------------------------------
    float l_tot = l_i + __shfl_xor(l_i, 32);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (qrow < p.n) {
        const bool live = qrow < seqlen;
        char *orow = o_base + (long long)qrow * p.os[2] * 2;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
                // d = 32*db + 8*rq + 4*g + 0..3
                union { T e[4]; u32x2_t u; } out4;
#pragma unroll
                for (int e = 0; e < 4; ++e) out4.e[e] = live ? (T)(oacc[db][rq * 4 + e] * inv) : (T)0.f;
                *reinterpret_cast<u32x2_t *>(orow + (32 * db + 8 * rq + 4 * g) * 2) = out4.u;
            }
    }
}

int check_tensors(const minf_qkvo *t) {
    if (!t || !t->q || !t->k || !t->v || !t->o) return MINF_ERR_INVALID_ARG;
    if (t->batch < 0 || t->heads_q <= 0 || t->heads_kv <= 0 || t->n < 0) return MINF_ERR_INVALID_ARG;
    if (t->heads_q % t->heads_kv != 0) return MINF_ERR_INVALID_ARG;
    if (t->head_dim != HD) return MINF_ERR_UNSUPPORTED;
    if (t->dtype != MINF_BF16 && t->dtype != MINF_F16) return MINF_ERR_UNSUPPORTED;
    const void *ptrs[4] = {t->q, t->k, t->v, t->o};
    const int64_t *strides[4] = {t->q_stride, t->k_stride, t->v_stride, t->o_stride};
    for (int i = 0; i < 4; ++i) {
        if (((uintptr_t)ptrs[i]) & 15) return MINF_ERR_ALIGNMENT;
        for (int j = 0; j < 3; ++j)
            if (strides[i][j] < 0 || (strides[i][j] & 7)) return MINF_ERR_ALIGNMENT;
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
    p.rows = (t->n + BM - 1) / BM;
    p.bc = p.bo = p.cc = p.ci = nullptr; p.nnz_s = p.nnz_v = 0;
    p.bidx = nullptr; p.max_blocks = 0; p.bidx_rows = 0;
    p.n_init = p.n_local = 0;
    p.total_wg = (long long)t->batch * t->heads_q * p.rows;
}

template <int MODE> int launch(const AttnParams &p, int dtype, void *stream) {
    if (p.total_wg == 0) return MINF_OK;
    const long long per_xcd = (p.total_wg + 7) >> 3;
    const long long grid = per_xcd * 8;
    if (grid > 0x7fffffffLL) return MINF_ERR_UNSUPPORTED;
    if (dtype == MINF_BF16)
        hipLaunchKernelGGL((attn_fwd_kernel<__bf16, MODE>), dim3((unsigned)grid), dim3(NTHREADS), 0,
                           (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL((attn_fwd_kernel<_Float16, MODE>), dim3((unsigned)grid), dim3(NTHREADS), 0,
                           (hipStream_t)stream, p);
    return minf_launch_status();
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
    return launch<MODE_VS>(p, t->dtype, stream);
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
    return launch<MODE_BS>(p, t->dtype, stream);
}

extern "C" int minf_ashape_attn_fwd(const minf_qkvo *t, int n_init, int n_local, void *stream) {
    int st = check_tensors(t);
    if (st) return st;
    if (n_init < 0 || n_local < 1) return MINF_ERR_INVALID_ARG;
    AttnParams p;
    fill_params(p, t);
    p.n_init = n_init; p.n_local = n_local;
    return launch<MODE_ASHAPE>(p, t->dtype, stream);
}

extern "C" int minf_dense_attn_fwd(const minf_qkvo *t, void *stream) {
    int st = check_tensors(t);
    if (st) return st;
    AttnParams p;
    fill_params(p, t);
    return launch<MODE_DENSE>(p, t->dtype, stream);
}
