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
constexpr int TILE_BYTES = BN * ROW_BYTES;          // 16 KB, rows unpadded, 16-byte chunks XOR-swizzled
constexpr int LDS_BYTES = 4 * TILE_BYTES + 1024;    // K x2, V x2 (double buffered) [+ merge scratch]

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
    // K and V double buffers as four separate LDS objects: the compiler only lets an LDS read
    // run ahead of an in-flight global->LDS copy when it can prove they touch different objects.
    __shared__ __attribute__((aligned(16))) char lds_k0[TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char lds_k1[TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char lds_v0[TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char lds_v1[TILE_BYTES];
    __shared__ float lds_ml[256];

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

    // ---- global -> LDS copies without a register round trip --------------------------------
    // global_load_lds_dwordx4: every lane fetches 16 bytes from its own global address and the
    // wave's 64 x 16 B land CONTIGUOUSLY in LDS at a wave-uniform base (lane i -> base + 16*i).
    // One instruction therefore fills 4 tile rows (16 lanes x 16 B each); wave w owns rows
    // 16*w .. 16*w+15 of every tile (4 instructions per matrix).  Bank-conflict-free reads need
    // the 16-byte chunks of a row permuted (K: chunk ^ row%16, V: chunk ^ 4*(row%4)); with DMA
    // the permutation is applied on the global side: lane (row, c') loads global chunk c'^swz(row).
    // Rows that do not exist (past seqlen, or padding of a gathered tile) are read from a
    // clamped, valid address: their scores are always masked to -inf, so their probabilities are
    // exactly 0 and the K/V contents never matter.
    const int cp_r = lane >> 4;                  // row inside the 4-row group
    const int cp_c = lane & 15;                  // LDS chunk
    // token ids of this lane's 4 rows of a gathered (column) tile
    auto gather_ids = [&](const Tile &t, int (&tok)[4]) {
        if (MODE == MODE_VS && t.gathered) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                tok[j] = ix.ci[ridx * p.nnz_v + t.start + min(16 * wave + 4 * j + cp_r, t.nvalid - 1)];
        }
    };
    auto copy_tile = [&](const Tile &t, const char *base, long long rowstride, bool is_v, const int (&gtok)[4],
                         char *ldsbuf) {
        const bool gathered = MODE == MODE_VS && t.gathered;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 16 * wave + 4 * j + cp_r;          // tile row
            const int tok = gathered ? gtok[j] : t.start + r;
            const int tk = max(0, min(tok, seqlen - 1));
            const int c = is_v ? (cp_c ^ ((r & 3) << 2)) : (cp_c ^ (r & 15));
            const char *gp = base + tk * rowstride + c * 16;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                             (__attribute__((address_space(3))) void *)(ldsbuf + (16 * wave + 4 * j) * ROW_BYTES),
                                             16, 0, 0);
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
    const int wrow_lo = row0 + rw * 32, wrow_hi = wrow_lo + 31;

    // K read: row 32*kw + l32, logical chunk 2*ks + g -> physical chunk ^ (row % 16)
    int k_rd_off[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) k_rd_off[ks] = (32 * kw + l32) * ROW_BYTES + (((2 * ks + g) ^ (l32 & 15)) << 4);
    // V transpose read: row 32*kw + 16*s2 + 8*jj + 4*g + rsub (row % 4 == rsub), logical chunk
    // 4*db + vc -> physical 4*(db ^ rsub) + vc
    const int v_rd_vc = (((lane >> 4) & 1) << 1) + ((lane & 3) >> 1);
    int v_rd_off[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
        v_rd_off[db] = (32 * kw + 4 * g + v_rd_rsub) * ROW_BYTES + ((((db ^ v_rd_rsub) << 2) + v_rd_vc) << 4) + ((lane & 1) << 3);
    // S^T of this wave: keys 32*kw + (0..31) of the tile in LDS x its 32 query rows
    auto qk_tile = [&](const char *kbuf) {
        f32x16_t s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            Frag a;
            a.u = *reinterpret_cast<const u32x4_t *>(kbuf + k_rd_off[ks]);
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

    auto pv_tile = [&](const Frag (&pf)[2], const char *vbuf) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                Frag vf;
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    vf.s4[jj] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) short4_t *)(vbuf + v_rd_off[db] + (16 * s2 + 8 * jj) * ROW_BYTES));
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
    // Step `it` (t0 = tile it, t1 = it+1, t2 = it+2; indices clamped to the last tile), with
    // K/V double buffered in LDS (buffer parity = tile parity):
    //   issue DMA  K(t2) -> Kbuf[it%2]   (held K(t0): last read before the previous barrier)
    //              V(t1) -> Vbuf[(it+1)%2]
    //   A : S_next = QK(t1) [Kbuf[(it+1)%2]]  ||  softmax(S_cur = scores of t0)
    //   B : O += P.V(t0)    [Vbuf[it%2]]
    //   wait for the DMA; barrier
    // One barrier per tile; the QK MFMAs of the next tile share a basic block with the softmax
    // VALU work of the current one.
    if (ntiles > 0) {
        const int last = ntiles - 1;
        Tile t0 = tile_at<MODE>(p, ix, ridx, m, nblk, 0);
        Tile t1 = tile_at<MODE>(p, ix, ridx, m, nblk, min(1, last));
        Tile t2 = tile_at<MODE>(p, ix, ridx, m, nblk, min(2, last));
        Tile t3 = tile_at<MODE>(p, ix, ridx, m, nblk, min(3, last));
        int tok0[4] = {0, 0, 0, 0}, tokV[4] = {0, 0, 0, 0}, tokK[4] = {0, 0, 0, 0}, tokN[4] = {0, 0, 0, 0};
        gather_ids(t0, tok0);
        gather_ids(t1, tokV);
        gather_ids(t2, tokK);
        gather_ids(t3, tokN);
        copy_tile(t0, k_base, k_row, false, tok0, lds_k0);
        copy_tile(t0, v_base, v_row, true, tok0, lds_v0);
        copy_tile(t1, k_base, k_row, false, tokV, lds_k1);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        f32x16_t s_a = qk_tile(lds_k0);
        __syncthreads();

        // on entry: Kbuf[(it+1)%2] = K(t1), Vbuf[it%2] = V(t0) landed; tokK/tokV/tokN = gathered
        // token ids of t2 / t1 / t3
        auto step = [&](f32x16_t &s_cur, f32x16_t &s_nxt, int it, auto parity) {
            constexpr int par = decltype(parity)::value;
            Frag pf[2];
            float alpha;
            bool rescale;
            copy_tile(t2, k_base, k_row, false, tokK, par ? lds_k1 : lds_k0);
            copy_tile(t1, v_base, v_row, true, tokV, par ? lds_v0 : lds_v1);
            const char *kb = par ? lds_k0 : lds_k1;
            if (needs_mask(t0)) {
                s_nxt = qk_tile(kb);
                softmax_tile(s_cur, t0, std::true_type{}, pf, alpha, rescale);
                interleave_hint();
            } else {
                s_nxt = qk_tile(kb);
                softmax_tile(s_cur, t0, std::false_type{}, pf, alpha, rescale);
                interleave_hint();
            }
            if (rescale) rescale_o(alpha);
            pv_tile(pf, par ? lds_v1 : lds_v0);
            t0 = t1;
            t1 = t2;
            t2 = t3;
            t3 = tile_at<MODE>(p, ix, ridx, m, nblk, min(it + 4, last));
#pragma unroll
            for (int i = 0; i < 4; ++i) { tokV[i] = tokK[i]; tokK[i] = tokN[i]; }
            gather_ids(t3, tokN);
            __builtin_amdgcn_s_waitcnt(0x0f70 | 0);   // vmcnt(0): the copies issued above have landed
            __syncthreads();
        };
        f32x16_t s_b;
        for (int it = 0;;) {
            step(s_a, s_b, it, std::integral_constant<int, 0>{});
            if (++it >= ntiles) break;
            step(s_b, s_a, it, std::integral_constant<int, 1>{});
            if (++it >= ntiles) break;
        }
    }

    // ---- merge the two key halves: waves kw=1 hand (m, l, O) to waves kw=0 through LDS ----
    __syncthreads();
    float *xo = reinterpret_cast<float *>(rw ? lds_k1 : lds_k0);       // [reg 0..63][lane]
    float *xml = lds_ml + rw * 128;                                      // [m|l][lane]
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
