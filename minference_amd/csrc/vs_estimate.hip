// Online vertical/slash pattern estimation for gfx950.
//
// For every (batch, query head): P = softmax(Q[-last_q:] . K^T / sqrt(d)) with the
// trailing last_q x last_q corner causally masked, then
//   vertical[c] = sum_i P[i, c]                      (column sums)
//   slash[j]    = sum_i P[i, i + j + 1 - last_q]     (diagonal sums; j <-> offset N-1-j)
// (reference minference/modules/minference_forward.py:599-614 and :110-116).
//
// Two sweeps over K, both on v_mfma_f32_32x32x16 with K and Q fragments in operand layout (the
// same registers serve as A or B operand, so swapping the operands transposes the score tile for
// free).  Q fragments are read straight from global memory; a K block is read straight from global
// memory too when the waves of a workgroup score different kv heads, and otherwise fetched once
// per workgroup into LDS (LDS-DMA, double buffered) and read from there by all four waves:
//   stats  : S^T = K.Q^T  -> lane <-> query row: running max / sum-of-exp in
//            registers, one (max, sum) pair per row per 2048-key chunk;
//   (every workgroup of the second sweep first combines the chunk pairs of its heads into the row
//   constants M_i = max_i + log2(sum_i): no kernel in between)
//   scores : S = Q.K^T    -> lane <-> key: p = exp2(s - M_row); column sums are
//            in-lane adds (+ one cross-half shuffle); the diagonal sums are formed in registers
//            with whole-wave lane shifts (one DPP add per query row, see est_scores_kernel; no
//            LDS tile, no atomics); the per-chunk window is written out whole;
//   finalize: stitch the chunk windows together (each diagonal gets at most two
//            pieces, added in a fixed order) and apply the forced +inf entries.
// Work split: a workgroup owns one 2048-key chunk of one group of up to four query heads that are
// neighbours in head order (with grouped-query attention: heads that read the same K): wave w
// scores head w % gw over key sub-range w / gw of the chunk (gw = heads per workgroup: 4, 2 or 1),
// so the K fragments that the four waves fetch are the same cache lines at the same time -- one
// trip to L2/HBM per kv head instead of one per query head.  The second sweep hands out its
// workgroups in the reverse order of the first, so that it starts on the K chunks that the first
// sweep touched last and finds part of K still cached.
// Arithmetic is fp32 on 16-bit inputs.  With `rounding` set (template parameter RR) every score is
// rounded where the reference's torch code rounds it on 16-bit inputs: the dot product to the input
// dtype (the einsum's result), then the product with sm_scale to the input dtype again (the division
// by sqrt(head_dim)), before the fp32 softmax (minference_forward.py:602-604).
#include "minf_common.h"
#include <math.h>
#include <type_traits>

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4_t;

constexpr int LQ = 64;          // query rows held per head (last_q <= LQ)
#ifndef EST_KC
#define EST_KC 2048
#endif
constexpr int KC = EST_KC;      // keys per workgroup
constexpr int EST_THREADS = 256;
constexpr int WIN = KC + LQ;    // diagonal window of one chunk
// A chunk is always summed as four pieces of KC/4 keys, each piece by one wave from its first key to
// its last, and the pieces are combined in ascending order -- whether one wave walks the whole chunk
// (four heads per workgroup) or four waves a piece each (one head per workgroup).  The scores of a
// head therefore do not depend, not even in the last bit, on which other heads share its launch.
constexpr int PIECE = KC / 4;
constexpr int PB = PIECE / 32;  // 32-key blocks per piece
constexpr int PWIN = PIECE + LQ;
static_assert(KC % 128 == 0, "a chunk is four pieces of whole 32-key blocks");

struct EstParams {
    const char *q, *k;
    long long qs[3], ks[3];     // element strides batch, head, token
    int batch, hq, hk, n, last_q;
    float scale_log2;
    float scale;                // sm_scale itself (the rounded form scales in the natural-log domain)
    int nchunks;
    float *stats;               // [B, Hq, nchunks, LQ, 2]
    float *win;                 // [B, Hq, nchunks, WIN]
    float *vertical, *slash;    // [B, Hq, N]
    int force_v, force_s;
    long long total_wg;
    // optional head selection: head_list[i], i < index_heads, are the query heads to score and i is
    // the head's position in the outputs and the workspace (index_heads = hq without a list)
    const int *head_list;
    int index_heads;
    int gw;                     // query heads per workgroup (waves w % gw), 4 / gw key sub-ranges each
    int nhc;                    // head groups: ceil(index_heads / gw)
};

union Frag {
    u32x4_t u;
    bf16x8_t b;
    f16x8_t h;
};

template <typename T> __device__ __forceinline__ f32x16_t mma(const Frag &a, const Frag &b, f32x16_t c);
template <> __device__ __forceinline__ f32x16_t mma<__bf16>(const Frag &a, const Frag &b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.b, b.b, c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x16_t mma<_Float16>(const Frag &a, const Frag &b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a.h, b.h, c, 0, 0, 0);
}

// Two values rounded to the 16-bit input format and back (round to nearest even; fp16 overflows to inf
// like torch's conversion): one packed conversion for the pair, then the two halves are widened again
// (bf16: a shift and a mask).
template <typename T> __device__ __forceinline__ void round_pair(float &a, float &b);
template <> __device__ __forceinline__ void round_pair<__bf16>(float &a, float &b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const bf16x2 p = __builtin_convertvector(f32x2{a, b}, bf16x2);
    const unsigned u = __builtin_bit_cast(unsigned, p);
    a = __uint_as_float(u << 16);
    b = __uint_as_float(u & 0xffff0000u);
}
template <> __device__ __forceinline__ void round_pair<_Float16>(float &a, float &b) {
    a = (float)(_Float16)a;
    b = (float)(_Float16)b;
}
// the scores the softmax sees, in the natural-log domain, rounded like the reference's bf16/fp16 torch
// ops: round(round(q.k) * sm_scale)
template <typename T> __device__ __forceinline__ void ref_logit_pair(float &a, float &b, float scale) {
    round_pair<T>(a, b);
    a *= scale;
    b *= scale;
    round_pair<T>(a, b);
}
constexpr float LOG2E = 1.4426950408889634f;

struct WgId { int b, h, hkv, chunk, slot, kq; bool valid, wave_valid; };

// Workgroup order: (batch, head group, chunk), contiguous per XCD: the chunks of one head group --
// i.e. of (mostly) one kv head -- are swept by consecutive workgroups of one XCD.  `reverse` flips
// the order (second sweep).  Wave `wave` of the workgroup gets head hc * gw + wave % gw.
__device__ __forceinline__ WgId decode_wg(const EstParams &p, int wave, bool reverse) {
    WgId w;
    const long long per_xcd = (p.total_wg + 7) >> 3;
    long long logical = (long long)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    w.valid = logical < p.total_wg;
    if (reverse) logical = p.total_wg - 1 - logical;
    const int group = p.hq / p.hk;
    long long rest = logical;
    w.chunk = (int)(rest % p.nchunks); rest /= p.nchunks;
    const int hc = (int)(rest % p.nhc);
    w.b = (int)(rest / p.nhc);
    w.kq = wave / p.gw;
    w.slot = hc * p.gw + wave % p.gw;
    w.wave_valid = w.valid && w.slot < p.index_heads;
    w.h = w.wave_valid ? (p.head_list ? p.head_list[w.slot] : w.slot) : 0;
    w.hkv = w.h / group;
    return w;
}

// Q fragments of one head: rows N-last_q+i, i = 32*blk + lane%32, d = 16*ks + 8*(lane/32) + 0..7
template <int KS>
__device__ __forceinline__ void load_q(const EstParams &p, const WgId &w, int lane, Frag (&qf)[2][KS]) {
    const int l32 = lane & 31, g = lane >> 5;
    const char *qb = p.q + ((long long)w.b * p.qs[0] + (long long)w.h * p.qs[1]) * 2;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        const int i = 32 * blk + l32;
        const int row = min(max(p.n - p.last_q + i, 0), p.n - 1);
        const char *rp = qb + (long long)row * p.qs[2] * 2 + g * 16;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[blk][ks].u = *reinterpret_cast<const u32x4_t *>(rp + ks * 32);
    }
}

// K fragments of one 32-key block starting at key c0 (rows clamped to n-1)
template <int KS>
__device__ __forceinline__ void load_k(const EstParams &p, const char *kb, int c0, int lane, Frag (&kf)[KS]) {
    const int l32 = lane & 31, g = lane >> 5;
    const int row = min(c0 + l32, p.n - 1);
    const char *rp = kb + (long long)row * p.ks[2] * 2 + g * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kf[ks].u = *reinterpret_cast<const u32x4_t *>(rp + ks * 32);
}

// K tiles shared through LDS.  When the heads of a workgroup read the same kv head (the usual
// case: the query heads of a kv group), the waves that sweep the same keys fetch every 32-key
// block of K once, together, straight into LDS (buffer_load ... lds, 16 bytes per lane, whole rows:
// fully coalesced) and read their MFMA operand fragments from there, instead of every wave
// fetching the same rows from global memory in 32-byte pieces.  Two buffers per key stream: the
// next block is on its way while this one is scored; one workgroup barrier per block.
// Rows are 2*HD bytes; their 16-byte chunks are XOR-permuted on the global-address side so that the
// fragment reads of 32 rows hit distinct banks (HD 128: chunk ^ row%16; HD 64: chunk ^ (row/2)%8).
template <int HD> struct KShare {
    static constexpr int ROWB = HD * 2, NCH = ROWB / 16, RPI = 64 / NCH, TILE = 32 * ROWB;
    static constexpr int MAXI = 16 / RPI;                    // copy instructions per wave at gw == 2
    static __device__ __forceinline__ int swz(int row) { return HD == 128 ? (row & 15) : ((row >> 1) & 7); }
    const char *kb;            // K of the common kv head
    char *tiles;               // this stream's two tiles
    long long rowstride;       // bytes
    int n, rows_w, row0_w, ninstr;
    int voff[MAXI];
    __device__ __forceinline__ void init(const EstParams &p, const char *kb_, char *tiles_, int lane, int ws) {
        kb = kb_; tiles = tiles_; rowstride = p.ks[2] * 2; n = p.n;
        rows_w = 32 / p.gw; row0_w = rows_w * ws; ninstr = rows_w / RPI;
        const int rin = lane / NCH, ch = lane % NCH;
#pragma unroll
        for (int j = 0; j < MAXI; ++j) voff[j] = rin * (int)rowstride + ((ch ^ swz(row0_w + RPI * j + rin)) << 4);
    }
    // this wave's share of the block of keys c0 .. c0+31 -> buffer `buf` (rows >= n are not fetched:
    // their scores are masked by the callers)
    __device__ __forceinline__ void copy(int c0, int buf) const {
#if defined(__HIP_DEVICE_COMPILE__)      // (the LDS-DMA builtins do not exist in the host pass, which would
                                         // then drop the kernels that use this function without a word)
        if (c0 >= n) return;
        const char *tb = kb + (long long)c0 * rowstride;
        const int nrows = min(32, n - c0);
        const __amdgpu_buffer_rsrc_t srd = __builtin_amdgcn_make_buffer_rsrc((void *)tb, 0, (nrows - 1) * (int)rowstride + ROWB, 0x00020000);
        const int lds0 = (int)(unsigned)(unsigned long long)(__attribute__((address_space(3))) char *)(tiles + buf * TILE) + row0_w * ROWB;
#pragma unroll
        for (int j = 0; j < MAXI; ++j)
            if (j < ninstr)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(srd, (__attribute__((address_space(3))) void *)(unsigned long long)(unsigned)(lds0 + RPI * j * ROWB),
                                                         16, voff[j], (row0_w + RPI * j) * (int)rowstride, 0, 0);
#endif
    }
    template <int KS> __device__ __forceinline__ void frags(int buf, int lane, Frag (&kf)[KS]) const {
        const int l32 = lane & 31, g = lane >> 5;
        const char *t = tiles + buf * TILE + l32 * ROWB;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kf[ks].u = *reinterpret_cast<const u32x4_t *>(t + (((2 * ks + g) ^ swz(l32)) << 4));
    }
};

// Do the (valid) heads of this workgroup read one kv head?  -> that head, or -1.  (All waves call
// this; it contains a workgroup barrier.)
__device__ __forceinline__ int common_kv_head(const EstParams &p, const WgId &w, int wave, int lane, int (&lds_hkv)[4]) {
    if (lane == 0) lds_hkv[wave] = w.wave_valid ? w.hkv : -1;
    __syncthreads();
    int common = -1;
    bool same = true;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int h = lds_hkv[v];
        if (h >= 0) { if (common < 0) common = h; else same = same && h == common; }
    }
    return __builtin_amdgcn_readfirstlane((p.gw >= 2 && same) ? common : -1);      // (uniform: keep it scalar)
}

// ---------------------------------------------------------------- stats sweep
template <typename T, int HD, bool RR>
__global__ __launch_bounds__(EST_THREADS, 3) void est_stats_kernel(const EstParams p) {
    constexpr int KS = HD / 16;       // k-steps of one 32x32 score block
    __shared__ float lds_m[16][LQ], lds_l[16][LQ];     // [head of the workgroup * 4 + piece][row]
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // wave-uniform: addresses built from it stay scalar
    const WgId w = decode_wg(p, wave, false);
    if (!w.valid) return;
    const int l32 = lane & 31, g = lane >> 5;
    const int nq = 4 / p.gw, klen = KC / nq;          // key sub-ranges per head, keys per wave
    const int ppw = p.gw;                             // pieces per wave (klen / PIECE)
    const int piece0 = (wave % p.gw) * 4 + w.kq * ppw; // this wave's first (head, piece) slot

    // lane <-> query rows i = l32 and 32 + l32; regs <-> keys 8*(r/4) + 4*g + r%4 of the block
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    int pieces_done = 0;
    // the running pair of a finished piece: merge the two lane halves, park it, start afresh
    auto flush_piece = [&]() {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const float mo = __shfl_xor(m_run[nb], 32), lo = __shfl_xor(l_run[nb], 32);
            const float m_new = fmaxf(m_run[nb], mo);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float l_new = l_run[nb] * __builtin_amdgcn_exp2f(m_run[nb] - m_use) + lo * __builtin_amdgcn_exp2f(mo - m_use);
            if (g == 0) {
                lds_m[piece0 + pieces_done][32 * nb + l32] = m_new;
                lds_l[piece0 + pieces_done][32 * nb + l32] = l_new;
            }
            m_run[nb] = -INFINITY;
            l_run[nb] = 0.f;
        }
        ++pieces_done;
    };
    __shared__ __attribute__((aligned(16))) char lds_kt[2][2 * KShare<HD>::TILE];
    __shared__ int lds_hkv[4];
    const int kv_common = common_kv_head(p, w, wave, lane, lds_hkv);       // (workgroup-uniform)
    Frag qf[2][KS];
    if (w.wave_valid) load_q(p, w, lane, qf);
    const int key_begin = w.chunk * KC + w.kq * klen;
    const int qpos0 = p.n - p.last_q;          // absolute position of query row 0
    const int nblk = klen / 32;
    // factor that takes a score to the log2 domain: the raw dot product needs sm_scale * log2(e), a
    // score that was already scaled and rounded only log2(e)
    const float sl2 = RR ? LOG2E : p.scale_log2;
    // scores one 32-key block whose K fragments are in kf
    auto score_block = [&](int c0, const Frag (&kf)[KS]) {
        f32x16_t st[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) st[nb][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) st[nb] = mma<T>(kf[ks], qf[nb][ks], st[nb]);
        }
        const bool edge = c0 + 31 > qpos0 || c0 + 32 > p.n;
        if constexpr (RR) {
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    float a = st[nb][r], b = st[nb][r + 1];
                    ref_logit_pair<T>(a, b, p.scale);
                    st[nb][r] = a; st[nb][r + 1] = b;
                }
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int i = 32 * nb + l32;
            // key c is visible to row i iff c <= qpos0 + i, c < n, i < last_q
            const int hi = (i < p.last_q ? min(qpos0 + i, p.n - 1) : -1) - c0 - 4 * g;
            if (edge) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int tkc = 8 * (r >> 2) + (r & 3);
                    st[nb][r] = (tkc <= hi) ? st[nb][r] : -INFINITY;
                }
            }
            // maximum of the raw scores (the scale is positive), three operands at a time
            float mx = fmaxf(fmaxf(st[nb][0], st[nb][1]), st[nb][2]);
#pragma unroll
            for (int r = 3; r + 1 < 16; r += 2) mx = fmaxf(fmaxf(mx, st[nb][r]), st[nb][r + 1]);
            mx = fmaxf(mx, st[nb][15]);
            const float m_new = fmaxf(m_run[nb], mx * sl2);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            float sum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) sum += __builtin_amdgcn_exp2f(fmaf(st[nb][r], sl2, -m_use));
            l_run[nb] = l_run[nb] * __builtin_amdgcn_exp2f(m_run[nb] - m_use) + sum;
            m_run[nb] = m_new;
        }
    };
    if (kv_common >= 0) {
        KShare<HD> ks_;
        ks_.init(p, p.k + ((long long)w.b * p.ks[0] + (long long)kv_common * p.ks[1]) * 2, lds_kt[w.kq & 1], lane, wave % p.gw);
        ks_.copy(key_begin, 0);
        for (int blk = 0; blk < nblk; ++blk) {
            const int c0 = key_begin + blk * 32;
            __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0): this wave's share of block blk is in LDS
            __syncthreads();                         // ... and everybody's; everyone is done with block blk-1
            if (blk + 1 < nblk) ks_.copy(c0 + 32, (blk + 1) & 1);
            if (w.wave_valid && c0 < p.n) {
                Frag kf[KS];
                ks_.template frags<KS>(blk & 1, lane, kf);
                score_block(c0, kf);
            }
            if (w.wave_valid && (blk + 1) % PB == 0) flush_piece();
        }
    } else if (w.wave_valid) {
        const char *kb = p.k + ((long long)w.b * p.ks[0] + (long long)w.hkv * p.ks[1]) * 2;
        Frag kf[KS], kn[KS];
        load_k(p, kb, key_begin, lane, kn);
        for (int blk = 0; blk < nblk; ++blk) {
            const int c0 = key_begin + blk * 32;
            if (c0 >= p.n) break;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kf[ks] = kn[ks];
            load_k(p, kb, min(c0 + 32, p.n - 1), lane, kn);      // next block, in flight during this one
            score_block(c0, kf);
            if ((blk + 1) % PB == 0) flush_piece();
        }
    }
    // (pieces past the end of the sequence: what is left of the running pair, then empty pairs)
    if (w.wave_valid)
        while (pieces_done < ppw) flush_piece();
    __syncthreads();
    // thread (hsub, row) folds the four pieces of head hsub's row in ascending order
    const int hsub = tid / LQ, row = tid % LQ;
    if (hsub < p.gw) {
        const WgId wh = decode_wg(p, hsub, false);
        if (wh.wave_valid) {
            float m = lds_m[hsub * 4][row], l = lds_l[hsub * 4][row];
            for (int pc = 1; pc < 4; ++pc) {
                const float mo = lds_m[hsub * 4 + pc][row], lo = lds_l[hsub * 4 + pc][row];
                const float m_new = fmaxf(m, mo);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                l = l * __builtin_amdgcn_exp2f(m - m_use) + lo * __builtin_amdgcn_exp2f(mo - m_use);
                m = m_new;
            }
            float *dst = p.stats + ((((long long)wh.b * p.index_heads + wh.slot) * p.nchunks + wh.chunk) * LQ + row) * 2;
            dst[0] = m;
            dst[1] = l;
        }
    }
}

// --------------------------------------------------------------- scores sweep
// Diagonal sums in registers.  A 32 x 32 probability block has one key per lane (n = lane % 32) and
// its rows in registers, two per register (row il in lanes 0-31, row il + 4 in lanes 32-63).
// v_permlane32_swap against a zero register turns each register into two 64-lane vectors "row il
// in lanes 0-31, zeros above"; then  acc = shift_up_one_lane(acc) + row_i  for i = 0 .. 31 (one
// v_add_f32 with the whole-wave DPP shift wave_shr:1 per row) leaves in lane L the sum of the
// diagonal n - i = L - 31: 16 swaps + 32 adds per block instead of 32 LDS writes, 64 LDS reads and
// 64 adds (LDS float atomics, tried first, run at a fraction of a lane per clock).  The 63 sums
// are added into the window of the block's piece in LDS (PIECE keys + 64 slots, private to the wave
// that walks the piece) with plain read-modify-write (one wave, in-order LDS: no race).
__device__ __forceinline__ float wave_shr1(float x) {      // lane L <- lane L - 1, lane 0 <- 0
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x138, 0xf, 0xf, true));
}

// (min 2 waves per SIMD: caps the kernel at 256 registers; it is latency bound and one resident
// wave per SIMD ran 1.4x slower)
template <typename T, int HD, bool RR>
__global__ __launch_bounds__(EST_THREADS, 2) void est_scores_kernel(const EstParams p) {
    constexpr int KS = HD / 16;
    __shared__ float lds_pwin[16][PWIN];               // [head of the workgroup * 4 + piece][slot]
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // wave-uniform: addresses built from it stay scalar
    const WgId w = decode_wg(p, wave, true);
    if (!w.valid) return;
    const int l32 = lane & 31, g = lane >> 5;
    const int nq = 4 / p.gw, klen = KC / nq;          // key sub-ranges per head, keys per wave
    const int ppw = p.gw;                             // pieces per wave (klen / PIECE)
    const long long bh = (long long)w.b * p.index_heads + w.slot;
    float *const wwin0 = lds_pwin[(wave % p.gw) * 4 + w.kq * ppw];   // this wave's ppw piece windows, contiguous

    for (int i = lane; i < ppw * PWIN; i += 64) wwin0[i] = 0.f;
    __syncthreads();

    __shared__ __attribute__((aligned(16))) char lds_kt[2][2 * KShare<HD>::TILE];
    __shared__ int lds_hkv[4];
    const int kv_common = common_kv_head(p, w, wave, lane, lds_hkv);       // (workgroup-uniform)
    Frag qf[2][KS];
    // lane <-> key; reg r of block mb <-> query row i = 32*mb + 8*(r/4) + 4*g + r%4
    float mrow[2][16];
    // Row constants M_i = max_i + log2(sum_i) of this wave's head, from the chunk statistics of the
    // first sweep (lane <-> row; every workgroup of a head repeats this small reduction instead of a
    // kernel of its own in between); rows that do not exist (i >= last_q) get +inf so that every
    // probability is 0.
    __shared__ float lds_row[4][LQ];
    if (w.wave_valid) {
        load_q(p, w, lane, qf);
        // two passes of independent loads (sixteen in flight) instead of one chain of dependent
        // rescales: the maximum over the chunks, then the sum of the chunk sums scaled to it
        const float2 *src = reinterpret_cast<const float2 *>(p.stats) + bh * p.nchunks * LQ + lane;
        float m = -INFINITY, l = 0.f;
        for (int c0 = 0; c0 < p.nchunks; c0 += 16) {
            float2 v[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) v[j] = src[(long long)min(c0 + j, p.nchunks - 1) * LQ];
#pragma unroll
            for (int j = 0; j < 16; ++j) m = fmaxf(m, v[j].x);
        }
        const float m_use = (m == -INFINITY) ? 0.f : m;
        for (int c0 = 0; c0 < p.nchunks; c0 += 16) {
            float2 v[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) v[j] = src[(long long)min(c0 + j, p.nchunks - 1) * LQ];
#pragma unroll
            for (int j = 0; j < 16; ++j) l += (c0 + j < p.nchunks) ? v[j].y * __builtin_amdgcn_exp2f(v[j].x - m_use) : 0.f;
        }
        lds_row[wave][lane] = (lane < p.last_q && l > 0.f) ? m + __builtin_amdgcn_logf(l) : INFINITY;
    }
    __syncthreads();
    if (w.wave_valid) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                mrow[mb][r] = lds_row[wave][32 * mb + 8 * (r >> 2) + 4 * g + (r & 3)];
    }
    const int key_begin = w.chunk * KC + w.kq * klen;
    const int qpos0 = p.n - p.last_q;
    const int rshift = LQ - p.last_q;          // rows are indexed as if last_q were 64
    float *vout = p.vertical + bh * p.n;
    const int nblk = klen / 32;
    // scores one 32-key block whose K fragments are in kf -> this lane's column sum (both lane halves)
    auto score_block = [&](int blk, int c0, const Frag (&kf)[KS]) -> float {
        // The block adds to 95 slots of the diagonal window, as two disjoint ranges: s1 + (0..63) and,
        // in lanes 32..62, s2 = s1 + 32.  Their old values are read now, a block's work ahead of the
        // add (window slot of lane L, row half mb: 32*blk + L + 32 - 32*mb - rshift = key - row + 63 - rshift).
        float *const wwin = wwin0 + (blk / PB) * PWIN;                  // the window of this block's piece
        const int s1 = 32 * (blk % PB) + lane - rshift, s2 = s1 + 32;
        const bool ok1 = s1 >= 0, ok2 = lane >= 32 && lane < 63 && s2 >= 0;
        const float w1 = ok1 ? wwin[s1] : 0.f;
        const float w2 = ok2 ? wwin[s2] : 0.f;
        const int c = c0 + l32;                 // this lane's key
        const bool edge = c0 + 31 > qpos0 || c0 + 32 > p.n;
        float colsum = 0.f;
        float pr[2][16];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
            f32x16_t sc;
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) sc = mma<T>(qf[mb][ks], kf[ks], sc);
            if constexpr (RR) {
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    float a = sc[r], b = sc[r + 1];
                    ref_logit_pair<T>(a, b, p.scale);
                    sc[r] = a; sc[r + 1] = b;
                }
            }
            const float sl2 = RR ? LOG2E : p.scale_log2;
#pragma unroll
            for (int r = 0; r < 16; ++r) pr[mb][r] = __builtin_amdgcn_exp2f(fmaf(sc[r], sl2, -mrow[mb][r]));
        }
        if (edge) {      // (a block of its own, kept one by the empty asm: merged into the straight-line code
                         // the 32 compares and selects would run for every block)
            asm volatile("");
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int i = 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);      // query row
                    pr[mb][r] = (c <= qpos0 + i && c < p.n) ? pr[mb][r] : 0.f;
                }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) colsum += pr[0][r] + pr[1][r];
        // the 63 diagonals d = n - il in [-31, 31] of each 32 x 32 block: rows in ascending order,
        // one lane shift between two rows, the two blocks' chains interleaved
        float dacc[2] = {0.f, 0.f};
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            float lo[2][4], hi[2][4];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(pr[mb][4 * q4 + j]), 0u, false, false);
                    lo[mb][j] = __uint_as_float(sw[0]);      // row 8*q4 + j     in lanes 0-31, zeros above
                    hi[mb][j] = __uint_as_float(sw[1]);      // row 8*q4 + 4 + j in lanes 0-31, zeros above
                }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) dacc[mb] = wave_shr1(dacc[mb]) + lo[mb][j];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) dacc[mb] = wave_shr1(dacc[mb]) + hi[mb][j];
        }
        // lane L of dacc[mb] is diagonal d = L - 31 of row half mb (lane 63 holds nothing).  Half 1 goes
        // to s1 + L; half 0 lies 32 slots higher: its lanes 0..31 join the upper lanes of half 1, its
        // lanes 32..62 go to s2.
        {
            auto sw = __builtin_amdgcn_permlane32_swap(0u, __float_as_uint(dacc[0]), false, false);
            const float v1 = dacc[1] + __uint_as_float(sw[0]);      // (0 | lanes 0..31 of half 0)
            if (ok1) wwin[s1] = w1 + v1;
            if (ok2) wwin[s2] = w2 + dacc[0];
        }
        return colsum + __shfl_xor(colsum, 32);
    };
    if (kv_common >= 0) {
        KShare<HD> ks_;
        ks_.init(p, p.k + ((long long)w.b * p.ks[0] + (long long)kv_common * p.ks[1]) * 2, lds_kt[w.kq & 1], lane, wave % p.gw);
        ks_.copy(key_begin, 0);
        float cs_prev = 0.f;                         // column sum of the previous block, stored a block later
        int c_prev = -1;                             // (so that no store is waited for with the copies)
        for (int blk = 0; blk < nblk; ++blk) {
            const int c0 = key_begin + blk * 32;
            __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0): this wave's share of block blk is in LDS
            __syncthreads();                         // ... and everybody's; everyone is done with block blk-1
            if (c_prev >= 0 && g == 0 && c_prev < p.n) vout[c_prev] = cs_prev;
            if (blk + 1 < nblk) ks_.copy(c0 + 32, (blk + 1) & 1);
            c_prev = -1;
            if (w.wave_valid && c0 < p.n) {
                Frag kf[KS];
                ks_.template frags<KS>(blk & 1, lane, kf);
                cs_prev = score_block(blk, c0, kf);
                c_prev = c0 + l32;
            }
        }
        if (c_prev >= 0 && g == 0 && c_prev < p.n) vout[c_prev] = cs_prev;
    } else if (w.wave_valid) {
        const char *kb = p.k + ((long long)w.b * p.ks[0] + (long long)w.hkv * p.ks[1]) * 2;
        Frag kf[KS], kn[KS];
        load_k(p, kb, key_begin, lane, kn);
        for (int blk = 0; blk < nblk; ++blk) {
            const int c0 = key_begin + blk * 32;
            if (c0 >= p.n) break;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kf[ks] = kn[ks];
            load_k(p, kb, min(c0 + 32, p.n - 1), lane, kn);      // next block, in flight during this one
            const float cs = score_block(blk, c0, kf);
            if (g == 0 && c0 + l32 < p.n) vout[c0 + l32] = cs;
        }
    }
    __syncthreads();
    // chunk window of head hsub, position q = (key - chunk0) + (last_q - 1 - i): piece pc contributes
    // its slot q - pc * PIECE; the pieces are added in ascending order
    for (int idx = tid; idx < p.gw * WIN; idx += EST_THREADS) {
        const int hsub = idx / WIN, q = idx - hsub * WIN;
        const WgId wh = decode_wg(p, hsub, true);
        if (!wh.wave_valid) continue;
        float acc = 0.f;
        for (int pc = 0; pc < 4; ++pc) {
            const int sl = q - pc * PIECE;
            if (sl >= 0 && sl < PWIN) acc += lds_pwin[hsub * 4 + pc][sl];
        }
        p.win[(((long long)wh.b * p.index_heads + wh.slot) * p.nchunks + wh.chunk) * WIN + q] = acc;
    }
}

// ------------------------------------------------------------------- finalize
__global__ __launch_bounds__(256) void est_finalize_kernel(const EstParams p) {
    const long long bh = blockIdx.y;
    const int j = (int)(blockIdx.x * 256 + threadIdx.x);
    if (j >= p.n) return;
    const int c = j / KC, off = j - c * KC;
    const float *wbase = p.win + bh * p.nchunks * WIN;
    // diagonal j lives at window position `off` of chunk c and, when off < LQ, also at
    // position KC + off of chunk c-1 (keys of the previous chunk seen by later rows)
    float v = wbase[(long long)c * WIN + off];
    if (c > 0 && off < LQ) v = wbase[(long long)(c - 1) * WIN + KC + off] + v;
    if (p.force_s > 0 && j >= p.n - p.force_s) v = INFINITY;
    p.slash[bh * p.n + j] = v;
    if (j < p.force_v) p.vertical[bh * p.n + j] = INFINITY;
}

int fill(EstParams &p, const void *q, const void *k, const int64_t *q_stride, const int64_t *k_stride,
         int batch, int heads_q, int heads_kv, int n, int head_dim, int dtype, float sm_scale,
         int last_q, int force_v, int force_s, float *vertical, float *slash, void *ws, size_t ws_bytes,
         const int32_t *head_list, int index_heads) {
    if (!q || !k || !vertical || !slash || !ws) return MINF_ERR_INVALID_ARG;
    if (head_list && index_heads <= 0) return MINF_ERR_INVALID_ARG;
    if (!head_list) index_heads = heads_q;
    if (batch < 0 || heads_q <= 0 || heads_kv <= 0 || n <= 0 || heads_q % heads_kv) return MINF_ERR_INVALID_ARG;
    if ((head_dim != 128 && head_dim != 64) || (dtype != MINF_BF16 && dtype != MINF_F16)) return MINF_ERR_UNSUPPORTED;
    if (last_q < 1 || last_q > LQ || force_v < 0 || force_s < 0) return MINF_ERR_INVALID_ARG;
    if (((uintptr_t)q & 15) || ((uintptr_t)k & 15)) return MINF_ERR_ALIGNMENT;
    for (int j = 0; j < 3; ++j)
        if ((q_stride[j] & 7) || (k_stride[j] & 7)) return MINF_ERR_ALIGNMENT;
    p.q = (const char *)q; p.k = (const char *)k;
    for (int j = 0; j < 3; ++j) { p.qs[j] = q_stride[j]; p.ks[j] = k_stride[j]; }
    p.batch = batch; p.hq = heads_q; p.hk = heads_kv; p.n = n;
    p.last_q = last_q < n ? last_q : n;
    p.scale_log2 = sm_scale * 1.4426950408889634f;
    p.scale = sm_scale;
    p.nchunks = (n + KC - 1) / KC;
    const long long bh = (long long)batch * index_heads;
    const size_t stats_b = (size_t)bh * p.nchunks * LQ * 2 * sizeof(float);
    const size_t win_b = (size_t)bh * p.nchunks * WIN * sizeof(float);
    if (ws_bytes < stats_b + win_b) return MINF_ERR_WORKSPACE;
    if ((uintptr_t)ws & 15) return MINF_ERR_ALIGNMENT;
    p.stats = (float *)ws;
    p.win = (float *)((char *)ws + stats_b);
    p.vertical = vertical; p.slash = slash;
    p.force_v = force_v; p.force_s = force_s;
    // heads per workgroup: neighbours in head order that (mostly) share a kv head
    const int group = heads_q / heads_kv;
    p.gw = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
    p.nhc = (index_heads + p.gw - 1) / p.gw;
    p.total_wg = (long long)batch * p.nhc * p.nchunks;
    p.head_list = head_list;
    p.index_heads = index_heads;
    return MINF_OK;
}

}  // namespace

extern "C" size_t minf_vs_estimate_workspace_bytes(int batch, int heads_q, int n) {
    if (batch <= 0 || heads_q <= 0 || n <= 0) return 0;
    const size_t bh = (size_t)batch * heads_q;
    const size_t nchunks = ((size_t)n + KC - 1) / KC;
    return bh * nchunks * LQ * 2 * sizeof(float) + bh * nchunks * WIN * sizeof(float);
}

static int estimate_launch(const void *q, const void *k, const int64_t *q_stride, const int64_t *k_stride,
                           int batch, int heads_q, int heads_kv, int n, int head_dim, int dtype, float sm_scale,
                           int last_q, int force_vertical, int force_slash, float *vertical, float *slash,
                           void *workspace, size_t workspace_bytes, const int32_t *head_list, int index_heads,
                           int rounding, void *stream) {
    EstParams p;
    if (rounding != MINF_ROUND_NONE && rounding != MINF_ROUND_INPUT_DTYPE) return MINF_ERR_INVALID_ARG;
    if (batch == 0) return MINF_OK;
    int st = fill(p, q, k, q_stride, k_stride, batch, heads_q, heads_kv, n, head_dim, dtype, sm_scale,
                  last_q, force_vertical, force_slash, vertical, slash, workspace, workspace_bytes,
                  head_list, index_heads);
    if (st) return st;
    const long long grid = ((p.total_wg + 7) >> 3) * 8;
    if (grid > 0x7fffffffLL) return MINF_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const long long bh = (long long)batch * p.index_heads;       // heads of the outputs
    const bool bf = dtype == MINF_BF16;
    const dim3 g((unsigned)grid), b(EST_THREADS);
    // (plain launches: a kernel template whose body holds lambdas is not instantiated for the host
    // when its address is only taken inside a generic lambda)
#define EST_LAUNCH_RR(kernel, RR)                                                                   \
    do {                                                                                            \
        if (head_dim == 128) {                                                                      \
            if (bf) hipLaunchKernelGGL((kernel<__bf16, 128, RR>), g, b, 0, s, p);                   \
            else hipLaunchKernelGGL((kernel<_Float16, 128, RR>), g, b, 0, s, p);                    \
        } else {                                                                                    \
            if (bf) hipLaunchKernelGGL((kernel<__bf16, 64, RR>), g, b, 0, s, p);                    \
            else hipLaunchKernelGGL((kernel<_Float16, 64, RR>), g, b, 0, s, p);                     \
        }                                                                                           \
    } while (0)
#define EST_LAUNCH(kernel)                                                                          \
    do {                                                                                            \
        if (rounding == MINF_ROUND_INPUT_DTYPE) EST_LAUNCH_RR(kernel, true);                        \
        else EST_LAUNCH_RR(kernel, false);                                                          \
    } while (0)
    EST_LAUNCH(est_stats_kernel);
    EST_LAUNCH(est_scores_kernel);
    hipLaunchKernelGGL(est_finalize_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)bh), dim3(256), 0, s, p);
#undef EST_LAUNCH
#undef EST_LAUNCH_RR
    return minf_launch_status();
}

extern "C" int minf_vs_estimate(const void *q, const void *k, const int64_t *q_stride,
                                const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                                int head_dim, int dtype, float sm_scale, int last_q, int force_vertical,
                                int force_slash, int rounding, float *vertical, float *slash, void *workspace,
                                size_t workspace_bytes, void *stream) {
    return estimate_launch(q, k, q_stride, k_stride, batch, heads_q, heads_kv, n, head_dim, dtype, sm_scale, last_q,
                           force_vertical, force_slash, vertical, slash, workspace, workspace_bytes, nullptr, 0,
                           rounding, stream);
}

extern "C" int minf_vs_estimate_heads(const void *q, const void *k, const int64_t *q_stride,
                                      const int64_t *k_stride, int batch, int heads_q, int heads_kv, int n,
                                      int head_dim, int dtype, float sm_scale, int last_q, int force_vertical,
                                      int force_slash, int rounding, const int32_t *head_list, int index_heads,
                                      float *vertical, float *slash, void *workspace,
                                      size_t workspace_bytes, void *stream) {
    if (!head_list) return MINF_ERR_INVALID_ARG;
    return estimate_launch(q, k, q_stride, k_stride, batch, heads_q, heads_kv, n, head_dim, dtype, sm_scale, last_q,
                           force_vertical, force_slash, vertical, slash, workspace, workspace_bytes, head_list,
                           index_heads, rounding, stream);
}
