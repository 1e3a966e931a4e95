// Block index of block-sparse attention for gfx950: mean-pool Q and K over 64-token blocks,
// score every (query block, key block) pair with the pooled vectors, keep the top-k key blocks
// per query block in ascending order (reference
// minference/ops/block_sparse_flash_attention.py:151-166, with the zero padding of :178-180
// folded in: the token axis is padded by 64 - n%64 zeros, a whole block when n%64 == 0).
//
//   bs_pool_kernel    one workgroup per (head, block): 64 rows x 128 dims of 16-bit input summed in
//                     fp32 (each thread 4 rows x 8 dims, then a fixed-order LDS reduction) -> mean.
//                     HBM-bound: reads Q and K once.
//   bs_scores_kernel  pooled Q . pooled K^T on the fp32 matrix cores (v_mfma_f32_32x32x2_f32), one
//                     wave per 32 query blocks x 32 key blocks, operands loaded straight from global
//                     memory in MFMA layout; applies the block-causal mask (-inf above the diagonal)
//                     and, optionally, forces the diagonal block and block 0 (+inf).
//   top-k             the shared radix-select kernel (ascending index order, ties -> lowest index).
//
// Arithmetic is fp32; with MINF_BS_ROUND_INPUT_DTYPE the pooled means and the pooled dot products
// are rounded to the input dtype, where the reference's torch code rounds them (its `mean` and
// `einsum` return bf16/fp16 tensors).
#include "minf_common.h"
#include <math.h>

extern "C" int minf_topk_indices(const float *scores, int rows, int n, int64_t row_stride, int k,
                                 int32_t *out, int64_t out_stride, int reverse_base, void *stream);
extern "C" int minf_topk_indices_block_causal(const float *scores, int rows, int n, int64_t row_stride, int k,
                                              int32_t *out, int64_t out_stride, int rows_per_head, void *stream);

namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4_t;

constexpr int HD = 128;
constexpr int BLK = 64;

struct PoolParams {
    const char *x;            // [batch, heads, n, hd] 16-bit, element strides below
    long long xs[3];
    int hd;                   // 64 or 128 input dims; the pooled rows are always 128 wide (zeros above hd)
    float *out;               // [batch*heads, rows, 128] fp32
    int heads, n, rows;
    int blk;                  // tokens per block: 64 or 32
    // optional head selection: `out` has out_heads heads and head i of it is head head_list[i] of x
    // (without a list: out_heads = heads, same numbering)
    const int *head_list;
    int out_heads;
    int round_out;            // round the means to the input dtype (stored as fp32 all the same)
};

template <typename T> __device__ __forceinline__ float to_f32(unsigned short bits);
template <> __device__ __forceinline__ float to_f32<__bf16>(unsigned short bits) {
    return __uint_as_float((unsigned)bits << 16);
}
template <> __device__ __forceinline__ float to_f32<_Float16>(unsigned short bits) {
    union { unsigned short u; _Float16 h; } c;
    c.u = bits;
    return (float)c.h;
}

template <typename T> __global__ __launch_bounds__(256) void bs_pool_kernel(const PoolParams p) {
    __shared__ float red[16][HD + 4];
    const int blk = blockIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / p.out_heads, slot = bh % p.out_heads;      // (grid: batch x out_heads)
    const int h = p.head_list ? p.head_list[slot] : slot;
    const int tid = (int)threadIdx.x;
    const int c = tid & 15, r4 = tid >> 4;
    const char *base = p.x + ((long long)b * p.xs[0] + (long long)h * p.xs[1]) * 2;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int tok = blk * p.blk + r4 + 16 * j;
        if (16 * j < p.blk && tok < p.n && c * 8 < p.hd) {
            const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(base + (long long)tok * p.xs[2] * 2 + c * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[2 * e] += to_f32<T>((unsigned short)(raw[e] & 0xffffu));
                acc[2 * e + 1] += to_f32<T>((unsigned short)(raw[e] >> 16));
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) red[r4][c * 8 + e] = acc[e];
    __syncthreads();
    if (tid < HD) {
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) s += red[r][tid];
        float mean = s / (float)p.blk;
        if (p.round_out) mean = (float)(T)mean;
        p.out[(((long long)b * p.out_heads + slot) * p.rows + blk) * HD + tid] = mean;
    }
}

constexpr int SCORE_CHUNK = 16;

struct ScoreParams {
    const float *qp, *kp;     // pooled [batch*heads_q, rows, 128], [batch*heads_kv, rows, 128]
    float *scores;            // [batch*heads_q, rows, pitch]
    int heads_q, heads_kv, rows, pitch, force;
    int mtiles, ntiles;
    int mquads;               // groups of four query tiles (one workgroup each per chunk)
    int nchunks;              // chunks of SCORE_CHUNK key tiles per group
    int skip_masked;
    const int *head_list;     // as in PoolParams; qp and scores have index_heads heads
    int index_heads;
    int round_dtype;          // -1: keep fp32 scores; MINF_BF16 / MINF_F16: round every score to that format
};

// lane l supplies row l%32 and, for MFMA step (s, j), contraction index 8*s + 4*(l/32) + j:
// sixteen 16-byte loads cover the lane's half of the 128-dim row.
__device__ __forceinline__ void load_operand(const float *base, int row, int rows, int g, f32x4_t (&x)[16]) {
    const float *src = base + (long long)min(row, rows - 1) * HD + 4 * g;
#pragma unroll
    for (int s = 0; s < 16; ++s) x[s] = *reinterpret_cast<const f32x4_t *>(src + 8 * s);
}

// One workgroup: four query tiles (one per wave, A operand held in registers) against one chunk of
// SCORE_CHUNK key tiles.  A key tile (32 pooled rows = 16 KB, contiguous in memory) is loaded once
// per workgroup with coalesced 16-byte loads, staged in LDS (two buffers, rows padded by 16 bytes so
// that the operand reads spread over the banks) and read from there by all four waves in MFMA
// layout: the matrix instructions then wait for LDS, whose latency two reads in flight cover, and
// not for L2 -- with the operand read straight from global memory the compiler keeps two of the
// sixteen loads in flight and the matrix pipe was 45 % busy.
constexpr int SCORE_PITCH = HD + 4;            // floats per staged row
__global__ __launch_bounds__(256, 3) void bs_scores_kernel(const ScoreParams p) {
    __shared__ __attribute__((aligned(16))) float lds_b[2][32 * SCORE_PITCH];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, g = lane >> 5;
    const int mq = p.mquads - 1 - (int)blockIdx.x / p.nchunks;    // heavy (late) query tiles first
    const int nt_begin = ((int)blockIdx.x % p.nchunks) * SCORE_CHUNK;
    const int bh = blockIdx.y;
    const int b = bh / p.index_heads, slot = bh % p.index_heads;   // (grid: batch x index_heads)
    const int h = p.head_list ? p.head_list[slot] : slot;
    const int hkv = h / (p.heads_q / p.heads_kv);
    const long long bs = bh;
    const float *qbase = p.qp + bs * p.rows * HD;
    const float *kbase = p.kp + ((long long)b * p.heads_kv + hkv) * p.rows * HD;
    float *out = p.scores + bs * p.rows * p.pitch;
    const int mt = 4 * mq + wave;                                  // this wave's query tile (may not exist)
    const int m0 = mt * 32;
    const bool have_q = mt < p.mtiles;
    // tiles wholly above the diagonal hold only -inf: when the selection that follows knows that
    // (rows of at most 4096 scores), they are neither computed nor stored; otherwise they are stored
    // without arithmetic.  The workgroup walks up to the last tile any of its waves needs.
    const int last_any = min(p.ntiles - 1, (min(4 * mq + 3, p.mtiles - 1) * 32 + 31) / 32);
    const int nt_stop = min(nt_begin + SCORE_CHUNK, p.skip_masked ? last_any + 1 : p.ntiles);
    if (nt_begin >= nt_stop) return;                               // (workgroup-uniform)
    const int last_mine = (m0 + 31) / 32;                          // last tile this wave computes

    f32x4_t aq[16];
    if (have_q) load_operand(qbase, m0 + l32, p.rows, g, aq);      // A operand: query blocks -> accumulator rows
    // staging: thread t moves the four 16-byte pieces t, t + 256, ... of the 16 KB tile
    auto fetch = [&](int nt, f32x4_t (&st)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int f = i * 256 + tid;                           // piece: row f / 32, floats 4 * (f % 32) ..
            const int row = min(nt * 32 + (f >> 5), p.rows - 1);
            st[i] = *reinterpret_cast<const f32x4_t *>(kbase + (long long)row * HD + 4 * (f & 31));
        }
    };
    auto stage = [&](int buf, const f32x4_t (&st)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int f = i * 256 + tid;
            *reinterpret_cast<f32x4_t *>(&lds_b[buf][(f >> 5) * SCORE_PITCH + 4 * (f & 31)]) = st[i];
        }
    };
    f32x4_t st[4];
    fetch(nt_begin, st);
    stage(0, st);
    for (int nt = nt_begin; nt < nt_stop; ++nt) {
        const int buf = (nt - nt_begin) & 1;
        __syncthreads();                       // tile nt is staged; everyone is done with tile nt - 1
        const bool more = nt + 1 < nt_stop;
        if (more) fetch(nt + 1, st);           // in flight during this tile's arithmetic
        const int n0 = nt * 32;
        if (have_q && !(p.skip_masked && nt > last_mine)) {
            f32x16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            if (nt <= last_mine) {
                // B operand: key blocks -> accumulator columns; lane l reads row l%32, floats 8 s + 4 g ..
                const float *brow = &lds_b[buf][l32 * SCORE_PITCH + 4 * g];
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    const f32x4_t bk = *reinterpret_cast<const f32x4_t *>(brow + 8 * s);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[s][j], bk[j], acc, 0, 0, 0);
                }
            }
            // accumulator element r of lane l: query block m0 + 8*(r/4) + 4*g + r%4, key block n0 + l%32,
            // so every store instruction writes two full 128-byte row segments
            const int ncol = n0 + l32;
            if (ncol < p.pitch) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int mrow = m0 + 8 * (r >> 2) + 4 * g + (r & 3);
                    float v = acc[r];
                    if (p.round_dtype == MINF_BF16) v = (float)(__bf16)v;
                    else if (p.round_dtype == MINF_F16) v = (float)(_Float16)v;
                    float x = ncol <= mrow ? v : -INFINITY;
                    if (p.force && (ncol == mrow || ncol == 0)) x = INFINITY;
                    if (mrow < p.rows) out[(long long)mrow * p.pitch + ncol] = x;
                }
            }
        }
        if (more) stage(buf ^ 1, st);          // (that buffer was last read for tile nt - 1)
    }
}

inline int padded_rows(int n) { return (n + (BLK - (n & (BLK - 1)))) / BLK; }
inline int score_pitch(int rows) { return (rows + 3) & ~3; }
inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
inline size_t workspace_for(int batch, int heads_q, int heads_kv, int rows) {
    return align256((size_t)batch * heads_q * rows * HD * 4) + align256((size_t)batch * heads_kv * rows * HD * 4) +
           align256((size_t)batch * heads_q * rows * score_pitch(rows) * 4);
}

}  // namespace

extern "C" int minf_bs_block_index_rows(int n) { return n < 0 ? 0 : padded_rows(n); }

namespace {

int block_index_impl(const void *q, const void *k, const int64_t *q_stride, const int64_t *k_stride, int batch,
                     int heads_q, int heads_kv, int n, int head_dim, int dtype, int blk, int rows, int top_k,
                     int flags, int32_t *block_index, void *workspace, size_t workspace_bytes,
                     void *stream, const int32_t *head_list = nullptr, int index_heads = 0) {
    if (!q || !k || !q_stride || !k_stride || !block_index) return MINF_ERR_INVALID_ARG;
    if (head_list && index_heads <= 0) return MINF_ERR_INVALID_ARG;
    if (!head_list) index_heads = heads_q;
    if (batch < 0 || heads_q <= 0 || heads_kv <= 0 || n <= 0 || top_k <= 0) return MINF_ERR_INVALID_ARG;
    if (heads_q % heads_kv != 0) return MINF_ERR_INVALID_ARG;
    if (flags & ~(MINF_BS_FORCE_DIAG_FIRST | MINF_BS_ROUND_INPUT_DTYPE)) return MINF_ERR_INVALID_ARG;
    const int force_diag_first = flags & MINF_BS_FORCE_DIAG_FIRST;
    const int rounded = (flags & MINF_BS_ROUND_INPUT_DTYPE) ? 1 : 0;
    if (head_dim != HD && head_dim != 64) return MINF_ERR_UNSUPPORTED;
    if (dtype != MINF_BF16 && dtype != MINF_F16) return MINF_ERR_UNSUPPORTED;
    if (((uintptr_t)q | (uintptr_t)k) & 15) return MINF_ERR_ALIGNMENT;
    for (int i = 0; i < 3; ++i)
        if ((q_stride[i] | k_stride[i]) & 7) return MINF_ERR_ALIGNMENT;
    if (batch == 0) return MINF_OK;
    const size_t need = workspace_for(batch, index_heads, heads_kv, rows);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15)) return MINF_ERR_WORKSPACE;
    const int pitch = score_pitch(rows);
    if ((long long)batch * index_heads * rows > 0x7fffffffLL || (long long)batch * index_heads > 65535) return MINF_ERR_UNSUPPORTED;

    char *ws = (char *)workspace;
    float *qp = (float *)ws;
    ws += align256((size_t)batch * index_heads * rows * HD * 4);
    float *kp = (float *)ws;
    ws += align256((size_t)batch * heads_kv * rows * HD * 4);
    float *scores = (float *)ws;
    hipStream_t st = (hipStream_t)stream;

    PoolParams pq{(const char *)q, {q_stride[0], q_stride[1], q_stride[2]}, head_dim, qp, heads_q, n, rows, blk, head_list, index_heads, rounded};
    PoolParams pk{(const char *)k, {k_stride[0], k_stride[1], k_stride[2]}, head_dim, kp, heads_kv, n, rows, blk, nullptr, heads_kv, rounded};
    if (dtype == MINF_BF16) {
        hipLaunchKernelGGL(bs_pool_kernel<__bf16>, dim3(rows, batch * index_heads), dim3(256), 0, st, pq);
        hipLaunchKernelGGL(bs_pool_kernel<__bf16>, dim3(rows, batch * heads_kv), dim3(256), 0, st, pk);
    } else {
        hipLaunchKernelGGL(bs_pool_kernel<_Float16>, dim3(rows, batch * index_heads), dim3(256), 0, st, pq);
        hipLaunchKernelGGL(bs_pool_kernel<_Float16>, dim3(rows, batch * heads_kv), dim3(256), 0, st, pk);
    }
    int status = minf_launch_status();
    if (status != MINF_OK) return status;

    const bool causal_topk = rows <= 64 * 64;      // one wave per row: reads only the stored prefix of a row
    ScoreParams sp{qp, kp, scores, heads_q, heads_kv, rows, pitch, force_diag_first ? 1 : 0,
                   (rows + 31) / 32, (pitch + 31) / 32, ((rows + 31) / 32 + 3) / 4,
                   ((pitch + 31) / 32 + SCORE_CHUNK - 1) / SCORE_CHUNK, causal_topk ? 1 : 0, head_list, index_heads,
                   rounded ? dtype : -1};
    hipLaunchKernelGGL(bs_scores_kernel, dim3(sp.mquads * sp.nchunks, batch * index_heads), dim3(256), 0, st, sp);
    status = minf_launch_status();
    if (status != MINF_OK) return status;

    const int kk = top_k < rows ? top_k : rows;
    if (causal_topk)
        return minf_topk_indices_block_causal(scores, batch * index_heads * rows, rows, pitch, kk, block_index, kk, rows, stream);
    return minf_topk_indices(scores, batch * index_heads * rows, rows, pitch, kk, block_index, kk, -1, stream);
}

}  // namespace

extern "C" size_t minf_bs_block_index_workspace_bytes(int batch, int heads_q, int heads_kv, int n) {
    if (batch <= 0 || heads_q <= 0 || heads_kv <= 0 || n <= 0) return 0;
    return workspace_for(batch, heads_q, heads_kv, padded_rows(n));
}

extern "C" int minf_bs_block_index(const void *q, const void *k, const int64_t *q_stride,
                                   const int64_t *k_stride, int batch, int heads_q, int heads_kv,
                                   int n, int head_dim, int dtype, int top_k, int flags,
                                   int32_t *block_index, void *workspace, size_t workspace_bytes,
                                   void *stream) {
    return block_index_impl(q, k, q_stride, k_stride, batch, heads_q, heads_kv, n, head_dim, dtype, BLK,
                            n > 0 ? padded_rows(n) : 0, top_k, flags, block_index, workspace,
                            workspace_bytes, stream);
}

extern "C" int minf_bs_block_index_heads(const void *q, const void *k, const int64_t *q_stride,
                                         const int64_t *k_stride, int batch, int heads_q, int heads_kv,
                                         int n, int head_dim, int dtype, int top_k, int flags,
                                         const int32_t *head_list, int index_heads,
                                         int32_t *block_index, void *workspace, size_t workspace_bytes,
                                         void *stream) {
    if (!head_list) return MINF_ERR_INVALID_ARG;
    return block_index_impl(q, k, q_stride, k_stride, batch, heads_q, heads_kv, n, head_dim, dtype, BLK,
                            n > 0 ? padded_rows(n) : 0, top_k, flags, block_index, workspace,
                            workspace_bytes, stream, head_list, index_heads);
}
extern "C" size_t minf_search_block_index_workspace_bytes(int batch, int heads_q, int heads_kv, int n) {
    if (batch <= 0 || heads_q <= 0 || heads_kv <= 0 || n <= 0) return 0;
    return workspace_for(batch, heads_q, heads_kv, (n + 31) / 32);
}

extern "C" int minf_search_block_index(const void *q, const void *k, const int64_t *q_stride,
                                       const int64_t *k_stride, int batch, int heads_q, int heads_kv,
                                       int n, int head_dim, int dtype, int top_k, int32_t *block_index,
                                       void *workspace, size_t workspace_bytes, void *stream) {
    return block_index_impl(q, k, q_stride, k_stride, batch, heads_q, heads_kv, n, head_dim, dtype, 32,
                            n > 0 ? (n + 31) / 32 : 0, top_k, 0, block_index, workspace, workspace_bytes, stream);
}
