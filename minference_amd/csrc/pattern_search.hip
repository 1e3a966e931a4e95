// Offline pattern search for gfx950: how much of the exact causal softmax mass does a candidate
// sparse pattern keep?  (reference minference/modules/minference_forward.py:129-227, where the
// whole N x N probability matrix is materialised and multiplied by N x N masks).
//
// Here nothing of size N x N exists.  A candidate is described by three flag arrays per head, one
// bit per candidate (up to 8 candidates are scored in one sweep):
//   col_flags[c]        bit t set: candidate t keeps key column c              (verticals, sinks)
//   diag_flags[o]       bit t set: candidate t keeps the diagonal query - key = o  (slashes, windows)
//   block_flags[R][C]   bit t set: candidate t keeps the 32 x 32 block (R, C)  (block-sparse)
// and element (r, c), c <= r, belongs to candidate t iff any of its three bits t is set.
//
//   pattern_recall_kernel  one workgroup per (head, 64 query rows), heavy row tiles first; its 4
//                     waves split the causal key blocks (32 keys each).  S^T = K.Q^T on
//                     v_mfma_f32_32x32x16 with fragments read straight from global memory in
//                     operand layout: lane <-> query row, registers <-> keys, so the running
//                     maximum, the running sum of exponentials and the 8 running masked sums are
//                     per-lane registers (online softmax, rescaled whenever the maximum grows).
//                     Lanes, then waves, are merged through LDS; the row tile's sum of
//                     masked/total ratios over its rows >= row_begin goes to a partial buffer.
//   pattern_recall_finalize  sums the partials of a head in a fixed order and divides by the
//                     number of rows (deterministic; no atomics).
//   flags_set_indices / flags_set_range  build the flag arrays from top-k index lists / ranges.
#include "minf_common.h"
#include <math.h>

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4_t;

constexpr int HD = 128;
constexpr int NC = 8;            // candidates per sweep (bits of a flag byte)
constexpr int TILE = 64;         // query rows per workgroup
constexpr int KB = 32;           // keys per block

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

struct RecallParams {
    const char *q, *k;
    long long qs[3], ks[3];      // element strides batch, head, token
    int hq, hk, n;
    float scale_log2;
    const unsigned char *col, *diag, *blk;   // blk may be null
    long long flag_pitch;        // bytes between heads of col / diag (>= n rounded up to 64)
    long long blk_pitch;         // bytes between block rows; a head has ceil(n/32) block rows
    int row_begin, tiles;
    float *partial;              // [batch*hq, tiles, NC]
};

// rows of one 32-row block of one head (or keys of a key block): row = first + lane%32, clamped;
// d = 16*ks + 8*(lane/32) + 0..7
__device__ __forceinline__ void load_frag(const char *base, long long tok_stride, int first, int n, int lane,
                                          Frag (&f)[8]) {
    const int row = min(first + (lane & 31), n - 1);
    const char *rp = base + (long long)row * tok_stride * 2 + (lane >> 5) * 16;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) f[ks].u = *reinterpret_cast<const u32x4_t *>(rp + ks * 32);
}

__device__ __forceinline__ unsigned load_u32_unaligned(const unsigned char *p) {
    unsigned w;
    __builtin_memcpy(&w, p, 4);
    return w;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct RowState {
    float m, z, zm[NC];
};

__device__ __forceinline__ void merge_into(RowState &a, float m, float z, const float (&zm)[NC]) {
    const float mn = fmaxf(a.m, m);
    const float mu = mn == -INFINITY ? 0.f : mn;
    const float fa = fast_exp2(a.m - mu), fb = fast_exp2(m - mu);
    a.z = a.z * fa + z * fb;
#pragma unroll
    for (int t = 0; t < NC; ++t) a.zm[t] = a.zm[t] * fa + zm[t] * fb;
    a.m = mn;
}

template <typename T> __global__ __launch_bounds__(256, 2) void pattern_recall_kernel(const RecallParams p) {
    __shared__ float lds[4][TILE][NC + 2];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, g = lane >> 5;
    const int head_lin = (int)blockIdx.y;                          // batch*hq + h
    const int rt = p.tiles - 1 - (int)blockIdx.x;                  // heavy (late) row tiles first
    const int b = head_lin / p.hq, h = head_lin % p.hq;
    const int hkv = h / (p.hq / p.hk);
    const char *qb = p.q + ((long long)b * p.qs[0] + (long long)h * p.qs[1]) * 2;
    const char *kbase = p.k + ((long long)b * p.ks[0] + (long long)hkv * p.ks[1]) * 2;
    const unsigned char *col = p.col + (long long)head_lin * p.flag_pitch;
    const unsigned char *diag = p.diag + (long long)head_lin * p.flag_pitch;
    const int brows = (p.n + KB - 1) / KB;
    const unsigned char *blk = p.blk ? p.blk + (long long)head_lin * brows * p.blk_pitch : nullptr;

    Frag qf[2][8];
    load_frag(qb, p.qs[2], rt * TILE, p.n, lane, qf[0]);
    load_frag(qb, p.qs[2], rt * TILE + 32, p.n, lane, qf[1]);

    RowState st[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        st[nb].m = -INFINITY;
        st[nb].z = 0.f;
#pragma unroll
        for (int t = 0; t < NC; ++t) st[nb].zm[t] = 0.f;
    }

    const int last_kb = min(2 * rt + 1, brows - 1);               // last key block any row of the tile sees
    Frag kf[8], kn[8];
    if (wave <= last_kb) load_frag(kbase, p.ks[2], wave * KB, p.n, lane, kn);
    for (int kb = wave; kb <= last_kb; kb += 4) {
        const int n0 = kb * KB;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) kf[ks] = kn[ks];
        if (kb + 4 <= last_kb) load_frag(kbase, p.ks[2], (kb + 4) * KB, p.n, lane, kn);

        // column flags of the lane's 16 keys: keys n0 + 8j + 4g + i, one aligned word per j
        unsigned cw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) cw[j] = *reinterpret_cast<const unsigned *>(col + n0 + 8 * j + 4 * g);

#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int rb = 2 * rt + nb;                            // 32-row block of this half
            if (kb > rb) continue;                                 // wholly above the diagonal
            f32x16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) acc = mma<T>(kf[ks], qf[nb][ks], acc);

            const int row = rb * 32 + l32;
            const unsigned bb = blk ? (unsigned)blk[(long long)min(rb, brows - 1) * p.blk_pitch + kb] : 0u;
            // diagonal flags: key i of group j has offset o0 - i, o0 = row - (n0 + 8j + 4g); the word
            // read at o0-3 holds it in byte 3-i.  Near the diagonal o0-3 may be negative: read at
            // 0 and shift the bytes up (offsets < 0 are above the diagonal and masked anyway).
            unsigned dw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int o0 = row - (n0 + 8 * j + 4 * g);
                const int base = min(max(o0 - 3, 0), (int)p.flag_pitch - 4);
                unsigned w = load_u32_unaligned(diag + base);
                const int up = base - (o0 - 3);                    // > 0 only when o0 < 3
                w = up >= 4 ? 0u : (w << (8 * max(up, 0)));
                dw[j] = w;
            }
            const bool on_diag = kb == rb;
            float s[16];
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = n0 + 8 * (r >> 2) + 4 * g + (r & 3);
                float x = acc[r] * p.scale_log2;
                if (on_diag && key > row) x = -INFINITY;
                s[r] = x;
                mx = fmaxf(mx, x);
            }
            const float mn = fmaxf(st[nb].m, mx);
            const float mu = mn == -INFINITY ? 0.f : mn;
            const float alpha = fast_exp2(st[nb].m - mu);
            float z = st[nb].z * alpha;
            float zm[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) zm[t] = st[nb].zm[t] * alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int j = r >> 2, i = r & 3;
                const float e = fast_exp2(s[r] - mu);
                const unsigned bits = (cw[j] >> (8 * i)) | (dw[j] >> (8 * (3 - i))) | bb;
                z += e;
#pragma unroll
                for (int t = 0; t < NC; ++t) zm[t] += (bits >> t) & 1u ? e : 0.f;
            }
            st[nb].m = mn;
            st[nb].z = z;
#pragma unroll
            for (int t = 0; t < NC; ++t) st[nb].zm[t] = zm[t];
        }
    }

    // merge the two lanes of a row (keys 4g + ...), then the four waves
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const float om = __shfl_xor(st[nb].m, 32);
        const float oz = __shfl_xor(st[nb].z, 32);
        float ozm[NC];
#pragma unroll
        for (int t = 0; t < NC; ++t) ozm[t] = __shfl_xor(st[nb].zm[t], 32);
        merge_into(st[nb], om, oz, ozm);
        if (g == 0) {
            float *dst = lds[wave][nb * 32 + l32];
            dst[0] = st[nb].m;
            dst[1] = st[nb].z;
#pragma unroll
            for (int t = 0; t < NC; ++t) dst[2 + t] = st[nb].zm[t];
        }
    }
    __syncthreads();
    if (wave == 0) {
        RowState a;
        a.m = lds[0][lane][0];
        a.z = lds[0][lane][1];
#pragma unroll
        for (int t = 0; t < NC; ++t) a.zm[t] = lds[0][lane][2 + t];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            float zm[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) zm[t] = lds[w][lane][2 + t];
            merge_into(a, lds[w][lane][0], lds[w][lane][1], zm);
        }
        const int row = rt * TILE + lane;
        const bool counted = row < p.n && row >= p.row_begin && a.z > 0.f;
        const float inv = counted ? 1.0f / a.z : 0.f;
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            float x = a.zm[t] * inv;
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d);     // fixed butterfly order
            if (lane == 0) p.partial[((long long)head_lin * p.tiles + rt) * NC + t] = x;
        }
    }
}

__global__ __launch_bounds__(64) void pattern_recall_finalize(const float *partial, int tiles, int n, int row_begin,
                                                              float *recall) {
    const int head_lin = (int)blockIdx.x, lane = (int)threadIdx.x;
    const float *src = partial + (long long)head_lin * tiles * NC;
    for (int t = 0; t < NC; ++t) {
        float x = 0.f;
        for (int i = lane; i < tiles; i += 64) x += src[(long long)i * NC + t];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d);
        // no rows to average over -> NaN, like the mean of an empty slice in the reference
        // (written as a bit pattern: the library is built without NaN semantics, under which the constant
        // itself is undefined)
        if (lane == 0) recall[head_lin * NC + t] = n > row_begin ? x / (float)(n - max(row_begin, 0)) : __uint_as_float(0x7fc00000u);
    }
}

__global__ void flags_set_indices_kernel(const int32_t *idx, long long idx_stride, int rows, int k, unsigned bit,
                                         unsigned char *flags, long long pitch, int limit) {
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i >= k) return;
    for (int row = (int)blockIdx.y; row < rows; row += (int)gridDim.y) {
        const int x = idx[(long long)row * idx_stride + i];
        if (x < 0 || x >= limit) continue;
        const long long off = (long long)row * pitch + x;
        atomicOr(reinterpret_cast<unsigned *>(flags + (off & ~3ll)), (1u << bit) << (8 * (int)(off & 3)));
    }
}

__global__ void flags_set_range_kernel(int begin, int end, int rows, unsigned bit, unsigned char *flags,
                                       long long pitch) {
    const int x = begin + (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (x >= end) return;
    for (int row = (int)blockIdx.y; row < rows; row += (int)gridDim.y) {
        const long long off = (long long)row * pitch + x;
        atomicOr(reinterpret_cast<unsigned *>(flags + (off & ~3ll)), (1u << bit) << (8 * (int)(off & 3)));
    }
}

}  // namespace

extern "C" size_t minf_pattern_recall_workspace_bytes(int batch, int heads_q, int n) {
    if (batch <= 0 || heads_q <= 0 || n <= 0) return 0;
    return (size_t)batch * heads_q * ((n + TILE - 1) / TILE) * NC * sizeof(float);
}

extern "C" int minf_pattern_recall(const void *q, const void *k, const int64_t *q_stride, const int64_t *k_stride,
                                   int batch, int heads_q, int heads_kv, int n, int head_dim, int dtype,
                                   float sm_scale, const uint8_t *col_flags, const uint8_t *diag_flags,
                                   int64_t flag_pitch, const uint8_t *block_flags, int64_t block_pitch,
                                   int row_begin, float *recall, void *workspace, size_t workspace_bytes,
                                   void *stream) {
    if (!q || !k || !q_stride || !k_stride || !col_flags || !diag_flags || !recall) return MINF_ERR_INVALID_ARG;
    if (batch < 0 || heads_q <= 0 || heads_kv <= 0 || n <= 0 || row_begin < 0) return MINF_ERR_INVALID_ARG;
    if (heads_q % heads_kv != 0) return MINF_ERR_INVALID_ARG;
    if (head_dim != HD) return MINF_ERR_UNSUPPORTED;
    if (dtype != MINF_BF16 && dtype != MINF_F16) return MINF_ERR_UNSUPPORTED;
    if (((uintptr_t)q | (uintptr_t)k) & 15) return MINF_ERR_ALIGNMENT;
    for (int i = 0; i < 3; ++i)
        if ((q_stride[i] | k_stride[i]) & 7) return MINF_ERR_ALIGNMENT;
    const int tiles = (n + TILE - 1) / TILE;
    if (flag_pitch < (int64_t)tiles * TILE || (flag_pitch & 3) || flag_pitch > 0x7fffffffLL) return MINF_ERR_INVALID_ARG;
    if (((uintptr_t)col_flags | (uintptr_t)diag_flags) & 3) return MINF_ERR_ALIGNMENT;
    if (block_flags && block_pitch < (n + KB - 1) / KB) return MINF_ERR_INVALID_ARG;
    if (batch == 0) return MINF_OK;
    if ((long long)batch * heads_q > 65535) return MINF_ERR_UNSUPPORTED;
    const size_t need = minf_pattern_recall_workspace_bytes(batch, heads_q, n);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3)) return MINF_ERR_WORKSPACE;

    RecallParams p;
    p.q = (const char *)q;
    p.k = (const char *)k;
    for (int i = 0; i < 3; ++i) {
        p.qs[i] = q_stride[i];
        p.ks[i] = k_stride[i];
    }
    p.hq = heads_q;
    p.hk = heads_kv;
    p.n = n;
    p.scale_log2 = sm_scale * 1.4426950408889634f;
    p.col = col_flags;
    p.diag = diag_flags;
    p.blk = block_flags;
    p.flag_pitch = flag_pitch;
    p.blk_pitch = block_pitch;
    p.row_begin = row_begin;
    p.tiles = tiles;
    p.partial = (float *)workspace;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(tiles, batch * heads_q);
    if (dtype == MINF_BF16)
        hipLaunchKernelGGL(pattern_recall_kernel<__bf16>, grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(pattern_recall_kernel<_Float16>, grid, dim3(256), 0, st, p);
    int status = minf_launch_status();
    if (status != MINF_OK) return status;
    hipLaunchKernelGGL(pattern_recall_finalize, dim3(batch * heads_q), dim3(64), 0, st, p.partial, tiles, n,
                       row_begin, recall);
    return minf_launch_status();
}

extern "C" int minf_flags_set_indices(const int32_t *idx, int rows, int k, int64_t idx_stride, int bit,
                                      uint8_t *flags, int64_t flag_pitch, int limit, void *stream) {
    if (!idx || !flags || rows < 0 || k < 0 || bit < 0 || bit >= NC || limit < 0) return MINF_ERR_INVALID_ARG;
    if (limit > flag_pitch || (flag_pitch & 3) || ((uintptr_t)flags & 3)) return MINF_ERR_INVALID_ARG;
    if (rows == 0 || k == 0) return MINF_OK;
    hipLaunchKernelGGL(flags_set_indices_kernel, dim3((k + 255) / 256, rows < 65535 ? rows : 65535), dim3(256), 0,
                       (hipStream_t)stream, idx, (long long)idx_stride, rows, k, (unsigned)bit, flags,
                       (long long)flag_pitch, limit);
    return minf_launch_status();
}

extern "C" int minf_flags_set_range(int begin, int end, int rows, int bit, uint8_t *flags, int64_t flag_pitch,
                                    void *stream) {
    if (!flags || rows < 0 || bit < 0 || bit >= NC || begin < 0) return MINF_ERR_INVALID_ARG;
    if (end > flag_pitch || (flag_pitch & 3) || ((uintptr_t)flags & 3)) return MINF_ERR_INVALID_ARG;
    if (rows == 0 || end <= begin) return MINF_OK;
    hipLaunchKernelGGL(flags_set_range_kernel, dim3((end - begin + 255) / 256, rows < 65535 ? rows : 65535),
                       dim3(256), 0, (hipStream_t)stream, begin, end, rows, (unsigned)bit, flags,
                       (long long)flag_pitch);
    return minf_launch_status();
}
