// A caller of libminf_hip.so that knows nothing about Python or torch: plain HIP runtime calls for
// memory, the C ABI of include/minf_hip.h for everything else.  It runs dense causal attention and
// the vertical-slash path (index build on the GPU, then the mixed sparse attention over those index
// tensors) on small ragged shapes and checks both against straightforward host loops.  Exit code 0
// and a final "c_caller ok" line mean success.  Built by __graft_entry__.build(); run by
// tests/test_gpu_cabi_caller.py.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

#include "../../include/minf_hip.h"

#define CHECK_HIP(x)                                                                  \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            return 2;                                                                 \
        }                                                                             \
    } while (0)
#define CHECK_MINF(x)                                                                       \
    do {                                                                                    \
        int s_ = (x);                                                                       \
        if (s_ != MINF_OK) {                                                                \
            fprintf(stderr, "%s:%d status %d (%s)\n", __FILE__, __LINE__, s_, minf_status_string(s_)); \
            return 3;                                                                       \
        }                                                                                   \
    } while (0)

static uint16_t to_bf16(float x) {           // round to nearest even
    uint32_t u;
    memcpy(&u, &x, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float x;
    memcpy(&x, &u, 4);
    return x;
}
static uint32_t lcg_state = 12345u;
static float lcg_normalish() {               // sum of four uniforms: roughly N(0, 1)
    float s = 0.f;
    for (int i = 0; i < 4; ++i) {
        lcg_state = lcg_state * 1664525u + 1013904223u;
        s += (float)(lcg_state >> 8) / 16777216.0f;
    }
    return (s - 2.0f) * 1.7320508f;
}

// masked softmax attention of one head on the host: keep(r, c) decides the mask
template <typename Keep>
static void host_attention(const std::vector<uint16_t> &q, const std::vector<uint16_t> &k,
                           const std::vector<uint16_t> &v, int n, int d, size_t qoff, size_t koff, Keep keep,
                           std::vector<float> &out) {
    out.assign((size_t)n * d, 0.f);
    std::vector<double> p(n);
    for (int r = 0; r < n; ++r) {
        double mx = -1e300;
        for (int c = 0; c < n; ++c) {
            if (!keep(r, c)) { p[c] = -1e300; continue; }
            double s = 0;
            for (int e = 0; e < d; ++e) s += (double)from_bf16(q[qoff + (size_t)r * d + e]) * from_bf16(k[koff + (size_t)c * d + e]);
            p[c] = s / sqrt((double)d);
            if (p[c] > mx) mx = p[c];
        }
        if (mx < -1e299) continue;
        double den = 0;
        for (int c = 0; c < n; ++c) { p[c] = p[c] < -1e299 ? 0.0 : exp(p[c] - mx); den += p[c]; }
        for (int c = 0; c < n; ++c) {
            if (p[c] == 0.0) continue;
            const double w = p[c] / den;
            for (int e = 0; e < d; ++e) out[(size_t)r * d + e] += (float)(w * from_bf16(v[koff + (size_t)c * d + e]));
        }
    }
}

static int compare(const char *what, const std::vector<uint16_t> &got, size_t off, const std::vector<float> &ref) {
    double mx = 0, mean = 0;
    for (size_t i = 0; i < ref.size(); ++i) {
        const double e = fabs((double)from_bf16(got[off + i]) - ref[i]);
        if (e > mx) mx = e;
        mean += e;
    }
    mean /= (double)ref.size();
    printf("%s: max-abs %.3e mean-abs %.3e\n", what, mx, mean);
    return (mx <= 2e-2 && mean <= 1e-3) ? 0 : 1;      // 16-bit output against the fp64 host result
}

int main() {
    const int B = 1, HQ = 4, HK = 2, N = 300, D = 128, ROWS = (N + 63) / 64;
    const size_t qn = (size_t)B * HQ * N * D, kn = (size_t)B * HK * N * D;
    std::vector<uint16_t> q(qn), k(kn), v(kn), o(qn);
    for (auto &x : q) x = to_bf16(lcg_normalish());
    for (auto &x : k) x = to_bf16(lcg_normalish());
    for (auto &x : v) x = to_bf16(lcg_normalish());
    printf("libminf_hip version %d\n", minf_version());
    if (minf_qkvo_size() != sizeof(minf_qkvo)) {
        fprintf(stderr, "this program and libminf_hip.so were built from different revisions of include/minf_hip.h "
                        "(minf_qkvo: %zu bytes here, %zu in the library): rebuild both\n", sizeof(minf_qkvo), minf_qkvo_size());
        return 3;
    }

    void *dq, *dk, *dv, *dout;
    CHECK_HIP(hipMalloc(&dq, qn * 2));
    CHECK_HIP(hipMalloc(&dk, kn * 2));
    CHECK_HIP(hipMalloc(&dv, kn * 2));
    CHECK_HIP(hipMalloc(&dout, qn * 2));
    CHECK_HIP(hipMemcpy(dq, q.data(), qn * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dk, k.data(), kn * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dv, v.data(), kn * 2, hipMemcpyHostToDevice));
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));

    minf_qkvo t;
    memset(&t, 0, sizeof t);
    t.q = dq; t.k = dk; t.v = dv; t.o = dout;
    const int64_t qs[3] = {(int64_t)HQ * N * D, (int64_t)N * D, D}, ks[3] = {(int64_t)HK * N * D, (int64_t)N * D, D};
    for (int i = 0; i < 3; ++i) { t.q_stride[i] = qs[i]; t.o_stride[i] = qs[i]; t.k_stride[i] = ks[i]; t.v_stride[i] = ks[i]; }
    t.batch = B; t.heads_q = HQ; t.heads_kv = HK; t.n = N; t.head_dim = D; t.dtype = MINF_BF16;
    t.seqlens = NULL;
    t.sm_scale = 1.0f / sqrtf((float)D);

    int bad = 0;
    std::vector<float> ref;
    // ---- dense causal attention -------------------------------------------------------------
    CHECK_MINF(minf_dense_attn_fwd(&t, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(o.data(), dout, qn * 2, hipMemcpyDeviceToHost));
    for (int h = 0; h < HQ; ++h) {
        host_attention(q, k, v, N, D, (size_t)h * N * D, (size_t)(h / (HQ / HK)) * N * D, [](int r, int c) { return c <= r; }, ref);
        bad |= compare("dense", o, (size_t)h * N * D, ref);
    }

    // ---- vertical-slash: index build, then the mixed sparse attention over the index tensors -----
    const int NV = 6, NS = 5;
    const int32_t vert[NV] = {0, 1, 2, 3, 77, 150}, slash[NS] = {200, 130, 64, 3, 0};      // ascending / descending
    std::vector<int32_t> hv((size_t)HQ * NV), hs((size_t)HQ * NS);
    for (int h = 0; h < HQ; ++h) {
        memcpy(&hv[(size_t)h * NV], vert, sizeof vert);
        memcpy(&hs[(size_t)h * NS], slash, sizeof slash);
    }
    const int32_t seqlen = N;
    int32_t *dseq, *dvi, *dsi, *dbc, *dbo, *dcc, *dci;
    CHECK_HIP(hipMalloc((void **)&dseq, 4));
    CHECK_HIP(hipMalloc((void **)&dvi, hv.size() * 4));
    CHECK_HIP(hipMalloc((void **)&dsi, hs.size() * 4));
    CHECK_HIP(hipMalloc((void **)&dbc, (size_t)HQ * ROWS * 4));
    CHECK_HIP(hipMalloc((void **)&dcc, (size_t)HQ * ROWS * 4));
    CHECK_HIP(hipMalloc((void **)&dbo, (size_t)HQ * ROWS * NS * 4));
    CHECK_HIP(hipMalloc((void **)&dci, (size_t)HQ * ROWS * NV * 4));
    CHECK_HIP(hipMemcpy(dseq, &seqlen, 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dvi, hv.data(), hv.size() * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dsi, hs.data(), hs.size() * 4, hipMemcpyHostToDevice));
    const size_t ws_bytes = minf_vs_index_workspace_bytes(B, HQ, NS, ROWS);
    void *dws;
    CHECK_HIP(hipMalloc(&dws, ws_bytes));
    CHECK_MINF(minf_vs_index_build_ws(dseq, dvi, dsi, dbc, dbo, dcc, dci, B, HQ, ROWS, NV, NS, 1, NULL, dws, ws_bytes, stream));
    CHECK_MINF(minf_vs_attn_fwd(&t, dbc, dbo, dcc, dci, ROWS, NS, NV, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(o.data(), dout, qn * 2, hipMemcpyDeviceToHost));
    std::vector<int32_t> bc((size_t)HQ * ROWS), cc((size_t)HQ * ROWS), bo((size_t)HQ * ROWS * NS), ci((size_t)HQ * ROWS * NV);
    CHECK_HIP(hipMemcpy(bc.data(), dbc, bc.size() * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(cc.data(), dcc, cc.size() * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(bo.data(), dbo, bo.size() * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(ci.data(), dci, ci.size() * 4, hipMemcpyDeviceToHost));
    // the mask the reference kernel realises from the index tensors (pit_sparse_flash_attention_v2.py:
    // 104-137): 64-key blocks with the causal test, gathered columns without it; what the slash list
    // {0, 3, 64, 130, 200} and the verticals must give is also checked directly on a few elements
    for (int h = 0; h < HQ; ++h) {
        auto keep = [&](int r, int c) {
            const size_t row = (size_t)h * ROWS + r / 64;
            for (int i = 0; i < bc[row]; ++i) {
                const int s = bo[row * NS + i];
                if (c >= s && c < s + 64 && c <= r) return true;
            }
            for (int i = 0; i < cc[row]; ++i)
                if (ci[row * NV + i] == c) return true;
            return false;
        };
        if (!keep(299, 299) || !keep(299, 296) || !keep(299, 99) || !keep(250, 77) || !keep(100, 0) || keep(100, 101)) {
            fprintf(stderr, "index tensors do not realise the expected mask (head %d)\n", h);
            bad |= 1;
        }
        host_attention(q, k, v, N, D, (size_t)h * N * D, (size_t)(h / (HQ / HK)) * N * D, keep, ref);
        bad |= compare("vertical-slash", o, (size_t)h * N * D, ref);
    }

    // ---- estimation + top-k: the forced entries come out first / last ----------------------------
    float *dvert, *dslash;
    int32_t *dtop;
    CHECK_HIP(hipMalloc((void **)&dvert, (size_t)HQ * N * 4));
    CHECK_HIP(hipMalloc((void **)&dslash, (size_t)HQ * N * 4));
    CHECK_HIP(hipMalloc((void **)&dtop, (size_t)HQ * 40 * 4));
    const size_t est_bytes = minf_vs_estimate_workspace_bytes(B, HQ, N);
    void *dest;
    CHECK_HIP(hipMalloc(&dest, est_bytes));
    CHECK_MINF(minf_vs_estimate(dq, dk, qs, ks, B, HQ, HK, N, D, MINF_BF16, t.sm_scale, 64, 30, 100, MINF_ROUND_INPUT_DTYPE, dvert, dslash, dest, est_bytes, stream));
    CHECK_MINF(minf_topk_indices(dvert, HQ, N, N, 40, dtop, 40, -1, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    std::vector<int32_t> top((size_t)HQ * 40);
    CHECK_HIP(hipMemcpy(top.data(), dtop, top.size() * 4, hipMemcpyDeviceToHost));
    for (int h = 0; h < HQ; ++h)
        for (int i = 0; i < 30; ++i)
            if (top[(size_t)h * 40 + i] != i) { fprintf(stderr, "forced vertical %d missing (head %d)\n", i, h); bad |= 1; }

    // ---- error behaviour: a status, not a crash ----------------------------------------------------
    t.head_dim = 96;
    if (minf_dense_attn_fwd(&t, stream) != MINF_ERR_UNSUPPORTED) { fprintf(stderr, "head_dim 96 was not rejected\n"); bad |= 1; }

    if (bad) { fprintf(stderr, "c_caller FAILED\n"); return 1; }
    printf("c_caller ok\n");
    return 0;
}
