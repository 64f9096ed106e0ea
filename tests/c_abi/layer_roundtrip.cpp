// One GCN layer, forward and backward, through the C ABI alone: plain HIP runtime calls for memory, no PyTorch.
//
// This is what a host written in C or C++ would do with include/plexus_hip.h.  Every result is compared with
// the CPU oracle's plain-C routines (oracle/oracle_kernels.c, fp64 accumulation) at the fp32 bar
// max|x - ref| / max|ref| <= 1e-5.  Exit status 0 = every comparison passed.
//
//   AGG = A.H, OUT = relu(AGG.W), loss / GRAD_OUT from the masked softmax cross-entropy,
//   GRAD_W = AGG^T.(GRAD_OUT * [OUT > 0]), GRAD_AGG = (GRAD_OUT * [OUT > 0]).W^T, GRAD_H = A^T.GRAD_AGG,
//   then one AdamW step on W          (plexus/gcn_conv.py:184-266, plexus/cross_entropy.py:19-114)
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "plexus_hip.h"

extern "C" {
void orc_csr_spmm_f32_acc64(int64_t M, const int64_t *rowptr, const int64_t *col, const float *val, const float *H, int64_t ldh,
                            int64_t D, float *Y, int64_t ldy);
void orc_gemm_f32_acc64(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                        float *C, int64_t ldc);
double orc_softmax_xent(int64_t M, int64_t C, const float *logits, int64_t ld, const int64_t *labels, int64_t num_nodes,
                        int64_t num_classes, double gscale, float *dlogits, int64_t ldd);
void orc_gcn_norm_csr(int64_t M, const int64_t *rowptr, const int64_t *col, const float *val, float *out);
}

namespace {

int g_failures = 0;

#define HIP_OK(expr)                                                                          \
    do {                                                                                      \
        hipError_t e__ = (expr);                                                              \
        if (e__ != hipSuccess) {                                                              \
            std::fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e__));                  \
            std::exit(2);                                                                     \
        }                                                                                     \
    } while (0)

#define PLX_OK_OR_DIE(expr)                                                                   \
    do {                                                                                      \
        int s__ = (expr);                                                                     \
        if (s__ != PLX_OK) {                                                                  \
            std::fprintf(stderr, "%s: %s: %s\n", #expr, plx_error_string(s__), plx_last_error()); \
            std::exit(2);                                                                     \
        }                                                                                     \
    } while (0)

uint64_t g_state = 0x9e3779b97f4a7c15ull;
uint64_t next_u64()
{  // splitmix64
    uint64_t z = (g_state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
float uniform(float lo, float hi) { return lo + (hi - lo) * (float)((next_u64() >> 40) * (1.0 / 16777216.0)); }

template <typename T>
T *to_device(const std::vector<T> &h)
{
    T *d = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d), std::max<size_t>(h.size(), 1) * sizeof(T)));
    if (!h.empty()) HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}
template <typename T>
T *device_alloc(size_t n)
{
    T *d = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d), std::max<size_t>(n, 1) * sizeof(T)));
    return d;
}
template <typename T>
std::vector<T> to_host(const T *d, size_t n)
{
    std::vector<T> h(n);
    HIP_OK(hipDeviceSynchronize());
    if (n) HIP_OK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

void compare(const char *what, const std::vector<float> &got, const std::vector<float> &ref, double tol = 1e-5)
{
    double err = 0.0, scale = 0.0;
    for (size_t i = 0; i < ref.size(); ++i) {
        err = std::max(err, std::fabs((double)got[i] - (double)ref[i]));
        scale = std::max(scale, std::fabs((double)ref[i]));
    }
    const double rel = scale > 0.0 ? err / scale : err;
    const bool ok = got.size() == ref.size() && rel <= tol && std::isfinite(rel);
    std::printf("%-28s %8zu elements  rel. error %.3e  %s\n", what, ref.size(), rel, ok ? "ok" : "FAILED");
    if (!ok) ++g_failures;
}

struct HostCsr {
    int64_t M = 0, K = 0;
    std::vector<int64_t> rowptr, col;
    std::vector<float> val;
    int64_t nnz() const { return (int64_t)col.size(); }
};

// random symmetric pattern with self loops; row 3 is a hub that touches every vertex, so it is split into segments
HostCsr make_graph(int64_t n, int64_t pairs)
{
    std::vector<std::vector<int64_t>> adj((size_t)n);
    for (int64_t e = 0; e < pairs; ++e) {
        const int64_t a = (int64_t)(next_u64() % (uint64_t)n), b = (int64_t)(next_u64() % (uint64_t)n);
        adj[(size_t)a].push_back(b);
        adj[(size_t)b].push_back(a);
    }
    for (int64_t v = 0; v < n; ++v) {
        adj[3].push_back(v);
        adj[(size_t)v].push_back(3);
        adj[(size_t)v].push_back(v);
    }
    HostCsr g;
    g.M = g.K = n;
    g.rowptr.push_back(0);
    for (auto &row : adj) {
        std::sort(row.begin(), row.end());
        row.erase(std::unique(row.begin(), row.end()), row.end());
        for (int64_t c : row) {
            g.col.push_back(c);
            g.val.push_back(1.0f);
        }
        g.rowptr.push_back((int64_t)g.col.size());
    }
    return g;
}

HostCsr transpose(const HostCsr &a)
{
    HostCsr t;
    t.M = a.K;
    t.K = a.M;
    t.rowptr.assign((size_t)a.K + 1, 0);
    for (int64_t c : a.col) ++t.rowptr[(size_t)c + 1];
    for (int64_t k = 0; k < a.K; ++k) t.rowptr[(size_t)k + 1] += t.rowptr[(size_t)k];
    t.col.resize(a.col.size());
    t.val.resize(a.val.size());
    std::vector<int64_t> fill(t.rowptr.begin(), t.rowptr.end() - 1);
    for (int64_t r = 0; r < a.M; ++r)
        for (int64_t j = a.rowptr[(size_t)r]; j < a.rowptr[(size_t)r + 1]; ++j) {
            const int64_t p = fill[(size_t)a.col[(size_t)j]]++;
            t.col[(size_t)p] = r;
            t.val[(size_t)p] = a.val[(size_t)j];
        }
    return t;
}

}  // namespace

int main()
{
    int n_dev = 0;
    if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev < 1) {
        std::fprintf(stderr, "no GPU\n");
        return 3;
    }
    HIP_OK(hipSetDevice(0));
    hipStream_t st = nullptr;
    HIP_OK(hipStreamCreate(&st));
    std::printf("libplexus_hip version %d\n", plx_version());

    const int64_t n = 5000, d_in = 100, d_out = 47, classes = 47;
    HostCsr a = make_graph(n, 40000);
    const int64_t nnz = a.nnz();
    std::printf("graph: %lld vertices, %lld stored entries\n", (long long)n, (long long)nnz);

    // ---- device copies; int64 indices as torch holds them, narrowed on the device ----
    int64_t *d_rowptr64 = to_device(a.rowptr), *d_col64 = to_device(a.col);
    float *d_ones = to_device(a.val);
    int32_t *d_rowptr = device_alloc<int32_t>((size_t)n + 1), *d_col = device_alloc<int32_t>((size_t)nnz);
    PLX_OK_OR_DIE(plx_csr_narrow_i64(n, nnz, d_rowptr64, d_col64, d_rowptr, d_col, st));

    // ---- GCN normalisation ----
    float *d_val = device_alloc<float>((size_t)nnz), *d_dinv = device_alloc<float>((size_t)n);
    PLX_OK_OR_DIE(plx_gcn_norm_csr_f32(n, d_rowptr, d_col, d_ones, d_val, d_dinv, st));
    std::vector<float> norm_ref((size_t)nnz);
    orc_gcn_norm_csr(n, a.rowptr.data(), a.col.data(), a.val.data(), norm_ref.data());
    compare("gcn normalisation", to_host(d_val, (size_t)nnz), norm_ref);
    a.val = norm_ref;  // the oracle continues from its own normalised values
    HIP_OK(hipMemcpy(d_val, norm_ref.data(), (size_t)nnz * sizeof(float), hipMemcpyHostToDevice));

    // ---- transpose on the device ----
    int32_t *d_rowptr_t = device_alloc<int32_t>((size_t)n + 1), *d_col_t = device_alloc<int32_t>((size_t)nnz);
    float *d_val_t = device_alloc<float>((size_t)nnz);
    const size_t tws_bytes = plx_csr_transpose_workspace_bytes(n, n, nnz);
    char *d_tws = device_alloc<char>(tws_bytes);
    PLX_OK_OR_DIE(plx_csr_transpose_f32(n, n, nnz, d_rowptr, d_col, d_val, d_rowptr_t, d_col_t, d_val_t, d_tws, tws_bytes, st));
    const HostCsr at = transpose(a);
    {
        const std::vector<int32_t> rp = to_host(d_rowptr_t, (size_t)n + 1), ci = to_host(d_col_t, (size_t)nnz);
        bool same = true;
        for (size_t i = 0; i < rp.size(); ++i) same = same && rp[i] == (int32_t)at.rowptr[i];
        for (size_t i = 0; i < ci.size(); ++i) same = same && ci[i] == (int32_t)at.col[i];
        std::printf("%-28s %8zu entries   indices %s\n", "transpose", ci.size(), same ? "identical  ok" : "DIFFER  FAILED");
        if (!same) ++g_failures;
        compare("transpose values", to_host(d_val_t, (size_t)nnz), at.val, 0.0);
    }

    // ---- plans (a short split length so that the hub row takes the segment path) ----
    plx_spmm_plan *plan = nullptr, *plan_t = nullptr;
    PLX_OK_OR_DIE(plx_spmm_plan_create(&plan, n, n, nnz, d_rowptr, d_col, 256, st));
    PLX_OK_OR_DIE(plx_spmm_plan_create(&plan_t, n, n, nnz, d_rowptr_t, d_col_t, 256, st));
    std::printf("plan: %lld split rows, %lld segments\n", (long long)plx_spmm_plan_info(plan, 3), (long long)plx_spmm_plan_info(plan, 4));
    const size_t sws_bytes = std::max(plx_spmm_workspace_bytes(plan, d_in), plx_spmm_workspace_bytes(plan_t, d_in));
    char *d_sws = device_alloc<char>(sws_bytes);

    // ---- operands ----
    std::vector<float> h((size_t)(n * d_in)), w((size_t)(d_in * d_out));
    for (float &x : h) x = uniform(-1.f, 1.f);
    const float bound = 1.0f / std::sqrt((float)d_out);  // plexus/gcn_conv.py:332-333
    for (float &x : w) x = uniform(-bound, bound);
    std::vector<int64_t> labels((size_t)n);
    for (int64_t &y : labels) y = (int64_t)(next_u64() % (uint64_t)classes);
    labels[7] = -1;  // an unlabeled vertex: zero loss and zero gradient row
    float *d_h = to_device(h), *d_w = to_device(w);
    int64_t *d_labels = to_device(labels);

    // ---- forward ----
    float *d_agg = device_alloc<float>((size_t)(n * d_in)), *d_out_act = device_alloc<float>((size_t)(n * d_out));
    PLX_OK_OR_DIE(plx_spmm_csr_f32(plan, d_val, d_h, d_in, d_in, d_agg, d_in, d_sws, sws_bytes, st));
    const size_t gws_bytes = plx_gemm_f32_split_workspace_bytes(std::max(d_in, d_out), std::max(d_in, d_out));
    char *d_gws = device_alloc<char>(gws_bytes);
    PLX_OK_OR_DIE(plx_gemm_nn_f32_split(n, d_out, d_in, d_agg, d_in, d_w, d_out, d_out_act, d_out, PLX_GEMM_RELU, d_gws, gws_bytes, st));
    float *d_out_plain = device_alloc<float>((size_t)(n * d_out));
    PLX_OK_OR_DIE(plx_gemm_nn_f32(n, d_out, d_in, d_agg, d_in, d_w, d_out, d_out_plain, d_out, PLX_GEMM_RELU, st));

    std::vector<float> agg_ref((size_t)(n * d_in)), out_ref((size_t)(n * d_out));
    orc_csr_spmm_f32_acc64(n, a.rowptr.data(), a.col.data(), a.val.data(), h.data(), d_in, d_in, agg_ref.data(), d_in);
    orc_gemm_f32_acc64(0, 0, n, d_out, d_in, agg_ref.data(), d_in, w.data(), d_out, out_ref.data(), d_out);
    for (float &x : out_ref) x = std::max(x, 0.f);
    compare("AGG = A.H", to_host(d_agg, agg_ref.size()), agg_ref);
    compare("OUT = relu(AGG.W) split", to_host(d_out_act, out_ref.size()), out_ref);
    compare("OUT = relu(AGG.W) fp32 mfma", to_host(d_out_plain, out_ref.size()), out_ref);

    // ---- loss ----
    float *d_loss = device_alloc<float>(1), *d_gout = device_alloc<float>((size_t)(n * d_out));
    const size_t xws_bytes = plx_softmax_xent_workspace_bytes(n, d_out);
    char *d_xws = device_alloc<char>(xws_bytes);
    PLX_OK_OR_DIE(plx_softmax_xent_f32(n, d_out, d_out_act, d_out, d_labels, n, classes, 0, 1.0f, d_loss, d_gout, d_out, d_xws, xws_bytes, st));
    std::vector<float> gout_ref((size_t)(n * d_out));
    const double loss_ref = orc_softmax_xent(n, d_out, out_ref.data(), d_out, labels.data(), n, classes, 1.0, gout_ref.data(), d_out);
    compare("loss", to_host(d_loss, 1), std::vector<float>{(float)loss_ref});
    compare("GRAD_OUT", to_host(d_gout, gout_ref.size()), gout_ref);

    // ---- backward ----
    float *d_gw = device_alloc<float>((size_t)(d_in * d_out)), *d_gagg = device_alloc<float>((size_t)(n * d_in));
    float *d_gh = device_alloc<float>((size_t)(n * d_in));
    const size_t tnws_bytes = plx_gemm_tn_workspace_bytes(n, d_out, d_in);
    char *d_tnws = device_alloc<char>(tnws_bytes);
    PLX_OK_OR_DIE(plx_gemm_tn_f32(n, d_out, d_in, d_agg, d_in, d_gout, d_out, d_gw, d_out, d_out_act, d_out, d_tnws, tnws_bytes, st));
    PLX_OK_OR_DIE(plx_gemm_nt_f32_split(n, d_in, d_out, d_gout, d_out, d_w, d_out, d_gagg, d_in, d_out_act, d_out, d_gws, gws_bytes, st));
    PLX_OK_OR_DIE(plx_spmm_csr_f32(plan_t, d_val_t, d_gagg, d_in, d_in, d_gh, d_in, d_sws, sws_bytes, st));

    std::vector<float> gmask(gout_ref);
    for (size_t i = 0; i < gmask.size(); ++i)
        if (!(out_ref[i] > 0.f)) gmask[i] = 0.f;
    std::vector<float> gw_ref((size_t)(d_in * d_out)), gagg_ref((size_t)(n * d_in)), gh_ref((size_t)(n * d_in));
    orc_gemm_f32_acc64(1, 0, d_in, d_out, n, agg_ref.data(), d_in, gmask.data(), d_out, gw_ref.data(), d_out);
    orc_gemm_f32_acc64(0, 1, n, d_in, d_out, gmask.data(), d_out, w.data(), d_out, gagg_ref.data(), d_in);
    orc_csr_spmm_f32_acc64(n, at.rowptr.data(), at.col.data(), at.val.data(), gagg_ref.data(), d_in, d_in, gh_ref.data(), d_in);
    compare("GRAD_W = AGG^T.G", to_host(d_gw, gw_ref.size()), gw_ref);
    compare("GRAD_AGG = G.W^T", to_host(d_gagg, gagg_ref.size()), gagg_ref);
    compare("GRAD_H = A^T.GRAD_AGG", to_host(d_gh, gh_ref.size()), gh_ref);

    // ---- GRAD_W on the bf16 matrix cores from exact splits, on operands whose rows take 128-bit loads: AGG^T . GRAD_AGG ----
    {
        const size_t sws2_bytes = plx_gemm_tn_f32_split_workspace_bytes(n, d_in, d_in);
        char *d_sws2 = device_alloc<char>(sws2_bytes);
        float *d_c2 = device_alloc<float>((size_t)(d_in * d_in));
        PLX_OK_OR_DIE(plx_gemm_tn_f32_split(n, d_in, d_in, d_agg, d_in, d_gagg, d_in, d_c2, d_in, nullptr, 0, nullptr, 0, 2.0f, d_sws2,
                                            sws2_bytes, st));
        const std::vector<float> agg_dev = to_host(d_agg, agg_ref.size()), gagg_dev = to_host(d_gagg, gagg_ref.size());
        std::vector<float> c2_ref((size_t)(d_in * d_in));
        orc_gemm_f32_acc64(1, 0, d_in, d_in, n, agg_dev.data(), d_in, gagg_dev.data(), d_in, c2_ref.data(), d_in);
        for (float &x : c2_ref) x *= 2.0f;
        compare("2 AGG^T.GRAD_AGG from splits", to_host(d_c2, c2_ref.size()), c2_ref);
        HIP_OK(hipFree(d_sws2));
        HIP_OK(hipFree(d_c2));
    }

    // ---- graph preparation: the normalised CSR straight from an edge list that lacks some self loops, and a permuted copy ----
    {
        std::vector<int64_t> e_row, e_col;
        for (int64_t r = 0; r < n; ++r)
            for (int64_t j = a.rowptr[(size_t)r]; j < a.rowptr[(size_t)r + 1]; ++j) {
                const int64_t c = a.col[(size_t)j];
                if (r == c && r % 5 == 0) continue;  // these vertices get their loop from the call
                e_row.push_back(r);
                e_col.push_back(c);
            }
        std::reverse(e_row.begin(), e_row.end());  // any order will do
        std::reverse(e_col.begin(), e_col.end());
        const int64_t n_edges = (int64_t)e_row.size();
        int64_t *d_erow = to_device(e_row), *d_ecol = to_device(e_col);
        int32_t *d_rp2 = device_alloc<int32_t>((size_t)n + 1), *d_ci2 = device_alloc<int32_t>((size_t)(n_edges + n));
        float *d_v2 = device_alloc<float>((size_t)(n_edges + n));
        const size_t nws_bytes = plx_gcn_norm_edges_workspace_bytes(n_edges, n);
        char *d_nws = device_alloc<char>(nws_bytes);
        int64_t nnz2 = 0;
        PLX_OK_OR_DIE(plx_gcn_norm_edges_f32(n_edges, d_erow, d_ecol, nullptr, n, 0, d_rp2, d_ci2, d_v2, &nnz2, d_nws, nws_bytes, st));
        const std::vector<int32_t> rp2 = to_host(d_rp2, (size_t)n + 1), ci2 = to_host(d_ci2, (size_t)std::min(nnz2, nnz));
        bool same = nnz2 == nnz;
        for (size_t i = 0; same && i < rp2.size(); ++i) same = rp2[i] == (int32_t)a.rowptr[i];
        for (size_t i = 0; same && i < ci2.size(); ++i) same = ci2[i] == (int32_t)a.col[i];
        std::printf("%-28s %8lld entries   indices %s\n", "normalised CSR from edges", (long long)nnz2, same ? "identical  ok" : "DIFFER  FAILED");
        if (!same) ++g_failures;
        else compare("its values", to_host(d_v2, (size_t)nnz), norm_ref);

        // out[new_col[c], i] = A^T[walk[i], c]: with A^T, walk = perm2 and new_col = the inverse of perm this is P.A.P2^T
        std::vector<int64_t> walk((size_t)n), new_id((size_t)n);
        for (int64_t i = 0; i < n; ++i) {
            walk[(size_t)i] = n - 1 - i;
            new_id[(size_t)i] = (i * 7 + 3) % n;  // a bijection: 7 and 5000 are coprime
        }
        int64_t *d_walk = to_device(walk), *d_new = to_device(new_id);
        int32_t *d_rp3 = device_alloc<int32_t>((size_t)n + 1), *d_ci3 = device_alloc<int32_t>((size_t)nnz);
        float *d_v3 = device_alloc<float>((size_t)nnz);
        const size_t pws_bytes = plx_csr_permute_transposed_workspace_bytes(n, n, nnz);
        char *d_pws = device_alloc<char>(pws_bytes);
        PLX_OK_OR_DIE(plx_csr_permute_transposed_f32(n, n, nnz, d_rowptr_t, d_col_t, d_val_t, d_walk, d_new, d_rp3, d_ci3, d_v3, d_pws,
                                                     pws_bytes, st));
        std::vector<std::vector<std::pair<int64_t, float>>> rows3((size_t)n);
        for (int64_t i = 0; i < n; ++i) {  // moved rows in ascending i, so every row of the result comes out ascending
            const int64_t src = walk[(size_t)i];
            for (int64_t j = at.rowptr[(size_t)src]; j < at.rowptr[(size_t)src + 1]; ++j)
                rows3[(size_t)new_id[(size_t)at.col[(size_t)j]]].push_back({i, at.val[(size_t)j]});
        }
        const std::vector<int32_t> rp3 = to_host(d_rp3, (size_t)n + 1), ci3 = to_host(d_ci3, (size_t)nnz);
        const std::vector<float> v3 = to_host(d_v3, (size_t)nnz);
        bool same3 = true;
        int64_t p = 0;
        for (int64_t r = 0; r < n && same3; ++r) {
            same3 = rp3[(size_t)r] == (int32_t)p;
            for (const auto &e : rows3[(size_t)r]) {
                same3 = same3 && ci3[(size_t)p] == (int32_t)e.first && v3[(size_t)p] == e.second;
                ++p;
            }
        }
        same3 = same3 && rp3[(size_t)n] == (int32_t)nnz;
        std::printf("%-28s %8lld entries   %s\n", "permuted CSR from A^T", (long long)nnz, same3 ? "identical  ok" : "DIFFER  FAILED");
        if (!same3) ++g_failures;
        void *mine[] = {d_erow, d_ecol, d_rp2, d_ci2, d_v2, d_nws, d_walk, d_new, d_rp3, d_ci3, d_v3, d_pws};
        for (void *q : mine) HIP_OK(hipFree(q));
    }

    // ---- one AdamW step on the weight (examples/train.py:155-159: lr 3e-3, no weight decay) ----
    float *d_m = device_alloc<float>(w.size()), *d_v = device_alloc<float>(w.size());
    HIP_OK(hipMemsetAsync(d_m, 0, w.size() * sizeof(float), st));
    HIP_OK(hipMemsetAsync(d_v, 0, w.size() * sizeof(float), st));
    PLX_OK_OR_DIE(plx_adamw_f32((int64_t)w.size(), d_w, d_gw, d_m, d_v, 3e-3, 0.9, 0.999, 1e-8, 0.0, 1, st));
    // from the gradient the device holds: the first step moves every weight by lr * sign(g), so a gradient within
    // rounding of zero must not be allowed to differ in sign between the two sides
    const std::vector<float> gw_dev = to_host(d_gw, gw_ref.size());
    std::vector<float> w_ref(w);
    for (size_t i = 0; i < w.size(); ++i) {
        const double g = gw_dev[i], m = 0.1 * g, v = 0.001 * g * g;
        w_ref[i] = (float)(w[i] - 3e-3 / (1.0 - 0.9) * m / (std::sqrt(v) / std::sqrt(1.0 - 0.999) + 1e-8));
    }
    compare("W after AdamW", to_host(d_w, w.size()), w_ref);

    // ---- error path: a call that cannot be served says so instead of running ----
    const int rc = plx_spmm_csr_f32(plan, d_val, d_h, d_in - 1, d_in, d_agg, d_in, d_sws, sws_bytes, st);
    std::printf("%-28s status %d (%s)  %s\n", "ldh < D is rejected", rc, plx_error_string(rc), rc == PLX_ERR_INVALID ? "ok" : "FAILED");
    if (rc != PLX_ERR_INVALID) ++g_failures;

    HIP_OK(hipStreamSynchronize(st));
    plx_spmm_plan_destroy(plan);
    plx_spmm_plan_destroy(plan_t);
    void *to_free[] = {d_rowptr64, d_col64, d_ones, d_rowptr, d_col, d_val, d_dinv, d_rowptr_t, d_col_t, d_val_t, d_tws, d_sws,
                       d_h, d_w, d_labels, d_agg, d_out_act, d_out_plain, d_gws, d_loss, d_gout, d_xws, d_gw, d_gagg, d_gh,
                       d_tnws, d_m, d_v};
    for (void *p : to_free) HIP_OK(hipFree(p));
    HIP_OK(hipStreamDestroy(st));
    std::printf(g_failures ? "FAILED: %d comparisons\n" : "all comparisons passed\n", g_failures);
    return g_failures ? 1 : 0;
}
