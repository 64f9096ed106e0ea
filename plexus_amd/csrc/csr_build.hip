// Building the operands of the SpMM on the device: the CSR of the transpose, and a CSR block from an
// edge list.
//
// The reference builds both on the host (plexus/utils/dataloader.py:343-368: mask the edge list to the
// rank's block, re-base, sparse_coo_tensor -> to_sparse_csr, and transpose(0, 1).to_sparse_csr()) and then
// copies them to the GPU.  For 10^8 entries that takes far longer than an epoch; here both are a stable
// radix sort (rocPRIM) plus a few streaming kernels, and the results are entry-for-entry what the host
// path produces: rows in order, columns ascending within a row, duplicates of an edge summed.
#include <cstring>  // rocPRIM's texture iterator calls memset without including it

#include <hip/hip_runtime.h>
#include <rocprim/rocprim.hpp>

#include <algorithm>
#include <cstdint>

#include "common.h"

namespace {

size_t align_up(size_t x) { return (x + 255) / 256 * 256; }

int bits_for(int64_t n)
{
    int b = 1;
    while (b < 63 && ((int64_t)1 << b) < n) ++b;
    return b;
}

// a fill kernel rather than a memset node: these calls are stream-ordered and may be recorded into a graph
__global__ void zero_i32_kernel(int64_t n, int32_t *__restrict__ out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = 0;
}

// rowptr[c] = first position i with sorted[i] >= c, for c in [0, n_rows]; positions are sorted ascending
template <typename KeyT, typename RowOf>
__global__ void rowptr_from_sorted_kernel(int64_t n, const KeyT *__restrict__ sorted, int64_t n_rows, int32_t *__restrict__ rowptr,
                                          RowOf row_of)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= n; i += stride) {
        const int64_t prev = i == 0 ? -1 : row_of(sorted[i - 1]);
        const int64_t cur = i == n ? n_rows : row_of(sorted[i]);
        for (int64_t r = prev + 1; r <= cur; ++r) rowptr[r] = (int32_t)i;
    }
}

// (row, value) of every stored entry as one 64-bit word, row in the upper half: the payload that travels through the
// sort by column.  A workgroup takes 1,024 consecutive entries; it finds the rows of its first and last entry by
// binary search once, and each entry then searches only between those (no steps at all inside a long row).
constexpr int kPackPerBlock = 1024;
__global__ void __launch_bounds__(256) pack_row_value_kernel(int64_t nnz, int64_t M, const int32_t *__restrict__ rowptr,
                                                             const float *__restrict__ val, uint64_t *__restrict__ packed)
{
    __shared__ int32_t bounds[2];
    const int64_t e0 = (int64_t)blockIdx.x * kPackPerBlock;
    const int64_t e1 = min(e0 + kPackPerBlock, nnz) - 1;
    if (threadIdx.x < 2) {
        const int64_t j = threadIdx.x == 0 ? e0 : e1;
        int64_t lo = 0, hi = M;  // invariant: rowptr[lo] <= j < rowptr[hi]
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if (rowptr[mid] <= j) lo = mid; else hi = mid;
        }
        bounds[threadIdx.x] = (int32_t)lo;
    }
    __syncthreads();
    const int32_t r_first = bounds[0], r_last = bounds[1];
    for (int64_t j = e0 + threadIdx.x; j <= e1; j += 256) {
        int32_t lo = r_first, hi = r_last + 1;  // the row of j is the last r in [r_first, r_last] with rowptr[r] <= j
        while (hi - lo > 1) {
            const int32_t mid = lo + ((hi - lo) >> 1);
            if (rowptr[mid] <= j) lo = mid; else hi = mid;
        }
        packed[j] = ((uint64_t)(uint32_t)lo << 32) | (uint64_t)__float_as_uint(val[j]);
    }
}

// transposed entry i: its column is the source row, its value the source value
__global__ void unpack_row_value_kernel(int64_t nnz, const uint64_t *__restrict__ packed, int32_t *__restrict__ col_t, float *__restrict__ val_t)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nnz; i += stride) {
        const uint64_t w = packed[i];
        col_t[i] = (int32_t)(w >> 32);
        val_t[i] = __uint_as_float((uint32_t)w);
    }
}

// edge list -> keys: (row - r0) * Kb + (col - c0) for edges inside the block, flag 0 otherwise
__global__ void block_keys_kernel(int64_t n, const int64_t *__restrict__ row, const int64_t *__restrict__ col, int64_t r0, int64_t r1,
                                  int64_t c0, int64_t c1, uint64_t *__restrict__ keys, uint8_t *__restrict__ flags)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t kb = c1 - c0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t r = row[i], c = col[i];
        const bool in = r >= r0 && r < r1 && c >= c0 && c < c1;
        keys[i] = in ? (uint64_t)((r - r0) * kb + (c - c0)) : 0u;
        flags[i] = in ? 1 : 0;
    }
}

struct RowOfColumnKey {
    __device__ int64_t operator()(int32_t k) const { return (int64_t)k; }
};
struct RowOfBlockKey {
    int64_t kb;
    __device__ int64_t operator()(uint64_t k) const { return (int64_t)(k / (uint64_t)kb); }
};

// ---- duplicates of sorted keys, summed in their input order ------------------------------------------------------
// head(i) = 1 where a run of equal keys starts.  An inclusive scan of it numbers the runs: the run of entry i is
// scan[i] - 1, and a row that starts at sorted position b starts at entry (b ? scan[b - 1] : 0) of the merged arrays.
struct RunHead {
    const uint64_t *keys;
    __device__ int32_t operator()(uint32_t i) const { return (i == 0 || keys[i] != keys[i - 1]) ? 1 : 0; }
};

struct HighField {
    __device__ int64_t operator()(uint64_t k) const { return (int64_t)(k >> 32); }
};
struct LowField {
    __device__ int64_t operator()(uint64_t k) const { return (int64_t)(k & 0xffffffffull); }
};

// rowptr of the merged entries: as rowptr_from_sorted_kernel, with positions translated through the run numbers
template <typename RowOf>
__global__ void rowptr_from_runs_kernel(int64_t n, const uint64_t *__restrict__ sorted, const int32_t *__restrict__ run_scan,
                                        int64_t n_rows, int32_t *__restrict__ rowptr, RowOf row_of)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= n; i += stride) {
        const int64_t prev = i == 0 ? -1 : min(row_of(sorted[i - 1]), n_rows);
        const int64_t cur = i == n ? n_rows : min(row_of(sorted[i]), n_rows);
        const int32_t at = i == 0 ? 0 : run_scan[i - 1];
        for (int64_t r = prev + 1; r <= cur; ++r) rowptr[r] = at;
    }
}

// one thread per sorted entry; the thread of a run's first entry adds the run up (runs are short: duplicates of one
// edge) and writes the merged entry.  Entries of rows >= n_rows (keys marked as dropped) are skipped.  With dinv the
// value is scaled by dinv[row] and dinv[col] (the symmetric normalisation).
template <typename RowOf, typename ColOf>
__global__ void merge_runs_kernel(int64_t n, const uint64_t *__restrict__ sorted, const float *__restrict__ w,
                                  const int32_t *__restrict__ run_scan, int64_t n_rows, const float *__restrict__ dinv,
                                  int32_t *__restrict__ col_out, float *__restrict__ val_out, RowOf row_of, ColOf col_of)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t k = sorted[i];
        if (i != 0 && sorted[i - 1] == k) continue;
        const int64_t r = row_of(k);
        if (r >= n_rows) continue;
        float s = w[i];
        for (int64_t j = i + 1; j < n && sorted[j] == k; ++j) s += w[j];
        const int64_t c = col_of(k);
        const int32_t p = run_scan[i] - 1;
        col_out[p] = (int32_t)c;
        val_out[p] = dinv ? (dinv[r] * s) * dinv[c] : s;
    }
}

// ---- GCN normalisation from an edge list --------------------------------------------------------------------------
// key of an edge: (row of the result) << 32 | (column of the result); edges that name a vertex outside [0, N) get
// (N, N) and fall behind every real entry.  A vertex seen with a self loop is marked.
__global__ void norm_keys_kernel(int64_t n, const int64_t *__restrict__ row, const int64_t *__restrict__ col,
                                 const float *__restrict__ weight, int64_t N, int transposed, uint64_t *__restrict__ keys,
                                 float *__restrict__ w_out, uint8_t *__restrict__ has_loop)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const uint64_t dropped = ((uint64_t)N << 32) | (uint64_t)N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t r = row[i], c = col[i];
        const bool in = r >= 0 && r < N && c >= 0 && c < N;
        const uint64_t hi = (uint64_t)(transposed ? c : r), lo = (uint64_t)(transposed ? r : c);
        keys[i] = in ? (hi << 32) | lo : dropped;
        w_out[i] = weight ? weight[i] : 1.f;
        if (in && r == c) has_loop[r] = 1;
    }
}

// the self loops that are missing, with weight 1, behind the edges (a vertex that has one keeps it)
__global__ void norm_loop_keys_kernel(int64_t N, const uint8_t *__restrict__ has_loop, uint64_t *__restrict__ keys,
                                      float *__restrict__ w_out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const uint64_t dropped = ((uint64_t)N << 32) | (uint64_t)N;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < N; v += stride) {
        keys[v] = has_loop[v] ? dropped : ((uint64_t)v << 32) | (uint64_t)v;
        w_out[v] = 1.f;
    }
}

__global__ void zero_u8_kernel(int64_t n, uint8_t *__restrict__ out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = 0;
}

// ---- rows and columns of a CSR matrix renumbered -------------------------------------------------------------------
__global__ void permuted_row_length_kernel(int64_t M, const int32_t *__restrict__ rowptr, const int64_t *__restrict__ perm_rows,
                                           int32_t *__restrict__ len, int32_t *__restrict__ out_of_range)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= M; i += stride) {
        if (i == M) { len[i] = 0; continue; }
        const int64_t r = perm_rows[i];
        const bool ok = r >= 0 && r < M;
        len[i] = ok ? rowptr[r + 1] - rowptr[r] : 0;
        if (!ok) *out_of_range = 1;
    }
}

// row of entry j by binary search between the rows of the workgroup's first and last entry (found once)
__device__ inline int32_t row_of_entry(const int32_t *__restrict__ rowptr, int32_t lo, int32_t hi, int64_t j)
{
    while (hi - lo > 1) {
        const int32_t mid = lo + ((hi - lo) >> 1);
        if (rowptr[mid] <= j) lo = mid; else hi = mid;
    }
    return lo;
}

__device__ inline void block_row_bounds(int64_t M, const int32_t *__restrict__ rowptr, int64_t e0, int64_t e1, int32_t *bounds)
{
    if (threadIdx.x < 2) {
        const int64_t j = threadIdx.x == 0 ? e0 : e1;
        int64_t lo = 0, hi = M;  // invariant: rowptr[lo] <= j < rowptr[hi]
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if (rowptr[mid] <= j) lo = mid; else hi = mid;
        }
        bounds[threadIdx.x] = (int32_t)lo;
    }
    __syncthreads();
}

// The source rows in their new order, column ids renumbered, ready for the sort by new column: entry j of that
// sequence lies in moved row i at offset j - moved_ptr[i]; it is the entry at the same offset of source row
// perm_rows[i].  Its key is the renumbered column, its payload (i, value) in one word.
__global__ void __launch_bounds__(256) gather_moved_rows_kernel(int64_t nnz, int64_t M, const int32_t *__restrict__ moved_ptr,
                                                                const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col,
                                                                const float *__restrict__ val, const int64_t *__restrict__ perm_rows,
                                                                const int64_t *__restrict__ new_col, int32_t *__restrict__ keys,
                                                                uint64_t *__restrict__ packed)
{
    __shared__ int32_t bounds[2];
    const int64_t e0 = (int64_t)blockIdx.x * kPackPerBlock;
    const int64_t e1 = min(e0 + kPackPerBlock, nnz) - 1;
    block_row_bounds(M, moved_ptr, e0, e1, bounds);
    const int32_t r_first = bounds[0], r_last = bounds[1];
    for (int64_t j = e0 + threadIdx.x; j <= e1; j += 256) {
        const int32_t i = row_of_entry(moved_ptr, r_first, r_last + 1, j);
        const int64_t src = (int64_t)rowptr[perm_rows[i]] + (j - moved_ptr[i]);
        keys[j] = (int32_t)new_col[col[src]];
        packed[j] = ((uint64_t)(uint32_t)i << 32) | (uint64_t)__float_as_uint(val[src]);
    }
}

__global__ void ids_in_range_kernel(int64_t n, const int64_t *__restrict__ ids, int64_t bound, int32_t *__restrict__ out_of_range)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        if (ids[i] < 0 || ids[i] >= bound) *out_of_range = 1;
}

unsigned blocks_for(int64_t n) { return (unsigned)std::max<int64_t>(1, std::min<int64_t>(plx::ceil_div(n, 256), 256 * 32)); }

struct TransposeLayout {
    size_t keys_out, pay_in, pay_out, temp, temp_bytes, total;
};

int transpose_layout(int64_t K, int64_t nnz, TransposeLayout &l)
{
    size_t temp = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, temp, (const int32_t *)nullptr, (int32_t *)nullptr, (const uint64_t *)nullptr,
                                             (uint64_t *)nullptr, (size_t)nnz, 0, (unsigned)bits_for(K), (hipStream_t)0);
    if (e != hipSuccess) return plx::fail(PLX_ERR_HIP, "csr_transpose: radix sort size query failed: %s", hipGetErrorString(e));
    size_t off = 0;
    l.keys_out = off; off += align_up(sizeof(int32_t) * (size_t)nnz);
    l.pay_in = off;   off += align_up(sizeof(uint64_t) * (size_t)nnz);
    l.pay_out = off;  off += align_up(sizeof(uint64_t) * (size_t)nnz);
    l.temp = off;     off += align_up(temp);
    l.temp_bytes = temp;
    l.total = off;
    return PLX_OK;
}

struct CooLayout {
    size_t keys, flags, keys_c, w_c, keys_s, w_s, run_scan, count, temp, temp_bytes, total;
};

size_t run_scan_temp_bytes(int64_t n)
{
    size_t t = 0;
    auto heads = rocprim::make_transform_iterator(rocprim::counting_iterator<uint32_t>(0), RunHead{nullptr});
    if (rocprim::inclusive_scan(nullptr, t, heads, (int32_t *)nullptr, (size_t)n, rocprim::plus<int32_t>(), (hipStream_t)0) != hipSuccess)
        return (size_t)-1;
    return t;
}

int coo_layout(int64_t n, int key_bits, CooLayout &l)
{
    size_t t1 = 0, t2 = 0;
    hipError_t e = rocprim::select(nullptr, t1, (const uint64_t *)nullptr, (const uint8_t *)nullptr, (uint64_t *)nullptr,
                                   (int64_t *)nullptr, (size_t)n, (hipStream_t)0);
    if (e == hipSuccess)
        e = rocprim::radix_sort_pairs(nullptr, t2, (const uint64_t *)nullptr, (uint64_t *)nullptr, (const float *)nullptr,
                                      (float *)nullptr, (size_t)n, 0, (unsigned)key_bits, (hipStream_t)0);
    const size_t t3 = run_scan_temp_bytes(n);
    if (e != hipSuccess || t3 == (size_t)-1)
        return plx::fail(PLX_ERR_HIP, "coo_to_csr: temporary-storage query failed: %s", hipGetErrorString(e));
    const size_t temp = std::max(t1, std::max(t2, t3));
    size_t off = 0;
    l.keys = off;     off += align_up(8 * (size_t)n);
    l.flags = off;    off += align_up((size_t)n);
    l.keys_c = off;   off += align_up(8 * (size_t)n);
    l.w_c = off;      off += align_up(4 * (size_t)n);
    l.keys_s = off;   off += align_up(8 * (size_t)n);
    l.w_s = off;      off += align_up(4 * (size_t)n);
    l.run_scan = off; off += align_up(4 * (size_t)n);
    l.count = off;    off += 256;
    l.temp = off;     off += align_up(temp);
    l.temp_bytes = temp;
    l.total = off;
    return PLX_OK;
}

// merged entries of sorted (key, weight) pairs: run numbers, row pointers, columns and summed values
template <typename RowOf, typename ColOf>
int merge_sorted(int64_t n, const uint64_t *sorted, const float *w, int32_t *run_scan, void *temp, size_t temp_bytes, int64_t n_rows,
                 const float *dinv, int32_t *rowptr, int32_t *col_out, float *val_out, RowOf row_of, ColOf col_of, hipStream_t st)
{
    auto heads = rocprim::make_transform_iterator(rocprim::counting_iterator<uint32_t>(0), RunHead{sorted});
    PLX_HIP_CHECK(rocprim::inclusive_scan(temp, temp_bytes, heads, run_scan, (size_t)n, rocprim::plus<int32_t>(), st));
    rowptr_from_runs_kernel<<<blocks_for(n + 1), 256, 0, st>>>(n, sorted, run_scan, n_rows, rowptr, row_of);
    PLX_LAUNCH_CHECK("rowptr_from_runs_kernel");
    merge_runs_kernel<<<blocks_for(n), 256, 0, st>>>(n, sorted, w, run_scan, n_rows, dinv, col_out, val_out, row_of, col_of);
    PLX_LAUNCH_CHECK("merge_runs_kernel");
    return PLX_OK;
}

struct ColOfBlockKey {
    int64_t kb;
    __device__ int64_t operator()(uint64_t k) const { return (int64_t)(k % (uint64_t)kb); }
};

struct NormLayout {
    size_t keys_a, keys_b, w_a, w_b, run_scan, segptr, dinv, has_loop, temp, temp_bytes, total;
    int field_bits;
};

int norm_layout(int64_t n_edges, int64_t N, NormLayout &l)
{
    const int64_t n = n_edges + N;
    l.field_bits = bits_for(N + 1);
    size_t t1 = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, t1, (const uint64_t *)nullptr, (uint64_t *)nullptr, (const float *)nullptr,
                                             (float *)nullptr, (size_t)n, 0, (unsigned)l.field_bits, (hipStream_t)0);
    const size_t t2 = run_scan_temp_bytes(n);
    if (e != hipSuccess || t2 == (size_t)-1)
        return plx::fail(PLX_ERR_HIP, "gcn_norm_edges: temporary-storage query failed: %s", hipGetErrorString(e));
    const size_t temp = std::max(t1, t2);
    size_t off = 0;
    l.keys_a = off;   off += align_up(8 * (size_t)n);
    l.keys_b = off;   off += align_up(8 * (size_t)n);
    l.w_a = off;      off += align_up(4 * (size_t)n);
    l.w_b = off;      off += align_up(4 * (size_t)n);
    l.run_scan = off; off += align_up(4 * (size_t)n);
    l.segptr = off;   off += align_up(4 * (size_t)(N + 2));
    l.dinv = off;     off += align_up(4 * (size_t)N);
    l.has_loop = off; off += align_up((size_t)N);
    l.temp = off;     off += align_up(temp);
    l.temp_bytes = temp;
    l.total = off;
    return PLX_OK;
}

struct PermuteLayout {
    size_t len, moved_ptr, flag, keys_in, sort, total;
    TransposeLayout t;
    size_t scan_temp;
};

int permute_layout(int64_t M, int64_t K, int64_t nnz, PermuteLayout &l)
{
    size_t t1 = 0;
    hipError_t e = rocprim::exclusive_scan(nullptr, t1, (const int32_t *)nullptr, (int32_t *)nullptr, (int32_t)0, (size_t)(M + 1),
                                           rocprim::plus<int32_t>(), (hipStream_t)0);
    if (e != hipSuccess) return plx::fail(PLX_ERR_HIP, "csr_permute: temporary-storage query failed: %s", hipGetErrorString(e));
    int rc = transpose_layout(K, nnz, l.t);
    if (rc != PLX_OK) return rc;
    l.scan_temp = t1;
    size_t off = 0;
    l.len = off;       off += align_up(4 * (size_t)(M + 1));
    l.moved_ptr = off; off += align_up(4 * (size_t)(M + 1));
    l.flag = off;      off += 256;
    l.keys_in = off;   off += align_up(4 * (size_t)nnz);
    l.sort = off;      off += std::max(l.t.total, align_up(t1));  // the scan's scratch is free again when the sort starts
    l.total = off;
    return PLX_OK;
}

}  // namespace

extern "C" {

size_t plx_csr_transpose_workspace_bytes(int64_t M, int64_t K, int64_t nnz)
{
    (void)M;
    if (nnz <= 0 || K <= 0) return 0;
    TransposeLayout l;
    if (transpose_layout(K, nnz, l) != PLX_OK) return 0;
    return l.total;
}

int plx_csr_transpose_f32(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, const float *val,
                          int32_t *rowptr_t, int32_t *col_t, float *val_t, void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(M >= 0 && K >= 0 && nnz >= 0, "csr_transpose: negative size");
    PLX_REQUIRE(M < (1ll << 31) - 1 && K < (1ll << 31) - 1 && nnz < (1ll << 31), "csr_transpose: sizes exceed int32 indexing");
    PLX_REQUIRE(rowptr_t != nullptr, "csr_transpose: NULL rowptr_t");
    hipStream_t st = plx::as_stream(stream);
    if (nnz == 0) {
        zero_i32_kernel<<<blocks_for(K + 1), 256, 0, st>>>(K + 1, rowptr_t);
        PLX_LAUNCH_CHECK("zero_i32_kernel");
        return PLX_OK;
    }
    PLX_REQUIRE(rowptr && col && val && col_t && val_t, "csr_transpose: NULL operand");
    TransposeLayout l;
    int rc = transpose_layout(K, nnz, l);
    if (rc != PLX_OK) return rc;
    if (workspace == nullptr || workspace_bytes < l.total)
        return plx::fail(PLX_ERR_WORKSPACE, "csr_transpose: workspace of %zu bytes needed, %zu given", l.total, workspace_bytes);
    PLX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "csr_transpose: workspace must be 256-byte aligned");
    char *ws = static_cast<char *>(workspace);
    int32_t *keys_out = reinterpret_cast<int32_t *>(ws + l.keys_out);
    uint64_t *pay_in = reinterpret_cast<uint64_t *>(ws + l.pay_in);
    uint64_t *pay_out = reinterpret_cast<uint64_t *>(ws + l.pay_out);

    pack_row_value_kernel<<<(unsigned)plx::ceil_div(nnz, kPackPerBlock), 256, 0, st>>>(nnz, M, rowptr, val, pay_in);
    PLX_LAUNCH_CHECK("pack_row_value_kernel");
    // stable sort by column: within a column the entries keep their source order, i.e. ascending source row; the
    // (row, value) words travel with the keys, so nothing is gathered afterwards
    size_t temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::radix_sort_pairs(ws + l.temp, temp, col, keys_out, pay_in, pay_out, (size_t)nnz, 0, (unsigned)bits_for(K), st));
    rowptr_from_sorted_kernel<int32_t><<<blocks_for(nnz + 1), 256, 0, st>>>(nnz, keys_out, K, rowptr_t, RowOfColumnKey());
    PLX_LAUNCH_CHECK("rowptr_from_sorted_kernel");
    unpack_row_value_kernel<<<blocks_for(nnz), 256, 0, st>>>(nnz, pay_out, col_t, val_t);
    PLX_LAUNCH_CHECK("unpack_row_value_kernel");
    return PLX_OK;
}

size_t plx_coo_block_to_csr_workspace_bytes(int64_t n_edges, int64_t block_rows, int64_t block_cols)
{
    if (n_edges <= 0) return 256;
    CooLayout l;
    if (coo_layout(n_edges, bits_for(std::max<int64_t>(block_rows, 1) * std::max<int64_t>(block_cols, 1)), l) != PLX_OK) return 0;
    return l.total;
}

int plx_coo_block_to_csr_f32(int64_t n_edges, const int64_t *row, const int64_t *col, const float *weight, int64_t r0, int64_t r1,
                             int64_t c0, int64_t c1, int32_t *rowptr, int32_t *col_out, float *val_out, int64_t *nnz_host,
                             void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(n_edges >= 0 && r0 <= r1 && c0 <= c1 && r0 >= 0 && c0 >= 0, "coo_to_csr: bad sizes");
    const int64_t Mb = r1 - r0, Kb = c1 - c0;
    PLX_REQUIRE(Mb < (1ll << 31) - 1 && Kb < (1ll << 31) - 1 && n_edges < (1ll << 31), "coo_to_csr: sizes exceed int32 indexing");
    PLX_REQUIRE(rowptr != nullptr && nnz_host != nullptr, "coo_to_csr: NULL output");
    hipStream_t st = plx::as_stream(stream);
    *nnz_host = 0;
    if (n_edges == 0 || Mb == 0 || Kb == 0) {
        zero_i32_kernel<<<blocks_for(Mb + 1), 256, 0, st>>>(Mb + 1, rowptr);
        PLX_LAUNCH_CHECK("zero_i32_kernel");
        return PLX_OK;
    }
    PLX_REQUIRE(row && col && weight && col_out && val_out, "coo_to_csr: NULL operand");
    const int key_bits = bits_for(Mb * Kb);
    CooLayout l;
    int rc = coo_layout(n_edges, key_bits, l);
    if (rc != PLX_OK) return rc;
    if (workspace == nullptr || workspace_bytes < l.total)
        return plx::fail(PLX_ERR_WORKSPACE, "coo_to_csr: workspace of %zu bytes needed, %zu given", l.total, workspace_bytes);
    PLX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "coo_to_csr: workspace must be 256-byte aligned");
    char *ws = static_cast<char *>(workspace);
    uint64_t *keys = reinterpret_cast<uint64_t *>(ws + l.keys);
    uint8_t *flags = reinterpret_cast<uint8_t *>(ws + l.flags);
    uint64_t *keys_c = reinterpret_cast<uint64_t *>(ws + l.keys_c);
    float *w_c = reinterpret_cast<float *>(ws + l.w_c);
    uint64_t *keys_s = reinterpret_cast<uint64_t *>(ws + l.keys_s);
    float *w_s = reinterpret_cast<float *>(ws + l.w_s);
    int32_t *run_scan = reinterpret_cast<int32_t *>(ws + l.run_scan);
    int64_t *count = reinterpret_cast<int64_t *>(ws + l.count);

    // 1. mask to the block and re-base (dataloader.py:343-354)
    block_keys_kernel<<<blocks_for(n_edges), 256, 0, st>>>(n_edges, row, col, r0, r1, c0, c1, keys, flags);
    PLX_LAUNCH_CHECK("block_keys_kernel");
    size_t temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::select(ws + l.temp, temp, keys, flags, keys_c, count, (size_t)n_edges, st));
    int64_t kept = 0;
    PLX_HIP_CHECK(hipMemcpyAsync(&kept, count, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    if (kept == 0) {
        zero_i32_kernel<<<blocks_for(Mb + 1), 256, 0, st>>>(Mb + 1, rowptr);
        PLX_LAUNCH_CHECK("zero_i32_kernel");
        return PLX_OK;
    }
    const float *w_in = weight;  // every edge kept (the block is the whole matrix): the weights are sorted from where they lie
    if (kept != n_edges) {
        temp = l.temp_bytes;
        PLX_HIP_CHECK(rocprim::select(ws + l.temp, temp, weight, flags, w_c, count, (size_t)n_edges, st));
        w_in = w_c;
    }
    // 2. sort by (row, col); the sort is stable, so duplicates of an edge are added in their input order
    temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::radix_sort_pairs(ws + l.temp, temp, kept == n_edges ? keys : keys_c, keys_s, w_in, w_s, (size_t)kept, 0,
                                            (unsigned)key_bits, st));
    // 3. coalesce duplicates (sparse_coo_tensor(...).to_sparse_csr() sums them, dataloader.py:356-367); row pointers
    //    and columns come from the same pass
    rc = merge_sorted(kept, keys_s, w_s, run_scan, ws + l.temp, l.temp_bytes, Mb, nullptr, rowptr, col_out, val_out, RowOfBlockKey{Kb},
                      ColOfBlockKey{Kb}, st);
    if (rc != PLX_OK) return rc;
    int32_t uniq = 0;
    PLX_HIP_CHECK(hipMemcpyAsync(&uniq, rowptr + Mb, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    *nnz_host = uniq;
    return PLX_OK;
}

size_t plx_gcn_norm_edges_workspace_bytes(int64_t n_edges, int64_t N)
{
    if (n_edges < 0 || N <= 0) return 256;
    NormLayout l;
    if (norm_layout(n_edges, N, l) != PLX_OK) return 0;
    return l.total;
}

int plx_gcn_norm_edges_f32(int64_t n_edges, const int64_t *row, const int64_t *col, const float *weight, int64_t N, int transposed,
                           int32_t *rowptr, int32_t *col_out, float *val_out, int64_t *nnz_host, void *workspace,
                           size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(n_edges >= 0 && N >= 0, "gcn_norm_edges: negative size");
    PLX_REQUIRE(N < (1ll << 31) - 1 && n_edges + N < (1ll << 31), "gcn_norm_edges: sizes exceed int32 indexing");
    PLX_REQUIRE(rowptr != nullptr && nnz_host != nullptr, "gcn_norm_edges: NULL output");
    hipStream_t st = plx::as_stream(stream);
    *nnz_host = 0;
    if (N == 0) {
        zero_i32_kernel<<<1, 256, 0, st>>>(1, rowptr);
        PLX_LAUNCH_CHECK("zero_i32_kernel");
        return PLX_OK;
    }
    PLX_REQUIRE((n_edges == 0 || (row && col)) && col_out && val_out, "gcn_norm_edges: NULL operand");
    NormLayout l;
    int rc = norm_layout(n_edges, N, l);
    if (rc != PLX_OK) return rc;
    if (workspace == nullptr || workspace_bytes < l.total)
        return plx::fail(PLX_ERR_WORKSPACE, "gcn_norm_edges: workspace of %zu bytes needed, %zu given", l.total, workspace_bytes);
    PLX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "gcn_norm_edges: workspace must be 256-byte aligned");
    char *ws = static_cast<char *>(workspace);
    uint64_t *keys_a = reinterpret_cast<uint64_t *>(ws + l.keys_a);
    uint64_t *keys_b = reinterpret_cast<uint64_t *>(ws + l.keys_b);
    float *w_a = reinterpret_cast<float *>(ws + l.w_a);
    float *w_b = reinterpret_cast<float *>(ws + l.w_b);
    int32_t *run_scan = reinterpret_cast<int32_t *>(ws + l.run_scan);
    int32_t *segptr = reinterpret_cast<int32_t *>(ws + l.segptr);
    float *dinv = reinterpret_cast<float *>(ws + l.dinv);
    uint8_t *has_loop = reinterpret_cast<uint8_t *>(ws + l.has_loop);
    const int64_t n = n_edges + N;
    const unsigned fb = (unsigned)l.field_bits;

    // 1. keys and weights of the edges, then of the self loops that are missing (the first step of T.GCNNorm, dataset.py:101)
    zero_u8_kernel<<<blocks_for(N), 256, 0, st>>>(N, has_loop);
    PLX_LAUNCH_CHECK("zero_u8_kernel");
    if (n_edges > 0) {
        norm_keys_kernel<<<blocks_for(n_edges), 256, 0, st>>>(n_edges, row, col, weight, N, transposed, keys_a, w_a, has_loop);
        PLX_LAUNCH_CHECK("norm_keys_kernel");
    }
    norm_loop_keys_kernel<<<blocks_for(N), 256, 0, st>>>(N, has_loop, keys_a + n_edges, w_a + n_edges);
    PLX_LAUNCH_CHECK("norm_loop_keys_kernel");
    // 2. a stable sort by the low field, then by the high field, leaves the entries ordered by (row, column) of the
    //    result.  The weighted in-degree is the sum over the edges that share a target: that is the low field of
    //    A-hat (read off between the two sorts) and the high field of its transpose (read off after both).
    size_t temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::radix_sort_pairs(ws + l.temp, temp, keys_a, keys_b, w_a, w_b, (size_t)n, 0, fb, st));
    if (!transposed) {
        rowptr_from_sorted_kernel<uint64_t><<<blocks_for(n + 1), 256, 0, st>>>(n, keys_b, N + 1, segptr, LowField());
        PLX_LAUNCH_CHECK("rowptr_from_sorted_kernel");
        rc = plx::row_sums_rsqrt(N, segptr, w_b, dinv, stream);
        if (rc != PLX_OK) return rc;
    }
    temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::radix_sort_pairs(ws + l.temp, temp, keys_b, keys_a, w_b, w_a, (size_t)n, 32, 32 + fb, st));
    if (transposed) {
        rowptr_from_sorted_kernel<uint64_t><<<blocks_for(n + 1), 256, 0, st>>>(n, keys_a, N + 1, segptr, HighField());
        PLX_LAUNCH_CHECK("rowptr_from_sorted_kernel");
        rc = plx::row_sums_rsqrt(N, segptr, w_a, dinv, stream);
        if (rc != PLX_OK) return rc;
    }
    // 3. duplicates summed, values scaled by 1/sqrt(d_row d_col), row pointers
    rc = merge_sorted(n, keys_a, w_a, run_scan, ws + l.temp, l.temp_bytes, N, dinv, rowptr, col_out, val_out, HighField(), LowField(), st);
    if (rc != PLX_OK) return rc;
    int32_t nnz = 0;
    PLX_HIP_CHECK(hipMemcpyAsync(&nnz, rowptr + N, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    *nnz_host = nnz;
    return PLX_OK;
}

size_t plx_csr_permute_transposed_workspace_bytes(int64_t M, int64_t K, int64_t nnz)
{
    if (M <= 0 || K <= 0 || nnz <= 0) return 256;
    PermuteLayout l;
    if (permute_layout(M, K, nnz, l) != PLX_OK) return 0;
    return l.total;
}

int plx_csr_permute_transposed_f32(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, const float *val,
                                   const int64_t *perm_rows, const int64_t *new_col, int32_t *rowptr_out, int32_t *col_out,
                                   float *val_out, void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(M >= 0 && K >= 0 && nnz >= 0, "csr_permute: negative size");
    PLX_REQUIRE(M < (1ll << 31) - 1 && K < (1ll << 31) - 1 && nnz < (1ll << 31), "csr_permute: sizes exceed int32 indexing");
    PLX_REQUIRE(rowptr_out != nullptr, "csr_permute: NULL rowptr_out");
    hipStream_t st = plx::as_stream(stream);
    if (nnz == 0 || M == 0 || K == 0) {
        zero_i32_kernel<<<blocks_for(K + 1), 256, 0, st>>>(K + 1, rowptr_out);
        PLX_LAUNCH_CHECK("zero_i32_kernel");
        return PLX_OK;
    }
    PLX_REQUIRE(rowptr && col && val && perm_rows && new_col && col_out && val_out, "csr_permute: NULL operand");
    PermuteLayout l;
    int rc = permute_layout(M, K, nnz, l);
    if (rc != PLX_OK) return rc;
    if (workspace == nullptr || workspace_bytes < l.total)
        return plx::fail(PLX_ERR_WORKSPACE, "csr_permute: workspace of %zu bytes needed, %zu given", l.total, workspace_bytes);
    PLX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "csr_permute: workspace must be 256-byte aligned");
    char *ws = static_cast<char *>(workspace);
    int32_t *len = reinterpret_cast<int32_t *>(ws + l.len);
    int32_t *moved_ptr = reinterpret_cast<int32_t *>(ws + l.moved_ptr);
    int32_t *out_of_range = reinterpret_cast<int32_t *>(ws + l.flag);
    int32_t *keys_in = reinterpret_cast<int32_t *>(ws + l.keys_in);
    char *sort_ws = ws + l.sort;
    int32_t *keys_out = reinterpret_cast<int32_t *>(sort_ws + l.t.keys_out);
    uint64_t *pay_in = reinterpret_cast<uint64_t *>(sort_ws + l.t.pay_in);
    uint64_t *pay_out = reinterpret_cast<uint64_t *>(sort_ws + l.t.pay_out);

    // 1. the source rows in their new order: lengths and where each begins; both maps checked for ids out of range
    zero_i32_kernel<<<1, 64, 0, st>>>(1, out_of_range);
    PLX_LAUNCH_CHECK("zero_i32_kernel");
    permuted_row_length_kernel<<<blocks_for(M + 1), 256, 0, st>>>(M, rowptr, perm_rows, len, out_of_range);
    PLX_LAUNCH_CHECK("permuted_row_length_kernel");
    ids_in_range_kernel<<<blocks_for(K), 256, 0, st>>>(K, new_col, K, out_of_range);
    PLX_LAUNCH_CHECK("ids_in_range_kernel");
    size_t temp = l.scan_temp;
    PLX_HIP_CHECK(rocprim::exclusive_scan(sort_ws, temp, len, moved_ptr, (int32_t)0, (size_t)(M + 1), rocprim::plus<int32_t>(), st));
    int32_t total = 0, stray = 0;
    PLX_HIP_CHECK(hipMemcpyAsync(&total, moved_ptr + M, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipMemcpyAsync(&stray, out_of_range, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    if (stray != 0) return plx::fail(PLX_ERR_INVALID, "csr_permute: a row or column id of the maps lies outside the matrix");
    if (total != nnz)
        return plx::fail(PLX_ERR_INVALID, "csr_permute: perm_rows is not a permutation of the rows (%d entries selected, %lld stored)",
                         total, (long long)nnz);
    // 2. keys (new column) and payloads (new row, value) in that order, then the stable sort by key of the
    //    transpose: within a new column the entries keep their order, i.e. ascending new row
    gather_moved_rows_kernel<<<(unsigned)plx::ceil_div(nnz, kPackPerBlock), 256, 0, st>>>(nnz, M, moved_ptr, rowptr, col, val, perm_rows,
                                                                                       new_col, keys_in, pay_in);
    PLX_LAUNCH_CHECK("gather_moved_rows_kernel");
    temp = l.t.temp_bytes;
    PLX_HIP_CHECK(rocprim::radix_sort_pairs(sort_ws + l.t.temp, temp, keys_in, keys_out, pay_in, pay_out, (size_t)nnz, 0,
                                            (unsigned)bits_for(K), st));
    rowptr_from_sorted_kernel<int32_t><<<blocks_for(nnz + 1), 256, 0, st>>>(nnz, keys_out, K, rowptr_out, RowOfColumnKey());
    PLX_LAUNCH_CHECK("rowptr_from_sorted_kernel");
    unpack_row_value_kernel<<<blocks_for(nnz), 256, 0, st>>>(nnz, pay_out, col_out, val_out);
    PLX_LAUNCH_CHECK("unpack_row_value_kernel");
    return PLX_OK;
}

}  // extern "C"
