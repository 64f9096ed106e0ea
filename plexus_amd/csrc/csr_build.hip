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

__global__ void split_keys_kernel(int64_t n, const int64_t *__restrict__ n_ptr, const uint64_t *__restrict__ keys, int64_t kb,
                                  int32_t *__restrict__ col)
{
    const int64_t total = n_ptr ? *n_ptr : n;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) col[i] = (int32_t)(keys[i] % (uint64_t)kb);
}

struct RowOfColumnKey {
    __device__ int64_t operator()(int32_t k) const { return (int64_t)k; }
};
struct RowOfBlockKey {
    int64_t kb;
    __device__ int64_t operator()(uint64_t k) const { return (int64_t)(k / (uint64_t)kb); }
};

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
    size_t keys, flags, keys_c, w_c, keys_s, w_s, keys_u, count, temp, temp_bytes, total;
};

int coo_layout(int64_t n, int key_bits, CooLayout &l)
{
    size_t t1 = 0, t2 = 0, t3 = 0;
    hipError_t e = rocprim::select(nullptr, t1, (const uint64_t *)nullptr, (const uint8_t *)nullptr, (uint64_t *)nullptr,
                                   (int64_t *)nullptr, (size_t)n, (hipStream_t)0);
    if (e == hipSuccess)
        e = rocprim::radix_sort_pairs(nullptr, t2, (const uint64_t *)nullptr, (uint64_t *)nullptr, (const float *)nullptr,
                                      (float *)nullptr, (size_t)n, 0, (unsigned)key_bits, (hipStream_t)0);
    if (e == hipSuccess)
        e = rocprim::reduce_by_key(nullptr, t3, (const uint64_t *)nullptr, (const float *)nullptr, (size_t)n, (uint64_t *)nullptr,
                                   (float *)nullptr, (int64_t *)nullptr, rocprim::plus<float>(), rocprim::equal_to<uint64_t>(),
                                   (hipStream_t)0);
    if (e != hipSuccess) return plx::fail(PLX_ERR_HIP, "coo_to_csr: temporary-storage query failed: %s", hipGetErrorString(e));
    const size_t temp = std::max(t1, std::max(t2, t3));
    size_t off = 0;
    l.keys = off;   off += align_up(8 * (size_t)n);
    l.flags = off;  off += align_up((size_t)n);
    l.keys_c = off; off += align_up(8 * (size_t)n);
    l.w_c = off;    off += align_up(4 * (size_t)n);
    l.keys_s = off; off += align_up(8 * (size_t)n);
    l.w_s = off;    off += align_up(4 * (size_t)n);
    l.keys_u = off; off += align_up(8 * (size_t)n);
    l.count = off;  off += 256;
    l.temp = off;   off += align_up(temp);
    l.temp_bytes = temp;
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
    uint64_t *keys_u = reinterpret_cast<uint64_t *>(ws + l.keys_u);
    int64_t *count = reinterpret_cast<int64_t *>(ws + l.count);

    // 1. mask to the block and re-base (dataloader.py:343-354)
    block_keys_kernel<<<blocks_for(n_edges), 256, 0, st>>>(n_edges, row, col, r0, r1, c0, c1, keys, flags);
    PLX_LAUNCH_CHECK("block_keys_kernel");
    size_t temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::select(ws + l.temp, temp, keys, flags, keys_c, count, (size_t)n_edges, st));
    temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::select(ws + l.temp, temp, weight, flags, w_c, count, (size_t)n_edges, st));
    int64_t kept = 0;
    PLX_HIP_CHECK(hipMemcpyAsync(&kept, count, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    if (kept == 0) {
        zero_i32_kernel<<<blocks_for(Mb + 1), 256, 0, st>>>(Mb + 1, rowptr);
        PLX_LAUNCH_CHECK("zero_i32_kernel");
        return PLX_OK;
    }
    // 2. sort by (row, col); the sort is stable, so duplicates of an edge are added in their input order
    temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::radix_sort_pairs(ws + l.temp, temp, keys_c, keys_s, w_c, w_s, (size_t)kept, 0, (unsigned)key_bits, st));
    // 3. coalesce duplicates (sparse_coo_tensor(...).to_sparse_csr() sums them, dataloader.py:356-367)
    temp = l.temp_bytes;
    PLX_HIP_CHECK(rocprim::reduce_by_key(ws + l.temp, temp, keys_s, w_s, (size_t)kept, keys_u, val_out, count, rocprim::plus<float>(),
                                         rocprim::equal_to<uint64_t>(), st));
    int64_t uniq = 0;
    PLX_HIP_CHECK(hipMemcpyAsync(&uniq, count, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    // 4. row pointers and columns from the unique keys
    rowptr_from_sorted_kernel<uint64_t><<<blocks_for(uniq + 1), 256, 0, st>>>(uniq, keys_u, Mb, rowptr, RowOfBlockKey{Kb});
    PLX_LAUNCH_CHECK("rowptr_from_sorted_kernel");
    split_keys_kernel<<<blocks_for(uniq), 256, 0, st>>>(uniq, nullptr, keys_u, Kb, col_out);
    PLX_LAUNCH_CHECK("split_keys_kernel");
    *nnz_host = uniq;
    return PLX_OK;
}

}  // extern "C"
