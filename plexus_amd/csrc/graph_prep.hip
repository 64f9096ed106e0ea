// Streaming kernels of the graph preprocessing that precedes the layer: vertex relabelling by a
// permutation (the products P.A.P2^T of plexus/utils/dataset.py:128-190 written as index maps) and the
// CSR -> edge-list expansion that to_edge_index performs there (:195-199).  All bandwidth-bound,
// one pass each, no atomics.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "common.h"

namespace {

// inv[perm[i]] = i; entries of perm outside [0, n) are skipped
__global__ void __launch_bounds__(256) invert_permutation_kernel(int64_t n, const int64_t *__restrict__ perm,
                                                                 int64_t *__restrict__ inv)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t p = perm[i];
        if (p >= 0 && p < n) inv[p] = i;
    }
}

// (row, col) -> (map_row[row], map_col[col]); an id outside its map gives -1 for that entry
__global__ void __launch_bounds__(256) relabel_edges_kernel(int64_t n_edges, const int64_t *row, const int64_t *col,
                                                            const int64_t *__restrict__ map_row, int64_t n_rows,
                                                            const int64_t *__restrict__ map_col, int64_t n_cols,
                                                            int64_t *row_out, int64_t *col_out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_edges; e += stride) {
        const int64_t r = row[e], c = col[e];
        row_out[e] = (r >= 0 && r < n_rows) ? map_row[r] : -1;
        col_out[e] = (c >= 0 && c < n_cols) ? map_col[c] : -1;
    }
}

// entry j belongs to the row r with rowptr[r] <= j < rowptr[r + 1].  A workgroup takes 2,048 consecutive entries,
// finds the rows of its first and last entry once, and every entry then searches only between those two (no steps
// at all inside a long row), so hub rows cost no more than others.
constexpr int kCooPerBlock = 2048;
__global__ void __launch_bounds__(256) csr_to_coo_kernel(int64_t M, int64_t nnz, const int32_t *__restrict__ rowptr,
                                                         const int32_t *__restrict__ col, int64_t *__restrict__ row_out,
                                                         int64_t *__restrict__ col_out)
{
    __shared__ int32_t bounds[2];
    const int64_t e0 = (int64_t)blockIdx.x * kCooPerBlock;
    const int64_t e1 = min(e0 + kCooPerBlock, nnz) - 1;
    if (threadIdx.x < 2) {
        const int64_t j = threadIdx.x == 0 ? e0 : e1;
        int64_t lo = 0, hi = M;  // the answer r satisfies lo <= r < hi
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if ((int64_t)rowptr[mid] <= j)
                lo = mid;
            else
                hi = mid;
        }
        bounds[threadIdx.x] = (int32_t)lo;
    }
    __syncthreads();
    const int32_t r_first = bounds[0], r_last = bounds[1];
    for (int64_t j = e0 + threadIdx.x; j <= e1; j += 256) {
        int32_t lo = r_first, hi = r_last + 1;
        while (hi - lo > 1) {
            const int32_t mid = lo + ((hi - lo) >> 1);
            if ((int64_t)rowptr[mid] <= j)
                lo = mid;
            else
                hi = mid;
        }
        row_out[j] = lo;
        col_out[j] = col[j];
    }
}

unsigned grid_for(int64_t n) { return (unsigned)std::max<int64_t>(1, std::min<int64_t>(plx::ceil_div(n, 256), 256 * 32)); }

}  // namespace

extern "C" {

int plx_invert_permutation_i64(int64_t n, const int64_t *perm, int64_t *inv, void *stream)
{
    PLX_REQUIRE(n >= 0, "invert_permutation: negative size");
    if (n == 0) return PLX_OK;
    PLX_REQUIRE(perm && inv && perm != inv, "invert_permutation: NULL or aliased operand");
    invert_permutation_kernel<<<grid_for(n), 256, 0, plx::as_stream(stream)>>>(n, perm, inv);
    PLX_LAUNCH_CHECK("invert_permutation_kernel");
    return PLX_OK;
}

int plx_relabel_edges_i64(int64_t n_edges, const int64_t *row, const int64_t *col, const int64_t *map_row, int64_t n_rows,
                          const int64_t *map_col, int64_t n_cols, int64_t *row_out, int64_t *col_out, void *stream)
{
    PLX_REQUIRE(n_edges >= 0 && n_rows >= 0 && n_cols >= 0, "relabel_edges: negative size");
    if (n_edges == 0) return PLX_OK;
    PLX_REQUIRE(row && col && row_out && col_out && (map_row || n_rows == 0) && (map_col || n_cols == 0),
                "relabel_edges: NULL operand");
    relabel_edges_kernel<<<grid_for(n_edges), 256, 0, plx::as_stream(stream)>>>(n_edges, row, col, map_row, n_rows, map_col,
                                                                               n_cols, row_out, col_out);
    PLX_LAUNCH_CHECK("relabel_edges_kernel");
    return PLX_OK;
}

int plx_csr_to_coo_i64(int64_t M, int64_t nnz, const int32_t *rowptr, const int32_t *col, int64_t *row_out, int64_t *col_out,
                       void *stream)
{
    PLX_REQUIRE(M >= 0 && nnz >= 0 && M < (1ll << 31) - 1 && nnz < (1ll << 31), "csr_to_coo: bad shape");
    if (nnz == 0) return PLX_OK;
    PLX_REQUIRE(M > 0 && rowptr && col && row_out && col_out, "csr_to_coo: NULL operand or entries without rows");
    csr_to_coo_kernel<<<(unsigned)plx::ceil_div(nnz, kCooPerBlock), 256, 0, plx::as_stream(stream)>>>(M, nnz, rowptr, col, row_out, col_out);
    PLX_LAUNCH_CHECK("csr_to_coo_kernel");
    return PLX_OK;
}

}  // extern "C"
