// Device-side construction of the SpMM plan: one pass over the row pointers and one over the columns validate the
// matrix and count the rows to split; the tables of those rows are then built with a stream compaction, a prefix sum
// and one workgroup per split row.  Only four counters and the two short tables that row-range products need on the host
// cross PCIe (the row pointers of a 2.4 M-row matrix alone are 10 MB, and looping over them on the host took longer
// than three products).
#include <cstring>  // rocPRIM's texture iterator calls memset without including it

#include <hip/hip_runtime.h>
#include <rocprim/rocprim.hpp>

#include <algorithm>

#include "common.h"
#include "plan_build.h"

namespace {

struct Counters {
    unsigned long long n_long, n_seg, bad_rowptr, bad_col;
};

__global__ void zero_counters_kernel(Counters *c)
{
    c->n_long = c->n_seg = c->bad_rowptr = c->bad_col = 0ull;
}

__device__ __forceinline__ int32_t parts_of(int32_t len, int32_t seg_len) { return len <= seg_len ? 0 : (len + seg_len - 1) / seg_len; }

__global__ void __launch_bounds__(256) scan_rows_kernel(int64_t M, int64_t nnz, const int32_t *__restrict__ rowptr, int32_t seg_len,
                                                        Counters *__restrict__ c)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    unsigned long long n_long = 0, n_seg = 0, bad = 0;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (first == 0) bad += (rowptr[0] != 0 ? 1u : 0u) + ((int64_t)rowptr[M] != nnz ? 1u : 0u);
    for (int64_t r = first; r < M; r += stride) {
        const int32_t a = rowptr[r], b = rowptr[r + 1];
        if (b < a) {
            ++bad;
            continue;
        }
        const int32_t p = parts_of(b - a, seg_len);
        if (p > 0) {
            ++n_long;
            n_seg += (unsigned long long)p;
        }
    }
    // integer sums: the totals do not depend on the order of the atomic additions
    if (n_long) atomicAdd(&c->n_long, n_long);
    if (n_seg) atomicAdd(&c->n_seg, n_seg);
    if (bad) atomicAdd(&c->bad_rowptr, bad);
}

__global__ void __launch_bounds__(256) scan_columns_kernel(int64_t nnz, const int32_t *__restrict__ col, int32_t K, Counters *__restrict__ c)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    unsigned long long bad = 0;
    for (; i < nnz; i += stride) bad += (unsigned int)col[i] >= (unsigned int)K ? 1u : 0u;
    if (bad) atomicAdd(&c->bad_col, bad);
}

struct IsLongRow {
    const int32_t *rowptr;
    int32_t seg_len;
    __device__ uint8_t operator()(int32_t r) const { return rowptr[r + 1] - rowptr[r] > seg_len ? 1 : 0; }
};

struct PartsOfLongRow {
    const int32_t *rowptr;
    const int32_t *long_rows;
    int32_t seg_len;
    __device__ int32_t operator()(int32_t q) const
    {
        const int32_t r = long_rows[q];
        return parts_of(rowptr[r + 1] - rowptr[r], seg_len);
    }
};

// one workgroup per split row: its segments, the first `len % parts` of them one entry longer
__global__ void __launch_bounds__(256) fill_segments_kernel(int32_t n_long, int32_t n_seg, const int32_t *__restrict__ rowptr, int32_t seg_len,
                                                            const int32_t *__restrict__ long_rows, int32_t *__restrict__ seg_first,
                                                            int32_t *__restrict__ seg_begin, int32_t *__restrict__ seg_end)
{
    const int32_t q = blockIdx.x;
    if (q == 0 && threadIdx.x == 0) seg_first[n_long] = n_seg;
    const int32_t r = long_rows[q];
    const int32_t a = rowptr[r], len = rowptr[r + 1] - a;
    const int32_t parts = parts_of(len, seg_len);
    const int32_t base = len / parts, extra = len % parts;
    const int32_t s0 = seg_first[q];
    for (int32_t s = threadIdx.x; s < parts; s += blockDim.x) {
        const int32_t begin = a + s * base + min(s, extra);
        seg_begin[s0 + s] = begin;
        seg_end[s0 + s] = begin + base + (s < extra ? 1 : 0);
    }
}

unsigned blocks_for(int64_t n, int64_t per_thread) { return (unsigned)std::max<int64_t>(1, std::min<int64_t>(plx::ceil_div(n, 256 * per_thread), 8192)); }

struct DeviceBlock {  // freed on every way out
    void *p = nullptr;
    ~DeviceBlock()
    {
        if (p) (void)hipFree(p);
    }
};

}  // namespace

namespace plx {

int build_plan_tables(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, int32_t seg_len, hipStream_t st,
                      PlanTables &out)
{
    out = PlanTables();
    // temporary storage of the compaction and the prefix sum, sized for the largest inputs they can get
    rocprim::counting_iterator<int32_t> rows_it(0);
    auto flags_it = rocprim::make_transform_iterator(rows_it, IsLongRow{rowptr, seg_len});
    size_t t_select = 0, t_scan = 0;
    hipError_t e = rocprim::select(nullptr, t_select, rows_it, flags_it, (int32_t *)nullptr, (unsigned long long *)nullptr, (size_t)M, st);
    if (e == hipSuccess) {
        auto parts_it = rocprim::make_transform_iterator(rows_it, PartsOfLongRow{rowptr, nullptr, seg_len});
        e = rocprim::exclusive_scan(nullptr, t_scan, parts_it, (int32_t *)nullptr, (int32_t)0, (size_t)std::max<int64_t>(M, 1),
                                    rocprim::plus<int32_t>(), st);
    }
    if (e != hipSuccess) return plx::fail(PLX_ERR_HIP, "plan_create: temporary-storage query failed: %s", hipGetErrorString(e));
    const size_t temp_bytes = std::max(t_select, t_scan);
    DeviceBlock scratch;
    e = hipMalloc(&scratch.p, 512 + temp_bytes);
    if (e != hipSuccess) return plx::fail(PLX_ERR_NOMEM, "plan_create: hipMalloc of %zu bytes failed: %s", 512 + temp_bytes, hipGetErrorString(e));
    Counters *d_counters = static_cast<Counters *>(scratch.p);
    unsigned long long *d_selected = reinterpret_cast<unsigned long long *>(static_cast<char *>(scratch.p) + 256);
    void *d_temp = static_cast<char *>(scratch.p) + 512;

    zero_counters_kernel<<<1, 1, 0, st>>>(d_counters);
    PLX_LAUNCH_CHECK("zero_counters_kernel");
    scan_rows_kernel<<<blocks_for(M, 4), 256, 0, st>>>(M, nnz, rowptr, seg_len, d_counters);
    PLX_LAUNCH_CHECK("scan_rows_kernel");
    if (nnz > 0) {
        scan_columns_kernel<<<blocks_for(nnz, 8), 256, 0, st>>>(nnz, col, (int32_t)K, d_counters);
        PLX_LAUNCH_CHECK("scan_columns_kernel");
    }
    Counters h{};
    PLX_HIP_CHECK(hipMemcpyAsync(&h, d_counters, sizeof(Counters), hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    PLX_REQUIRE(h.bad_rowptr == 0,
                "plan_create: rowptr decreases, does not start at 0 or does not end at nnz=%lld (%llu violations)", (long long)nnz,
                h.bad_rowptr);
    PLX_REQUIRE(h.bad_col == 0, "plan_create: %llu column indices lie outside [0, %lld)", h.bad_col, (long long)K);
    PLX_REQUIRE(h.n_seg < (1ull << 31), "plan_create: %llu segments exceed int32 indexing", h.n_seg);
    out.n_long = (int64_t)h.n_long;
    out.n_seg = (int64_t)h.n_seg;
    if (out.n_long == 0) return PLX_OK;

    const int64_t nl = out.n_long, ns = out.n_seg;
    const size_t total = (size_t)nl + (size_t)(nl + 1) + 2 * (size_t)ns;
    e = hipMalloc(reinterpret_cast<void **>(&out.tables), total * sizeof(int32_t));
    if (e != hipSuccess) {
        out.tables = nullptr;
        return plx::fail(PLX_ERR_NOMEM, "plan_create: hipMalloc of %zu bytes failed: %s", total * sizeof(int32_t), hipGetErrorString(e));
    }
    int32_t *long_rows = out.tables, *seg_first = long_rows + nl, *seg_begin = seg_first + nl + 1, *seg_end = seg_begin + ns;
    auto cleanup = [&](int rc) {
        (void)hipFree(out.tables);
        out.tables = nullptr;
        return rc;
    };
    size_t temp = temp_bytes;
    e = rocprim::select(d_temp, temp, rows_it, flags_it, long_rows, d_selected, (size_t)M, st);
    if (e == hipSuccess) {
        auto parts_it = rocprim::make_transform_iterator(rows_it, PartsOfLongRow{rowptr, long_rows, seg_len});
        temp = temp_bytes;
        e = rocprim::exclusive_scan(d_temp, temp, parts_it, seg_first, (int32_t)0, (size_t)nl, rocprim::plus<int32_t>(), st);
    }
    if (e != hipSuccess) return cleanup(plx::fail(PLX_ERR_HIP, "plan_create: building the segment tables failed: %s", hipGetErrorString(e)));
    fill_segments_kernel<<<(unsigned)nl, 256, 0, st>>>((int32_t)nl, (int32_t)ns, rowptr, seg_len, long_rows, seg_first, seg_begin, seg_end);
    e = hipGetLastError();
    out.h_long_rows.resize((size_t)nl);
    out.h_seg_first.resize((size_t)nl + 1);
    if (e == hipSuccess) e = hipMemcpyAsync(out.h_long_rows.data(), long_rows, sizeof(int32_t) * (size_t)nl, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipMemcpyAsync(out.h_seg_first.data(), seg_first, sizeof(int32_t) * (size_t)(nl + 1), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return cleanup(plx::fail(PLX_ERR_HIP, "plan_create: segment tables: %s", hipGetErrorString(e)));
    return PLX_OK;
}

}  // namespace plx
