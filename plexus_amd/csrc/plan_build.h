// Row analysis behind plx_spmm_plan_create, on the device: validation of the CSR arrays and the tables of the rows
// that are split into segments.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

namespace plx {

struct PlanTables {
    int64_t n_long = 0, n_seg = 0;
    int32_t *tables = nullptr;  // device: long_rows[n_long] | seg_first[n_long + 1] | seg_begin[n_seg] | seg_end[n_seg]
    std::vector<int32_t> h_long_rows, h_seg_first;  // host copies of the first two
};

// Checks that rowptr runs from 0 to nnz without decreasing and that every column lies in [0, K); finds the rows longer
// than seg_len, in ascending order, and cuts each into ceil(len / seg_len) near-equal segments (the first len % parts
// segments one entry longer) -- the tables plx_spmm_segments_host builds on the host.  Synchronises `st`; what it
// allocates besides `tables` it frees before returning.  Returns a plx_status.
int build_plan_tables(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, int32_t seg_len, hipStream_t st,
                      PlanTables &out);

}  // namespace plx
