// Hub-row pass of the SpMM (spmm_hub.hip): the longest rows of A, multiplied window by window so that the rows of H
// they gather are shared through the L2 of an XCD.  Tables, their construction and the launcher used by spmm.hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <vector>

namespace plx {
namespace hub {

constexpr int kHubRanges = 8;        // column ranges, one per XCD (workgroup b works on range b % 8)
constexpr int kHubGroups = 32;       // workgroups per range, one per compute unit of an XCD
constexpr int kWaves = 8;            // wavefronts per workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kHubRowsPerWave = 36;  // (slot, range) sums a wavefront owns: 8 x 36 rows x 128 columns x 4 bytes = 144 KB of LDS
constexpr int kHubVec = 4;           // elements of a row of H per lane: half a wavefront reads 128 columns
constexpr int kHubTile = 32 * kHubVec;
constexpr int kHubSlots = kHubGroups * kWaves * kHubRowsPerWave;  // 9,216 slots: a hub row takes one per part
// The wide layout, for bf16 rows of 512 bytes and more: half a wavefront reads 256 columns with 16 bytes per lane, so a
// sum is 256 floats and a wavefront owns half as many of them (8 x 18 x 256 x 4 bytes: the same 144 KB); the parts of a
// hub row are twice as long, so about as many rows find a slot.
constexpr int kHubRowsPerWaveWide = 18;
constexpr int kHubTileWide = 256;
constexpr int kHubStreams = kHubRanges * kHubGroups * kWaves;     // one per wavefront of the pass
constexpr int kHubWindow = 4096;     // columns per window: 2 MB of 512-byte rows, half of an XCD's L2
constexpr int kHubMaxWindows = 4096;  // windows per range a plan may have
constexpr int kHubPace = 1;          // windows a wavefront may run ahead of the slowest of its workgroup (measured, hub pass of the
                                     // 2.45 M-node graph: none 1.36 ms and 6.1 GB fetched, 0 / 1 / 2 / 3: 1.35 / 1.27 / 1.30 / 1.31 ms, 1: 3.9 GB)
constexpr int kHubMaxPolls = 4096;   // of a wavefront waiting for the others, then it goes on regardless
constexpr int kHubPartFactor = 16;   // a hub row is cut into parts of at most kHubPartFactor * seg_len entries (8 / 16 / 32 / 64 on the
                                     // 2.45 M-node graph: 6,530 / 8,170 / 8,820 / 9,074 hub rows, product 5.73 / 5.69 / 5.67 / 5.68 ms)
constexpr int kHubPartFactorWide = 32;
constexpr int64_t kHubMaxBytes = 1ll << 32;  // rows of H are addressed with 32-bit byte offsets

// Device tables of a plan's hub pass.  A slot is a part of a hub row; the slots are dealt over the wavefronts by size.
struct HubPlan {
    int32_t n_rows = 0;    // hub rows
    int32_t n_slots = 0;   // slots in use
    int64_t entries = 0;   // entries of A in hub rows
    int64_t stored = 0;    // entries of the streams, padding included
    double mean_run = 0;   // entries per (slot, window): how long a wavefront adds into one sum before it changes
    int32_t window = 0, n_windows = 0, windows_per_range = 0;
    int32_t rows_per_wave = 0;     // kHubRowsPerWave, or kHubRowsPerWaveWide for the wide layout
    int32_t slot_cap = 0;          // kHubGroups * kWaves * rows_per_wave: slots of the layout, used or not
    void *block = nullptr;         // one device allocation behind every pointer below
    const int32_t *hub_row = nullptr;         // [slot_cap] row of a slot, -1 for an empty slot
    const int32_t *rows = nullptr;            // [n_rows] hub rows, longest first
    const int32_t *row_slot_first = nullptr;  // [n_rows + 1]
    const int32_t *row_slots = nullptr;       // [n_slots] slots of a row, in part order
    const int64_t *stream_first = nullptr;    // [kHubStreams] first entry of a wavefront's stream
    const int32_t *stream_total = nullptr;    // [kHubStreams] entries of the stream (stored padded to whole batches of 64)
    const int32_t *stream_pos = nullptr;      // [stored] position of an entry in the CSR arrays
    const uint8_t *stream_run = nullptr;      // [stored] its slot among the wavefront's rows_per_wave
    const int32_t *stream_mark = nullptr;     // [kHubStreams][windows_per_range] batch of the stream in which a window begins
    const uint8_t *long_is_hub = nullptr;     // [n_long] flags over the plan's split rows
    const uint8_t *seg_is_hub = nullptr;      // [n_seg] flags over their segments
    std::vector<int32_t> h_rows_sorted;       // hub rows in ascending order (host), to intersect with a row range
};

// Chooses the hub rows among the split rows (`long_rows`, ascending, with their segments in seg_first), longest first
// while slots last, and builds the tables, in the regular layout (128-column tiles, kHubRowsPerWave sums per wavefront,
// parts of kHubPartFactor * seg_len entries) or the wide one.  Leaves `out` empty (block == nullptr) when no row
// qualifies or the chosen rows hold fewer than `min_entries` entries.  Synchronises
// `st`.  Returns a plx_status.
int build_hub_plan(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, int32_t seg_len, int64_t n_long,
                   int64_t n_seg, const int32_t *long_rows, const int32_t *seg_first, const std::vector<int32_t> &h_long_rows,
                   int64_t min_entries, bool wide, hipStream_t st, HubPlan &out);
void free_hub_plan(HubPlan &hp);

// bytes of the partial sums of a pass over D columns in either layout (both hold 8 ranges x 147,456 bytes per 128 columns
// of a 128- or 256-column tile)
size_t partial_bytes(int64_t D, bool wide);

// One pass: Y[r] for the hub rows r in [row_begin, row_end).  `d_read` = columns of a row of H that may be read (a
// multiple of kHubVec: D itself, or D rounded up where the row pitch covers it).  Rows of H: K * ldh * sizeof(T) <
// kHubMaxBytes, 16-byte aligned (fp32) or 8-byte aligned (bf16) base and pitch; a plan in the wide layout takes bf16
// rows only, 16-byte aligned, with d_read a multiple of 8.  `run_pass`: compute the partial sums of
// every hub row into `partial` (false: they are there from an earlier call with the same operands); `run_reduce`: add
// up the hub rows of the range.
int launch(const HubPlan &hp, const int32_t *col, const float *val, const void *H, int64_t ldh, int64_t D, int64_t d_read, bool bf16,
           int64_t row_begin, int64_t row_end, void *Y, int64_t ldy, float *partial, hipStream_t st, bool run_pass = true,
           bool run_reduce = true);

}  // namespace hub
}  // namespace plx
