// The rows of A with the most entries ("hub rows"), multiplied window by window.
//
// On a power-law graph a third of the entries sit in a few thousand rows.  Taken row by row they gather rows of H
// from all over the matrix like every other row and miss the cache four times out of five.  Here all of them walk
// the columns together: the columns are cut into kHubRanges ranges, one per XCD, and every range into windows of
// kHubWindow columns whose rows of H fit the XCD's L2; the kHubGroups workgroups of a range go through its windows
// in the same order, each adding the entries that its own rows have in the window, so that a row of H fetched for
// one hub row is found in L2 by the others that reference it.
//
// A hub row is cut into parts of bounded length ("slots": part s of S takes the s-th S-th of the row's entries inside
// every window), and the slots are dealt over the wavefronts by size.  A workgroup keeps the sums of its slots for its
// range in LDS for the whole pass; a wavefront owns kHubRowsPerWave of them, so no two wavefronts touch the same sum
// and no sum needs an atomic or a barrier (all that wavefronts tell each other is the window they are in, so that
// none runs far ahead of the rows of H the others still share: "pacing" in the kernel).  The entries of a slot inside a window are a contiguous run of the CSR
// arrays (columns are sorted within a row); the plan writes out, for every wavefront, the runs of its slots window
// after window as one stream of positions.  The partial sums of the kHubRanges ranges of a slot go to memory and a
// second kernel adds them, slot by slot and range by range, into the row of Y: the order of every sum is fixed by
// the plan, so the result does not change from call to call or with the row range of the call.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <functional>
#include <numeric>
#include <queue>
#include <utility>
#include <type_traits>
#include <vector>

#include "common.h"
#include "spmm_hub.h"

#ifndef PLX_HUB_U
#define PLX_HUB_U 8
#endif

namespace {

using plx::kWave;
using namespace plx::hub;

struct HubArgs {
    const int32_t *col;
    const float *val;
    const void *H;
    int64_t ldh;
    int32_t D, d_read;
    const int32_t *hub_row;
    const int64_t *stream_first;
    const int32_t *stream_total;
    const int32_t *stream_pos;
    const uint8_t *stream_run;
    const int32_t *stream_mark;  // [streams][windows_per_range] batch in which a window of the range begins
    int32_t windows_per_range;
    int32_t pace;                // windows a wavefront may be ahead of the slowest of its workgroup (< 0: no pacing)
    int32_t n_rows;
    const int32_t *rows;
    const int32_t *row_slot_first;
    const int32_t *row_slots;
    int32_t row_begin, row_end;
    float *partial;  // [kHubRanges][slot_cap][ldp]
    int64_t ldp;
    int32_t slot_cap;  // slots of the plan's layout (kHubGroups * kWaves * sums per wavefront)
};

// The VEC elements of a row of H that a lane reads, as they lie in memory: converted to fp32 only where they are added
// up, so that nothing between a load and its use touches the loaded registers.
template <typename T, int VEC>
struct RawVec;
template <>
struct RawVec<float, 4> {
    float4 r;
    __device__ __forceinline__ void load(const void *p) { r = *reinterpret_cast<const float4 *>(p); }
    __device__ __forceinline__ void widen(float (&o)[4]) const
    {
        o[0] = r.x;
        o[1] = r.y;
        o[2] = r.z;
        o[3] = r.w;
    }
};
template <>
struct RawVec<uint16_t, 4> {
    uint2 r;
    __device__ __forceinline__ void load(const void *p) { r = *reinterpret_cast<const uint2 *>(p); }
    __device__ __forceinline__ void widen(float (&o)[4]) const
    {
        o[0] = __uint_as_float(r.x << 16);
        o[1] = __uint_as_float(r.x & 0xffff0000u);
        o[2] = __uint_as_float(r.y << 16);
        o[3] = __uint_as_float(r.y & 0xffff0000u);
    }
};
template <>
struct RawVec<uint16_t, 8> {
    uint4 r;
    __device__ __forceinline__ void load(const void *p) { r = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ void widen(float (&o)[8]) const
    {
        o[0] = __uint_as_float(r.x << 16);
        o[1] = __uint_as_float(r.x & 0xffff0000u);
        o[2] = __uint_as_float(r.y << 16);
        o[3] = __uint_as_float(r.y & 0xffff0000u);
        o[4] = __uint_as_float(r.z << 16);
        o[5] = __uint_as_float(r.z & 0xffff0000u);
        o[6] = __uint_as_float(r.w << 16);
        o[7] = __uint_as_float(r.w & 0xffff0000u);
    }
};

// One wavefront = one stream: the entries of its RPW slots inside its range of columns, window after
// window, written out by the plan as positions in the CSR arrays (stream_pos) and slot numbers (stream_run), padded
// to whole batches of 64.  A batch moves through four stages, one per turn of the loop, so that no load is waited for
// in the turn that issues it: positions and slots (coalesced) -> column and value of every entry (gathered) -> byte
// offset of the row of H and value into LDS, run boundaries as a bit mask -> rows of H.  The vector memory pipeline
// takes as long for a 64-lane load of 4 or 8 bytes per lane as for one of 16, so a row of H (a tile of LPR * VEC
// columns of it) is read by LPR lanes, 16 bytes per lane where the rows allow it, and the 64 / LPR lane groups go
// through different entries: group g through entries g * LPR ... of the batch, one per step, U steps at a time, the
// loads of one set of steps in flight while the set before is added up.  Every turn issues the same
// loads whatever it finds (past the end of the stream they repeat its last batch), so the counter of outstanding
// loads the hardware waits on has a fixed meaning.
template <typename T, int VEC, int LPR, int RPW>
__global__ void __launch_bounds__(kThreads, 1) spmm_hub_kernel(const HubArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TW = LPR * VEC;   // columns of H covered by a wavefront
    constexpr int G = kWave / LPR;  // lane groups: group g goes through entries g * STEPS ... of a batch, one per step
    constexpr int STEPS = kWave / G;
    constexpr int U = PLX_HUB_U;    // steps (G entries each) per set of loads
    constexpr int SETS = STEPS / U;
    static_assert(SETS == 2 || SETS == 4, "the steps of a batch are two or four sets");
    static_assert(VEC == 4 || VEC == 8, "a lane reads 4 or 8 elements");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int grp = lane / LPR;
    const int range = blockIdx.x % kHubRanges;  // workgroups go to the XCDs in turn
    const int group = blockIdx.x / kHubRanges;
    const int dl = (lane % LPR) * VEC;  // this lane's columns inside the tile
    const int d0 = blockIdx.y * TW + dl;
    // a lane whose columns lie past the readable width gathers the first columns instead; its sums are never stored
    const bool ok = d0 + VEC <= p.d_read;
    const int off = ok ? d0 : 0;

    float *acc = lds + (size_t)wave * RPW * TW;  // [RPW][TW], this wavefront's sums
    uint2 *ring = reinterpret_cast<uint2 *>(lds + (size_t)kWaves * RPW * TW) + wave * 3 * kWave;  // [3][64] (offset, value)
    for (int i = lane; i < RPW * TW; i += kWave) acc[i] = 0.f;
    // window each wavefront of the workgroup is in (pacing, below)
    int *progress = reinterpret_cast<int *>(reinterpret_cast<uint2 *>(lds + (size_t)kWaves * RPW * TW) + kWaves * 3 * kWave);
    if (lane == 0) progress[wave] = 0;
    __syncthreads();

    const int slot0 = (group * kWaves + wave) * RPW;
    const int stream = (range * kHubGroups + group) * kWaves + wave;
    const int64_t sbase = p.stream_first[stream];
    const int total = p.stream_total[stream];
    const int nb = (total + kWave - 1) / kWave;  // batches
    const char *__restrict__ Hb = static_cast<const char *>(p.H);
    const uint32_t row_bytes = (uint32_t)(p.ldh * (int64_t)sizeof(T));
    const uint32_t lane_off = (uint32_t)off * (uint32_t)sizeof(T);

    if (nb > 0) {
        struct Listed { int pos, run; };
        struct Read { int c, run; float v; };
        struct Ready { int run; uint64_t starts; int left; const uint2 *mine; };
        auto list = [&](int k) {
            const int64_t at = sbase + (int64_t)min(k, nb - 1) * kWave + lane;
            Listed x;
            x.pos = p.stream_pos[at];
            x.run = p.stream_run[at];
            return x;
        };
        auto read = [&](const Listed &x) {
            Read y;
            y.c = p.col[x.pos];
            y.v = p.val[x.pos];
            y.run = x.run;
            return y;
        };
        int carry = -1;  // slot of the last entry this lane's group had in the batch before: where the group stands
        auto ready = [&](const Read &y, int k, int slot) {
            Ready z;
            uint2 *dst = ring + slot * kWave;
            dst[lane] = make_uint2((uint32_t)y.c * row_bytes, __float_as_uint(y.v));
            int before = __shfl_up(y.run, 1, kWave);
            if (lane % STEPS == 0) before = carry;
            z.left = min(max(total - k * kWave, 0), kWave);
            z.starts = __ballot(y.run != before && lane < z.left);
            carry = __shfl(y.run, grp * STEPS + STEPS - 1, kWave);
            z.run = y.run;
            z.mine = dst + grp * STEPS;
            plx::wave_lds_fence();
            return z;
        };
        struct Rows { RawVec<T, VEC> h[U]; float v[U]; };
        auto fetch = [&](const Ready &z, int g, Rows &r) {
#pragma unroll
            for (int u = 0; u < U; u += 2) {
                const uint4 e = *reinterpret_cast<const uint4 *>(z.mine + g * U + u);  // two entries of this group
                r.v[u] = __uint_as_float(e.y);
                r.v[u + 1] = __uint_as_float(e.w);
                r.h[u].load(Hb + (e.x + lane_off));
                r.h[u + 1].load(Hb + (e.z + lane_off));
            }
        };
        int cur = -1;  // the slot this group is summing
        float sum[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) sum[k] = 0.f;
        // Products are summed in registers while the slot stays the same and added to the slot's sum in LDS when it
        // changes; several groups may hold the same slot, so they add to LDS one after the other.
        auto flush = [&](int run) {
            if (cur >= 0) {
#pragma unroll
                for (int k = 0; k < VEC; k += 4) {
                    float4 t = *reinterpret_cast<float4 *>(acc + cur * TW + dl + k);
                    t.x += sum[k];
                    t.y += sum[k + 1];
                    t.z += sum[k + 2];
                    t.w += sum[k + 3];
                    *reinterpret_cast<float4 *>(acc + cur * TW + dl + k) = t;
                }
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum[k] = 0.f;
            cur = run;
        };
        uint64_t every_group = 0;  // bit g * STEPS for every group g
#pragma unroll
        for (int g = 0; g < G; ++g) every_group |= 1ull << (g * STEPS);
        auto consume = [&](const Ready &z, int s, const Rows &r, auto checked) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = s * U + u;
                if ((z.starts >> i) & every_group) {
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        if ((z.starts >> (g * STEPS + i)) & 1) {
                            const int run = __builtin_amdgcn_readlane(z.run, g * STEPS + i);
                            if (grp == g) flush(run);
                            plx::wave_lds_fence();
                        }
                    }
                }
                if (!decltype(checked)::value || grp * STEPS + i < z.left) {
                    float hv[VEC];
                    r.h[u].widen(hv);
#pragma unroll
                    for (int k = 0; k < VEC; ++k) sum[k] = fmaf(r.v[u], hv[k], sum[k]);
                }
            }
        };
        auto add_up = [&](const Ready &z, int s, const Rows &r) {
            if (z.left == kWave) consume(z, s, r, std::false_type{});
            else consume(z, s, r, std::true_type{});
        };

        Rows ra, rb;
        Listed l0 = list(0), l1 = list(1), l2 = list(2);
        Read r0 = read(l0), r1 = read(l1);
        int s_now = 0, s_next = 1, s_free = 2;
        Ready now = ready(r0, 0, s_now), next = ready(r1, 1, s_next);
        Read rd = read(l2);
        Listed li = list(3);
        fetch(now, 0, ra);
        // Pacing: the rows of H of a window stay in L2 only while the wavefronts that share them are in the same few
        // windows.  Left alone they drift apart by the random walk of their entry counts; here a wavefront that enters a
        // window waits until the slowest wavefront of its workgroup is at most `pace` windows behind.  The wait reads
        // LDS only, ends when the others move on (they never wait for a wavefront ahead of them, and a wavefront that has
        // finished counts as far ahead), and is cut off after a fixed number of polls whatever happens.
        const int32_t *marks = p.stream_mark + (int64_t)stream * p.windows_per_range;
        int w_next = 1;
        int mark_next = p.pace >= 0 && w_next < p.windows_per_range ? marks[w_next] : 0x7fffffff;
        for (int k = 0; k < nb; ++k) {
            if (k >= mark_next) {
                while (w_next < p.windows_per_range && k >= mark_next) {
                    ++w_next;
                    mark_next = w_next < p.windows_per_range ? marks[w_next] : 0x7fffffff;
                }
                const int here = w_next - 1;
                if (lane == 0) __hip_atomic_store(&progress[wave], here, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                for (int polls = 0; polls < kHubMaxPolls; ++polls) {
                    int slowest = 0x7fffffff;
#pragma unroll
                    for (int x = 0; x < kWaves; ++x)
                        slowest = min(slowest, __hip_atomic_load(&progress[x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
                    if (slowest >= here - p.pace) break;
                    __builtin_amdgcn_s_sleep(8);
                }
            }
            const Ready after = ready(rd, k + 2, s_free);
            rd = read(li);
            li = list(k + 4);
            if constexpr (SETS == 4) {
                fetch(now, 1, rb);
                add_up(now, 0, ra);
                fetch(now, 2, ra);
                add_up(now, 1, rb);
                fetch(now, 3, rb);
                add_up(now, 2, ra);
                fetch(next, 0, ra);
                add_up(now, 3, rb);
            } else {
                fetch(now, 1, rb);
                add_up(now, 0, ra);
                fetch(next, 0, ra);
                add_up(now, 1, rb);
            }
            now = next;
            next = after;
            const int t = s_now;
            s_now = s_next;
            s_next = s_free;
            s_free = t;
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (grp == g) flush(-1);
            plx::wave_lds_fence();
        }
    }

    if (lane == 0) __hip_atomic_store(&progress[wave], 0x7fffffff, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);  // done: nobody waits for this wavefront

    // the sums of this range: P[range][slot][ldp]
    if (grp == 0 && ok) {
        for (int r = 0; r < RPW; ++r) {
            if (p.hub_row[slot0 + r] < 0) continue;
            float *dst = p.partial + ((int64_t)range * p.slot_cap + slot0 + r) * p.ldp + blockIdx.y * TW + dl;
#pragma unroll
            for (int k = 0; k < VEC; ++k)
                if (blockIdx.y * TW + dl + k < p.D) dst[k] = acc[r * TW + dl + k];
        }
    }
}

// Y[hub row] = sum of the partial sums of the row's slots (its parts, in order) over the ranges (in range order).
// A workgroup owns a hub row: 8 chains x 32 lanes, each lane a float4.  Chain c adds partial sums c, c + 8, ... of
// the (slot, range) list in order; the 8 chain sums are then added in chain order, so the summation order is fixed.
template <typename TOUT>
__global__ void __launch_bounds__(256) spmm_hub_reduce_kernel(const HubArgs p, TOUT *__restrict__ Y, int64_t ldy)
{
    __shared__ float4 part[8][32];
    const int q = blockIdx.x;
    const int row = p.rows[q];
    if (row < p.row_begin || row >= p.row_end) return;
    const int s0 = p.row_slot_first[q], n = (p.row_slot_first[q + 1] - s0) * kHubRanges;
    const int chain = threadIdx.x >> 5, l = threadIdx.x & 31;
    for (int d0 = 0; d0 < p.D; d0 += kHubTile) {
        const int d = d0 + l * 4;  // ldp is a multiple of kHubTile (128 or 256): the float4 at d lies inside the padded partial row
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        auto at = [&](int j) {
            const int slot = p.row_slots[s0 + j / kHubRanges], x = j % kHubRanges;
            return *reinterpret_cast<const float4 *>(p.partial + ((int64_t)x * p.slot_cap + slot) * p.ldp + d);
        };
        auto add = [&](const float4 &t) {
            acc.x += t.x;
            acc.y += t.y;
            acc.z += t.z;
            acc.w += t.w;
        };
        int j = chain;
        for (; j + 24 < n; j += 32) {  // four loads in flight, added in the order of the list
            const float4 t0 = at(j), t1 = at(j + 8), t2 = at(j + 16), t3 = at(j + 24);
            add(t0);
            add(t1);
            add(t2);
            add(t3);
        }
        for (; j < n; j += 8) add(at(j));
        __syncthreads();  // the chain sums of the tile before have been read
        part[chain][l] = acc;
        __syncthreads();
        if (chain == 0) {
            float4 s = part[0][l];
#pragma unroll
            for (int c = 1; c < 8; ++c) {
                s.x += part[c][l].x;
                s.y += part[c][l].y;
                s.z += part[c][l].z;
                s.w += part[c][l].w;
            }
            const float v[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (d + e >= p.D) break;
                if constexpr (sizeof(TOUT) == 4) {
                    Y[(int64_t)row * ldy + d + e] = v[e];
                } else {
                    uint32_t u = __float_as_uint(v[e]);
                    if ((u & 0x7fffffffu) > 0x7f800000u) u = (u >> 16) | 0x40u;
                    else u = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
                    Y[(int64_t)row * ldy + d + e] = (uint16_t)u;
                }
            }
        }
    }
}

// ---- construction of the streams ----
struct BuildArgs {
    const int32_t *rowptr;
    const int32_t *col;
    const int32_t *hub_row;   // [slot cap]
    const int32_t *hub_part;  // [slot cap] part | parts << 16
    int32_t window, windows_per_range, n_windows;
    int32_t rows_per_wave;    // slots of a wavefront (at most 64: one lane follows one slot)
    const int64_t *stream_first;  // fill
    int32_t *stream_total;        // count
    int32_t *stream_pos;          // fill
    uint8_t *stream_run;          // fill
    int32_t *stream_mark;         // fill
};

// One wavefront per stream.  Lane l follows slot l of the wavefront through the windows of the range: the entries of
// the slot's row inside a window (found by bisection over the row's sorted columns) and the slot's share of them.
// FILL = false adds up the stream's length; FILL = true writes the stream: the runs of a window one after the other,
// 64 entries per step (entry f of the window belongs to the last slot whose exclusive prefix of run lengths is <= f).
template <bool FILL>
__global__ void __launch_bounds__(64) hub_streams_kernel(const BuildArgs b)
{
    __shared__ int prefix[kWave];
    __shared__ int delta[kWave];
    const int lane = threadIdx.x;
    const int stream = blockIdx.x;
    const int wave = stream % kWaves, group = (stream / kWaves) % kHubGroups, range = stream / (kWaves * kHubGroups);
    const int slot = (group * kWaves + wave) * b.rows_per_wave + min(lane, b.rows_per_wave - 1);
    const int row = lane < b.rows_per_wave ? b.hub_row[slot] : -1;
    int lo_pos = 0, end_pos = 0, part = 0, parts = 1;
    if (row >= 0) {
        lo_pos = b.rowptr[row];
        end_pos = b.rowptr[row + 1];
        part = b.hub_part[slot] & 0xffff;
        parts = b.hub_part[slot] >> 16;
    }
    auto first_at_least = [&](int from, int64_t target) {  // first position in [from, end_pos] whose column is >= target
        int lo = from, hi = end_pos;
        while (lo < hi) {
            const int mid = lo + ((hi - lo) >> 1);
            if ((int64_t)b.col[mid] < target) lo = mid + 1; else hi = mid;
        }
        return lo;
    };
    const int w_begin = range * b.windows_per_range, w_end = min(w_begin + b.windows_per_range, b.n_windows);
    int p0 = row >= 0 ? first_at_least(lo_pos, (int64_t)w_begin * b.window) : 0;
    int64_t length = 0;  // of this lane's runs (count) / of the stream so far (fill)
    const int64_t base = FILL ? b.stream_first[stream] : 0;
    for (int w = w_begin; w < w_end; ++w) {
        int p1 = p0;
        if (row >= 0) p1 = w + 1 == b.n_windows ? end_pos : first_at_least(p0, (int64_t)(w + 1) * b.window);
        const int64_t n_all = p1 - p0;
        const int begin = p0 + (int)(n_all * part / parts), end = p0 + (int)(n_all * (part + 1) / parts);
        p0 = p1;
        const int n = row >= 0 ? end - begin : 0;
        if constexpr (!FILL) {
            length += n;
        } else {
            if (lane == 0) b.stream_mark[(int64_t)stream * b.windows_per_range + (w - w_begin)] = (int32_t)(length / kWave);
            int incl = n;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const int t = __shfl_up(incl, o, kWave);
                if (lane >= o) incl += t;
            }
            const int total = __shfl(incl, kWave - 1, kWave);
            __syncthreads();
            prefix[lane] = incl - n;
            delta[lane] = begin - (incl - n);
            __syncthreads();
            for (int f = lane; f < total; f += kWave) {
                int lo = 0, hi = b.rows_per_wave;  // prefix[lo] <= f < prefix[hi] (prefix[rows_per_wave ..] = total)
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (prefix[mid] <= f) lo = mid; else hi = mid;
                }
                b.stream_pos[base + length + f] = f + delta[lo];
                b.stream_run[base + length + f] = (uint8_t)lo;
            }
            length += total;
        }
    }
    if constexpr (!FILL) {
        int64_t sum = length;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
        if (lane == 0) b.stream_total[stream] = (int32_t)sum;
    } else {
        for (int w = w_end - w_begin + lane; w < b.windows_per_range; w += kWave) b.stream_mark[(int64_t)stream * b.windows_per_range + w] = 0x7fffffff;
        // padding up to a whole batch: a valid position (entry 0 of the matrix), a slot number no wavefront has
        const int64_t padded = (length + kWave - 1) / kWave * kWave;
        for (int64_t f = length + lane; f < padded; f += kWave) {
            b.stream_pos[base + f] = 0;
            b.stream_run[base + f] = 255;
        }
    }
}

// flags of the hub rows among the split rows of the plan and of their segments; one workgroup per hub row
__global__ void __launch_bounds__(64) hub_flags_kernel(int32_t n_long, const int32_t *__restrict__ long_rows, const int32_t *__restrict__ seg_first,
                                                       const int32_t *__restrict__ rows, uint8_t *__restrict__ long_is_hub,
                                                       uint8_t *__restrict__ seg_is_hub)
{
    const int32_t row = rows[blockIdx.x];
    int lo = 0, hi = n_long;  // position of the row among the split rows (it is one of them)
    while (lo < hi) {
        const int mid = lo + ((hi - lo) >> 1);
        if (long_rows[mid] < row) lo = mid + 1; else hi = mid;
    }
    if (threadIdx.x == 0) long_is_hub[lo] = 1;
    for (int s = seg_first[lo] + threadIdx.x; s < seg_first[lo + 1]; s += blockDim.x) seg_is_hub[s] = 1;
}

__global__ void __launch_bounds__(256) row_lengths_kernel(int64_t n, const int32_t *__restrict__ rowptr, const int32_t *__restrict__ rows,
                                                          int32_t *__restrict__ len)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) len[i] = rowptr[rows[i] + 1] - rowptr[rows[i]];
}

// The streams are cut out of a row by bisection over its columns, so the columns of a hub row must ascend (equal
// neighbours are harmless).  One workgroup per split row; *unsorted receives the number of rows that do not comply.
__global__ void __launch_bounds__(256) rows_ascend_kernel(const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col,
                                                          const int32_t *__restrict__ rows, int32_t *__restrict__ unsorted)
{
    __shared__ int bad;
    if (threadIdx.x == 0) bad = 0;
    __syncthreads();
    const int32_t r = rows[blockIdx.x];
    const int32_t a = rowptr[r], b = rowptr[r + 1];
    int mine = 0;
    for (int32_t i = a + 1 + (int32_t)threadIdx.x; i < b; i += (int32_t)blockDim.x) mine |= col[i] < col[i - 1] ? 1 : 0;
    if (mine) bad = 1;  // every writer stores the same value
    __syncthreads();
    if (threadIdx.x == 0 && bad) atomicAdd(unsorted, 1);
}

struct DeviceBlock {  // freed on every way out
    void *p = nullptr;
    ~DeviceBlock()
    {
        if (p) (void)hipFree(p);
    }
};

template <typename T, int VEC, int LPR, int RPW = kHubRowsPerWave>
int launch_t(const HubArgs &a, void *Y, int64_t ldy, hipStream_t st, bool run_pass, bool run_reduce)
{
    constexpr int TW = LPR * VEC;
    const size_t shm = ((size_t)kWaves * RPW * TW) * sizeof(float) + (size_t)kWaves * 3 * kWave * sizeof(uint2) + kWaves * sizeof(int);
    static_assert(((size_t)kWaves * RPW * TW) * sizeof(float) + (size_t)kWaves * 3 * kWave * sizeof(uint2) + kWaves * sizeof(int) <= 160 * 1024,
                  "the sums of a workgroup, its rings and its progress words fit the LDS of a compute unit");
    static std::atomic<uint64_t> allowed{0};  // devices on which this instantiation may take its LDS
    const int rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&spmm_hub_kernel<T, VEC, LPR, RPW>), shm, allowed);
    if (rc != PLX_OK) return rc;
    dim3 grid(kHubRanges * kHubGroups, (unsigned)plx::ceil_div(a.D, TW), 1);
    if (run_pass) {
        spmm_hub_kernel<T, VEC, LPR, RPW><<<grid, kThreads, shm, st>>>(a);
        PLX_LAUNCH_CHECK("spmm_hub_kernel");
    }
    if (run_reduce) {
        spmm_hub_reduce_kernel<T><<<(unsigned)a.n_rows, 256, 0, st>>>(a, static_cast<T *>(Y), ldy);
        PLX_LAUNCH_CHECK("spmm_hub_reduce_kernel");
    }
    return PLX_OK;
}

}  // namespace

namespace plx {
namespace hub {

size_t partial_bytes(int64_t D, bool wide)
{
    const int64_t tile = wide ? kHubTileWide : kHubTile, slots = (int64_t)kHubGroups * kWaves * (wide ? kHubRowsPerWaveWide : kHubRowsPerWave);
    return (size_t)kHubRanges * (size_t)slots * (size_t)(ceil_div(D, tile) * tile) * sizeof(float);
}

void free_hub_plan(HubPlan &hp)
{
    if (hp.block) (void)hipFree(hp.block);
    hp = HubPlan();
}

int build_hub_plan(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, int32_t seg_len, int64_t n_long,
                   int64_t n_seg, const int32_t *long_rows, const int32_t *seg_first, const std::vector<int32_t> &h_long_rows,
                   int64_t min_entries, bool wide, hipStream_t st, HubPlan &out)
{
    (void)M;
    out = HubPlan();
    const int rows_per_wave = wide ? kHubRowsPerWaveWide : kHubRowsPerWave;
    const int slot_cap = kHubGroups * kWaves * rows_per_wave;
    if (n_long <= 0 || K <= 0 || nnz <= 0) return PLX_OK;

    // lengths of the split rows, and whether their columns ascend, to the host
    std::vector<int32_t> len((size_t)n_long + 1);
    {
        DeviceBlock d_len;
        PLX_HIP_CHECK(hipMalloc(&d_len.p, sizeof(int32_t) * ((size_t)n_long + 1)));
        int32_t *d = static_cast<int32_t *>(d_len.p);
        PLX_HIP_CHECK(hipMemsetAsync(d + n_long, 0, sizeof(int32_t), st));
        row_lengths_kernel<<<(unsigned)ceil_div(n_long, 256), 256, 0, st>>>(n_long, rowptr, long_rows, d);
        PLX_LAUNCH_CHECK("row_lengths_kernel");
        rows_ascend_kernel<<<(unsigned)n_long, 256, 0, st>>>(rowptr, col, long_rows, d + n_long);
        PLX_LAUNCH_CHECK("rows_ascend_kernel");
        PLX_HIP_CHECK(hipMemcpyAsync(len.data(), d_len.p, sizeof(int32_t) * ((size_t)n_long + 1), hipMemcpyDeviceToHost, st));
        PLX_HIP_CHECK(hipStreamSynchronize(st));
    }
    if (len[(size_t)n_long] != 0)
        return plx::fail(PLX_ERR_UNSUPPORTED, "hub plan: the columns of %d of the %lld split rows do not ascend; the hub pass needs them sorted "
                         "within each row (the products without it do not)", len[(size_t)n_long], (long long)n_long);
    len.pop_back();
    // longest first (ties: lower row first); a row takes ceil(len / part_len) slots, rows are taken while slots last
    std::vector<int32_t> order((size_t)n_long);
    std::iota(order.begin(), order.end(), 0);
    const size_t keep = std::min<size_t>((size_t)n_long, (size_t)slot_cap);
    auto longer = [&](int32_t x, int32_t y) { return len[(size_t)x] != len[(size_t)y] ? len[(size_t)x] > len[(size_t)y] : x < y; };
    std::partial_sort(order.begin(), order.begin() + (ptrdiff_t)keep, order.end(), longer);
    const int64_t part_len = (int64_t)seg_len * (wide ? kHubPartFactorWide : kHubPartFactor);
    struct Slot { int32_t row, part, parts, q; int64_t size; };
    std::vector<Slot> slots;
    std::vector<int32_t> rows, row_slot_first{0};
    int64_t entries = 0;
    for (size_t i = 0; i < keep; ++i) {
        const int32_t q = order[i];
        const int64_t l = len[(size_t)q];
        const int64_t parts = ceil_div(l, part_len);
        if ((int64_t)slots.size() + parts > slot_cap) continue;  // a shorter row may still fit
        for (int64_t s = 0; s < parts; ++s) slots.push_back(Slot{h_long_rows[(size_t)q], (int32_t)s, (int32_t)parts, (int32_t)rows.size(), l / parts});
        rows.push_back(h_long_rows[(size_t)q]);
        row_slot_first.push_back((int32_t)slots.size());
        entries += l;
    }
    if (rows.empty() || entries < min_entries) return PLX_OK;
    // The slots go to the wavefronts largest first, each to the wavefront with the fewest entries so far that still has
    // room: wavefronts with equal loads pass through the windows side by side, which is what keeps a window's rows of H
    // in L2 while they are shared (a wavefront 5 % short of the others ends the pass four windows ahead of them).
    std::vector<int32_t> by_size(slots.size());
    std::iota(by_size.begin(), by_size.end(), 0);
    std::stable_sort(by_size.begin(), by_size.end(), [&](int32_t x, int32_t y) { return slots[(size_t)x].size > slots[(size_t)y].size; });
    std::vector<int32_t> hub_row((size_t)slot_cap, -1), hub_part((size_t)slot_cap, 1 << 16), row_slots(slots.size());
    {
        constexpr int kBins = kHubGroups * kWaves;
        using Bin = std::pair<int64_t, int32_t>;  // (entries, wavefront): the least loaded first, ties by number
        std::priority_queue<Bin, std::vector<Bin>, std::greater<Bin>> bins;
        // numbered so that consecutive wavefronts lie in different workgroups: few slots then spread over the chip
        for (int32_t b = 0; b < kBins; ++b) bins.push(Bin{0, b});
        std::vector<int32_t> held((size_t)kBins, 0);
        for (size_t k = 0; k < by_size.size(); ++k) {
            const Slot &sl = slots[(size_t)by_size[k]];
            Bin bin = bins.top();
            bins.pop();
            const int32_t b = bin.second, group = b % kHubGroups, wave = b / kHubGroups;
            const int32_t id = (group * kWaves + wave) * rows_per_wave + held[(size_t)b];
            hub_row[(size_t)id] = sl.row;
            hub_part[(size_t)id] = sl.part | (sl.parts << 16);
            row_slots[(size_t)row_slot_first[(size_t)sl.q] + (size_t)sl.part] = id;
            bin.first += sl.size;
            if (++held[(size_t)b] < rows_per_wave) bins.push(bin);
        }
    }

    const int32_t window = kHubWindow;
    const int32_t wpr = (int32_t)ceil_div(ceil_div(K, kHubRanges), window);
    const int32_t n_windows = wpr * kHubRanges;
    if (wpr > kHubMaxWindows) return PLX_OK;  // beyond 134 M columns the per-window tables outgrow their use: no hub pass

    // the small tables and the stream lengths
    const size_t n_rows = rows.size(), n_slots = slots.size();
    auto up16 = [](size_t x) { return (x + 15) / 16 * 16; };
    const size_t o_hub_row = 0, o_hub_part = o_hub_row + up16(sizeof(int32_t) * slot_cap), o_rows = o_hub_part + up16(sizeof(int32_t) * slot_cap),
                 o_rsf = o_rows + up16(sizeof(int32_t) * n_rows), o_rs = o_rsf + up16(sizeof(int32_t) * (n_rows + 1)),
                 o_first = o_rs + up16(sizeof(int32_t) * n_slots), o_total = o_first + up16(sizeof(int64_t) * kHubStreams),
                 o_mark = o_total + up16(sizeof(int32_t) * kHubStreams), o_lflag = o_mark + up16(sizeof(int32_t) * (size_t)kHubStreams * (size_t)wpr),
                 o_sflag = o_lflag + up16((size_t)n_long),
                 small_bytes = o_sflag + up16((size_t)n_seg);
    DeviceBlock small;
    PLX_HIP_CHECK(hipMalloc(&small.p, small_bytes));
    char *sb = static_cast<char *>(small.p);
    PLX_HIP_CHECK(hipMemcpyAsync(sb + o_hub_row, hub_row.data(), sizeof(int32_t) * slot_cap, hipMemcpyHostToDevice, st));
    PLX_HIP_CHECK(hipMemcpyAsync(sb + o_hub_part, hub_part.data(), sizeof(int32_t) * slot_cap, hipMemcpyHostToDevice, st));
    BuildArgs b{};
    b.rowptr = rowptr;
    b.col = col;
    b.hub_row = reinterpret_cast<const int32_t *>(sb + o_hub_row);
    b.hub_part = reinterpret_cast<const int32_t *>(sb + o_hub_part);
    b.window = window;
    b.windows_per_range = wpr;
    b.n_windows = n_windows;
    b.rows_per_wave = rows_per_wave;
    b.stream_total = reinterpret_cast<int32_t *>(sb + o_total);
    hub_streams_kernel<false><<<kHubStreams, 64, 0, st>>>(b);
    PLX_LAUNCH_CHECK("hub_streams_kernel (count)");
    std::vector<int32_t> totals((size_t)kHubStreams);
    PLX_HIP_CHECK(hipMemcpyAsync(totals.data(), sb + o_total, sizeof(int32_t) * kHubStreams, hipMemcpyDeviceToHost, st));
    PLX_HIP_CHECK(hipStreamSynchronize(st));
    std::vector<int64_t> first((size_t)kHubStreams);
    int64_t stored = 0, counted = 0;
    for (int i = 0; i < kHubStreams; ++i) {
        first[(size_t)i] = stored;
        stored += ceil_div(totals[(size_t)i], kWave) * kWave;
        counted += totals[(size_t)i];
    }
    PLX_REQUIRE(counted == entries, "hub plan: the streams hold %lld entries, the hub rows %lld", (long long)counted, (long long)entries);

    // everything in one block: the small tables, then the streams
    const size_t o_pos = up16(small_bytes), o_run = o_pos + up16(sizeof(int32_t) * (size_t)stored), bytes = o_run + up16((size_t)stored);
    DeviceBlock block;
    hipError_t e = hipMalloc(&block.p, bytes);
    if (e != hipSuccess) return plx::fail(PLX_ERR_NOMEM, "hub plan: hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    char *bb = static_cast<char *>(block.p);
    PLX_HIP_CHECK(hipMemcpyAsync(bb, sb, o_rows, hipMemcpyDeviceToDevice, st));  // hub_row, hub_part
    PLX_HIP_CHECK(hipMemcpyAsync(bb + o_rows, rows.data(), sizeof(int32_t) * n_rows, hipMemcpyHostToDevice, st));
    PLX_HIP_CHECK(hipMemcpyAsync(bb + o_rsf, row_slot_first.data(), sizeof(int32_t) * (n_rows + 1), hipMemcpyHostToDevice, st));
    PLX_HIP_CHECK(hipMemcpyAsync(bb + o_rs, row_slots.data(), sizeof(int32_t) * n_slots, hipMemcpyHostToDevice, st));
    PLX_HIP_CHECK(hipMemcpyAsync(bb + o_first, first.data(), sizeof(int64_t) * kHubStreams, hipMemcpyHostToDevice, st));
    PLX_HIP_CHECK(hipMemcpyAsync(bb + o_total, totals.data(), sizeof(int32_t) * kHubStreams, hipMemcpyHostToDevice, st));
    PLX_HIP_CHECK(hipMemsetAsync(bb + o_lflag, 0, o_pos - o_lflag, st));
    b.hub_row = reinterpret_cast<const int32_t *>(bb + o_hub_row);
    b.hub_part = reinterpret_cast<const int32_t *>(bb + o_hub_part);
    b.stream_first = reinterpret_cast<const int64_t *>(bb + o_first);
    b.stream_total = nullptr;
    b.stream_pos = reinterpret_cast<int32_t *>(bb + o_pos);
    b.stream_run = reinterpret_cast<uint8_t *>(bb + o_run);
    b.stream_mark = reinterpret_cast<int32_t *>(bb + o_mark);
    hub_streams_kernel<true><<<kHubStreams, 64, 0, st>>>(b);
    PLX_LAUNCH_CHECK("hub_streams_kernel (fill)");
    hub_flags_kernel<<<(unsigned)n_rows, 64, 0, st>>>((int32_t)n_long, long_rows, seg_first, reinterpret_cast<const int32_t *>(bb + o_rows),
                                                      reinterpret_cast<uint8_t *>(bb + o_lflag), reinterpret_cast<uint8_t *>(bb + o_sflag));
    PLX_LAUNCH_CHECK("hub_flags_kernel");
    PLX_HIP_CHECK(hipStreamSynchronize(st));  // the host vectors above are read by the copies

    out.n_rows = (int32_t)n_rows;
    out.n_slots = (int32_t)n_slots;
    out.entries = entries;
    out.mean_run = (double)entries / ((double)n_slots * (double)n_windows);
    out.stored = stored;
    out.window = window;
    out.n_windows = n_windows;
    out.windows_per_range = wpr;
    out.rows_per_wave = rows_per_wave;
    out.slot_cap = slot_cap;
    out.block = block.p;
    block.p = nullptr;
    out.hub_row = reinterpret_cast<const int32_t *>(bb + o_hub_row);
    out.rows = reinterpret_cast<const int32_t *>(bb + o_rows);
    out.row_slot_first = reinterpret_cast<const int32_t *>(bb + o_rsf);
    out.row_slots = reinterpret_cast<const int32_t *>(bb + o_rs);
    out.stream_first = reinterpret_cast<const int64_t *>(bb + o_first);
    out.stream_total = reinterpret_cast<const int32_t *>(bb + o_total);
    out.stream_pos = reinterpret_cast<const int32_t *>(bb + o_pos);
    out.stream_run = reinterpret_cast<const uint8_t *>(bb + o_run);
    out.stream_mark = reinterpret_cast<const int32_t *>(bb + o_mark);
    out.long_is_hub = reinterpret_cast<const uint8_t *>(bb + o_lflag);
    out.seg_is_hub = reinterpret_cast<const uint8_t *>(bb + o_sflag);
    out.h_rows_sorted = rows;
    std::sort(out.h_rows_sorted.begin(), out.h_rows_sorted.end());
    return PLX_OK;
}

int launch(const HubPlan &hp, const int32_t *col, const float *val, const void *H, int64_t ldh, int64_t D, int64_t d_read, bool bf16,
           int64_t row_begin, int64_t row_end, void *Y, int64_t ldy, float *partial, hipStream_t st, bool run_pass, bool run_reduce)
{
    PLX_REQUIRE(hp.block != nullptr && partial != nullptr, "hub pass: no tables or no room for the partial sums");
    PLX_REQUIRE(d_read % kHubVec == 0 && d_read <= ldh, "hub pass: readable width %lld", (long long)d_read);
    HubArgs a{};
    a.col = col;
    a.val = val;
    a.H = H;
    a.ldh = ldh;
    a.D = (int32_t)D;
    a.d_read = (int32_t)d_read;
    a.hub_row = hp.hub_row;
    a.stream_first = hp.stream_first;
    a.stream_total = hp.stream_total;
    a.stream_pos = hp.stream_pos;
    a.stream_run = hp.stream_run;
    a.stream_mark = hp.stream_mark;
    a.windows_per_range = hp.windows_per_range;
    a.pace = kHubPace;
    a.n_rows = hp.n_rows;
    a.rows = hp.rows;
    a.row_slot_first = hp.row_slot_first;
    a.row_slots = hp.row_slots;
    a.row_begin = (int32_t)row_begin;
    a.row_end = (int32_t)row_end;
    a.partial = partial;
    a.slot_cap = hp.slot_cap;
    if (hp.rows_per_wave == kHubRowsPerWaveWide) {
        // bf16 rows of 512 bytes and more: half a wavefront reads 256 columns, 16 bytes per lane, in one tile (in 128-column
        // tiles every stream, column index and value is read once per tile and a load carries 8 bytes per lane)
        PLX_REQUIRE(bf16 && d_read % 8 == 0, "hub pass: the wide layout takes bf16 rows in multiples of 8 columns");
        a.ldp = ceil_div(D, kHubTileWide) * kHubTileWide;
        return launch_t<uint16_t, 8, 32, kHubRowsPerWaveWide>(a, Y, ldy, st, run_pass, run_reduce);
    }
    a.ldp = ceil_div(D, kHubTile) * kHubTile;  // every kernel's tile divides kHubTile
    // fp32 rows of at most 256 bytes are read by a quarter of a wavefront, four entries per load instruction
    // (bf16 rows read 16 bytes per lane by a quarter of a wavefront were measured too: no faster than 8 bytes by a half)
    if (!bf16) return D <= 64 ? launch_t<float, 4, 16>(a, Y, ldy, st, run_pass, run_reduce) : launch_t<float, 4, 32>(a, Y, ldy, st, run_pass, run_reduce);
    return launch_t<uint16_t, 4, 32>(a, Y, ldy, st, run_pass, run_reduce);
}

}  // namespace hub
}  // namespace plx
