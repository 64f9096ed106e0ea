// CSR SpMM  Y = A . H  for gfx950.
//
// Work decomposition (no atomics, fixed summation order):
//   * one 64-lane wavefront per task; a task is either a whole row of A (rows of at most
//     seg_len non-zeros) or one segment of a longer row;
//   * segment tasks come first in the grid (they are the longest) and write fp32 partial rows to a
//     workspace; a second small kernel adds the partial rows of each split row in segment order;
//   * inside a task the 64 lanes are cut into G = 64 / LPR groups of LPR lanes.  A group covers
//     one row of H with VEC-element (up to 128-bit) loads per lane, so one gather instruction of
//     the wavefront pulls G rows of H.  Group g handles non-zeros g, g+G, g+2G, ... of the task;
//     the G partial sums are combined with cross-lane shuffles at the end;
//   * column indices and values are read 64 at a time, one per lane (coalesced), and handed to the
//     groups through cross-lane permutes, so no lane re-reads them from memory;
//   * for rows of H wider than 64 lanes x VEC, each lane keeps NACC accumulator vectors; rows wider
//     than that are tiled over gridDim.y.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <mutex>
#include <vector>

#include "common.h"
#include "plan_build.h"
#include "spmm_hub.h"
#include "plexus_hip_diag.h"

// Scratch of plx_spmm_csr_f32_static: fp32 partial rows of the split rows.  Every GPU the library runs on holds its own
// copy of this array, at its own address, until the process ends.
constexpr size_t kStaticScratchBytes = PLX_SPMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

using plx::kWave;

struct SpmmArgs {
    const int32_t *rowptr;
    const int32_t *col;
    const float *val;
    const void *H;
    void *Y;
    float *ws;
    const int32_t *seg_begin;
    const int32_t *seg_end;
    int64_t ldh;
    int64_t ldy;
    int64_t ldws;
    int32_t M;         // rows are [row_begin, row_end)
    int32_t n_seg;     // segment tasks of this launch
    int32_t D;
    int32_t seg_len;
    int32_t row_begin;
    int32_t row_end;
    int32_t seg_base;  // index of the first segment task in the plan's tables
    int32_t y_vec;     // 1: rows of Y take VEC-wide stores; 0: element stores, each guarded by the width D
    const uint8_t *seg_skip;  // flags over the plan's segments: tasks left to the hub pass (or NULL)
};

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;  // quiet the NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                  // round to nearest even
    return u >> 16;
}

// ---- VEC-element loads / stores, fp32 or bf16 storage, fp32 in registers ----
template <typename T, int VEC>
struct VecIO;

template <>
struct VecIO<float, 1> {
    static __device__ __forceinline__ void load(const float *p, float (&o)[1]) { o[0] = *p; }
    static __device__ __forceinline__ void store(float *p, const float (&v)[1]) { *p = v[0]; }
};
template <>
struct VecIO<float, 2> {
    static __device__ __forceinline__ void load(const float *p, float (&o)[2])
    {
        const float2 t = *reinterpret_cast<const float2 *>(p);
        o[0] = t.x;
        o[1] = t.y;
    }
    static __device__ __forceinline__ void store(float *p, const float (&v)[2])
    {
        *reinterpret_cast<float2 *>(p) = make_float2(v[0], v[1]);
    }
};
template <>
struct VecIO<float, 4> {
    static __device__ __forceinline__ void load(const float *p, float (&o)[4])
    {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        o[0] = t.x;
        o[1] = t.y;
        o[2] = t.z;
        o[3] = t.w;
    }
    static __device__ __forceinline__ void store(float *p, const float (&v)[4])
    {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <>
struct VecIO<uint16_t, 1> {
    static __device__ __forceinline__ void load(const uint16_t *p, float (&o)[1]) { o[0] = bf16_to_f32(*p); }
    static __device__ __forceinline__ void store(uint16_t *p, const float (&v)[1]) { *p = (uint16_t)f32_to_bf16(v[0]); }
};
template <>
struct VecIO<uint16_t, 2> {
    static __device__ __forceinline__ void load(const uint16_t *p, float (&o)[2])
    {
        const uint32_t t = *reinterpret_cast<const uint32_t *>(p);
        o[0] = __uint_as_float(t << 16);
        o[1] = __uint_as_float(t & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(uint16_t *p, const float (&v)[2])
    {
        *reinterpret_cast<uint32_t *>(p) = f32_to_bf16(v[0]) | (f32_to_bf16(v[1]) << 16);
    }
};
template <>
struct VecIO<uint16_t, 4> {
    static __device__ __forceinline__ void load(const uint16_t *p, float (&o)[4])
    {
        const uint2 t = *reinterpret_cast<const uint2 *>(p);
        o[0] = __uint_as_float(t.x << 16);
        o[1] = __uint_as_float(t.x & 0xffff0000u);
        o[2] = __uint_as_float(t.y << 16);
        o[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(uint16_t *p, const float (&v)[4])
    {
        uint2 t;
        t.x = f32_to_bf16(v[0]) | (f32_to_bf16(v[1]) << 16);
        t.y = f32_to_bf16(v[2]) | (f32_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2 *>(p) = t;
    }
};
template <>
struct VecIO<uint16_t, 8> {
    static __device__ __forceinline__ void load(const uint16_t *p, float (&o)[8])
    {
        const uint4 t = *reinterpret_cast<const uint4 *>(p);
        const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = __uint_as_float(w[i] << 16);
            o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(uint16_t *p, const float (&v)[8])
    {
        uint4 t;
        t.x = f32_to_bf16(v[0]) | (f32_to_bf16(v[1]) << 16);
        t.y = f32_to_bf16(v[2]) | (f32_to_bf16(v[3]) << 16);
        t.z = f32_to_bf16(v[4]) | (f32_to_bf16(v[5]) << 16);
        t.w = f32_to_bf16(v[6]) | (f32_to_bf16(v[7]) << 16);
        *reinterpret_cast<uint4 *>(p) = t;
    }
};

// fp32 store of a VEC-element register vector (the workspace is fp32 whatever the storage type)
template <int VEC>
__device__ __forceinline__ void store_f32(float *p, const float (&v)[VEC])
{
    if constexpr (VEC == 8) {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        VecIO<float, VEC>::store(p, v);
    }
}

__device__ __forceinline__ void store_elem(float *p, float v) { *p = v; }
__device__ __forceinline__ void store_elem(uint16_t *p, float v) { *p = (uint16_t)f32_to_bf16(v); }

// value of `x` held by lane `src`; `src` differs between lane groups when G > 1
template <int G>
__device__ __forceinline__ int pick_i(int x, int src)
{
    if constexpr (G == 1)
        return __builtin_amdgcn_readlane(x, src);
    else
        return __shfl(x, src, kWave);
}
template <int G>
__device__ __forceinline__ float pick_f(float x, int src)
{
    return __int_as_float(pick_i<G>(__float_as_int(x), src));
}

// R > 1: every lane group keeps R accumulator sets ("chains") and entry number q of a task (counted from the task's
// first entry) goes to chain q mod (G * R) -- group q mod G, set (q / G) mod R.  The chains are added pairwise in the
// order a kernel with G * R lane groups adds its groups, so the sum has the same bits as that kernel's.
template <typename TIN, typename TOUT, int VEC, int LPR, int NACC, int R = 1>
__global__ void __launch_bounds__(256) spmm_csr_kernel(const SpmmArgs p)
{
    constexpr int G = kWave / LPR;
    static_assert(G == 1 || NACC == 1, "several accumulator vectors only with one group");
    static_assert((R & (R - 1)) == 0 && R >= 1 && G * R <= kWave, "chains per group: a power of two");
    // gathers kept in flight per lane = U * NACC; U is a multiple of R so that the chain of a load is known statically
    constexpr int U0 = (G >= 8) ? 1 : (G == 4) ? 2 : (G == 2) ? 4 : (NACC <= 2 ? 4 : (NACC <= 4 ? 2 : 1));
    constexpr int U = U0 > R ? U0 : R;
    constexpr int TILE = LPR * VEC * NACC;

    const int lane = threadIdx.x & (kWave - 1);
    const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t task = (int64_t)blockIdx.x * 4 + wid;
    const int g = lane / LPR;
    const int t = lane % LPR;
    const int d0 = blockIdx.y * TILE;

    int a, b;
    bool to_ws;
    int64_t out_row;
    if (task < p.n_seg) {
        if (p.seg_skip != nullptr && p.seg_skip[p.seg_base + task]) return;
        a = p.seg_begin[p.seg_base + task];
        b = p.seg_end[p.seg_base + task];
        to_ws = true;
        out_row = p.seg_base + task;  // partial rows are indexed by the plan-wide segment number
    } else {
        const int64_t r = p.row_begin + (task - p.n_seg);
        if (r >= p.row_end) return;
        a = p.rowptr[r];
        b = p.rowptr[r + 1];
        if (b - a > p.seg_len) return;  // split row: its segments are separate tasks
        to_ws = false;
        out_row = r;
    }
    a = __builtin_amdgcn_readfirstlane(a);
    b = __builtin_amdgcn_readfirstlane(b);

    // element offsets of this lane's vectors inside a row of H; lanes past the row width
    // gather element 0 instead (a valid address) and never store
    int off[NACC];
    bool ok[NACC];
#pragma unroll
    for (int k = 0; k < NACC; ++k) {
        const int e = d0 + (t + k * LPR) * VEC;
        ok[k] = e < p.D;
        off[k] = ok[k] ? e : 0;
    }

    float acc[R][NACC][VEC];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int k = 0; k < NACC; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[r][k][e] = 0.f;

    const TIN *__restrict__ Hp = static_cast<const TIN *>(p.H);

    for (int j0 = a; j0 < b; j0 += kWave) {
        const int n = min(kWave, b - j0);
        int cl = 0;
        float vl = 0.f;
        if (lane < n) {
            cl = p.col[j0 + lane];
            vl = p.val[j0 + lane];
        }
        int i = 0;
        for (; i + G * U <= n; i += G * U) {
            int c[U];
            float v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int src = i + u * G + g;
                c[u] = pick_i<G>(cl, src);
                v[u] = pick_f<G>(vl, src);
            }
            float h[U][NACC][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const TIN *row = Hp + (int64_t)c[u] * p.ldh;
#pragma unroll
                for (int k = 0; k < NACC; ++k) VecIO<TIN, VEC>::load(row + off[k], h[u][k]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < NACC; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[u % R][k][e] = fmaf(v[u], h[u][k][e], acc[u % R][k][e]);
        }
        if constexpr (R == 1) {
            for (; i < n; i += G) {
                const int src = i + g;
                const int c = pick_i<G>(cl, src & (kWave - 1));
                const float v = pick_f<G>(vl, src & (kWave - 1));
                if (src < n) {
                    const TIN *row = Hp + (int64_t)c * p.ldh;
#pragma unroll
                    for (int k = 0; k < NACC; ++k) {
                        float h[VEC];
                        VecIO<TIN, VEC>::load(row + off[k], h);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[0][k][e] = fmaf(v, h[e], acc[0][k][e]);
                    }
                }
            }
        } else {
            // fewer than G * U entries are left; i is a multiple of G * U, so step u continues chain u mod R
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int src = i + u * G + g;
                const int c = pick_i<G>(cl, src & (kWave - 1));
                const float v = pick_f<G>(vl, src & (kWave - 1));
                if (src < n) {
                    const TIN *row = Hp + (int64_t)c * p.ldh;
#pragma unroll
                    for (int k = 0; k < NACC; ++k) {
                        float h[VEC];
                        VecIO<TIN, VEC>::load(row + off[k], h);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[u % R][k][e] = fmaf(v, h[e], acc[u % R][k][e]);
                    }
                }
            }
        }
    }

    // combine the G group sums: group g ^ 1, g ^ 2, ... (fixed order), chain set by chain set
    if constexpr (G > 1) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int o = LPR; o < kWave; o <<= 1)
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[r][0][e] += __shfl_xor(acc[r][0][e], o, kWave);
    }
    // then the chain sets, continuing the same pairwise order
#pragma unroll
    for (int s = 1; s < R; s <<= 1)
#pragma unroll
        for (int r = 0; r < R; r += 2 * s)
#pragma unroll
            for (int k = 0; k < NACC; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[r][k][e] += acc[r + s][k][e];

    if (g == 0) {
        if (to_ws) {
            float *dst = p.ws + out_row * p.ldws;
#pragma unroll
            for (int k = 0; k < NACC; ++k)
                if (ok[k]) store_f32<VEC>(dst + off[k], acc[0][k]);
        } else {
            TOUT *dst = static_cast<TOUT *>(p.Y) + out_row * p.ldy;
            if (p.y_vec) {
#pragma unroll
                for (int k = 0; k < NACC; ++k)
                    if (ok[k]) VecIO<TOUT, VEC>::store(dst + off[k], acc[0][k]);
            } else {
#pragma unroll
                for (int k = 0; k < NACC; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        if (ok[k] && off[k] + e < p.D) store_elem(dst + off[k] + e, acc[0][k][e]);
            }
        }
    }
}

// Y[row q] = sum over the segments of split row q.  A workgroup owns one split row and 64 of its
// columns: 16 chains x 16 lanes, each lane a float4.  Chain c adds segments c, c + 16, ... in order;
// the 16 chain sums are then added in chain order, so the summation order is fixed.
template <typename TOUT>
__global__ void __launch_bounds__(256) spmm_reduce_split_rows(const float *__restrict__ ws, int64_t ldws,
                                                              const int32_t *__restrict__ long_rows,
                                                              const int32_t *__restrict__ seg_first, int32_t q_base,
                                                              int32_t D, TOUT *__restrict__ Y, int64_t ldy,
                                                              const uint8_t *__restrict__ long_skip)
{
    __shared__ float4 part[16][16];
    const int q = q_base + blockIdx.x;
    if (long_skip != nullptr && long_skip[q]) return;  // a hub row: the hub pass writes it
    const int chain = threadIdx.x >> 4;
    const int l = threadIdx.x & 15;
    const int d = blockIdx.y * 64 + l * 4;
    const int s0 = seg_first[q];
    const int s1 = seg_first[q + 1];
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d < D) {  // ldws is a multiple of 4, so the float4 at d stays inside the padded workspace row
        for (int i = s0 + chain; i < s1; i += 16) {
            const float4 t = *reinterpret_cast<const float4 *>(ws + (int64_t)i * ldws + d);
            acc.x += t.x;
            acc.y += t.y;
            acc.z += t.z;
            acc.w += t.w;
        }
    }
    part[chain][l] = acc;
    __syncthreads();
    if (chain == 0 && d < D) {
        float4 s = part[0][l];
#pragma unroll
        for (int c = 1; c < 16; ++c) {
            s.x += part[c][l].x;
            s.y += part[c][l].y;
            s.z += part[c][l].z;
            s.w += part[c][l].w;
        }
        const float v[4] = {s.x, s.y, s.z, s.w};
        TOUT *dst = Y + (int64_t)long_rows[q] * ldy + d;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (d + e < D) {
                if constexpr (sizeof(TOUT) == 4)
                    dst[e] = v[e];
                else
                    dst[e] = (uint16_t)f32_to_bf16(v[e]);
            }
        }
    }
}

__global__ void narrow_i64_kernel(int64_t n, const int64_t *__restrict__ src, int32_t *__restrict__ dst)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = (int32_t)src[i];
}

// Diagnostic: what the memory system gives to the access pattern of the SpMM when nothing else is in the
// way -- uniformly random rows of a dense table, 128-bit loads, G rows per wavefront instruction, 8 loads in
// flight per lane, row numbers from a hash (no index stream, no arithmetic worth mentioning).
__device__ __forceinline__ uint32_t mix32(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

template <int LPR>
__global__ void __launch_bounds__(256) random_gather_kernel(const float4 *__restrict__ table, uint32_t rows, int64_t ld4, int iters,
                                                            float *__restrict__ sink)
{
    constexpr int G = kWave / LPR;
    constexpr int U = 8;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = (uint32_t)((blockIdx.x * 256 + threadIdx.x) >> 6);
    const int g = lane / LPR, t = lane % LPR;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int it = 0; it < iters; it += U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t r = mix32((wave * 1315423911u) ^ (uint32_t)((it + u) * G + g) * 2654435761u) % rows;
            v[u] = table[(int64_t)r * ld4 + t];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc.x += v[u].x;
            acc.y += v[u].y;
            acc.z += v[u].z;
            acc.w += v[u].w;
        }
    }
    if (acc.x + acc.y + acc.z + acc.w == 1.2345678e30f) sink[0] = 1.f;  // keeps the loads alive
}

int64_t ws_ld(int64_t D) { return (D + 3) / 4 * 4; }

// ---- staging of H into rows that start on 128-byte lines ----
// A gathered row that starts on a line touches ceil(row bytes / 128) lines; one that starts anywhere touches up to one
// more (602 fp32: 19 against 19.8 on average), and the lines fetched are what a launch costs.  When every row of H
// is gathered many times, copying H once into line-aligned rows pays: 232,965 x 602 fp32 under 114.6 M entries,
// 0.2 ms for the copy, 34.0 -> 30.9 ms for the product.  The values and their order are the same, so is the result.
constexpr int64_t kLine = 128;

// mean number of lines touched by rows of `row_bytes` bytes whose start offsets inside a line are the multiples of
// `granule` (a power of two up to 128)
double mean_lines(int64_t row_bytes, int64_t granule)
{
    double sum = 0.0;
    int n = 0;
    for (int64_t off = 0; off < kLine; off += granule, ++n) sum += (double)((off + row_bytes + kLine - 1) / kLine);
    return sum / n;
}

int64_t offset_granule(uintptr_t base, int64_t pitch_bytes)
{
    int64_t g = kLine;
    while (g > 1 && (base % g != 0 || pitch_bytes % g != 0)) g >>= 1;
    return g;
}

// leading dimension (elements) of the staged copy, or 0 when staging does not pay
int64_t staged_ld(int64_t K, int64_t nnz, int64_t D, int64_t elem, uintptr_t base, int64_t ldh)
{
    if (K <= 0) return 0;
    const int64_t row_bytes = D * elem;
    const int64_t g = offset_granule(base, ldh * elem);
    if (g == kLine) return 0;  // rows already start on lines
    const double aligned = (double)((row_bytes + kLine - 1) / kLine);
    const double saved = mean_lines(row_bytes, g) - aligned;  // lines per gathered row
    if (saved < 0.3) return 0;
    // the copy reads and writes H once; the gathers save `saved` lines each.  Stage when the saving is at least three
    // times the bytes of a row per row of H (a copy streams, a gather does not: margin for that)
    if ((double)nnz * saved * (double)kLine < 3.0 * (double)K * (double)row_bytes) return 0;
    return (row_bytes + kLine - 1) / kLine * kLine / elem;
}

template <typename T, int VEC>
__global__ void __launch_bounds__(256) stage_rows_kernel(int64_t K, int32_t D, const T *__restrict__ src, int64_t lds,
                                                         T *__restrict__ dst, int64_t ldd)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= K) return;
    const T *s = src + row * lds;
    T *d = dst + row * ldd;
    for (int c = lane * VEC; c < D; c += kWave * VEC) {
        float v[VEC];
        VecIO<T, VEC>::load(s + c, v);
        VecIO<T, VEC>::store(d + c, v);
    }
}

}  // namespace

struct plx_spmm_plan {
    int64_t M, K, nnz;
    const int32_t *rowptr;
    const int32_t *col;
    int32_t seg_len;
    int64_t n_long, n_seg;
    int32_t *tables;  // device: long_rows[n_long] | seg_first[n_long+1] | seg_begin[n_seg] | seg_end[n_seg]
    const int32_t *long_rows, *seg_first, *seg_begin, *seg_end;
    std::vector<int32_t> h_long_rows, h_seg_first;  // host copies, to cut row ranges out of the plan
    int slicing = 0;  // 0: column slices of H where the cost model says so, 1: whenever rows exceed a slice, -1: never
    plx::hub::HubPlan hub;  // tables of the hub pass (empty: no hub pass)
    plx::hub::HubPlan hub_wide;  // the same in the wide layout, for bf16 rows of 512 bytes and more (empty: those take `hub`)
    int hub_mode = 0;       // 0: hub pass where the tables exist and the operands allow it, -1: never
};

namespace {

template <typename TIN, typename TOUT, int VEC, int LPR, int NACC, int R = 1>
void launch_variant(const SpmmArgs &a, dim3 grid, hipStream_t st)
{
    spmm_csr_kernel<TIN, TOUT, VEC, LPR, NACC, R><<<grid, 256, 0, st>>>(a);
}

template <typename TIN, typename TOUT, int VEC>
int launch_for_vec(const SpmmArgs &a, int lpr, int nacc, dim3 grid, hipStream_t st)
{
    switch (lpr) {
        case 4: launch_variant<TIN, TOUT, VEC, 4, 1>(a, grid, st); return 0;
        case 8: launch_variant<TIN, TOUT, VEC, 8, 1>(a, grid, st); return 0;
        case 16: launch_variant<TIN, TOUT, VEC, 16, 1>(a, grid, st); return 0;
        case 32: launch_variant<TIN, TOUT, VEC, 32, 1>(a, grid, st); return 0;
        default: break;
    }
    switch (nacc) {
        case 1: launch_variant<TIN, TOUT, VEC, 64, 1>(a, grid, st); return 0;
        case 2: launch_variant<TIN, TOUT, VEC, 64, 2>(a, grid, st); return 0;
        case 3: launch_variant<TIN, TOUT, VEC, 64, 3>(a, grid, st); return 0;
        case 4: launch_variant<TIN, TOUT, VEC, 64, 4>(a, grid, st); return 0;
        case 5: launch_variant<TIN, TOUT, VEC, 64, 5>(a, grid, st); return 0;
        case 6: launch_variant<TIN, TOUT, VEC, 64, 6>(a, grid, st); return 0;
        case 7: launch_variant<TIN, TOUT, VEC, 64, 7>(a, grid, st); return 0;
        case 8: launch_variant<TIN, TOUT, VEC, 64, 8>(a, grid, st); return 0;
        default: return -1;
    }
}

// the one-pass kernel summing in the order of the column-sliced product (kSliceChains chains): lpr 32 -> two lane
// groups with two chains each, lpr 64 -> one group with four chains and at most two accumulator vectors
template <typename TIN, typename TOUT, int VEC>
int launch_chained(const SpmmArgs &a, int lpr, int nacc, dim3 grid, hipStream_t st)
{
    if (lpr == 32) { launch_variant<TIN, TOUT, VEC, 32, 1, 2>(a, grid, st); return 0; }
    if (lpr == 64 && nacc == 1) { launch_variant<TIN, TOUT, VEC, 64, 1, 4>(a, grid, st); return 0; }
    if (lpr == 64 && nacc == 2) { launch_variant<TIN, TOUT, VEC, 64, 2, 4>(a, grid, st); return 0; }
    return -1;
}

// ---- column slices of H ----
// A wide H is gathered in passes over slices of kSliceBytes per row when its rows, taken whole, overflow the last-level
// cache while one slice of every row stays in it: on a 233 K-row graph with 492 entries per row, 602 fp32 columns take
// 31.0 ms in one pass and 18.4 ms in ten passes over 64-column slices (a pass re-reads the index and value arrays, 8 of
// the 264 bytes an entry then costs).  A slice is one quarter of a wavefront's 64 x 16 bytes, so a pass runs with four
// lane groups; products that cannot be sliced in place (row ranges, operands that are not line-aligned and have no
// room to be copied) use the one-pass kernel with the same four chains per sum, hence the same bits.
constexpr int64_t kSliceBytes = 256;
constexpr int kSliceChains = 4;

bool sliced_plan(const plx_spmm_plan *plan, int64_t D, int64_t elem)
{
    const int64_t row_bytes = D * elem;
    if (row_bytes <= kSliceBytes || plan->K <= 0 || plan->M <= 0 || plan->slicing < 0) return false;
    if (plan->slicing > 0) return true;
    if (plan->K * row_bytes <= (64ll << 20)) return false;     // whole rows stay cached as they are
    if (plan->K * kSliceBytes > (128ll << 20)) return false;   // not even a slice of every row would
    return plan->nnz >= 32 * plan->K && plan->nnz >= 32 * plan->M;  // every row of H is gathered often, rows of A are long
}

// Slices are read with 16-byte loads from line-aligned rows; a last slice that is not a multiple of 16 bytes wide is
// read past its width, which is safe inside the padded rows of a staged copy but not inside a caller's tensor.
bool sliceable_in_place(uintptr_t base, int64_t ldh, int64_t D, int64_t elem)
{
    return offset_granule(base, ldh * elem) == kLine && (D * elem) % 16 == 0;
}

// leading dimension (elements) of the staged copy of H that a whole-matrix product of this plan and width wants, or 0:
// line-aligned rows either because column slices need them or because alignment alone repays the copy
int64_t wanted_stage_ld(const plx_spmm_plan *plan, int64_t D, int64_t elem, uintptr_t base, int64_t ldh)
{
    if (sliced_plan(plan, D, elem)) {
        if (sliceable_in_place(base, ldh, D, elem)) return 0;
        return (D * elem + kLine - 1) / kLine * kLine / elem;
    }
    return staged_ld(plan->K, plan->nnz, D, elem, base, ldh);
}

// room for the partial sums of the hub pass, or 0 when this plan and width do not use it (column slices and the hub
// pass answer different shapes of matrix; a product takes one or the other)
// The pass saves memory traffic in proportion to the bytes of a row of H and costs instructions per entry and per change
// of sum, so narrow rows do not repay it: measured on the 2.45 M-node power-law graph (7.4 entries per slot and window)
// and on a 4.19 M-node R-MAT block (3 per slot and window), fp32: 512-byte rows 7.6 -> 6.0 and 4.1 -> 3.5 ms, 256-byte
// rows 3.6 -> 3.1 and 2.3 -> 2.4 ms, 128-byte rows 2.3 -> 2.5 and 1.8 -> 2.1 ms; bf16 rows count by the 256 bytes that the
// 128 columns of a tile hold (256 columns: 7.3 -> 6.7 and 4.2 -> 4.3 ms).  The rule looks at the plan and the width only,
// so a whole product and its row ranges choose alike.
// which tables a product of this width and element size takes: the wide layout for bf16 rows of 512 bytes and more
// where the plan has it (the operand must also allow 16-byte loads: wide_ok), else the regular one by the rule above
enum HubChoice { kHubNone = 0, kHubRegular = 1, kHubWide = 2 };

bool hub_regular_pays(const plx_spmm_plan *plan, int64_t D, int64_t elem)
{
    if (plan->hub.block == nullptr) return false;
    const int64_t tile_bytes = std::min<int64_t>(D, plx::hub::kHubTile) * elem;  // of a row of H, per load of the pass
    return !(tile_bytes < 256 || (tile_bytes < 512 && plan->hub.mean_run < 4.0));
}

HubChoice hub_choice(const plx_spmm_plan *plan, int64_t D, int64_t elem, bool wide_ok)
{
    if (plan->hub_mode < 0 || sliced_plan(plan, D, elem)) return kHubNone;
    if (elem == 2 && D * elem >= 512 && plan->hub_wide.block != nullptr && wide_ok) return kHubWide;
    return hub_regular_pays(plan, D, elem) ? kHubRegular : kHubNone;
}

// sized for whichever tables the operand may turn out to allow
size_t hub_workspace_bytes(const plx_spmm_plan *plan, int64_t D, int64_t elem)
{
    size_t bytes = 0;
    if (hub_choice(plan, D, elem, true) == kHubWide) bytes = plx::hub::partial_bytes(D, true);
    if (hub_choice(plan, D, elem, false) == kHubRegular) bytes = std::max(bytes, plx::hub::partial_bytes(D, false));
    return bytes;
}

// scratch of a product of width D whose elements take `elem` bytes: partial rows of the split rows, partial sums of the
// hub pass, and room for a line-aligned copy of H where contiguous rows of that type would want one
size_t workspace_need(const plx_spmm_plan *plan, int64_t D, int64_t elem)
{
    if (!plan || D <= 0) return 0;
    const size_t seg_bytes = (size_t)plan->n_seg * (size_t)ws_ld(D) * sizeof(float);
    const int64_t ld_st = wanted_stage_ld(plan, D, elem, 0, D);
    const size_t hub_bytes = hub_workspace_bytes(plan, D, elem);
    if (ld_st == 0) return seg_bytes + hub_bytes;
    return (size_t)kLine + (size_t)plan->K * (size_t)ld_st * (size_t)elem + seg_bytes + hub_bytes;
}

// `may_stage` = false: the workspace holds the partial rows of the split rows and nothing else (H is gathered where
// it lies; same values in the same order, so the same result)
template <typename T>
int spmm_impl(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, const float *val, const T *H, int64_t ldh,
              int64_t D, T *Y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream, bool may_stage = true,
              int parts = 3, int hub_stage = 0)
{
    // hub_stage, for a product computed range by range with one workspace: 0 = this call stands alone (a range that holds
    // a hub row runs the whole pass); 1 = first range of a sequence: the pass runs now, for every hub row, and leaves its
    // partial sums in the workspace; 2 = a later range: the partial sums are there, only this range's hub rows are added up
    PLX_REQUIRE(plan != nullptr, "spmm: plan is NULL");
    PLX_REQUIRE(row_begin >= 0 && row_begin <= row_end && row_end <= plan->M, "spmm: row range [%lld, %lld) outside [0, %lld)",
                (long long)row_begin, (long long)row_end, (long long)plan->M);
    PLX_REQUIRE(D >= 0 && D <= (1ll << 21), "spmm: bad feature width D=%lld (at most 2,097,152)", (long long)D);
    if (row_begin == row_end || D == 0) return PLX_OK;
    PLX_REQUIRE((val || plan->nnz == 0) && H && Y, "spmm: NULL operand (val=%p H=%p Y=%p)", (const void *)val, (const void *)H, (void *)Y);
    PLX_REQUIRE(ldh >= D && ldy >= D, "spmm: leading dimension smaller than D (ldh=%lld ldy=%lld D=%lld)",
                (long long)ldh, (long long)ldy, (long long)D);
    // sized for this element type: the hub pass and the column slices go by the bytes of a row, so a bf16 product may
    // need room that the fp32 product of the same width does not (each type has its size query)
    const size_t seg_bytes = (size_t)plan->n_seg * (size_t)ws_ld(D) * sizeof(float);
    const size_t hub_bytes = may_stage ? hub_workspace_bytes(plan, D, sizeof(T)) : 0;
    const size_t need = may_stage ? workspace_need(plan, D, sizeof(T)) : seg_bytes;
    if (need > 0 && (workspace == nullptr || workspace_bytes < need))
        return plx::fail(PLX_ERR_WORKSPACE, "spmm: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    PLX_REQUIRE(need == 0 || (reinterpret_cast<uintptr_t>(workspace) % 16) == 0, "spmm: workspace not 16-byte aligned");
    hipStream_t st = plx::as_stream(stream);

    constexpr int kMaxVec = 16 / (int)sizeof(T);
    constexpr int64_t kElem = (int64_t)sizeof(T);
    const bool whole = row_begin == 0 && row_end == plan->M;
    const bool sliced = sliced_plan(plan, D, kElem);

    // Whole-matrix products stage H into line-aligned rows when that pays and the workspace has the room (the size
    // query reserves it for contiguous fp32 rows); the partial rows of split rows follow the staged copy.
    char *ws_base = static_cast<char *>(workspace);
    const T *const H0 = H;  // the operand as the caller passed it
    const int64_t ldh0 = ldh;
    bool h_is_staged = false;  // H points at the copy: rows on 128-byte lines, padded to whole lines
    if (may_stage && whole) {
        const int64_t ld_st = wanted_stage_ld(plan, D, kElem, reinterpret_cast<uintptr_t>(H), ldh);
        const size_t st_bytes = (size_t)plan->K * (size_t)ld_st * sizeof(T);
        const size_t pad = ws_base ? (size_t)((kLine - reinterpret_cast<uintptr_t>(ws_base) % kLine) % kLine) : 0;
        if (ld_st > 0 && ws_base != nullptr && workspace_bytes >= pad + st_bytes + seg_bytes + hub_bytes) {
            T *staged = reinterpret_cast<T *>(ws_base + pad);
            const unsigned sblocks = (unsigned)plx::ceil_div(plan->K, 4);
            int sv = kMaxVec;
            while (sv > 1 && (D % sv || ldh % sv || reinterpret_cast<uintptr_t>(H) % (sv * sizeof(T)))) sv >>= 1;
            switch (sv) {
                case 1: stage_rows_kernel<T, 1><<<sblocks, 256, 0, st>>>(plan->K, (int32_t)D, H, ldh, staged, ld_st); break;
                case 2: stage_rows_kernel<T, 2><<<sblocks, 256, 0, st>>>(plan->K, (int32_t)D, H, ldh, staged, ld_st); break;
                case 4: stage_rows_kernel<T, 4><<<sblocks, 256, 0, st>>>(plan->K, (int32_t)D, H, ldh, staged, ld_st); break;
                default:
                    if constexpr (kMaxVec == 8) stage_rows_kernel<T, 8><<<sblocks, 256, 0, st>>>(plan->K, (int32_t)D, H, ldh, staged, ld_st);
                    break;
            }
            PLX_LAUNCH_CHECK("stage_rows_kernel");
            H = staged;
            ldh = ld_st;
            h_is_staged = true;
            ws_base += pad + st_bytes;  // a multiple of 128 bytes past an aligned address
        }
    }

    // ---- the hub pass takes the longest rows when the plan has its tables and the caller's H suits its loads ----
    // (4-element vectors at 32-bit byte offsets).  The choice looks at the operand as the caller passed it, so a whole
    // product and a row range of it choose alike, and a row range runs the whole pass when it holds a hub row: the sums
    // of a hub row are then the same bits whatever range it is computed in and wherever H is gathered from.
    bool use_hub = false, hub_in_range = false;
    const T *hub_h = H0;
    int64_t hub_ldh = ldh0;
    const plx::hub::HubPlan *hp = nullptr;
    if (hub_bytes > 0) {
        auto fits = [&](int64_t q) {  // q-element vectors at 32-bit byte offsets
            return D % q == 0 && ldh0 % q == 0 && reinterpret_cast<uintptr_t>(H0) % (q * sizeof(T)) == 0 && plan->K * ldh0 * kElem < plx::hub::kHubMaxBytes;
        };
        const HubChoice choice = hub_choice(plan, D, kElem, fits(8));
        if (choice == kHubWide) hp = &plan->hub_wide;
        else if (choice == kHubRegular && fits(4)) hp = &plan->hub;
    }
    if (hp != nullptr) {
        const auto &hr = hp->h_rows_sorted;
        hub_in_range = std::lower_bound(hr.begin(), hr.end(), (int32_t)row_begin) != std::lower_bound(hr.begin(), hr.end(), (int32_t)row_end);
        use_hub = hub_in_range || hub_stage == 1;
        if (h_is_staged && plan->K * ldh * kElem < plx::hub::kHubMaxBytes) {
            hub_h = H;
            hub_ldh = ldh;
        }
    }
    float *hub_partial = reinterpret_cast<float *>(ws_base + seg_bytes);  // seg_bytes is a multiple of 16
    if (use_hub && (ws_base == nullptr || (size_t)(ws_base - static_cast<char *>(workspace)) + seg_bytes + hub_bytes > workspace_bytes))
        return plx::fail(PLX_ERR_WORKSPACE, "spmm: the partial sums of the hub pass need %zu bytes behind the %zu of the split rows, %zu given",
                         hub_bytes, seg_bytes, workspace_bytes);
    auto hub_pass = [&]() -> int {
        if (!use_hub || !(parts & 2)) return PLX_OK;
        return plx::hub::launch(*hp, plan->col, val, hub_h, hub_ldh, D, D, sizeof(T) == 2, row_begin, row_end, Y, ldy, hub_partial, st,
                                /*run_pass=*/hub_stage != 2, /*run_reduce=*/hub_in_range);
    };

    SpmmArgs a;
    a.seg_skip = use_hub ? hp->seg_is_hub : nullptr;
    a.rowptr = plan->rowptr;
    a.col = plan->col;
    a.val = val;
    a.ws = reinterpret_cast<float *>(ws_base);
    a.seg_begin = plan->seg_begin;
    a.seg_end = plan->seg_end;
    a.ldh = ldh;
    a.ldy = ldy;
    // split rows inside the range, and their segments
    const auto lr_begin = plan->h_long_rows.begin(), lr_end = plan->h_long_rows.end();
    const int64_t q0 = std::lower_bound(lr_begin, lr_end, (int32_t)row_begin) - lr_begin;
    const int64_t q1 = std::lower_bound(lr_begin, lr_end, (int32_t)row_end) - lr_begin;
    const int64_t s0 = q1 > q0 ? plan->h_seg_first[(size_t)q0] : 0;
    const int64_t s1 = q1 > q0 ? plan->h_seg_first[(size_t)q1] : 0;
    a.M = (int32_t)plan->M;
    a.n_seg = (int32_t)(s1 - s0);
    a.seg_len = plan->seg_len;
    a.row_begin = (int32_t)row_begin;
    a.row_end = (int32_t)row_end;
    a.seg_base = (int32_t)s0;
    const int64_t tasks = (row_end - row_begin) + (s1 - s0);
    auto reduce_split_rows = [&](T *y, int64_t d) -> int {
        if (q1 > q0) {
            dim3 rgrid((unsigned)(q1 - q0), (unsigned)plx::ceil_div(d, 64), 1);
            spmm_reduce_split_rows<T><<<rgrid, 256, 0, st>>>(a.ws, a.ldws, plan->long_rows, plan->seg_first, (int32_t)q0, (int32_t)d, y, ldy,
                                                             use_hub ? hp->long_is_hub : nullptr);
            PLX_LAUNCH_CHECK("spmm_reduce_split_rows");
        }
        return PLX_OK;
    };

    // ---- passes over column slices: whole matrix, rows of H (as they lie or as staged) on 128-byte lines ----
    if (sliced && whole && (h_is_staged || sliceable_in_place(reinterpret_cast<uintptr_t>(H), ldh, D, kElem))) {
        static_assert(kWave / 16 == kSliceChains, "a slice is covered by 16 lanes, so a pass sums in kSliceChains lane groups");
        constexpr int64_t kW = kSliceBytes / kElem;  // columns per slice; 16 lanes x 16 bytes cover one
        const bool y_vec = reinterpret_cast<uintptr_t>(Y) % 16 == 0 && (ldy * kElem) % 16 == 0;
        a.ldws = ws_ld(kW);
        dim3 grid((unsigned)plx::ceil_div(tasks, 4), 1, 1);
        for (int64_t c0 = 0; c0 < D; c0 += kW) {
            const int64_t w = std::min<int64_t>(kW, D - c0);
            a.H = H + c0;
            a.Y = Y + c0;
            a.D = (int32_t)w;
            a.y_vec = (y_vec && w % kMaxVec == 0) ? 1 : 0;  // a ragged last slice loads past its width (inside the padded row) and stores by element
            launch_variant<T, T, kMaxVec, 16, 1>(a, grid, st);
            PLX_LAUNCH_CHECK("spmm_csr_kernel (column slice)");
            const int rc = reduce_split_rows(Y + c0, w);
            if (rc != PLX_OK) return rc;
        }
        return PLX_OK;
    }

    auto widest = [&](const T *h, int64_t ld_h) {
        int v = kMaxVec;
        while (v > 1 && (D % v || ld_h % v || ldy % v || reinterpret_cast<uintptr_t>(h) % (v * sizeof(T)) ||
                         reinterpret_cast<uintptr_t>(Y) % (v * sizeof(T))))
            v >>= 1;
        return v;
    };
    int vec = widest(H, ldh);
    const int64_t units = D / vec;
    int lpr = 4;
    while (lpr < kWave && lpr < units) lpr <<= 1;
    int nacc = 1, tiles = 1;
    if (lpr == kWave) {
        const int64_t chunks = plx::ceil_div(units, kWave);
        tiles = (int)plx::ceil_div(chunks, sliced ? 2 : 8);  // the chained kernel keeps four sums per accumulator vector
        nacc = (int)plx::ceil_div(chunks, tiles);
    }
    a.H = H;
    a.Y = Y;
    a.ldws = ws_ld(D);
    a.D = (int32_t)D;
    a.y_vec = 1;

    dim3 grid((unsigned)plx::ceil_div(tasks, 4), (unsigned)tiles, 1);
    int rc = -1;
    if (!(parts & 1)) return hub_pass();  // measurement of the hub pass alone
    if (sliced) {  // one pass, summed in the order of the sliced product
        switch (vec) {
            case 1: rc = launch_chained<T, T, 1>(a, lpr, nacc, grid, st); break;
            case 2: rc = launch_chained<T, T, 2>(a, lpr, nacc, grid, st); break;
            case 4: rc = launch_chained<T, T, 4>(a, lpr, nacc, grid, st); break;
            case 8:
                if constexpr (kMaxVec == 8) rc = launch_chained<T, T, 8>(a, lpr, nacc, grid, st);
                break;
            default: break;
        }
    } else {
        switch (vec) {
            case 1: rc = launch_for_vec<T, T, 1>(a, lpr, nacc, grid, st); break;
            case 2: rc = launch_for_vec<T, T, 2>(a, lpr, nacc, grid, st); break;
            case 4: rc = launch_for_vec<T, T, 4>(a, lpr, nacc, grid, st); break;
            case 8:
                if constexpr (kMaxVec == 8) rc = launch_for_vec<T, T, 8>(a, lpr, nacc, grid, st);
                break;
            default: break;
        }
    }
    if (rc != 0) return plx::fail(PLX_ERR_UNSUPPORTED, "spmm: no kernel for vec=%d lpr=%d nacc=%d%s", vec, lpr, nacc, sliced ? " (chained)" : "");
    PLX_LAUNCH_CHECK("spmm_csr_kernel");
    rc = reduce_split_rows(Y, D);
    if (rc != PLX_OK) return rc;
    return hub_pass();
}

// ---- the product without a caller's workspace: partial rows of the split rows in a static device array ----
// In host code `scratch` is only a handle of the symbol; the address of the array on a device comes from
// hipGetSymbolAddress with that device current, once per device (every device has its own copy).
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int static_scratch(void **out)
{
    int dev = -1;
    PLX_HIP_CHECK(hipGetDevice(&dev));
    PLX_REQUIRE(dev >= 0 && dev < kMaxDevices, "spmm_static: device ordinal %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        PLX_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        PLX_REQUIRE(ptr != nullptr, "spmm_static: hipGetSymbolAddress returned NULL");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return PLX_OK;
}

// the tables of the hub pass (regular or wide layout), kept when the hub rows hold at least `min_entries` entries
int build_hub(plx_spmm_plan *p, int64_t min_entries, bool wide, hipStream_t st)
{
    if (p->n_long == 0) return PLX_OK;
    plx::hub::HubPlan hp;
    const int rc = plx::hub::build_hub_plan(p->M, p->K, p->nnz, p->rowptr, p->col, p->seg_len, p->n_long, p->n_seg, p->long_rows, p->seg_first,
                                            p->h_long_rows, min_entries, wide, st, hp);
    if (rc != PLX_OK) return rc;
    (wide ? p->hub_wide : p->hub) = std::move(hp);
    return PLX_OK;
}

}  // namespace

extern "C" {

int plx_csr_narrow_i64(int64_t M, int64_t nnz, const int64_t *rowptr64, const int64_t *col64, int32_t *rowptr32,
                       int32_t *col32, void *stream)
{
    PLX_REQUIRE(M >= 0 && nnz >= 0, "csr_narrow: negative size");
    PLX_REQUIRE(nnz < (1ll << 31) && M < (1ll << 31) - 1, "csr_narrow: M=%lld nnz=%lld do not fit int32", (long long)M,
                (long long)nnz);
    PLX_REQUIRE(rowptr64 && rowptr32, "csr_narrow: NULL rowptr");
    PLX_REQUIRE(nnz == 0 || (col64 && col32), "csr_narrow: NULL col");
    hipStream_t st = plx::as_stream(stream);
    {
        const int64_t n = M + 1;
        const unsigned blocks = (unsigned)std::min<int64_t>(plx::ceil_div(n, 256), 65536);
        narrow_i64_kernel<<<blocks, 256, 0, st>>>(n, rowptr64, rowptr32);
        PLX_LAUNCH_CHECK("narrow_i64_kernel");
    }
    if (nnz > 0) {
        const unsigned blocks = (unsigned)std::min<int64_t>(plx::ceil_div(nnz, 256), 65536);
        narrow_i64_kernel<<<blocks, 256, 0, st>>>(nnz, col64, col32);
        PLX_LAUNCH_CHECK("narrow_i64_kernel");
    }
    return PLX_OK;
}

int plx_spmm_segments_host(int64_t M, const int32_t *rowptr_host, int32_t seg_len, int64_t *n_long, int64_t *n_seg,
                           int32_t *long_rows_host, int32_t *seg_first_host, int64_t cap_long, int32_t *seg_begin_host,
                           int32_t *seg_end_host, int64_t cap_seg)
{
    PLX_REQUIRE(M >= 0 && rowptr_host != nullptr && seg_len > 0, "spmm_segments: bad arguments");
    PLX_REQUIRE(n_long != nullptr && n_seg != nullptr, "spmm_segments: NULL count outputs");
    int64_t nl = 0, ns = 0;
    for (int64_t r = 0; r < M; ++r) {
        const int64_t a = rowptr_host[r], b = rowptr_host[r + 1];
        PLX_REQUIRE(b >= a, "spmm_segments: rowptr decreases at row %lld", (long long)r);
        const int64_t len = b - a;
        if (len <= seg_len) continue;
        const int64_t parts = plx::ceil_div(len, seg_len);
        const int64_t base = len / parts, extra = len % parts;  // the first `extra` segments get one more
        if (long_rows_host && nl < cap_long) long_rows_host[nl] = (int32_t)r;
        if (seg_first_host && nl < cap_long) seg_first_host[nl] = (int32_t)ns;
        int64_t pos = a;
        for (int64_t s = 0; s < parts; ++s) {
            const int64_t l = base + (s < extra ? 1 : 0);
            if (seg_begin_host && ns < cap_seg) seg_begin_host[ns] = (int32_t)pos;
            if (seg_end_host && ns < cap_seg) seg_end_host[ns] = (int32_t)(pos + l);
            pos += l;
            ++ns;
        }
        ++nl;
    }
    if (seg_first_host && nl <= cap_long) seg_first_host[nl] = (int32_t)ns;
    *n_long = nl;
    *n_seg = ns;
    return PLX_OK;
}

int plx_spmm_plan_create(plx_spmm_plan **out, int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr,
                         const int32_t *col, int32_t seg_len, void *stream)
{
    PLX_REQUIRE(out != nullptr, "plan_create: NULL output");
    *out = nullptr;
    PLX_REQUIRE(M >= 0 && K >= 0 && nnz >= 0, "plan_create: negative size");
    // the kernels step through the entries 64 at a time with 32-bit positions
    PLX_REQUIRE(M < (1ll << 31) - 1 && K < (1ll << 31) && nnz < (1ll << 31) - 64, "plan_create: sizes exceed int32 indexing");
    PLX_REQUIRE(rowptr != nullptr, "plan_create: NULL rowptr");
    PLX_REQUIRE(nnz == 0 || col != nullptr, "plan_create: NULL col");
    // default split length, from measurements: 1,024 entries on graphs with short rows (the 2.45 M-node power-law graph:
    // 1,024 / 4,096 / 16,384 give 7.27 / 7.32 / 7.93 ms), 4,096 where rows hold hundreds of entries on average (the
    // 233 K-node R-MAT graph at D = 602: 36.6 / 33.6 / 36.9 ms)
    if (seg_len <= 0) seg_len = (M > 0 && nnz / M >= 128) ? 4096 : 1024;
    hipStream_t st = plx::as_stream(stream);

    // validation and the tables of the split rows, on the device
    plx::PlanTables t;
    const int rc = plx::build_plan_tables(M, K, nnz, rowptr, col, seg_len, st, t);
    if (rc != PLX_OK) return rc;

    plx_spmm_plan *p = new (std::nothrow) plx_spmm_plan();
    if (!p) {
        if (t.tables) (void)hipFree(t.tables);
        return plx::fail(PLX_ERR_NOMEM, "plan_create: host allocation failed");
    }
    p->M = M;
    p->K = K;
    p->nnz = nnz;
    p->rowptr = rowptr;
    p->col = col;
    p->seg_len = seg_len;
    p->n_long = t.n_long;
    p->n_seg = t.n_seg;
    p->tables = t.tables;
    p->long_rows = p->seg_first = p->seg_begin = p->seg_end = nullptr;
    if (t.n_long > 0) {
        p->h_long_rows = std::move(t.h_long_rows);
        p->h_seg_first = std::move(t.h_seg_first);
        p->long_rows = p->tables;
        p->seg_first = p->tables + t.n_long;
        p->seg_begin = p->seg_first + t.n_long + 1;
        p->seg_end = p->seg_begin + t.n_seg;
    }
    // The hub pass pays where H is far larger than the caches (its rows are then fetched again for almost every
    // entry), rows are short on average (wide-row matrices take column slices instead) and the long rows hold a good
    // part of the entries: measured on the 2.45 M-node power-law graph, 128 fp32 columns, 33 % of the entries in hub
    // rows: 7.3 ms without, 5.7 ms with.
    if (t.n_long > 0 && M > 0 && nnz / M < 128 && K * 512 >= (128ll << 20)) {
        const int hrc = build_hub(p, nnz / 8, false, st);
        // no room for the tables, or rows whose columns do not ascend: the plan works without them
        if (hrc != PLX_OK && hrc != PLX_ERR_NOMEM && hrc != PLX_ERR_UNSUPPORTED) {
            plx_spmm_plan_destroy(p);
            return hrc;
        }
    }
    *out = p;
    return PLX_OK;
}

int plx_spmm_plan_build_hub(plx_spmm_plan *plan, void *stream)
{
    PLX_REQUIRE(plan != nullptr, "plan_build_hub: plan is NULL");
    if (plan->hub.block != nullptr) return PLX_OK;
    return build_hub(plan, 1, false, plx::as_stream(stream));
}

int plx_spmm_plan_build_hub_wide(plx_spmm_plan *plan, void *stream)
{
    PLX_REQUIRE(plan != nullptr, "plan_build_hub_wide: plan is NULL");
    if (plan->hub_wide.block != nullptr) return PLX_OK;
    return build_hub(plan, 1, true, plx::as_stream(stream));
}

int plx_spmm_plan_set_hub(plx_spmm_plan *plan, int mode)
{
    PLX_REQUIRE(plan != nullptr, "plan_set_hub: plan is NULL");
    PLX_REQUIRE(mode >= -1 && mode <= 0, "plan_set_hub: mode must be -1 or 0");
    plan->hub_mode = mode;
    return PLX_OK;
}

int plx_spmm_plan_destroy(plx_spmm_plan *plan)
{
    if (!plan) return PLX_OK;
    plx::hub::free_hub_plan(plan->hub);
    plx::hub::free_hub_plan(plan->hub_wide);
    if (plan->tables) (void)hipFree(plan->tables);
    delete plan;
    return PLX_OK;
}

int64_t plx_spmm_plan_info(const plx_spmm_plan *plan, int what)
{
    if (!plan) return -1;
    switch (what) {
        case 0: return plan->M;
        case 1: return plan->K;
        case 2: return plan->nnz;
        case 3: return plan->n_long;
        case 4: return plan->n_seg;
        case 5: return plan->seg_len;
        case 6: return plan->hub.n_rows;
        case 7: return plan->hub.entries;
        case 8: return (plan->hub.stored + plan->hub_wide.stored) * 5;  // bytes of the streams, both layouts
        case 9: return plan->hub_wide.n_rows;
        case 10: return plan->hub_wide.entries;
        default: return -1;
    }
}

int plx_spmm_plan_tables_host(const plx_spmm_plan *plan, int32_t *long_rows_host, int32_t *seg_first_host, int32_t *seg_begin_host,
                              int32_t *seg_end_host)
{
    PLX_REQUIRE(plan != nullptr, "plan_tables_host: plan is NULL");
    if (plan->n_long == 0) {
        if (seg_first_host) seg_first_host[0] = 0;
        return PLX_OK;
    }
    const size_t nl = (size_t)plan->n_long, ns = (size_t)plan->n_seg;
    if (long_rows_host) PLX_HIP_CHECK(hipMemcpy(long_rows_host, plan->long_rows, nl * sizeof(int32_t), hipMemcpyDeviceToHost));
    if (seg_first_host) PLX_HIP_CHECK(hipMemcpy(seg_first_host, plan->seg_first, (nl + 1) * sizeof(int32_t), hipMemcpyDeviceToHost));
    if (seg_begin_host) PLX_HIP_CHECK(hipMemcpy(seg_begin_host, plan->seg_begin, ns * sizeof(int32_t), hipMemcpyDeviceToHost));
    if (seg_end_host) PLX_HIP_CHECK(hipMemcpy(seg_end_host, plan->seg_end, ns * sizeof(int32_t), hipMemcpyDeviceToHost));
    return PLX_OK;
}

int64_t plx_spmm_plan_hub_info(const plx_spmm_plan *plan, int wide, int what)
{
    if (!plan) return -1;
    const plx::hub::HubPlan &hp = wide ? plan->hub_wide : plan->hub;
    switch (what) {
        case 0: return hp.n_rows;
        case 1: return hp.n_slots;
        case 2: return hp.entries;
        case 3: return hp.stored;
        case 4: return hp.window;
        case 5: return hp.n_windows;
        case 6: return hp.windows_per_range;
        case 7: return hp.rows_per_wave;
        case 8: return hp.slot_cap;
        case 9: return hp.block != nullptr ? plx::hub::kHubStreams : 0;
        default: return -1;
    }
}

int plx_spmm_plan_hub_tables_host(const plx_spmm_plan *plan, int wide, int32_t *hub_row_host, int32_t *rows_host, int32_t *row_slot_first_host,
                                  int32_t *row_slots_host, int64_t *stream_first_host, int32_t *stream_total_host, int32_t *stream_pos_host,
                                  uint8_t *stream_run_host, int32_t *stream_mark_host)
{
    PLX_REQUIRE(plan != nullptr, "plan_hub_tables_host: plan is NULL");
    const plx::hub::HubPlan &hp = wide ? plan->hub_wide : plan->hub;
    PLX_REQUIRE(hp.block != nullptr, "plan_hub_tables_host: the plan has no hub tables in that layout");
    const size_t streams = (size_t)plx::hub::kHubStreams;
    auto get = [](void *dst, const void *src, size_t bytes) { return (dst == nullptr || bytes == 0) ? hipSuccess : hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost); };
    PLX_HIP_CHECK(get(hub_row_host, hp.hub_row, sizeof(int32_t) * (size_t)hp.slot_cap));
    PLX_HIP_CHECK(get(rows_host, hp.rows, sizeof(int32_t) * (size_t)hp.n_rows));
    PLX_HIP_CHECK(get(row_slot_first_host, hp.row_slot_first, sizeof(int32_t) * ((size_t)hp.n_rows + 1)));
    PLX_HIP_CHECK(get(row_slots_host, hp.row_slots, sizeof(int32_t) * (size_t)hp.n_slots));
    PLX_HIP_CHECK(get(stream_first_host, hp.stream_first, sizeof(int64_t) * streams));
    PLX_HIP_CHECK(get(stream_total_host, hp.stream_total, sizeof(int32_t) * streams));
    PLX_HIP_CHECK(get(stream_pos_host, hp.stream_pos, sizeof(int32_t) * (size_t)hp.stored));
    PLX_HIP_CHECK(get(stream_run_host, hp.stream_run, (size_t)hp.stored));
    PLX_HIP_CHECK(get(stream_mark_host, hp.stream_mark, sizeof(int32_t) * streams * (size_t)hp.windows_per_range));
    return PLX_OK;
}

// The room for the line-aligned copy of H is decided for contiguous rows of the element type (an operand laid out
// otherwise is staged only if it fits what the caller brought).
size_t plx_spmm_workspace_bytes(const plx_spmm_plan *plan, int64_t D) { return workspace_need(plan, D, 4); }
size_t plx_spmm_workspace_bytes_bf16(const plx_spmm_plan *plan, int64_t D) { return workspace_need(plan, D, 2); }

int plx_spmm_plan_set_slicing(plx_spmm_plan *plan, int mode)
{
    PLX_REQUIRE(plan != nullptr, "plan_set_slicing: plan is NULL");
    PLX_REQUIRE(mode >= -1 && mode <= 1, "plan_set_slicing: mode must be -1, 0 or 1");
    plan->slicing = mode;
    return PLX_OK;
}

int plx_spmm_csr_f32(const plx_spmm_plan *plan, const float *val, const float *H, int64_t ldh, int64_t D, float *Y,
                     int64_t ldy, void *workspace, size_t workspace_bytes, void *stream)
{
    return spmm_impl<float>(plan, 0, plan ? plan->M : 0, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream);
}

int plx_spmm_csr_rows_f32(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, const float *val, const float *H,
                          int64_t ldh, int64_t D, float *Y, int64_t ldy, void *workspace, size_t workspace_bytes,
                          void *stream)
{
    return spmm_impl<float>(plan, row_begin, row_end, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream);
}

int plx_spmm_csr_chunk_f32(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, int first_chunk, const float *val, const float *H,
                           int64_t ldh, int64_t D, float *Y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream)
{
    return spmm_impl<float>(plan, row_begin, row_end, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream, true, 3, first_chunk ? 1 : 2);
}

size_t plx_spmm_static_scratch_bytes(void) { return kStaticScratchBytes; }

int plx_spmm_csr_f32_static(const plx_spmm_plan *plan, const float *val, const float *H, int64_t ldh, int64_t D, float *Y,
                            int64_t ldy, void *stream)
{
    PLX_REQUIRE(plan != nullptr, "spmm_static: plan is NULL");
    PLX_REQUIRE(D >= 0 && D <= (1ll << 21), "spmm_static: bad feature width D=%lld (at most 2,097,152)", (long long)D);
    const size_t need = (size_t)plan->n_seg * (size_t)ws_ld(D) * sizeof(float);
    if (need > kStaticScratchBytes)
        return plx::fail(PLX_ERR_WORKSPACE,
                         "spmm_static: the %lld segments of the split rows need %zu bytes of partial sums at D=%lld, the static "
                         "scratch holds %zu; use plx_spmm_csr_f32 with a workspace",
                         (long long)plan->n_seg, need, (long long)D, kStaticScratchBytes);
    void *ptr = nullptr;
    const int rc = static_scratch(&ptr);
    if (rc != PLX_OK) return rc;
    // every partial row is written in full (columns < D) by its segment task before the reduction reads it, so nothing
    // of an earlier call has to be cleared
    return spmm_impl<float>(plan, 0, plan->M, val, H, ldh, D, Y, ldy, ptr, kStaticScratchBytes, stream, /*may_stage=*/false);
}

int plx_diag_spmm_parts_f32(const plx_spmm_plan *plan, const float *val, const float *H, int64_t ldh, int64_t D, float *Y, int64_t ldy,
                            void *workspace, size_t workspace_bytes, int parts, void *stream)
{
    PLX_REQUIRE(parts >= 1 && parts <= 3, "diag_spmm_parts: parts must be 1 (row kernel), 2 (hub pass) or 3 (both)");
    PLX_REQUIRE(plan != nullptr, "diag_spmm_parts: plan is NULL");
    return spmm_impl<float>(plan, 0, plan->M, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream, true, parts);
}

int plx_diag_random_gather_f32(const float *table, int64_t rows, int64_t ld, int64_t D, int64_t n_gathers, int64_t *gathers_done,
                               float *sink, void *stream)
{
    PLX_REQUIRE(table && sink && gathers_done, "random_gather: NULL argument");
    PLX_REQUIRE(rows >= 1 && rows < (1ll << 32) && ld >= D && ld % 4 == 0 && reinterpret_cast<uintptr_t>(table) % 16 == 0,
                "random_gather: bad table shape or alignment");
    PLX_REQUIRE(D == 16 || D == 32 || D == 64 || D == 128 || D == 256, "random_gather: D must be 16, 32, 64, 128 or 256");
    const int lpr = (int)(D / 4);
    const int gpi = kWave / lpr;                 // rows per wavefront instruction
    const int64_t waves = 256ll * 32 * 4;        // 32 workgroups of 4 wavefronts per compute unit
    int64_t iters = std::max<int64_t>(8, n_gathers / (waves * gpi) / 8 * 8);
    PLX_REQUIRE(iters < (1ll << 30), "random_gather: too many gathers");
    *gathers_done = waves * gpi * iters;
    hipStream_t st = plx::as_stream(stream);
    const unsigned blocks = (unsigned)(waves / 4);
    const float4 *t4 = reinterpret_cast<const float4 *>(table);
    switch (lpr) {
        case 4: random_gather_kernel<4><<<blocks, 256, 0, st>>>(t4, (uint32_t)rows, ld / 4, (int)iters, sink); break;
        case 8: random_gather_kernel<8><<<blocks, 256, 0, st>>>(t4, (uint32_t)rows, ld / 4, (int)iters, sink); break;
        case 16: random_gather_kernel<16><<<blocks, 256, 0, st>>>(t4, (uint32_t)rows, ld / 4, (int)iters, sink); break;
        case 32: random_gather_kernel<32><<<blocks, 256, 0, st>>>(t4, (uint32_t)rows, ld / 4, (int)iters, sink); break;
        default: random_gather_kernel<64><<<blocks, 256, 0, st>>>(t4, (uint32_t)rows, ld / 4, (int)iters, sink); break;
    }
    PLX_LAUNCH_CHECK("random_gather_kernel");
    return PLX_OK;
}

int plx_spmm_csr_bf16(const plx_spmm_plan *plan, const float *val, const uint16_t *H, int64_t ldh, int64_t D,
                      uint16_t *Y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream)
{
    return spmm_impl<uint16_t>(plan, 0, plan ? plan->M : 0, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream);
}

int plx_spmm_csr_rows_bf16(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, const float *val, const uint16_t *H,
                           int64_t ldh, int64_t D, uint16_t *Y, int64_t ldy, void *workspace, size_t workspace_bytes,
                           void *stream)
{
    return spmm_impl<uint16_t>(plan, row_begin, row_end, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream);
}

int plx_spmm_csr_chunk_bf16(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, int first_chunk, const float *val,
                            const uint16_t *H, int64_t ldh, int64_t D, uint16_t *Y, int64_t ldy, void *workspace, size_t workspace_bytes,
                            void *stream)
{
    return spmm_impl<uint16_t>(plan, row_begin, row_end, val, H, ldh, D, Y, ldy, workspace, workspace_bytes, stream, true, 3, first_chunk ? 1 : 2);
}

}  // extern "C"
