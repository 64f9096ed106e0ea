// Dense products of the GCN layer on the gfx950 matrix cores, fp32 in / fp32 accumulate.
//
//   NN  C[M x N] = A[M x K] . B[K x N]            OUT      = AGG . W
//   NT  C[M x N] = (A*mask)[M x K] . B[N x K]^T   GRAD_AGG = GRAD_OUT . W^T
//   TN  C[K x N] = A[M x K]^T . (B*mask)[M x N]   GRAD_W   = AGG^T . GRAD_OUT   (split over M)
//
// All three are "tall-skinny": one dimension is the node count (millions), the others are feature
// widths (tens to hundreds).  One kernel template covers them.  A workgroup of four wavefronts owns
// a 128 x BN output tile (each wavefront 32 x BN = TN tiles of v_mfma_f32_32x32x2_f32) and walks
// the contraction in chunks of 32.  Chunks are fetched global -> registers -> LDS with two LDS
// buffers, so the fetch of chunk c+1 overlaps the MFMAs of chunk c.
//
// LDS tile layouts are chosen so that the global side is always read along contiguous memory:
//   "x-major"  T[x][k] (row stride 36 floats): rows of the source are rows of the tile; a lane reads
//              four consecutive k with one 128-bit LDS load;
//   "k-major"  T[k][x]: the source is already contraction-major (B of NN, both operands of TN); a
//              lane reads single floats, consecutive lanes consecutive x.
// Both layouts agree on which k a lane feeds to MFMA number (s, m) of a chunk: k = 8 s + 4 h + m with
// h = lane / 32, which is a permutation of the chunk and therefore leaves the product unchanged.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "common.h"

#ifndef PLX_GEMM_LEAN
#define PLX_GEMM_LEAN 1  // 0: always use the general kernel (for A/B timing)
#endif

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 128;   // output rows per workgroup
constexpr int kBK = 32;    // contraction chunk
constexpr int kXS = 36;    // row stride of an x-major tile (floats)
constexpr int kThreads = 256;

enum Mode { kNN = 0, kNT = 1, kTN = 2 };

struct GemmArgs {
    const float *A;
    const float *B;
    float *C;
    const float *mask;
    int64_t lda, ldb, ldc, ldmask;
    int64_t M, N, K;       // as in the header of each entry point
    int64_t rows_per_split;  // TN only
    float *ws;             // TN only: partial tiles [split][Kpad][Npad]
    int64_t ws_ld, ws_slab;
    unsigned flags;
    float alpha;           // NN / NT: C = epilogue(alpha * product)
    int a_vec, b_vec, m_vec;  // 1 when 128-bit global loads of that operand are legal
    // when set, the launch does nothing unless one of these n_run_if device words (a few at most) is non-zero: the
    // fp32 redo of a split product whose operands turned out to hold Inf / NaN
    const unsigned *run_if;
    int n_run_if;
};

__device__ __forceinline__ bool guard_says_skip(const GemmArgs &g)
{
    if (g.run_if == nullptr) return false;
    unsigned any = 0;
    for (int i = 0; i < g.n_run_if; ++i) any |= g.run_if[i];
    return any == 0;
}

// ROWS x COLS tile of a row-major source, fetched as float4 per thread, zero-filled outside the source
template <int ROWS, int COLS, int STRIDE>
struct Tile {
    static constexpr int kV4PerRow = COLS / 4;
    static constexpr int kPer = ROWS * COLS / 4 / kThreads;
    static_assert(ROWS * COLS / 4 % kThreads == 0 && kPer >= 1, "tile does not divide over the workgroup");
    float4 reg[kPer];

    __device__ __forceinline__ void fetch(const float *__restrict__ src, int64_t ld, int64_t r0, int64_t c0, int64_t nrows,
                                          int64_t ncols, int vec_ok, const float *__restrict__ mask, int64_t ldm,
                                          int mvec_ok)
    {
#pragma unroll
        for (int p = 0; p < kPer; ++p) {
            const int idx = p * kThreads + threadIdx.x;
            const int64_t r = r0 + idx / kV4PerRow;
            const int64_t c = c0 + (idx % kV4PerRow) * 4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r < nrows && c < ncols) {
                const float *q = src + r * ld + c;
                if (vec_ok && c + 3 < ncols) {
                    v = *reinterpret_cast<const float4 *>(q);
                } else {
                    v.x = q[0];
                    if (c + 1 < ncols) v.y = q[1];
                    if (c + 2 < ncols) v.z = q[2];
                    if (c + 3 < ncols) v.w = q[3];
                }
                if (mask != nullptr) {
                    const float *mq = mask + r * ldm + c;
                    float4 m = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (mvec_ok && c + 3 < ncols) {
                        m = *reinterpret_cast<const float4 *>(mq);
                    } else {
                        m.x = mq[0];
                        if (c + 1 < ncols) m.y = mq[1];
                        if (c + 2 < ncols) m.z = mq[2];
                        if (c + 3 < ncols) m.w = mq[3];
                    }
                    v.x = m.x > 0.f ? v.x : 0.f;
                    v.y = m.y > 0.f ? v.y : 0.f;
                    v.z = m.z > 0.f ? v.z : 0.f;
                    v.w = m.w > 0.f ? v.w : 0.f;
                }
            }
            reg[p] = v;
        }
    }

    __device__ __forceinline__ void stash(float *lds) const
    {
#pragma unroll
        for (int p = 0; p < kPer; ++p) {
            const int idx = p * kThreads + threadIdx.x;
            const int r = idx / kV4PerRow;
            const int c = (idx % kV4PerRow) * 4;
            *reinterpret_cast<float4 *>(lds + r * STRIDE + c) = reg[p];
        }
    }
};

// Second level of the sum over rows in the TN product.  ON = false: no state, no code.
constexpr int kFlushChunks = 8;  // 8 chunks of 32 rows = 128 accumulation steps of the 32x32x2 MFMA
template <bool ON, int TN>
struct TotalsTN {
    __device__ __forceinline__ void chunk_done(floatx16 (&)[TN], int &) {}
    __device__ __forceinline__ void finish(floatx16 (&)[TN]) {}
};
template <int TN>
struct TotalsTN<true, TN> {
    float tot[TN][16];
    __device__ __forceinline__ TotalsTN()
    {
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) tot[t][v] = 0.f;
    }
    __device__ __forceinline__ void flush(floatx16 (&acc)[TN])
    {
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                tot[t][v] += acc[t][v];
                acc[t][v] = 0.f;
            }
    }
    __device__ __forceinline__ void chunk_done(floatx16 (&acc)[TN], int &since_flush)
    {
        if (++since_flush == kFlushChunks) {  // uniform over the workgroup
            since_flush = 0;
            flush(acc);
        }
    }
    // leaves the totals in acc for the common store code
    __device__ __forceinline__ void finish(floatx16 (&acc)[TN])
    {
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[t][v] += tot[t][v];
    }
};

// one output tile; `bx` is the workgroup's first grid coordinate (row tile of NN / NT, stretch of rows of TN)
template <int MODE, int TN>
__device__ __forceinline__ void gemm_f32_tile(const GemmArgs &g, float *lds, const int64_t bx)
{
    constexpr int BN = 32 * TN;
    constexpr bool kAX = (MODE != kTN);  // A tile x-major?
    constexpr bool kBX = (MODE == kNT);  // B tile x-major?
    constexpr int kAStride = kAX ? kXS : kBM;
    constexpr int kBStride = kBX ? kXS : BN;
    constexpr int kASize = kAX ? kBM * kXS : kBK * kBM;
    constexpr int kBSize = kBX ? BN * kXS : kBK * BN;
    using ATile = Tile<(kAX ? kBM : kBK), (kAX ? kBK : kBM), kAStride>;
    using BTile = Tile<(kBX ? BN : kBK), (kBX ? kBK : BN), kBStride>;

    auto a_buf = [&](int i) { return lds + i * kASize; };
    auto b_buf = [&](int i) { return lds + 2 * kASize + i * kBSize; };

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 31;
    const int h = lane >> 5;

    // output tile origin and contraction range
    int64_t row0, col0, kbeg, kend;
    if constexpr (MODE == kTN) {
        row0 = (int64_t)blockIdx.y * kBM;  // rows of C = columns of A
        col0 = (int64_t)blockIdx.z * BN;
        kbeg = bx * g.rows_per_split;
        kend = min(kbeg + g.rows_per_split, g.M);
    } else {
        row0 = bx * kBM;
        col0 = (int64_t)blockIdx.y * BN;
        kbeg = 0;
        kend = g.K;
    }

    ATile at;
    BTile bt;
    auto fetch = [&](int64_t k0) {
        if constexpr (MODE == kNN) {
            at.fetch(g.A, g.lda, row0, k0, g.M, g.K, g.a_vec, nullptr, 0, 0);
            bt.fetch(g.B, g.ldb, k0, col0, g.K, g.N, g.b_vec, nullptr, 0, 0);
        } else if constexpr (MODE == kNT) {
            at.fetch(g.A, g.lda, row0, k0, g.M, g.K, g.a_vec, g.mask, g.ldmask, g.m_vec);
            bt.fetch(g.B, g.ldb, col0, k0, g.N, g.K, g.b_vec, nullptr, 0, 0);
        } else {
            at.fetch(g.A, g.lda, k0, row0, kend, g.K, g.a_vec, nullptr, 0, 0);
            bt.fetch(g.B, g.ldb, k0, col0, kend, g.N, g.b_vec, g.mask, g.ldmask, g.m_vec);
        }
    };

    floatx16 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

    // TN sums over the rows of the matrices, thousands of them per workgroup: every kFlushChunks chunks the accumulators
    // of the matrix cores are added into a second set of totals and cleared, so that the rounding error grows with
    // sqrt(kFlushChunks * 16) + sqrt(chunks / kFlushChunks) steps instead of sqrt(chunks * 16)
    TotalsTN<MODE == kTN, TN> tot;

    int buf = 0;
    if (kbeg < kend) {
        fetch(kbeg);
        at.stash(a_buf(0));
        bt.stash(b_buf(0));
    }
    __syncthreads();

    int since_flush = 0;
    for (int64_t k0 = kbeg; k0 < kend; k0 += kBK) {
        const bool more = k0 + kBK < kend;
        if (more) fetch(k0 + kBK);

        const float *as = a_buf(buf);
        const float *bs = b_buf(buf);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            float a[4];
            if constexpr (kAX) {
                const float4 t4 = *reinterpret_cast<const float4 *>(as + (wave * 32 + li) * kXS + 8 * s + 4 * h);
                a[0] = t4.x;
                a[1] = t4.y;
                a[2] = t4.z;
                a[3] = t4.w;
            } else {
#pragma unroll
                for (int m = 0; m < 4; ++m) a[m] = as[(8 * s + 4 * h + m) * kAStride + wave * 32 + li];
            }
            float b[TN][4];
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                if constexpr (kBX) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(bs + (t * 32 + li) * kXS + 8 * s + 4 * h);
                    b[t][0] = t4.x;
                    b[t][1] = t4.y;
                    b[t][2] = t4.z;
                    b[t][3] = t4.w;
                } else {
#pragma unroll
                    for (int m = 0; m < 4; ++m) b[t][m] = bs[(8 * s + 4 * h + m) * kBStride + t * 32 + li];
                }
            }
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[m], b[t][m], acc[t], 0, 0, 0);
        }

        if (more) {
            at.stash(a_buf(buf ^ 1));
            bt.stash(b_buf(buf ^ 1));
        }
        tot.chunk_done(acc, since_flush);
        __syncthreads();
        buf ^= 1;
    }
    tot.finish(acc);

    // accumulator register v of a lane is C[8 (v / 4) + 4 h + v % 4][lane % 32] of the 32 x 32 tile
    float *out;
    int64_t ldo, nrows, ncols;
    if constexpr (MODE == kTN) {
        if (g.ws != nullptr) {
            out = g.ws + bx * g.ws_slab;
            ldo = g.ws_ld;
        } else {
            out = g.C;
            ldo = g.ldc;
        }
        nrows = g.K;
        ncols = g.N;
    } else {
        out = g.C;
        ldo = g.ldc;
        nrows = g.M;
        ncols = g.N;
    }
    const bool relu = (g.flags & PLX_GEMM_RELU) != 0;
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        const int64_t c = col0 + t * 32 + li;
        if (c >= ncols) continue;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t r = row0 + wave * 32 + 8 * (v / 4) + 4 * h + (v % 4);
            if (r < nrows) {
                float x = acc[t][v];
                if (MODE != kTN || g.ws == nullptr) x *= g.alpha;  // partial tiles are scaled when they are added up
                if (relu) x = fmaxf(x, 0.f);
                out[r * ldo + c] = x;
            }
        }
    }
}

// NN / NT: a workgroup walks the row tiles bx, bx + gridDim.x, ... (one each unless the launch is a guarded one, whose grid
// is small so that it costs little when it has nothing to do); TN: one stretch of rows per workgroup
template <int MODE, int TN>
__global__ void __launch_bounds__(kThreads) gemm_f32_kernel(const GemmArgs g)
{
    constexpr int BN = 32 * TN;
    constexpr int kASize = (MODE != kTN) ? kBM * kXS : kBK * kBM;
    constexpr int kBSize = (MODE == kNT) ? BN * kXS : kBK * BN;
    __shared__ __attribute__((aligned(16))) float lds[2 * (kASize + kBSize)];
    if (guard_says_skip(g)) return;
    if constexpr (MODE == kTN) {
        gemm_f32_tile<MODE, TN>(g, lds, (int64_t)blockIdx.x);
    } else {
        const int64_t row_tiles = (g.M + kBM - 1) / kBM;
        for (int64_t bx = blockIdx.x; bx < row_tiles; bx += gridDim.x) {
            gemm_f32_tile<MODE, TN>(g, lds, bx);
            __syncthreads();  // the next tile's first chunk overwrites the buffers
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Lean variant for aligned operands (every base 16-byte aligned, every leading dimension and the
// contraction / column extents multiples of 4).  Same tiling and LDS layouts as gemm_f32_kernel; the
// difference is the cost of a fetch: one 64-bit multiply per thread and tile, then pointer steps and
// 32-bit compares.  In the general kernel the per-element guards and 64-bit address products amount to
// ~8 vector-ALU instructions per MFMA, which is what keeps its MFMA pipe half idle.
// ---------------------------------------------------------------------------------------------------
template <int MODE, int TN, bool MASKED>
__device__ __forceinline__ void gemm_f32_vec_tile(const GemmArgs &g, float *lds, const int64_t bx)
{
    constexpr int BN = 32 * TN;
    constexpr bool kAX = (MODE != kTN);
    constexpr bool kBX = (MODE == kNT);
    constexpr int kAStride = kAX ? kXS : kBM;
    constexpr int kBStride = kBX ? kXS : BN;
    constexpr int kASize = kAX ? kBM * kXS : kBK * kBM;
    constexpr int kBSize = kBX ? BN * kXS : kBK * BN;
    // float4 per tile row and rows covered by one pass of the 256 threads
    constexpr int kAV = (kAX ? kBK : kBM) / 4, kARows = kAX ? kBM : kBK, kAPass = kThreads / kAV;
    constexpr int kBV = (kBX ? kBK : BN) / 4, kBRows = kBX ? BN : kBK, kBPass = kThreads / kBV;
    constexpr int kAPer = (kARows + kAPass - 1) / kAPass, kBPer = (kBRows + kBPass - 1) / kBPass;


    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 31;
    const int h = lane >> 5;

    int64_t row0, col0, kbeg, kend;
    if constexpr (MODE == kTN) {
        row0 = (int64_t)blockIdx.y * kBM;
        col0 = (int64_t)blockIdx.z * BN;
        kbeg = bx * g.rows_per_split;
        kend = min(kbeg + g.rows_per_split, g.M);
    } else {
        row0 = bx * kBM;
        col0 = (int64_t)blockIdx.y * BN;
        kbeg = 0;
        kend = g.K;
    }

    // thread coordinates inside the A and B tiles: (row of the first pass, float4 index in the row)
    const int ar = threadIdx.x / kAV, av = (threadIdx.x % kAV) * 4;
    const int br = threadIdx.x / kBV, bv = (threadIdx.x % kBV) * 4;
    // source row / column of element (0, 0) of each tile at contraction offset kbeg, and the extents left
    const float *pa, *pb, *pm = nullptr;
    int64_t a_step, b_step, m_step = 0;  // pointer advance per pass (rows of the tile)
    int64_t a_adv, b_adv, m_adv = 0;     // pointer advance per chunk
    int a_rows_left, a_cols_left, b_rows_left, b_cols_left;  // relative to this thread's first element
    if constexpr (MODE == kNN) {
        pa = g.A + (row0 + ar) * g.lda + av;             a_step = (int64_t)kAPass * g.lda; a_adv = kBK;
        pb = g.B + (int64_t)br * g.ldb + col0 + bv;      b_step = (int64_t)kBPass * g.ldb; b_adv = (int64_t)kBK * g.ldb;
        a_rows_left = (int)min(max(g.M - row0 - ar, (int64_t)0), (int64_t)kBM);  a_cols_left = (int)min(g.K - av, (int64_t)1 << 30);
        b_rows_left = (int)min(g.K - br, (int64_t)1 << 30);                       b_cols_left = (int)min(max(g.N - col0 - bv, (int64_t)0), (int64_t)BN);
    } else if constexpr (MODE == kNT) {
        pa = g.A + (row0 + ar) * g.lda + av;             a_step = (int64_t)kAPass * g.lda; a_adv = kBK;
        if constexpr (MASKED) { pm = g.mask + (row0 + ar) * g.ldmask + av; m_step = (int64_t)kAPass * g.ldmask; m_adv = kBK; }
        pb = g.B + (col0 + br) * g.ldb + bv;             b_step = (int64_t)kBPass * g.ldb; b_adv = kBK;
        a_rows_left = (int)min(max(g.M - row0 - ar, (int64_t)0), (int64_t)kBM);  a_cols_left = (int)min(g.K - av, (int64_t)1 << 30);
        b_rows_left = (int)min(max(g.N - col0 - br, (int64_t)0), (int64_t)BN);   b_cols_left = (int)min(g.K - bv, (int64_t)1 << 30);
    } else {
        pa = g.A + (kbeg + ar) * g.lda + row0 + av;      a_step = (int64_t)kAPass * g.lda; a_adv = (int64_t)kBK * g.lda;
        pb = g.B + (kbeg + br) * g.ldb + col0 + bv;      b_step = (int64_t)kBPass * g.ldb; b_adv = (int64_t)kBK * g.ldb;
        if constexpr (MASKED) { pm = g.mask + (kbeg + br) * g.ldmask + col0 + bv; m_step = (int64_t)kBPass * g.ldmask; m_adv = (int64_t)kBK * g.ldmask; }
        a_rows_left = (int)min(kend - kbeg - ar, (int64_t)1 << 30);  a_cols_left = (int)min(max(g.K - row0 - av, (int64_t)0), (int64_t)kBM);
        b_rows_left = (int)min(kend - kbeg - br, (int64_t)1 << 30);  b_cols_left = (int)min(max(g.N - col0 - bv, (int64_t)0), (int64_t)BN);
    }
    // which of (rows, cols) shrinks as the contraction advances
    constexpr bool kAContrRows = (MODE == kTN);            // A tile rows are contraction indices (k-major)
    constexpr bool kBContrRows = (MODE != kNT);            // B tile rows are contraction indices

    // a mask travels beside its chunk and is applied when the chunk is stored to LDS, so that a fetch only issues loads
    constexpr int kMPer = !MASKED ? 1 : (MODE == kNT ? kAPer : kBPer);
    float4 ra[kAPer], rb[kBPer], rmask[kMPer];
    auto masked = [](float4 v, float4 m) {
        return make_float4(m.x > 0.f ? v.x : 0.f, m.y > 0.f ? v.y : 0.f, m.z > 0.f ? v.z : 0.f, m.w > 0.f ? v.w : 0.f);
    };
    auto fetch = [&]() {
        {
            const float *q = pa;
            const float *mq = pm;
#pragma unroll
            for (int p = 0; p < kAPer; ++p) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (p * kAPass < a_rows_left && a_cols_left > 0 && (kARows % kAPass == 0 || ar + p * kAPass < kARows)) {
                    v = *reinterpret_cast<const float4 *>(q);
                    if constexpr (MASKED && MODE == kNT) rmask[p] = *reinterpret_cast<const float4 *>(mq);
                } else if constexpr (MASKED && MODE == kNT) {
                    rmask[p] = v;
                }
                ra[p] = v;
                q += a_step;
                if constexpr (MASKED && MODE == kNT) mq += m_step;
            }
        }
        {
            const float *q = pb;
            const float *mq = pm;
#pragma unroll
            for (int p = 0; p < kBPer; ++p) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (p * kBPass < b_rows_left && b_cols_left > 0 && (kBRows % kBPass == 0 || br + p * kBPass < kBRows)) {
                    v = *reinterpret_cast<const float4 *>(q);
                    if constexpr (MASKED && MODE == kTN) rmask[p] = *reinterpret_cast<const float4 *>(mq);
                } else if constexpr (MASKED && MODE == kTN) {
                    rmask[p] = v;
                }
                rb[p] = v;
                q += b_step;
                if constexpr (MASKED && MODE == kTN) mq += m_step;
            }
        }
        // advance to the next chunk
        pa += a_adv;
        pb += b_adv;
        if constexpr (MASKED) pm += m_adv;
        if constexpr (kAContrRows) a_rows_left -= kBK; else a_cols_left -= kBK;
        if constexpr (kBContrRows) b_rows_left -= kBK; else b_cols_left -= kBK;
    };
    const int a_st = ar * kAStride + av, b_st = br * kBStride + bv;
    auto stash = [&](int buf) {
        float *as = lds + buf * kASize + a_st;
        float *bs = lds + 2 * kASize + buf * kBSize + b_st;
#pragma unroll
        for (int p = 0; p < kAPer; ++p)
            if (kARows % kAPass == 0 || ar + p * kAPass < kARows)
                *reinterpret_cast<float4 *>(as + p * kAPass * kAStride) = (MASKED && MODE == kNT) ? masked(ra[p], rmask[MASKED && MODE == kNT ? p : 0]) : ra[p];
#pragma unroll
        for (int p = 0; p < kBPer; ++p)
            if (kBRows % kBPass == 0 || br + p * kBPass < kBRows)
                *reinterpret_cast<float4 *>(bs + p * kBPass * kBStride) = (MASKED && MODE == kTN) ? masked(rb[p], rmask[MASKED && MODE == kTN ? p : 0]) : rb[p];
    };

    floatx16 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

    TotalsTN<MODE == kTN, TN> tot;  // second-level totals of the long sum over rows (see gemm_f32_kernel)
    int since_flush = 0;
    int buf = 0;
    if (kbeg < kend) {
        fetch();
        stash(0);
    }
    __syncthreads();
    for (int64_t k0 = kbeg; k0 < kend; k0 += kBK) {
        const bool more = k0 + kBK < kend;
        if (more) fetch();
        const float *as = lds + buf * kASize;
        const float *bs = lds + 2 * kASize + buf * kBSize;
#pragma unroll
        for (int s = 0; s < kBK / 8; ++s) {
            float a[4];
            if constexpr (kAX) {
                const float4 t4 = *reinterpret_cast<const float4 *>(as + (wave * 32 + li) * kXS + 8 * s + 4 * h);
                a[0] = t4.x; a[1] = t4.y; a[2] = t4.z; a[3] = t4.w;
            } else {
#pragma unroll
                for (int m = 0; m < 4; ++m) a[m] = as[(8 * s + 4 * h + m) * kAStride + wave * 32 + li];
            }
            float b[TN][4];
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                if constexpr (kBX) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(bs + (t * 32 + li) * kXS + 8 * s + 4 * h);
                    b[t][0] = t4.x; b[t][1] = t4.y; b[t][2] = t4.z; b[t][3] = t4.w;
                } else {
#pragma unroll
                    for (int m = 0; m < 4; ++m) b[t][m] = bs[(8 * s + 4 * h + m) * kBStride + t * 32 + li];
                }
            }
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[m], b[t][m], acc[t], 0, 0, 0);
        }
        if (more) stash(buf ^ 1);
        tot.chunk_done(acc, since_flush);
        __syncthreads();
        buf ^= 1;
    }
    tot.finish(acc);

    float *out;
    int64_t ldo, nrows, ncols;
    if constexpr (MODE == kTN) {
        if (g.ws != nullptr) {
            out = g.ws + bx * g.ws_slab;
            ldo = g.ws_ld;
        } else {
            out = g.C;
            ldo = g.ldc;
        }
        nrows = g.K;
        ncols = g.N;
    } else {
        out = g.C;
        ldo = g.ldc;
        nrows = g.M;
        ncols = g.N;
    }
    const bool relu = (g.flags & PLX_GEMM_RELU) != 0;
    const int64_t rbase = row0 + wave * 32 + 4 * h;
    const int rows_left = (int)min(max(nrows - rbase, (int64_t)0), (int64_t)64);
    const int cols_left = (int)min(max(ncols - col0 - li, (int64_t)0), (int64_t)BN);
    float *prow = out + rbase * ldo + col0 + li;
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
#pragma unroll
        for (int vv = 0; vv < 4; ++vv) {
            if (8 * v4 + vv < rows_left) {
                float *q = prow + (int64_t)(8 * v4 + vv) * ldo;
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    float x = acc[t][4 * v4 + vv];
                    if (MODE != kTN || g.ws == nullptr) x *= g.alpha;  // partial tiles are scaled when they are added up
                    if (relu) x = fmaxf(x, 0.f);
                    if (t * 32 < cols_left) q[t * 32] = x;
                }
            }
        }
    }
}

template <int MODE, int TN, bool MASKED>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) gemm_f32_vec_kernel(const GemmArgs g)
{
    constexpr int BN = 32 * TN;
    constexpr int kASize = (MODE != kTN) ? kBM * kXS : kBK * kBM;
    constexpr int kBSize = (MODE == kNT) ? BN * kXS : kBK * BN;
    __shared__ __attribute__((aligned(16))) float lds[2 * (kASize + kBSize)];
    if (guard_says_skip(g)) return;
    if constexpr (MODE == kTN) {
        gemm_f32_vec_tile<MODE, TN, MASKED>(g, lds, (int64_t)blockIdx.x);
    } else {
        const int64_t row_tiles = (g.M + kBM - 1) / kBM;
        for (int64_t bx = blockIdx.x; bx < row_tiles; bx += gridDim.x) {
            gemm_f32_vec_tile<MODE, TN, MASKED>(g, lds, bx);
            __syncthreads();  // the next tile's first chunk overwrites the buffers
        }
    }
}

// C[e] = sum over splits of ws[s][e], s ascending within four interleaved chains that are then
// added in chain order -- a fixed order, so the result does not depend on scheduling.
__global__ void __launch_bounds__(256) gemm_tn_reduce(const float *__restrict__ ws, int64_t ws_ld, int64_t ws_slab,
                                                      int splits, int64_t rows, int64_t cols, float *__restrict__ C,
                                                      int64_t ldc, double alpha, const unsigned *__restrict__ run_if)
{
    if (run_if != nullptr && *run_if == 0u) return;  // the guarded redo of a split product: nothing to add up
    // 16 output elements per workgroup, 16 interleaved chains per element (chain j adds the partial tiles
    // j, j + 16, ... in order); the chains are then added in chain order: the same sum whatever the timing
    __shared__ double part[16][17];
    const int e_local = threadIdx.x & 15;
    const int chain = threadIdx.x >> 4;
    const int64_t e = (int64_t)blockIdx.x * 16 + e_local;
    const int64_t total = rows * cols;
    double s = 0.0;  // the partial tiles are added in fp64 and the sum is rounded once
    int64_t r = 0, c = 0;
    if (e < total) {
        r = e / cols;
        c = e % cols;
        const float *p = ws + r * ws_ld + c + (int64_t)chain * ws_slab;
        const int64_t step = 16 * ws_slab;
        int i = chain;
        for (; i + 48 < splits; i += 64) {  // four loads in flight per chain
            const float v0 = p[0], v1 = p[step], v2 = p[2 * step], v3 = p[3 * step];
            s = (((s + (double)v0) + (double)v1) + (double)v2) + (double)v3;
            p += 4 * step;
        }
        for (; i < splits; i += 16) {
            s += (double)p[0];
            p += step;
        }
    }
    part[chain][e_local] = s;
    __syncthreads();
    if (chain == 0 && e < total) {
        double t = part[0][e_local];
#pragma unroll
        for (int j = 1; j < 16; ++j) t += part[j][e_local];
        C[r * ldc + c] = (float)(t * alpha);  // alpha = 1 changes nothing
    }
}

int vec_ok(const float *p, int64_t ld) { return (p == nullptr || (reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0)) ? 1 : 0; }

int pick_tn(int64_t n) { return n <= 32 ? 1 : (n <= 64 ? 2 : 4); }

template <int MODE, bool MASKED>
void launch_vec(const GemmArgs &g, int tn, dim3 grid, hipStream_t st)
{
    switch (tn) {
        case 1: gemm_f32_vec_kernel<MODE, 1, MASKED><<<grid, kThreads, 0, st>>>(g); break;
        case 2: gemm_f32_vec_kernel<MODE, 2, MASKED><<<grid, kThreads, 0, st>>>(g); break;
        default: gemm_f32_vec_kernel<MODE, 4, MASKED><<<grid, kThreads, 0, st>>>(g); break;
    }
}

template <int MODE>
void launch_gemm(const GemmArgs &g, int tn, dim3 grid, hipStream_t st)
{
    // aligned operands and extents that are multiples of 4 -> the lean kernel; anything else -> the general one
    const bool ext4 = (MODE == kTN) ? (g.K % 4 == 0 && g.N % 4 == 0) : (MODE == kNN ? (g.K % 4 == 0 && g.N % 4 == 0) : g.K % 4 == 0);
    const bool vec = g.a_vec && g.b_vec && (g.mask == nullptr || g.m_vec) && ext4 && PLX_GEMM_LEAN;
    if (vec) {
        if (g.mask != nullptr && MODE != kNN) launch_vec<MODE, true>(g, tn, grid, st);
        else launch_vec<MODE, false>(g, tn, grid, st);
        return;
    }
    switch (tn) {
        case 1: gemm_f32_kernel<MODE, 1><<<grid, kThreads, 0, st>>>(g); break;
        case 2: gemm_f32_kernel<MODE, 2><<<grid, kThreads, 0, st>>>(g); break;
        default: gemm_f32_kernel<MODE, 4><<<grid, kThreads, 0, st>>>(g); break;
    }
}

// Row tiles of an NN / NT launch.  A guarded launch (one that runs only if a split product has raised its flag, which is
// rare) takes a grid of at most 1,024 workgroups that walk the row tiles: 19,000 workgroups that all return at once still
// keep the GPU busy for 15 us.
unsigned guarded_grid(int64_t row_tiles, const unsigned *run_if)
{
    return (unsigned)(run_if != nullptr ? std::min<int64_t>(row_tiles, 1024) : row_tiles);
}

int check_common(const char *who, int64_t M, int64_t N, int64_t K, const void *A, const void *B, const void *C)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && K >= 0, "%s: negative dimension", who);
    PLX_REQUIRE(N < (1ll << 30) && K < (1ll << 30), "%s: dimension too large", who);
    if (M == 0 || N == 0) return 1;
    PLX_REQUIRE(C != nullptr, "%s: NULL output", who);
    PLX_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "%s: NULL operand", who);
    return PLX_OK;
}

// TN split policy: enough workgroups to fill 256 compute units a few times over, at least 256 rows each
int64_t tn_splits(int64_t M, int64_t N, int64_t K)
{
    const int64_t tiles = plx::ceil_div(K, kBM) * plx::ceil_div(N, 32 * pick_tn(N));
    int64_t want = std::max<int64_t>(1, 512 / tiles);
    int64_t by_rows = std::max<int64_t>(1, M / 256);
    return std::max<int64_t>(1, std::min(want, by_rows));
}

int gemm_nn_impl(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                 int64_t ldc, unsigned flags, const unsigned *run_if, int n_run_if, void *stream)
{
    int rc = check_common("gemm_nn", M, N, K, A, B, C);
    if (rc != PLX_OK) return rc < 0 ? rc : PLX_OK;
    PLX_REQUIRE(lda >= K && ldb >= N && ldc >= N, "gemm_nn: leading dimension too small");
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.M = M; g.N = N; g.K = K; g.flags = flags; g.alpha = 1.f;
    g.a_vec = vec_ok(A, lda); g.b_vec = vec_ok(B, ldb);
    g.run_if = run_if; g.n_run_if = n_run_if;
    const int tn = pick_tn(N);
    dim3 grid(guarded_grid(plx::ceil_div(M, kBM), run_if), (unsigned)plx::ceil_div(N, 32 * tn), 1);
    launch_gemm<kNN>(g, tn, grid, plx::as_stream(stream));
    PLX_LAUNCH_CHECK("gemm_f32_kernel<NN>");
    return PLX_OK;
}

int gemm_nt_impl(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                 int64_t ldc, const float *mask, int64_t ldmask, const unsigned *run_if, int n_run_if, void *stream, float alpha = 1.f)
{
    int rc = check_common("gemm_nt", M, N, K, A, B, C);
    if (rc != PLX_OK) return rc < 0 ? rc : PLX_OK;
    PLX_REQUIRE(lda >= K && ldb >= K && ldc >= N, "gemm_nt: leading dimension too small");
    PLX_REQUIRE(mask == nullptr || ldmask >= K, "gemm_nt: mask leading dimension too small");
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.mask = mask; g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldmask = ldmask;
    g.M = M; g.N = N; g.K = K; g.alpha = alpha;
    g.a_vec = vec_ok(A, lda); g.b_vec = vec_ok(B, ldb); g.m_vec = vec_ok(mask, ldmask);
    g.run_if = run_if; g.n_run_if = n_run_if;
    const int tn = pick_tn(N);
    dim3 grid(guarded_grid(plx::ceil_div(M, kBM), run_if), (unsigned)plx::ceil_div(N, 32 * tn), 1);
    launch_gemm<kNT>(g, tn, grid, plx::as_stream(stream));
    PLX_LAUNCH_CHECK("gemm_f32_kernel<NT>");
    return PLX_OK;
}

size_t tn_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const int64_t splits = tn_splits(M, N, K);
    if (splits <= 1) return 0;
    const int64_t ld = (N + 3) / 4 * 4;
    return (size_t)splits * (size_t)K * (size_t)ld * sizeof(float);
}

// run_if != NULL: nothing runs (and C is left alone) unless that device word is non-zero
int gemm_tn_impl(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                 const float *mask, int64_t ldmask, void *workspace, size_t workspace_bytes, const unsigned *run_if, float alpha, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm_tn: negative dimension");
    if (K == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(C != nullptr, "gemm_tn: NULL output");
    PLX_REQUIRE(M == 0 || (A != nullptr && B != nullptr), "gemm_tn: NULL operand");
    PLX_REQUIRE(lda >= K && ldb >= N && ldc >= N, "gemm_tn: leading dimension too small");
    PLX_REQUIRE(mask == nullptr || ldmask >= N, "gemm_tn: mask leading dimension too small");
    hipStream_t st = plx::as_stream(stream);
    const int64_t splits = tn_splits(std::max<int64_t>(M, 1), N, K);
    const size_t need = tn_workspace_bytes(M, N, K);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need))
        return plx::fail(PLX_ERR_WORKSPACE, "gemm_tn: workspace of %zu bytes needed, %zu given", need, workspace_bytes);

    GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.mask = mask; g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldmask = ldmask;
    g.M = M; g.N = N; g.K = K; g.alpha = alpha;
    g.a_vec = vec_ok(A, lda); g.b_vec = vec_ok(B, ldb); g.m_vec = vec_ok(mask, ldmask);
    g.run_if = run_if; g.n_run_if = run_if != nullptr ? 1 : 0;
    // every split covers a multiple of the 32-row chunk so that chunk boundaries do not depend on the split
    g.rows_per_split = plx::ceil_div(plx::ceil_div(std::max<int64_t>(M, 1), splits), kBK) * kBK;
    const int64_t used = plx::ceil_div(std::max<int64_t>(M, 1), g.rows_per_split);
    const bool through_ws = splits > 1;  // else one workgroup per tile writes C itself
    if (through_ws) {
        g.ws = static_cast<float *>(workspace);
        g.ws_ld = (N + 3) / 4 * 4;
        g.ws_slab = K * g.ws_ld;
    }
    const int tn = pick_tn(N);
    dim3 grid((unsigned)used, (unsigned)plx::ceil_div(K, kBM), (unsigned)plx::ceil_div(N, 32 * tn));
    launch_gemm<kTN>(g, tn, grid, st);
    PLX_LAUNCH_CHECK("gemm_f32_kernel<TN>");
    if (through_ws) {
        const int64_t total = K * N;
        gemm_tn_reduce<<<(unsigned)plx::ceil_div(total, 16), 256, 0, st>>>(g.ws, g.ws_ld, g.ws_slab, (int)used, K, N, C, ldc, (double)alpha, run_if);
        PLX_LAUNCH_CHECK("gemm_tn_reduce");
    }
    return PLX_OK;
}

}  // namespace

// the same two products, launched so that they run only if a device flag is set (used by the split products)
namespace plx {
size_t gemm_tn_f32_workspace_bytes(int64_t M, int64_t N, int64_t K) { return tn_workspace_bytes(M, N, K); }
int64_t gemm_tn_f32_splits(int64_t M, int64_t N, int64_t K) { return tn_splits(std::max<int64_t>(M, 1), N, K); }
int gemm_tn_f32_if(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                   const float *mask, int64_t ldmask, void *workspace, size_t workspace_bytes, const unsigned *run_if, float alpha, void *stream)
{
    return gemm_tn_impl(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, workspace, workspace_bytes, run_if, alpha, stream);
}
// C[e] = alpha * (sum over the partial tiles ws[s][e], s < splits), the tiles added in 16 interleaved chains and the
// chains in order, in fp64, rounded once
int gemm_tn_reduce_tiles(const float *ws, int64_t ws_ld, int64_t ws_slab, int splits, int64_t K, int64_t N, float *C, int64_t ldc, float alpha,
                         void *stream)
{
    gemm_tn_reduce<<<(unsigned)ceil_div(K * N, 16), 256, 0, as_stream(stream)>>>(ws, ws_ld, ws_slab, splits, K, N, C, ldc, (double)alpha, nullptr);
    PLX_LAUNCH_CHECK("gemm_tn_reduce");
    return PLX_OK;
}
int gemm_nn_f32_if(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                   int64_t ldc, unsigned flags, const unsigned *run_if, int n_run_if, void *stream)
{
    return gemm_nn_impl(M, N, K, A, lda, B, ldb, C, ldc, flags, run_if, n_run_if, stream);
}
int gemm_nt_f32_if(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                   int64_t ldc, const float *mask, int64_t ldmask, const unsigned *run_if, int n_run_if, void *stream, float alpha)
{
    return gemm_nt_impl(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, run_if, n_run_if, stream, alpha);
}
}  // namespace plx

extern "C" {

int plx_gemm_nn_f32(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, unsigned flags, void *stream)
{
    if (flags & PLX_GEMM_DROPOUT)  // this entry point carries no p / seed / offset
        return plx::fail(PLX_ERR_UNSUPPORTED, "gemm_nn: PLX_GEMM_DROPOUT needs plx_gemm_nn_f32_split_dropout, or plx_dropout_f32 after this product");
    return gemm_nn_impl(M, N, K, A, lda, B, ldb, C, ldc, flags, nullptr, 0, stream);
}

int plx_gemm_nt_f32(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, const float *mask, int64_t ldmask, void *stream)
{
    return gemm_nt_impl(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, nullptr, 0, stream);
}

size_t plx_gemm_tn_workspace_bytes(int64_t M, int64_t N, int64_t K) { return tn_workspace_bytes(M, N, K); }

int plx_gemm_tn_f32(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, const float *mask, int64_t ldmask, void *workspace,
                    size_t workspace_bytes, void *stream)
{
    return gemm_tn_impl(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, workspace, workspace_bytes, nullptr, 1.f, stream);
}

}  // extern "C"
