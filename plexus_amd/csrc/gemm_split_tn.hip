// GRAD_W = AGG^T . (GRAD_OUT * mask) for fp32 storage on the bf16 matrix cores:
//     C[K x N] = alpha * A[M x K]^T . (B * mask)[M x N],   the contraction running over the M rows of both operands.
//
// Both operands are large, so both are split on the fly: a chunk of 32 rows of A and of B is read as fp32, every value
// is split exactly into three bf16 pieces (split.h) and the pieces are written to LDS TRANSPOSED -- a thread holds the
// same four columns of two consecutive rows, and the piece words of a row pair (row 2j in the low half, row 2j + 1 in the
// high half) are what a lane of v_mfma_f32_32x32x16_bf16 wants side by side: its 8 consecutive contraction elements of
// one column are four such words, one 128-bit LDS read.  Six piece products per 32 x 32 x 16 block, as in the NT forms,
// make the product memory-bound where the fp32 MFMA is compute-bound (2.45 M rows, 128 x 128: 0.82 ms on the fp32 MFMA
// at 70 % MFMA busy).  The mask can be read as one bit per element (the sign bits the forward product wrote).
//
// A workgroup owns a 128 x BN tile of C and one stretch of the rows: some of its wavefronts fetch, split and store the
// chunks, the others multiply them (32 rows of the tile each, and half of its columns when there are eight of them).  Chunks are requested three ahead into two register
// sets and pass through two LDS buffers, one workgroup barrier per chunk.  As in the fp32 kernel the accumulators are added into a second set every
// 256 rows, the stretches' partial tiles go to the workspace, and a second kernel adds them in a fixed order in fp64.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdint>

#include "bf16.h"
#include "common.h"
#include "split.h"

namespace {

using namespace plx::split;

constexpr int kRows = 32;          // rows of both operands per chunk (the contraction)
constexpr int kSW = 20;            // 32-bit words per row of a plane: 16 row pairs + 4 of padding (80 bytes: 128-bit reads conflict-free)
constexpr int kTileK = 128;        // columns of A per workgroup = rows of its tile of C
constexpr int kFlushChunks = 8;    // chunks between two flushes of the accumulators into the totals: 256 rows
constexpr size_t kFlagBytes = 256;

struct TnArgs {
    const float *A, *B, *mask;
    const uint32_t *mask_bits;  // bit c % 32 of word [row * ldw + c / 32]: element (row, c) of B counts
    int64_t lda, ldb, ldmask, ldw;
    int64_t M, N, K;
    int64_t rows_per_split;
    float *ws;  // partial tiles [split][K][ws_ld]
    int64_t ws_ld, ws_slab;
    unsigned *nonfinite;  // raised when an operand holds a value the split cannot carry
};

__global__ void zero_flag_kernel(unsigned *flag) { *flag = 0u; }

constexpr int kNP = 8;  // wavefronts that fetch, split and store
constexpr int kNC = 4;  // wavefronts that multiply
constexpr int kThreads = 64 * (kNP + kNC);
static_assert((kNP == 4 || kNP == 8) && (kNC == 4 || kNC == 8), "four or eight wavefronts per role");

// TNW: 32-column tiles of the workgroup's 128 x 32 TNW tile of C (2 or 4); MASK: 0 none, 1 fp32 values, 2 bits.  The
// operands are 16-byte aligned with leading dimensions, K and N multiples of 4: every access is a 128-bit load.
// The wavefronts of a workgroup have two roles: kNP of them fetch, split and store the chunks (vector ALU, LDS writes),
// kNC multiply them (matrix cores, LDS reads), so that the splitting of chunk c + 1 runs beside the products of chunk c.
// The hardware deals the wavefronts of a workgroup to the four SIMDs of its compute unit in turn (w, w + 4, w + 8, ...
// share one), so the first kNC wavefronts multiply and the rest split: every SIMD gets its share of both.
// BVEC = false: B is read element by element (rows that are not 16-byte aligned, any N: the 47-wide gradient of a last
// layer), without a mask; a splitting thread then owns single columns cq, cq + kQ, ... of B's tile instead of groups of four.
template <int TNW, int MASK, bool BVEC = true>
__global__ void __launch_bounds__(kThreads, 1) gemm_split_tn_kernel(const TnArgs g)
{
    static_assert(BVEC || MASK == 0, "element loads of B come without a mask");
    constexpr int BN = 32 * TNW;
    constexpr int TNH = kNC == 8 ? TNW / 2 : TNW;               // tiles per multiplying wavefront
    constexpr int kAWords = 3 * kTileK * kSW, kBWords = 3 * BN * kSW;  // words of the planes of one buffer
    constexpr int kBuf = kAWords + kBWords;
    constexpr int kQ = kNP * 4;                                 // 4-column groups covered by one pass of the splitting threads
    constexpr int kAItems = 32 / kQ;                            // (row pair, 4-column group) items of A per splitting thread
    constexpr int kBItems = BVEC ? (BN / 4 + kQ - 1) / kQ : 1;  // ... of B
    constexpr int kBCols = BVEC ? 1 : (BN + kQ - 1) / kQ;       // (row pair, column) items of B per splitting thread, element loads
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];  // [2][kBuf]

    const int hw_wave = threadIdx.x >> 6;
    const bool producer = hw_wave >= kNC;
    const int wave = producer ? hw_wave - kNC : hw_wave;  // number within the role
    const int64_t row0 = (int64_t)blockIdx.y * kTileK;  // rows of C = columns of A
    const int64_t col0 = (int64_t)blockIdx.z * BN;      // columns of C = columns of B
    const int64_t mbeg = (int64_t)blockIdx.x * g.rows_per_split;
    const int64_t mend = min(mbeg + g.rows_per_split, g.M);
    const int64_t n_chunks = mbeg < mend ? (mend - mbeg + kRows - 1) / kRows : 0;

    // planes of column groups outside the matrices are never written again
    for (int i = threadIdx.x; i < 2 * kBuf; i += kThreads) lds[i] = 0u;
    __syncthreads();

    if (producer) {
        // ---- thread (mp, cq) owns rows 2 mp and 2 mp + 1 of a chunk and the column groups cq, cq + kQ, ... of both tiles ----
        const int tid = wave * 64 + (int)(threadIdx.x & 63);
        const int mp = tid & 15;
        const int cq = tid >> 4;  // 0 .. kQ - 1
        // A column group that lies outside the matrices (K or N below the tile's width) is read all the same -- from the
        // first columns of the tile, so that the loop has no branch around a load -- and its pieces go to a corner of LDS
        // that nobody reads, while its own place in the planes keeps the zeros written at the start.
        bool a_ok[kAItems], b_ok[kBItems];
        const float *pa[kAItems], *pb[kBItems], *pm[MASK == 1 ? kBItems : 1];
        const uint32_t *pw[MASK == 2 ? kBItems : 1];
        int bit0[kBItems];
        bool bs_ok[kBCols];
        const float *pbs[kBCols];
#pragma unroll
        for (int p = 0; p < kBCols; ++p) {
            const int c = cq + kQ * p;
            bs_ok[p] = !BVEC && c < BN && col0 + c < g.N;
            pbs[p] = g.B + (mbeg + 2 * mp) * g.ldb + (bs_ok[p] ? col0 + c : col0);
        }
#pragma unroll
        for (int p = 0; p < kAItems; ++p) {
            const int64_t col = row0 + 4 * (cq + kQ * p);
            a_ok[p] = col < g.K;
            pa[p] = g.A + (mbeg + 2 * mp) * g.lda + (a_ok[p] ? col : row0);
        }
#pragma unroll
        for (int p = 0; p < kBItems; ++p) {
            const int64_t col = col0 + 4 * (cq + kQ * p);
            b_ok[p] = BVEC && 4 * (cq + kQ * p) < BN && col < g.N;
            const int64_t c = b_ok[p] ? col : col0;
            pb[p] = g.B + (mbeg + 2 * mp) * g.ldb + c;
            if constexpr (MASK == 1) pm[p] = g.mask + (mbeg + 2 * mp) * g.ldmask + c;
            if constexpr (MASK == 2) pw[p] = g.mask_bits + (mbeg + 2 * mp) * g.ldw + c / 32;
            bit0[p] = (int)(c % 32);
        }

        struct Regs {
            float4 a[kAItems][2], b[kBItems][2], m[MASK == 1 ? kBItems : 1][2];
            uint32_t w[MASK == 2 ? kBItems : 1][2];
            float bs[kBCols][2];
        };
        int64_t m_next = mbeg;  // first row of the chunk the next fetch brings
        auto advance = [&]() {
#pragma unroll
            for (int p = 0; p < kAItems; ++p) pa[p] += (int64_t)kRows * g.lda;
#pragma unroll
            for (int p = 0; p < kBItems; ++p) {
                pb[p] += (int64_t)kRows * g.ldb;
                if constexpr (MASK == 1) pm[p] += (int64_t)kRows * g.ldmask;
                if constexpr (MASK == 2) pw[p] += (int64_t)kRows * g.ldw;
            }
            if constexpr (!BVEC) {
#pragma unroll
                for (int p = 0; p < kBCols; ++p) pbs[p] += (int64_t)kRows * g.ldb;
            }
            m_next += kRows;
        };
        // a chunk whose 32 rows all exist: loads and nothing else (no branch, so that the waits the compiler places before
        // the use of one register set can leave the loads of the other set in flight)
        auto fetch_whole = [&](Regs &r) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int p = 0; p < kAItems; ++p) r.a[p][j] = *reinterpret_cast<const float4 *>(pa[p] + j * g.lda);
                if constexpr (BVEC) {
#pragma unroll
                    for (int p = 0; p < kBItems; ++p) {
                        r.b[p][j] = *reinterpret_cast<const float4 *>(pb[p] + j * g.ldb);
                        if constexpr (MASK == 1) r.m[p][j] = *reinterpret_cast<const float4 *>(pm[p] + j * g.ldmask);
                        if constexpr (MASK == 2) r.w[p][j] = pw[p][j * g.ldw];
                    }
                } else {
#pragma unroll
                    for (int p = 0; p < kBCols; ++p) r.bs[p][j] = pbs[p][j * g.ldb];
                }
            }
            advance();
        };
        // any chunk: rows past the end of the stretch count as zeros
        auto fetch_any = [&](Regs &r) {
            const int rows_left = (int)min(max(mend - m_next - 2 * mp, (int64_t)0), (int64_t)2);
            const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bool row_ok = j < rows_left;
#pragma unroll
                for (int p = 0; p < kAItems; ++p) r.a[p][j] = row_ok ? *reinterpret_cast<const float4 *>(pa[p] + j * g.lda) : zero;
                if constexpr (BVEC) {
#pragma unroll
                    for (int p = 0; p < kBItems; ++p) {
                        r.b[p][j] = row_ok ? *reinterpret_cast<const float4 *>(pb[p] + j * g.ldb) : zero;
                        if constexpr (MASK == 1) r.m[p][j] = row_ok ? *reinterpret_cast<const float4 *>(pm[p] + j * g.ldmask) : zero;
                        if constexpr (MASK == 2) r.w[p][j] = row_ok ? pw[p][j * g.ldw] : 0u;
                    }
                } else {
#pragma unroll
                    for (int p = 0; p < kBCols; ++p) r.bs[p][j] = row_ok ? pbs[p][j * g.ldb] : 0.f;
                }
            }
            advance();
        };
        // where the pieces of an item go: word mp of the plane rows of its four columns, in buffer 0 (the other buffer and
        // the other planes at fixed distances), or the unread corner behind the buffers
        int a_dst[kAItems], b_dst[kBItems];
#pragma unroll
        for (int p = 0; p < kAItems; ++p) a_dst[p] = a_ok[p] ? (4 * (cq + kQ * p)) * kSW + mp : 2 * kBuf + mp;
#pragma unroll
        for (int p = 0; p < kBItems; ++p) b_dst[p] = b_ok[p] ? kAWords + (4 * (cq + kQ * p)) * kSW + mp : 2 * kBuf + mp;
        // the pieces of (row 2 mp, row 2 mp + 1) of one column are one word per plane
        // (returns true if one of the eight values is one the split cannot carry)
        auto stash_quad = [&](uint32_t *dst, int plane_words, const float4 &r0, const float4 &r1) -> bool {
            const float x0[4] = {r0.x, r0.y, r0.z, r0.w}, x1[4] = {r1.x, r1.y, r1.z, r1.w};
            bool care = false;
            uint32_t piece[3][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) care |= split2_checked(x0[e], x1[e], piece[0][e], piece[1][e], piece[2][e]);
            // plane by plane: four stores at fixed distances from one address pair up into two-word store instructions
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                uint32_t *const d = dst + q * plane_words;
#pragma unroll
                for (int e = 0; e < 4; ++e) d[e * kSW] = piece[q][e];
            }
            return care;
        };
        auto stash = [&](int buf, const Regs &r) {
            uint32_t *base = lds + buf * kBuf;
            bool care = false;
#pragma unroll
            for (int p = 0; p < kAItems; ++p)
                care |= stash_quad(a_ok[p] ? base + a_dst[p] : lds + a_dst[p], a_ok[p] ? kTileK * kSW : 0, r.a[p][0], r.a[p][1]);
            if constexpr (!BVEC) {
#pragma unroll
                for (int p = 0; p < kBCols; ++p) {
                    uint32_t p0, p1, p2;
                    care |= split2_checked(r.bs[p][0], r.bs[p][1], p0, p1, p2);
                    uint32_t *dst = bs_ok[p] ? base + kAWords + (cq + kQ * p) * kSW + mp : lds + 2 * kBuf + mp;
                    const int plane_words = bs_ok[p] ? BN * kSW : 0;
                    dst[0] = p0;
                    dst[plane_words] = p1;
                    dst[2 * plane_words] = p2;
                }
            }
#pragma unroll
            for (int p = 0; p < kBItems; ++p) {
                if constexpr (!BVEC) continue;
                if (4 * (cq + kQ * p) >= BN && kBItems * kQ * 4 > BN) continue;  // a pass that reaches past the tile (compile-time shape)
                float4 b0 = r.b[p][0], b1 = r.b[p][1];
                if constexpr (MASK == 1) {
                    const float4 m0 = r.m[p][0], m1 = r.m[p][1];
                    b0 = make_float4(m0.x > 0.f ? b0.x : 0.f, m0.y > 0.f ? b0.y : 0.f, m0.z > 0.f ? b0.z : 0.f, m0.w > 0.f ? b0.w : 0.f);
                    b1 = make_float4(m1.x > 0.f ? b1.x : 0.f, m1.y > 0.f ? b1.y : 0.f, m1.z > 0.f ? b1.z : 0.f, m1.w > 0.f ? b1.w : 0.f);
                }
                if constexpr (MASK == 2) {
                    const uint32_t w0 = r.w[p][0] >> bit0[p], w1 = r.w[p][1] >> bit0[p];
                    b0 = make_float4((w0 & 1u) ? b0.x : 0.f, (w0 & 2u) ? b0.y : 0.f, (w0 & 4u) ? b0.z : 0.f, (w0 & 8u) ? b0.w : 0.f);
                    b1 = make_float4((w1 & 1u) ? b1.x : 0.f, (w1 & 2u) ? b1.y : 0.f, (w1 & 4u) ? b1.z : 0.f, (w1 & 8u) ? b1.w : 0.f);
                }
                care |= stash_quad(b_ok[p] ? base + b_dst[p] : lds + b_dst[p], b_ok[p] ? BN * kSW : 0, b0, b1);
            }
            if (__builtin_expect(care, 0)) *g.nonfinite = 1u;
        };
        // Chunk c lives in register set c % 2 from its fetch (three steps before its products) to its stash (one before).
        // At the top of a double step c (even): chunk c is in buffer 0, chunk c + 1 in r1, chunk c + 2 in r0.
        Regs r0, r1;
        int64_t c = 0;
        if (n_chunks >= 6) {
            // steady state, straight-line: every chunk fetched here (up to c + 4 <= n_chunks - 2) is whole
            fetch_whole(r0);
            fetch_whole(r1);
            stash(0, r0);
            fetch_whole(r0);
            __syncthreads();
            for (; c + 6 <= n_chunks; c += 2) {
                stash(1, r1);
                fetch_whole(r1);
                __syncthreads();
                stash(0, r0);
                fetch_whole(r0);
                __syncthreads();
            }
        } else {
            if (n_chunks > 0) {
                fetch_any(r0);
                if (n_chunks > 1) fetch_any(r1);
                stash(0, r0);
                if (n_chunks > 2) fetch_any(r0);
            }
            __syncthreads();
        }
        for (; c < n_chunks; c += 2) {  // the last steps of the stretch, and short stretches
            if (c + 1 < n_chunks) stash(1, r1);
            if (c + 3 < n_chunks) fetch_any(r1);
            __syncthreads();
            if (c + 1 < n_chunks) {
                if (c + 2 < n_chunks) stash(0, r0);
                if (c + 4 < n_chunks) fetch_any(r0);
                __syncthreads();
            }
        }
        return;
    }

    // ---- the multiplying wavefronts: rows 32 kb ... of the tile, column tiles nh TNH ... ----
    const int lane = threadIdx.x & 63;
    const int li = lane & 31;
    const int h = lane >> 5;
    const int kb = wave & 3;
    const int nh = wave >> 2;  // 0 when four wavefronts multiply
    floatx16 acc[TNH];
    float tot[TNH][16];
#pragma unroll
    for (int t = 0; t < TNH; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc[t][v] = 0.f;
            tot[t][v] = 0.f;
        }
    auto flush = [&]() {
#pragma unroll
        for (int t = 0; t < TNH; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                tot[t][v] += acc[t][v];
                acc[t][v] = 0.f;
            }
    };
    // a lane reads row li of its 32-row block of a plane: words 8 s + 4 h ... + 3 are contraction rows 16 s + 8 h ... + 7
    const uint16_t *const a_src = reinterpret_cast<const uint16_t *>(lds) + ((kb * 32 + li) * kSW + 4 * h) * 2;
    const uint16_t *const b_src = reinterpret_cast<const uint16_t *>(lds + kAWords) + ((nh * TNH * 32 + li) * kSW + 4 * h) * 2;
    // With two column tiles per wavefront the pieces of B are read one tile ahead of their products into a second register set
    // (the order is pinned: an empty asm statement takes each tile's accumulator, a scheduling barrier follows).  With four tiles
    // the 128 accumulators and totals leave no registers for that set (12 wavefronts: 168 registers each), and the pieces are
    // read where they are used.
    constexpr bool kAheadB = TNH <= 2;
    auto compute = [&](int buf) {
        const uint16_t *as = a_src + buf * kBuf * 2, *bs = b_src + buf * kBuf * 2;
        if constexpr (!kAheadB) {
#pragma unroll
            for (int s = 0; s < kRows / 16; ++s) {
                const bf16x8 a0 = *reinterpret_cast<const bf16x8 *>(as + 16 * s);
                const bf16x8 a1 = *reinterpret_cast<const bf16x8 *>(as + 16 * s + kTileK * kSW * 2);
                const bf16x8 a2 = *reinterpret_cast<const bf16x8 *>(as + 16 * s + 2 * kTileK * kSW * 2);
#pragma unroll
                for (int t = 0; t < TNH; ++t) {
                    const uint16_t *bt = bs + t * 32 * kSW * 2 + 16 * s;
                    const bf16x8 b0 = *reinterpret_cast<const bf16x8 *>(bt);
                    const bf16x8 b1 = *reinterpret_cast<const bf16x8 *>(bt + BN * kSW * 2);
                    const bf16x8 b2 = *reinterpret_cast<const bf16x8 *>(bt + 2 * BN * kSW * 2);
                    acc[t] = mfma6(a0, a1, a2, b0, b1, b2, acc[t]);
                }
            }
            return;
        }
        auto load_b = [&](bf16x8(&b)[3], int sub, int t) __attribute__((always_inline)) {
            const uint16_t *bt = bs + t * 32 * kSW * 2 + 16 * sub;
            b[0] = *reinterpret_cast<const bf16x8 *>(bt);
            b[1] = *reinterpret_cast<const bf16x8 *>(bt + BN * kSW * 2);
            b[2] = *reinterpret_cast<const bf16x8 *>(bt + 2 * BN * kSW * 2);
        };
        bf16x8 bb[2][3];
        load_b(bb[0], 0, 0);
#pragma unroll
        for (int sub = 0; sub < kRows / 16; ++sub) {
            const bf16x8 a0 = *reinterpret_cast<const bf16x8 *>(as + 16 * sub);
            const bf16x8 a1 = *reinterpret_cast<const bf16x8 *>(as + 16 * sub + kTileK * kSW * 2);
            const bf16x8 a2 = *reinterpret_cast<const bf16x8 *>(as + 16 * sub + 2 * kTileK * kSW * 2);
#pragma unroll
            for (int t = 0; t < TNH; ++t) {
                const int group = sub * TNH + t;
                if (t + 1 < TNH) load_b(bb[(group + 1) & 1], sub, t + 1);
                else if (sub + 1 < kRows / 16) load_b(bb[(group + 1) & 1], sub + 1, 0);
                acc[t] = mfma6(a0, a1, a2, bb[group & 1][0], bb[group & 1][1], bb[group & 1][2], acc[t]);
                asm volatile("" : "+v"(acc[t]));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    __syncthreads();  // chunk 0 is in buffer 0
    int since_flush = 0;
    for (int64_t c = 0; c < n_chunks; ++c) {
        compute((int)(c & 1));
        if (++since_flush == kFlushChunks) {
            since_flush = 0;
            flush();
        }
        __syncthreads();  // chunk c + 1 is in the other buffer; this one may be overwritten
    }
    flush();

    // register v of a lane is row 8 (v / 4) + 4 h + v % 4, column lane % 32 of each 32 x 32 block
    float *out = g.ws + (int64_t)blockIdx.x * g.ws_slab;
#pragma unroll
    for (int t = 0; t < TNH; ++t) {
        const int64_t c = col0 + (nh * TNH + t) * 32 + li;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t r = row0 + kb * 32 + 8 * (v / 4) + 4 * h + (v % 4);
            if (c < g.N && r < g.K) out[r * g.ws_ld + c] = tot[t][v];
        }
    }
}

template <int TNW, int MASK, bool BVEC = true>
int launch_one(const TnArgs &g, dim3 grid, hipStream_t st)
{
    // two buffers of planes and the corner that takes the pieces of column groups outside the matrices
    constexpr size_t shm = ((size_t)2 * 3 * (kTileK + 32 * TNW) * kSW + 4 * kSW) * sizeof(uint32_t);
    static_assert(shm <= 160 * 1024, "two buffers of planes fit the LDS of a compute unit");
    static std::atomic<uint64_t> allowed{0};  // devices on which this instantiation may take its LDS
    const int rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_split_tn_kernel<TNW, MASK, BVEC>), shm, allowed);
    if (rc != PLX_OK) return rc;
    gemm_split_tn_kernel<TNW, MASK, BVEC><<<grid, kThreads, shm, st>>>(g);
    PLX_LAUNCH_CHECK("gemm_split_tn_kernel");
    return PLX_OK;
}

template <int TNW>
int launch_mask(const TnArgs &g, int mask, dim3 grid, hipStream_t st)
{
    switch (mask) {
        case 0: return launch_one<TNW, 0>(g, grid, st);
        case 1: return launch_one<TNW, 1>(g, grid, st);
        default: return launch_one<TNW, 2>(g, grid, st);
    }
}

int tile_cols(int64_t N) { return N <= 64 ? 64 : 128; }

// one workgroup per compute unit (its two buffers take most of the LDS), so the stretches of rows are as many as fill the
// chip once: equal work for all, no second round with a tail
int64_t split_count(int64_t M, int64_t N, int64_t K)
{
    const int64_t tiles = plx::ceil_div(K, kTileK) * plx::ceil_div(N, tile_cols(N));
    const int64_t want = std::max<int64_t>(1, 256 / tiles);
    const int64_t by_rows = std::max<int64_t>(1, M / 1024);
    return std::max<int64_t>(1, std::min(want, by_rows));
}

size_t partial_bytes(int64_t M, int64_t N, int64_t K)
{
    const int64_t ld = (N + 3) / 4 * 4;
    return (size_t)split_count(M, N, K) * (size_t)K * (size_t)ld * sizeof(float);
}

bool aligned16(const void *p, int64_t ld) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0); }

}  // namespace

extern "C" {

size_t plx_gemm_tn_f32_split_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    // the partial tiles, shared with the fp32 MFMA product that redoes the work when an operand holds Inf or NaN, and the
    // flag word that tells it to
    return std::max(partial_bytes(M, N, K), plx::gemm_tn_f32_workspace_bytes(M, N, K)) + kFlagBytes;
}

int plx_gemm_tn_f32_split(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                          const float *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw, float alpha, void *workspace,
                          size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && K >= 0 && N < (1ll << 30) && K < (1ll << 30), "gemm_tn_split: bad dimension");
    if (K == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(C != nullptr, "gemm_tn_split: NULL output");
    PLX_REQUIRE(M == 0 || (A != nullptr && B != nullptr), "gemm_tn_split: NULL operand");
    PLX_REQUIRE(lda >= K && ldb >= N && ldc >= N, "gemm_tn_split: leading dimension too small");
    PLX_REQUIRE(mask == nullptr || ldmask >= N, "gemm_tn_split: mask leading dimension too small");
    PLX_REQUIRE(mask_bits == nullptr || (mask != nullptr && ldw >= (N + 31) / 32),
                "gemm_tn_split: a bit mask comes with the fp32 mask it stands for and a pitch of at least ceil(N / 32) words");
    const size_t need = plx_gemm_tn_f32_split_workspace_bytes(std::max<int64_t>(M, 1), N, K);
    if (workspace == nullptr || workspace_bytes < need)
        return plx::fail(PLX_ERR_WORKSPACE, "gemm_tn_split: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    PLX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, "gemm_tn_split: workspace must be 16-byte aligned");
    hipStream_t st = plx::as_stream(stream);
    unsigned *flag = reinterpret_cast<unsigned *>(static_cast<char *>(workspace) + (need - kFlagBytes));
    zero_flag_kernel<<<1, 1, 0, st>>>(flag);
    PLX_LAUNCH_CHECK("zero_flag_kernel");

    TnArgs g{};
    g.A = A; g.B = B; g.mask = mask; g.mask_bits = mask_bits;
    g.lda = lda; g.ldb = ldb; g.ldmask = ldmask; g.ldw = ldw;
    g.M = M; g.N = N; g.K = K;
    const int64_t splits = split_count(std::max<int64_t>(M, 1), N, K);
    g.rows_per_split = plx::ceil_div(plx::ceil_div(std::max<int64_t>(M, 1), splits), kRows) * kRows;  // whole chunks, whatever the split
    const int64_t used = plx::ceil_div(std::max<int64_t>(M, 1), g.rows_per_split);
    g.ws = static_cast<float *>(workspace);
    g.ws_ld = (N + 3) / 4 * 4;
    g.ws_slab = K * g.ws_ld;
    g.nonfinite = flag;
    // the split kernel reads with 128-bit loads; operands that do not allow them go to the fp32 MFMA kernel as they are
    const bool bits = mask_bits != nullptr && reinterpret_cast<uintptr_t>(mask_bits) % 4 == 0;
    const bool a_vec = M > 0 && aligned16(A, lda) && K % 4 == 0;
    const bool vec = a_vec && aligned16(B, ldb) && (bits || aligned16(mask, ldmask)) && N % 4 == 0;
    // B in rows that do not take 128-bit loads (the 47-wide gradient of a last layer): read element by element, when it is at most
    // 64 columns wide and comes without a mask
    const bool b_scalar = !vec && a_vec && mask == nullptr && N <= 64;
    if (!vec && !b_scalar)
        return plx::gemm_tn_f32_if(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, workspace, need - kFlagBytes, nullptr, alpha, stream);
    const int mode = mask == nullptr ? 0 : (bits ? 2 : 1);
    const int bn = tile_cols(N);
    dim3 grid((unsigned)used, (unsigned)plx::ceil_div(K, kTileK), (unsigned)plx::ceil_div(N, bn));
    int rc = b_scalar ? launch_one<2, 0, false>(g, grid, st) : (bn == 64 ? launch_mask<2>(g, mode, grid, st) : launch_mask<4>(g, mode, grid, st));
    if (rc != PLX_OK) return rc;
    rc = plx::gemm_tn_reduce_tiles(g.ws, g.ws_ld, g.ws_slab, (int)used, K, N, C, ldc, alpha, stream);
    if (rc != PLX_OK) return rc;
    // Inf / NaN / values next to FLT_MAX in either operand: the fp32 MFMA kernel redoes the product (a launch that is
    // always enqueued and returns at once unless the flag is set)
    return plx::gemm_tn_f32_if(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, workspace, need - kFlagBytes, flag, alpha, stream);
}

}  // extern "C"
