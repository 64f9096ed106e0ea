// Dense products of the GCN layer with bf16 storage and fp32 accumulation (v_mfma_f32_32x32x16_bf16).
//
//   NT  C[M x N] (bf16) = epilogue(alpha * (A*mask)[M x K] . B[N x K]^T)
//         forward  OUT      = AGG . W        with B = W^T stored [N_out x K_in]  (+ ReLU, + dropout)
//         backward GRAD_AGG = GRAD_OUT . W^T with B = W   stored [K_in x N_out]  (+ ReLU/dropout mask, alpha = 1/(1-p))
//   TN  C[K x N] (fp32) = alpha * A[M x K]^T . (B*mask)[M x N]          GRAD_W = AGG^T . GRAD_OUT
//
// With bf16 storage these tall-skinny products are bound by HBM, not by the matrix cores (the MFMA
// rate is 16x the fp32 one), so the kernels are built around wide memory accesses:
//   * operands are fetched as 16-byte vectors (8 bf16) along contiguous memory;
//   * an MFMA lane needs 8 consecutive contraction indices of one row/column.  For NT both operands
//     are already contraction-contiguous ("x-major" LDS tiles, one 128-bit LDS read per fragment).  For
//     TN the contraction runs over the rows of both operands, so tiles are transposed on their way into
//     LDS: a thread loads the same 8 columns of two consecutive rows and writes eight 32-bit words
//     (row pair packed) down a column of the transposed tile;
//   * the NT output goes through LDS so that every lane stores 16 bytes of one output row; the dropout
//     generator (Philox-4x32-10) is called once per 8 consecutive elements there.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "bf16.h"
#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 128;      // output rows per workgroup
constexpr int kBK = 64;       // contraction chunk (bf16 elements)
constexpr int kS = kBK + 8;   // LDS row stride in bf16 elements: 144 bytes, keeps 128-bit reads conflict-free
constexpr int kThreads = 256;

struct Bf16Args {
    const uint16_t *A;
    const uint16_t *B;
    const uint16_t *mask;
    void *C;
    int64_t lda, ldb, ldc, ldmask;
    int64_t M, N, K;
    float alpha;
    unsigned flags;
    uint32_t thresh16;   // keep iff 16-bit lane >= thresh16
    float keep_scale;    // 1 / (1 - p)
    uint32_t seed_lo, seed_hi, off_lo, off_hi;
    int a_vec, b_vec, c_vec, m_vec;
    int c_flat;  // resident NT kernel: C 16-byte aligned and contiguous (ldc == N), N <= 64, no dropout, no sign bits: half panels leave as flat runs
    // the mask as one bit per element (bit c % 32 of word [row * ldw + c / 32]): read in place of `mask` by the resident NT
    // kernel and the whole-tile TN kernel, written for C (its positive elements) by the resident NT kernel
    const uint32_t *mask_bits;
    int64_t ldw;
    uint32_t *relu_bits;
    int64_t ldw_out;
    // TN only
    int64_t rows_per_split;
    float *ws;
    int64_t ws_ld, ws_slab;
};

__device__ __forceinline__ uint4 zero4() { return make_uint4(0u, 0u, 0u, 0u); }

// 8 consecutive bf16 of a row, zero beyond `valid` elements; 16-byte load when allowed
__device__ __forceinline__ uint4 load8(const uint16_t *q, int valid, int vec_ok)
{
    if (valid >= 8 && vec_ok) return *reinterpret_cast<const uint4 *>(q);
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) e[i] = i < valid ? (uint32_t)q[i] : 0u;
    return make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
}

__device__ __forceinline__ uint32_t mask2(uint32_t v, uint32_t m)
{
    const uint32_t lo = plx::bf16_positive(m & 0xffffu) ? 0x0000ffffu : 0u;
    const uint32_t hi = plx::bf16_positive(m >> 16) ? 0xffff0000u : 0u;
    return v & (lo | hi);
}

// the same with the mask as 8 bits, bit e for element e
__device__ __forceinline__ uint32_t keep2(uint32_t v, uint32_t b) { return v & (((b & 1u) ? 0x0000ffffu : 0u) | ((b & 2u) ? 0xffff0000u : 0u)); }
__device__ __forceinline__ uint4 mask8_bits(uint4 v, uint32_t b) { return make_uint4(keep2(v.x, b), keep2(v.y, b >> 2), keep2(v.z, b >> 4), keep2(v.w, b >> 6)); }

__device__ __forceinline__ uint4 mask8(uint4 v, uint4 m) { return make_uint4(mask2(v.x, m.x), mask2(v.y, m.y), mask2(v.z, m.z), mask2(v.w, m.w)); }

// ------------------------------------------------------------------------------------------------
// NT: C = epilogue(alpha * (A*mask) . B^T), A [M x K], B [N x K], both contraction-contiguous
// ------------------------------------------------------------------------------------------------
// VEC: every operand is 16-byte aligned with a leading dimension that is a multiple of 8 and K % 8 == 0,
// so a tile is made of whole 16-byte vectors: no element-wise paths, and addressing is one 64-bit
// multiply per thread and tile plus pointer steps (address arithmetic per vector would otherwise cost more
// vector-ALU time than the MFMAs take).
template <int TN, bool MASKED, bool VEC>
__global__ void __launch_bounds__(kThreads) gemm_bf16_nt_kernel(const Bf16Args g)
{
    constexpr int BN = 32 * TN;
    constexpr int kAVec = kBM * kBK / 8 / kThreads;                       // 16-byte vectors per thread and chunk, A tile
    constexpr int kBVec = (BN * kBK / 8 + kThreads - 1) / kThreads;       // B tile
    constexpr int kTile = (kBM + BN) * kS;                                // bf16 elements per buffer
    constexpr int kCS = BN + 4;                                           // fp32 row stride of the staged output
    constexpr int kAhead = 4;                                             // chunks of A fetched in one go
    static_assert(4 * 32 * kCS * 4 <= 2 * kTile * 2, "staged output must fit the operand buffers");

    __shared__ __attribute__((aligned(16))) uint16_t lds[2 * kTile];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 31;
    const int h = lane >> 5;

    // Workgroup -> tile mapping.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with
    // its own L2; the column tiles of one row panel are therefore given to consecutive workgroups of the
    // SAME XCD (ids b, b + 8, ...), so that the row panel of A is read from HBM once and from that L2 after.
    const int64_t n_ct = (g.N + BN - 1) / BN;
    const int64_t n_rp = (g.M + kBM - 1) / kBM;
    const int64_t bid = blockIdx.x;
    const int64_t xcd = bid % 8, slot = bid / 8;
    const int64_t rp = (slot / n_ct) * 8 + xcd;
    if (rp >= n_rp) return;
    const int64_t row0 = rp * kBM;
    const int64_t col0 = (slot % n_ct) * BN;

    // thread (rt, kq) owns vector kq of rows rt, rt + 32, ... of a tile
    const int rt = threadIdx.x >> 3;
    const int kq = threadIdx.x & 7;
    const uint16_t *pa = g.A + (row0 + rt) * g.lda + kq * 8;
    const uint16_t *pm = MASKED ? g.mask + (row0 + rt) * g.ldmask + kq * 8 : nullptr;
    const uint16_t *pb = g.B + (col0 + rt) * g.ldb + kq * 8;
    const int a_rows = (int)min(max(g.M - row0 - rt, (int64_t)0), (int64_t)kBM);  // rows rt + 32 p with 32 p < a_rows exist
    const int b_rows = (int)min(max(g.N - col0 - rt, (int64_t)0), (int64_t)BN);
    const int K = (int)g.K;

    // A is bound by HBM latency, not by the matrix cores (one chunk is 16 MFMAs): all loads of up to
    // kAhead chunks are issued back to back before the first one is consumed.  B (the weight) comes from
    // L2 and keeps the usual one-chunk-ahead prefetch.
    // the mask is kept beside its chunk and applied when the chunk is stored to LDS: applying it at the load
    // would make every fetch wait for its own data and undo the prefetch
    uint4 ra[kAhead][kAVec], rm[MASKED ? kAhead : 1][kAVec], rb[kBVec];
    auto fetch_a = [&](int k0, uint4(&dst)[kAVec], uint4(&mdst)[kAVec]) {
        const int k = k0 + kq * 8;
#pragma unroll
        for (int p = 0; p < kAVec; ++p) {
            uint4 v = zero4(), m = zero4();
            if (32 * p < a_rows && k < K) {
                if constexpr (VEC) {
                    v = *reinterpret_cast<const uint4 *>(pa + (int64_t)(32 * p) * g.lda + k0);
                    if constexpr (MASKED) m = *reinterpret_cast<const uint4 *>(pm + (int64_t)(32 * p) * g.ldmask + k0);
                } else {
                    const int valid = min(8, K - k);
                    v = load8(pa + (int64_t)(32 * p) * g.lda + k0, valid, g.a_vec);
                    if constexpr (MASKED) m = load8(pm + (int64_t)(32 * p) * g.ldmask + k0, valid, g.m_vec);
                }
            }
            dst[p] = v;
            if constexpr (MASKED) mdst[p] = m;
        }
    };
    auto fetch_b = [&](int k0) {
        const int k = k0 + kq * 8;
#pragma unroll
        for (int p = 0; p < kBVec; ++p) {
            uint4 v = zero4();
            if (32 * p < b_rows && k < K) {
                if constexpr (VEC)
                    v = *reinterpret_cast<const uint4 *>(pb + (int64_t)(32 * p) * g.ldb + k0);
                else
                    v = load8(pb + (int64_t)(32 * p) * g.ldb + k0, min(8, K - k), g.b_vec);
            }
            rb[p] = v;
        }
    };
    const int st_off = rt * kS + kq * 8;
    auto stash = [&](int buf, const uint4(&a)[kAVec], const uint4(&m)[kAVec]) {
        uint16_t *as = lds + buf * kTile + st_off;
        uint16_t *bs = as + kBM * kS;
#pragma unroll
        for (int p = 0; p < kAVec; ++p) *reinterpret_cast<uint4 *>(as + 32 * p * kS) = MASKED ? mask8(a[p], m[p]) : a[p];
#pragma unroll
        for (int p = 0; p < kBVec; ++p)
            if (32 * p < BN) *reinterpret_cast<uint4 *>(bs + 32 * p * kS) = rb[p];
    };

    floatx16 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

    int buf = 0;
    for (int kk = 0; kk < K; kk += kAhead * kBK) {
#pragma unroll
        for (int c = 0; c < kAhead; ++c) fetch_a(kk + c * kBK, ra[c], rm[MASKED ? c : 0]);  // chunks past K come back as zeros
        fetch_b(kk);
        stash(buf, ra[0], rm[0]);
        __syncthreads();
#pragma unroll
        for (int c = 0; c < kAhead; ++c) {
            const int k0 = kk + c * kBK;
            if (k0 >= K) break;
            const bool more = (c + 1 < kAhead) && (k0 + kBK < K);
            if (more) fetch_b(k0 + kBK);
            const uint16_t *as = lds + buf * kTile;
            const uint16_t *bs = as + kBM * kS;
#pragma unroll
            for (int s = 0; s < kBK / 16; ++s) {
                const bf16x8 a = *reinterpret_cast<const bf16x8 *>(as + (wave * 32 + li) * kS + 16 * s + 8 * h);
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    const bf16x8 b = *reinterpret_cast<const bf16x8 *>(bs + (t * 32 + li) * kS + 16 * s + 8 * h);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
                }
            }
            if (more) stash(buf ^ 1, ra[(c + 1) % kAhead], rm[MASKED ? (c + 1) % kAhead : 0]);
            __syncthreads();
            buf ^= 1;
        }
    }

    // stage the wavefront's 32 x BN fp32 tile in LDS (register v of a lane is row 8 (v / 4) + 4 h + v % 4,
    // column lane % 32 of each 32 x 32 tile), then hand out 8 consecutive columns of one row per lane
    float *cs = reinterpret_cast<float *>(lds) + wave * 32 * kCS;
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) cs[(8 * (v / 4) + 4 * h + (v % 4)) * kCS + t * 32 + li] = acc[t][v];
    __syncthreads();

    const bool relu = (g.flags & PLX_GEMM_RELU) != 0;
    const bool drop = (g.flags & PLX_GEMM_DROPOUT) != 0;
    uint16_t *C = static_cast<uint16_t *>(g.C);
    constexpr int kVecPerRow = BN / 8;
#pragma unroll
    for (int it = 0; it < 32 * kVecPerRow / 64; ++it) {
        const int id = it * 64 + lane;
        const int rl = id / kVecPerRow;
        const int cq = id % kVecPerRow;
        const int64_t r = row0 + wave * 32 + rl;
        const int64_t c = col0 + cq * 8;
        if (r >= g.M || c >= g.N) continue;
        const float4 lo = *reinterpret_cast<const float4 *>(cs + rl * kCS + cq * 8);
        const float4 hi = *reinterpret_cast<const float4 *>(cs + rl * kCS + cq * 8 + 4);
        float x[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x[e] *= g.alpha;
            if (relu) x[e] = fmaxf(x[e], 0.f);
        }
        const int valid = (int)min((int64_t)8, g.N - c);
        if (drop) {
            const uint64_t e0 = (uint64_t)r * (uint64_t)g.N + (uint64_t)c;
            if ((e0 & 7u) == 0) {
                const uint64_t q = e0 >> 3;
                const plx::Philox4 rnd = plx::philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), g.off_lo, g.off_hi, g.seed_lo, g.seed_hi);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = plx::dropout_lane16(rnd, e) >= g.thresh16 ? x[e] * g.keep_scale : 0.f;
            } else {
                for (int e = 0; e < valid; ++e) {
                    const uint64_t ee = e0 + e;
                    const uint64_t q = ee >> 3;
                    const plx::Philox4 rnd = plx::philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), g.off_lo, g.off_hi, g.seed_lo, g.seed_hi);
                    x[e] = plx::dropout_lane16(rnd, (int)(ee & 7u)) >= g.thresh16 ? x[e] * g.keep_scale : 0.f;
                }
            }
        }
        uint16_t *dst = C + r * g.ldc + c;
        if (valid == 8 && g.c_vec) {
            *reinterpret_cast<uint4 *>(dst) = make_uint4(plx::pack_bf16x2(x[0], x[1]), plx::pack_bf16x2(x[2], x[3]),
                                                         plx::pack_bf16x2(x[4], x[5]), plx::pack_bf16x2(x[6], x[7]));
        } else {
            for (int e = 0; e < valid; ++e) dst[e] = (uint16_t)plx::f32_to_bf16(x[e]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// NT for a weight of at most 256 x 256 and an output that allows 16-byte stores: B stays in LDS for the life of a 512-thread
// workgroup and every wavefront streams its own 32-row panels of A through a private LDS tile, so the main
// loop has no workgroup barrier (the wavefronts of a SIMD overlap one's MFMAs with the other's staging).  A chunk
// is 32 rows x 32 contraction elements, two 16-byte vectors per lane, requested kRing positions ahead.  The output
// tile goes through the private tile 16 rows x 32 columns at a time, so that a lane holds 8 consecutive columns of
// a row for the dropout generator and stores 16 bytes.
// ------------------------------------------------------------------------------------------------
constexpr int kRWaves = 8;
constexpr int kRCK = 32;                 // contraction elements per chunk
constexpr int kRAS = kRCK + 8;           // stride of the private tile in bf16 elements (80 bytes)
constexpr int kRMax = 256;               // largest N and K
constexpr int kRBS = kRMax + 8;          // stride of the resident B (528 bytes)
constexpr int kRPrivate = 32 * kRAS;     // bf16 elements of a private tile (2,560 bytes; also 16 x 36 floats of staging)
constexpr int kRCS = 36;                 // fp32 stride of the staged half tile
constexpr size_t kRLdsBytes = ((size_t)kRMax * kRBS + (size_t)kRWaves * kRPrivate) * sizeof(uint16_t);
static_assert(16 * kRCS * 4 <= kRPrivate * 2, "staged half tile must fit the private tile");

// KS: chunk positions of a panel, 8 (K <= 256) or 4 (K <= 128).
// FAST: A (and the mask) take 16-byte loads and K is a multiple of 8, at least 8.  Every request is then an unconditional
// load from an address clamped into the matrix (rows past the end repeat the last row and are never stored; columns
// past K repeat the last eight and meet the zero padding of B), with no branch around it, and every position is
// multiplied: the wait the compiler places before a chunk is used can then name how many younger requests may stay in
// flight, where loads inside branches make it wait for all of them.
// MASK: 0 none, 1 bf16 values beside A (positive keeps the element), 2 one bit per element (FAST only; the KS words of a
// panel row come with the panel's first chunk and stay in registers, so the ring is as deep as without a mask)
// WBITS: also write the sign bits of C (a kernel of its own, so that the others do not carry its registers)
template <int TN, int MASK, bool FAST = false, int KS = 8, bool WBITS = false>
__global__ void __launch_bounds__(kRWaves * 64, 1) gemm_bf16_nt_resident_kernel(const Bf16Args g)
{
    constexpr bool MASKED = MASK == 1;
    constexpr bool BITS = MASK == 2;
    static_assert(!BITS || FAST, "the bit mask is read by the unconditional kernel only");
    constexpr int kSteps = KS;             // chunk positions of a panel (positions past K are skipped)
    constexpr int kRing = (MASKED || FAST || TN > 4) ? 4 : KS;  // register slots = positions ahead that a chunk is requested
    static_assert(KS == 8 || (FAST && KS == 4), "the guarded kernel walks all eight positions");
    extern __shared__ __attribute__((aligned(16))) uint16_t rlds[];
    uint16_t *const bres = rlds;  // [kRMax][kRBS]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in every lane: panel arithmetic stays scalar
    const int li = lane & 31;
    const int h = lane >> 5;
    uint16_t *const apriv = rlds + kRMax * kRBS + wave * kRPrivate;
    const int K = (int)g.K, N = (int)g.N;

    // B[N x K] -> LDS, zero beyond N and K up to the tile edges that the MFMAs read
    {
        const int kp = FAST ? KS * kRCK : (K + kRCK - 1) / kRCK * kRCK, vec_per_row = kp / 8;
        const int items = 32 * TN * vec_per_row;
        for (int id = threadIdx.x; id < items; id += kRWaves * 64) {
            const int row = id / vec_per_row, q = id % vec_per_row;
            uint4 v = zero4();
            if (row < N && q * 8 < K) v = load8(g.B + (int64_t)row * g.ldb + q * 8, min(8, K - q * 8), g.b_vec);
            *reinterpret_cast<uint4 *>(bres + row * kRBS + q * 8) = v;
        }
    }
    __syncthreads();

    const int n_kc = (K + kRCK - 1) / kRCK;
    const int64_t n_panels = (g.M + 31) / 32;
    const int64_t first = (int64_t)blockIdx.x * kRWaves + wave, stride = (int64_t)gridDim.x * kRWaves;
    if (first >= n_panels) return;

    // lane (r, half) owns elements 16 half .. 16 half + 15 of row r of a chunk
    const int r = lane >> 1, half = lane & 1;
    int64_t f_panel = first;
    int f_kc = 0;
    uint4 ring[kRing][2], mring[MASKED ? kRing : 1][2];
    uint4 pb_cur[KS / 4], pb_next[KS / 4];  // bit mask: word kc of the lane's row covers chunk position kc
#pragma unroll
    for (int q = 0; q < KS / 4; ++q) pb_cur[q] = pb_next[q] = make_uint4(~0u, ~0u, ~0u, ~0u);
    // byte offsets of a lane's row inside a panel (in the last panel: clamped to the last row of the matrix) and of the last
    // eight columns, to which a lane's columns are clamped; the host keeps 128 leading dimensions below 2^32 bytes for the
    // unconditional kernel
    uint32_t a_off = 0, a_off_last = 0, m_off = 0, m_off_last = 0, w_off = 0, w_off_last = 0;
    const uint32_t k_last = 2u * (uint32_t)(K - 8);
    if constexpr (FAST) {
        const uint32_t row_last = (uint32_t)min(r, (int)(g.M - (n_panels - 1) * 32) - 1);
        a_off = (uint32_t)r * (uint32_t)g.lda * 2u;
        a_off_last = row_last * (uint32_t)g.lda * 2u;
        if constexpr (MASKED) m_off = (uint32_t)r * (uint32_t)g.ldmask * 2u, m_off_last = row_last * (uint32_t)g.ldmask * 2u;
        if constexpr (BITS) w_off = (uint32_t)r * (uint32_t)g.ldw * 4u, w_off_last = row_last * (uint32_t)g.ldw * 4u;
    }
    // `pos`, `of_panel`: the position a request is for (the unconditional form takes them from its caller, where they are
    // compile-time and loop-invariant values; the guarded form follows its cursor)
    auto fetch = [&](uint4(&dst)[2], uint4(&mdst)[2], int pos, int64_t of_panel) __attribute__((always_inline)) {
        if constexpr (FAST) {
            // the panel's address is the same in every lane (scalar arithmetic); a lane adds a 32-bit byte offset that does
            // not depend on the panel, except that the rows of the last panel are clamped into the matrix
            const int64_t panel = min(of_panel, n_panels - 1);
            const bool last = panel == n_panels - 1;
            const char *const pa = reinterpret_cast<const char *>(g.A) + panel * 64 * g.lda;
            const char *const pm = MASKED ? reinterpret_cast<const char *>(g.mask) + panel * 64 * g.ldmask : nullptr;
            if constexpr (BITS) {
                if (pos == 0) {
                    const char *const pw = reinterpret_cast<const char *>(g.mask_bits) + panel * 128 * g.ldw + (last ? w_off_last : w_off);
#pragma unroll
                    for (int q = 0; q < KS / 4; ++q) pb_next[q] = *reinterpret_cast<const uint4 *>(pw + 16 * q);
                }
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t k_off = min((uint32_t)(pos * kRCK * 2 + half * 32 + 16 * j), k_last);
                dst[j] = *reinterpret_cast<const uint4 *>(pa + ((last ? a_off_last : a_off) + k_off));
                if constexpr (MASKED) mdst[j] = *reinterpret_cast<const uint4 *>(pm + ((last ? m_off_last : m_off) + k_off));
            }
            return;
        }
        if (f_kc < n_kc && f_panel < n_panels) {
            const int64_t row = f_panel * 32 + r;
            const int k = f_kc * kRCK + half * 16;
            const uint16_t *pa = g.A + row * g.lda + k;
            const uint16_t *pm = MASKED ? g.mask + row * g.ldmask + k : nullptr;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 v = zero4(), m = zero4();
                if (row < g.M && k + 8 * j < K) {  // element loads when an operand does not allow 16-byte ones
                    const int valid = min(8, K - k - 8 * j);
                    v = load8(pa + 8 * j, valid, g.a_vec);
                    if constexpr (MASKED) m = load8(pm + 8 * j, valid, g.m_vec);
                }
                dst[j] = v;
                if constexpr (MASKED) mdst[j] = m;
            }
        }
        if (++f_kc == kSteps) {
            f_kc = 0;
            f_panel += stride;
        }
    };

    floatx16 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

    uint16_t *const a_dst = apriv + r * kRAS + half * 16;
    const uint16_t *const a_src = apriv + li * kRAS + 8 * h;
    const uint16_t *const b_src = bres + li * kRBS + 8 * h;

    int64_t cur_panel = first;
    auto step = [&](int kc, uint4(&cur)[2], uint4(&mcur)[2]) __attribute__((always_inline)) {
        const bool live = FAST || kc < n_kc;  // the unconditional kernel multiplies every position: no branch around its requests
        if (live) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 v = cur[j];
                if constexpr (MASKED) v = mask8(v, mcur[j]);
                if constexpr (BITS) {
                    const uint4 w4 = pb_cur[kc >> 2];
                    const uint32_t word = (kc & 3) == 0 ? w4.x : ((kc & 3) == 1 ? w4.y : ((kc & 3) == 2 ? w4.z : w4.w));
                    v = mask8_bits(v, word >> (16 * half + 8 * j));
                }
                *reinterpret_cast<uint4 *>(a_dst + 8 * j) = v;
            }
            plx::wave_lds_fence();  // the chunk other lanes stored is read below
        }
        fetch(cur, mcur, (kc + kRing) % kSteps, cur_panel + ((kc + kRing) / kSteps) * stride);
        if (live) {
#pragma unroll
            for (int s = 0; s < kRCK / 16; ++s) {
                const bf16x8 a = *reinterpret_cast<const bf16x8 *>(a_src + 16 * s);
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    const bf16x8 b = *reinterpret_cast<const bf16x8 *>(b_src + t * 32 * kRBS + kc * kRCK + 16 * s);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
                }
            }
            plx::wave_lds_fence();  // the next position (or the epilogue) overwrites the private tile
        }
    };

    const bool relu = (g.flags & PLX_GEMM_RELU) != 0;
    const bool drop = (g.flags & PLX_GEMM_DROPOUT) != 0;
    uint16_t *const C = static_cast<uint16_t *>(g.C);
    float *const cs = reinterpret_cast<float *>(apriv);
    const int srow = lane >> 2, scq = lane & 3;  // staged half tile: this lane reads 8 columns of row srow

    uint32_t wkeep[2][(TN + 3) / 4] = {};
    // a finished panel: scaling, ReLU, dropout, sign bits, stores; leaves the accumulators zero
    auto finish_panel = [&](int64_t panel) __attribute__((always_inline)) {
        // register v of a lane is row 8 (v / 4) + 4 h + v % 4, column lane % 32 of each 32 x 32 block
        // A contiguous C whose rows are not multiples of 16 bytes (47 columns): 16 rows of it are still one aligned run of 32 N
        // bytes.  The half panel is staged row-major as bf16 without padding (N <= 64 here)
        // and leaves in 16-byte stores.
        if constexpr (TN <= 2) if (g.c_flat) {  // (N <= 64: the wider kernels have no registers to spare for a second epilogue)
            uint16_t *const stage = apriv;  // [16][N]
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
                for (int t = 0; t < TN; ++t) {
#pragma unroll
                    for (int v = 0; v < 8; ++v) {
                        float x = acc[t][8 * pass + v] * g.alpha;
                        if (relu) x = fmaxf(x, 0.f);
                        if (li + t * 32 < N) stage[(8 * (v / 4) + 4 * h + (v % 4)) * N + t * 32 + li] = (uint16_t)plx::f32_to_bf16(x);
                        acc[t][8 * pass + v] = 0.f;
                    }
                }
                plx::wave_lds_fence();
                const int64_t row_first = panel * 32 + 16 * pass;
                const int valid = (int)min(max(g.M - row_first, (int64_t)0), (int64_t)16) * N;  // elements of this half panel that exist
                uint16_t *const dst = C + row_first * N;
                for (int i = 8 * lane; i < valid; i += 512) {
                    if (i + 8 <= valid) {
                        *reinterpret_cast<uint4 *>(dst + i) = *reinterpret_cast<const uint4 *>(stage + i);
                    } else {
                        for (int e = i; e < valid; ++e) dst[e] = stage[e];
                    }
                }
                plx::wave_lds_fence();  // the next half, or the next panel's first chunk, overwrites the staging
            }
            return;
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) {
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
                for (int v = 0; v < 8; ++v) cs[(8 * (v / 4) + 4 * h + (v % 4)) * kRCS + li] = acc[t][8 * pass + v];
                plx::wave_lds_fence();  // staged by all lanes, read back transposed
                const float4 lo = *reinterpret_cast<const float4 *>(cs + srow * kRCS + scq * 8);
                const float4 hi = *reinterpret_cast<const float4 *>(cs + srow * kRCS + scq * 8 + 4);
                plx::wave_lds_fence();  // before the next pass (or the next panel's chunks) overwrites the tile
                const int64_t row = panel * 32 + 16 * pass + srow;
                const int col = t * 32 + scq * 8;
                uint32_t positive = 0;  // bit e: element col + e of this row is stored positive
                if (row < g.M && col < N) {
                    float x[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        x[e] *= g.alpha;
                        if (relu) x[e] = fmaxf(x[e], 0.f);
                    }
                    if (drop) {
                        const uint64_t q = ((uint64_t)row * (uint64_t)N + (uint64_t)col) >> 3;  // N % 8 == 0: 8 aligned elements
                        const plx::Philox4 rnd = plx::philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), g.off_lo, g.off_hi, g.seed_lo, g.seed_hi);
#pragma unroll
                        for (int e = 0; e < 8; ++e) x[e] = plx::dropout_lane16(rnd, e) >= g.thresh16 ? x[e] * g.keep_scale : 0.f;
                    }
                    const uint4 packed = make_uint4(plx::pack_bf16x2(x[0], x[1]), plx::pack_bf16x2(x[2], x[3]),
                                                    plx::pack_bf16x2(x[4], x[5]), plx::pack_bf16x2(x[6], x[7]));
                    *reinterpret_cast<uint4 *>(C + row * g.ldc + col) = packed;
                    if constexpr (WBITS) {
                        // a stored bf16 is positive exactly when its 16 bits, read as a signed integer, are: two packed
                        // integer operations turn both halves of a word into 0 or 1
                        typedef short short2_t __attribute__((ext_vector_type(2)));
                        const uint32_t pk[4] = {packed.x, packed.y, packed.z, packed.w};
                        uint32_t both = 0;  // bit 2 e: element 2 e; bit 16 + 2 e: element 2 e + 1
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            short2_t hv = __builtin_bit_cast(short2_t, pk[e]);
                            hv = __builtin_elementwise_max(__builtin_elementwise_min(hv, (short2_t){1, 1}), (short2_t){0, 0});
                            both |= __builtin_bit_cast(uint32_t, hv) << (2 * e);
                        }
                        positive = (both & 0x55u) | ((both >> 15) & 0xaau);
                    }
                }
                if constexpr (WBITS) {
                    // the four lanes of a row hold its 32 columns of this tile: one word, which lane t % 4 of them keeps, so
                    // that a row's words leave in two stores of all 64 lanes per half panel rather than one of 16 per tile
                    int word = (int)(positive << (8 * scq));
                    word |= __builtin_amdgcn_update_dpp(0, word, 0xB1, 0xF, 0xF, true);  // lanes 1 0 3 2 of the quad
                    word |= __builtin_amdgcn_update_dpp(0, word, 0x4E, 0xF, 0xF, true);  // lanes 2 3 0 1
                    if ((t & 3) == scq) wkeep[pass][t >> 2] = (uint32_t)word;
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
        }
        if constexpr (WBITS) {
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                const int64_t row = panel * 32 + 16 * pass + srow;
#pragma unroll
                for (int q = 0; q < (TN + 3) / 4; ++q)
                    if (row < g.M && (scq + 4 * q) * 32 < N) g.relu_bits[row * g.ldw_out + scq + 4 * q] = wkeep[pass][q];
            }
        }
    };

#pragma unroll
    for (int i = 0; i < kRing; ++i) fetch(ring[i], mring[MASKED ? i : 0], i, first);

    if constexpr (FAST) {
        // The positions run as a pipeline inside the wavefront: the pieces of B are read kPiecesAhead products before the product
        // that takes them (B is resident, so this runs across positions and panels), the next position of A goes to the
        // private tile in the middle of the current one -- the tile is free once the current position's operands are in
        // registers -- and comes back as operands before the current one ends.  The order written here is pinned: an empty
        // asm statement takes each product's result as its operand, and a scheduling barrier follows.
        constexpr int kPiecesAhead = (MASKED && TN > 6) ? 1 : 4;  // (the widest kernel that carries mask values has registers for one)
        constexpr int kPer = 2 * TN;   // products of a position
        constexpr int kStoreAt = TN;   // the product before which the next position is stored
        static_assert(kRing == 4 && (kSteps * kPer) % kPiecesAhead == 0, "buffers are chosen by compile-time counts");
        bf16x8 aa[2][2], bq[kPiecesAhead];
        auto load_a = [&](bf16x8(&a)[2]) __attribute__((always_inline)) {
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) a[sub] = *reinterpret_cast<const bf16x8 *>(a_src + 16 * sub);
        };
        auto load_b = [&](bf16x8 &b, int kc, int idx) __attribute__((always_inline)) {
            b = *reinterpret_cast<const bf16x8 *>(b_src + (idx % TN) * 32 * kRBS + kc * kRCK + 16 * (idx / TN));
        };
        auto store_chunk = [&](const uint4(&c)[2], const uint4(&mc)[2], const uint4(&pb)[KS / 4], int kc) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 v = c[j];
                if constexpr (MASKED) v = mask8(v, mc[j]);
                if constexpr (BITS) {
                    const uint4 w4 = pb[kc >> 2];
                    const uint32_t word = (kc & 3) == 0 ? w4.x : ((kc & 3) == 1 ? w4.y : ((kc & 3) == 2 ? w4.z : w4.w));
                    v = mask8_bits(v, word >> (16 * half + 8 * j));
                }
                *reinterpret_cast<uint4 *>(a_dst + 8 * j) = v;
            }
        };
        if constexpr (BITS) {
#pragma unroll
            for (int q = 0; q < KS / 4; ++q) pb_cur[q] = pb_next[q];
        }
        store_chunk(ring[0], mring[0], pb_cur, 0);
        plx::wave_lds_fence();
        load_a(aa[0]);
#pragma unroll
        for (int d = 0; d < kPiecesAhead; ++d) load_b(bq[d], (d / kPer) % kSteps, d % kPer);
        plx::wave_lds_fence();

        for (int64_t panel = first; panel < n_panels; panel += stride) {
#pragma unroll
            for (int kc = 0; kc < kSteps; ++kc) {
                const bool wrap = kc + 1 == kSteps;  // the next position is the first of this wavefront's next panel
                const int nc = wrap ? 0 : kc + 1, slot = (kc + 1) % kRing;
#pragma unroll
                for (int idx = 0; idx < kPer; ++idx) {
                    const int count = kc * kPer + idx;  // products since the panel began
                    if (idx == kStoreAt) {
                        plx::wave_lds_fence();  // after the loads of this position's operands (and a finished panel's staging)
                        store_chunk(ring[slot], mring[MASKED ? slot : 0], wrap ? pb_next : pb_cur, nc);
                        if constexpr (BITS) {
                            if (wrap) {  // before a request replaces them with the bits of the panel after
#pragma unroll
                                for (int q = 0; q < KS / 4; ++q) pb_cur[q] = pb_next[q];
                            }
                        }
                        // requests go out for two positions at a time, which share their 128-byte lines: positions kc + 4
                        // and kc + 5 into the slots of positions kc and kc + 1, both stored by now
                        if ((kc & 1) == 0) {
                            fetch(ring[kc % kRing], mring[MASKED ? kc % kRing : 0], (kc + kRing) % kSteps, panel + ((kc + kRing) / kSteps) * stride);
                            fetch(ring[slot], mring[MASKED ? slot : 0], (kc + 1 + kRing) % kSteps, panel + ((kc + 1 + kRing) / kSteps) * stride);
                        }
                        plx::wave_lds_fence();
                        load_a(aa[(kc + 1) & 1]);
                        plx::wave_lds_fence();
                    }
                    acc[idx % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aa[kc & 1][idx / TN], bq[count % kPiecesAhead], acc[idx % TN], 0, 0, 0);
                    asm volatile("" : "+v"(acc[idx % TN]));
                    const int ahead = count + kPiecesAhead;  // the product that takes the piece read now, into the buffer just used
                    load_b(bq[count % kPiecesAhead], (ahead / kPer) % kSteps, ahead % kPer);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            plx::wave_lds_fence();  // the staging of the panel comes after the loads of the next position's operands
            finish_panel(panel);
        }
        return;
    }

    for (int64_t panel = first; panel < n_panels; panel += stride) {
        cur_panel = panel;
        if constexpr (BITS) {  // the bits that came with this panel's first chunk; the steps below fetch the next panel's
#pragma unroll
            for (int q = 0; q < KS / 4; ++q) pb_cur[q] = pb_next[q];
        }
#pragma unroll
        for (int i = 0; i < kSteps; ++i) step(i, ring[i % kRing], mring[MASKED ? i % kRing : 0]);
        finish_panel(panel);
    }
}

template <int TN, int MASK, bool FAST, int KS, bool WBITS = false>
int launch_nt_resident_one(const Bf16Args &g, unsigned blocks, hipStream_t st)
{
    static std::atomic<uint64_t> allowed{0};  // devices on which this instantiation may take its LDS
    const int rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_bf16_nt_resident_kernel<TN, MASK, FAST, KS, WBITS>), kRLdsBytes,
                                          allowed);
    if (rc != PLX_OK) return rc;
    gemm_bf16_nt_resident_kernel<TN, MASK, FAST, KS, WBITS><<<blocks, kRWaves * 64, kRLdsBytes, st>>>(g);
    return PLX_OK;
}

// operands that take 16-byte loads go to the kernel whose requests are unconditional, with as many chunk positions as K needs
// whether the resident kernel can read the mask of this product as bits: the unconditional form, rows of bits that take
// 16-byte loads and hold a word for every chunk position the kernel walks
// the unconditional kernel's lanes address a panel with 32-bit byte offsets
bool resident_offsets_fit(const Bf16Args &g)
{
    const int64_t ld_max = (int64_t)1 << 24;
    return g.lda < ld_max && g.ldmask < ld_max && g.ldw < ld_max;
}

bool resident_takes_bits(const Bf16Args &g)
{
    if (g.mask_bits == nullptr || !(g.a_vec && g.K % 8 == 0 && g.K >= 8) || !resident_offsets_fit(g)) return false;
    const int64_t words = g.K <= 4 * kRCK ? 4 : 8;
    return reinterpret_cast<uintptr_t>(g.mask_bits) % 16 == 0 && g.ldw % 4 == 0 && g.ldw >= words;
}

template <int TN, bool MASKED>
int launch_nt_resident(const Bf16Args &g, unsigned blocks, hipStream_t st)
{
    if constexpr (MASKED) {
        if (resident_takes_bits(g)) {
            if (g.K <= 4 * kRCK) return launch_nt_resident_one<TN, 2, true, 4>(g, blocks, st);
            return launch_nt_resident_one<TN, 2, true, 8>(g, blocks, st);
        }
    }
    constexpr int MASK = MASKED ? 1 : 0;
    if (g.a_vec && g.m_vec && g.K % 8 == 0 && g.K >= 8 && resident_offsets_fit(g)) {
        if constexpr (!MASKED) {
            if (g.relu_bits != nullptr) {
                if (g.K <= 4 * kRCK) return launch_nt_resident_one<TN, 0, true, 4, true>(g, blocks, st);
                return launch_nt_resident_one<TN, 0, true, 8, true>(g, blocks, st);
            }
        }
        if (g.K <= 4 * kRCK) return launch_nt_resident_one<TN, MASK, true, 4>(g, blocks, st);
        return launch_nt_resident_one<TN, MASK, true, 8>(g, blocks, st);
    }
    return launch_nt_resident_one<TN, MASK, false, 8>(g, blocks, st);
}

// ------------------------------------------------------------------------------------------------
// TN: C[K x N] (fp32) = alpha * A[M x K]^T . (B*mask)[M x N]; contraction over the rows of both
// ------------------------------------------------------------------------------------------------
template <int TN, bool MASKED, bool VEC>
__global__ void __launch_bounds__(kThreads) gemm_bf16_tn_kernel(const Bf16Args g)
{
    constexpr int BN = 32 * TN;
    constexpr int kAItems = 32 * (kBM / 8) / kThreads;                      // (row pair, 8-column vector) items per thread
    constexpr int kBItems = (32 * (BN / 8) + kThreads - 1) / kThreads;
    constexpr int kTile = (kBM + BN) * kS;

    __shared__ __attribute__((aligned(16))) uint16_t lds[2 * kTile];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 31;
    const int h = lane >> 5;
    const int64_t row0 = (int64_t)blockIdx.y * kBM;  // rows of C = columns of A
    const int64_t col0 = (int64_t)blockIdx.z * BN;   // columns of C = columns of B
    const int64_t mbeg = (int64_t)blockIdx.x * g.rows_per_split;
    const int64_t mend = min(mbeg + g.rows_per_split, g.M);

    // thread (mp, cq0) owns the row pair (2 mp, 2 mp + 1) and the column vectors cq0, cq0 + 8, ... of a chunk;
    // pointers walk down the rows chunk by chunk, so a fetch costs pointer steps and 32-bit compares only
    const int mp = threadIdx.x & 31;
    const int cq0 = threadIdx.x >> 5;
    const uint16_t *pa = g.A + (mbeg + 2 * mp) * g.lda + row0 + cq0 * 8;
    const uint16_t *pb = g.B + (mbeg + 2 * mp) * g.ldb + col0 + cq0 * 8;
    const uint16_t *pm = MASKED ? g.mask + (mbeg + 2 * mp) * g.ldmask + col0 + cq0 * 8 : nullptr;
    const int a_cols = (int)min(max(g.K - row0 - cq0 * 8, (int64_t)0), (int64_t)kBM);  // columns 64 p + e with 64 p + e < a_cols exist
    const int b_cols = (int)min(max(g.N - col0 - cq0 * 8, (int64_t)0), (int64_t)BN);

    uint4 ra[kAItems][2], rb[kBItems][2], rmk[MASKED ? kBItems : 1][2];  // mask applied at the stash, not at the load
    auto fetch = [&](int64_t m0) {
        const int rows_left = (int)min(mend - m0 - 2 * mp, (int64_t)2);  // 2: both rows of the pair exist
#pragma unroll
        for (int p = 0; p < kAItems; ++p) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 v = zero4();
                if (j < rows_left && 64 * p < a_cols) {
                    if constexpr (VEC)
                        v = *reinterpret_cast<const uint4 *>(pa + j * g.lda + 64 * p);
                    else
                        v = load8(pa + j * g.lda + 64 * p, min(8, a_cols - 64 * p), g.a_vec);
                }
                ra[p][j] = v;
            }
        }
#pragma unroll
        for (int p = 0; p < kBItems; ++p) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 v = zero4(), mk = zero4();
                if (j < rows_left && 64 * p < b_cols && 64 * p + cq0 * 8 < BN) {
                    if constexpr (VEC) {
                        v = *reinterpret_cast<const uint4 *>(pb + j * g.ldb + 64 * p);
                        if constexpr (MASKED) mk = *reinterpret_cast<const uint4 *>(pm + j * g.ldmask + 64 * p);
                    } else {
                        const int valid = min(8, b_cols - 64 * p);
                        v = load8(pb + j * g.ldb + 64 * p, valid, g.b_vec);
                        if constexpr (MASKED) mk = load8(pm + j * g.ldmask + 64 * p, valid, g.m_vec);
                    }
                }
                rb[p][j] = v;
                if constexpr (MASKED) rmk[p][j] = mk;
            }
        }
        pa += (int64_t)kBK * g.lda;
        pb += (int64_t)kBK * g.ldb;
        if constexpr (MASKED) pm += (int64_t)kBK * g.ldmask;
    };
    // transposed stash: word e of the pair holds (row 2 mp, row 2 mp + 1) of column 8 cq + e
    auto stash_pair = [&](uint16_t *t, int mp, int cq, const uint4 &r0, const uint4 &r1) {
        const uint32_t a[4] = {r0.x, r0.y, r0.z, r0.w};
        const uint32_t b[4] = {r1.x, r1.y, r1.z, r1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t lo = (e & 1) ? (a[e >> 1] >> 16) : (a[e >> 1] & 0xffffu);
            const uint32_t hi = (e & 1) ? (b[e >> 1] >> 16) : (b[e >> 1] & 0xffffu);
            *reinterpret_cast<uint32_t *>(t + (cq * 8 + e) * kS + 2 * mp) = lo | (hi << 16);
        }
    };
    auto stash = [&](int buf) {
        uint16_t *at = lds + buf * kTile;
        uint16_t *bt = at + kBM * kS;
#pragma unroll
        for (int p = 0; p < kAItems; ++p) stash_pair(at, mp, cq0 + 8 * p, ra[p][0], ra[p][1]);
#pragma unroll
        for (int p = 0; p < kBItems; ++p)
            if (cq0 + 8 * p < BN / 8) {
                if constexpr (MASKED)
                    stash_pair(bt, mp, cq0 + 8 * p, mask8(rb[p][0], rmk[p][0]), mask8(rb[p][1], rmk[p][1]));
                else
                    stash_pair(bt, mp, cq0 + 8 * p, rb[p][0], rb[p][1]);
            }
    };

    floatx16 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

    int buf = 0;
    if (mbeg < mend) {
        fetch(mbeg);
        stash(0);
    }
    __syncthreads();
    for (int64_t m0 = mbeg; m0 < mend; m0 += kBK) {
        const bool more = m0 + kBK < mend;
        if (more) fetch(m0 + kBK);
        const uint16_t *at = lds + buf * kTile;
        const uint16_t *bt = at + kBM * kS;
#pragma unroll
        for (int s = 0; s < kBK / 16; ++s) {
            const bf16x8 a = *reinterpret_cast<const bf16x8 *>(at + (wave * 32 + li) * kS + 16 * s + 8 * h);
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const bf16x8 b = *reinterpret_cast<const bf16x8 *>(bt + (t * 32 + li) * kS + 16 * s + 8 * h);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
            }
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    float *out;
    int64_t ldo;
    float scale;
    if (g.ws != nullptr) {
        out = g.ws + (int64_t)blockIdx.x * g.ws_slab;
        ldo = g.ws_ld;
        scale = 1.f;  // alpha is applied when the partial tiles are added
    } else {
        out = static_cast<float *>(g.C);
        ldo = g.ldc;
        scale = g.alpha;
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        const int64_t c = col0 + t * 32 + li;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t r = row0 + wave * 32 + 8 * (v / 4) + 4 * h + (v % 4);
            if (c < g.N && r < g.K) out[r * ldo + c] = acc[t][v] * scale;
        }
    }
}

// The same product for K and N up to 256 where one of them exceeds 128: with 128 x 128 tiles a workgroup reads half of A
// and half of B, so every operand crosses the memory system twice.  Here one workgroup of 16 wavefronts owns the whole
// 256 x 256 tile of C for its stretch of rows: A, B and the mask are read once.  Wavefront w multiplies the 32 rows
// 32 (w % 8) of C by the column half w / 8.  Operands take 128-bit loads (K and N multiples of 8).  A chunk is requested
// right after the previous one has been stored to LDS, so its loads are in flight for a whole turn of the loop; whole
// chunks are fetched without a branch (a thread whose columns lie beyond K or N reads column 0 and stores nothing), so
// the compiler waits for exactly the loads it is about to use; the last, partial chunk of a stretch is fetched with guards.
// Stretches, chunk order and the order of the products inside a chunk are those of the tiled kernel: the same bits.
constexpr int kWThreads = 1024;
constexpr int kWTile = 512 * kS;  // bf16 elements per buffer: 256 columns of A and 256 of B, one LDS row each
constexpr size_t kWLdsBytes = 2 * (size_t)kWTile * sizeof(uint16_t);

// MASK: 0 none, 1 bf16 values beside B, 2 one bit per element (a thread's 8 columns of a row are one byte), 3 none and B of at
// most 64 columns in rows that take no 16-byte loads (the 47-wide gradient of a last layer), read element by element: a thread
// then owns columns cq and cq + 32 of B
template <int MASK>
__global__ void __launch_bounds__(kWThreads) gemm_bf16_tn_wide_kernel(const Bf16Args g)
{
    constexpr bool MASKED = MASK == 1;
    constexpr bool BITS = MASK == 2;
    constexpr bool BSC = MASK == 3;
    extern __shared__ __attribute__((aligned(16))) uint16_t lds_w[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 31;
    const int h = lane >> 5;
    const int rb = wave & 7, ch = wave >> 3;
    const int64_t mbeg = (int64_t)blockIdx.x * g.rows_per_split;
    const int64_t mend = min(mbeg + g.rows_per_split, g.M);

    // thread (mp, cq): row pair (2 mp, 2 mp + 1) of a chunk, columns 8 cq .. 8 cq + 7 of A and of B
    const int mp = threadIdx.x & 31;
    const int cq = threadIdx.x >> 5;
    const bool a_ok = cq * 8 < g.K, b_ok = !BSC && cq * 8 < g.N;
    const bool bs_ok[2] = {BSC && cq < g.N, BSC && cq + 32 < g.N};
    const uint16_t *pbs = g.B + (mbeg + 2 * mp) * g.ldb;
    uint32_t rbs[2][2] = {{0u, 0u}, {0u, 0u}};
    const uint16_t *pa = g.A + (mbeg + 2 * mp) * g.lda + (a_ok ? cq * 8 : 0);
    const uint16_t *pb = g.B + (mbeg + 2 * mp) * g.ldb + (b_ok ? cq * 8 : 0);
    const uint16_t *pm = MASKED ? g.mask + (mbeg + 2 * mp) * g.ldmask + (b_ok ? cq * 8 : 0) : nullptr;
    const uint8_t *pbit = BITS ? reinterpret_cast<const uint8_t *>(g.mask_bits) + (mbeg + 2 * mp) * g.ldw * 4 + (b_ok ? cq : 0) : nullptr;

    uint4 ra[2], rb2[2], rmk[2];
    uint32_t rbit[2] = {0u, 0u};
    auto advance = [&]() {
        pa += (int64_t)kBK * g.lda;
        pb += (int64_t)kBK * g.ldb;
        if constexpr (MASKED) pm += (int64_t)kBK * g.ldmask;
        if constexpr (BITS) pbit += (int64_t)kBK * g.ldw * 4;
        if constexpr (BSC) pbs += (int64_t)kBK * g.ldb;
    };
    auto fetch_whole = [&]() {  // all 64 rows of the chunk exist
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ra[j] = *reinterpret_cast<const uint4 *>(pa + j * g.lda);
            if constexpr (!BSC) rb2[j] = *reinterpret_cast<const uint4 *>(pb + j * g.ldb);
            if constexpr (MASKED) rmk[j] = *reinterpret_cast<const uint4 *>(pm + j * g.ldmask);
            if constexpr (BITS) rbit[j] = pbit[j * g.ldw * 4];
            if constexpr (BSC) {
#pragma unroll
                for (int p = 0; p < 2; ++p) rbs[p][j] = pbs[j * g.ldb + (bs_ok[p] ? cq + 32 * p : 0)];
            }
        }
        advance();
    };
    auto fetch_any = [&](int64_t m0) {
        const int rows_left = (int)min(max(mend - m0 - 2 * mp, (int64_t)0), (int64_t)2);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ra[j] = zero4();
            rb2[j] = zero4();
            rmk[j] = zero4();
            if (j < rows_left) {
                ra[j] = *reinterpret_cast<const uint4 *>(pa + j * g.lda);
                if constexpr (!BSC) rb2[j] = *reinterpret_cast<const uint4 *>(pb + j * g.ldb);
                if constexpr (MASKED) rmk[j] = *reinterpret_cast<const uint4 *>(pm + j * g.ldmask);
                if constexpr (BITS) rbit[j] = pbit[j * g.ldw * 4];
            }
            if constexpr (BSC) {
#pragma unroll
                for (int p = 0; p < 2; ++p) rbs[p][j] = j < rows_left ? (uint32_t)pbs[j * g.ldb + (bs_ok[p] ? cq + 32 * p : 0)] : 0u;
            }
        }
        advance();
    };
    // transposed stash: word e of the pair holds (row 2 mp, row 2 mp + 1) of column 8 cq + e
    auto stash_pair = [&](uint16_t *t, const uint4 &r0, const uint4 &r1) {
        const uint32_t a[4] = {r0.x, r0.y, r0.z, r0.w};
        const uint32_t b[4] = {r1.x, r1.y, r1.z, r1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t lo = (e & 1) ? (a[e >> 1] >> 16) : (a[e >> 1] & 0xffffu);
            const uint32_t hi = (e & 1) ? (b[e >> 1] >> 16) : (b[e >> 1] & 0xffffu);
            *reinterpret_cast<uint32_t *>(t + (cq * 8 + e) * kS + 2 * mp) = lo | (hi << 16);
        }
    };
    auto stash = [&](int buf) {
        uint16_t *at = lds_w + buf * kWTile;
        uint16_t *bt = at + 256 * kS;
        if (a_ok) stash_pair(at, ra[0], ra[1]);
        if constexpr (BSC) {
#pragma unroll
            for (int p = 0; p < 2; ++p)
                if (bs_ok[p]) *reinterpret_cast<uint32_t *>(bt + (cq + 32 * p) * kS + 2 * mp) = rbs[p][0] | (rbs[p][1] << 16);
        }
        if (b_ok) {
            if constexpr (MASKED)
                stash_pair(bt, mask8(rb2[0], rmk[0]), mask8(rb2[1], rmk[1]));
            else if constexpr (BITS)
                stash_pair(bt, mask8_bits(rb2[0], rbit[0]), mask8_bits(rb2[1], rbit[1]));
            else
                stash_pair(bt, rb2[0], rb2[1]);
        }
    };

    floatx16 acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
    const bool works = rb * 32 < g.K && ch * 128 < g.N;  // uniform over the wavefront
    auto compute = [&](int buf) {
        if (!works) return;
        const uint16_t *at = lds_w + buf * kWTile;
        const uint16_t *bt = at + (256 + ch * 128) * kS;
#pragma unroll
        for (int s = 0; s < kBK / 16; ++s) {
            const bf16x8 a = *reinterpret_cast<const bf16x8 *>(at + (rb * 32 + li) * kS + 16 * s + 8 * h);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const bf16x8 b = *reinterpret_cast<const bf16x8 *>(bt + (t * 32 + li) * kS + 16 * s + 8 * h);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
            }
        }
    };

    const int64_t rows = max(mend - mbeg, (int64_t)0);
    const int64_t n_chunks = (rows + kBK - 1) / kBK;
    const int64_t n_whole = rows / kBK;  // chunks 0 .. n_whole - 1 have all their rows
    // chunk 0 into buffer 0, chunk 1 requested
    if (n_chunks > 0) {
        if (n_whole > 0) fetch_whole(); else fetch_any(mbeg);
        stash(0);
    }
    if (n_chunks > 1) {
        if (n_whole > 1) fetch_whole(); else fetch_any(mbeg + kBK);
    }
    __syncthreads();
    int64_t c = 0;
    for (; c + 2 < n_whole; ++c) {  // steady state: chunk c in LDS, c + 1 in registers, c + 2 whole and about to be requested
        compute((int)(c & 1));
        stash((int)((c + 1) & 1));
        fetch_whole();
        __syncthreads();
    }
    for (; c < n_chunks; ++c) {
        compute((int)(c & 1));
        if (c + 1 < n_chunks) stash((int)((c + 1) & 1));
        if (c + 2 < n_chunks) fetch_any(mbeg + (c + 2) * kBK);
        __syncthreads();
    }

    float *out = g.ws + (int64_t)blockIdx.x * g.ws_slab;  // always split over the rows: alpha is applied when the partial tiles are added
    if (works) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int64_t col = ch * 128 + t * 32 + li;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t r = rb * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                if (col < g.N && r < g.K) out[r * g.ws_ld + col] = acc[t][v];
            }
        }
    }
}

// C[e] = alpha * sum over splits of ws[s][e]; four interleaved chains, added in chain order
__global__ void __launch_bounds__(256) gemm_bf16_tn_reduce(const float *__restrict__ ws, int64_t ws_ld, int64_t ws_slab,
                                                           int splits, int64_t rows, int64_t cols, float alpha,
                                                           float *__restrict__ C, int64_t ldc)
{
    __shared__ float part[4][64];
    const int e_local = threadIdx.x & 63;
    const int chain = threadIdx.x >> 6;
    const int64_t e = (int64_t)blockIdx.x * 64 + e_local;
    const int64_t total = rows * cols;
    float s = 0.f;
    int64_t r = 0, c = 0;
    if (e < total) {
        r = e / cols;
        c = e % cols;
        const float *p = ws + r * ws_ld + c;
        for (int i = chain; i < splits; i += 4) s += p[(int64_t)i * ws_slab];
    }
    part[chain][e_local] = s;
    __syncthreads();
    if (chain == 0 && e < total)
        C[r * ldc + c] = alpha * (((part[0][e_local] + part[1][e_local]) + part[2][e_local]) + part[3][e_local]);
}

// Y = bf16(X) or bf16(X^T): 32 x 32 tiles through LDS so that both sides are accessed along rows
__global__ void __launch_bounds__(256) cast_f32_bf16_kernel(int64_t M, int64_t N, const float *__restrict__ X, int64_t ldx,
                                                            uint16_t *__restrict__ Y, int64_t ldy, int transpose)
{
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const int64_t r0 = (int64_t)blockIdx.x * 32, c0 = (int64_t)blockIdx.y * 32;
    for (int j = ty; j < 32; j += 8) {
        const int64_t r = r0 + j, c = c0 + tx;
        tile[j][tx] = (r < M && c < N) ? X[r * ldx + c] : 0.f;
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        if (transpose) {
            const int64_t r = c0 + j, c = r0 + tx;  // Y is [N x M]
            if (r < N && c < M) Y[r * ldy + c] = (uint16_t)plx::f32_to_bf16(tile[tx][j]);
        } else {
            const int64_t r = r0 + j, c = c0 + tx;
            if (r < M && c < N) Y[r * ldy + c] = (uint16_t)plx::f32_to_bf16(tile[j][tx]);
        }
    }
}

int vec16(const void *p, int64_t ld) { return (p == nullptr || (reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 8 == 0)) ? 1 : 0; }
int pick_tn(int64_t n) { return n <= 32 ? 1 : (n <= 64 ? 2 : 4); }

int64_t tn_splits(int64_t M, int64_t N, int64_t K)
{
    const int64_t tiles = plx::ceil_div(K, kBM) * plx::ceil_div(N, 32 * pick_tn(N));
    const int64_t want = std::max<int64_t>(1, 1024 / tiles);
    const int64_t by_rows = std::max<int64_t>(1, M / 512);
    return std::max<int64_t>(1, std::min(want, by_rows));
}

template <bool MASKED, bool VEC>
void launch_nt(const Bf16Args &g, int tn, dim3 grid, hipStream_t st)
{
    switch (tn) {
        case 1: gemm_bf16_nt_kernel<1, MASKED, VEC><<<grid, kThreads, 0, st>>>(g); break;
        case 2: gemm_bf16_nt_kernel<2, MASKED, VEC><<<grid, kThreads, 0, st>>>(g); break;
        default: gemm_bf16_nt_kernel<4, MASKED, VEC><<<grid, kThreads, 0, st>>>(g); break;
    }
}

template <bool MASKED, bool VEC>
void launch_tn(const Bf16Args &g, int tn, dim3 grid, hipStream_t st)
{
    switch (tn) {
        case 1: gemm_bf16_tn_kernel<1, MASKED, VEC><<<grid, kThreads, 0, st>>>(g); break;
        case 2: gemm_bf16_tn_kernel<2, MASKED, VEC><<<grid, kThreads, 0, st>>>(g); break;
        default: gemm_bf16_tn_kernel<4, MASKED, VEC><<<grid, kThreads, 0, st>>>(g); break;
    }
}

}  // namespace

extern "C" {

int plx_gemm_nt_bf16(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                     uint16_t *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, float alpha, unsigned flags,
                     float dropout_p, uint64_t seed, uint64_t offset, void *stream)
{
    return plx_gemm_nt_bf16_bits(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, nullptr, 0, nullptr, 0, alpha, flags, dropout_p, seed,
                                 offset, stream);
}

int plx_gemm_nt_bf16_bits(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                          uint16_t *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw,
                          uint32_t *relu_bits, int64_t ldw_out, float alpha, unsigned flags, float dropout_p, uint64_t seed,
                          uint64_t offset, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm_nt_bf16: negative dimension");
    PLX_REQUIRE(N < (1ll << 30) && K < (1ll << 30), "gemm_nt_bf16: dimension too large");
    PLX_REQUIRE(M < (1ll << 40), "gemm_nt_bf16: too many rows");
    if (M == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(C != nullptr, "gemm_nt_bf16: NULL output");
    PLX_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "gemm_nt_bf16: NULL operand");
    PLX_REQUIRE(lda >= K && ldb >= K && ldc >= N, "gemm_nt_bf16: leading dimension too small");
    PLX_REQUIRE(mask == nullptr || ldmask >= K, "gemm_nt_bf16: mask leading dimension too small");
    PLX_REQUIRE(mask_bits == nullptr || (mask != nullptr && ldw >= (K + 31) / 32),
                "gemm_nt_bf16: a bit mask comes with the bf16 mask it stands for and a pitch of at least ceil(K / 32) words");
    PLX_REQUIRE(relu_bits == nullptr || ldw_out >= (N + 31) / 32, "gemm_nt_bf16: pitch of the sign bits smaller than ceil(N / 32) words");
    PLX_REQUIRE(!(flags & PLX_GEMM_DROPOUT) || (dropout_p >= 0.f && dropout_p < 1.f), "gemm_nt_bf16: dropout p=%g outside [0, 1)",
                (double)dropout_p);
    Bf16Args g{};
    g.A = A; g.B = B; g.mask = mask; g.C = C;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldmask = ldmask;
    g.M = M; g.N = N; g.K = K;
    g.alpha = alpha; g.flags = flags;
    g.thresh16 = (uint32_t)std::min<long long>(65535, llroundf(dropout_p * 65536.f));
    g.keep_scale = 1.f / (1.f - dropout_p);
    g.seed_lo = (uint32_t)seed; g.seed_hi = (uint32_t)(seed >> 32);
    g.off_lo = (uint32_t)offset; g.off_hi = (uint32_t)(offset >> 32);
    g.a_vec = vec16(A, lda); g.b_vec = vec16(B, ldb); g.c_vec = vec16(C, ldc); g.m_vec = vec16(mask, ldmask);
    g.mask_bits = mask_bits; g.ldw = ldw; g.relu_bits = relu_bits; g.ldw_out = ldw_out;
    const int tn = pick_tn(N);
    // one workgroup per (row panel, column tile); row panels are rounded up to a multiple of 8 for the XCD mapping
    const int64_t n_ct = plx::ceil_div(N, 32 * tn);
    const int64_t blocks = plx::ceil_div(plx::ceil_div(M, kBM), 8) * 8 * n_ct;
    PLX_REQUIRE(blocks < (1ll << 31), "gemm_nt_bf16: too many tiles");
    dim3 grid((unsigned)blocks, 1, 1);
    const bool vec = g.a_vec && g.b_vec && g.m_vec && K % 8 == 0;
    hipStream_t st = plx::as_stream(stream);
    g.c_flat = (!(g.c_vec && N % 8 == 0) && reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc == N && N <= 64 && (flags & PLX_GEMM_DROPOUT) == 0 &&
                relu_bits == nullptr) ? 1 : 0;
    const bool resident = ((g.c_vec && N % 8 == 0) || g.c_flat) && N <= kRMax && K <= kRMax && K > 0;
    if (relu_bits != nullptr && !(resident && mask == nullptr && g.a_vec && K % 8 == 0 && K >= 8))  // only one form of the kernel writes them
        return plx::fail(PLX_ERR_UNSUPPORTED, "gemm_nt_bf16: sign bits are written for N, K <= %d with N and K multiples of 8, 16-byte rows of A "
                                              "and C, and no mask", kRMax);
    if (resident) {
        const unsigned rblocks = (unsigned)std::min<int64_t>(plx::ceil_div(M, 32 * kRWaves), 256);
        const int rtn = (int)plx::ceil_div(N, 32);
        int rc = PLX_OK;
#define PLX_RES(T_) (mask != nullptr ? launch_nt_resident<T_, true>(g, rblocks, st) : launch_nt_resident<T_, false>(g, rblocks, st))
        switch (rtn) {
            case 1: rc = PLX_RES(1); break;
            case 2: rc = PLX_RES(2); break;
            case 3: case 4: rc = PLX_RES(4); break;
            case 5: case 6: rc = PLX_RES(6); break;
            default: rc = PLX_RES(8); break;
        }
#undef PLX_RES
        if (rc != PLX_OK) return rc;
        PLX_LAUNCH_CHECK("gemm_bf16_nt_resident_kernel");
        return PLX_OK;
    }
    if (mask != nullptr) {
        if (vec) launch_nt<true, true>(g, tn, grid, st);
        else launch_nt<true, false>(g, tn, grid, st);
    } else {
        if (vec) launch_nt<false, true>(g, tn, grid, st);
        else launch_nt<false, false>(g, tn, grid, st);
    }
    PLX_LAUNCH_CHECK("gemm_bf16_nt_kernel");
    return PLX_OK;
}

size_t plx_gemm_tn_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const int64_t splits = tn_splits(M, N, K);
    if (splits <= 1) return 0;
    const int64_t ld = (N + 3) / 4 * 4;
    return (size_t)splits * (size_t)K * (size_t)ld * sizeof(float);
}

int plx_gemm_tn_bf16(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                     float *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, float alpha, void *workspace,
                     size_t workspace_bytes, void *stream)
{
    return plx_gemm_tn_bf16_bits(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, nullptr, 0, alpha, workspace, workspace_bytes, stream);
}

int plx_gemm_tn_bf16_bits(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                          float *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw,
                          float alpha, void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm_tn_bf16: negative dimension");
    if (K == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(C != nullptr, "gemm_tn_bf16: NULL output");
    PLX_REQUIRE(M == 0 || (A != nullptr && B != nullptr), "gemm_tn_bf16: NULL operand");
    PLX_REQUIRE(lda >= K && ldb >= N && ldc >= N, "gemm_tn_bf16: leading dimension too small");
    PLX_REQUIRE(mask == nullptr || ldmask >= N, "gemm_tn_bf16: mask leading dimension too small");
    PLX_REQUIRE(mask_bits == nullptr || (mask != nullptr && ldw >= (N + 31) / 32),
                "gemm_tn_bf16: a bit mask comes with the bf16 mask it stands for and a pitch of at least ceil(N / 32) words");
    hipStream_t st = plx::as_stream(stream);
    const int64_t splits = tn_splits(std::max<int64_t>(M, 1), N, K);
    const size_t need = plx_gemm_tn_bf16_workspace_bytes(M, N, K);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need))
        return plx::fail(PLX_ERR_WORKSPACE, "gemm_tn_bf16: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    Bf16Args g{};
    g.A = A; g.B = B; g.mask = mask; g.C = C;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldmask = ldmask;
    g.M = M; g.N = N; g.K = K; g.alpha = alpha;
    g.a_vec = vec16(A, lda); g.b_vec = vec16(B, ldb); g.m_vec = vec16(mask, ldmask);
    g.mask_bits = mask_bits; g.ldw = ldw;  // read by the whole-tile kernel; the tiled one takes the values
    g.rows_per_split = plx::ceil_div(plx::ceil_div(std::max<int64_t>(M, 1), splits), kBK) * kBK;
    const int64_t used = plx::ceil_div(std::max<int64_t>(M, 1), g.rows_per_split);
    if (splits > 1) {
        g.ws = static_cast<float *>(workspace);
        g.ws_ld = (N + 3) / 4 * 4;
        g.ws_slab = K * g.ws_ld;
    }
    const int tn = pick_tn(N);
    dim3 grid((unsigned)used, (unsigned)plx::ceil_div(K, kBM), (unsigned)plx::ceil_div(N, 32 * tn));
    const bool vec = g.a_vec && g.b_vec && g.m_vec && K % 8 == 0 && N % 8 == 0;
    const bool b_scalar = !vec && splits > 1 && g.a_vec && K % 8 == 0 && K <= 256 && N <= 64 && mask == nullptr;
    if (b_scalar) {
        // a narrow B in rows without 16-byte alignment: the whole-tile kernel reads it element by element
        static std::atomic<uint64_t> allowed_s{0};
        const int rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_bf16_tn_wide_kernel<3>), kWLdsBytes, allowed_s);
        if (rc != PLX_OK) return rc;
        gemm_bf16_tn_wide_kernel<3><<<(unsigned)used, kWThreads, kWLdsBytes, st>>>(g);
        PLX_LAUNCH_CHECK("gemm_bf16_tn_wide_kernel");
    } else if (vec && splits > 1 && K <= 256 && N <= 256 && (K > kBM || N > 128)) {
        // more than one 128 x 128 tile, at most 256 x 256: one workgroup per stretch holds the whole tile and reads every operand once
        static std::atomic<uint64_t> allowed_b{0}, allowed_m{0}, allowed_p{0};
        int rc;
        if (g.mask_bits != nullptr) {  // a row of bits holds at least ceil(N / 32) words: the bytes this kernel reads
            rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_bf16_tn_wide_kernel<2>), kWLdsBytes, allowed_b);
            if (rc == PLX_OK) gemm_bf16_tn_wide_kernel<2><<<(unsigned)used, kWThreads, kWLdsBytes, st>>>(g);
        } else if (mask != nullptr) {
            rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_bf16_tn_wide_kernel<1>), kWLdsBytes, allowed_m);
            if (rc == PLX_OK) gemm_bf16_tn_wide_kernel<1><<<(unsigned)used, kWThreads, kWLdsBytes, st>>>(g);
        } else {
            rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_bf16_tn_wide_kernel<0>), kWLdsBytes, allowed_p);
            if (rc == PLX_OK) gemm_bf16_tn_wide_kernel<0><<<(unsigned)used, kWThreads, kWLdsBytes, st>>>(g);
        }
        if (rc != PLX_OK) return rc;
        PLX_LAUNCH_CHECK("gemm_bf16_tn_wide_kernel");
    } else if (mask != nullptr) {
        if (vec) launch_tn<true, true>(g, tn, grid, st);
        else launch_tn<true, false>(g, tn, grid, st);
    } else {
        if (vec) launch_tn<false, true>(g, tn, grid, st);
        else launch_tn<false, false>(g, tn, grid, st);
    }
    PLX_LAUNCH_CHECK("gemm_bf16_tn_kernel");
    if (splits > 1) {
        gemm_bf16_tn_reduce<<<(unsigned)plx::ceil_div(K * N, 64), 256, 0, st>>>(g.ws, g.ws_ld, g.ws_slab, (int)used, K, N, alpha, C, ldc);
        PLX_LAUNCH_CHECK("gemm_bf16_tn_reduce");
    }
    return PLX_OK;
}

int plx_cast_f32_bf16(int64_t M, int64_t N, const float *X, int64_t ldx, uint16_t *Y, int64_t ldy, int transpose, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0, "cast_f32_bf16: negative shape");
    if (M == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(X && Y, "cast_f32_bf16: NULL operand");
    PLX_REQUIRE(ldx >= N && ldy >= (transpose ? M : N), "cast_f32_bf16: leading dimension too small");
    PLX_REQUIRE(N <= 32ll * 65535, "cast_f32_bf16: too many columns");
    dim3 grid((unsigned)plx::ceil_div(M, 32), (unsigned)plx::ceil_div(N, 32), 1);
    cast_f32_bf16_kernel<<<grid, 256, 0, plx::as_stream(stream)>>>(M, N, X, ldx, Y, ldy, transpose);
    PLX_LAUNCH_CHECK("cast_f32_bf16_kernel");
    return PLX_OK;
}

}  // extern "C"
