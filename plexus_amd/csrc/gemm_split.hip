// fp32 dense products of the GCN layer on the bf16 matrix cores: every fp32 operand is split exactly into three
// bf16 pieces, x = x0 + x1 + x2 (8 + 8 + 8 mantissa bits, each piece the round-to-nearest bf16 of what the
// previous ones left), and the product is accumulated in fp32 from the six piece products
//     a0.b0 + a0.b1 + a1.b0 + a1.b1 + a0.b2 + a2.b0
// -- the terms left out (a1.b2, a2.b1, a2.b2) are below 2^-24 of the result, the rounding level of an fp32
// product.  v_mfma_f32_32x32x16_bf16 runs at 16 times the rate of the fp32 MFMA, so six of them still cost
// 2.7 times less matrix-core time, which moves these tall-skinny products from the MFMA bound to the HBM bound.
//
//   NT form   C[M x N] = epilogue((A*mask)[M x K] . Bp[N x K]^T)     A, mask, C fp32 in memory;
//             Bp = the three bf16 planes of the small operand, made once per call by split_planes_kernel:
//               forward   OUT      = AGG . W         Bp = planes of W^T   (+ ReLU)
//               backward  GRAD_AGG = GRAD_OUT . W^T  Bp = planes of W     (+ ReLU mask on GRAD_OUT)
//             (GRAD_W = AGG^T . GRAD_OUT, the reduction over the rows, runs on the fp32 MFMA: gemm.hip)
//
// The large operand is read as fp32 with 128-bit loads, split in registers and stored to LDS as three bf16
// planes; an MFMA lane then reads its 8 consecutive contraction elements of a plane with one 128-bit LDS load.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "bf16.h"
#include "common.h"
#include "split.h"

namespace {

using namespace plx::split;

constexpr int kBM = 128;     // rows of the large operand per workgroup tile
constexpr int kBK = 32;      // contraction chunk
constexpr int kS = kBK + 8;  // LDS row stride of a plane in bf16 elements (80 bytes: 128-bit reads conflict-free)
constexpr int kThreads = 256;

// four floats at an address that is a multiple of 4 only
struct __attribute__((packed, aligned(4))) Float4Align4 {
    float x, y, z, w;
};

struct SplitArgs {
    const float *A;
    const float *mask;
    const uint16_t *Bp;  // [3][Np][Kp] bf16 planes, zero padded
    float *C;
    int64_t lda, ldmask, ldc;
    int64_t M, N, K;
    int64_t Np, Kp;
    unsigned flags;
    unsigned *nonfinite;  // device word raised when an operand holds a value the split cannot carry
    int a_vec;  // A (and mask) 16-byte aligned, leading dimensions and K multiples of 4: 128-bit loads
    int c_vec;  // C 16-byte aligned, ldc and N multiples of 4: 128-bit stores
    int c_flat;  // C 16-byte aligned and contiguous (ldc == N), N <= 64, no sign bits asked for: half panels leave as flat runs of 16-byte stores
    // dropout after the ReLU (resident NT kernel): element e = row * N + col is kept iff 16-bit lane e % 8 of
    // Philox-4x32-10(counter = (e / 8, offset), key = seed) is >= thresh16, and then scaled by keep_scale
    uint32_t thresh16, seed_lo, seed_hi, off_lo, off_hi;
    float keep_scale;
    // sign bits: bit c % 32 of word [row * ldw + c / 32] says that element (row, c) is positive
    uint32_t *relu_bits;        // written beside C (resident NT kernel), or NULL
    const uint32_t *mask_bits;  // the mask of A in that form (resident NT kernel, 128-bit loads of A), or NULL
    int64_t ldw;
};

// One flag word behind the planes in the workspace: cleared by split_planes_kernel, raised by the product kernel
// when it meets such a value in either operand (it sees every element of both; in the planes of the small operand
// all of them show as Inf / NaN first pieces).
constexpr size_t kFlagBytes = 256;

// the three bf16 planes of a small fp32 matrix, optionally transposed: P[p][n][k] = piece p of alpha * X(n, k) with
// X(n, k) = B[k][n] (transpose) or B[n][k]; zero outside N x K.  Also clears the flag word.
__global__ void __launch_bounds__(256) split_planes_kernel(const float *__restrict__ B, int64_t ldb, int transpose, int64_t N,
                                                           int64_t K, int64_t Np, int64_t Kp, uint16_t *__restrict__ P,
                                                           unsigned *__restrict__ flag, float alpha)
{
    const int64_t total = Np * Kp;
    if (blockIdx.x == 0 && threadIdx.x == 0) *flag = 0u;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = i / Kp, k = i % Kp;
        float x = 0.f;
        if (n < N && k < K) x = (transpose ? B[k * ldb + n] : B[n * ldb + k]) * alpha;  // alpha = 1 leaves the bits alone
        uint32_t p0, p1, p2;
        split2(x, 0.f, p0, p1, p2);
        P[i] = (uint16_t)p0;
        P[total + i] = (uint16_t)p1;
        P[2 * total + i] = (uint16_t)p2;
    }
}

// ------------------------------------------------------------------------------------------------
// NT form.  Workgroups are persistent: workgroup b takes the row panels b, b + gridDim.x, ... and, per panel,
// every column tile; the steps (panel, column tile, chunk) form one software pipeline in which the global
// loads of step q + 1 are in flight while the MFMAs of step q run.  AVEC = 4: A (and mask) 16-byte aligned with
// leading dimensions that are multiples of 4 and K % 4 == 0, read with 128-bit loads.  AVEC = 2: everything a
// multiple of 2 elements / 8 bytes (rows of 602 elements), read with pairs of 64-bit loads.
// ------------------------------------------------------------------------------------------------
template <int TN, bool MASKED, int AVEC>
__global__ void __launch_bounds__(kThreads, 2) gemm_split_nt_kernel(const SplitArgs g)
{
    constexpr int BN = 32 * TN;
    constexpr int kAVec = kBM * kBK / 4 / kThreads;  // float4 per thread and chunk of A: 4
    constexpr int kBItems = 3 * BN * (kBK / 8);      // 16-byte vectors of the three B planes per chunk
    constexpr int kBVec = (kBItems + kThreads - 1) / kThreads;
    constexpr int kAPlane = kBM * kS, kBPlane = BN * kS;

    __shared__ __attribute__((aligned(16))) uint16_t lds[3 * kAPlane + 3 * kBPlane];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & 31;
    const int h = lane >> 5;
    const int rt = threadIdx.x >> 3;  // thread (rt, kq) owns float4 kq of rows rt, rt + 32, rt + 64, rt + 96 of a chunk
    const int kq = threadIdx.x & 7;

    const int64_t n_rp = (g.M + kBM - 1) / kBM;
    const int n_ct = (int)((g.N + BN - 1) / BN);
    const int n_kc = (int)((g.K + kBK - 1) / kBK);
    const int K = (int)g.K;
    const int64_t my_panels = n_rp > (int64_t)blockIdx.x ? (n_rp - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const int64_t steps = my_panels * n_ct * n_kc;
    if (steps == 0) return;

    // Step q of the pipeline is (row panel, column tile, chunk), chunk fastest.  A is fetched two steps ahead
    // (HBM latency), the B planes one step ahead (L2).  Both fetch cursors advance without divisions, and
    // everything that does not depend on the step (offsets inside a chunk, LDS addresses) is computed once.
    int64_t a_rp = blockIdx.x;
    int a_ct = 0, a_kc = 0;
    int b_ct = 0, b_kc = 0;
    const int64_t lda32 = 32 * g.lda, ldm32 = 32 * g.ldmask;

    // the mask travels beside its chunk and is applied when the chunk is split, so that a fetch only issues loads
    auto fetch_a = [&](float4(&dst)[kAVec], float4(&mdst)[kAVec]) __attribute__((always_inline)) {
        const int64_t row = a_rp * kBM + rt;
        const int k = a_kc * kBK + kq * 4;
        const int rows_left = (int)min(g.M - row, (int64_t)kBM);  // rows row + 32 p with 32 p < rows_left exist
        const float *pa = g.A + row * g.lda + k;
        const float *pm = MASKED ? g.mask + row * g.ldmask + k : nullptr;
#pragma unroll
        for (int p = 0; p < kAVec; ++p) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f), m = v;
            if (32 * p < rows_left && k < K) {
                if constexpr (AVEC == 4) {
                    v = *reinterpret_cast<const float4 *>(pa);
                    if constexpr (MASKED) m = *reinterpret_cast<const float4 *>(pm);
                } else {  // K is even: a pair lies inside the row or past its end as a whole
                    const float2 lo = *reinterpret_cast<const float2 *>(pa);
                    v.x = lo.x;
                    v.y = lo.y;
                    if constexpr (MASKED) {
                        const float2 mlo = *reinterpret_cast<const float2 *>(pm);
                        m.x = mlo.x;
                        m.y = mlo.y;
                    }
                    if (k + 2 < K) {
                        const float2 hi = *reinterpret_cast<const float2 *>(pa + 2);
                        v.z = hi.x;
                        v.w = hi.y;
                        if constexpr (MASKED) {
                            const float2 mhi = *reinterpret_cast<const float2 *>(pm + 2);
                            m.z = mhi.x;
                            m.w = mhi.y;
                        }
                    }
                }
            }
            dst[p] = v;
            if constexpr (MASKED) mdst[p] = m;
            pa += lda32;
            if constexpr (MASKED) pm += ldm32;
        }
        if (++a_kc == n_kc) {
            a_kc = 0;
            if (++a_ct == n_ct) {
                a_ct = 0;
                a_rp += gridDim.x;
            }
        }
    };

    // B items of this thread: (plane, row, 16-byte vector) -> offset inside a chunk of the planes / inside LDS
    int b_goff[kBVec], b_loff[kBVec];
    bool b_plane0[kBVec];
    bool b_first_pass = true;
#pragma unroll
    for (int j = 0; j < kBVec; ++j) {
        const int id = min((int)threadIdx.x + j * kThreads, kBItems - 1);  // surplus threads repeat the last item
        const int plane = id / (BN * 4), rem = id % (BN * 4);
        b_plane0[j] = plane == 0;
        b_goff[j] = (int)(plane * g.Np * g.Kp + (int64_t)(rem >> 2) * g.Kp + (rem & 3) * 8);  // planes hold < 2^31 elements
        b_loff[j] = 3 * kAPlane + plane * kBPlane + (rem >> 2) * kS + (rem & 3) * 8;
    }
    u32x4 rb[kBVec];
    auto fetch_b = [&]() __attribute__((always_inline)) {
        // planes are zero padded to Np x Kp, so no guards
        const uint16_t *pb = g.Bp + ((int64_t)b_ct * BN) * g.Kp + b_kc * kBK;
#pragma unroll
        for (int j = 0; j < kBVec; ++j) rb[j] = *reinterpret_cast<const u32x4 *>(pb + b_goff[j]);
        if (b_first_pass) {  // every chunk of the planes passes here once per workgroup: look for Inf / NaN in plane 0
#pragma unroll
            for (int j = 0; j < kBVec; ++j)
                if (b_plane0[j] && __builtin_expect(plane0_nonfinite(rb[j]), 0)) *g.nonfinite = 1u;
        }
        if (++b_kc == n_kc) {
            b_kc = 0;
            if (++b_ct == n_ct) {
                b_ct = 0;
                b_first_pass = false;
            }
        }
    };
    uint16_t *const a_dst = lds + rt * kS + kq * 4;
    auto stash = [&](const float4(&a)[kAVec], const float4(&am)[kAVec]) __attribute__((always_inline)) {
        int care = 0;
#pragma unroll
        for (int p = 0; p < kAVec; ++p) {
            float4 v = a[p];
            if constexpr (MASKED) {
                const float4 m = am[p];
                v = make_float4(m.x > 0.f ? v.x : 0.f, m.y > 0.f ? v.y : 0.f, m.z > 0.f ? v.z : 0.f, m.w > 0.f ? v.w : 0.f);
            }
            care |= needs_care(v);
            uint32_t lo0, lo1, lo2, hi0, hi1, hi2;
            split2(v.x, v.y, lo0, lo1, lo2);
            split2(v.z, v.w, hi0, hi1, hi2);
            uint16_t *dst = a_dst + 32 * p * kS;
            *reinterpret_cast<uint2 *>(dst) = make_uint2(lo0, hi0);
            *reinterpret_cast<uint2 *>(dst + kAPlane) = make_uint2(lo1, hi1);
            *reinterpret_cast<uint2 *>(dst + 2 * kAPlane) = make_uint2(lo2, hi2);
        }
        if (__builtin_expect(care, 0)) *g.nonfinite = 1u;
#pragma unroll
        for (int j = 0; j < kBVec; ++j)
            if ((int)threadIdx.x + j * kThreads < kBItems) *reinterpret_cast<u32x4 *>(lds + b_loff[j]) = rb[j];
    };

    floatx16 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

    const uint16_t *const as = lds + (wave * 32 + li) * kS + 8 * h;
    const uint16_t *const bs = lds + 3 * kAPlane + li * kS + 8 * h;
    int64_t rp = blockIdx.x;  // the step being computed
    int ct = 0, kc = 0;
    const bool relu = (g.flags & PLX_GEMM_RELU) != 0;

    auto step = [&](int64_t q, float4(&cur)[kAVec], float4(&mcur)[kAVec]) __attribute__((always_inline)) {
        stash(cur, mcur);
        __syncthreads();
        if (q + 2 < steps) fetch_a(cur, mcur);
        if (q + 1 < steps) fetch_b();
#pragma unroll
        for (int s = 0; s < kBK / 16; ++s) {
            const bf16x8 a0 = *reinterpret_cast<const bf16x8 *>(as + 16 * s);
            const bf16x8 a1 = *reinterpret_cast<const bf16x8 *>(as + kAPlane + 16 * s);
            const bf16x8 a2 = *reinterpret_cast<const bf16x8 *>(as + 2 * kAPlane + 16 * s);
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const uint16_t *bt = bs + t * 32 * kS + 16 * s;
                const bf16x8 b0 = *reinterpret_cast<const bf16x8 *>(bt);
                const bf16x8 b1 = *reinterpret_cast<const bf16x8 *>(bt + kBPlane);
                const bf16x8 b2 = *reinterpret_cast<const bf16x8 *>(bt + 2 * kBPlane);
                acc[t] = mfma6(a0, a1, a2, b0, b1, b2, acc[t]);
            }
        }
        if (++kc == n_kc) {
            // the tile is complete: register v of a lane is row 8 (v / 4) + 4 h + v % 4, column lane % 32 of each 32 x 32 block
            const int64_t r0 = rp * kBM + wave * 32 + 4 * h;
            const int c0 = ct * BN + li;
            float *pc = g.C + r0 * g.ldc + c0;
            const int rows_left = (int)min(g.M - r0, (int64_t)32);  // row r0 + d exists iff d < rows_left
            const int N = (int)g.N;
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const bool col_ok = c0 + t * 32 < N;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int d = 8 * (v / 4) + (v % 4);
                    float x = acc[t][v];
                    if (relu) x = fmaxf(x, 0.f);
                    if (col_ok && d < rows_left) pc[(int64_t)d * g.ldc + t * 32] = x;
                    acc[t][v] = 0.f;
                }
            }
            kc = 0;
            if (++ct == n_ct) {
                ct = 0;
                rp += gridDim.x;
            }
        }
        __syncthreads();
    };

    float4 ra0[kAVec], ra1[kAVec], m0[kAVec], m1[kAVec];  // m0 / m1 are dead registers without a mask
    fetch_a(ra0, m0);
    fetch_b();
    if (steps > 1) fetch_a(ra1, m1);
    for (int64_t q = 0; q < steps; q += 2) {
        step(q, ra0, m0);
        if (q + 1 < steps) step(q + 1, ra1, m1);
    }
}

// ------------------------------------------------------------------------------------------------
// NT form for a small operand of at most 128 x 128 (the layer widths of the benchmark network): the three
// planes of B stay in LDS for the life of the workgroup, and every wavefront streams its own 32-row panels
// of A through a private LDS tile.  There is no workgroup barrier after the planes are loaded, so the eight
// wavefronts of a workgroup drift apart and the matrix cores of a SIMD run one wavefront's MFMAs while the
// other wavefront splits and stages its next chunk.  A chunk is 32 rows x 16 contraction elements (two float4
// per lane); chunks are requested kRing steps before they are used.
// ------------------------------------------------------------------------------------------------
constexpr int kRWaves = 8;            // wavefronts per workgroup
constexpr int kRCK = 16;              // contraction elements per chunk
constexpr int kRAS = kRCK + 8;        // stride of the private A tile (48 bytes: 128-bit reads conflict-free)
constexpr int kRMaxK = 128, kRMaxN = 128;
constexpr int kRBS = kRMaxK + 8;      // stride of the resident B planes (272 bytes)
constexpr int kRAPlane = 32 * kRAS;   // bf16 elements of one private plane
constexpr size_t kRLdsBytes = ((size_t)3 * kRMaxN * kRBS + (size_t)kRWaves * 3 * kRAPlane) * sizeof(uint16_t);

// MASK: 0 none, 1 fp32 values beside A (mask > 0 keeps the element), 2 one bit per element
// DROP: dropout after the ReLU, for N a multiple of 8 (a call of the generator then covers 8 columns of one row)
// KS: chunk positions of a panel, 8 (K <= 128) or 4 (K <= 64)
// FAST: A (and the fp32 mask) take 128-bit loads and K >= 4.  Every request is then an unconditional load from an address
// clamped into the matrix (rows past the end repeat the last row and are never stored; columns past K repeat the last
// four and meet the zero padding of the planes), with no branch around it: the wait the compiler places before a
// chunk is used can then name how many younger requests may stay in flight, where loads inside branches make it wait
// for all of them -- which is what decides the speed of this kernel.
// ROWS16 = false (unconditional kernel without a mask): the rows of A are only 4-byte aligned and K is any number from 4 up (the
// 47-wide gradient of a last layer).  The same 16-byte requests -- the compiler emits them for 4-byte aligned data, which this
// hardware reads -- except that the vector which would reach past the end of a row is requested from the row's last four
// elements and shifted into place when it is used.
template <int TN, int MASK, bool DROP = false, bool FAST = false, int KS = 8, bool ROWS16 = true>
__global__ void __launch_bounds__(kRWaves * 64, 1) gemm_split_nt_resident_kernel(const SplitArgs g)
{
    constexpr bool MASKED = MASK == 1;      // the fp32 mask travels in registers beside its chunk
    constexpr bool BITS = MASK == 2;        // the bit mask of a panel row is four words, loaded once per panel
    constexpr int kSteps = KS;              // chunk positions of a panel (positions past K are skipped)
    constexpr int kRing = (MASKED || FAST) ? 4 : KS;  // register slots = how many positions ahead a chunk is requested
    static_assert(KS == 8 || (FAST && KS == 4), "the guarded kernel walks all eight positions");
    static_assert(ROWS16 || (FAST && MASK == 0 && !DROP), "rows without 16-byte alignment: the plain unconditional kernel only");
    extern __shared__ __attribute__((aligned(16))) uint16_t rlds[];
    uint16_t *const bres = rlds;                               // [3][kRMaxN][kRBS]
    constexpr int kBPlane = kRMaxN * kRBS;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in every lane: panel arithmetic stays scalar
    const int li = lane & 31;
    const int h = lane >> 5;
    uint16_t *const apriv = rlds + 3 * kBPlane + wave * 3 * kRAPlane;  // [3][32][kRAS], this wavefront's

    // the planes of B: [3][Np][Kp] in memory -> LDS, 16-byte vectors; rows and columns past Np / Kp stay unread
    // (the unconditional kernel multiplies all KS chunk positions of all TN column tiles: what lies past Np x Kp is zero)
    {
        const int rows = FAST ? 32 * TN : (int)g.Np;
        const int vec_per_row = (FAST ? kRCK * KS : (int)g.Kp) / 8;
        const int items = 3 * rows * vec_per_row;
        for (int id = threadIdx.x; id < items; id += kRWaves * 64) {
            const int plane = id / (rows * vec_per_row), rem = id % (rows * vec_per_row);
            const int row = rem / vec_per_row, q = rem % vec_per_row;
            u32x4 v = u32x4{0u, 0u, 0u, 0u};
            if (row < (int)g.Np && q * 8 < (int)g.Kp) v = *reinterpret_cast<const u32x4 *>(g.Bp + ((int64_t)plane * g.Np + row) * g.Kp + q * 8);
            *reinterpret_cast<u32x4 *>(bres + plane * kBPlane + row * kRBS + q * 8) = v;
            if (plane == 0 && __builtin_expect(plane0_nonfinite(v), 0)) *g.nonfinite = 1u;  // Inf / NaN in the small operand
        }
    }
    __syncthreads();

    const int K = (int)g.K;
    const int n_kc = (K + kRCK - 1) / kRCK;
    const int64_t n_panels = (g.M + 31) / 32;
    const int64_t first = (int64_t)blockIdx.x * kRWaves + wave, stride = (int64_t)gridDim.x * kRWaves;
    if (first >= n_panels) return;

    // lane (r, kq) owns float4 kq of rows r and r + 16 of a chunk.  The fetch cursor walks the positions
    // (panel, 0 .. kSteps - 1) in order and loads the ones that hold data.
    const int r = lane >> 2, kq = lane & 3;
    int64_t f_panel = first;
    int f_kc = 0;
    const int64_t lda16 = 16 * g.lda, ldm16 = 16 * g.ldmask;
    float4 ring[kRing][2], mring[MASKED ? kRing : 1][2];
    // Bit mask: a 64-lane load takes the memory pipeline as long for 4 bytes per lane as for 16, so the bits are not
    // fetched chunk by chunk; the 128 bits of rows r and r + 16 of a panel come with its first chunk and stay in registers.
    static_assert(!BITS || FAST || kRing == kSteps, "the guarded kernel makes the bits that came with a panel's first chunk current at the panel's start");
    u32x4 pb_cur[2], pb_next[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) pb_cur[p] = pb_next[p] = u32x4{~0u, ~0u, ~0u, ~0u};
    // byte offsets of a lane's two rows inside a panel (in the last panel: rows clamped to the last row of the matrix) and of
    // the last four columns, to which a lane's four columns are clamped; the host keeps 128 leading dimensions below 2^32
    // bytes for this kernel
    uint32_t a_off[2], a_off_last[2], m_off[2], m_off_last[2], w_off[2], w_off_last[2];
    const uint32_t k_last = 4u * (uint32_t)(K - 4);
    if constexpr (FAST) {
        const int rows_last = (int)(g.M - (n_panels - 1) * 32);  // 1 ... 32
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const uint32_t row = r + 16 * p, row_last = min(r + 16 * p, rows_last - 1);
            a_off[p] = row * (uint32_t)g.lda * 4u;
            a_off_last[p] = row_last * (uint32_t)g.lda * 4u;
            m_off[p] = MASKED ? row * (uint32_t)g.ldmask * 4u : 0u;
            m_off_last[p] = MASKED ? row_last * (uint32_t)g.ldmask * 4u : 0u;
            w_off[p] = BITS ? row * (uint32_t)g.ldw * 4u : 0u;
            w_off_last[p] = BITS ? row_last * (uint32_t)g.ldw * 4u : 0u;
        }
    }
    // `pos`, `of_panel`: the position a request is for (the unconditional form takes them from its caller, where they are
    // compile-time and loop-invariant values; the guarded form follows its cursor)
    auto fetch = [&](float4(&dst)[2], float4(&mdst)[2], int pos, int64_t of_panel) __attribute__((always_inline)) {
        if constexpr (FAST) {
            // the panel's address is the same in every lane (scalar arithmetic); a lane adds a 32-bit byte offset that does
            // not depend on the panel, except that the rows of the last panel are clamped into the matrix
            const int64_t panel = min(of_panel, n_panels - 1);
            const bool last = panel == n_panels - 1;
            const char *const pa = reinterpret_cast<const char *>(g.A) + panel * 128 * g.lda;
            const char *const pm = MASKED ? reinterpret_cast<const char *>(g.mask) + panel * 128 * g.ldmask : nullptr;
            const char *const pw = BITS ? reinterpret_cast<const char *>(g.mask_bits) + panel * 128 * g.ldw : nullptr;
            const uint32_t k_off = min((uint32_t)(pos * kRCK * 4 + kq * 16), k_last);
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                if constexpr (ROWS16) {
                    dst[p] = *reinterpret_cast<const float4 *>(pa + ((last ? a_off_last[p] : a_off[p]) + k_off));
                } else {
                    const Float4Align4 v = *reinterpret_cast<const Float4Align4 *>(pa + ((last ? a_off_last[p] : a_off[p]) + k_off));
                    dst[p] = make_float4(v.x, v.y, v.z, v.w);
                }
                if constexpr (MASKED) mdst[p] = *reinterpret_cast<const float4 *>(pm + ((last ? m_off_last[p] : m_off[p]) + k_off));
                if constexpr (BITS) {
                    if (pos == 0) pb_next[p] = *reinterpret_cast<const u32x4 *>(pw + (last ? w_off_last[p] : w_off[p]));
                }
            }
            return;
        }
        if (f_kc < n_kc && f_panel < n_panels) {
            const int64_t row = f_panel * 32 + r;
            const int k = f_kc * kRCK + kq * 4;
            const int rows_left = (int)min(g.M - row, (int64_t)32);  // rows row + 16 p with 16 p < rows_left exist
            const float *pa = g.A + row * g.lda + k;
            const float *pm = MASKED ? g.mask + row * g.ldmask + k : nullptr;
            if constexpr (BITS) {
                if (f_kc == 0) {
#pragma unroll
                    for (int p = 0; p < 2; ++p)
                        if (16 * p < rows_left) pb_next[p] = *reinterpret_cast<const u32x4 *>(g.mask_bits + (row + 16 * p) * g.ldw);
                }
            }
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f), m = make_float4(1.f, 1.f, 1.f, 1.f);
                if (16 * p < rows_left && k < K) {
                    if (g.a_vec) {
                        v = *reinterpret_cast<const float4 *>(pa);
                        if constexpr (MASKED) m = *reinterpret_cast<const float4 *>(pm);
                    } else {  // any alignment, any K: element loads
                        v.x = pa[0];
                        if (k + 1 < K) v.y = pa[1];
                        if (k + 2 < K) v.z = pa[2];
                        if (k + 3 < K) v.w = pa[3];
                        if constexpr (MASKED) {
                            m.x = pm[0];
                            if (k + 1 < K) m.y = pm[1];
                            if (k + 2 < K) m.z = pm[2];
                            if (k + 3 < K) m.w = pm[3];
                        }
                    }
                }
                dst[p] = v;
                if constexpr (MASKED) mdst[p] = m;
                pa += lda16;
                if constexpr (MASKED) pm += ldm16;
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

    uint16_t *const a_dst = apriv + r * kRAS + kq * 4;
    const uint16_t *const a_src = apriv + li * kRAS + 8 * h;
    const uint16_t *const b_src = bres + li * kRBS + 8 * h;
    const bool relu = (g.flags & PLX_GEMM_RELU) != 0;
    const int N = (int)g.N;

    int64_t cur_panel = first;
    // one position: split the chunk into the private tile, hand its registers to the position kRing ahead, multiply
    auto step = [&](int kc, float4(&cur)[2], float4(&mcur)[2]) __attribute__((always_inline)) {
        const bool live = FAST || kc < n_kc;  // the unconditional kernel multiplies every position: no branch around its requests
        if (live) {
            int care = 0;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                float4 v = cur[p];
                if constexpr (MASKED) {
                    const float4 m = mcur[p];
                    v = make_float4(m.x > 0.f ? v.x : 0.f, m.y > 0.f ? v.y : 0.f, m.z > 0.f ? v.z : 0.f, m.w > 0.f ? v.w : 0.f);
                }
                if constexpr (BITS) {
                    // chunk kc holds contraction elements 16 kc ...: bits 16 (kc % 2) + 4 kq ... of word kc / 2
                    const uint32_t mb = pb_cur[p][kc >> 1] >> (16 * (kc & 1) + 4 * kq);
                    v = make_float4((mb & 1u) ? v.x : 0.f, (mb & 2u) ? v.y : 0.f, (mb & 4u) ? v.z : 0.f, (mb & 8u) ? v.w : 0.f);
                }
                care |= needs_care(v);
                uint32_t lo0, lo1, lo2, hi0, hi1, hi2;
                split2(v.x, v.y, lo0, lo1, lo2);
                split2(v.z, v.w, hi0, hi1, hi2);
                uint16_t *dst = a_dst + 16 * p * kRAS;
                *reinterpret_cast<uint2 *>(dst) = make_uint2(lo0, hi0);
                *reinterpret_cast<uint2 *>(dst + kRAPlane) = make_uint2(lo1, hi1);
                *reinterpret_cast<uint2 *>(dst + 2 * kRAPlane) = make_uint2(lo2, hi2);
            }
            if (__builtin_expect(care, 0)) *g.nonfinite = 1u;
            plx::wave_lds_fence();  // the pieces other lanes stored are read below
        }
        fetch(cur, mcur, (kc + kRing) % kSteps, cur_panel + ((kc + kRing) / kSteps) * stride);
        if (live) {
            const bf16x8 a0 = *reinterpret_cast<const bf16x8 *>(a_src);
            const bf16x8 a1 = *reinterpret_cast<const bf16x8 *>(a_src + kRAPlane);
            const bf16x8 a2 = *reinterpret_cast<const bf16x8 *>(a_src + 2 * kRAPlane);
            const uint16_t *bk = b_src + kc * kRCK;
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const bf16x8 b0 = *reinterpret_cast<const bf16x8 *>(bk + t * 32 * kRBS);
                const bf16x8 b1 = *reinterpret_cast<const bf16x8 *>(bk + t * 32 * kRBS + kBPlane);
                const bf16x8 b2 = *reinterpret_cast<const bf16x8 *>(bk + t * 32 * kRBS + 2 * kBPlane);
                acc[t] = mfma6(a0, a1, a2, b0, b1, b2, acc[t]);
            }
            plx::wave_lds_fence();  // the next position overwrites the private tile
        }
    };

    // a finished panel: ReLU, dropout, sign bits, stores; leaves the accumulators zero
    auto finish_panel = [&](int64_t panel) __attribute__((always_inline)) {
        // the panel is complete: register v of a lane is row 8 (v / 4) + 4 h + v % 4, column lane % 32 of each 32 x 32 block
        const int64_t r0 = panel * 32 + 4 * h;
        float *pc = g.C + r0 * g.ldc + li;
        const int rows_left = (int)min(g.M - r0, (int64_t)32);
        // Dropout: one call of the generator gives the 16-bit lanes of 8 consecutive columns of a row, and an accumulator
        // register holds one column of a row, so the keep bits go through LDS: lane (row li, half h) makes the bits of
        // columns 32 t + 16 h ... + 15 of its row for every tile t (two calls each), stored as halves of the 32-bit word
        // [t][row] in the private tile (idle between the last product of a panel and the first chunk of the next); a
        // lane then reads the words of its four consecutive rows with one 128-bit load per four registers.
        uint32_t *const keep_words = reinterpret_cast<uint32_t *>(apriv);  // [TN][32]
        if constexpr (DROP) {
            const uint64_t row = (uint64_t)(panel * 32 + li);
            const uint64_t q_row = row * (uint64_t)(N >> 3);
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                uint32_t bits = 0;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint64_t q = q_row + (uint64_t)(4 * t + 2 * h + j);
                    const plx::Philox4 rnd = plx::philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), g.off_lo, g.off_hi, g.seed_lo, g.seed_hi);
#pragma unroll
                    for (int e = 0; e < 8; ++e) bits |= (plx::dropout_lane16(rnd, e) >= g.thresh16 ? 1u : 0u) << (8 * j + e);
                }
                reinterpret_cast<uint16_t *>(keep_words)[(t * 32 + li) * 2 + h] = (uint16_t)bits;
            }
            plx::wave_lds_fence();
        }
        // C in 128-bit stores: a 64-lane store takes the memory pipeline as long for 4 bytes per lane as for 16, and the 64
        // narrow stores of a panel fill the wavefront's queue of outstanding memory operations, behind which the requests of
        // the next panel wait.  The tile goes through the private LDS tile (32 rows of 36 floats: exactly its size), where a
        // lane picks up four consecutive columns of four rows; 16 stores per panel instead of 64.
        if constexpr (FAST && !DROP) {
            if (g.c_vec) {
                float *const stage = reinterpret_cast<float *>(apriv);  // [32][36]
                const int rr = lane >> 3, c4 = (lane & 7) * 4;
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    const bool col_ok = li + t * 32 < N;
                    uint32_t word = 0;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int d = 8 * (v / 4) + (v % 4);
                        float x = acc[t][v];
                        if (relu) x = fmaxf(x, 0.f);
                        stage[(d + 4 * h) * 36 + li] = x;
                        if (g.relu_bits != nullptr) {
                            const uint64_t votes = __ballot(col_ok && x > 0.f);
                            if (li == v) word = h ? (uint32_t)(votes >> 32) : (uint32_t)votes;
                        }
                        acc[t][v] = 0.f;
                    }
                    if (g.relu_bits != nullptr && li < 16) {
                        const int d = 8 * (li / 4) + (li % 4);
                        if (d < rows_left && t * 32 < N) g.relu_bits[(r0 + d) * g.ldw + t] = word;
                    }
                    plx::wave_lds_fence();
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int64_t row = panel * 32 + rr + 8 * j;
                        const float4 x4 = *reinterpret_cast<const float4 *>(stage + (rr + 8 * j) * 36 + c4);
                        if (row < g.M && t * 32 + c4 < N) *reinterpret_cast<float4 *>(g.C + row * g.ldc + t * 32 + c4) = x4;
                    }
                    plx::wave_lds_fence();  // the next tile, or the next panel's first chunk, overwrites the staging
                }
                return;
            }
            // A contiguous C whose rows are not multiples of 16 bytes (47 columns): 16 rows of it are still one aligned run of
            // 64 N bytes.  The half panel is staged row-major without padding (16 N floats fit the private tile; N <= 64 here)
            // and leaves in ceil(4 N / 64) stores of 16 bytes per lane instead of 16 TN stores of 4.
            if constexpr (TN <= 2) if (g.c_flat) {  // (N <= 64: the widest kernel has no registers to spare for a third epilogue)
                float *const stage = reinterpret_cast<float *>(apriv);  // [16][N]
#pragma unroll
                for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
                    for (int t = 0; t < TN; ++t) {
#pragma unroll
                        for (int v = 0; v < 8; ++v) {
                            const int d = 8 * (v / 4) + (v % 4) + 4 * h;  // row within the half panel
                            float x = acc[t][8 * pass + v];
                            if (relu) x = fmaxf(x, 0.f);
                            if (li + t * 32 < N) stage[d * N + t * 32 + li] = x;
                            acc[t][8 * pass + v] = 0.f;
                        }
                    }
                    plx::wave_lds_fence();
                    const int64_t row_first = panel * 32 + 16 * pass;
                    const int valid = (int)min(max(g.M - row_first, (int64_t)0), (int64_t)16) * N;  // floats of this half panel that exist
                    float *const dst = g.C + row_first * N;
                    for (int i = 4 * lane; i < valid; i += 256) {
                        if (i + 4 <= valid) {
                            *reinterpret_cast<float4 *>(dst + i) = *reinterpret_cast<const float4 *>(stage + i);
                        } else {
                            for (int e = i; e < valid; ++e) dst[e] = stage[e];
                        }
                    }
                    plx::wave_lds_fence();  // the next half, or the next panel's first chunk, overwrites the staging
                }
                return;
            }
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            const bool col_ok = li + t * 32 < N;
            uint32_t word = 0;  // lane li < 16 of half h collects the sign bits of row r0 + d(li), columns 32 t ... 32 t + 31
            u32x4 keep4[4];
            if constexpr (DROP) {
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) keep4[v4] = *reinterpret_cast<const u32x4 *>(keep_words + t * 32 + 8 * v4 + 4 * h);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 8 * (v / 4) + (v % 4);
                float x = acc[t][v];
                if (relu) x = fmaxf(x, 0.f);
                if constexpr (DROP) x = ((keep4[v / 4][v % 4] >> li) & 1u) ? x * g.keep_scale : 0.f;
                if (col_ok && d < rows_left) pc[(int64_t)d * g.ldc + t * 32] = x;
                if (g.relu_bits != nullptr) {  // one vote of the wavefront gives the words of two rows
                    const uint64_t votes = __ballot(col_ok && x > 0.f);
                    if (li == v) word = h ? (uint32_t)(votes >> 32) : (uint32_t)votes;
                }
                acc[t][v] = 0.f;
            }
            if (g.relu_bits != nullptr && li < 16) {
                const int d = 8 * (li / 4) + (li % 4);
                // a row holds ceil(N / 32) words: tiles that lie past N altogether (N <= 96 under four tiles) have none
                if (d < rows_left && t * 32 < N) g.relu_bits[(r0 + d) * g.ldw + t] = word;
            }
        }
        if constexpr (DROP) plx::wave_lds_fence();  // the next panel's first chunk overwrites the keep bits
    };

#pragma unroll
    for (int i = 0; i < kRing; ++i) fetch(ring[i], mring[MASKED ? i : 0], i, first);

    if constexpr (FAST) {
        // The positions run as a pipeline inside the wavefront.  While the matrix cores multiply position i out of registers,
        // the vector ALU splits position i + 1, the pieces go to the private tile (free once the pieces of position i have
        // been read), come back as the operands of position i + 1, and the pieces of B are read one column tile ahead of
        // their products.  A wavefront issues in order, so what shall overlap has to alternate in the instruction stream:
        // every product is followed by at most one half split (six or seven vector instructions, less than the 28 cycles a
        // product leaves free), and the order written here is pinned -- an empty asm statement after each product and each
        // half split takes their results as operands, and a scheduling barrier follows.
        constexpr int kStoreAt = TN >= 4 ? 18 : (TN == 2 ? 8 : 4);  // the product before which the next position is stored
        static_assert((kSteps * TN) % 2 == 0, "operand buffers alternate with the parity of a compile-time count");
        constexpr bool kAheadB = !(MASKED && TN > 1);
        bool unsplittable = false;  // a value the split cannot carry was met
        bf16x8 aa[2][3], bb[2][3];
        auto load_a = [&](bf16x8(&a)[3]) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 3; ++q) a[q] = *reinterpret_cast<const bf16x8 *>(a_src + q * kRAPlane);
        };
        auto load_b = [&](bf16x8(&b)[3], int kc, int t) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 3; ++q) b[q] = *reinterpret_cast<const bf16x8 *>(b_src + kc * kRCK + t * 32 * kRBS + q * kBPlane);
        };
        auto masked = [&](const float4 &a, const float4 &m, const u32x4 &bits, int kc) __attribute__((always_inline)) -> float4 {
            float4 v = a;
            if constexpr (!ROWS16) {
                // this lane's columns are kc 16 + 4 kq ...; the request was clamped to K - 4, so what it brought lies `over`
                // elements to the right of its place, and the elements past K count as zero
                const int over = kc * kRCK + kq * 4 - (K - 4);
                if (over > 0) {
                    v.x = over == 1 ? a.y : over == 2 ? a.z : over == 3 ? a.w : 0.f;
                    v.y = over == 1 ? a.z : over == 2 ? a.w : 0.f;
                    v.z = over == 1 ? a.w : 0.f;
                    v.w = 0.f;
                }
            }
            if constexpr (MASKED) v = make_float4(m.x > 0.f ? v.x : 0.f, m.y > 0.f ? v.y : 0.f, m.z > 0.f ? v.z : 0.f, m.w > 0.f ? v.w : 0.f);
            if constexpr (BITS) {
                // chunk kc holds contraction elements 16 kc ...: bits 16 (kc % 2) + 4 kq ... of word kc / 2
                const uint32_t mb = bits[kc >> 1] >> (16 * (kc & 1) + 4 * kq);
                v = make_float4((mb & 1u) ? v.x : 0.f, (mb & 2u) ? v.y : 0.f, (mb & 4u) ? v.z : 0.f, (mb & 8u) ? v.w : 0.f);
            }
            return v;
        };
        auto store_pieces = [&](const uint32_t(&w)[2][6]) __attribute__((always_inline)) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                uint16_t *dst = a_dst + 16 * p * kRAS;
                *reinterpret_cast<uint2 *>(dst) = make_uint2(w[p][0], w[p][3]);
                *reinterpret_cast<uint2 *>(dst + kRAPlane) = make_uint2(w[p][1], w[p][4]);
                *reinterpret_cast<uint2 *>(dst + 2 * kRAPlane) = make_uint2(w[p][2], w[p][5]);
            }
        };

        // position 0 of the first panel, with nothing to multiply meanwhile
        {
            if constexpr (BITS) {
#pragma unroll
                for (int p = 0; p < 2; ++p) pb_cur[p] = pb_next[p];
            }
            uint32_t w[2][6];
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const float4 v = masked(ring[0][p], mring[0][p], pb_cur[p], 0);
                float rx, ry;
                split2_first(v.x, v.y, w[p][0], rx, ry);
                unsplittable |= split2_second(rx, ry, w[p][1], w[p][2]);
                split2_first(v.z, v.w, w[p][3], rx, ry);
                unsplittable |= split2_second(rx, ry, w[p][4], w[p][5]);
            }
            store_pieces(w);
            plx::wave_lds_fence();
            load_a(aa[0]);
            if constexpr (kAheadB) load_b(bb[0], 0, 0);
            plx::wave_lds_fence();
        }

        for (int64_t panel = first; panel < n_panels; panel += stride) {
#pragma unroll
            for (int kc = 0; kc < kSteps; ++kc) {
                const bool wrap = kc + 1 == kSteps;  // the next position is the first of this wavefront's next panel
                const int nc = wrap ? 0 : kc + 1, slot = (kc + 1) % kRing;
                float4(&nxt)[2] = ring[slot];
                float4(&mnxt)[2] = mring[MASKED ? slot : 0];
                // the next position: eight values of a lane, four half-split pairs (j = 2 p + half of the float4)
                float x[4], y[4], rx[4], ry[4];
                uint32_t w[2][6];
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    const float4 v = masked(nxt[p], mnxt[p], wrap ? pb_next[p] : pb_cur[p], nc);
                    x[2 * p] = v.x, y[2 * p] = v.y, x[2 * p + 1] = v.z, y[2 * p + 1] = v.w;
                }
                if constexpr (BITS) {
                    if (wrap) {  // before the request below replaces them with the bits of the panel after
#pragma unroll
                        for (int p = 0; p < 2; ++p) pb_cur[p] = pb_next[p];
                    }
                }
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    const int group = kc * TN + t;  // which of the two buffers of B holds this column tile's pieces
                    // the pieces of B one column tile ahead (the first tile of the next position after the last); the kernel
                    // that also carries fp32 mask values has no registers for that and reads them where they are used
                    if constexpr (kAheadB) {
                        if (t + 1 < TN) load_b(bb[(group + 1) & 1], kc, t + 1);
                        else load_b(bb[(group + 1) & 1], nc, 0);
                    } else {
                        load_b(bb[group & 1], kc, t);
                    }
#pragma unroll
                    for (int m = 0; m < 6; ++m) {
                        const int idx = 6 * t + m;
                        if (idx == kStoreAt) {  // every half split lies before this product
                            plx::wave_lds_fence();  // after the loads of this position's pieces (and a finished panel's staging)
                            store_pieces(w);
                            // requests go out for two positions at a time, which share their 128-byte lines: positions
                            // kc + 4 and kc + 5 into the slots of positions kc and kc + 1, both split by now
                            if ((kc & 1) == 0) {
                                fetch(ring[kc % kRing], mring[MASKED ? kc % kRing : 0], (kc + kRing) % kSteps, panel + ((kc + kRing) / kSteps) * stride);
                                fetch(nxt, mnxt, (kc + 1 + kRing) % kSteps, panel + ((kc + 1 + kRing) / kSteps) * stride);
                            }
                            plx::wave_lds_fence();
                            load_a(aa[(kc + 1) & 1]);
                            plx::wave_lds_fence();
                        }
                        // the six piece products in the order of mfma6 (the smallest terms first)
                        const bf16x8(&a)[3] = aa[kc & 1];
                        const bf16x8(&b)[3] = bb[group & 1];
                        const bf16x8 am = (m == 0) ? a[2] : (m == 2 || m == 3) ? a[1] : a[0];
                        const bf16x8 bm = (m == 0 || m == 3 || m == 5) ? b[0] : (m == 1) ? b[2] : b[1];
                        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am, bm, acc[t], 0, 0, 0);
                        asm volatile("" : "+v"(acc[t]));
#pragma unroll
                        for (int k = 0; k < 8; ++k) {  // half split k = 2 j + second half, after product k kStoreAt / 8
                            if (k * kStoreAt / 8 != idx) continue;
                            const int j = k >> 1, p = j >> 1, o = 3 * (j & 1);
                            if ((k & 1) == 0) {
                                split2_first(x[j], y[j], w[p][o], rx[j], ry[j]);
                                asm volatile("" : "+v"(w[p][o]), "+v"(rx[j]), "+v"(ry[j]));
                            } else {
                                unsplittable |= split2_second(rx[j], ry[j], w[p][o + 1], w[p][o + 2]);
                                asm volatile("" : "+v"(w[p][o + 1]), "+v"(w[p][o + 2]));
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            if (__builtin_expect(unsplittable, 0)) *g.nonfinite = 1u;
            plx::wave_lds_fence();  // the staging of the panel comes after the loads of the next position's pieces
            finish_panel(panel);
        }
        return;
    }

    for (int64_t panel = first; panel < n_panels; panel += stride) {
        cur_panel = panel;
        if constexpr (BITS) {  // the bits that came with this panel's first chunk; the steps below fetch the next panel's
#pragma unroll
            for (int p = 0; p < 2; ++p) pb_cur[p] = pb_next[p];
        }
#pragma unroll
        for (int i = 0; i < kSteps; ++i) step(i, ring[i % kRing], mring[MASKED ? i % kRing : 0]);
        finish_panel(panel);
    }
}

template <int TN, int MASK, bool DROP, bool FAST, int KS, bool ROWS16 = true>
int launch_resident_one(const SplitArgs &g, unsigned blocks, hipStream_t st)
{
    static std::atomic<uint64_t> allowed{0};  // devices on which this instantiation may take its LDS
    const int rc = plx::allow_dynamic_lds(reinterpret_cast<const void *>(&gemm_split_nt_resident_kernel<TN, MASK, DROP, FAST, KS, ROWS16>),
                                          kRLdsBytes, allowed);
    if (rc != PLX_OK) return rc;
    gemm_split_nt_resident_kernel<TN, MASK, DROP, FAST, KS, ROWS16><<<blocks, kRWaves * 64, kRLdsBytes, st>>>(g);
    return PLX_OK;
}

// operands that take 128-bit loads go to the kernel whose requests are unconditional, with as many chunk positions as K needs
template <int TN, int MASK, bool DROP = false>
int launch_resident(const SplitArgs &g, unsigned blocks, hipStream_t st)
{
    // (its lanes address a panel with 32-bit byte offsets)
    const int64_t ld_max = (int64_t)1 << 24;
    if (g.a_vec && g.K >= 4 && g.lda < ld_max && g.ldmask < ld_max && g.ldw < ld_max) {
        if (g.K <= 64) return launch_resident_one<TN, MASK, DROP, true, 4>(g, blocks, st);
        return launch_resident_one<TN, MASK, DROP, true, 8>(g, blocks, st);
    }
    if constexpr (MASK == 0 && !DROP) {  // rows of A without 16-byte alignment, or a K that is not a multiple of 4
        // (four column tiles over eight positions: the shifting does not fit the registers, the guarded form below takes those)
        if (g.K >= 4 && g.lda < ld_max) {
            if (g.K <= 64) return launch_resident_one<TN, 0, false, true, 4, false>(g, blocks, st);
            if constexpr (TN <= 2) return launch_resident_one<TN, 0, false, true, 8, false>(g, blocks, st);
        }
    }
    return launch_resident_one<TN, MASK, DROP, false, 8>(g, blocks, st);
}

template <int MASK, bool DROP = false>
int launch_resident_tn(const SplitArgs &g, int tn, unsigned blocks, hipStream_t st)
{
    switch (tn) {
        case 1: return launch_resident<1, MASK, DROP>(g, blocks, st);
        case 2: return launch_resident<2, MASK, DROP>(g, blocks, st);
        default: return launch_resident<4, MASK, DROP>(g, blocks, st);
    }
}

// Dropout of a matrix in place, for the products whose kernel does not apply it (weights beyond 128 x 128, widths that
// are not multiples of 8, the fp32 MFMA kernels): thread i takes call i of the generator, i.e. elements 8 i ... 8 i + 7
// of the row-major numbering e = row * N + col.  Runs only if *run_if is set (run_if == NULL: always).
struct DropArgs {
    uint32_t thresh16, seed_lo, seed_hi, off_lo, off_hi;
    float keep_scale;
};

__global__ void __launch_bounds__(256) dropout_f32_kernel(int64_t M, int64_t N, float *__restrict__ X, int64_t ldx, const DropArgs a,
                                                          const unsigned *__restrict__ run_if)
{
    if (run_if != nullptr && *run_if == 0u) return;
    const uint64_t total = (uint64_t)M * (uint64_t)N;
    const uint64_t calls = (total + 7) / 8;
    for (uint64_t q = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; q < calls; q += (uint64_t)gridDim.x * blockDim.x) {
        const plx::Philox4 rnd = plx::philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), a.off_lo, a.off_hi, a.seed_lo, a.seed_hi);
        uint64_t e = q * 8;
        uint64_t r = e / (uint64_t)N, c = e % (uint64_t)N;
#pragma unroll
        for (int i = 0; i < 8; ++i, ++e) {
            if (e >= total) break;
            float *px = X + (int64_t)r * ldx + (int64_t)c;
            *px = plx::dropout_lane16(rnd, i) >= a.thresh16 ? *px * a.keep_scale : 0.f;
            if (++c == (uint64_t)N) {
                c = 0;
                ++r;
            }
        }
    }
}

int launch_dropout(int64_t M, int64_t N, float *X, int64_t ldx, const DropArgs &a, const unsigned *run_if, hipStream_t st)
{
    const int64_t calls = (M * N + 7) / 8;
    if (calls == 0) return PLX_OK;
    // (a guarded launch, which seldom has anything to do, takes a small grid: returning at once from 150,000 workgroups takes 50 us)
    const int64_t max_blocks = run_if != nullptr ? 2048 : 1 << 20;
    dropout_f32_kernel<<<(unsigned)std::min<int64_t>(plx::ceil_div(calls, 256), max_blocks), 256, 0, st>>>(M, N, X, ldx, a, run_if);
    PLX_LAUNCH_CHECK("dropout_f32_kernel");
    return PLX_OK;
}

int drop_args(const char *who, float p, uint64_t seed, uint64_t offset, DropArgs &a)
{
    PLX_REQUIRE(p >= 0.f && p < 1.f, "%s: dropout p=%g outside [0, 1)", who, (double)p);
    a.thresh16 = (uint32_t)std::min<long long>(65535, llroundf(p * 65536.f));
    a.keep_scale = 1.f / (1.f - p);
    a.seed_lo = (uint32_t)seed;
    a.seed_hi = (uint32_t)(seed >> 32);
    a.off_lo = (uint32_t)offset;
    a.off_hi = (uint32_t)(offset >> 32);
    return PLX_OK;
}

// sign bits of a matrix: word [row * ldw + w] = bits of columns 32 w ... 32 w + 31 (columns past N: 0).  Runs only if
// *run_if is set (run_if == NULL: always): the bits a product wrote beside C are wrong once the guarded fp32 launch has
// redone C.
__global__ void __launch_bounds__(256) sign_bits_kernel(int64_t M, int64_t N, const float *__restrict__ X, int64_t ldx,
                                                        uint32_t *__restrict__ bits, int64_t ldw, const unsigned *__restrict__ run_if)
{
    if (run_if != nullptr && *run_if == 0u) return;
    // a wavefront takes 64 consecutive columns of a row: one element per lane, one vote, two words
    const int lane = threadIdx.x & 63;
    const int64_t groups = (N + 63) / 64;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6, waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t i = wave; i < M * groups; i += waves) {
        const int64_t row = i / groups, c0 = (i % groups) * 64;
        const bool positive = c0 + lane < N && X[row * ldx + c0 + lane] > 0.f;
        const uint64_t votes = __ballot(positive);
        if (lane == 0) bits[row * ldw + c0 / 32] = (uint32_t)votes;
        if (lane == 32 && c0 + 32 < N) bits[row * ldw + c0 / 32 + 1] = (uint32_t)(votes >> 32);
    }
}

int launch_sign_bits(int64_t M, int64_t N, const float *X, int64_t ldx, uint32_t *bits, int64_t ldw, const unsigned *run_if, hipStream_t st)
{
    const int64_t items = M * ((N + 63) / 64);  // one wavefront each
    if (items == 0) return PLX_OK;
    // (a guarded launch, which seldom has anything to do, takes a small grid)
    const int64_t max_blocks = run_if != nullptr ? 2048 : 1 << 16;
    sign_bits_kernel<<<(unsigned)std::min<int64_t>(plx::ceil_div(items, 4), max_blocks), 256, 0, st>>>(M, N, X, ldx, bits, ldw, run_if);
    PLX_LAUNCH_CHECK("sign_bits_kernel");
    return PLX_OK;
}

int pick_tn(int64_t n) { return n <= 32 ? 1 : (n <= 64 ? 2 : 4); }

template <bool MASKED, int AVEC>
void launch_nt(const SplitArgs &g, int tn, unsigned blocks, hipStream_t st)
{
    switch (tn) {
        case 1: gemm_split_nt_kernel<1, MASKED, AVEC><<<blocks, kThreads, 0, st>>>(g); break;
        case 2: gemm_split_nt_kernel<2, MASKED, AVEC><<<blocks, kThreads, 0, st>>>(g); break;
        default: gemm_split_nt_kernel<4, MASKED, AVEC><<<blocks, kThreads, 0, st>>>(g); break;
    }
}

bool aligned16(const void *p, int64_t ld) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0); }
bool aligned8(const void *p, int64_t ld) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % 8 == 0 && ld % 2 == 0); }

int64_t round_up(int64_t x, int64_t q) { return (x + q - 1) / q * q; }

// C = epilogue((A*mask) . X^T) with X (N x K) = B^T (transpose_b) or B
// `drop` (forward only): dropout after the ReLU; `alpha` (backward only): the product is scaled by it, through the
// planes of the small operand
int nt_form(const char *who, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
            int transpose_b, float *C, int64_t ldc, const float *mask, int64_t ldmask, unsigned flags, void *workspace,
            size_t workspace_bytes, void *stream, uint32_t *relu_bits = nullptr, const uint32_t *mask_bits = nullptr, int64_t ldw = 0,
            const DropArgs *drop = nullptr, float alpha = 1.f)
{
    if (drop == nullptr && (flags & PLX_GEMM_DROPOUT) != 0)  // this entry point carries no p / seed / offset
        return plx::fail(PLX_ERR_UNSUPPORTED, "%s: PLX_GEMM_DROPOUT needs plx_gemm_nn_f32_split_dropout", who);
    PLX_REQUIRE(M >= 0 && N >= 0 && K > 0 && N < (1ll << 30) && K < (1ll << 30), "%s: bad dimension", who);
    if (M == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(C != nullptr && A != nullptr && B != nullptr, "%s: NULL operand", who);
    PLX_REQUIRE(lda >= K && ldc >= N && (mask == nullptr || ldmask >= K), "%s: leading dimension too small", who);
    PLX_REQUIRE(relu_bits == nullptr || ldw >= (N + 31) / 32, "%s: pitch of the sign bits smaller than ceil(N / 32) words", who);
    PLX_REQUIRE(mask_bits == nullptr || (mask != nullptr && ldw >= (K + 31) / 32),
                "%s: a bit mask comes with the fp32 mask it stands for and a pitch of at least ceil(K / 32) words", who);
    const int tn = pick_tn(N);
    const int64_t Np = round_up(N, 32 * tn), Kp = round_up(std::max<int64_t>(K, 1), kBK);
    const bool vec = aligned16(A, lda) && aligned16(mask, ldmask) && K % 4 == 0;
    const bool vec2 = aligned8(A, lda) && aligned8(mask, ldmask) && K % 2 == 0;
    const bool resident = Np <= kRMaxN && Kp <= kRMaxK;  // this kernel also reads A element by element
    PLX_REQUIRE(vec || vec2 || resident,
                "%s: for weights beyond 128 x 128, A and mask must be 8-byte aligned with leading dimensions and K multiples of 2", who);
    const size_t plane_bytes = (size_t)3 * Np * Kp * sizeof(uint16_t);  // a multiple of 16
    const size_t need = plane_bytes + kFlagBytes;
    if (workspace == nullptr || workspace_bytes < need)
        return plx::fail(PLX_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
    PLX_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, "%s: workspace must be 16-byte aligned", who);
    hipStream_t st = plx::as_stream(stream);
    uint16_t *planes = static_cast<uint16_t *>(workspace);
    unsigned *flag_words = reinterpret_cast<unsigned *>(static_cast<char *>(workspace) + plane_bytes);
    PLX_REQUIRE(M < (1ll << 40), "%s: too many rows", who);
    split_planes_kernel<<<(unsigned)std::min<int64_t>(plx::ceil_div(Np * Kp, 256), 4096), 256, 0, st>>>(B, ldb, transpose_b, N, K, Np,
                                                                                                    Kp, planes, flag_words, alpha);
    PLX_LAUNCH_CHECK("split_planes_kernel");
    const unsigned mm_flags = flags & ~PLX_GEMM_DROPOUT;  // what the fp32 MFMA launch understands
    // Inf / NaN / values next to FLT_MAX in either operand: the split product is then meaningless and the fp32 MFMA
    // kernel redoes it.  That
    // launch is always enqueued and returns at once unless the flag word is set.
    auto redo = [&]() -> int {
        if (transpose_b) {
            int rc = plx::gemm_nn_f32_if(M, N, K, A, lda, B, ldb, C, ldc, mm_flags, flag_words, 1, stream);
            if (rc == PLX_OK && drop != nullptr) rc = launch_dropout(M, N, C, ldc, *drop, flag_words, st);
            if (rc != PLX_OK || relu_bits == nullptr) return rc;
            return launch_sign_bits(M, N, C, ldc, relu_bits, ldw, flag_words, st);  // of the C that launch wrote, if it ran
        }
        return plx::gemm_nt_f32_if(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, flag_words, 1, stream, alpha);
    };
    // dropout that the product's kernel does not apply: a pass over C, and the sign bits after it
    auto drop_after = [&]() -> int {
        int rc = launch_dropout(M, N, C, ldc, *drop, nullptr, st);
        if (rc == PLX_OK && relu_bits != nullptr) rc = launch_sign_bits(M, N, C, ldc, relu_bits, ldw, nullptr, st);
        return rc;
    };
    SplitArgs g{};
    g.A = A; g.mask = mask; g.Bp = planes; g.C = C; g.lda = lda; g.ldmask = ldmask; g.ldc = ldc;
    g.M = M; g.N = N; g.K = K; g.Np = Np; g.Kp = Kp; g.flags = mm_flags; g.a_vec = vec;
    g.c_vec = (reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc % 4 == 0 && N % 4 == 0) ? 1 : 0;
    g.c_flat = (!g.c_vec && reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc == N && N <= 64 && relu_bits == nullptr) ? 1 : 0;
    g.nonfinite = flag_words;
    g.ldw = ldw;
    if (drop != nullptr) {
        g.thresh16 = drop->thresh16; g.keep_scale = drop->keep_scale;
        g.seed_lo = drop->seed_lo; g.seed_hi = drop->seed_hi; g.off_lo = drop->off_lo; g.off_hi = drop->off_hi;
    }
    if (resident && drop != nullptr) {
        const unsigned blocks = (unsigned)std::min<int64_t>(plx::ceil_div(M, 32 * kRWaves), 256);
        const bool fused = N % 8 == 0;
        g.relu_bits = fused ? relu_bits : nullptr;
        int rc = fused ? launch_resident_tn<0, true>(g, tn, blocks, st) : launch_resident_tn<0>(g, tn, blocks, st);
        if (rc != PLX_OK) return rc;
        PLX_LAUNCH_CHECK("gemm_split_nt_resident_kernel");
        if (!fused && (rc = drop_after()) != PLX_OK) return rc;
        return redo();
    }
    if (resident) {
        const unsigned blocks = (unsigned)std::min<int64_t>(plx::ceil_div(M, 32 * kRWaves), 256);
        g.relu_bits = relu_bits;
        // the bit mask is read with the 128-bit loads of A; other layouts take the fp32 mask
        const bool bits = mask_bits != nullptr && vec && ldw % 4 == 0 && reinterpret_cast<uintptr_t>(mask_bits) % 16 == 0;
        g.mask_bits = bits ? mask_bits : nullptr;
        const int rc = bits ? launch_resident_tn<2>(g, tn, blocks, st)
                            : (mask != nullptr ? launch_resident_tn<1>(g, tn, blocks, st) : launch_resident_tn<0>(g, tn, blocks, st));
        if (rc != PLX_OK) return rc;
        PLX_LAUNCH_CHECK("gemm_split_nt_resident_kernel");
        return redo();
    }
    const unsigned blocks = (unsigned)std::min<int64_t>(plx::ceil_div(M, kBM), 2 * 256);
    if (vec) {
        if (mask != nullptr) launch_nt<true, 4>(g, tn, blocks, st); else launch_nt<false, 4>(g, tn, blocks, st);
    } else {
        if (mask != nullptr) launch_nt<true, 2>(g, tn, blocks, st); else launch_nt<false, 2>(g, tn, blocks, st);
    }
    PLX_LAUNCH_CHECK("gemm_split_nt_kernel");
    if (drop != nullptr) {
        const int rc = drop_after();
        if (rc != PLX_OK) return rc;
    } else if (relu_bits != nullptr) {  // this kernel does not write them: a pass over C does
        const int rc = launch_sign_bits(M, N, C, ldc, relu_bits, ldw, nullptr, st);
        if (rc != PLX_OK) return rc;
    }
    return redo();
}

}  // namespace

extern "C" {

size_t plx_gemm_f32_split_workspace_bytes(int64_t N, int64_t K)
{
    if (N <= 0 || K < 0) return 0;
    const int64_t Np = round_up(N, 32 * pick_tn(N)), Kp = round_up(std::max<int64_t>(K, 1), kBK);
    return (size_t)3 * Np * Kp * sizeof(uint16_t) + kFlagBytes;
}

int plx_gemm_nn_f32_split(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                          int64_t ldc, unsigned flags, void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(ldb >= N, "gemm_nn_split: leading dimension too small");
    return nt_form("gemm_nn_split", M, N, K, A, lda, B, ldb, 1, C, ldc, nullptr, 0, flags, workspace, workspace_bytes, stream);
}

int plx_gemm_nt_f32_split(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                          int64_t ldc, const float *mask, int64_t ldmask, void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(ldb >= K, "gemm_nt_split: leading dimension too small");
    return nt_form("gemm_nt_split", M, N, K, A, lda, B, ldb, 0, C, ldc, mask, ldmask, 0u, workspace, workspace_bytes, stream);
}

int plx_gemm_nn_f32_split_bits(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                               int64_t ldc, unsigned flags, uint32_t *sign_bits, int64_t ldw, void *workspace, size_t workspace_bytes,
                               void *stream)
{
    PLX_REQUIRE(ldb >= N, "gemm_nn_split_bits: leading dimension too small");
    PLX_REQUIRE(sign_bits != nullptr, "gemm_nn_split_bits: NULL sign bits");
    return nt_form("gemm_nn_split_bits", M, N, K, A, lda, B, ldb, 1, C, ldc, nullptr, 0, flags, workspace, workspace_bytes, stream,
                   sign_bits, nullptr, ldw);
}

int plx_gemm_nt_f32_split_bits(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                               int64_t ldc, const float *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(ldb >= K, "gemm_nt_split_bits: leading dimension too small");
    PLX_REQUIRE(mask_bits != nullptr, "gemm_nt_split_bits: NULL bit mask");
    return nt_form("gemm_nt_split_bits", M, N, K, A, lda, B, ldb, 0, C, ldc, mask, ldmask, 0u, workspace, workspace_bytes, stream,
                   nullptr, mask_bits, ldw);
}

int plx_gemm_nn_f32_split_dropout(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                                  int64_t ldc, unsigned flags, float dropout_p, uint64_t seed, uint64_t offset, uint32_t *sign_bits,
                                  int64_t ldw, void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(ldb >= N, "gemm_nn_split_dropout: leading dimension too small");
    DropArgs d{};
    const int rc = drop_args("gemm_nn_split_dropout", dropout_p, seed, offset, d);
    if (rc != PLX_OK) return rc;
    const bool drop = (flags & PLX_GEMM_DROPOUT) != 0 && dropout_p > 0.f;
    return nt_form("gemm_nn_split_dropout", M, N, K, A, lda, B, ldb, 1, C, ldc, nullptr, 0, drop ? flags : (flags & ~PLX_GEMM_DROPOUT),
                   workspace, workspace_bytes, stream, sign_bits, nullptr, ldw, drop ? &d : nullptr);
}

int plx_gemm_nt_f32_split_scaled(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                                 int64_t ldc, const float *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw, float alpha,
                                 void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(ldb >= K, "gemm_nt_split_scaled: leading dimension too small");
    return nt_form("gemm_nt_split_scaled", M, N, K, A, lda, B, ldb, 0, C, ldc, mask, ldmask, 0u, workspace, workspace_bytes, stream,
                   nullptr, mask_bits, ldw, nullptr, alpha);
}

int plx_dropout_f32(int64_t M, int64_t N, float *X, int64_t ldx, float dropout_p, uint64_t seed, uint64_t offset, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && ldx >= N && M < (1ll << 40) && N < (1ll << 30), "dropout: bad dimension or pitch");
    if (M == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(X != nullptr, "dropout: NULL operand");
    DropArgs d{};
    const int rc = drop_args("dropout", dropout_p, seed, offset, d);
    if (rc != PLX_OK) return rc;
    return launch_dropout(M, N, X, ldx, d, nullptr, plx::as_stream(stream));
}

int plx_sign_bits_f32(int64_t M, int64_t N, const float *X, int64_t ldx, uint32_t *sign_bits, int64_t ldw, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0 && ldx >= N && ldw >= (N + 31) / 32, "sign_bits: bad dimension or pitch");
    if (M == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(X != nullptr && sign_bits != nullptr, "sign_bits: NULL operand");
    return launch_sign_bits(M, N, X, ldx, sign_bits, ldw, nullptr, plx::as_stream(stream));
}

}  // extern "C"
