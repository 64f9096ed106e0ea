// Row-softmax cross-entropy: loss and d(loss)/d(logits) in one pass over the logits.
//
// A group of LPR lanes (LPR = power of two >= min(C, 64)) owns one row, so a wavefront covers
// 64 / LPR consecutive rows -- consecutive rows are contiguous in memory when ld == C, which keeps
// the loads of a wavefront in one contiguous span.  The row maximum and the row sum are reduced
// with cross-lane shuffles inside the group.  Each workgroup adds the losses of its rows in a
// fixed order and writes one partial; a one-workgroup kernel adds the partials in order (in fp64)
// and divides by the node count.  No atomics.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "bf16.h"
#include "common.h"

namespace {

constexpr int kXentMaxBlocks = 4096;
constexpr int kMaxPerLane = 16;  // classes per lane kept in registers: C <= 64 * 16

// element access for fp32 (float) or bf16 (uint16_t bit pattern) storage; the arithmetic is fp32
template <typename T>
__device__ __forceinline__ float ld_elem(const void *base, int64_t i)
{
    if constexpr (sizeof(T) == 4)
        return static_cast<const float *>(base)[i];
    else
        return plx::bf16_to_f32(static_cast<const uint16_t *>(base)[i]);
}
template <typename T>
__device__ __forceinline__ void st_elem(void *base, int64_t i, float v)
{
    if constexpr (sizeof(T) == 4)
        static_cast<float *>(base)[i] = v;
    else
        static_cast<uint16_t *>(base)[i] = (uint16_t)plx::f32_to_bf16(v);
}

struct XentArgs {
    const void *logits;
    const int64_t *labels;
    void *dlogits;
    float *partials;
    int64_t ld, ldd;
    int64_t M, C, num_nodes, num_classes, row_offset;
    float scale;  // gscale / num_nodes
};

template <typename T, int LPR, int PER>
__global__ void __launch_bounds__(256) softmax_xent_kernel(const XentArgs p)
{
    constexpr int RPW = 64 / LPR;  // rows per wavefront
    __shared__ float wsum[4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int grp = lane / LPR;
    const int t = lane % LPR;
    const int64_t cv = min(p.C, p.num_classes);
    const int64_t rows_per_block = 4 * RPW;
    const int64_t n_groups = (p.M + rows_per_block - 1) / rows_per_block;

    float loss_acc = 0.f;  // per lane; only lane t == 0 of a group adds
    for (int64_t gb = blockIdx.x; gb < n_groups; gb += gridDim.x) {
        const int64_t r = gb * rows_per_block + wave * RPW + grp;
        const bool row_ok = r < p.M;
        const int64_t xoff = (row_ok ? r : 0) * p.ld;
        float v[PER];
        float mx = -INFINITY;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int64_t c = t + (int64_t)k * LPR;
            v[k] = (row_ok && c < cv) ? ld_elem<T>(p.logits, xoff + c) : -INFINITY;
            mx = fmaxf(mx, v[k]);
        }
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        float den = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            v[k] = (v[k] == -INFINITY) ? 0.f : expf(v[k] - mx);
            den += v[k];
        }
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) den += __shfl_xor(den, o, 64);

        const int64_t y = row_ok ? p.labels[r] : -1;
        const bool invalid_node = (p.row_offset + r >= p.num_nodes) || (y < 0);
        const bool label_ok = (y >= 0) && (y < p.C);
        const float inv = invalid_node ? 0.f : 1.f / den;
        float py = 0.f;  // probability of the labelled class, held by the lane that owns it
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int64_t c = t + (int64_t)k * LPR;
            const float prob = v[k] * inv;
            const bool hit = label_ok && c == y;
            if (hit) py = prob;
            if (row_ok && c < p.C && p.dlogits != nullptr) st_elem<T>(p.dlogits, r * p.ldd + c, (prob - (hit ? 1.f : 0.f)) * p.scale);
        }
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) py += __shfl_xor(py, o, 64);  // one lane holds it, the rest 0
        if (t == 0 && row_ok && label_ok) loss_acc += -logf(fmaxf(py, 1e-9f));
    }
    // fixed-order sum over the lanes of the wavefront, then over the four wavefronts
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) loss_acc += __shfl_xor(loss_acc, o, 64);
    if (lane == 0) wsum[wave] = loss_acc;
    __syncthreads();
    if (threadIdx.x == 0) p.partials[blockIdx.x] = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
}

// Narrow rows (C up to a few hundred): a workgroup stages a tile of R consecutive rows in LDS with
// coalesced loads, one lane then owns one row (row stride C | 1, so lanes hit distinct banks), and the
// gradient tile goes back with coalesced stores.  Every lane is busy whatever C is, which the
// group-per-row kernel above cannot offer for widths like 47.
template <typename T>
__global__ void __launch_bounds__(256) softmax_xent_tiled_kernel(const XentArgs p, int R, int CP)
{
    extern __shared__ float tile[];
    __shared__ float wsum[4];
    const int C = (int)p.C;
    const int cv = (int)min(p.C, p.num_classes);
    const int64_t n_tiles = (p.M + R - 1) / R;
    const int step_r = 256 / C, step_c = 256 % C;
    float loss_acc = 0.f;
    for (int64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
        const int64_t row0 = t * R;
        const int rows = (int)min((int64_t)R, p.M - row0);
        const int count = rows * C;
        // stage: element i of the tile is (i / C, i % C); (r, c) advance without divisions
        int r = (int)threadIdx.x / C, c = (int)threadIdx.x % C;
        for (int i = threadIdx.x; i < count; i += 256) {
            tile[r * CP + c] = ld_elem<T>(p.logits, (row0 + r) * p.ld + c);
            r += step_r;
            c += step_c;
            if (c >= C) {
                c -= C;
                ++r;
            }
        }
        __syncthreads();
        if ((int)threadIdx.x < rows) {
            float *x = tile + threadIdx.x * CP;
            const int64_t row = row0 + threadIdx.x;
            float mx = -INFINITY;
            for (int k = 0; k < cv; ++k) mx = fmaxf(mx, x[k]);
            float den = 0.f;
            for (int k = 0; k < cv; ++k) {
                const float e = expf(x[k] - mx);
                x[k] = e;
                den += e;
            }
            const int64_t y = p.labels[row];
            const bool invalid_node = (p.row_offset + row >= p.num_nodes) || (y < 0);
            const bool label_ok = (y >= 0) && (y < p.C);
            const float inv = invalid_node ? 0.f : 1.f / den;
            float py = 0.f;
            for (int k = 0; k < C; ++k) {
                const float prob = k < cv ? x[k] * inv : 0.f;
                const bool hit = label_ok && k == (int)y;
                if (hit) py = prob;
                x[k] = (prob - (hit ? 1.f : 0.f)) * p.scale;
            }
            if (label_ok) loss_acc += -logf(fmaxf(py, 1e-9f));
        }
        __syncthreads();
        if (p.dlogits != nullptr) {
            r = (int)threadIdx.x / C;
            c = (int)threadIdx.x % C;
            for (int i = threadIdx.x; i < count; i += 256) {
                st_elem<T>(p.dlogits, (row0 + r) * p.ldd + c, tile[r * CP + c]);
                r += step_r;
                c += step_c;
                if (c >= C) {
                    c -= C;
                    ++r;
                }
            }
        }
        __syncthreads();
    }
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) loss_acc += __shfl_xor(loss_acc, o, 64);
    if (lane == 0) wsum[threadIdx.x >> 6] = loss_acc;
    __syncthreads();
    if (threadIdx.x == 0) p.partials[blockIdx.x] = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
}

// Same tiling for C <= CMAX <= 64 with the row held in registers: a lane reads its row from LDS once,
// does max / exp / sum / gradient on registers (statically unrolled, so the LDS reads are issued in one
// batch) and writes the gradient row back once -- 2 LDS accesses per element instead of 5.
// Requires that the rows are contiguous in memory (ld == ldd == C) and C is odd, so a tile is rows * C
// consecutive elements, copied in and out with 128-bit accesses into an unpadded LDS tile (CP == C) whose
// per-row pass is free of bank conflicts because the row stride is odd.  (Rotating the visit order by the
// lane index makes even C conflict-free too, but the run-time LDS addresses cost more than the copy saves.)
template <typename T, int CMAX, int R>
__global__ void __launch_bounds__(256) softmax_xent_tiled_reg_kernel(const XentArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float tile[];
    __shared__ float wsum[4];
    constexpr int EPV = 16 / (int)sizeof(T);  // elements per 128-bit access
    constexpr int kVecs = (R * CMAX + EPV * 256 - 1) / (EPV * 256);  // 128-bit vectors of a tile per thread, at most
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int C = (int)p.C;
    const int cv = (int)min(p.C, p.num_classes);
    const int64_t n_tiles = (p.M + R - 1) / R;
    float loss_acc = 0.f;
    // The tile after the one being worked on is already on its way from memory: its vectors are requested into
    // registers before the row phase of the current tile and written to LDS when that tile has been stored, so the
    // loads of a workgroup overlap its own exponentials and stores, not only those of its neighbours on the compute unit.
    u32x4 pre[kVecs];
    auto request = [&](int64_t t) {
        const int64_t row0 = t * R;
        const int vecs = (int)min((int64_t)R, p.M - row0) * C / EPV;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const T *>(p.logits) + row0 * C);
#pragma unroll
        for (int j = 0; j < kVecs; ++j) {
            const int i = j * 256 + (int)threadIdx.x;
            if (i < vecs) pre[j] = __builtin_nontemporal_load(src + i);
        }
    };
    if ((int64_t)blockIdx.x < n_tiles) request(blockIdx.x);
    for (int64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
        const int64_t row0 = t * R;
        const int rows = (int)min((int64_t)R, p.M - row0);
        const int count = rows * C;
        const int vecs = count / EPV;
#pragma unroll
        for (int j = 0; j < kVecs; ++j) {
            const int i = j * 256 + (int)threadIdx.x;
            if (i < vecs) {
                if constexpr (sizeof(T) == 4) {
                    reinterpret_cast<u32x4 *>(tile)[i] = pre[j];
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        tile[i * 8 + 2 * q] = __uint_as_float(pre[j][q] << 16);
                        tile[i * 8 + 2 * q + 1] = __uint_as_float(pre[j][q] & 0xffff0000u);
                    }
                }
            }
        }
        for (int i = vecs * EPV + threadIdx.x; i < count; i += 256) tile[i] = ld_elem<T>(p.logits, row0 * C + i);
        __syncthreads();
        if (t + gridDim.x < n_tiles) request(t + gridDim.x);
        if ((int)threadIdx.x < rows) {
            float *x = tile + threadIdx.x * C;
            const int64_t row = row0 + threadIdx.x;
            float v[CMAX];
            float mx = -INFINITY;
#pragma unroll
            for (int k = 0; k < CMAX; ++k) {
                v[k] = k < cv ? x[k] : -INFINITY;
                mx = fmaxf(mx, v[k]);
            }
            float den = 0.f;
#pragma unroll
            for (int k = 0; k < CMAX; ++k) {
                v[k] = expf(v[k] - mx);  // exp(-inf) = 0 for the slots that hold no valid class
                den += v[k];
            }
            const int64_t y = p.labels[row];
            const bool invalid_node = (p.row_offset + row >= p.num_nodes) || (y < 0);
            const bool label_ok = (y >= 0) && (y < p.C);
            const float inv = invalid_node ? 0.f : 1.f / den;
            float py = 0.f;
#pragma unroll
            for (int k = 0; k < CMAX; ++k) {
                const float prob = v[k] * inv;
                const bool hit = label_ok && k == (int)y;
                if (hit) py = prob;
                if (k < C) x[k] = (prob - (hit ? 1.f : 0.f)) * p.scale;
            }
            if (label_ok) loss_acc += -logf(fmaxf(py, 1e-9f));
        }
        __syncthreads();
        if (p.dlogits != nullptr) {
            // the gradient is read next by another kernel, long after this one: stores that do not linger in the caches
            u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<T *>(p.dlogits) + row0 * C);
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const int i = j * 256 + (int)threadIdx.x;
                if (i < vecs) {
                    if constexpr (sizeof(T) == 4) {
                        __builtin_nontemporal_store(reinterpret_cast<const u32x4 *>(tile)[i], dst + i);
                    } else {
                        const float4 lo = reinterpret_cast<const float4 *>(tile)[2 * i];
                        const float4 hi = reinterpret_cast<const float4 *>(tile)[2 * i + 1];
                        u32x4 o;
                        o[0] = plx::pack_bf16x2(lo.x, lo.y);
                        o[1] = plx::pack_bf16x2(lo.z, lo.w);
                        o[2] = plx::pack_bf16x2(hi.x, hi.y);
                        o[3] = plx::pack_bf16x2(hi.z, hi.w);
                        __builtin_nontemporal_store(o, dst + i);
                    }
                }
            }
            for (int i = vecs * EPV + threadIdx.x; i < count; i += 256) st_elem<T>(p.dlogits, row0 * C + i, tile[i]);
        }
        __syncthreads();
    }
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) loss_acc += __shfl_xor(loss_acc, o, 64);
    if (lane == 0) wsum[threadIdx.x >> 6] = loss_acc;
    __syncthreads();
    if (threadIdx.x == 0) p.partials[blockIdx.x] = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
}

template <typename T>
static void launch_tiled_reg(const XentArgs &a, int64_t C, int R, unsigned blocks, size_t shm, hipStream_t st)
{
    if (R == 256) {  // C <= 47
        if (C <= 16) softmax_xent_tiled_reg_kernel<T, 16, 256><<<blocks, 256, shm, st>>>(a);
        else if (C <= 32) softmax_xent_tiled_reg_kernel<T, 32, 256><<<blocks, 256, shm, st>>>(a);
        else softmax_xent_tiled_reg_kernel<T, 48, 256><<<blocks, 256, shm, st>>>(a);
    } else {
        softmax_xent_tiled_reg_kernel<T, 64, 128><<<blocks, 256, shm, st>>>(a);
    }
}

__global__ void __launch_bounds__(256) xent_finish_kernel(const float *__restrict__ partials, int n, double inv_nodes,
                                                          float *__restrict__ loss)
{
    __shared__ double part[256];
    double s = 0.0;
    for (int i = threadIdx.x; i < n; i += 256) s += (double)partials[i];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) part[threadIdx.x] += part[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss = (float)(part[0] * inv_nodes);
}

template <typename T, int LPR>
int launch_xent(const XentArgs &a, int per, unsigned blocks, hipStream_t st)
{
    if constexpr (LPR < 64) {
        if (per != 1) return -1;
        softmax_xent_kernel<T, LPR, 1><<<blocks, 256, 0, st>>>(a);
        return 0;
    } else {
        switch (per) {
            case 1: softmax_xent_kernel<T, LPR, 1><<<blocks, 256, 0, st>>>(a); return 0;
            case 2: softmax_xent_kernel<T, LPR, 2><<<blocks, 256, 0, st>>>(a); return 0;
            case 4: softmax_xent_kernel<T, LPR, 4><<<blocks, 256, 0, st>>>(a); return 0;
            case 8: softmax_xent_kernel<T, LPR, 8><<<blocks, 256, 0, st>>>(a); return 0;
            case 16: softmax_xent_kernel<T, LPR, 16><<<blocks, 256, 0, st>>>(a); return 0;
            default: return -1;
        }
    }
}

}  // namespace

extern "C" {

size_t plx_softmax_xent_workspace_bytes(int64_t M, int64_t C)
{
    (void)M;
    (void)C;
    return (size_t)kXentMaxBlocks * sizeof(float);
}

}  // extern "C"

namespace {
template <typename T>
int softmax_xent_impl(int64_t M, int64_t C, const T *logits, int64_t ld, const int64_t *labels, int64_t num_nodes,
                      int64_t num_classes, int64_t row_offset, float gscale, float *loss, T *dlogits, int64_t ldd,
                      void *workspace, size_t workspace_bytes, void *stream)
{
    PLX_REQUIRE(M >= 0 && C >= 1, "softmax_xent: bad shape M=%lld C=%lld", (long long)M, (long long)C);
    PLX_REQUIRE(C <= 64 * kMaxPerLane, "softmax_xent: at most %d classes are supported, got %lld", 64 * kMaxPerLane,
                (long long)C);
    PLX_REQUIRE(num_nodes >= 1 && num_classes >= 1, "softmax_xent: num_nodes and num_classes must be positive");
    PLX_REQUIRE(loss != nullptr, "softmax_xent: NULL loss");
    PLX_REQUIRE(M == 0 || (logits != nullptr && labels != nullptr), "softmax_xent: NULL input");
    PLX_REQUIRE(ld >= C && (dlogits == nullptr || ldd >= C), "softmax_xent: leading dimension smaller than C");
    if (workspace == nullptr || workspace_bytes < plx_softmax_xent_workspace_bytes(M, C))
        return plx::fail(PLX_ERR_WORKSPACE, "softmax_xent: workspace of %zu bytes needed, %zu given",
                         plx_softmax_xent_workspace_bytes(M, C), workspace_bytes);
    hipStream_t st = plx::as_stream(stream);

    int lpr = 1;
    while (lpr < 64 && lpr < C) lpr <<= 1;
    int per = 1;
    while ((int64_t)lpr * per < C) per <<= 1;

    XentArgs a;
    a.logits = logits;
    a.labels = labels;
    a.dlogits = dlogits;
    a.partials = static_cast<float *>(workspace);
    a.ld = ld;
    a.ldd = ldd;
    a.M = M;
    a.C = C;
    a.num_nodes = num_nodes;
    a.num_classes = num_classes;
    a.row_offset = row_offset;
    a.scale = gscale / (float)num_nodes;

    unsigned blocks;
    // Which kernel, from measurements on 2,449,029 rows (fp32, ms): the tiled kernels win up to about 88 classes
    // (C = 80: 0.67 against 0.71 for a lane group per row), beyond that the lane groups win by far (C = 100: 0.89
    // against 0.75, C = 172: 2.5 against 0.91).
    if (C >= 2 && C <= 88) {
        // rows contiguous and tile origins 16-byte aligned (R is a multiple of 8): copy tiles with 128-bit accesses
        const bool contig = C <= 64 && (C & 1) && ld == C && (dlogits == nullptr || ldd == C) &&
                            reinterpret_cast<uintptr_t>(logits) % 16 == 0 && reinterpret_cast<uintptr_t>(dlogits) % 16 == 0;
        const int CP = contig ? (int)C : ((int)C | 1);
        // rows per tile: 256 or 128 for the vector-copy kernel; the element-copy kernel runs best with tiles of at
        // most 26 KB, so that six or more workgroups share a compute unit and overlap their copy and row phases
        // (C = 47 in rows of 48: 0.53 ms with 256 rows, 0.39 with 128; C = 40: 0.44 / 0.29; C = 64: 0.60 / 0.54 with 64)
        int R = C <= 47 ? 256 : 128;
        if (!contig)
            while (R > 32 && (size_t)R * CP * sizeof(float) > 26 * 1024) R >>= 1;
        blocks = (unsigned)std::max<int64_t>(1, std::min<int64_t>(plx::ceil_div(M, R), kXentMaxBlocks));
        const size_t shm = (size_t)R * CP * sizeof(float);
        if (contig) launch_tiled_reg<T>(a, C, R, blocks, shm, st);
        else softmax_xent_tiled_kernel<T><<<blocks, 256, shm, st>>>(a, R, CP);
        PLX_LAUNCH_CHECK("softmax_xent_tiled_kernel");
    } else {
        const int64_t rows_per_block = 4 * (64 / lpr);
        blocks = (unsigned)std::max<int64_t>(1, std::min<int64_t>(plx::ceil_div(M, rows_per_block), kXentMaxBlocks));
        int rc = -1;
        switch (lpr) {
            case 1: rc = launch_xent<T, 1>(a, per, blocks, st); break;
            case 64: rc = launch_xent<T, 64>(a, per, blocks, st); break;
            default: break;
        }
        if (rc != 0) return plx::fail(PLX_ERR_UNSUPPORTED, "softmax_xent: no kernel for C=%lld", (long long)C);
        PLX_LAUNCH_CHECK("softmax_xent_kernel");
    }
    xent_finish_kernel<<<1, 256, 0, st>>>(a.partials, (int)blocks, 1.0 / (double)num_nodes, loss);
    PLX_LAUNCH_CHECK("xent_finish_kernel");
    return PLX_OK;
}

}  // namespace

extern "C" {

int plx_softmax_xent_f32(int64_t M, int64_t C, const float *logits, int64_t ld, const int64_t *labels,
                         int64_t num_nodes, int64_t num_classes, int64_t row_offset, float gscale, float *loss,
                         float *dlogits, int64_t ldd, void *workspace, size_t workspace_bytes, void *stream)
{
    return softmax_xent_impl<float>(M, C, logits, ld, labels, num_nodes, num_classes, row_offset, gscale, loss, dlogits, ldd,
                                    workspace, workspace_bytes, stream);
}

int plx_softmax_xent_bf16(int64_t M, int64_t C, const uint16_t *logits, int64_t ld, const int64_t *labels,
                          int64_t num_nodes, int64_t num_classes, int64_t row_offset, float gscale, float *loss,
                          uint16_t *dlogits, int64_t ldd, void *workspace, size_t workspace_bytes, void *stream)
{
    return softmax_xent_impl<uint16_t>(M, C, logits, ld, labels, num_nodes, num_classes, row_offset, gscale, loss, dlogits,
                                       ldd, workspace, workspace_bytes, stream);
}

}  // extern "C"
