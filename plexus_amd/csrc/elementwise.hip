// Bandwidth-bound helpers of the GCN layer: ReLU forward/backward for callers that keep the
// activation outside the layer, and the symmetric GCN normalisation of a CSR matrix.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "bf16.h"
#include "common.h"

namespace {

// These passes are bound by HBM.  What reaches the highest rates here: one 128-bit item per thread with a grid
// that covers the tensor (no grid-stride loop), and non-temporal accesses, since nothing is read twice.
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load_nt(const float *q)
{
    const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(q));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void store_nt(float *q, float4 x)
{
    const f32x4 t = {x.x, x.y, x.z, x.w};
    __builtin_nontemporal_store(t, reinterpret_cast<f32x4 *>(q));
}

// one item (float4 when everything is 16-byte aligned, else one element) per thread; FLAT: rows are contiguous
// in all operands, so the matrix is addressed as one long row without a division
template <bool BWD, bool VEC4, bool FLAT>
__global__ void __launch_bounds__(256) relu_kernel(int64_t M, int64_t N, const float *in, int64_t ldi, const float *ref,
                                                   int64_t ldr, float *out, int64_t ldo)  // out may alias in (or ref)
{
    const int64_t per_row = VEC4 ? N / 4 : N;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M * per_row) return;
    const int64_t r = FLAT ? 0 : i / per_row;
    const int64_t c = (FLAT ? i : i % per_row) * (VEC4 ? 4 : 1);
    if constexpr (VEC4) {
        const float4 x = load_nt(in + r * ldi + c);
        float4 y;
        if constexpr (BWD) {
            const float4 m = load_nt(ref + r * ldr + c);
            y = make_float4(m.x > 0.f ? x.x : 0.f, m.y > 0.f ? x.y : 0.f, m.z > 0.f ? x.z : 0.f, m.w > 0.f ? x.w : 0.f);
        } else {
            y = make_float4(fmaxf(x.x, 0.f), fmaxf(x.y, 0.f), fmaxf(x.z, 0.f), fmaxf(x.w, 0.f));
        }
        store_nt(out + r * ldo + c, y);
    } else {
        const float x = in[r * ldi + c];
        if constexpr (BWD)
            out[r * ldo + c] = ref[r * ldr + c] > 0.f ? x : 0.f;
        else
            out[r * ldo + c] = fmaxf(x, 0.f);
    }
}

bool aligned4(const void *p, int64_t ld) { return reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0; }

// rows of `row_bytes` bytes from one pitch to another; UNIT = bytes per thread item (16 when everything is 16-byte
// aligned, else 4 or 2)
template <typename UNIT>
__global__ void __launch_bounds__(256) copy_rows_kernel(int64_t M, int64_t units_per_row, const char *__restrict__ src, int64_t src_pitch,
                                                        char *__restrict__ dst, int64_t dst_pitch)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M * units_per_row) return;
    const int64_t r = i / units_per_row, c = i % units_per_row;
    reinterpret_cast<UNIT *>(dst + r * dst_pitch)[c] = reinterpret_cast<const UNIT *>(src + r * src_pitch)[c];
}

// d^-1/2 of the row sums.  A wavefront sums one row; rows longer than kLongRow entries (the hubs of a power-law
// graph: one row of the benchmark graph holds 1.1 M entries) are left to the whole workgroup afterwards, with four
// loads in flight per thread.  Both orders of summation are fixed.
constexpr int kLongRow = 4096;

__global__ void __launch_bounds__(256) row_dinv_kernel(int64_t M, const int32_t *__restrict__ rowptr,
                                                       const float *__restrict__ val, float *__restrict__ dinv)
{
    __shared__ float part[4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t r = (int64_t)blockIdx.x * 4 + wave;
    if (r < M) {
        const int a = rowptr[r], b = rowptr[r + 1];
        if (b - a <= kLongRow) {
            float s = 0.f;
            for (int j = a + lane; j < b; j += 64) s += val[j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
            if (lane == 0) dinv[r] = s > 0.f ? 1.f / sqrtf(s) : 0.f;
        }
    }
    for (int q = 0; q < 4; ++q) {  // the long rows among this workgroup's four, one after the other
        const int64_t rq = (int64_t)blockIdx.x * 4 + q;
        if (rq >= M) break;
        const int a = rowptr[rq], b = rowptr[rq + 1];
        if (b - a <= kLongRow) continue;  // uniform over the workgroup
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        int j = a + threadIdx.x;
        for (; j + 768 < b; j += 1024) {
            s0 += val[j];
            s1 += val[j + 256];
            s2 += val[j + 512];
            s3 += val[j + 768];
        }
        for (; j < b; j += 256) s0 += val[j];
        float s = (s0 + s1) + (s2 + s3);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        __syncthreads();
        if (lane == 0) part[wave] = s;
        __syncthreads();
        if (threadIdx.x == 0) {
            const float t = (part[0] + part[1]) + (part[2] + part[3]);
            dinv[rq] = t > 0.f ? 1.f / sqrtf(t) : 0.f;
        }
    }
}

// out[j] = dinv[row(j)] val[j] dinv[col[j]], entry by entry; the row of an entry is found by binary search in the row
// pointer (small against the entries, so it stays in cache), which costs a hub row no more than any other.  The number
// of entries is read from the row pointer on the device, so the host does not have to know it.
__global__ void __launch_bounds__(256) gcn_scale_kernel(int64_t M, const int32_t *__restrict__ rowptr,
                                                        const int32_t *__restrict__ col, const float *__restrict__ val,
                                                        const float *__restrict__ dinv, float *__restrict__ out)
{
    const int64_t nnz = rowptr[M];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < nnz; j += stride) {
        int64_t lo = 0, hi = M;  // rowptr[lo] <= j < rowptr[hi]
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if ((int64_t)rowptr[mid] <= j)
                lo = mid;
            else
                hi = mid;
        }
        out[j] = (dinv[lo] * val[j]) * dinv[col[j]];
    }
}

// one pass over (p, g, m, v): 16 bytes read and 12 written per element; one item per thread
template <bool VEC4>
__global__ void __launch_bounds__(256) adamw_kernel(int64_t n, float *__restrict__ p, const float *__restrict__ g,
                                                    float *__restrict__ m, float *__restrict__ v, float decay,
                                                    float one_minus_b1, float b2, float one_minus_b2, float step_size,
                                                    float inv_bc2_sqrt, float eps)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (VEC4 ? n / 4 : n)) return;
    if constexpr (VEC4) {
        float4 pp = load_nt(p + 4 * i);
        const float4 gg = load_nt(g + 4 * i);
        float4 mm = load_nt(m + 4 * i);
        float4 vv = load_nt(v + 4 * i);
        float *pe = &pp.x, *me = &mm.x, *ve = &vv.x;
        const float *ge = &gg.x;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            me[e] = me[e] + (ge[e] - me[e]) * one_minus_b1;
            ve[e] = ve[e] * b2 + (ge[e] * ge[e]) * one_minus_b2;
            const float denom = sqrtf(ve[e]) * inv_bc2_sqrt + eps;
            pe[e] = pe[e] * decay - step_size * (me[e] / denom);
        }
        store_nt(p + 4 * i, pp);
        store_nt(m + 4 * i, mm);
        store_nt(v + 4 * i, vv);
    } else {
        const float ge = g[i];
        const float me = m[i] + (ge - m[i]) * one_minus_b1;
        const float ve = v[i] * b2 + (ge * ge) * one_minus_b2;
        const float denom = sqrtf(ve) * inv_bc2_sqrt + eps;
        p[i] = p[i] * decay - step_size * (me / denom);
        m[i] = me;
        v[i] = ve;
    }
}

// AdamW with a bf16 gradient; optionally refreshes a bf16 copy of the parameter in the same pass
// (14 bytes read and 12 or 14 written per element; VEC4: four elements per thread, 128-bit fp32 and 64-bit bf16 accesses)
template <bool VEC4>
__global__ void __launch_bounds__(256) adamw_grad_bf16_kernel(int64_t n, float *__restrict__ p, const uint16_t *__restrict__ g,
                                                              float *__restrict__ m, float *__restrict__ v, float decay,
                                                              float one_minus_b1, float b2, float one_minus_b2,
                                                              float step_size, float inv_bc2_sqrt, float eps,
                                                              uint16_t *__restrict__ p16)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (VEC4 ? n / 4 : n)) return;
    if constexpr (VEC4) {
        float4 pp = load_nt(p + 4 * i);
        const uint2 gw = reinterpret_cast<const uint2 *>(g)[i];
        float4 mm = load_nt(m + 4 * i);
        float4 vv = load_nt(v + 4 * i);
        const float ge[4] = {__uint_as_float(gw.x << 16), __uint_as_float(gw.x & 0xffff0000u), __uint_as_float(gw.y << 16),
                             __uint_as_float(gw.y & 0xffff0000u)};
        float *pe = &pp.x, *me = &mm.x, *ve = &vv.x;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            me[e] = me[e] + (ge[e] - me[e]) * one_minus_b1;
            ve[e] = ve[e] * b2 + (ge[e] * ge[e]) * one_minus_b2;
            const float denom = sqrtf(ve[e]) * inv_bc2_sqrt + eps;
            pe[e] = pe[e] * decay - step_size * (me[e] / denom);
        }
        store_nt(p + 4 * i, pp);
        store_nt(m + 4 * i, mm);
        store_nt(v + 4 * i, vv);
        if (p16 != nullptr) reinterpret_cast<uint2 *>(p16)[i] = make_uint2(plx::pack_bf16x2(pp.x, pp.y), plx::pack_bf16x2(pp.z, pp.w));
    } else {
        const float ge = plx::bf16_to_f32(g[i]);
        const float me = m[i] + (ge - m[i]) * one_minus_b1;
        const float ve = v[i] * b2 + (ge * ge) * one_minus_b2;
        const float denom = sqrtf(ve) * inv_bc2_sqrt + eps;
        const float pe = p[i] * decay - step_size * (me / denom);
        p[i] = pe;
        m[i] = me;
        v[i] = ve;
        if (p16 != nullptr) p16[i] = (uint16_t)plx::f32_to_bf16(pe);
    }
}

int relu_common(bool bwd, int64_t M, int64_t N, const float *in, int64_t ldi, const float *ref, int64_t ldr, float *out,
                int64_t ldo, void *stream)
{
    PLX_REQUIRE(M >= 0 && N >= 0, "relu: negative shape");
    if (M == 0 || N == 0) return PLX_OK;
    PLX_REQUIRE(in && out && (!bwd || ref), "relu: NULL operand");
    PLX_REQUIRE(ldi >= N && ldo >= N && (!bwd || ldr >= N), "relu: leading dimension smaller than N");
    const bool flat = ldi == N && ldo == N && (!bwd || ldr == N);  // contiguous rows everywhere: one long row
    if (flat) {
        N *= M;
        M = 1;
        ldi = ldo = ldr = N;
    }
    const bool v4 = N % 4 == 0 && aligned4(in, ldi) && aligned4(out, ldo) && (!bwd || aligned4(ref, ldr));
    const int64_t total = M * (v4 ? N / 4 : N);
    const int64_t nblocks = plx::ceil_div(total, 256);
    PLX_REQUIRE(nblocks < (1ll << 31), "relu: tensor too large for one launch");
    const unsigned blocks = (unsigned)nblocks;
    hipStream_t st = plx::as_stream(stream);
#define PLX_RELU_LAUNCH(B, V, F) relu_kernel<B, V, F><<<blocks, 256, 0, st>>>(M, N, in, ldi, ref, ldr, out, ldo)
    if (bwd) {
        if (v4) {
            if (flat) PLX_RELU_LAUNCH(true, true, true); else PLX_RELU_LAUNCH(true, true, false);
        } else {
            if (flat) PLX_RELU_LAUNCH(true, false, true); else PLX_RELU_LAUNCH(true, false, false);
        }
    } else {
        if (v4) {
            if (flat) PLX_RELU_LAUNCH(false, true, true); else PLX_RELU_LAUNCH(false, true, false);
        } else {
            if (flat) PLX_RELU_LAUNCH(false, false, true); else PLX_RELU_LAUNCH(false, false, false);
        }
    }
#undef PLX_RELU_LAUNCH
    PLX_LAUNCH_CHECK("relu_kernel");
    return PLX_OK;
}

// y[i] = x[i] * (*scale): the upstream gradient of a scalar loss lives on the device and is read there, so the
// host never waits for it.  T = float or bf16 bits.  VEC: one 128-bit item per thread over the first
// n - n % kPer elements, and one more thread for the few elements left over; otherwise one element per thread.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256) scale_by_device_scalar_kernel(int64_t n, const T *x, const float *__restrict__ scale, T *y)
{
    constexpr int kPer = 16 / (int)sizeof(T);
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float s = *scale;
    auto one = [&](int64_t e) {
        if constexpr (sizeof(T) == 4)
            y[e] = x[e] * s;
        else
            y[e] = (uint16_t)plx::f32_to_bf16(plx::bf16_to_f32(x[e]) * s);
    };
    if constexpr (!VEC) {
        if (i < n) one(i);
    } else {
        const int64_t items = n / kPer;
        if (i > items) return;
        if (i == items) {
            for (int64_t e = items * kPer; e < n; ++e) one(e);
        } else if constexpr (sizeof(T) == 4) {
            const float4 v = load_nt(x + 4 * i);
            store_nt(y + 4 * i, make_float4(v.x * s, v.y * s, v.z * s, v.w * s));
        } else {
            const uint4 v = reinterpret_cast<const uint4 *>(x)[i];
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o[j] = plx::pack_bf16x2(__uint_as_float(w[j] << 16) * s, __uint_as_float(w[j] & 0xffff0000u) * s);
            reinterpret_cast<uint4 *>(y)[i] = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
}

template <typename T>
int scale_common(int64_t n, const T *x, const float *scale, T *y, void *stream)
{
    PLX_REQUIRE(n >= 0, "scale: negative size");
    if (n == 0) return PLX_OK;
    PLX_REQUIRE(x && scale && y, "scale: NULL operand");
    constexpr int kPer = 16 / (int)sizeof(T);
    const bool vec = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
    const int64_t nblocks = plx::ceil_div(vec ? n / kPer + 1 : n, 256);
    PLX_REQUIRE(nblocks < (1ll << 31), "scale: tensor too large for one launch");
    hipStream_t st = plx::as_stream(stream);
    if (vec)
        scale_by_device_scalar_kernel<T, true><<<(unsigned)nblocks, 256, 0, st>>>(n, x, scale, y);
    else
        scale_by_device_scalar_kernel<T, false><<<(unsigned)nblocks, 256, 0, st>>>(n, x, scale, y);
    PLX_LAUNCH_CHECK("scale_by_device_scalar_kernel");
    return PLX_OK;
}

}  // namespace

int plx::row_sums_rsqrt(int64_t M, const int32_t *rowptr, const float *val, float *dinv, void *stream)
{
    if (M <= 0) return PLX_OK;
    row_dinv_kernel<<<(unsigned)plx::ceil_div(M, 4), 256, 0, plx::as_stream(stream)>>>(M, rowptr, val, dinv);
    PLX_LAUNCH_CHECK("row_dinv_kernel");
    return PLX_OK;
}

extern "C" {

int plx_scale_by_device_scalar_f32(int64_t n, const float *x, const float *scale, float *y, void *stream)
{
    return scale_common<float>(n, x, scale, y, stream);
}

int plx_scale_by_device_scalar_bf16(int64_t n, const uint16_t *x, const float *scale, uint16_t *y, void *stream)
{
    return scale_common<uint16_t>(n, x, scale, y, stream);
}

int plx_copy_rows(int64_t M, int64_t row_bytes, const void *src, int64_t src_pitch_bytes, void *dst, int64_t dst_pitch_bytes,
                  void *stream)
{
    PLX_REQUIRE(M >= 0 && row_bytes >= 0, "copy_rows: negative size");
    if (M == 0 || row_bytes == 0) return PLX_OK;
    PLX_REQUIRE(src != nullptr && dst != nullptr, "copy_rows: NULL operand");
    PLX_REQUIRE(src_pitch_bytes >= row_bytes && dst_pitch_bytes >= row_bytes, "copy_rows: pitch smaller than a row");
    const uintptr_t all = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | (uintptr_t)row_bytes |
                          (uintptr_t)src_pitch_bytes | (uintptr_t)dst_pitch_bytes;
    PLX_REQUIRE(all % 2 == 0, "copy_rows: addresses, pitches and the row length must be multiples of 2 bytes");
    hipStream_t st = plx::as_stream(stream);
    const char *s = static_cast<const char *>(src);
    char *d = static_cast<char *>(dst);
    auto blocks = [&](int64_t unit) { return (unsigned)plx::ceil_div(M * (row_bytes / unit), 256); };
    PLX_REQUIRE(M * row_bytes / 2 < (1ll << 39), "copy_rows: too large");
    if (all % 16 == 0) copy_rows_kernel<uint4><<<blocks(16), 256, 0, st>>>(M, row_bytes / 16, s, src_pitch_bytes, d, dst_pitch_bytes);
    else if (all % 4 == 0) copy_rows_kernel<uint32_t><<<blocks(4), 256, 0, st>>>(M, row_bytes / 4, s, src_pitch_bytes, d, dst_pitch_bytes);
    else copy_rows_kernel<uint16_t><<<blocks(2), 256, 0, st>>>(M, row_bytes / 2, s, src_pitch_bytes, d, dst_pitch_bytes);
    PLX_LAUNCH_CHECK("copy_rows_kernel");
    return PLX_OK;
}

int plx_relu_f32(int64_t M, int64_t N, const float *X, int64_t ldx, float *Y, int64_t ldy, void *stream)
{
    return relu_common(false, M, N, X, ldx, nullptr, 0, Y, ldy, stream);
}

int plx_relu_bwd_f32(int64_t M, int64_t N, const float *dY, int64_t lddy, const float *Y, int64_t ldy, float *dX,
                     int64_t lddx, void *stream)
{
    return relu_common(true, M, N, dY, lddy, Y, ldy, dX, lddx, stream);
}

// The hyperparameters arrive as doubles, as Python holds them, and are rounded to fp32 only where torch's optimizer
// rounds them (1 - beta as a double first), so that the moments match torch.optim.AdamW to fp32 rounding.
struct AdamScalars {
    float decay, one_minus_b1, b2, one_minus_b2, step_size, inv_bc2_sqrt, eps;
};

static AdamScalars adam_scalars(double lr, double beta1, double beta2, double eps, double weight_decay, int64_t step)
{
    const double bc1 = 1.0 - std::pow(beta1, (double)step);
    const double bc2 = 1.0 - std::pow(beta2, (double)step);
    AdamScalars a;
    a.decay = (float)(1.0 - lr * weight_decay);
    a.one_minus_b1 = (float)(1.0 - beta1);
    a.b2 = (float)beta2;
    a.one_minus_b2 = (float)(1.0 - beta2);
    a.step_size = (float)(lr / bc1);
    a.inv_bc2_sqrt = (float)(1.0 / std::sqrt(bc2));
    a.eps = (float)eps;
    return a;
}

int plx_adamw_f32(int64_t n, float *param, const float *grad, float *exp_avg, float *exp_avg_sq, double lr, double beta1,
                  double beta2, double eps, double weight_decay, int64_t step, void *stream)
{
    PLX_REQUIRE(n >= 0 && step >= 1, "adamw: bad size or step (n=%lld step=%lld)", (long long)n, (long long)step);
    if (n == 0) return PLX_OK;
    PLX_REQUIRE(param && grad && exp_avg && exp_avg_sq, "adamw: NULL operand");
    PLX_REQUIRE(beta1 >= 0.0 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0, "adamw: betas must lie in [0, 1)");
    const AdamScalars a = adam_scalars(lr, beta1, beta2, eps, weight_decay, step);
    const bool v4 = n % 4 == 0 && reinterpret_cast<uintptr_t>(param) % 16 == 0 && reinterpret_cast<uintptr_t>(grad) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(exp_avg) % 16 == 0 && reinterpret_cast<uintptr_t>(exp_avg_sq) % 16 == 0;
    const int64_t count = v4 ? n / 4 : n;
    PLX_REQUIRE(plx::ceil_div(count, 256) < (1ll << 31), "adamw: tensor too large for one launch");
    const unsigned blocks = (unsigned)plx::ceil_div(count, 256);
    hipStream_t st = plx::as_stream(stream);
    if (v4)
        adamw_kernel<true><<<blocks, 256, 0, st>>>(n, param, grad, exp_avg, exp_avg_sq, a.decay, a.one_minus_b1, a.b2, a.one_minus_b2,
                                                   a.step_size, a.inv_bc2_sqrt, a.eps);
    else
        adamw_kernel<false><<<blocks, 256, 0, st>>>(n, param, grad, exp_avg, exp_avg_sq, a.decay, a.one_minus_b1, a.b2, a.one_minus_b2,
                                                    a.step_size, a.inv_bc2_sqrt, a.eps);
    PLX_LAUNCH_CHECK("adamw_kernel");
    return PLX_OK;
}

int plx_adamw_f32_grad_bf16(int64_t n, float *param, const uint16_t *grad, float *exp_avg, float *exp_avg_sq, double lr,
                            double beta1, double beta2, double eps, double weight_decay, int64_t step, uint16_t *param_bf16,
                            void *stream)
{
    PLX_REQUIRE(n >= 0 && step >= 1, "adamw: bad size or step (n=%lld step=%lld)", (long long)n, (long long)step);
    if (n == 0) return PLX_OK;
    PLX_REQUIRE(param && grad && exp_avg && exp_avg_sq, "adamw: NULL operand");
    PLX_REQUIRE(beta1 >= 0.0 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0, "adamw: betas must lie in [0, 1)");
    const AdamScalars a = adam_scalars(lr, beta1, beta2, eps, weight_decay, step);
    const bool v4 = n % 4 == 0 && reinterpret_cast<uintptr_t>(param) % 16 == 0 && reinterpret_cast<uintptr_t>(grad) % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(exp_avg) % 16 == 0 && reinterpret_cast<uintptr_t>(exp_avg_sq) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(param_bf16) % 8 == 0;
    PLX_REQUIRE(plx::ceil_div(v4 ? n / 4 : n, 256) < (1ll << 31), "adamw: tensor too large for one launch");
    const unsigned blocks = (unsigned)plx::ceil_div(v4 ? n / 4 : n, 256);
    hipStream_t st = plx::as_stream(stream);
    if (v4)
        adamw_grad_bf16_kernel<true><<<blocks, 256, 0, st>>>(n, param, grad, exp_avg, exp_avg_sq, a.decay, a.one_minus_b1, a.b2,
                                                             a.one_minus_b2, a.step_size, a.inv_bc2_sqrt, a.eps, param_bf16);
    else
        adamw_grad_bf16_kernel<false><<<blocks, 256, 0, st>>>(n, param, grad, exp_avg, exp_avg_sq, a.decay, a.one_minus_b1, a.b2,
                                                              a.one_minus_b2, a.step_size, a.inv_bc2_sqrt, a.eps, param_bf16);
    PLX_LAUNCH_CHECK("adamw_grad_bf16_kernel");
    return PLX_OK;
}

int plx_gcn_norm_csr_f32(int64_t M, const int32_t *rowptr, const int32_t *col, const float *val_in, float *val_out,
                         float *dinv, void *stream)
{
    PLX_REQUIRE(M >= 0 && M < (1ll << 31) - 1, "gcn_norm: bad row count");
    if (M == 0) return PLX_OK;
    PLX_REQUIRE(rowptr && col && val_in && val_out && dinv, "gcn_norm: NULL operand");
    hipStream_t st = plx::as_stream(stream);
    int rc = plx::row_sums_rsqrt(M, rowptr, val_in, dinv, stream);
    if (rc != PLX_OK) return rc;
    gcn_scale_kernel<<<256 * 32, 256, 0, st>>>(M, rowptr, col, val_in, dinv, val_out);
    PLX_LAUNCH_CHECK("gcn_scale_kernel");
    return PLX_OK;
}

}  // extern "C"
