// bf16 <-> fp32 helpers shared by the kernels (bf16 travels as raw uint16 bit patterns) and the
// counter-based generator behind the fused dropout.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace plx {

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint32_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// two fp32 -> packed bf16 pair with the hardware conversion (v_cvt_pk_bf16_f32: round to nearest even)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const float2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// true where the bf16 value is > 0 (positive sign, non-zero magnitude)
__device__ __forceinline__ bool bf16_positive(uint32_t bits16) { return (bits16 & 0x8000u) == 0 && (bits16 & 0x7fffu) != 0; }

// Philox-4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11).  One call yields 4 x 32 random bits.
struct Philox4 {
    uint32_t v[4];
};

__host__ __device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1)
{
    constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)M0 * c0;
        const uint64_t p1 = (uint64_t)M1 * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0;
        c1 = n1;
        c2 = n2;
        c3 = n3;
        k0 += W0;
        k1 += W1;
    }
    Philox4 out;
    out.v[0] = c0;
    out.v[1] = c1;
    out.v[2] = c2;
    out.v[3] = c3;
    return out;
}

// Dropout keep decision of element e of a logical matrix (row-major linear index):
//   call q = e / 8 of Philox(counter = (q, offset), key = seed) gives eight 16-bit lanes
//   (word w = (e % 8) / 2, low half for even e); the element is kept iff its lane >= thresh16,
//   thresh16 = round(p * 65536).
__host__ __device__ __forceinline__ uint32_t dropout_lane16(const Philox4 &r, int slot)
{
    const uint32_t w = r.v[slot >> 1];
    return (slot & 1) ? (w >> 16) : (w & 0xffffu);
}

}  // namespace plx
