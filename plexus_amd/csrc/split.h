// Exact three-way bf16 splits of fp32 values and the six-product accumulation on the bf16 matrix cores: shared by the
// split products (gemm_split.hip: NT forms, gemm_split_tn.hip: the reduction over the rows).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "bf16.h"

namespace plx {
namespace split {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // plain vector type: register arrays of it stay in registers

// x = p0 + p1 + p2 exactly (bf16 pieces, round to nearest even each); pieces of 2 values packed per word.  Holds for
// every value that needs_care() does not name.
__device__ __forceinline__ void split2(float x, float y, uint32_t &p0, uint32_t &p1, uint32_t &p2)
{
    p0 = plx::pack_bf16x2(x, y);
    const float rx = x - __uint_as_float(p0 << 16), ry = y - __uint_as_float(p0 & 0xffff0000u);
    p1 = plx::pack_bf16x2(rx, ry);
    const float sx = rx - __uint_as_float(p1 << 16), sy = ry - __uint_as_float(p1 & 0xffff0000u);
    p2 = plx::pack_bf16x2(sx, sy);
}

// The same split; true if x or y is a value the split cannot carry (see needs_care): the first piece of such a value is Inf
// or NaN, which leaves NaN as the last residual, and no other value does.  One compare for the two values.
__device__ __forceinline__ bool split2_checked(float x, float y, uint32_t &p0, uint32_t &p1, uint32_t &p2)
{
    p0 = plx::pack_bf16x2(x, y);
    const float rx = x - __uint_as_float(p0 << 16), ry = y - __uint_as_float(p0 & 0xffff0000u);
    p1 = plx::pack_bf16x2(rx, ry);
    const float sx = rx - __uint_as_float(p1 << 16), sy = ry - __uint_as_float(p1 & 0xffff0000u);
    p2 = plx::pack_bf16x2(sx, sy);
    return __builtin_isunordered(sx, sy);
}

// The same split in two halves, for kernels that place them between other instructions: the first half gives the first
// piece and what it leaves, the second the other two pieces and the same answer as split2_checked.
__device__ __forceinline__ void split2_first(float x, float y, uint32_t &p0, float &rx, float &ry)
{
    p0 = plx::pack_bf16x2(x, y);
    rx = x - __uint_as_float(p0 << 16);
    ry = y - __uint_as_float(p0 & 0xffff0000u);
}
__device__ __forceinline__ bool split2_second(float rx, float ry, uint32_t &p1, uint32_t &p2)
{
    p1 = plx::pack_bf16x2(rx, ry);
    const float sx = rx - __uint_as_float(p1 << 16), sy = ry - __uint_as_float(p1 & 0xffff0000u);
    p2 = plx::pack_bf16x2(sx, sy);
    return __builtin_isunordered(sx, sy);
}

// Values the split cannot carry: Inf and NaN (Inf times a zero piece is NaN, where the fp32 product gives Inf), and finite
// values of 0x7f7f8000 (3.3895e38) or more in magnitude, whose rounding to bf16 overflows.  One compare per element
// (NaN fails the "less than").  A kernel that meets one raises the flag word of its call, and the whole product is then
// redone by the fp32 MFMA kernel.
__device__ __forceinline__ int needs_care(float x) { return !(fabsf(x) < 3.3895313892515355e38f) ? 1 : 0; }
__device__ __forceinline__ int needs_care(const float4 &v) { return needs_care(v.x) | needs_care(v.y) | needs_care(v.z) | needs_care(v.w); }

// true if one of the eight bf16 values of a first-plane vector is Inf or NaN
__device__ __forceinline__ bool plane0_nonfinite(const u32x4 &v)
{
    uint32_t t = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) t |= (v[i] & 0x7f807f80u) + 0x00800080u;
    return (t & 0x80008000u) != 0u;
}

// six piece products of one 32 x 32 x 16 block, smallest terms first
__device__ __forceinline__ floatx16 mfma6(bf16x8 a0, bf16x8 a1, bf16x8 a2, bf16x8 b0, bf16x8 b1, bf16x8 b2, floatx16 acc)
{
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, b0, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b2, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc, 0, 0, 0);
    return acc;
}

}  // namespace split
}  // namespace plx
