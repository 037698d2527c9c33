// Device helpers of the chunked backward kernel.
#pragma once

#include "lfw_chunk.hpp"

namespace t2fw {
namespace bwd {

template <typename E> __device__ __forceinline__ uint2 packq(float a, float b, float c, float d) {
    return make_uint2(E::pack2(a, b), E::pack2(c, d));
}

template <typename E> __device__ __forceinline__ uint2 pack4v(const floatx4 &v) {
    return make_uint2(E::pack2(v[0], v[1]), E::pack2(v[2], v[3]));
}

__device__ __forceinline__ uint2 ld2(const u16 *p) { return *reinterpret_cast<const uint2 *>(p); }
__device__ __forceinline__ uint4 ld4(const u16 *p) { return *reinterpret_cast<const uint4 *>(p); }
__device__ __forceinline__ uint4 cat(uint2 a, uint2 b) { return make_uint4(a.x, a.y, b.x, b.y); }

template <typename E> __device__ __forceinline__ void unpack4(uint2 v, float (&o)[4]) {
    o[0] = E::to_f32((u16)(v.x & 0xffff));
    o[1] = E::to_f32((u16)(v.x >> 16));
    o[2] = E::to_f32((u16)(v.y & 0xffff));
    o[3] = E::to_f32((u16)(v.y >> 16));
}

// Sums over the four 16-lane rows of a wave with the gfx950 lane-swap instructions (VALU, no LDS
// round trip).  permlane16_swap(v, v) returns {rows [0,0,2,2] of v, rows [1,1,3,3] of v};
// permlane32_swap(v, v) returns {lower half in both halves, upper half in both halves}.
struct RowSums {
    float odd;      // this lane's value in the odd row of its row pair (rows 1 or 3)
    float pair;     // sum over the lane's row pair
    float hi;       // pair sum of rows 2 and 3
    float all;      // sum over the four rows
};
__device__ __forceinline__ RowSums row_sums(float a) {
    RowSums r;
    const u32 ab = __float_as_uint(a);
    const auto s16 = __builtin_amdgcn_permlane16_swap(ab, ab, false, false);
    r.odd = __uint_as_float(s16[1]);
    r.pair = __uint_as_float(s16[0]) + r.odd;
    const u32 pb = __float_as_uint(r.pair);
    const auto s32 = __builtin_amdgcn_permlane32_swap(pb, pb, false, false);
    r.hi = __uint_as_float(s32[1]);
    r.all = __uint_as_float(s32[0]) + r.hi;
    return r;
}

// Reverse running sum over the 16 tokens of a block, without LDS traffic: lane (g, r) holds d[i] for
// token 4g+i of its channel; on return d[i] = carry + sum of the tokens >= 4g+i, and carry has taken
// in the whole block.
__device__ __forceinline__ void reverse_running_sum_swap(float (&d)[4], float &carry, int g) {
    d[2] += d[3];
    d[1] += d[2];
    d[0] += d[1];
    const RowSums t = row_sums(d[0]);
    // rows above this one: the odd partner (for even rows) and the upper pair (for rows 0 and 1)
    const float higher = ((g & 1) ? 0.f : t.odd) + (g < 2 ? t.hi : 0.f) + carry;
#pragma unroll
    for (int i = 0; i < 4; ++i) d[i] += higher;
    carry += t.all;
}

}  // namespace bwd
}  // namespace t2fw
