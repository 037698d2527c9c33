// Device helpers shared by the chunked backward kernels (whole-row and split-by-side variants).
#pragma once

#include "lfw_chunk.hpp"

// Build-time diagnostic (-DT2FW_PHASE_TIMERS): workgroup 0 accumulates shader-clock ticks
// per phase into row_flags[64..]; off in the shipped library.
#ifdef T2FW_PHASE_TIMERS
#define PHASE_BEGIN() unsigned long long ph_t = __builtin_amdgcn_s_memtime(); unsigned long long ph_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}; int ph_sel = 0
#define PHASE_MARK(i) { const unsigned long long ph_n = __builtin_amdgcn_s_memtime(); ph_acc[(i) + ph_sel] += ph_n - ph_t; ph_t = ph_n; }
#define PHASE_END(slot) if (b == 0 && (tid & 63) == 0) { for (int ph_i = 0; ph_i < 8; ++ph_i) p.row_flags[64 + (slot) * 8 + ph_i] = (int)(ph_acc[ph_i] & 0x7fffffff); }
#define PHASE_SELECT(v) ph_sel = (v)
#else
#define PHASE_BEGIN()
#define PHASE_MARK(i)
#define PHASE_END(slot)
#define PHASE_SELECT(v)
#endif

namespace t2fw {
namespace bwd {

// ---- stage schedule ----------------------------------------------------------------------
// Chunks are visited from the last one down; a chunk with nb blocks takes nb "R" stages
// (blocks 0..nb-1) followed by nb "B" stages (blocks nb-1..0).
struct StageInfo {
    int chunk;
    int block;      // block inside the chunk
    bool bmode;     // false: recompute sweep, true: backward sweep
};

// 32-bit arithmetic only; NB is a power of two, so the divisions are shifts.
template <int NB> struct Schedule {
    int NC, total, nb_last;
    __device__ Schedule(int64_t T, int64_t NC_, int C) {
        NC = (int)NC_;
        const int len_last = (int)(T - (NC_ - 1) * C);
        nb_last = (len_last + CH_L - 1) / CH_L;
        total = 2 * nb_last + (NC - 1) * 2 * NB;
    }
    __device__ StageInfo at(int s) const {
        StageInfo r;
        int local, nb;
        if (s < 2 * nb_last) {
            r.chunk = NC - 1;
            local = s;
            nb = nb_last;
        } else {
            const unsigned s2 = (unsigned)(s - 2 * nb_last);
            r.chunk = NC - 2 - (int)(s2 / (2u * NB));
            local = (int)(s2 % (2u * NB));
            nb = NB;
        }
        r.bmode = local >= nb;
        r.block = r.bmode ? 2 * nb - 1 - local : local;
        return r;
    }
};

template <typename E> __device__ __forceinline__ uint2 packq(float a, float b, float c, float d) {
    return make_uint2(E::pack2(a, b), E::pack2(c, d));
}

template <typename E> __device__ __forceinline__ uint2 pack4v(const floatx4 &v) {
    return make_uint2(E::pack2(v[0], v[1]), E::pack2(v[2], v[3]));
}

template <typename IOE> __device__ __forceinline__ u32 gate_check(const u16 (&g)[CH_L]) {
    u16 mx = 0;
#pragma unroll
    for (int t = 0; t < CH_L; ++t) {
        const u16 m1 = (u16)(g[t] - 1);      // gates must lie in (0, 1]: 0 < bits <= bits(1.0)
        mx = m1 > mx ? m1 : mx;
    }
    return (mx >= IOE::ONE_BITS) ? 1u : 0u;
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

// Reverse running sum over the 16 tokens of a block: lane (g, r) holds d[i] for token 4g+i of its channel;
// returns the inclusive suffix sums plus `carry`, and updates carry to the value at token 0.
__device__ __forceinline__ void reverse_running_sum(float (&d)[4], float &carry, int g, int r) {
    d[2] += d[3];
    d[1] += d[2];
    d[0] += d[1];
    const float tot = d[0];
    const float t16 = __shfl_down(tot, 16, 64), t32 = __shfl_down(tot, 32, 64), t48 = __shfl_down(tot, 48, 64);
    const float higher = (g < 3 ? t16 : 0.f) + (g < 2 ? t32 : 0.f) + (g < 1 ? t48 : 0.f) + carry;
#pragma unroll
    for (int i = 0; i < 4; ++i) d[i] += higher;
    carry = __shfl(d[0], r, 64);
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

// As reverse_running_sum, without LDS traffic: lane (g, r) holds d[i] for token 4g+i of its channel.
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
