// Block-wise matrix-core form of the delta rule for D = M = 64, fp32 / fp16 / bf16 tensors (dfw_chunk_fwd.hip,
// dfw_chunk_bwd.hip): shared layout constants and device helpers.
//
// Inside a block of L = 16 steps that starts from the state S0 (all matrices with one row per step):
//   A  = strictly lower triangle of K K^T        Bq = strictly lower triangle of Q K^T
//   Delta = Tm (V - K S0^T),  Tm = (I + A)^-1    (the block's delta_t = v_t - S_{t-1} k_t)
//   O  = Q S0^T + Bq Delta                       S_L = S0 + Delta^T K
// A is nilpotent (A^16 = 0), so Tm = (I - A)(I + A^2)(I + A^4)(I + A^8): three squarings and a few more
// 16 x 16 products on the matrix cores instead of a 16-step substitution.  Tm and the transformed keys
// K' = Tm K do not depend on the state, so they are prepared ahead of the sequential pass, whose chain per
// block is then only  S0 -> Delta = Tm V - K' S0^T -> S_L.  The backward pass uses Tm transposed the same way.
//
// Precision: the matrix cores take bf16, so every operand (an fp32 or fp16 input, an fp32 intermediate) is
// split into a bf16 head and a bf16 remainder (x = hi + lo up to 2^-17 of x) and a product runs as three MFMAs
// (hi*hi + hi*lo + lo*hi) with fp32 accumulation: results carry fp32-level rounding (measured against the
// fp64 oracle: 3e-5 of max|ref|), not the 2^-9 of a single bf16 operand, before they are rounded to the tensors'
// type.  A caller that prefers speed asks for the heads alone (T2FW_FLAG_BF16_OPERANDS; template parameter
// SP = false below).
//
// Tensor element types: the kernels are templates over an element policy E (ElF32, El16<Fp16>, El16<Bf16>) that
// says how a lane moves elements between global memory and registers; all arithmetic is the same.
#pragma once

#include "lfw_chunk.hpp"
#include "lfw_chunk_bwd_dev.hpp"

namespace t2fw {

#if defined(__HIPCC__)
namespace dfwc {

using namespace bwd;

constexpr int DL = 16;                        // block length
constexpr int DNB = 2;                        // blocks per stage (one workgroup barrier per stage)
constexpr int DTS = 72;                       // row stride (elements) of token-major tiles [16 tokens][64 channels]
constexpr int DCS = 20;                       // row stride of channel-major tiles [64 channels][16 tokens]
constexpr int TM_TILE = DL * DTS * 2;         // bytes of one token-major tile (one of hi / lo)
constexpr int CM_TILE = CH_N * DCS * 2;       // bytes of one channel-major tile
constexpr int ST_TILE = 64 * 8;               // a 16 x 16 matrix as a packed MFMA operand: 8 bytes per lane

// ---- element types of the tensors ----------------------------------------------------------------------
// elem: the type in memory.  A value that is loaded ahead of its use stays in the form it was loaded in (elem,
// Raw16) and is converted where it is used: a conversion next to the load would wait for the load there.
struct ElF32 {
    typedef float elem;
    struct Raw16 {          // sixteen consecutive channels of one token
        float4 v[4];
    };
    static __device__ __forceinline__ float f(elem x) { return x; }
    static __device__ __forceinline__ elem e(float x) { return x; }
    static __device__ __forceinline__ Raw16 load16(const elem *p) {
        Raw16 r;
#pragma unroll
        for (int a = 0; a < 4; ++a) r.v[a] = reinterpret_cast<const float4 *>(p)[a];
        return r;
    }
    static __device__ __forceinline__ void floats(const Raw16 &r, float (&o)[16]) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            o[4 * a] = r.v[a].x; o[4 * a + 1] = r.v[a].y; o[4 * a + 2] = r.v[a].z; o[4 * a + 3] = r.v[a].w;
        }
    }
    // four consecutive elements, 16-byte aligned
    static __device__ __forceinline__ floatx4 load4(const elem *p) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        return floatx4{t.x, t.y, t.z, t.w};
    }
    static __device__ __forceinline__ void store4(elem *p, const floatx4 &v) {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <typename IOE> struct El16 {          // IOE = Fp16 or Bf16 (lfw_chunk.hpp)
    typedef u16 elem;
    struct Raw16 {
        uint4 v[2];
    };
    static __device__ __forceinline__ float f(elem x) { return IOE::to_f32(x); }
    static __device__ __forceinline__ elem e(float x) { return cvt1<IOE>(x); }
    static __device__ __forceinline__ Raw16 load16(const elem *p) {
        Raw16 r;
        r.v[0] = reinterpret_cast<const uint4 *>(p)[0];
        r.v[1] = reinterpret_cast<const uint4 *>(p)[1];
        return r;
    }
    static __device__ __forceinline__ void floats(const Raw16 &r, float (&o)[16]) {
        const u32 w[8] = {r.v[0].x, r.v[0].y, r.v[0].z, r.v[0].w, r.v[1].x, r.v[1].y, r.v[1].z, r.v[1].w};
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            o[2 * a] = IOE::to_f32((u16)(w[a] & 0xffffu));
            o[2 * a + 1] = IOE::to_f32((u16)(w[a] >> 16));
        }
    }
    // four consecutive elements, 8-byte aligned
    static __device__ __forceinline__ floatx4 load4(const elem *p) {
        float o[4];
        unpack4<IOE>(*reinterpret_cast<const uint2 *>(p), o);
        return floatx4{o[0], o[1], o[2], o[3]};
    }
    static __device__ __forceinline__ void store4(elem *p, const floatx4 &v) { *reinterpret_cast<uint2 *>(p) = packq<IOE>(v[0], v[1], v[2], v[3]); }
};

// An operand of a 16-deep (Sp2) or 32-deep (Sp4) contraction as bf16 head and remainder.  SP = false (the
// caller asked for T2FW_FLAG_BF16_OPERANDS): the head alone, one MFMA per product, 2^-9 per operand.
template <bool SP> struct Sp2 {
    uint2 hi, lo;
};
template <bool SP> struct Sp4 {
    uint4 hi, lo;
};

template <bool SP> __device__ __forceinline__ Sp2<SP> split4(float a, float b, float c, float d) {
    Sp2<SP> o;
    o.hi = packq<Bf16>(a, b, c, d);
    if constexpr (SP)
        o.lo = packq<Bf16>(a - Bf16::to_f32((u16)(o.hi.x & 0xffffu)), b - Bf16::to_f32((u16)(o.hi.x >> 16)),
                           c - Bf16::to_f32((u16)(o.hi.y & 0xffffu)), d - Bf16::to_f32((u16)(o.hi.y >> 16)));
    else
        o.lo = make_uint2(0u, 0u);
    return o;
}
template <bool SP> __device__ __forceinline__ Sp2<SP> split4(const floatx4 &v) { return split4<SP>(v[0], v[1], v[2], v[3]); }
template <bool SP> __device__ __forceinline__ Sp4<SP> cat(const Sp2<SP> &a, const Sp2<SP> &b) {
    Sp4<SP> o;
    o.hi = bwd::cat(a.hi, b.hi);
    o.lo = bwd::cat(a.lo, b.lo);
    return o;
}

// c + a b with split operands (the smaller terms first); chains of one MFMA form only
template <bool SP> __device__ __forceinline__ floatx4 mma16(const Sp2<SP> &a, const Sp2<SP> &b, floatx4 c) {
    if constexpr (SP) {
        c = Bf16::mfma16(a.lo, b.hi, c);
        c = Bf16::mfma16(a.hi, b.lo, c);
    }
    return Bf16::mfma16(a.hi, b.hi, c);
}
template <bool SP> __device__ __forceinline__ floatx4 mma32(const Sp4<SP> &a, const Sp4<SP> &b, floatx4 c) {
    if constexpr (SP) {
        c = Bf16::mfma32(a.lo, b.hi, c);
        c = Bf16::mfma32(a.hi, b.lo, c);
    }
    return Bf16::mfma32(a.hi, b.hi, c);
}

// ---- tiles in LDS: a head tile followed by a remainder tile of the same shape ----------------------
// token-major [16][DTS]: channel c of a token sits at tm_pos(c), so that the sixteen channels a matrix lane
// (r, g) pairs with its accumulators (16 j + 4 g + e) are contiguous at 16 g
typedef __attribute__((address_space(3))) short4_t *lds_tr_ptr;
template <bool SP> struct TmTile {
    const u16 *hi, *lo;
    __device__ __forceinline__ TmTile(const unsigned char *base) : hi(reinterpret_cast<const u16 *>(base)), lo(reinterpret_cast<const u16 *>(base + TM_TILE)) {}
    // A / B operand "row `row`, the lane's accumulator channels", halves h = 0, 1 of the 64-deep contraction
    __device__ __forceinline__ Sp4<SP> acc_order(int row, int g, int h) const {
        Sp4<SP> o;
        o.hi = ld4(hi + row * DTS + 16 * g + 8 * h);
        o.lo = SP ? ld4(lo + row * DTS + 16 * g + 8 * h) : make_uint4(0u, 0u, 0u, 0u);
        return o;
    }
    // A / B operand "row `row`" for products of two token-major tiles (any fixed channel order)
    __device__ __forceinline__ Sp4<SP> any_order(int row, int g, int h) const {
        Sp4<SP> o;
        o.hi = ld4(hi + row * DTS + 8 * g + 32 * h);
        o.lo = SP ? ld4(lo + row * DTS + 8 * g + 32 * h) : make_uint4(0u, 0u, 0u, 0u);
        return o;
    }
    // A operand "channel 16 j + r, tokens 4 g .. 4 g + 3" for lane (r, g): a column of the tile, through the
    // transposing LDS read (lane r of a 16-lane group fetches the 8 bytes of token 4 g + r / 4 that hold channels
    // 16 j + 4 (r % 4) .. + 3; the hardware hands lane r the four tokens of channel 16 j + r)
    __device__ __forceinline__ Sp2<SP> column(int j, int r, int g) const {
        const int o = (4 * g + (r >> 2)) * DTS + 16 * (r & 3) + 4 * j;
        Sp2<SP> v;
        v.hi = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(hi + o)));
        v.lo = SP ? __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(lo + o))) : make_uint2(0u, 0u);
        return v;
    }
};
// channel-major [64][DCS]: A operand "channel `ch`, tokens 4 g .. 4 g + 3"
template <bool SP> struct CmTile {
    const u16 *hi, *lo;
    __device__ __forceinline__ CmTile(const unsigned char *base) : hi(reinterpret_cast<const u16 *>(base)), lo(reinterpret_cast<const u16 *>(base + CM_TILE)) {}
    __device__ __forceinline__ Sp2<SP> tokens(int ch, int g) const {
        Sp2<SP> o;
        o.hi = ld2(hi + ch * DCS + 4 * g);
        o.lo = SP ? ld2(lo + ch * DCS + 4 * g) : make_uint2(0u, 0u);
        return o;
    }
};
// Four result tiles [channel 16 j + 4 g + e][token r] (j = 0 .. 3) of a lane are the sixteen channels that
// tm_pos puts at 16 g of token row r: stored as head and remainder of a token-major tile
template <bool SP> __device__ __forceinline__ void store_tm_from_acc(unsigned char *tile, int r, int g, const floatx4 (&v)[4]) {
    u16 *hi = reinterpret_cast<u16 *>(tile), *lo = reinterpret_cast<u16 *>(tile + TM_TILE);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const Sp2<SP> s = split4<SP>(v[j]);
        *reinterpret_cast<uint2 *>(hi + r * DTS + 16 * g + 4 * j) = s.hi;
        if constexpr (SP) *reinterpret_cast<uint2 *>(lo + r * DTS + 16 * g + 4 * j) = s.lo;
    }
}

// a 16 x 16 matrix in the accumulator layout (lane (r, g): rows 4 g + e of column r), packed: read back by
// the same lane it is at once the B operand "X" and the A operand "X transposed" of a 16-deep product
template <bool SP> __device__ __forceinline__ void st_store(unsigned char *tile, int lane, const Sp2<SP> &v) {
    reinterpret_cast<uint2 *>(tile)[lane] = v.hi;
    if constexpr (SP) reinterpret_cast<uint2 *>(tile + ST_TILE)[lane] = v.lo;
}
template <bool SP> __device__ __forceinline__ Sp2<SP> st_load(const unsigned char *tile, int lane) {
    Sp2<SP> o;
    o.hi = reinterpret_cast<const uint2 *>(tile)[lane];
    o.lo = SP ? reinterpret_cast<const uint2 *>(tile + ST_TILE)[lane] : make_uint2(0u, 0u);
    return o;
}

// ---- the state-independent 16 x 16 algebra of a block ------------------------------------------------
// In the accumulator layout lane (r, g) holds rows 4 g + e of column r.  From the symmetric K K^T (`kk`) both
// triangles: acc(A) (column < row) and acc(A^T) (row < column).  A matrix held in the accumulator layout is the
// B operand "X" and the A operand "X^T" of a 16-deep product, so acc(X Y) = mfma(acc(X^T), acc(Y)) without any
// data movement; squaring X and X^T side by side gives the powers 2, 4, 8 of A and of A^T, then
//   P1 = (I + A^4)(I + A^8) = I + A^4 + A^8 + A^12,   P2^T = ((I - A)(I + A^2))^T = I - A^T + (A^2)^T - (A^3)^T,
//   Tm = P2 P1:   acc(Tm^T) = mfma(acc(P1), acc(P2^T)),   acc(Tm) = mfma(acc(P2^T), acc(P1)).
template <bool SP> struct BlockInverse {
    Sp2<SP> p1, p2t;
    __device__ __forceinline__ BlockInverse(const floatx4 &kk, int r, int g) {
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
        floatx4 a, at, eye;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 4 * g + e;
            a[e] = r < row ? kk[e] : 0.f;
            at[e] = row < r ? kk[e] : 0.f;
            eye[e] = row == r ? 1.f : 0.f;
        }
        const Sp2<SP> x1 = split4<SP>(a), x1t = split4<SP>(at);
        const floatx4 a2 = mma16(x1t, x1, zero), a2t = mma16(x1, x1t, zero);
        const Sp2<SP> x2 = split4<SP>(a2), x2t = split4<SP>(a2t);
        const floatx4 a3t = mma16(x1, x2t, zero);                       // (A^3)^T = A^T (A^2)^T
        const floatx4 a4 = mma16(x2t, x2, zero), a4t = mma16(x2, x2t, zero);
        const Sp2<SP> x4 = split4<SP>(a4), x4t = split4<SP>(a4t);
        const floatx4 a8 = mma16(x4t, x4, zero);
        const floatx4 a12 = mma16(x4t, split4<SP>(a8), zero);               // A^12 = A^4 A^8
        p1 = split4<SP>(eye + a4 + a8 + a12);
        p2t = split4<SP>(eye - at + a2t - a3t);
    }
    __device__ __forceinline__ floatx4 acc_tm_transposed() const { return mma16(p1, p2t, floatx4{0.f, 0.f, 0.f, 0.f}); }
    __device__ __forceinline__ floatx4 acc_tm() const { return mma16(p2t, p1, floatx4{0.f, 0.f, 0.f, 0.f}); }
};

// ---- staging of a [T, 64] array into tiles (one wave per array) ---------------------------------------
// sixteen elements of one lane: token lane >> 2, channels 16 (lane & 3) .. + 15.  Rows at or past T read as zero.
// Loads are issued unconditionally (rows at or past T are read from row T - 1 and zeroed when the tile is
// built): a load inside a branch would make every later wait for a load a wait for all of them.
template <typename E> __device__ __forceinline__ typename E::Raw16 load_tm(const typename E::elem *row0, int tok0, int T, int lane) {
    const int t = min(tok0 + (lane >> 2), T - 1);
    return E::load16(row0 + (size_t)t * CH_N + 16 * (lane & 3));
}
template <bool SP, typename E> __device__ __forceinline__ void store_tm(unsigned char *tile, int lane, const typename E::Raw16 &r, int tok0, int T, float sign = 1.f) {
    u16 *hi = reinterpret_cast<u16 *>(tile), *lo = reinterpret_cast<u16 *>(tile + TM_TILE);
    const int o = (lane >> 2) * DTS + 4 * (lane & 3);
    const float keep = tok0 + (lane >> 2) < T ? sign : 0.f;
    float v[16];
    E::floats(r, v);
#pragma unroll
    for (int a = 0; a < 4; ++a) {          // channels 16 q + 4 a + e sit at 16 a + 4 q + e
        const Sp2<SP> s = split4<SP>(v[4 * a] * keep, v[4 * a + 1] * keep, v[4 * a + 2] * keep, v[4 * a + 3] * keep);
        *reinterpret_cast<uint2 *>(hi + o + 16 * a) = s.hi;
        if constexpr (SP) *reinterpret_cast<uint2 *>(lo + o + 16 * a) = s.lo;
    }
}

// ---- staging pipeline shared by the backward kernels ---------------------------------------------------
// LDS as rings of stages: raw tiles live three stages (built two stages ahead of the slab waves, read by the
// matrix waves one stage ahead and by the slab waves), the matrix waves' results two.
template <int RAW_BLOCK, int ST_BLOCK, int NBLK> struct Ring {
    static constexpr int ST = 3 * NBLK * RAW_BLOCK;
    static constexpr int SMEM = ST + 2 * NBLK * ST_BLOCK;
    static __device__ __forceinline__ unsigned char *raw(unsigned char *smem, int stage, int bb) {
        return smem + ((stage % 3) * NBLK + bb) * RAW_BLOCK;
    }
    static __device__ __forceinline__ unsigned char *st(unsigned char *smem, int stage, int bb) {
        return smem + ST + ((stage & 1) * NBLK + bb) * ST_BLOCK;
    }
};

// One wave stages NJOBS arrays for every stage, two stages ahead of the slab waves.  An array is loaded once,
// token-major (four 16-byte loads per lane and block for fp32 tensors, two for 16-bit ones), and written as a token-major tile; where a channel-major
// tile of the same array is wanted too, the wave reads its own token-major tile back with the transposing LDS
// read and writes that (the loads of a second layout were what the wave waited for: a wave can have 63 memory
// instructions outstanding, and a channel-major tile loaded directly is sixteen 4-byte loads per lane).
// Loads are unconditional and issued SETS - 1 stages before their tiles are built, into the register set that the
// stage before has left (SETS sets in turn; the stage loop is unrolled SETS times so that no register copy waits
// for a load).  tok0_of(stage, bb): first token of a block (at or past T: a block of zeros).
template <typename E> struct PrepJob {
    const typename E::elem *src;       // token 0 of the batch row
    int tm_off;             // byte offset of the token-major tile inside a block's raw tiles; < 0: the wave's scratch tile
    int cm_off;             // byte offset of the channel-major tile; < 0: none
    float sign;             // the token-major tile holds sign * src
    bool cm_negated;        // the channel-major tile holds the negative of the token-major one
};
template <typename RING, int NBLK, int NJOBS, bool SP, int SETS, typename E, typename TOK0>
__device__ __forceinline__ void prep_wave_jobs(unsigned char *smem, const PrepJob<E> (&jobs)[NJOBS], int T, int nstages, int lane,
                                               TOK0 tok0_of, unsigned char *scratch_tile) {
    static_assert(SETS == 2 || SETS == 3, "two or three register sets");
    const int r = lane & 15, g = lane >> 4;
    typedef typename E::Raw16 Raw16;
    Raw16 set_a[NJOBS][NBLK], set_b[NJOBS][NBLK], set_c[SETS == 3 ? NJOBS : 1][SETS == 3 ? NBLK : 1];
    auto load = [&](auto &regs, int stage) {
#pragma unroll
        for (int a = 0; a < NJOBS; ++a)
#pragma unroll
            for (int bb = 0; bb < NBLK; ++bb) regs[a][bb] = load_tm<E>(jobs[a].src, tok0_of(stage, bb), T, lane);
    };
    // stage `stage` out of `cur`; the loads of stage + SETS - 1 into `far` (the set that stage - 1 has left)
    auto stage_body = [&](int stage, auto &cur, auto &far) {
        load(far, min(stage + SETS - 1, nstages - 1));
#pragma unroll
        for (int a = 0; a < NJOBS; ++a)
#pragma unroll
            for (int bb = 0; bb < NBLK; ++bb) {
                unsigned char *const raw = RING::raw(smem, stage, bb);
                unsigned char *const tm = jobs[a].tm_off >= 0 ? raw + jobs[a].tm_off : scratch_tile;
                store_tm<SP, E>(tm, lane, cur[a][bb], tok0_of(stage, bb), T, jobs[a].sign);
                if (jobs[a].cm_off >= 0) {
                    // DS operations of one wave execute in order: the reads below see the tile just written
                    const TmTile<SP> own(tm);
                    u16 *const hi = reinterpret_cast<u16 *>(raw + jobs[a].cm_off), *const lo = reinterpret_cast<u16 *>(raw + jobs[a].cm_off + CM_TILE);
                    const u32 flip = jobs[a].cm_negated ? 0x80008000u : 0u;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const Sp2<SP> col = own.column(j, r, g);          // channel 16 j + r, tokens 4 g .. 4 g + 3
                        const int o = (16 * j + r) * DCS + 4 * g;
                        *reinterpret_cast<uint2 *>(hi + o) = make_uint2(col.hi.x ^ flip, col.hi.y ^ flip);
                        if constexpr (SP) *reinterpret_cast<uint2 *>(lo + o) = make_uint2(col.lo.x ^ flip, col.lo.y ^ flip);
                    }
                }
            }
        __syncthreads();
    };
    load(set_a, 0);
    int stage = 0;
    if constexpr (SETS == 3) {
        load(set_b, min(1, nstages - 1));
        for (; stage + 3 <= nstages; stage += 3) {
            stage_body(stage, set_a, set_c);
            stage_body(stage + 1, set_b, set_a);
            stage_body(stage + 2, set_c, set_b);
        }
        if (stage < nstages) stage_body(stage, set_a, set_c);
        if (stage + 1 < nstages) stage_body(stage + 1, set_b, set_a);
    } else {
        for (; stage + 2 <= nstages; stage += 2) {
            stage_body(stage, set_a, set_b);
            stage_body(stage + 1, set_b, set_a);
        }
        if (stage < nstages) stage_body(stage, set_a, set_b);
    }
    __syncthreads();        // the two ticks in which the other waves finish
    __syncthreads();
}

}  // namespace dfwc
#endif  // __HIPCC__

}  // namespace t2fw
