// Chunk-parallel matrix-core form of the decay-rule recurrence for D = K = 64, 16-bit tensors.
//
// A chunk is the CL = 32 or 64 steps between two checkpoints.  With prefix products taken from the
// chunk start, a_t[d] = prod_{r<=t} f_r[d], b_t[k] = prod_{r<=t} fkey_r[k], and
//   qs_t = q_t*b_t   kt_t = k_t/b_t   xt_t = x_t/a_t   gs_t = g_t*a_t
// everything inside a chunk is a dense contraction of those four [CL, 64] tiles with each other,
// with the chunk-start state S0 (the checkpoint) and with the adjoint entering the chunk from the
// future (lfw_par_bwd.hip).  Only the chunk-to-chunk hand-over of the adjoint is sequential; its
// per-chunk increments are a light pass of their own that reads four of the inputs, the hand-over
// itself is elementwise, and the rest runs as one workgroup per (batch row, chunk) over the whole grid.
//
// Range: the scalings are taken relative to the MIDDLE of the chunk (a'_t = a_t / a_mid, likewise
// b'), so that 1/a'_t and a'_t each grow over half a chunk only: the form needs the gate products of
// both halves of every chunk to stay above PAR_MIN_PRODUCT (operands are bf16, which has the exponent
// range of fp32) and gates in (0, 1].  Rows that violate this are flagged and redone with the exact
// scan.  The state and the adjoint enter the products scaled to the same reference:
// S0' = (a_mid (x) b_mid) * S0 and Gh' = (a_CL/a_mid (x) b_CL/b_mid) * Ge, all factors <= 1.  These two
// carry the half-chunk products of BOTH sides, down to PAR_MIN_PRODUCT^2 = 2^-160, which no 32-bit
// exponent holds, while what they are multiplied with carries the inverse of one side's product: they
// are stored times PAR_STATE_SHIFT, and the contractions with them are multiplied by PAR_STATE_UNSHIFT
// before anything else is added.
//
// Lane layout ("C layout"): a workgroup has 8 waves = (side, channel block cb); side 0 owns the value
// side (x, f, g_out), side 1 the key side (k, f_key, q).  Lane (i = lane & 15, kg = lane >> 4) of
// wave (side, cb) owns channel 16 cb + i of its side and the tokens 16 m + 4 kg + j (m < CL / 16,
// j < 4) of the chunk.  That is the layout in which an MFMA returns a 16 x 16 result tile with rows
// = tokens and columns = channels (lane holds rows 4 kg + j of column i), and in which a lane's four
// consecutive tokens of a tile are one B operand of a 16-deep contraction over tokens: scaled
// operands of the own side go from registers straight into the matrix cores, and every per-element
// factor (prefix products, their inverses) stays in the lane that needs it for the output scaling.
// The other side's tiles are read from LDS, where they are stored channel-major [64][CMS], through
// the transposing LDS read of gfx950 (ds_read_b64_tr_b16), which hands lane i the four consecutive
// channels of token i that an A operand needs.
#pragma once

#include "lfw_chunk.hpp"
#include "lfw_chunk_bwd_dev.hpp"

namespace t2fw {

// Backward, three launches: the adjoint's per-chunk increments sum_t gs_t (x) qs_t and gate products
// (one workgroup per (row, chunk)); their scan over the chunks of a row, last to first, which leaves
// the adjoint entering every chunk (Gh', bf16) in place of the increments and writes d_s0 (elementwise,
// eight workgroups per row); and the gradients (one workgroup per (row, chunk)).
constexpr int PAR_NVEC = 6;            // per (row, chunk): totA, totB, refA, refB, sfxA, sfxB, [64] floats each
struct ParBwdArgs {
    const void *g_out, *g_state, *x, *f, *q, *k, *f_key, *ckpt;
    void *d_x, *d_f, *d_q, *d_k, *d_f_key, *d_s0;
    void *gh;                          // scratch [B, NC, 64, 64] bf16: adjoint increments, then Gh'
    float *vecs;                       // scratch [B, NC, PAR_NVEC, 64]
    int32_t *chunk_flags;              // scratch [B * NC]: 1 for chunks this form cannot take
    int32_t *row_flags;                // [B]: 1 for rows with such a chunk (their results are not valid)
    int64_t B, T, NC;
    int32_t C;                         // checkpoint interval = chunk length: 32 or 64
    int32_t heads;                     // as in ChunkFwdArgs
};

int par_backward(const ParBwdArgs &a, int dtype, hipStream_t stream);

#if defined(__HIPCC__)
namespace par {

using namespace bwd;

constexpr int PAR_THREADS = 512;
constexpr int CMS = 72;                          // row stride (elements) of channel-major tiles [64][CMS]
constexpr int CM_BYTES = CH_N * CMS * 2;
// smallest chunk gate product this form accepts: 1 / product scales operands that are then
// multiplied by values and summed in fp32, which has to stay far below 2^128
constexpr float PAR_MIN_PRODUCT = 8.271806125530277e-25f;     // 2^-80
// S0' and Gh' are stored times 2^44: an element of magnitude 2^-10 under two half-chunk products of 2^-80
// is still a normal bf16 number (2^-126), and the one contraction of S0' with Gh' (both shifted, 64
// terms) stays finite up to |S0| |Ge| = 2^34, beyond what two fp16 tensors can hold.  The factor goes
// onto one side's product before the other side's is multiplied in, so that no intermediate leaves
// the range either.
constexpr float PAR_STATE_SHIFT = 17592186044416.0f;          // 2^44
constexpr float PAR_STATE_UNSHIFT = 5.684341886080802e-14f;   // 2^-44

typedef __attribute__((address_space(3))) short4_t *lds_short4_ptr;

// Transposing LDS read: the 16 lanes of a row group read rows row0 .. row0 + 3, columns
// col0 .. col0 + 15 of a 16-bit matrix with `stride` elements per row; lane i returns the four
// elements (row0 .. row0 + 3, col0 + i).  (Lane i fetches 8 bytes of row row0 + i / 4 at column
// col0 + 4 (i % 4); the hardware redistributes them.)
__device__ __forceinline__ uint2 lds_tr4(const u16 *m, int row0, int col0, int stride, int i) {
    const u16 *p = m + (row0 + (i >> 2)) * stride + col0 + 4 * (i & 3);
    const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(p));
    return __builtin_bit_cast(uint2, v);
}

// Contraction over the 64 channels of a side runs as two MFMAs of depth 32 (h = 0, 1); lane kg
// supplies, as element e of its eight, channel 32 h + 16 (e / 4) + 4 kg + e % 4.  Any assignment
// works as long as both operands use the same one; this one lets both halves of an operand come
// from one aligned 8-byte read each.
//
// Operand "rows of a token tile": lane i = token tok0 + i of a channel-major tile, channels as above.
__device__ __forceinline__ uint4 tok_rows_op(const u16 *tile, int tok0, int h, int i, int kg) {
    return cat(lds_tr4(tile, 32 * h + 4 * kg, tok0, CMS, i), lds_tr4(tile, 32 * h + 16 + 4 * kg, tok0, CMS, i));
}
// Operand "row of a [64][CMS] matrix": lane i = row row0 + i, columns = channels as above
__device__ __forceinline__ uint4 mat_rows_op(const u16 *mat, int row0, int h, int i, int kg) {
    const u16 *p = mat + (row0 + i) * CMS + 32 * h + 4 * kg;
    return cat(ld2(p), ld2(p + 16));
}
// Operand "column of a [64][CMS] matrix": lane i = column col0 + i, rows = channels as above
__device__ __forceinline__ uint4 mat_cols_op(const u16 *mat, int col0, int h, int i, int kg) {
    return cat(lds_tr4(mat, 32 * h + 4 * kg, col0, CMS, i), lds_tr4(mat, 32 * h + 16 + 4 * kg, col0, CMS, i));
}

// ---- cross-row scans over the four 16-lane rows of a wave (lane-swap instructions, no LDS) -------
struct RowScan {
    float lower;    // combination of the rows below this lane's row (identity for row 0)
    float all;      // combination of the four rows
};
__device__ __forceinline__ RowScan row_scan_mul(float v, int kg) {
    const u32 vb = __float_as_uint(v);
    const auto s16 = __builtin_amdgcn_permlane16_swap(vb, vb, false, false);     // {even row of the pair, odd row}
    const float ev = __uint_as_float(s16[0]);
    const float pair = ev * __uint_as_float(s16[1]);
    const u32 pb = __float_as_uint(pair);
    const auto s32 = __builtin_amdgcn_permlane32_swap(pb, pb, false, false);     // {rows 0-1, rows 2-3}
    const float lo = __uint_as_float(s32[0]);
    RowScan r;
    r.all = lo * __uint_as_float(s32[1]);
    r.lower = ((kg & 1) ? ev : 1.0f) * ((kg & 2) ? lo : 1.0f);
    return r;
}
__device__ __forceinline__ RowScan row_scan_add(float v, int kg) {
    const u32 vb = __float_as_uint(v);
    const auto s16 = __builtin_amdgcn_permlane16_swap(vb, vb, false, false);
    const float ev = __uint_as_float(s16[0]);
    const float pair = ev + __uint_as_float(s16[1]);
    const u32 pb = __float_as_uint(pair);
    const auto s32 = __builtin_amdgcn_permlane32_swap(pb, pb, false, false);
    const float lo = __uint_as_float(s32[0]);
    RowScan r;
    r.all = lo + __uint_as_float(s32[1]);
    r.lower = ((kg & 1) ? ev : 0.0f) + ((kg & 2) ? lo : 0.0f);
    return r;
}

// ---- one lane's share of a chunk of one side ------------------------------------------------------
// NT = CL / 16 token tiles; element [m][j] is token 16 m + 4 kg + j of the chunk.
template <int NT> struct LaneChunk {
    float pre[NT][4];     // gate products from the origin up to and including the token
    float off[NT];        // gate product up to the token before [m][0]
    float tot;            // the whole chunk's gate product (the same in every lane of the channel)
    float ref;            // the product of the first half of the chunk (tokens 0 .. CL / 2 - 1)
    float sfx;            // the product of the second half
    u32 bad;              // a gate outside (0, 1] or a half-chunk product below PAR_MIN_PRODUCT
};

// Raw 16-bit loads of one array: this lane's NT * 4 tokens of channel c, two tokens per register
// (the loads write the low and the high half of a register directly).  ubase: the array at the
// chunk's first token, channel 0 (the same for the whole workgroup, so that a token's address is a
// scalar base plus the lane's fixed offset, whatever the token stride); lane_off = 4 kg * ts + c; ts:
// elements between consecutive tokens; n_left: tokens from the lane's first token to the end of the
// sequence (tokens at or past the end are read from the last one).
typedef unsigned short us2 __attribute__((ext_vector_type(2)));
template <int NT> struct RawTokens {
    us2 p[NT][2];
    __device__ __forceinline__ u16 at(int m, int j) const { return (j & 1) ? p[m][j >> 1].y : p[m][j >> 1].x; }
};

// a value that is the same in every lane, moved to scalar registers (the compiler computes 64-bit
// divisions in vector registers and would otherwise keep what is derived from them there)
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
    const u32 lo = __builtin_amdgcn_readfirstlane((u32)(unsigned long long)v);
    const u32 hi = __builtin_amdgcn_readfirstlane((u32)((unsigned long long)v >> 32));
    return (int64_t)(((unsigned long long)hi << 32) | lo);
}

template <int NT, bool FULL>
__device__ __forceinline__ void load_tokens(RawTokens<NT> &r, const u16 *ubase, u32 lane_off, u32 ts, int n_left) {
#pragma unroll
    for (int m = 0; m < NT; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u16 v;
            if (FULL) {
                const u16 *const tok = ubase + (size_t)(16 * m + j) * ts;      // wave-uniform
                v = tok[lane_off];
            } else {
                const int o = min(16 * m + j, n_left - 1);
                v = ubase[lane_off + (u32)o * ts];
            }
            if (j & 1)
                r.p[m][j >> 1].y = v;
            else
                r.p[m][j >> 1].x = v;
        }
}

// Gates -> prefix products (and the range verdict).  FULL = false: tokens at or past n_left act as
// identity (gate 1).
//
// Origin of pre and off: the chunk start (MID = false), or the middle of the chunk (MID = true), that
// is pre = a_t / a_mid, from 1 / ref down to 1 over the first half and from 1 down to sfx over the
// second.  The second half's products are then built from 1 at the middle, not from the chunk start and
// divided: the product of both halves may lie far below the smallest fp32 number while each half is in
// range.
//
// Gates below 2^-12 (an exactly zero gate above all, which an fp16 sigmoid returns below a logit of
// about -17) enter as 2^-12.  The forward's state after such a step holds at most 2^-24 of what was there
// before it; here 2^-12 of it leaks through, 2.4e-4 of a term that the operands' bf16 rounding already
// perturbs by 2^-9.  The floor is this high for the gate gradient of that very step: gate * d_gate is
// what the sweeps produce (lfw_par_bwd.hip), with an absolute error of fp32 rounding (2^-24) of the
// terms that cancel in it, and d_gate = that / gate with the floored gate is then good to 2^-12 of those
// terms.  (d_gate at a step does not depend on the step's own gate, so the floored gate gives the right
// value.)
template <typename IOE, int NT, bool FULL, bool MID>
__device__ __forceinline__ void gate_scan(LaneChunk<NT> &lc, float (&gate)[NT][4], const RawTokens<NT> &raw, int kg,
                                          int n_left) {
    us2 mx = {0, 0};
    const us2 floor_bits = {IOE::BWD_FLOOR_BITS, IOE::BWD_FLOOR_BITS};
#pragma unroll
    for (int m = 0; m < NT; ++m)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            us2 bits = raw.p[m][jj];
            if (!FULL) {
                if (!(16 * m + 2 * jj < n_left)) bits.x = IOE::ONE_BITS;
                if (!(16 * m + 2 * jj + 1 < n_left)) bits.y = IOE::ONE_BITS;
            }
            mx = __builtin_elementwise_max(mx, bits);      // > bits(1.0): above one, negative, NaN
            bits = __builtin_elementwise_max(bits, floor_bits);      // gates in [0, 2^-12) count as 2^-12
            gate[m][2 * jj] = IOE::to_f32(bits.x);
            gate[m][2 * jj + 1] = IOE::to_f32(bits.y);
        }
    float carry = 1.0f, second = 1.0f;
#pragma unroll
    for (int m = 0; m < NT; ++m) {
        float l[4];
        l[0] = gate[m][0];
#pragma unroll
        for (int j = 1; j < 4; ++j) l[j] = l[j - 1] * gate[m][j];
        const RowScan s = row_scan_mul(l[3], kg);
        lc.off[m] = carry * s.lower;
        carry *= s.all;
        if (m == NT / 2 - 1) {
            lc.ref = carry;
            if (MID) carry = 1.0f;
        }
        if (m >= NT / 2) second *= s.all;
#pragma unroll
        for (int j = 0; j < 4; ++j) lc.pre[m][j] = lc.off[m] * l[j];
    }
    lc.tot = MID ? lc.ref * second : carry;
    lc.sfx = second;
    if (MID) {
        const float r = __builtin_amdgcn_rcpf(lc.ref);
#pragma unroll
        for (int m = 0; m < NT / 2; ++m) {
            lc.off[m] *= r;
#pragma unroll
            for (int j = 0; j < 4; ++j) lc.pre[m][j] *= r;
        }
    }
    const u16 hi = mx.x > mx.y ? mx.x : mx.y;
    lc.bad = (hi > IOE::ONE_BITS || !(lc.ref >= PAR_MIN_PRODUCT) || !(second >= PAR_MIN_PRODUCT)) ? 1u : 0u;
}

// 1 / pre: one reciprocal per run of four tokens, the others by multiplying the gates back in
template <int NT>
__device__ __forceinline__ void inverse_products(float (&inv)[NT][4], const LaneChunk<NT> &lc, const float (&gate)[NT][4]) {
#pragma unroll
    for (int m = 0; m < NT; ++m) {
        inv[m][3] = __builtin_amdgcn_rcpf(lc.pre[m][3]);
#pragma unroll
        for (int j = 2; j >= 0; --j) inv[m][j] = inv[m][j + 1] * gate[m][j + 1];
    }
}

template <typename IOE, int NT, bool FULL>
__device__ __forceinline__ void to_floats(float (&v)[NT][4], const RawTokens<NT> &raw, int n_left) {
#pragma unroll
    for (int m = 0; m < NT; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) v[m][j] = (FULL || 16 * m + j < n_left) ? IOE::to_f32(raw.at(m, j)) : 0.0f;
}

// v * s for the lane's tokens, packed to bf16 pairs: [m] is one B operand (four consecutive tokens)
template <int NT>
__device__ __forceinline__ void scale_pack(uint2 (&p)[NT], const float (&v)[NT][4], const float (&s)[NT][4]) {
#pragma unroll
    for (int m = 0; m < NT; ++m)
        p[m] = packq<Bf16>(v[m][0] * s[m][0], v[m][1] * s[m][1], v[m][2] * s[m][2], v[m][3] * s[m][3]);
}

// the lane's packed tokens -> its channel's row of a channel-major tile
template <int NT> __device__ __forceinline__ void store_cm(u16 *tile, int c, int kg, const uint2 (&p)[NT]) {
#pragma unroll
    for (int m = 0; m < NT; ++m) *reinterpret_cast<uint2 *>(tile + c * CMS + 16 * m + 4 * kg) = p[m];
}

// MFMA result tile (rows 4 kg + j, column i) -> 16-bit A/B operand of a 16-deep contraction over its
// rows, keeping rows < column (LOWER: strictly below the diagonal of the transposed tile, i.e.
// row index < column index) or rows > column, or everything
enum { KEEP_ALL = 0, KEEP_ROW_LT_COL = 1, KEEP_ROW_GT_COL = 2 };
template <int KEEP> __device__ __forceinline__ uint2 mask_pack(const floatx4 &t, int i, int kg) {
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = 4 * kg + j;
        const bool keep = KEEP == KEEP_ALL || (KEEP == KEEP_ROW_LT_COL ? row < i : row > i);
        v[j] = keep ? t[j] : 0.0f;
    }
    return packq<Bf16>(v[0], v[1], v[2], v[3]);
}

// diagonal of a 16 x 16 result tile, redistributed: lane (i, kg) receives elements (4 kg + j, 4 kg + j)
__device__ __forceinline__ void tile_diagonal(float (&d)[4], const floatx4 &t, int kg) {
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = __shfl(t[j], 20 * kg + j, 64);
}

// Operand tiles are re-read from LDS where they are used; without this the compiler merges the
// reads of a whole sweep and keeps all of them in registers.
__device__ __forceinline__ void lds_fence() { asm volatile("" ::: "memory"); }

}  // namespace par
#endif  // __HIPCC__

}  // namespace t2fw
