// Chunked (matrix-core) form of the decay-rule recurrence for D = K = 64, 16-bit I/O.
//
// The rank-1-separable gate lets a block of L = 16 steps be written as small dense
// contractions.  With a_t[d] = prod_{r<=t} f_r[d], b_t[k] = prod_{r<=t} fkey_r[k] (products
// from the block start), suffix products ca_t = a_L/a_t, cb_t = b_L/b_t and
//   qs_t = q_t*b_t,  kh_t = k_t*cb_t,  kt_t = kh_t/b_L (= k_t/b_t),
//   xh_t = x_t*ca_t, xt_t = xh_t/a_L (= x_t/a_t),  gs_t = g_t*a_t
// the block is
//   P[t,s]  = qs_t . kt_s                       (t >= s)
//   o_t     = a_t * ( S0 qs_t + sum_{s<=t} P[t,s] xt_s )
//   S_L     = (a_L (x) b_L) * S0 + sum_s xh_s (x) kh_s
// Only the intra-block terms use an inverse (1/b_L, 1/a_L over 16 steps); everything that
// crosses block boundaries is scaled by factors <= 1, so the form holds for any gates in
// (0, 1] whose 16-step products stay above 2^-100.  Rows that violate this (or have gates
// outside (0, 1]) are flagged and recomputed with the exact scan: by the forward kernel itself,
// per workgroup (a whole row, or the 32 value channels a workgroup of the split launch owns:
// value channels are independent recurrences, so the other 32 keep their chunked results unless
// their own or the key-side gates are flagged too), and by a launch of the exact backward kernel
// after the chunked backward.
//
// All contractions run on MFMA with 16-bit operands (type OP) and fp32 accumulation; the
// state itself is carried in fp32 accumulator registers for the whole sequence.
#pragma once

#include "common.hpp"

namespace t2fw {

struct ChunkFwdArgs {
    const void *x, *f, *q, *k, *f_key, *s0;
    void *out, *next_state, *ckpt;     // ckpt may be null
    int32_t *row_flags;                // [2 * chunk_rows_padded(B)]: set to 1 for rows the chunked form cannot take
    int32_t *par_hint;                 // same shape, may be null: set to 1 for rows the chunk-parallel backward may decline
                                       // (a 16-step gate product below PAR_HINT_MIN_PRODUCT, or what row_flags reports)
    int64_t B, T, NC;
    int32_t C;                         // checkpoint interval, multiple of 32
    int32_t heads;                     // 1: rows are [T, 64] slabs; H > 1: row b is head b % H of a [B / H, T, H, 64] tensor
    // rows the chunked form cannot take are redone in place with the exact scan (0: only reported);
    // launch geometry of that scan for a 64 x 64 state (set by chunk_forward)
    int32_t redo, scan_kg, scan_tb, scan_ntiles;
};

struct ChunkBwdArgs {
    const void *g_out, *g_state, *x, *f, *q, *k, *f_key, *ckpt;
    void *d_x, *d_f, *d_q, *d_k, *d_f_key, *d_s0;
    int32_t *row_flags;                // as for the forward
    const int32_t *row_select;         // null: every row; else only rows b with row_select[b] != 0 (the others report "not flagged")
    int64_t B, T, NC;
    int32_t C;
    int32_t redo;                      // nonzero: a workgroup whose row the chunked form cannot take redoes its side
                                       // of that row with the exact scan, inside the kernel
    int32_t scan_kg, scan_ntiles;      // geometry of the exact scan body for a 64 x 64 state (set by the launcher)
    int32_t heads;                     // as for the forward (inputs, g_out and the five [.., T, .., 64] gradients)
};

// Kernels that split a batch row over two workgroups index them as half * chunk_rows_padded(B) + row
// and use two flag slots per row, row_flags[row] and row_flags[chunk_rows_padded(B) + row].
__host__ __device__ inline int64_t chunk_rows_padded(int64_t B) { return (B + 7) / 8 * 8; }

// op: 0 = bf16 operands, 1 = fp16 operands (fp16 I/O only); split: two workgroups per batch row
int chunk_forward(const ChunkFwdArgs &a, int dtype, int op, bool split, hipStream_t stream);
// two workgroups per batch row (one per side of the state)
int chunk_backward(const ChunkBwdArgs &a, int dtype, int op, hipStream_t stream);
constexpr int64_t CHUNK_MAX_T = 1 << 24;      // the kernels address a batch row with 32-bit offsets: T * heads must stay below this

#if defined(__HIPCC__)

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef unsigned short u16;
typedef unsigned int u32;

// MFMA chaining rule used by the kernels: an accumulator is only ever chained (result fed back
// as the C operand) through MFMAs of the SAME form.  The result of a 16x16x32 chain and the
// result of a 16x16x16 product are combined with VALU adds, never by feeding one form's
// result straight into the other form's C operand: with only three instructions between a
// 16x16x32 and a dependent 16x16x16 the latter was observed to read a partly written C on
// gfx950 (two of the four result elements wrong); VALU reads of MFMA results are interlocked
// by the compiler's wait states.
// 16-bit element types as raw bits + conversions ---------------------------------------
// A row none of whose 16-step gate products is below this is inside the chunk-parallel backward's range
// (products over half a chunk, i.e. one or two blocks, at or above 2^-80).
constexpr float PAR_HINT_MIN_PRODUCT = 9.094947017729282e-13f;      // 2^-40

struct Bf16 {
    using io_type = __hip_bfloat16;      // the same tensor element as the exact kernels see it
    static constexpr u16 ONE_BITS = 0x3F80;
    static constexpr u16 FLOOR_BITS = 0x3380;        // 2^-24: gates enter the forward's products no smaller
    static constexpr u16 BWD_FLOOR_BITS = 0x3980;    // 2^-12: ... and the chunk-parallel backward's
    // As the tensors' type: results of size 2^28 and more are representable, which is where an intermediate of the
    // matrix-core forms (the result times up to 1 / product) can leave fp32: the kernels then look at what they
    // store and hand rows with an inf or NaN to the exact recurrence.  With fp16 tensors such a result is beyond
    // the type anyway, and no operand can overflow (values up to 2^16, 1 / product up to 2^100).
    static constexpr bool CHECK_RESULTS = true;
    // smallest 16-step gate product accepted with operands of this type: the inverse
    // 1/product scales the intra-block operands and must stay far from overflow
    static constexpr float MIN_PRODUCT = 7.8886090522101181e-31f;   // 2^-100
    static __device__ __forceinline__ float to_f32(u16 v) { return __uint_as_float((u32)v << 16); }
    // products of raw 16-bit values
    static __device__ __forceinline__ float mul(u16 a, float x) { return to_f32(a) * x; }
    static __device__ __forceinline__ float mul2(u16 a, u16 b) { return to_f32(a) * to_f32(b); }
    static __device__ __forceinline__ u32 pack2(float lo, float hi) {
        floatx2 v = {lo, hi};
        return __builtin_bit_cast(u32, __builtin_convertvector(v, bf16x2_t));
    }
    static __device__ __forceinline__ floatx4 mfma32(uint4 a, uint4 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                            __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ floatx4 mfma16(uint2 a, uint2 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a),
                                                              __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
    }
};

struct Fp16 {
    using io_type = __half;
    static constexpr u16 ONE_BITS = 0x3C00;
    static constexpr u16 FLOOR_BITS = 0x0001;        // 2^-24, the smallest positive fp16
    static constexpr u16 BWD_FLOOR_BITS = 0x0C00;    // 2^-12
    static constexpr bool CHECK_RESULTS = false;     // see Bf16
    static constexpr float MIN_PRODUCT = 0.00390625f;               // 2^-8
    static __device__ __forceinline__ float to_f32(u16 v) { return (float)__builtin_bit_cast(_Float16, v); }
    // products of raw 16-bit values (a fused form with fp16 operands converted on the fly exists,
    // v_fma_mix_f32, but measured slower here than the separate conversion it saves)
    static __device__ __forceinline__ float mul(u16 a, float x) { return to_f32(a) * x; }
    static __device__ __forceinline__ float mul2(u16 a, u16 b) { return to_f32(a) * to_f32(b); }
    static __device__ __forceinline__ u32 pack2(float lo, float hi) {
        floatx2 v = {lo, hi};
        return __builtin_bit_cast(u32, __builtin_convertvector(v, f16x2_t));
    }
    static __device__ __forceinline__ floatx4 mfma32(uint4 a, uint4 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                           __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ floatx4 mfma16(uint2 a, uint2 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a),
                                                          __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
    }
};

template <typename E> __device__ __forceinline__ u16 cvt1(float v) { return (u16)(E::pack2(v, 0.f) & 0xffffu); }

constexpr int CH_THREADS = 256;
constexpr int CH_L = 16;        // block length
constexpr int CH_STEP = 32;     // tokens prepared per iteration (two blocks)
constexpr int CH_N = 64;        // D = K = 64

// LDS strides (in elements) chosen so the MFMA operand reads are bank-conflict free
constexpr int TS = 72;          // token-major tiles [32 tokens][64 ch] of 16-bit: row stride
constexpr int CS = 36;          // channel-major tiles [64 ch][32 tokens] of 16-bit / fp32: row stride
constexpr int OS = 68;          // output tile [32 tokens][64 ch] of 16-bit: row stride

// Position of channel c = 16j + 4g + e inside the row of a token-major tile whose rows are also
// contracted against a wave's own accumulators: 16g + 4j + e.  The 16 values lane (r, g) pairs
// with its accumulator elements (channels 16j + 4g + e, j = 0..3) are then contiguous (two
// 16-byte reads).  Products between two such tiles are indifferent to the order.
__device__ __forceinline__ int tm_pos(int c) { return 16 * ((c >> 2) & 3) + 4 * (c >> 4) + (c & 3); }

#endif  // __HIPCC__

}  // namespace t2fw
