// Forward scan of the decay rule in chunked matrix-core form (see lfw_chunk.hpp for the
// algebra).  One workgroup of 12 waves owns one batch row.  Matrix wave w keeps the
// 16 x 64 slab S[16w:16w+16, :] of the state in fp32 accumulator registers for the whole
// sequence, runs the MFMA phase of a 32-token step and stores the outputs itself.  Eight
// prep waves build the scaled 16-bit operand tiles of the next step in LDS: a wave takes
// one side (key or value), one of the step's two 16-token blocks and eight of its tokens,
// a lane one channel.  Raw inputs go from global memory straight to the prep waves'
// registers (two-byte loads, coalesced over the wave's 64 channels), two steps ahead of
// their use; one workgroup barrier per step hands the double-buffered tiles over.
//
// The rows S[d, :] of the state never interact, so a batch row can also be split over two
// workgroups by value channel (d < 32 / d >= 32): each then runs two matrix waves, the whole
// key-side preparation (duplicated) and half of the value-side one.  The launcher does this
// when twice the batch still fits the CUs of the device.
//
// Replaces lfw_cuda_fwd_kernel + the output einsum of the reference
// (t2fw/csrc/lfw_kernel.cu:18-59, t2fw/csrc/lfw.cpp:45); semantics t2fw/torch.py:21-31.
#include <algorithm>
#include <type_traits>

#include "lfw_chunk.hpp"
#include "lfw_scan_body.hpp"

namespace t2fw {
namespace {

constexpr int FWD_THREADS = 768;          // one workgroup per batch row: 4 matrix + 8 prep waves
constexpr int FWD_THREADS_HALF = 512;     // two per batch row: 2 matrix + 4 key-side + 2 value-side prep waves

// ---- LDS layout of one operand buffer (bytes) -------------------------------------------
constexpr int OFF_QT = 0;                                  // qs  token-major  [32][TS] u16, channels at tm_pos
constexpr int OFF_KT = OFF_QT + CH_STEP * TS * 2;          // kt  token-major  [32][TS] u16, channels at tm_pos
constexpr int OFF_KH = OFF_KT + CH_STEP * TS * 2;          // kh  channel-major [64][CS] u16
constexpr int OFF_XT = OFF_KH + CH_N * CS * 2;             // xt  channel-major
constexpr int OFF_XH = OFF_XT + CH_N * CS * 2;             // xh  channel-major
constexpr int OFF_AS = OFF_XH + CH_N * CS * 2;             // a_t channel-major [64][CS] f32
constexpr int OFF_BL = OFF_AS + CH_N * CS * 4;             // b_L [2][64] f32
constexpr int OFF_AL = OFF_BL + 2 * CH_N * 4;              // a_L [2][64] f32
constexpr int OPS_BYTES = OFF_AL + 2 * CH_N * 4;
// Two stages of two steps each: a workgroup barrier every 64 tokens, the prep waves one stage ahead.
constexpr int OFF_VERDICT = 4 * OPS_BYTES;      // one int: some prep wave of this workgroup flagged the row
constexpr int FWD_SMEM = OFF_VERDICT + 16;
static_assert(FWD_SMEM <= 160 * 1024, "forward operand buffers exceed the LDS of one CU");
static_assert(OPS_BYTES % 16 == 0, "operand buffers must keep 16-byte alignment");

// ---- raw inputs --------------------------------------------------------------------------
// One prep lane: the gate at its eight tokens, the gate at the block's other eight tokens, and
// NV value arrays (key side: k and q, value side: x) at its own tokens.
template <int NV> struct RawSet {
    u16 gown[8], goth[8], val[NV][8];
};

// gate, val0, val1 (NV = 2 only): wave-uniform addresses of token 0 of the batch row; tok_own / tok_oth:
// first of the eight own / other tokens; lane_bytes = 2 * channel.  All sixteen tokens must exist.
// Consecutive tokens are ts elements apart.  HEADS = false: ts = 64, the token inside the half is an
// immediate offset.  HEADS = true: ts is a run-time multiple of 64; tok_blk is the block's first
// token (wave-uniform) and own_off[t] / oth_off[t] are the lane's byte offsets of its own / other
// eight tokens from there (channel included; kept in registers for the whole sequence).
template <int NV, bool HEADS>
__device__ __forceinline__ void raw_issue(RawSet<NV> &r, const u16 *gate, const u16 *val0, const u16 *val1, int tok_own,
                                          int tok_oth, u32 lane_bytes, int tok_blk, u32 ts, const u32 (&own_off)[8],
                                          const u32 (&oth_off)[8]) {
    const u16 *const val[2] = {val0, val1};
    if constexpr (!HEADS) {
        auto at = [&](const u16 *base, int tok) -> const u16 * {
            return reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base + (u32)tok * CH_N) + lane_bytes);
        };
        const u16 *go = at(gate, tok_own), *gx = at(gate, tok_oth);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.goth[t] = gx[t * CH_N];
#pragma unroll
        for (int t = 0; t < 8; ++t) r.gown[t] = go[t * CH_N];
#pragma unroll
        for (int a = 0; a < NV; ++a) {
            const u16 *va = at(val[a], tok_own);
#pragma unroll
            for (int t = 0; t < 8; ++t) r.val[a][t] = va[t * CH_N];
        }
    } else {
        auto ld = [&](const u16 *base, u32 off) -> u16 {
            return *reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base + (u32)tok_blk * ts) + off);
        };
#pragma unroll
        for (int t = 0; t < 8; ++t) r.goth[t] = ld(gate, oth_off[t]);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.gown[t] = ld(gate, own_off[t]);
#pragma unroll
        for (int a = 0; a < NV; ++a) {
#pragma unroll
            for (int t = 0; t < 8; ++t) r.val[a][t] = ld(val[a], own_off[t]);
        }
    }
}

// The same for the last, partial step of a sequence: tokens past the end are read from the last
// one (and replaced by raw_take_tail).
template <int NV>
__device__ __forceinline__ void raw_issue_tail(RawSet<NV> &r, const u16 *gate, const u16 *val0, const u16 *val1,
                                               int tok_own, int tok_oth, int T, u32 lane_bytes, u32 ts) {
    const u16 *const val[2] = {val0, val1};
    auto at = [&](const u16 *base, int tok) -> const u16 * {
        return reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base + (u32)min(tok, T - 1) * ts) +
                                             lane_bytes);
    };
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        r.goth[t] = *at(gate, tok_oth + t);
        r.gown[t] = *at(gate, tok_own + t);
#pragma unroll
        for (int a = 0; a < NV; ++a) r.val[a][t] = *at(val[a], tok_own + t);
    }
}

template <int NV> struct RawF {
    float gown[8], goth_prod, val[NV][8];
    u32 bad;      // own gates outside [0, 1]
};

// Gates enter the products no smaller than FLOOR_BITS (2^-24): an exactly zero gate, which an fp16
// sigmoid returns below a logit of about -17, would make the block's prefix products zero and their
// inverses infinite.  What the floor lets through from before such a step, 2^-24 of the state, is far
// below the rounding of the 16-bit outputs.
template <typename IOE> __device__ __forceinline__ u16 floor_gate(u16 bits) {
    return bits > IOE::FLOOR_BITS ? bits : IOE::FLOOR_BITS;
}

// Registers -> floats.
template <typename IOE, int NV> __device__ __forceinline__ RawF<NV> raw_take(const RawSet<NV> &r) {
    RawF<NV> f;
    // the loads complete in order: one wait for the last of them covers the whole set
    asm volatile("" ::"v"(r.val[NV - 1][7]));
    u16 mx = 0;
    float po = 1.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        mx = r.gown[t] > mx ? r.gown[t] : mx;     // gates must lie in [0, 1]: bits <= bits(1.0) (negative, NaN: above)
        f.gown[t] = IOE::to_f32(floor_gate<IOE>(r.gown[t]));
        po *= IOE::to_f32(floor_gate<IOE>(r.goth[t]));
#pragma unroll
        for (int a = 0; a < NV; ++a) f.val[a][t] = IOE::to_f32(r.val[a][t]);
    }
    f.bad = (mx > IOE::ONE_BITS) ? 1u : 0u;
    f.goth_prod = po;
    return f;
}

// Partial step: tokens past the end act as identity (gate 1, everything else 0).
template <typename IOE, int NV>
__device__ __forceinline__ RawF<NV> raw_take_tail(const RawSet<NV> &r, int tok_own, int tok_oth, int T) {
    RawF<NV> f;
    u16 mx = 0;
    float po = 1.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        if (tok_oth + t < T) po *= IOE::to_f32(floor_gate<IOE>(r.goth[t]));
        const bool own = tok_own + t < T;
        const u16 gb = own ? r.gown[t] : (u16)0;
        mx = gb > mx ? gb : mx;
        f.gown[t] = own ? IOE::to_f32(floor_gate<IOE>(r.gown[t])) : 1.0f;
#pragma unroll
        for (int a = 0; a < NV; ++a) f.val[a][t] = own ? IOE::to_f32(r.val[a][t]) : 0.0f;
    }
    f.bad = (mx > IOE::ONE_BITS) ? 1u : 0u;
    f.goth_prod = po;
    return f;
}

// eight tokens of one channel as four packed pairs
struct Packed8 {
    u32 p[4];
};
template <typename OPE> __device__ __forceinline__ Packed8 pack8(const float (&v)[8]) {
    Packed8 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.p[i] = OPE::pack2(v[2 * i], v[2 * i + 1]);
    return r;
}
// token-major: tile[(tok0 + t) * TS + tm_pos(c)]
__device__ __forceinline__ void write_tm8(unsigned char *tile, int c, int tok0, const Packed8 &v) {
    u16 *tm = reinterpret_cast<u16 *>(tile) + tok0 * TS + tm_pos(c);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        tm[(2 * i) * TS] = (u16)(v.p[i] & 0xffffu);
        tm[(2 * i + 1) * TS] = (u16)(v.p[i] >> 16);
    }
}
// channel-major: tile[c * CS + tok0 + t]
__device__ __forceinline__ void write_cm8(unsigned char *tile, int c, int tok0, const Packed8 &v) {
    uint2 *cm = reinterpret_cast<uint2 *>(tile + (c * CS + tok0) * 2);
    cm[0] = make_uint2(v.p[0], v.p[1]);
    cm[1] = make_uint2(v.p[2], v.p[3]);
}

// Prefix and suffix scalings of one half block (h = 0: tokens 0..7, h = 1: tokens 8..15):
//   pre[t] = prod_{r<=t} gate_r from the block start, hat = v * prod_{r>t} gate_r, til = hat / total.
template <typename OPE, int NV>
__device__ __forceinline__ float scale_half(const RawF<NV> &f, int h, float (&pre)[8], float (&hat)[8], float (&til)[8],
                                            u32 &bad, float &min_tot) {
    float run = h ? f.goth_prod : 1.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        run *= f.gown[t];
        pre[t] = run;
    }
    const float tot = h ? run : run * f.goth_prod;
    bad |= f.bad;
    min_tot = fminf(min_tot, tot);       // the smallest 16-step product of the row decides at the end
    const float itot = __builtin_amdgcn_rcpf(tot);
    float sfx = h ? 1.0f : f.goth_prod;
#pragma unroll
    for (int t = 7; t >= 0; --t) {
        hat[t] = f.val[0][t] * sfx;      // scaled to the block end   (<= |v|)
        til[t] = hat[t] * itot;          // scaled to the block start (v / prefix)
        sfx *= f.gown[t];
    }
    return tot;
}

// One side of the prep work for the whole sequence: KEY = true builds qs, kt (token-major), kh
// (channel-major) and b_L from f_key, k, q; KEY = false builds xt, xh, a_t and a_L from f, x.
// c: this lane's channel; hh: block of the step (wave-uniform); h: token half (wave-uniform, or
// per lane when a wave covers both halves of 32 channels); flag_slot: where this workgroup
// reports rows the chunked form cannot take.
template <typename IOE, typename OPE, bool KEY, bool HEADS>
__device__ __forceinline__ void fwd_prep_side(const ChunkFwdArgs &p, unsigned char *smem, int tid, int64_t b, int c,
                                              int hh, int h, int64_t flag_slot) {
    constexpr int NV = KEY ? 2 : 1;
    const int T = (int)p.T;                                // the launcher admits T < 2^24 only
    const int64_t row_off = row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N;
    const u32 ts = HEADS ? (u32)p.heads * CH_N : (u32)CH_N;        // elements between consecutive tokens
    const u16 *const gate = reinterpret_cast<const u16 *>(KEY ? p.f_key : p.f) + row_off;
    const u16 *const val0 = reinterpret_cast<const u16 *>(KEY ? p.k : p.x) + row_off;
    const u16 *const val1 = reinterpret_cast<const u16 *>(p.q) + row_off;      // key side only
    const int nfull = T / CH_STEP;                         // full 32-token steps; a partial one may follow
    const int off_own = CH_L * hh + 8 * h, off_oth = CH_L * hh + 8 * (1 - h);   // inside a step
    const u32 lane_bytes = 2u * (u32)c;
    u32 own_off[8], oth_off[8];                            // HEADS only: vector offsets of the sixteen tokens
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        own_off[t] = HEADS ? lane_bytes + 2u * (u32)(8 * h + t) * ts : 0u;
        oth_off[t] = HEADS ? lane_bytes + 2u * (u32)(8 * (1 - h) + t) * ts : 0u;
    }
    u32 bad = 0;
    float min_tot = 1.0f;

    // this wave's share of the operand tiles of step n
    auto build = [&](const RawF<NV> &f, int n) {
        unsigned char *ops = smem + (n & 3) * OPS_BYTES;
        float pre[8], hat[8], til[8];
        const float tot = scale_half<OPE, NV>(f, h, pre, hat, til, bad, min_tot);
        const int tok0 = CH_L * hh + 8 * h;
        if constexpr (KEY) {
            float qs[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) qs[t] = f.val[1][t] * pre[t];
            write_tm8(ops + OFF_QT, c, tok0, pack8<OPE>(qs));
            write_tm8(ops + OFF_KT, c, tok0, pack8<OPE>(til));
            write_cm8(ops + OFF_KH, c, tok0, pack8<OPE>(hat));
            if (h == 0) reinterpret_cast<float *>(ops + OFF_BL)[hh * CH_N + c] = tot;
        } else {
            write_cm8(ops + OFF_XT, c, tok0, pack8<OPE>(til));
            write_cm8(ops + OFF_XH, c, tok0, pack8<OPE>(hat));
            float4 *AS = reinterpret_cast<float4 *>(ops + OFF_AS + (c * CS + tok0) * 4);
            AS[0] = make_float4(pre[0], pre[1], pre[2], pre[3]);
            AS[1] = make_float4(pre[4], pre[5], pre[6], pre[7]);
            if (h == 0) reinterpret_cast<float *>(ops + OFF_AL)[hh * CH_N + c] = tot;
        }
    };
    auto issue = [&](RawSet<NV> &r, int step, u32 lb) {
        const int st = min(step, nfull - 1);       // past the last full step: that step again (never used)
        raw_issue<NV, HEADS>(r, gate, val0, val1, st * CH_STEP + off_own, st * CH_STEP + off_oth, lb,
                             st * CH_STEP + CH_L * hh, ts, own_off, oth_off);
    };
    // builds the tiles of full step n, which r holds; r then takes step n + 2
    auto prepare = [&](RawSet<NV> &r, int n) {
        const RawF<NV> f = raw_take<IOE, NV>(r);
        // The loads that refill r must come after the conversions above, or they need registers
        // (and a wait) of their own: tie their address to the converted values.
        u32 lb = lane_bytes;
        if constexpr (KEY) {
            asm volatile("" : "+v"(lb)
                         : "v"(f.gown[0]), "v"(f.gown[1]), "v"(f.gown[2]), "v"(f.gown[3]), "v"(f.gown[4]), "v"(f.gown[5]),
                           "v"(f.gown[6]), "v"(f.gown[7]), "v"(f.val[0][0]), "v"(f.val[0][1]), "v"(f.val[0][2]),
                           "v"(f.val[0][3]), "v"(f.val[0][4]), "v"(f.val[0][5]), "v"(f.val[0][6]), "v"(f.val[0][7]),
                           "v"(f.val[NV - 1][0]), "v"(f.val[NV - 1][1]), "v"(f.val[NV - 1][2]), "v"(f.val[NV - 1][3]),
                           "v"(f.val[NV - 1][4]), "v"(f.val[NV - 1][5]), "v"(f.val[NV - 1][6]), "v"(f.val[NV - 1][7]),
                           "v"(f.goth_prod), "v"(f.bad));
        } else {
            asm volatile("" : "+v"(lb)
                         : "v"(f.gown[0]), "v"(f.gown[1]), "v"(f.gown[2]), "v"(f.gown[3]), "v"(f.gown[4]), "v"(f.gown[5]),
                           "v"(f.gown[6]), "v"(f.gown[7]), "v"(f.val[0][0]), "v"(f.val[0][1]), "v"(f.val[0][2]),
                           "v"(f.val[0][3]), "v"(f.val[0][4]), "v"(f.val[0][5]), "v"(f.val[0][6]), "v"(f.val[0][7]),
                           "v"(f.goth_prod), "v"(f.bad));
        }
        if constexpr (HEADS) {      // the token offsets carry the same dependency (and stay in registers)
            asm volatile(""
                         : "+v"(own_off[0]), "+v"(own_off[1]), "+v"(own_off[2]), "+v"(own_off[3]), "+v"(own_off[4]),
                           "+v"(own_off[5]), "+v"(own_off[6]), "+v"(own_off[7])
                         : "v"(lb));
            asm volatile(""
                         : "+v"(oth_off[0]), "+v"(oth_off[1]), "+v"(oth_off[2]), "+v"(oth_off[3]), "+v"(oth_off[4]),
                           "+v"(oth_off[5]), "+v"(oth_off[6]), "+v"(oth_off[7])
                         : "v"(lb));
        }
        issue(r, n + 2, lb);
        build(f, n);
    };

    // Full steps alternate between two register sets.  The loop always does a whole pair (set A,
    // then set B) with no exit in between, so that the order of the loads in flight is the same on
    // every path into it; an odd count peels the first step off.  A stage is two steps: the barrier
    // that publishes the tiles comes after every odd step and after the last one.
    const int nsteps = nfull + (nfull * CH_STEP < T ? 1 : 0);
    auto publish = [&](int n) {
        if ((n & 1) || n == nsteps - 1) __syncthreads();
    };
    if (nfull > 0) {
        RawSet<NV> setA, setB;
        int n = 0;
        if (nfull & 1) {
            issue(setB, 0, lane_bytes);
            issue(setA, 1, lane_bytes);
            prepare(setB, 0);
            publish(0);
            n = 1;
        } else {
            issue(setA, 0, lane_bytes);
            issue(setB, 1, lane_bytes);
        }
        for (; n < nfull; n += 2) {
            prepare(setA, n);
            publish(n);
            prepare(setB, n + 1);
            publish(n + 1);
        }
    }
    if (nfull * CH_STEP < T) {      // the partial step at the end
        RawSet<NV> r;
        const int t_own = nfull * CH_STEP + off_own, t_oth = nfull * CH_STEP + off_oth;
        raw_issue_tail<NV>(r, gate, val0, val1, t_own, t_oth, T, lane_bytes, ts);
        build(raw_take_tail<IOE, NV>(r, t_own, t_oth, T), nfull);
        publish(nfull);
    }
    if (bad || !(min_tot >= OPE::MIN_PRODUCT)) {
        p.row_flags[flag_slot] = 1;
        *reinterpret_cast<volatile int *>(smem + OFF_VERDICT) = 1;
    }
    // what the chunk-parallel backward will make of this row: with every 16-step product at or above
    // PAR_HINT_MIN_PRODUCT its products over half a chunk (one or two blocks) are inside its range
    if (p.par_hint != nullptr && (bad || !(min_tot >= PAR_HINT_MIN_PRODUCT))) p.par_hint[flag_slot] = 1;
}

template <typename E> __device__ __forceinline__ uint2 pack4(const floatx4 &v) {
    return make_uint2(E::pack2(v[0], v[1]), E::pack2(v[2], v[3]));
}

// state slab of one wave <-> global [64][64] state of one row (16-bit I/O)
template <typename IOE>
__device__ __forceinline__ void store_state(const floatx4 (&S)[4], u16 *dst, int d, int g) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uint2 *>(dst + d * CH_N + 16 * j + 4 * g) = pack4<IOE>(S[j]);
}

template <typename IOE, typename OPE, bool HEADS>
__device__ __forceinline__ void fwd_matrix_waves(const ChunkFwdArgs &p, unsigned char *smem, int tid, int64_t b,
                                                 int dbase, int64_t flag_slot, bool clear_other_slot) {
    const int w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int d = dbase + 16 * w + r;          // this lane's state row (value channel)
    const int T = (int)p.T;
    u16 *ckpt = reinterpret_cast<u16 *>(p.ckpt);
    u16 *const out = reinterpret_cast<u16 *>(p.out) + row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N;
    const u32 ts = HEADS ? (u32)p.heads * CH_N : (u32)CH_N;        // elements between consecutive tokens
    // S[j][i]: value channel d, key channel 16j + 4g + i
    floatx4 S[4];
    {
        const u16 *s0 = reinterpret_cast<const u16 *>(p.s0) + b * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint2 v = *reinterpret_cast<const uint2 *>(s0 + d * CH_N + 16 * j + 4 * g);
            S[j][0] = IOE::to_f32((u16)(v.x & 0xffff));
            S[j][1] = IOE::to_f32((u16)(v.x >> 16));
            S[j][2] = IOE::to_f32((u16)(v.y & 0xffff));
            S[j][3] = IOE::to_f32((u16)(v.y >> 16));
        }
    }
    int until_ckpt = 0;
    int64_t chunk = 0;
    float omax = 0.f;
    if (tid == 0) {
        p.row_flags[flag_slot] = 0;
        if (clear_other_slot) p.row_flags[chunk_rows_padded(p.B) + b] = 0;
        if (p.par_hint != nullptr) {
            p.par_hint[flag_slot] = 0;
            if (clear_other_slot) p.par_hint[chunk_rows_padded(p.B) + b] = 0;
        }
        *reinterpret_cast<volatile int *>(smem + OFF_VERDICT) = 0;
    }
    // One step (two blocks).  FULL: all 32 tokens exist, which leaves the body without a branch
    // around its stores, so that the LDS reads of the whole step can be scheduled ahead of the
    // matrix products that use them.
    // BAR: the step is the first of its stage and starts with the workgroup barrier.
    auto step = [&](int n, auto full_c, auto bar_c) {
        constexpr bool FULL = decltype(full_c)::value;
        if constexpr (decltype(bar_c)::value) {
            __syncthreads();        // the operand tiles of steps n and n + 1 are in LDS
        }
        const unsigned char *ops = smem + (n & 3) * OPS_BYTES;
        const u16 *QT = reinterpret_cast<const u16 *>(ops + OFF_QT);
        const u16 *KT = reinterpret_cast<const u16 *>(ops + OFF_KT);
        const u16 *KH = reinterpret_cast<const u16 *>(ops + OFF_KH);
        const u16 *XT = reinterpret_cast<const u16 *>(ops + OFF_XT);
        const u16 *XH = reinterpret_cast<const u16 *>(ops + OFF_XH);
        const float *AS = reinterpret_cast<const float *>(ops + OFF_AS);
        const float *BL = reinterpret_cast<const float *>(ops + OFF_BL);
        const float *AL = reinterpret_cast<const float *>(ops + OFF_AL);
        if (ckpt != nullptr) {          // checkpoint interval is a multiple of the step
            if (until_ckpt == 0) {
                store_state<IOE>(S, ckpt + (b * p.NC + chunk) * (CH_N * CH_N), d, g);
                until_ckpt = p.C;
                ++chunk;
            }
            until_ckpt -= CH_STEP;
        }
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int tok0 = CH_L * hh;
            // P^T[s,t] = kt_s . qs_t, kept for s <= t, as the A operand of the intra product
            const u16 *krow = KT + (tok0 + r) * TS + 8 * g;
            const u16 *qrow = QT + (tok0 + r) * TS + 8 * g;
            floatx4 pt = {0.f, 0.f, 0.f, 0.f};
            pt = OPE::mfma32(*reinterpret_cast<const uint4 *>(krow), *reinterpret_cast<const uint4 *>(qrow), pt);
            pt = OPE::mfma32(*reinterpret_cast<const uint4 *>(krow + 32), *reinterpret_cast<const uint4 *>(qrow + 32), pt);
#pragma unroll
            for (int i = 0; i < 4; ++i) pt[i] = (4 * g + i <= r) ? pt[i] : 0.f;
            const uint2 pa = pack4<OPE>(pt);
            // o[t,d] = a_t[d] * ( sum_k qs_t[k] S0[d,k] + sum_{s<=t} P[t,s] xt_s[d] )
            const u16 *qperm = QT + (tok0 + r) * TS + 16 * g;     // channels 16j + 4g + e, j = 0..3, contiguous
            const uint2 s0p = pack4<OPE>(S[0]), s1p = pack4<OPE>(S[1]), s2p = pack4<OPE>(S[2]), s3p = pack4<OPE>(S[3]);
            floatx4 o = {0.f, 0.f, 0.f, 0.f};
            o = OPE::mfma32(*reinterpret_cast<const uint4 *>(qperm), make_uint4(s0p.x, s0p.y, s1p.x, s1p.y), o);
            o = OPE::mfma32(*reinterpret_cast<const uint4 *>(qperm + 8), make_uint4(s2p.x, s2p.y, s3p.x, s3p.y), o);
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            const floatx4 oi = OPE::mfma16(pa, *reinterpret_cast<const uint2 *>(XT + d * CS + tok0 + 4 * g), zero);
            const float4 as = *reinterpret_cast<const float4 *>(AS + d * CS + tok0 + 4 * g);
            const float asv[4] = {as.x, as.y, as.z, as.w};
            // 16 lanes write 32 contiguous bytes of a token row; the four waves complete the row
            const int tg = n * CH_STEP + tok0 + 4 * g;
            u16 *const po = out + ((u32)tg * ts + (u32)d);      // the four tokens: immediate offsets (folded rows)
            float res[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                res[i] = (o[i] + oi[i]) * asv[i];
                if constexpr (IOE::CHECK_RESULTS) omax = __builtin_fmaf(res[i], 0.0f, omax);        // 0 until a result is inf or NaN, then NaN
            }
            if constexpr (FULL) {
#pragma unroll
                for (int i = 0; i < 4; ++i) po[i * ts] = cvt1<IOE>(res[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (tg + i < T) po[i * ts] = cvt1<IOE>(res[i]);
            }
            // S_L = (a_L (x) b_L) * S0 + sum_s xh_s (x) kh_s
            const float aL = AL[hh * CH_N + d];
            const uint2 xh = *reinterpret_cast<const uint2 *>(XH + d * CS + tok0 + 4 * g);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 bl = *reinterpret_cast<const float4 *>(BL + hh * CH_N + 16 * j + 4 * g);
                S[j][0] *= aL * bl.x;
                S[j][1] *= aL * bl.y;
                S[j][2] *= aL * bl.z;
                S[j][3] *= aL * bl.w;
                S[j] = OPE::mfma16(*reinterpret_cast<const uint2 *>(KH + (16 * j + r) * CS + tok0 + 4 * g), xh, S[j]);
            }
        }
    };
    const int nfull = T / CH_STEP;
    int n = 0;
    for (; n + 1 < nfull; n += 2) {
        step(n, std::true_type{}, std::true_type{});
        step(n + 1, std::true_type{}, std::false_type{});
    }
    if (n < nfull) step(n, std::true_type{}, std::true_type{});
    if (nfull * CH_STEP < T) {
        if (nfull & 1)
            step(nfull, std::false_type{}, std::false_type{});
        else
            step(nfull, std::false_type{}, std::true_type{});
    }
    store_state<IOE>(S, reinterpret_cast<u16 *>(p.next_state) + b * (CH_N * CH_N), d, g);
    // A result that is not finite (an operand scaled by 1 / product left the range of its type, or a product of
    // scaled operands that of fp32) hands the row to the exact recurrence like a gate outside the range does.
    if constexpr (IOE::CHECK_RESULTS) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) omax = __builtin_fmaf(S[j][i], 0.0f, omax);
    }
    if (!(omax == 0.0f)) {
        p.row_flags[flag_slot] = 1;
        *reinterpret_cast<volatile int *>(smem + OFF_VERDICT) = 1;
        if (p.par_hint != nullptr) p.par_hint[flag_slot] = 1;
    }
}

// End of a workgroup's work on its (part of a) batch row.  A barrier publishes the prep waves'
// verdict; if the chunked form could not take the row, the workgroup's first SCAN_THREADS threads
// redo value channels of tiles [tile0, tile1) with the exact scan, in place, and everyone else
// leaves (a workgroup barrier only waits for the waves that are still there).
template <typename IOE>
__device__ __forceinline__ void fwd_redo_if_flagged(const ChunkFwdArgs &p, unsigned char *smem, int tid, int64_t b,
                                                    int tile0, int tile1) {
    __syncthreads();
    if (tid >= SCAN_THREADS || !p.redo) return;
    if (*reinterpret_cast<volatile int *>(smem + OFF_VERDICT) == 0) return;
    ScanFwdArgs sa{};
    sa.x = p.x; sa.f = p.f; sa.q = p.q; sa.k = p.k; sa.f_key = p.f_key; sa.s0 = p.s0;
    sa.out = p.out; sa.next_state = p.next_state; sa.ckpt = p.ckpt;
    sa.B = p.B; sa.T = p.T; sa.D = CH_N; sa.K = CH_N; sa.NC = p.NC;
    sa.C = p.C; sa.kg = p.scan_kg; sa.tb = p.scan_tb; sa.ntiles = p.scan_ntiles; sa.heads = p.heads;
    for (int tile = tile0; tile < tile1; ++tile) {
        __syncthreads();        // the tiles of the chunked form, or of the tile before, are no longer read
        scan::fwd_scan_body_kg<typename IOE::io_type, 4, 16>(sa, b, tile);
    }
}

template <typename IOE, typename OPE, bool HEADS>
__global__ __launch_bounds__(FWD_THREADS) void lfw_fwd_chunk_kernel(ChunkFwdArgs p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int64_t b = blockIdx.x;
    // every wave executes exactly ceil(number of steps / 2) workgroup barriers
    if (tid < 256) {
        fwd_matrix_waves<IOE, OPE, HEADS>(p, smem, tid, b, 0, b, true);
    } else {
        // prep wave pw: (side, block of the step, token half); each SIMD gets one wave of each side
        const int pw = __builtin_amdgcn_readfirstlane((tid - 256) >> 6);
        const int hh = (pw >> 1) & 1, h = pw >> 2;
        if (((pw ^ h) & 1) == 0)
            fwd_prep_side<IOE, OPE, true, HEADS>(p, smem, tid - 256, b, tid & 63, hh, h, b);
        else
            fwd_prep_side<IOE, OPE, false, HEADS>(p, smem, tid - 256, b, tid & 63, hh, h, b);
    }
    fwd_redo_if_flagged<IOE>(p, smem, tid, b, 0, p.scan_ntiles);
}

// Two workgroups per batch row: blockIdx = half * rows_padded + row with rows_padded a multiple of
// 8, so that the two halves of a row land on the same XCD and share its L2 for the key-side
// inputs both of them read.  Each half reports flagged rows in a slot of its own (the value-side
// gates it checks are its own 32 channels): row_flags[row] and row_flags[rows_padded + row].
template <typename IOE, typename OPE, bool HEADS>
__global__ __launch_bounds__(FWD_THREADS_HALF) void lfw_fwd_chunk_half_kernel(ChunkFwdArgs p, int rows_padded) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int half = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - half * rows_padded;
    if (b >= p.B) return;
    const int64_t slot = (int64_t)half * rows_padded + b;
    // waves: 0, 1 matrix; 2..5 key side (block, token half); 6, 7 value side (block; a lane takes
    // one of the half's 32 channels and one token half).  SIMD i runs waves i and i + 4.
    if (tid < 128) {
        fwd_matrix_waves<IOE, OPE, HEADS>(p, smem, tid, b, 32 * half, slot, false);
    } else if (tid < 384) {
        const int pw = __builtin_amdgcn_readfirstlane((tid - 128) >> 6);
        fwd_prep_side<IOE, OPE, true, HEADS>(p, smem, tid - 128, b, tid & 63, pw & 1, pw >> 1, slot);
    } else {
        const int pw = __builtin_amdgcn_readfirstlane((tid - 384) >> 6);
        fwd_prep_side<IOE, OPE, false, HEADS>(p, smem, tid - 128, b, 32 * half + (tid & 31), pw, (tid >> 5) & 1, slot);
    }
    // this half's value channels are half of the scan's tiles
    fwd_redo_if_flagged<IOE>(p, smem, tid, b, half * (p.scan_ntiles / 2), (half + 1) * (p.scan_ntiles / 2));
}

template <typename IOE, typename OPE, bool HEADS> int launch(const ChunkFwdArgs &a, bool split, hipStream_t stream) {
    if (a.B > 0x1fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    if (a.heads < 1 || a.T * a.heads >= CHUNK_MAX_T)
        return fail(T2FW_ERR_UNSUPPORTED, "T=%lld with %d heads is too long for 32-bit row offsets", (long long)a.T, a.heads);
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    if (split) {
        auto kern = lfw_fwd_chunk_half_kernel<IOE, OPE, HEADS>;
        int rc = enable_lds(reinterpret_cast<const void *>(kern), FWD_SMEM, "hipFuncSetAttribute(forward chunk kernel, two workgroups per row)");
        if (rc) return rc;
        const int rows_padded = (int)chunk_rows_padded(a.B);
        hipLaunchKernelGGL(kern, dim3(2u * (unsigned)rows_padded), dim3(FWD_THREADS_HALF), FWD_SMEM, stream, a, rows_padded);
        return check_hip(hipGetLastError(), "lfw_fwd_chunk_half_kernel launch");
    }
    auto kern = lfw_fwd_chunk_kernel<IOE, OPE, HEADS>;
    int rc = enable_lds(reinterpret_cast<const void *>(kern), FWD_SMEM, "hipFuncSetAttribute(forward chunk kernel)");
    if (rc) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)a.B), dim3(FWD_THREADS), FWD_SMEM, stream, a);
    return check_hip(hipGetLastError(), "lfw_fwd_chunk_kernel launch");
}

}  // namespace

int chunk_forward(const ChunkFwdArgs &args, int dtype, int op, bool split, hipStream_t stream) {
    ChunkFwdArgs a = args;
    {   // geometry of the exact scan for a 64 x 64 state, as lfw_scan.hip chooses it
        const ScanGeom g = scan_geometry(CH_N);
        a.scan_kg = g.kg;
        int tb = 32;
        tb = std::min(tb, scan::PFC * SCAN_THREADS / (g.kg * g.kpl));
        tb = std::min(tb, scan::PFR * SCAN_THREADS / g.rows);
        a.scan_tb = tb;
        a.scan_ntiles = CH_N / g.rows;
        if (g.kpl != 4 || g.kg != 16 || a.scan_ntiles % 2 != 0)
            return fail(T2FW_ERR_UNSUPPORTED, "unexpected scan geometry for a 64 x 64 state");
        // the body runs in this kernel's LDS, below the verdict word
        const size_t need = scan_fwd_lds_bytes(tb, g.kg, g.kpl, g.rows);
        if (need > (size_t)OFF_VERDICT)
            return fail(T2FW_ERR_UNSUPPORTED, "the exact scan body needs %zu bytes of LDS, the forward kernel has %d", need,
                        OFF_VERDICT);
    }
    if (a.heads == 1) {
        if (dtype == T2FW_F16)
            return op == 1 ? launch<Fp16, Fp16, false>(a, split, stream) : launch<Fp16, Bf16, false>(a, split, stream);
        if (dtype == T2FW_BF16) return launch<Bf16, Bf16, false>(a, split, stream);
    } else {
        if (dtype == T2FW_F16)
            return op == 1 ? launch<Fp16, Fp16, true>(a, split, stream) : launch<Fp16, Bf16, true>(a, split, stream);
        if (dtype == T2FW_BF16) return launch<Bf16, Bf16, true>(a, split, stream);
    }
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
