// Backward pass of the decay rule in chunked matrix-core form, two workgroups per batch row, with
// stages of TWO blocks (32 tokens).  Block algebra, sides and operand names: lfw_chunk_bwd.hip.
//
// What differs from lfw_chunk_bwd.hip is the work of the eight prep waves and the stage length:
//   * a B stage covers a pair of blocks as an R stage does, so a chunk of four blocks takes two R
//     and two B stages (four workgroup barriers instead of six);
//   * a prep wave is (block of the pair, own / other side, token half) in both kinds of stage, and in
//     a B stage one lane builds the prefix-scaled AND the suffix-scaled operands of its side from
//     one set of gate conversions and one 16-step product: 32 two-byte loads and about 125 VALU
//     instructions where the one-role-per-wave form needs 48 loads and about 190 for the same tiles;
//   * raw inputs are kept in two register sets that are refilled in place, two stages ahead, after
//     their contents have been converted (the refill's address depends on the converted values, so
//     the compiler cannot hoist the loads above the conversions).
//
// Replaces lfw_cuda_bwd_kernel and the six einsums of the reference
// (t2fw/csrc/lfw_kernel.cu:61-102, t2fw/csrc/lfw.cpp:84-93).
#include <type_traits>

#include "lfw_chunk_bwd_dev.hpp"

namespace t2fw {
namespace {

using namespace bwd;

constexpr int PB_THREADS = 768;
constexpr int CC = 20;   // channel-major 16-token tiles: row stride in elements

// ---- LDS layout: a stage buffer holds the tiles of its two blocks, one region per block ---------
constexpr int TM_TILE = CH_L * TS * 2;       // token-major 16-bit tile [16][TS], channels permuted (tm_pos)
constexpr int CM_TILE = CH_N * CC * 2;       // channel-major 16-bit tile [64][CC]
constexpr int CF_TILE = CH_N * CC * 4;       // channel-major fp32 tile [64][CC]
enum { TM_AOS = 0, TM_VOT, TM_VOH, TM_NUM };
enum { CM_AOS = 0, CM_VOH, CM_AS, CM_VT, CM_VH, CM_NUM };      // R stages use CM_VOH and CM_VH only
enum { F_RG = 0, F_IP, F_PP, F_NUM };        // 1/own gate, 1/own prefix, own prefix
constexpr int OFF_TM = 0;
constexpr int OFF_CM = OFF_TM + TM_NUM * TM_TILE;
constexpr int OFF_CF = OFF_CM + CM_NUM * CM_TILE;
constexpr int OFF_LV = OFF_CF + F_NUM * CF_TILE;      // 16-step gate products [other side, own side][64] f32
constexpr int BLOCK_BYTES = OFF_LV + 2 * CH_N * 4;
constexpr int STAGE_BYTES = 2 * BLOCK_BYTES;
constexpr int PB_SMEM = 2 * STAGE_BYTES;
static_assert(PB_SMEM <= 160 * 1024, "backward stage buffers exceed the LDS of one CU");
static_assert(BLOCK_BYTES % 16 == 0, "block regions must keep 16-byte alignment");

// ---- stage schedule ----------------------------------------------------------------------
// Chunks are visited from the last one down; a chunk with M pairs of blocks takes M R stages
// (pairs 0..M-1, forward in time), then M B stages (pairs M-1..0).  The last chunk of a sequence
// may have fewer pairs, its last pair one block, its last block fewer than 16 tokens.
template <int NB> struct PairSchedule {
    static constexpr int MP = NB / 2, PER = 2 * MP;      // pairs and stages of a full chunk
    int NC, C, n_last, m_last, total;
    __device__ PairSchedule(int64_t T, int64_t NC_, int C_) {
        NC = (int)NC_;
        C = C_;
        const int len_last = (int)(T - (NC_ - 1) * C_);
        m_last = (len_last + 2 * CH_L - 1) / (2 * CH_L);
        n_last = 2 * m_last;
        total = n_last + (NC - 1) * PER;
    }
    // stage s -> first token of its pair of blocks, and whether it is a B stage (wave-uniform)
    __device__ void at(int s, int &tok, bool &bmode) const {
        int chunk, local, m;
        if (s < n_last) {
            chunk = NC - 1;
            local = s;
            m = m_last;
        } else {
            const unsigned s2 = (unsigned)(s - n_last);
            chunk = NC - 2 - (int)(s2 / (unsigned)PER);
            local = (int)(s2 % (unsigned)PER);
            m = MP;
        }
        bmode = local >= m;
        const int pair = bmode ? 2 * m - 1 - local : local;
        tok = chunk * C + pair * 2 * CH_L;
    }
};

// ---- raw inputs --------------------------------------------------------------------------
// A prep lane works on one channel and eight tokens of one block; it needs the gate at those
// tokens and at the block's other eight, and the value and the adjoint array of its side at its own
// tokens (R stages do not use the adjoint; it is loaded all the same, so that every stage has the
// same number of loads in flight and the waits for them can be exact).
struct RawSet {
    u16 gown[8], goth[8], val[8], adj[8];
};
struct RawF {
    float gown[8], val[8], adj[8], poth;
    u32 bad;
};

// Where the sixteen tokens of a block are, seen from a prep lane (as in lfw_chunk_bwd.hip).
template <bool HEADS> struct TokenMap {
    u32 ts, voff_own, voff_oth, shift_own, shift_oth, tok_off[8];
    __device__ __forceinline__ TokenMap(u32 ts_, int h, int c) {
        ts = HEADS ? ts_ : (u32)CH_N;
        voff_own = (u32)(8 * h * CH_N + c) * 2u;
        voff_oth = (u32)(8 * (1 - h) * CH_N + c) * 2u;
        shift_own = 8u * (u32)h * ts;
        shift_oth = 8u * (u32)(1 - h) * ts;
#pragma unroll
        for (int t = 0; t < 8; ++t) tok_off[t] = 2u * ((u32)c + (u32)t * ts);
    }
};

// gate, val, adj: wave-uniform addresses of the block's first token; all sixteen tokens exist
template <bool HEADS>
__device__ __forceinline__ void raw_issue(RawSet &r, const u16 *gate, const u16 *val, const u16 *adj, TokenMap<HEADS> &m) {
    if constexpr (!HEADS) {
        auto at = [&](const u16 *base, u32 voff, int t) -> u16 {
            return *reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base + t * CH_N) + voff);
        };
#pragma unroll
        for (int t = 0; t < 8; ++t) r.goth[t] = at(gate, m.voff_oth, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.gown[t] = at(gate, m.voff_own, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.val[t] = at(val, m.voff_own, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.adj[t] = at(adj, m.voff_own, t);
    } else {
        auto at = [&](const u16 *base, int t) -> u16 {
            return *reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base) + m.tok_off[t]);
        };
        const u16 *const go = gate + m.shift_own, *const gx = gate + m.shift_oth;
        const u16 *const vo = val + m.shift_own, *const ao = adj + m.shift_own;
#pragma unroll
        for (int t = 0; t < 8; ++t) r.goth[t] = at(gx, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.gown[t] = at(go, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.val[t] = at(vo, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.adj[t] = at(ao, t);
    }
}

// The same for a block that reaches past the end of the sequence (or lies past it): tokens past the
// end are read from the last one, with the same number of loads, and replaced when the set is taken.
// row_*: token 0 of the batch row.
__device__ __forceinline__ void raw_issue_tail(RawSet &r, const u16 *row_gate, const u16 *row_val, const u16 *row_adj,
                                               int tok_own, int tok_oth, int T, u32 cbytes, u32 ts) {
    auto at = [&](const u16 *base, int tok) -> u16 {
        return *reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base + (u32)min(tok, T - 1) * ts) + cbytes);
    };
#pragma unroll
    for (int t = 0; t < 8; ++t) r.goth[t] = at(row_gate, tok_oth + t);
#pragma unroll
    for (int t = 0; t < 8; ++t) r.gown[t] = at(row_gate, tok_own + t);
#pragma unroll
    for (int t = 0; t < 8; ++t) r.val[t] = at(row_val, tok_own + t);
#pragma unroll
    for (int t = 0; t < 8; ++t) r.adj[t] = at(row_adj, tok_own + t);
}

template <typename IOE> __device__ __forceinline__ u32 gate_check8(const u16 (&g)[8]) {
    u16 mx = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const u16 m1 = (u16)(g[t] - 1);      // gates must lie in (0, 1]: 0 < bits <= bits(1.0)
        mx = m1 > mx ? m1 : mx;
    }
    return (mx >= IOE::ONE_BITS) ? 1u : 0u;
}


// Registers -> floats, with the gate range check (gates must lie in (0, 1]) and the product of the
// other half's gates.  TAIL: tokens at or past T act as identity (gate 1, everything else 0).
template <typename IOE, bool TAIL>
__device__ __forceinline__ RawF raw_take(const RawSet &r, int tok_own, int tok_oth, int T) {
    RawF f;
    // the loads complete in order: one wait for the last of them covers the whole set
    asm volatile("" ::"v"(r.adj[7]));
    float po = 1.0f;
    u16 mx = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const bool own = !TAIL || tok_own + t < T;
        const u16 m1 = own ? (u16)(r.gown[t] - 1) : (u16)0;      // 0 < bits <= bits(1.0)
        mx = m1 > mx ? m1 : mx;
        f.gown[t] = own ? IOE::to_f32(r.gown[t]) : 1.0f;
        f.val[t] = own ? IOE::to_f32(r.val[t]) : 0.0f;
        f.adj[t] = own ? IOE::to_f32(r.adj[t]) : 0.0f;
        if (!TAIL || tok_oth + t < T) po *= IOE::to_f32(r.goth[t]);
    }
    f.poth = po;
    f.bad = (mx >= IOE::ONE_BITS) ? 1u : 0u;
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


__device__ __forceinline__ void write_tm8(unsigned char *blk, int tile, int c, int t0, const Packed8 &v) {
    u16 *tm = reinterpret_cast<u16 *>(blk + OFF_TM + tile * TM_TILE) + t0 * TS + tm_pos(c);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        tm[(2 * i) * TS] = (u16)(v.p[i] & 0xffffu);
        tm[(2 * i + 1) * TS] = (u16)(v.p[i] >> 16);
    }
}

__device__ __forceinline__ void write_cm8(unsigned char *blk, int tile, int c, int t0, const Packed8 &v) {
    uint2 *cm = reinterpret_cast<uint2 *>(blk + OFF_CM + tile * CM_TILE + (c * CC + t0) * 2);
    cm[0] = make_uint2(v.p[0], v.p[1]);
    cm[1] = make_uint2(v.p[2], v.p[3]);
}

__device__ __forceinline__ void write_cf8(unsigned char *blk, int tile, int c, int t0, const float (&v)[8]) {
    float4 *cf = reinterpret_cast<float4 *>(blk + OFF_CF + tile * CF_TILE + (c * CC + t0) * 4);
    cf[0] = make_float4(v[0], v[1], v[2], v[3]);
    cf[1] = make_float4(v[4], v[5], v[6], v[7]);
}

__device__ __forceinline__ float *lv_vec(unsigned char *blk, int own) {
    return reinterpret_cast<float *>(blk + OFF_LV) + own * CH_N;
}
__device__ __forceinline__ const float *lv_vec(const unsigned char *blk, int own) {
    return reinterpret_cast<const float *>(blk + OFF_LV) + own * CH_N;
}

// One prep lane's share of a stage: tokens 8h..8h+7 of one block, channel c, own or other side.
//   R stage: the suffix-scaled values (VH | VOH, channel-major) and the 16-step gate product.
//   B stage, other side: AOS (token- and channel-major), VOH (both), VOT (token-major), L_other.
//   B stage, own side  : AS, VH, VT (channel-major), 1/gate, 1/prefix, prefix (side 1), L_own.
template <typename OPE>
__device__ __forceinline__ void prep_lane(const RawF &f, unsigned char *blk, bool bmode, int own, int h, int c,
                                          bool want_pp, u32 &bad) {
    const int t0 = 8 * h;
    const float base = h ? f.poth : 1.0f;
    float pre[8];
    float run = base;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        run *= f.gown[t];
        pre[t] = run;
    }
    const float tot = h ? run : run * f.poth;
    bad |= (tot >= OPE::MIN_PRODUCT) ? 0u : 1u;
    const float itot = __builtin_amdgcn_rcpf(tot);
    float hat[8], til[8], inv[8];
    float sfx = h ? 1.0f : f.poth;
#pragma unroll
    for (int t = 7; t >= 0; --t) {
        inv[t] = sfx * itot;             // 1 / prefix_t
        hat[t] = f.val[t] * sfx;         // scaled to the block end
        til[t] = hat[t] * itot;          // scaled to the block start
        sfx *= f.gown[t];
    }
    if (h == 0) lv_vec(blk, own)[c] = tot;
    const Packed8 hp = pack8<OPE>(hat);
    if (!bmode) {
        write_cm8(blk, own ? CM_VH : CM_VOH, c, t0, hp);
        return;
    }
    bad |= f.bad;                        // every block's gates are range-checked in its B stage
    float v[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) v[t] = f.adj[t] * pre[t];
    const Packed8 vp = pack8<OPE>(v), tp = pack8<OPE>(til);
    if (!own) {
        write_tm8(blk, TM_AOS, c, t0, vp);
        write_cm8(blk, CM_AOS, c, t0, vp);
        write_cm8(blk, CM_VOH, c, t0, hp);
        write_tm8(blk, TM_VOH, c, t0, hp);
        write_tm8(blk, TM_VOT, c, t0, tp);
    } else {
        float rg[8];                     // 1/gate_t = prefix_{t-1} / prefix_t
        rg[0] = base * inv[0];
#pragma unroll
        for (int t = 1; t < 8; ++t) rg[t] = pre[t - 1] * inv[t];
        write_cm8(blk, CM_AS, c, t0, vp);
        write_cm8(blk, CM_VH, c, t0, hp);
        write_cm8(blk, CM_VT, c, t0, tp);
        write_cf8(blk, F_RG, c, t0, rg);
        write_cf8(blk, F_IP, c, t0, inv);
        if (want_pp) write_cf8(blk, F_PP, c, t0, pre);
    }
}

template <typename IOE, typename OPE, int NB, bool HEADS>
__device__ __forceinline__ void pair_prep_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b,
                                                int side) {
    const int pw = __builtin_amdgcn_readfirstlane(tid >> 6), c = tid & 63;
    // (block of the pair, own / other side, token half); each SIMD gets an own-side and an other-side wave
    const int jb = (pw >> 1) & 1, own = pw & 1, h = pw >> 2;
    const int T = (int)p.T;                              // the launcher admits T * heads < 2^24 only
    const int64_t row_off = row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N;
    const u16 *const x = reinterpret_cast<const u16 *>(p.x) + row_off, *const f = reinterpret_cast<const u16 *>(p.f) + row_off;
    const u16 *const g = reinterpret_cast<const u16 *>(p.g_out) + row_off, *const k = reinterpret_cast<const u16 *>(p.k) + row_off;
    const u16 *const fk = reinterpret_cast<const u16 *>(p.f_key) + row_off, *const q = reinterpret_cast<const u16 *>(p.q) + row_off;
    // this wave's side of the state: value side = (x, f, g_out), key side = (k, f_key, q)
    const bool value_side = (side == 0) == (own == 1);
    const u16 *const gate = value_side ? f : fk, *const val = value_side ? x : k, *const adj = value_side ? g : q;
    const PairSchedule<NB> sched(p.T, p.NC, p.C);
    TokenMap<HEADS> tmap(HEADS ? (u32)p.heads * CH_N : (u32)CH_N, h, c);
    const u32 ts = tmap.ts;                              // elements between consecutive tokens
    u32 bad = 0;
    PHASE_BEGIN();

    // Raw inputs of stage st (clamped to the last stage: that stage again, never used) -> registers.
    // ANY: the block may reach past the end of the sequence or lie past it (last chunk only); the
    // loads then go through clamped per-token addresses, which is correct for every block but slow.
    auto issue = [&](RawSet &r, int st, auto any_c) {
        int tok;
        bool bmode;
        sched.at(min(st, sched.total - 1), tok, bmode);
        tok += jb * CH_L;                                // this wave's block of the pair
        if constexpr (decltype(any_c)::value)
            raw_issue_tail(r, gate, val, adj, tok + 8 * h, tok + 8 * (1 - h), T, 2u * (u32)c, ts);
        else
            raw_issue<HEADS>(r, gate + (u32)tok * ts, val + (u32)tok * ts, adj + (u32)tok * ts, tmap);
    };
    // builds this wave's tiles of stage s from r, which then takes the raw inputs of stage s + 2
    auto prepare = [&](RawSet &r, int s, auto any_c) {
        constexpr bool ANY = decltype(any_c)::value;
        int tok;
        bool bmode;
        sched.at(s, tok, bmode);
        tok += jb * CH_L;
        const RawF fl = raw_take<IOE, ANY>(r, tok + 8 * h, tok + 8 * (1 - h), T);
        // The loads that refill r must come after the conversions above, or they need registers (and
        // a wait) of their own: tie their addresses to the converted values.
        asm volatile(""
                     : "+v"(tmap.voff_own), "+v"(tmap.voff_oth)
                     : "v"(fl.gown[0]), "v"(fl.gown[1]), "v"(fl.gown[2]), "v"(fl.gown[3]), "v"(fl.gown[4]), "v"(fl.gown[5]),
                       "v"(fl.gown[6]), "v"(fl.gown[7]), "v"(fl.val[0]), "v"(fl.val[1]), "v"(fl.val[2]), "v"(fl.val[3]),
                       "v"(fl.val[4]), "v"(fl.val[5]), "v"(fl.val[6]), "v"(fl.val[7]), "v"(fl.poth), "v"(fl.bad));
        asm volatile(""
                     : "+v"(tmap.voff_own), "+v"(tmap.voff_oth)
                     : "v"(fl.adj[0]), "v"(fl.adj[1]), "v"(fl.adj[2]), "v"(fl.adj[3]), "v"(fl.adj[4]), "v"(fl.adj[5]),
                       "v"(fl.adj[6]), "v"(fl.adj[7]));
        if constexpr (HEADS) {
#pragma unroll
            for (int t = 0; t < 8; ++t) asm volatile("" : "+v"(tmap.tok_off[t]) : "v"(tmap.voff_own));
        }
        issue(r, s + 2, any_c);
        prep_lane<OPE>(fl, smem + (s & 1) * STAGE_BYTES + jb * BLOCK_BYTES, bmode, own, h, c, side == 1, bad);
        PHASE_MARK(bmode ? 2 : 0);
        __syncthreads();
        PHASE_MARK(bmode ? 3 : 1);
    };

    // The stages of every chunk come in pairs (as many R as B stages), so the two register sets
    // simply alternate and the order of the loads in flight is the same on every path.  The stages
    // of the last chunk (first in this order), whose blocks may be partial or missing, and the two
    // refills they issue go through the general loader; everything after that is full blocks.
    RawSet setA, setB;
    issue(setA, 0, std::true_type{});
    issue(setB, 1, std::true_type{});
    int s = 0;
    for (; s < sched.n_last; s += 2) {
        prepare(setA, s, std::true_type{});
        prepare(setB, s + 1, std::true_type{});
    }
    for (; s < sched.total; s += 2) {
        prepare(setA, s, std::false_type{});
        prepare(setB, s + 1, std::false_type{});
    }
    // Both workgroups of a row see all four gates' blocks and reach the same verdict, so either
    // order of their writes leaves the same flag.
    if (bad) p.row_flags[b] = 1;
    PHASE_END(4 + (tid >> 6));
}

template <typename IOE, typename OPE, int NB, bool HEADS, int SIDE>
__device__ __forceinline__ void pair_matrix_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b) {
    constexpr int side = SIDE;
    const int w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int ch = 16 * w + r;       // this lane's own-side channel
    const int T = (int)p.T;                              // the launcher admits T * heads < 2^24 only
    const int64_t NC = p.NC;
    const int C = p.C;
    const u16 *ckpt = reinterpret_cast<const u16 *>(p.ckpt) + b * NC * (CH_N * CH_N);
    const int nb_last = (int)((p.T - (NC - 1) * C + CH_L - 1) / CH_L);
    const int64_t row_off = row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N;
    const u32 ts = HEADS ? (u32)p.heads * CH_N : (u32)CH_N;       // elements between consecutive tokens
    u16 *const d_val = reinterpret_cast<u16 *>(side == 0 ? p.d_x : p.d_k) + row_off;
    u16 *const d_gate = reinterpret_cast<u16 *>(side == 0 ? p.d_f : p.d_f_key) + row_off;
    u16 *const d_adj = reinterpret_cast<u16 *>(p.d_q) + row_off;

    // S[j][i], G[j][i]: own channel ch, other channel 16j + 4g + i
    floatx4 S[4], G[4];
    uint4 sv[NB][2];                  // block-start states as 16-bit MFMA operands (other channels 0..31, 32..63)
    uint2 pf[4];                      // checkpoint prefetch, packed I/O type
    // memory is [d][k]: side 0 reads 4 adjacent k of row d = ch, side 1 gathers column k = ch
    auto load_state = [&](const u16 *m, uint2 (&dst)[4]) {
        if (side == 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) dst[j] = ld2(m + ch * CH_N + 16 * j + 4 * g);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u16 *col = m + (16 * j + 4 * g) * CH_N + ch;
                dst[j] = make_uint2((u32)col[0] | ((u32)col[CH_N] << 16), (u32)col[2 * CH_N] | ((u32)col[3 * CH_N] << 16));
            }
        }
    };
    auto take_state = [&](const uint2 (&src)[4], floatx4 (&dst)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float t[4];
            unpack4<IOE>(src[j], t);
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[j][i] = t[i];
        }
    };
    load_state(reinterpret_cast<const u16 *>(p.g_state) + b * (CH_N * CH_N), pf);
    take_state(pf, G);
    load_state(ckpt + (NC - 1) * (CH_N * CH_N), pf);
    float carry = 0.f;
    int s = 0;
    if (tid == 0) {      // both flag slots of the row (the backward kernels report in the first)
        p.row_flags[b] = 0;
        p.row_flags[chunk_rows_padded(p.B) + b] = 0;
    }
    PHASE_BEGIN();

    // every stage starts with the workgroup barrier that publishes its operand tiles
    for (int64_t chunk = NC - 1; chunk >= 0; --chunk) {
        const int nb = chunk == NC - 1 ? nb_last : NB;
        take_state(pf, S);
        if (chunk > 0) load_state(ckpt + (chunk - 1) * (CH_N * CH_N), pf);
        // ---- R stages: block-start states, forward in time
#pragma unroll
        for (int i2 = 0; i2 < NB; i2 += 2) {
            if (i2 < nb) {
                __syncthreads();
                PHASE_MARK(3);
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) {
                    const int i = i2 + jb;
                    if (i < nb) {
                        const unsigned char *blk = stage + jb * BLOCK_BYTES;
                        const u16 *VOHc = reinterpret_cast<const u16 *>(blk + OFF_CM + CM_VOH * CM_TILE);
                        const u16 *VHc = reinterpret_cast<const u16 *>(blk + OFF_CM + CM_VH * CM_TILE);
                        const float *LX = lv_vec(blk, 0), *LO = lv_vec(blk, 1);
                        {
                            const uint2 a0 = pack4v<OPE>(S[0]), a1 = pack4v<OPE>(S[1]), a2 = pack4v<OPE>(S[2]),
                                        a3 = pack4v<OPE>(S[3]);
                            sv[i][0] = cat(a0, a1);
                            sv[i][1] = cat(a2, a3);
                        }
                        const float lo = LO[ch];
                        const uint2 vhc = ld2(VHc + ch * CC + 4 * g);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float4 lx = *reinterpret_cast<const float4 *>(LX + 16 * j + 4 * g);
                            S[j][0] *= lo * lx.x; S[j][1] *= lo * lx.y; S[j][2] *= lo * lx.z; S[j][3] *= lo * lx.w;
                            S[j] = OPE::mfma16(ld2(VOHc + (16 * j + r) * CC + 4 * g), vhc, S[j]);
                        }
                    }
                }
                PHASE_MARK(0);
                ++s;
            }
        }
        // ---- re-anchor the running sum of the gate gradient: sum over the other side of Gb * S_end
        {
            float us = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) us += G[j][i] * S[j][i];
            carry = row_sums(us).all;
        }
        // ---- B stages: pairs last to first, inside a pair the later block first
#pragma unroll
        for (int i2 = NB - 2; i2 >= 0; i2 -= 2) {
            if (i2 < nb) {
                __syncthreads();
                PHASE_MARK(2);
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
#pragma unroll
                for (int jb = 1; jb >= 0; --jb) {
                    const int i = i2 + jb;
                    if (i < nb) {
                        const unsigned char *blk = stage + jb * BLOCK_BYTES;
                        const u16 *AOS = reinterpret_cast<const u16 *>(blk + OFF_TM + TM_AOS * TM_TILE);
                        const u16 *VOT = reinterpret_cast<const u16 *>(blk + OFF_TM + TM_VOT * TM_TILE);
                        const u16 *VOH = reinterpret_cast<const u16 *>(blk + OFF_TM + TM_VOH * TM_TILE);
                        const u16 *AOSc = reinterpret_cast<const u16 *>(blk + OFF_CM + CM_AOS * CM_TILE);
                        const u16 *ASc = reinterpret_cast<const u16 *>(blk + OFF_CM + CM_AS * CM_TILE);
                        const u16 *VTc = reinterpret_cast<const u16 *>(blk + OFF_CM + CM_VT * CM_TILE);
                        const float *LX = lv_vec(blk, 0), *LO = lv_vec(blk, 1);
                        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                        const uint4 sb0 = sv[i][0], sb1 = sv[i][1];      // the state at the start of this block
                        // the 16x16 token-token product, in both orientations (full contraction over 64 channels)
                        const int ro = r * TS + 8 * g;
                        const uint4 vot_lo = ld4(VOT + ro), vot_hi = ld4(VOT + ro + 32);
                        const uint4 aos_lo = ld4(AOS + ro), aos_hi = ld4(AOS + ro + 32);
                        floatx4 pt1 = OPE::mfma32(vot_hi, aos_hi, OPE::mfma32(vot_lo, aos_lo, zero));   // P[t=r][s=4g+i]
                        floatx4 pt2 = OPE::mfma32(aos_hi, vot_hi, OPE::mfma32(aos_lo, vot_lo, zero));   // P[r'=4g+i][t=r]
                        float pd[4];     // diagonal for this lane's tokens 4g+i
        #pragma unroll
                        for (int ii = 0; ii < 4; ++ii) pd[ii] = __shfl(pt1[ii], 20 * g + ii, 64);
        #pragma unroll
                        for (int ii = 0; ii < 4; ++ii) {
                            pt1[ii] = (4 * g + ii < r) ? pt1[ii] : 0.f;
                            pt2[ii] = (4 * g + ii > r) ? pt2[ii] : 0.f;
                        }
                        const uint2 pa_o = pack4v<OPE>(pt1), pa_v = pack4v<OPE>(pt2);
                        const uint2 vtc = ld2(VTc + ch * CC + 4 * g), asc = ld2(ASc + ch * CC + 4 * g);
                        const float lo = LO[ch];
                        const int po = r * TS + 16 * g;
                        // o' uses the block-start state
                        floatx4 oa = OPE::mfma32(ld4(AOS + po + 8), sb1, OPE::mfma32(ld4(AOS + po), sb0, zero));
                        oa += OPE::mfma16(pa_o, vtc, zero);
                        // v' uses the adjoint entering the block, scaled to the block end on the own side
                        floatx4 ga[4];
        #pragma unroll
                        for (int j = 0; j < 4; ++j) ga[j] = G[j] * lo;
                        const uint4 gp0 = cat(pack4v<OPE>(ga[0]), pack4v<OPE>(ga[1]));
                        const uint4 gp1 = cat(pack4v<OPE>(ga[2]), pack4v<OPE>(ga[3]));
                        floatx4 va = OPE::mfma32(ld4(VOH + po + 8), gp1, OPE::mfma32(ld4(VOH + po), gp0, zero));
                        va += OPE::mfma16(pa_v, asc, zero);
                        // adjoint of the previous block
        #pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float4 lx = *reinterpret_cast<const float4 *>(LX + 16 * j + 4 * g);
                            ga[j][0] *= lx.x; ga[j][1] *= lx.y; ga[j][2] *= lx.z; ga[j][3] *= lx.w;
                            G[j] = OPE::mfma16(ld2(AOSc + (16 * j + r) * CC + 4 * g), asc, ga[j]);
                        }
                        // ---- gradients for tokens 4g+i, channel ch
                        {
                            float asv[4], vtv[4], du[4];
                            unpack4<OPE>(asc, asv);
                            unpack4<OPE>(vtc, vtv);
        #pragma unroll
                            for (int ii = 0; ii < 4; ++ii) du[ii] = oa[ii] * asv[ii] - va[ii] * vtv[ii];
                            reverse_running_sum_swap(du, carry, g);
                            const float *cf = reinterpret_cast<const float *>(blk + OFF_CF) + ch * CC + 4 * g;
                            const float4 rg = *reinterpret_cast<const float4 *>(cf + F_RG * (CF_TILE / 4));
                            const float4 ip = *reinterpret_cast<const float4 *>(cf + F_IP * (CF_TILE / 4));
                            const float rgv[4] = {rg.x, rg.y, rg.z, rg.w}, ipv[4] = {ip.x, ip.y, ip.z, ip.w};
                            // 16 lanes write 32 contiguous bytes of a token row; the four waves complete the row.
                            // Only the last block of the sequence can reach past its end.
                            const int tg = (int)chunk * C + i * CH_L + 4 * g;         // this lane's first token
                            const u32 go = (u32)tg * ts + (u32)ch;
                            float ppv[4] = {0.f, 0.f, 0.f, 0.f};
                            if (side == 1) {
                                const float4 pp = *reinterpret_cast<const float4 *>(cf + F_PP * (CF_TILE / 4));
                                ppv[0] = pp.x; ppv[1] = pp.y; ppv[2] = pp.z; ppv[3] = pp.w;
                            }
                            // one address per array; the four tokens are immediate offsets from it (folded rows)
                            u16 *const pv = d_val + go, *const pg = d_gate + go, *const pa = d_adj + go;
                            auto store = [&](int ii) {
                                pv[ii * ts] = cvt1<IOE>(ipv[ii] * (va[ii] + asv[ii] * pd[ii]));
                                pg[ii * ts] = cvt1<IOE>(du[ii] * rgv[ii]);
                                if (side == 1) pa[ii * ts] = cvt1<IOE>(ppv[ii] * (oa[ii] + vtv[ii] * pd[ii]));
                            };
                            if ((int)chunk * C + (i + 1) * CH_L <= T) {
        #pragma unroll
                                for (int ii = 0; ii < 4; ++ii) store(ii);
                            } else {
        #pragma unroll
                                for (int ii = 0; ii < 4; ++ii)
                                    if (tg + ii < T) store(ii);
                            }
                        }
                    }
                }
                PHASE_MARK(1);
                ++s;
            }
        }
    }
    // d_s0 = adjoint after the first block (value side only: rows of [d][k] are contiguous there)
    if (side == 0) {
        u16 *ds = reinterpret_cast<u16 *>(p.d_s0) + b * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint2 *>(ds + ch * CH_N + 16 * j + 4 * g) = pack4v<IOE>(G[j]);
    }
    PHASE_END(tid >> 6);
}

template <typename IOE, typename OPE, int NB, bool HEADS>
__global__ __launch_bounds__(PB_THREADS) void lfw_bwd_pair_kernel(ChunkBwdArgs p, int rows_padded) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    // blockIdx = side * rows_padded + row with rows_padded a multiple of 8: the two workgroups of a
    // row land on the same XCD and share its L2 for the inputs both of them read
    const int side = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - side * rows_padded;
    if (b >= p.B) return;
    // both branches execute one workgroup barrier per stage
    if (tid < 256) {
        if (side == 0)
            pair_matrix_waves<IOE, OPE, NB, HEADS, 0>(p, smem, tid, b);
        else
            pair_matrix_waves<IOE, OPE, NB, HEADS, 1>(p, smem, tid, b);
    } else {
        pair_prep_waves<IOE, OPE, NB, HEADS>(p, smem, tid - 256, b, side);
    }
}

template <typename IOE, typename OPE, int NB, bool HEADS> int launch(const ChunkBwdArgs &a, hipStream_t stream) {
    auto kern = lfw_bwd_pair_kernel<IOE, OPE, NB, HEADS>;
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, PB_SMEM),
                       "hipFuncSetAttribute(backward pair kernel)");
    if (rc) return rc;
    if (a.B > 0x1fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    if (a.heads < 1 || a.T * a.heads >= CHUNK_MAX_T)
        return fail(T2FW_ERR_UNSUPPORTED, "T=%lld with %d heads is too long for 32-bit row offsets", (long long)a.T, a.heads);
    const int rows_padded = (int)((a.B + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(2u * (unsigned)rows_padded), dim3(PB_THREADS), PB_SMEM, stream, a, rows_padded);
    return check_hip(hipGetLastError(), "lfw_bwd_pair_kernel launch");
}

template <typename IOE, typename OPE> int by_nb(const ChunkBwdArgs &a, hipStream_t stream) {
    if (a.C == 64) return a.heads == 1 ? launch<IOE, OPE, 4, false>(a, stream) : launch<IOE, OPE, 4, true>(a, stream);
    if (a.C == 32) return a.heads == 1 ? launch<IOE, OPE, 2, false>(a, stream) : launch<IOE, OPE, 2, true>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the pair-stage backward kernel takes checkpoint intervals 32 or 64");
}

}  // namespace

int chunk_backward_pair(const ChunkBwdArgs &a, int dtype, int op, hipStream_t stream) {
    if (dtype == T2FW_F16) return op == 1 ? by_nb<Fp16, Fp16>(a, stream) : by_nb<Fp16, Bf16>(a, stream);
    if (dtype == T2FW_BF16) return by_nb<Bf16, Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
