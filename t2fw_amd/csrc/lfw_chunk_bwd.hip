// Backward pass of the decay rule in chunked matrix-core form (block algebra: lfw_chunk.hpp),
// two workgroups per batch row.
//
// With G = dL/dS flowing backwards in time, Gb the adjoint entering a 16-step block from the
// future, S0 the state at the block start and the block-local scalings of lfw_chunk.hpp
// (qs, kt, kh, xt, xh, gs = g*a_t):
//   P[t,s] = qs_t.kt_s      W[t,s] = gs_t.xt_s
//   o'_t  = a_t  * ( S0 qs_t            + sum_{s<t} P[t,s] xt_s )       (output without its own write)
//   dq'_t = b_t  * ( S0^T gs_t          + sum_{s<t} W[t,s] kt_s )
//   dx'_t = 1/a_t* ( (a_L*Gb) kh_t      + sum_{r>t} P[r,t] gs_r )
//   dk'_t = 1/b_t* ( (b_L*Gb)^T xh_t    + sum_{r>t} W[r,t] qs_r )
//   dx_t = dx'_t + g_t P[t,t]   dq_t = dq'_t + k_t W[t,t]   dk_t = dk'_t + q_t W[t,t]
//   f_t*df_t   = u_t,  u_t = u_{t+1} + g_t.o'_t  - x_t.dx'_t   (elementwise; reverse running sum)
//   fk_t*dfk_t = v_t,  v_t = v_{t+1} + q_t.dq'_t - k_t.dk'_t
//   Gb_prev = (a_L (x) b_L)*Gb + sum_t gs_t (x) qs_t
// u and v are re-anchored at every checkpoint boundary from the states themselves
// (u = rowsum(Gb*S_end), v = colsum(Gb*S_end)), so rounding does not accumulate over T.
//
// The recurrence is symmetric under (x, f, g_out, D) <-> (k, f_key, q, K) with the state
// transposed, so the two sides get a workgroup (and a CU) each and nothing is exchanged:
//   side 0 ("value side"): own = (x, f, g_out), other = (k, f_key, q); writes d_x, d_f, d_s0
//   side 1 ("key side")  : own = (k, f_key, q), other = (x, f, g_out); writes d_k, d_f_key, d_q
// In the names below V = own value (x | k), A = own adjoint (g_out | q), VO / AO the other
// side's, a suffix S / T / H = scaled by the gate prefix / divided by it / scaled by the
// gate suffix (qs, kt, kh ... above).  With own channel c, other channel e:
//   P[t,s]  = AOS_t . VOT_s                                         (contraction over e)
//   o'_t[c] = sum_e S0[c,e] AOS_t[e] + sum_{s<t} P[t,s] VT_s[c]
//   v'_t[c] = sum_e (L_own[c] Gb[c,e]) VOH_t[e] + sum_{r>t} P[r,t] AS_r[c]
//   d_own_gate_t = RG_t * (carry + sum_{r>=t} o'_r AS_r - v'_r VT_r)
//   d_V_t = IP_t * (v'_t + AS_t P[t,t])        d_A_t = PP_t * (o'_t + VT_t P[t,t])   (side 1 only)
//   Gb <- L_own[c] L_other[e] Gb[c,e] + sum_t AS_t[c] AOS_t[e]
//
// A workgroup has 12 waves.  Matrix wave w (of 4) holds, in fp32 accumulators, the slab of S and
// of Gb for own channels 16w..16w+15 (all other channels), so that every contraction is local to
// a wave.  Chunks (one per checkpoint) are visited last to first.  A chunk needs a forward sweep
// over its blocks ("R" work: the block-start states, recomputed from the checkpoint and kept as
// 16-bit MFMA operands in registers) before its blocks can be visited last to first ("B" work:
// gradients and the adjoint).  R work is light for the matrix waves and heavy for the prep waves, B
// work the other way round, and with one workgroup barrier per stage a stage is as long as the
// slower of the two; so a stage here carries the B work of a pair of blocks of chunk c AND the R
// work of a pair of blocks of chunk c - 1, which no dependence forbids (R needs only the checkpoint):
//   prologue     R pairs of the last chunk
//   transition   c -> c - 1, for k = 0 .. NB/2 - 1:  B pair NB/2 - 1 - k of chunk c, R pair k of chunk c - 1
//   epilogue     B pairs of chunk 0
// The states recomputed for chunk c - 1 go to the registers of the pair of chunk c that the same
// stage has just finished with (the two pairs are swapped into place after the transition).
//
// Eight prep waves build the operand tiles of the next stage in double-buffered LDS: (block of the
// pair, own / other side, token half) for the B and for the R part.  In the B part one lane builds
// the prefix-scaled AND the suffix-scaled operands of its side from one set of gate conversions and
// one 16-step product.  Raw inputs go from global memory straight to registers, one set per part,
// refilled in place one stage ahead after their contents have been converted (the refill's address
// depends on the converted values, so the compiler cannot hoist the loads above the conversions);
// the matrix waves store the gradients themselves.
//
// Replaces lfw_cuda_bwd_kernel and the six einsums of the reference
// (t2fw/csrc/lfw_kernel.cu:61-102, t2fw/csrc/lfw.cpp:84-93).
#include <type_traits>

#include "lfw_chunk_bwd_dev.hpp"
#include "lfw_scan_body.hpp"

namespace t2fw {
namespace {

using namespace bwd;

constexpr int BW_THREADS = 768;
constexpr int CC = 20;   // channel-major 16-token tiles: row stride in elements

// ---- LDS layout: a stage buffer holds the B tiles of two blocks, then the R tiles of two blocks -----
constexpr int TM_TILE = CH_L * TS * 2;       // token-major 16-bit tile [16][TS], channels permuted (tm_pos)
constexpr int CM_TILE = CH_N * CC * 2;       // channel-major 16-bit tile [64][CC]
constexpr int CF_TILE = CH_N * CC * 4;       // channel-major fp32 tile [64][CC]
enum { TM_AOS = 0, TM_VOT, TM_VOH, TM_NUM };
enum { CM_AOS = 0, CM_VOH, CM_AS, CM_VT, CM_VH, CM_NUM };
enum { F_RG = 0, F_IP, F_NUM };              // 1/own gate, 1/own prefix (the prefix itself is its reciprocal)
constexpr int OFF_TM = 0;
constexpr int OFF_CM = OFF_TM + TM_NUM * TM_TILE;
constexpr int OFF_CF = OFF_CM + CM_NUM * CM_TILE;
constexpr int OFF_LV = OFF_CF + F_NUM * CF_TILE;      // 16-step gate products [other side, own side][64] f32
constexpr int BLOCK_BYTES = OFF_LV + 2 * CH_N * 4;
// R tiles of one block: VOH, VH (channel-major) and the gate products
constexpr int ROFF_VOH = 0, ROFF_VH = CM_TILE, ROFF_LV = 2 * CM_TILE;
constexpr int RBLOCK_BYTES = ROFF_LV + 2 * CH_N * 4;
constexpr int OFF_RPART = 2 * BLOCK_BYTES;
constexpr int STAGE_BYTES = OFF_RPART + 2 * RBLOCK_BYTES;
// after the two stage buffers: per matrix wave, room to park its fp32 state slab (64 lanes x 16 floats)
// while the B part of a stage needs the registers
constexpr int OFF_PARK = 2 * STAGE_BYTES;
constexpr int OFF_VERDICT = OFF_PARK + 4 * 64 * 16 * 4;      // one int: a prep wave of this workgroup flagged the row
constexpr int BW_SMEM = OFF_VERDICT + 16;
static_assert(BW_SMEM <= 160 * 1024, "backward stage buffers exceed the LDS of one CU");
static_assert(BLOCK_BYTES % 16 == 0 && RBLOCK_BYTES % 16 == 0, "tile regions must keep 16-byte alignment");

// ---- stage schedule ----------------------------------------------------------------------
// The last chunk of a sequence may have fewer pairs of blocks than a full one, its last pair one
// block, its last block fewer than 16 tokens.
template <int NB> struct StageSchedule {
    static constexpr int MP = NB / 2;                    // pairs of a full chunk
    int NC, C, nb_last, m_last, m0, n_trans, total;
    __device__ StageSchedule(int64_t T, int64_t NC_, int C_) {
        NC = (int)NC_;
        C = C_;
        const int len_last = (int)(T - (NC_ - 1) * C_);
        nb_last = (len_last + CH_L - 1) / CH_L;
        m_last = (nb_last + 1) / 2;
        m0 = NC == 1 ? m_last : MP;                      // pairs of chunk 0
        n_trans = (NC - 1) * MP;
        total = m_last + n_trans + m0;
    }
    // stage s -> first tokens of the pairs of blocks of its B and R parts (wave-uniform)
    struct Desc {
        int tok_b, tok_r;
        bool has_b, has_r;
    };
    __device__ Desc at(int s) const {
        Desc d;
        d.tok_b = 0;
        d.tok_r = 0;
        if (s < m_last) {
            d.has_b = false;
            d.has_r = true;
            d.tok_r = (NC - 1) * C + s * 2 * CH_L;
        } else if (s - m_last < n_trans) {
            const unsigned s2 = (unsigned)(s - m_last);
            const int c = NC - 1 - (int)(s2 / (unsigned)MP), k = (int)(s2 % (unsigned)MP), pb = MP - 1 - k;
            d.has_b = 2 * pb < (c == NC - 1 ? nb_last : NB);
            d.tok_b = c * C + pb * 2 * CH_L;
            d.has_r = true;
            d.tok_r = (c - 1) * C + k * 2 * CH_L;
        } else {
            const int k = s - m_last - n_trans;
            d.has_b = true;
            d.has_r = false;
            d.tok_b = (m0 - 1 - k) * 2 * CH_L;
        }
        return d;
    }
};

// ---- raw inputs --------------------------------------------------------------------------
// A prep lane works on one channel and eight tokens of one block; it needs the gate at those
// tokens and at the block's other eight, the value array of its side at its own tokens and, for the
// B part (ADJ), the adjoint array as well.
struct RawSet {
    u16 gown[8], goth[8], val[8], adj[8];
};
struct RawF {
    float gown[8], val[8], adj[8], poth;
    u32 bad;
};

// Where the sixteen tokens of a block are, seen from a prep lane.  Consecutive tokens are ts elements
// apart.  HEADS = false: ts = 64; the token half and the channel make up a constant vector offset
// (voff_own / voff_oth), the token inside the half is an immediate one.  HEADS = true: ts is a
// run-time multiple of 64; the token half moves the scalar base (shift_own / shift_oth elements) and
// tok_off[t] = 2 * (channel + t * ts) is the vector offset of token t of a half.
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
template <bool HEADS, bool ADJ>
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
        if constexpr (ADJ) {
#pragma unroll
            for (int t = 0; t < 8; ++t) r.adj[t] = at(adj, m.voff_own, t);
        }
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
        if constexpr (ADJ) {
#pragma unroll
            for (int t = 0; t < 8; ++t) r.adj[t] = at(ao, t);
        }
    }
}

// The same for a block that reaches past the end of the sequence (or lies past it): tokens past the
// end are read from the last one, with the same number of loads, and replaced when the set is taken.
// row_*: token 0 of the batch row.
template <bool ADJ>
__device__ __forceinline__ void raw_issue_any(RawSet &r, const u16 *row_gate, const u16 *row_val, const u16 *row_adj,
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
    if constexpr (ADJ) {
#pragma unroll
        for (int t = 0; t < 8; ++t) r.adj[t] = at(row_adj, tok_own + t);
    }
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
// other half's gates.  ANY: tokens at or past T act as identity (gate 1, everything else 0).
template <typename IOE, bool ANY, bool ADJ>
__device__ __forceinline__ RawF raw_take(const RawSet &r, int tok_own, int tok_oth, int T) {
    RawF f;
    // the loads complete in order: one wait for the last of them covers the whole set
    if constexpr (ADJ)
        asm volatile("" ::"v"(r.adj[7]));
    else
        asm volatile("" ::"v"(r.val[7]));
    float po = 1.0f;
    u16 mx = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const bool own = !ANY || tok_own + t < T;
        const u16 m1 = own ? (u16)(r.gown[t] - 1) : (u16)0;      // 0 < bits <= bits(1.0)
        mx = m1 > mx ? m1 : mx;
        f.gown[t] = own ? IOE::to_f32(r.gown[t]) : 1.0f;
        f.val[t] = own ? IOE::to_f32(r.val[t]) : 0.0f;
        if constexpr (ADJ) f.adj[t] = own ? IOE::to_f32(r.adj[t]) : 0.0f;
        if (!ANY || tok_oth + t < T) po *= IOE::to_f32(r.goth[t]);
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

// Gate scalings of one half block (tokens 8h..8h+7) of one channel: pre = prod_{r<=t} gate_r from the
// block start, inv = 1 / pre, hat = v * prod_{r>t} gate_r (scaled to the block end), til = hat / total
// (scaled to the block start); returns the 16-step product.
template <typename OPE>
__device__ __forceinline__ float scale_half(const RawF &f, int h, float (&pre)[8], float (&hat)[8], float (&til)[8],
                                            float (&inv)[8], u32 &bad) {
    float run = h ? f.poth : 1.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        run *= f.gown[t];
        pre[t] = run;
    }
    const float tot = h ? run : run * f.poth;
    bad |= (tot >= OPE::MIN_PRODUCT) ? 0u : 1u;
    const float itot = __builtin_amdgcn_rcpf(tot);
    float sfx = h ? 1.0f : f.poth;
#pragma unroll
    for (int t = 7; t >= 0; --t) {
        inv[t] = sfx * itot;
        hat[t] = f.val[t] * sfx;
        til[t] = hat[t] * itot;
        sfx *= f.gown[t];
    }
    return tot;
}

// R part, one prep lane (tokens 8h..8h+7 of one block, channel c, own or other side): the
// suffix-scaled values (VH | VOH, channel-major) and the 16-step gate product.
template <typename OPE>
__device__ __forceinline__ void prep_lane_r(const RawF &f, unsigned char *rblk, int own, int h, int c, u32 &bad) {
    float pre[8], hat[8], til[8], inv[8];
    const float tot = scale_half<OPE>(f, h, pre, hat, til, inv, bad);
    if (h == 0) reinterpret_cast<float *>(rblk + ROFF_LV)[own * CH_N + c] = tot;
    const Packed8 hp = pack8<OPE>(hat);
    uint2 *cm = reinterpret_cast<uint2 *>(rblk + (own ? ROFF_VH : ROFF_VOH) + (c * CC + 8 * h) * 2);
    cm[0] = make_uint2(hp.p[0], hp.p[1]);
    cm[1] = make_uint2(hp.p[2], hp.p[3]);
}

// B part, one prep lane.
//   other side: AOS (token- and channel-major), VOH (both), VOT (token-major), L_other
//   own side  : AS, VH, VT (channel-major), 1/gate, 1/prefix, L_own
template <typename OPE>
__device__ __forceinline__ void prep_lane_b(const RawF &f, unsigned char *blk, int own, int h, int c, u32 &bad) {
    const int t0 = 8 * h;
    float pre[8], hat[8], til[8], inv[8];
    const float tot = scale_half<OPE>(f, h, pre, hat, til, inv, bad);
    bad |= f.bad;                        // every block's gates are range-checked in its B part
    if (h == 0) lv_vec(blk, own)[c] = tot;
    float v[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) v[t] = f.adj[t] * pre[t];
    const Packed8 vp = pack8<OPE>(v), hp = pack8<OPE>(hat), tp = pack8<OPE>(til);
    if (!own) {
        write_tm8(blk, TM_AOS, c, t0, vp);
        write_cm8(blk, CM_AOS, c, t0, vp);
        write_cm8(blk, CM_VOH, c, t0, hp);
        write_tm8(blk, TM_VOH, c, t0, hp);
        write_tm8(blk, TM_VOT, c, t0, tp);
    } else {
        float rg[8];                     // 1/gate_t = prefix_{t-1} / prefix_t
        rg[0] = (h ? f.poth : 1.0f) * inv[0];
#pragma unroll
        for (int t = 1; t < 8; ++t) rg[t] = pre[t - 1] * inv[t];
        write_cm8(blk, CM_AS, c, t0, vp);
        write_cm8(blk, CM_VH, c, t0, hp);
        write_cm8(blk, CM_VT, c, t0, tp);
        write_cf8(blk, F_RG, c, t0, rg);
        write_cf8(blk, F_IP, c, t0, inv);
    }
}

template <typename IOE, typename OPE, int NB, bool HEADS>
__device__ __forceinline__ void bwd_prep_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b,
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
    const StageSchedule<NB> sched(p.T, p.NC, p.C);
    TokenMap<HEADS> tmap(HEADS ? (u32)p.heads * CH_N : (u32)CH_N, h, c);
    const u32 ts = tmap.ts;                              // elements between consecutive tokens
    u32 bad = 0;

    // Raw inputs of a part of a stage -> registers; tok: first token of the part's pair of blocks.
    // ANY: the block may reach past the end of the sequence or lie past it; the loads then go through
    // clamped per-token addresses, which is correct for every block but slow.
    auto issue = [&](RawSet &r, int tok, auto any_c, auto adj_c) {
        constexpr bool ADJ = decltype(adj_c)::value;
        tok += jb * CH_L;                                // this wave's block of the pair
        if constexpr (decltype(any_c)::value)
            raw_issue_any<ADJ>(r, gate, val, adj, tok + 8 * h, tok + 8 * (1 - h), T, 2u * (u32)c, ts);
        else
            raw_issue<HEADS, ADJ>(r, gate + (u32)tok * ts, val + (u32)tok * ts, adj + (u32)tok * ts, tmap);
    };
    // The loads that refill a set must come after the conversion of its contents, or they need
    // registers (and a wait) of their own: their addresses are tied to the converted values.
    auto tie = [&](const RawF &fl, auto adj_c) {
        asm volatile(""
                     : "+v"(tmap.voff_own), "+v"(tmap.voff_oth)
                     : "v"(fl.gown[0]), "v"(fl.gown[1]), "v"(fl.gown[2]), "v"(fl.gown[3]), "v"(fl.gown[4]), "v"(fl.gown[5]),
                       "v"(fl.gown[6]), "v"(fl.gown[7]), "v"(fl.val[0]), "v"(fl.val[1]), "v"(fl.val[2]), "v"(fl.val[3]),
                       "v"(fl.val[4]), "v"(fl.val[5]), "v"(fl.val[6]), "v"(fl.val[7]), "v"(fl.poth), "v"(fl.bad));
        if constexpr (decltype(adj_c)::value) {
            asm volatile(""
                         : "+v"(tmap.voff_own), "+v"(tmap.voff_oth)
                         : "v"(fl.adj[0]), "v"(fl.adj[1]), "v"(fl.adj[2]), "v"(fl.adj[3]), "v"(fl.adj[4]), "v"(fl.adj[5]),
                           "v"(fl.adj[6]), "v"(fl.adj[7]));
        }
        if constexpr (HEADS) {
#pragma unroll
            for (int t = 0; t < 8; ++t) asm volatile("" : "+v"(tmap.tok_off[t]) : "v"(tmap.voff_own));
        }
    };
    // One stage: this wave's tiles of the B part from setB and of the R part from setR; each set takes
    // the raw inputs of the next stage as soon as its contents are converted.  A part that the stage
    // does not have still loads (from the start of the row): the number of loads in flight is the
    // same on every path, so the waits for them are exact.
    RawSet setB, setR;
    using Desc = typename StageSchedule<NB>::Desc;
    auto stage = [&](int s, const Desc cur, auto any_cur, auto any_next) {
        constexpr bool ANY = decltype(any_cur)::value;
        const Desc nxt = sched.at(min(s + 1, sched.total - 1));
        unsigned char *const buf = smem + (s & 1) * STAGE_BYTES;
        {
            const int tok = cur.tok_b + jb * CH_L;
            const RawF fl = raw_take<IOE, ANY, true>(setB, tok + 8 * h, tok + 8 * (1 - h), T);
            tie(fl, std::true_type{});
            issue(setB, nxt.tok_b, any_next, std::true_type{});
            if (cur.has_b) prep_lane_b<OPE>(fl, buf + jb * BLOCK_BYTES, own, h, c, bad);
        }
        {
            const int tok = cur.tok_r + jb * CH_L;
            const RawF fl = raw_take<IOE, ANY, false>(setR, tok + 8 * h, tok + 8 * (1 - h), T);
            tie(fl, std::false_type{});
            issue(setR, nxt.tok_r, any_next, std::false_type{});
            if (cur.has_r) prep_lane_r<OPE>(fl, buf + OFF_RPART + jb * RBLOCK_BYTES, own, h, c, bad);
        }
        __syncthreads();
    };
    // Blocks can be partial or missing only in the last chunk, i.e. in the prologue and the first
    // transition: those stages go through the general loader unless that chunk is full.  Parts that a
    // stage does not have load from the start of the row, which the fast loader may do as soon as the
    // row has more than one chunk (or one full one).
    const bool last_full = p.T % p.C == 0;
    const int n1 = last_full ? 0 : sched.m_last + min(sched.NC - 1, 1) * StageSchedule<NB>::MP;
    const int n2 = (sched.NC > 1 || last_full) ? sched.total : sched.m_last + sched.n_trans;
    {
        const Desc d0 = sched.at(0);
        if (n1 > 0) {
            issue(setB, d0.tok_b, std::true_type{}, std::true_type{});
            issue(setR, d0.tok_r, std::true_type{}, std::false_type{});
        } else {
            issue(setB, d0.tok_b, std::false_type{}, std::true_type{});
            issue(setR, d0.tok_r, std::false_type{}, std::false_type{});
        }
    }
    for (int s = 0; s < sched.total; ++s) {
        const Desc cur = sched.at(s);
        const bool any_cur = s < n1 || s >= n2, any_next = s + 1 < n1 || s + 1 >= n2;
        if (any_cur) {
            if (any_next)
                stage(s, cur, std::true_type{}, std::true_type{});
            else
                stage(s, cur, std::true_type{}, std::false_type{});
        } else {
            if (any_next)
                stage(s, cur, std::false_type{}, std::true_type{});
            else
                stage(s, cur, std::false_type{}, std::false_type{});
        }
    }
    // Both workgroups of a row see all four gates' blocks and reach the same verdict, so either
    // order of their writes leaves the same flag.
    if (bad) {
        p.row_flags[b] = 1;
        *reinterpret_cast<volatile int *>(smem + OFF_VERDICT) = 1;
    }
}

template <typename IOE, typename OPE, int NB, bool HEADS, int SIDE>
__device__ __forceinline__ void bwd_matrix_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b) {
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
    float chk = 0.f;         // 0 until a stored result is inf or NaN, then NaN
    int s = 0;
    if (tid == 0) {      // both flag slots of the row (the backward kernels report in the first)
        p.row_flags[b] = 0;
        p.row_flags[chunk_rows_padded(p.B) + b] = 0;
        *reinterpret_cast<volatile int *>(smem + OFF_VERDICT) = 0;      // published by the first stage's barrier
    }

    // R part of a stage: the states at the start of blocks i2 and i2 + 1 of a chunk with nbc blocks
    // (S runs forward over them), as MFMA operands into d0 and d1
    auto r_pair = [&](const unsigned char *stage, int nbc, int i2, uint4 (&d0)[2], uint4 (&d1)[2]) {
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
            if (i2 + jb < nbc) {
                const unsigned char *rblk = stage + OFF_RPART + jb * RBLOCK_BYTES;
                const u16 *VOHc = reinterpret_cast<const u16 *>(rblk + ROFF_VOH);
                const u16 *VHc = reinterpret_cast<const u16 *>(rblk + ROFF_VH);
                const float *LX = reinterpret_cast<const float *>(rblk + ROFF_LV), *LO = LX + CH_N;
                {
                    const uint2 a0 = pack4v<OPE>(S[0]), a1 = pack4v<OPE>(S[1]), a2 = pack4v<OPE>(S[2]),
                                a3 = pack4v<OPE>(S[3]);
                    uint4(&d)[2] = jb ? d1 : d0;
                    d[0] = cat(a0, a1);
                    d[1] = cat(a2, a3);
                }
                // (the index is made opaque so that the byte offset is formed here, from the channel, instead of
                // living in a register of its own across the stages: at this kernel's register limit that register
                // is spilled, and its reload after the gradient stores makes the wave wait for those stores)
                int ch_here = ch;
                asm volatile("" : "+v"(ch_here));
                const float lo = LO[ch_here];
                const uint2 vhc = ld2(VHc + ch * CC + 4 * g);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float4 lx = *reinterpret_cast<const float4 *>(LX + 16 * j + 4 * g);
                    S[j][0] *= lo * lx.x; S[j][1] *= lo * lx.y; S[j][2] *= lo * lx.z; S[j][3] *= lo * lx.w;
                    S[j] = OPE::mfma16(ld2(VOHc + (16 * j + r) * CC + 4 * g), vhc, S[j]);
                }
            }
        }
    };
    // B part of a stage: blocks i2 + 1 and i2 (in that order) of chunk `chunk`, which has nb blocks
    auto b_pair = [&](const unsigned char *stage, int64_t chunk, int nb, auto i2_c) {
        constexpr int i2 = decltype(i2_c)::value;
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
                // (the index is made opaque so that the byte offset is formed here, from the channel, instead of
                // living in a register of its own across the stages: at this kernel's register limit that register
                // is spilled, and its reload after the gradient stores makes the wave wait for those stores)
                int ch_here = ch;
                asm volatile("" : "+v"(ch_here));
                const float lo = LO[ch_here];
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
                    float ppv[4] = {0.f, 0.f, 0.f, 0.f};        // own prefix = 1 / (1 / prefix)
                    if (side == 1) {
#pragma unroll
                        for (int ii = 0; ii < 4; ++ii) ppv[ii] = __builtin_amdgcn_rcpf(ipv[ii]);
                    }
                    // one address per array; the four tokens are immediate offsets from it (folded rows)
                    u16 *const pv = d_val + go, *const pg = d_gate + go, *const pa = d_adj + go;
                    auto store = [&](int ii) {
                        const float rv = ipv[ii] * (va[ii] + asv[ii] * pd[ii]), rg = du[ii] * rgv[ii];
                        if constexpr (IOE::CHECK_RESULTS) chk = __builtin_fmaf(rv, 0.0f, __builtin_fmaf(rg, 0.0f, chk));
                        pv[ii * ts] = cvt1<IOE>(rv);
                        pg[ii * ts] = cvt1<IOE>(rg);
                        if (side == 1) {
                            const float ra = ppv[ii] * (oa[ii] + vtv[ii] * pd[ii]);
                            if constexpr (IOE::CHECK_RESULTS) chk = __builtin_fmaf(ra, 0.0f, chk);
                            pa[ii * ts] = cvt1<IOE>(ra);
                        }
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
    };
    // re-anchor the running sum of the gate gradient: sum over the other side of Gb * S_end
    auto anchor = [&]() {
        float us = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) us += G[j][i] * S[j][i];
        carry = row_sums(us).all;
    };
    constexpr int MP = NB / 2;

    // every stage starts with the workgroup barrier that publishes its operand tiles
    // ---- prologue: R pairs of the last chunk
    take_state(pf, S);
    if (NC > 1) load_state(ckpt + (NC - 2) * (CH_N * CH_N), pf);
#pragma unroll
    for (int k = 0; k < MP; ++k) {
        if (2 * k < nb_last) {
            __syncthreads();
            r_pair(smem + (s & 1) * STAGE_BYTES, nb_last, 2 * k, sv[2 * k], sv[2 * k + 1]);
            ++s;
        }
    }
    anchor();
    // ---- transitions: B pairs of chunk c, last to first, each with an R pair of chunk c - 1
    // (the running state S of the R work is kept out of the registers while a B part runs: as the raw
    // checkpoint before the chunk's first R pair, parked in LDS between its R pairs)
    float4 *const park = reinterpret_cast<float4 *>(smem + OFF_PARK) + tid * 4;
    for (int64_t chunk = NC - 1; chunk >= 1; --chunk) {
        const int nb = chunk == NC - 1 ? nb_last : NB;
        {
            __syncthreads();
            const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
            b_pair(stage, chunk, nb, std::integral_constant<int, NB - 2>{});
            take_state(pf, S);
            if (chunk > 1) load_state(ckpt + (chunk - 2) * (CH_N * CH_N), pf);
            // the registers of the pair just done take the first pair of the chunk below
            r_pair(stage, NB, 0, sv[NB - 2], sv[NB - 1]);
            if constexpr (MP == 2) {
#pragma unroll
                for (int j = 0; j < 4; ++j) park[j] = make_float4(S[j][0], S[j][1], S[j][2], S[j][3]);
            }
            ++s;
        }
        if constexpr (MP == 2) {
            __syncthreads();
            const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
            b_pair(stage, chunk, nb, std::integral_constant<int, 0>{});
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 v = park[j];
                S[j][0] = v.x; S[j][1] = v.y; S[j][2] = v.z; S[j][3] = v.w;
            }
            r_pair(stage, NB, 2, sv[0], sv[1]);
            ++s;
            // ... which leaves the two pairs in each other's place
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const uint4 t = sv[i][e];
                    sv[i][e] = sv[(i + 2) % NB][e];
                    sv[(i + 2) % NB][e] = t;
                }
        }
        anchor();
    }
    // ---- epilogue: B pairs of chunk 0
    {
        const int nb = NC == 1 ? nb_last : NB;
        if (NB - 2 < nb && MP == 2) {
            __syncthreads();
            b_pair(smem + (s & 1) * STAGE_BYTES, 0, nb, std::integral_constant<int, NB - 2>{});
            ++s;
        }
        {
            __syncthreads();
            b_pair(smem + (s & 1) * STAGE_BYTES, 0, nb, std::integral_constant<int, 0>{});
            ++s;
        }
    }
    // d_s0 = adjoint after the first block (value side only: rows of [d][k] are contiguous there)
    if (side == 0) {
        u16 *ds = reinterpret_cast<u16 *>(p.d_s0) + b * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint2 *>(ds + ch * CH_N + 16 * j + 4 * g) = pack4v<IOE>(G[j]);
    }
    // A result that is not finite (a scaled operand or a product of scaled operands left the range of its type)
    // hands this side of the row to the exact recurrence, like a gate outside the range does.
    if constexpr (IOE::CHECK_RESULTS) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) chk = __builtin_fmaf(G[j][i], 0.0f, chk);
    }
    if (!(chk == 0.0f)) {
        p.row_flags[b] = 1;
        *reinterpret_cast<volatile int *>(smem + OFF_VERDICT) = 1;
    }
}

template <typename IOE, typename OPE, int NB, bool HEADS>
__global__ __launch_bounds__(BW_THREADS) void lfw_bwd_chunk_kernel(ChunkBwdArgs p, int rows_padded) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    // blockIdx = side * rows_padded + row with rows_padded a multiple of 8: the two workgroups of a
    // row land on the same XCD and share its L2 for the inputs both of them read
    const int side = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - side * rows_padded;
    if (b >= p.B) return;
    if (p.row_select != nullptr && p.row_select[b] == 0) {      // not this kernel's row: nothing to redo after it either
        if (tid == 0) {
            p.row_flags[b] = 0;
            p.row_flags[rows_padded + b] = 0;
        }
        return;
    }
    // both branches execute one workgroup barrier per stage
    if (tid < 256) {
        if (side == 0)
            bwd_matrix_waves<IOE, OPE, NB, HEADS, 0>(p, smem, tid, b);
        else
            bwd_matrix_waves<IOE, OPE, NB, HEADS, 1>(p, smem, tid, b);
    } else {
        bwd_prep_waves<IOE, OPE, NB, HEADS>(p, smem, tid - 256, b, side);
    }
    // A barrier publishes the prep waves' verdict.  If the chunked form could not take the row, the first
    // SCAN_THREADS threads redo this workgroup's side of it with the exact scan, in place, and everyone
    // else leaves (a workgroup barrier only waits for the waves that are still there).  The scan body
    // needs more registers than this kernel's waves have: it spills here, which only such rows pay for.
    __syncthreads();
    if (tid >= SCAN_THREADS || !p.redo) return;
    if (*reinterpret_cast<volatile int *>(smem + OFF_VERDICT) == 0) return;
    ScanBwdArgs sa{};
    sa.g_out = p.g_out; sa.g_state = p.g_state; sa.x = p.x; sa.f = p.f; sa.q = p.q; sa.k = p.k; sa.f_key = p.f_key;
    sa.ckpt = p.ckpt;
    sa.d_x = p.d_x; sa.d_f = p.d_f; sa.d_q = p.d_q; sa.d_k = p.d_k; sa.d_f_key = p.d_f_key; sa.d_s0 = p.d_s0;
    sa.B = p.B; sa.T = p.T; sa.D = CH_N; sa.K = CH_N; sa.NC = p.NC;
    sa.C = p.C; sa.kg = p.scan_kg; sa.use_sub = 1; sa.ntiles = p.scan_ntiles; sa.heads = p.heads;
    for (int tile = 0; tile < p.scan_ntiles; ++tile) {
        __syncthreads();        // the stage buffers, or the tile before, are no longer read
        if (side == 0)
            scan::bwd_scan_body_kg<typename IOE::io_type, 4, 0, 16, 1>(sa, b, tile);
        else
            scan::bwd_scan_body_kg<typename IOE::io_type, 4, 1, 16, 1>(sa, b, tile);
    }
}

template <typename IOE, typename OPE, int NB, bool HEADS> int launch(const ChunkBwdArgs &a, hipStream_t stream) {
    auto kern = lfw_bwd_chunk_kernel<IOE, OPE, NB, HEADS>;
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    int rc = enable_lds(reinterpret_cast<const void *>(kern), BW_SMEM, "hipFuncSetAttribute(backward chunk kernel)");
    if (rc) return rc;
    if (a.B > 0x1fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    if (a.heads < 1 || a.T * a.heads >= CHUNK_MAX_T)
        return fail(T2FW_ERR_UNSUPPORTED, "T=%lld with %d heads is too long for 32-bit row offsets", (long long)a.T, a.heads);
    const int rows_padded = (int)((a.B + 7) / 8 * 8);
    ChunkBwdArgs a2 = a;
    {
        // the exact scan body for flagged rows: 16 lanes per state row, four columns per lane, the
        // segment-start states of a chunk in LDS (which this kernel's allocation holds with room to spare)
        const ScanGeom g = scan_geometry(CH_N);
        if (g.kg != 16 || g.kpl != 4) return fail(T2FW_ERR_UNSUPPORTED, "unexpected scan geometry for a 64 x 64 state");
        a2.scan_kg = g.kg;
        a2.scan_ntiles = (CH_N + g.rows - 1) / g.rows;
        // the body runs in this kernel's LDS, below the verdict word
        const size_t need = scan_bwd_lds_bytes(scan::SegLen<4>::value, g.kg, g.kpl, g.rows, a.C, true);
        if (need > (size_t)OFF_VERDICT)
            return fail(T2FW_ERR_UNSUPPORTED, "the exact scan body needs %zu bytes of LDS, the block-wise backward kernel has %d",
                        need, OFF_VERDICT);
    }
    hipLaunchKernelGGL(kern, dim3(2u * (unsigned)rows_padded), dim3(BW_THREADS), BW_SMEM, stream, a2, rows_padded);
    return check_hip(hipGetLastError(), "lfw_bwd_chunk_kernel launch");
}

template <typename IOE, typename OPE> int by_nb(const ChunkBwdArgs &a, hipStream_t stream) {
    if (a.C == 64) return a.heads == 1 ? launch<IOE, OPE, 4, false>(a, stream) : launch<IOE, OPE, 4, true>(a, stream);
    if (a.C == 32) return a.heads == 1 ? launch<IOE, OPE, 2, false>(a, stream) : launch<IOE, OPE, 2, true>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked backward kernel takes checkpoint intervals 32 or 64");
}

}  // namespace

int chunk_backward(const ChunkBwdArgs &a, int dtype, int op, hipStream_t stream) {
    if (dtype == T2FW_F16) return op == 1 ? by_nb<Fp16, Fp16>(a, stream) : by_nb<Fp16, Bf16>(a, stream);
    if (dtype == T2FW_BF16) return by_nb<Bf16, Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
