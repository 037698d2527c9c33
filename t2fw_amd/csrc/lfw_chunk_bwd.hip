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
// a wave.  Chunks are visited last to first; inside a chunk a forward sweep ("R" stages, two
// blocks per stage) recomputes the block-start states from the checkpoint and keeps them as
// 16-bit MFMA operands in registers, then the blocks are visited last to first ("B" stages).
// Eight prep waves (B stages: 4 roles x 2 token halves; R stages: 2 blocks x 2 sides x 2 token
// halves) build the operand tiles of the next stage in double-buffered LDS; one barrier per
// stage.  Raw inputs go from global memory straight to the prep waves' registers two stages
// ahead, and the matrix waves store the gradients themselves.
//
// Replaces lfw_cuda_bwd_kernel and the six einsums of the reference
// (t2fw/csrc/lfw_kernel.cu:61-102, t2fw/csrc/lfw.cpp:84-93).
#include <type_traits>

#include "lfw_chunk_bwd_dev.hpp"

namespace t2fw {
namespace {

using namespace bwd;

constexpr int SP_THREADS = 768;
constexpr int CC = 20;   // channel-major 16-token tiles: row stride in elements

// ---- LDS layout of one stage buffer (bytes) ----------------------------------------------
constexpr int TM_TILE = CH_L * TS * 2;       // token-major 16-bit tile [16][TS], channels permuted (tm_pos)
constexpr int CM_TILE = CH_N * CC * 2;       // channel-major 16-bit tile [64][CC]
constexpr int CF_TILE = CH_N * CC * 4;       // channel-major fp32 tile [64][CC]
enum { TM_AOS = 0, TM_VOT, TM_VOH, TM_NUM };
// B stages use the named tiles; an R stage covers two blocks j = 0, 1 and uses tiles 2j (VOH) and 2j+1 (VH)
enum { CM_AOS = 0, CM_VOH, CM_AS, CM_VT, CM_VH, CM_NUM };
enum { F_RG = 0, F_IP, F_PP, F_NUM };        // 1/own gate, 1/own prefix, own prefix
constexpr int OFF_TM = 0;
constexpr int OFF_CM = OFF_TM + TM_NUM * TM_TILE;
constexpr int OFF_CF = OFF_CM + CM_NUM * CM_TILE;
// 16-step gate products, [block j of an R stage][other side, own side][64] f32 (B stages: j = 0)
constexpr int OFF_LV = OFF_CF + F_NUM * CF_TILE;
constexpr int STAGE_BYTES = OFF_LV + 4 * CH_N * 4;
constexpr int SP_SMEM = 2 * STAGE_BYTES;
static_assert(SP_SMEM <= 160 * 1024, "backward stage buffers exceed the LDS of one CU");
static_assert(STAGE_BYTES % 16 == 0, "stage buffers must keep 16-byte alignment");

__device__ __forceinline__ float *lv_vec(unsigned char *stage, int j, int own) {
    return reinterpret_cast<float *>(stage + OFF_LV) + (2 * j + own) * CH_N;
}
__device__ __forceinline__ const float *lv_vec(const unsigned char *stage, int j, int own) {
    return reinterpret_cast<const float *>(stage + OFF_LV) + (2 * j + own) * CH_N;
}

// ---- stage schedule ----------------------------------------------------------------------
// Chunks are visited from the last one down; a chunk with nb blocks takes ceil(nb/2) "R"
// stages of two blocks each (forward in time), then nb "B" stages (blocks nb-1..0).
// A stage is one int: (first token of its first block) * 2 + (1 for a B stage).
// NB = 1 means a checkpoint per block (C = 16): the state at every block start comes from memory, so
// only the last block of the sequence takes an R stage (for the state at the end of the sequence).
template <int NB> struct SplitSchedule {
    static constexpr unsigned PER_CHUNK = NB == 1 ? 1 : NB / 2 + NB;
    int NC, C, total, nb_last, st_last;
    __device__ SplitSchedule(int64_t T, int64_t NC_, int C_) {
        NC = (int)NC_;
        C = C_;
        const int len_last = (int)(T - (NC_ - 1) * C_);
        nb_last = (len_last + CH_L - 1) / CH_L;
        st_last = (nb_last + 1) / 2 + nb_last;
        total = st_last + (NC - 1) * (int)PER_CHUNK;
    }
};

// The same schedule as a forward iterator: cur() is SplitSchedule::at of the stage it stands on;
// advancing past the last stage leaves it there.  The stages of a chunk are one byte each in a
// 64-bit table, (block << 1) | (1 for a B stage), so that a step costs a few scalar instructions.
template <int NB> struct StageIter {
    static __host__ __device__ constexpr uint64_t table_of(int nb) {
        uint64_t t = 0;
        const int nr = (nb + 1) / 2;
        for (int l = 0; l < nr + nb; ++l) {
            const uint64_t e = l < nr ? (uint64_t)(2 * l) << 1 : ((uint64_t)(nb - 1 - (l - nr)) << 1) | 1u;
            t |= e << (8 * l);
        }
        return t;
    }
    uint64_t table;     // of the chunk it stands in
    int base2;          // (first token of that chunk) * 2
    int local, count;   // stage inside the chunk, stages of the chunk
    int C2, left;       // 2 * C; stages after the current one
    __device__ StageIter(const SplitSchedule<NB> &sc)
        : base2((sc.NC - 1) * sc.C * 2), local(0), count(sc.st_last), C2(2 * sc.C), left(sc.total - 1) {
        table = sc.nb_last == 1 ? table_of(1) : sc.nb_last == 2 ? table_of(2) : sc.nb_last == 3 ? table_of(3) : table_of(4);
    }
    __device__ void advance() {
        if (left > 0) {
            --left;
            ++local;
            if (local == count) {
                base2 -= C2;
                local = 0;
                count = (int)SplitSchedule<NB>::PER_CHUNK;
                table = NB == 1 ? (uint64_t)1 /* one B stage, block 0 */ : table_of(NB);
            }
        }
    }
    __device__ int cur() const {
        const int e = (int)(table >> (8 * local)) & 0xff;       // (block << 1) | bmode
        return base2 + (e >> 1) * (2 * CH_L) + (e & 1);
    }
};
static_assert(SplitSchedule<4>::PER_CHUNK <= 8, "a chunk's stages must fit the 64-bit table");

// ---- raw inputs --------------------------------------------------------------------------
// A prep thread works on one channel and eight tokens; it needs the gate at those tokens, the
// gate at the block's other eight tokens and one value (or adjoint) array at its own tokens:
// 24 two-byte loads, coalesced over the wave's 64 channels.  They go straight to registers,
// two stages ahead of their use: the block's first token of an array is a scalar base, the
// lane's channel and token half a constant vector offset, the token inside the half an
// immediate one (for rows that are heads of a [B, T, H, 64] tensor see TokenMap).
struct RawSet {
    u16 gown[8], goth[8], val[8];
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
        for (int t = 0; t < 8; ++t) {
            tok_off[t] = 2u * ((u32)c + (u32)t * ts);
        }
    }
};

// gate, val: wave-uniform addresses of the block's first token
template <bool HEADS>
__device__ __forceinline__ void raw_issue(RawSet &r, const u16 *gate, const u16 *val, TokenMap<HEADS> &m) {
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
    } else {
        // The offsets are made opaque at every use: they then stay in eight 32-bit registers (no
        // re-derivation from the channel, no widened copies hoisted out of the loops), which is the
        // form the scalar-base addressing mode of the loads takes.
#pragma unroll
        for (int t = 0; t < 8; ++t) asm volatile("" : "+v"(m.tok_off[t]));
        auto at = [&](const u16 *base, int t) -> u16 {
            return *reinterpret_cast<const u16 *>(reinterpret_cast<const unsigned char *>(base) + m.tok_off[t]);
        };
        const u16 *const go = gate + m.shift_own, *const gx = gate + m.shift_oth, *const vo = val + m.shift_own;
#pragma unroll
        for (int t = 0; t < 8; ++t) r.goth[t] = at(gx, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.gown[t] = at(go, t);
#pragma unroll
        for (int t = 0; t < 8; ++t) r.val[t] = at(vo, t);
    }
}

// The same for a block that reaches past the end of the sequence (T % 16 != 0, last chunk only):
// tokens past the end are read from the last one, with the same number of loads, and replaced by
// raw_patch_tail when the set is taken.  row_gate, row_val: token 0 of the batch row.
__device__ __forceinline__ void raw_issue_tail(RawSet &r, const u16 *row_gate, const u16 *row_val, int tok_own,
                                               int tok_oth, int T, int c, u32 ts) {
    auto at = [&](const u16 *base, int tok) -> u16 { return base[(u32)min(tok, T - 1) * ts + c]; };
#pragma unroll
    for (int t = 0; t < 8; ++t) r.goth[t] = at(row_gate, tok_oth + t);
#pragma unroll
    for (int t = 0; t < 8; ++t) r.gown[t] = at(row_gate, tok_own + t);
#pragma unroll
    for (int t = 0; t < 8; ++t) r.val[t] = at(row_val, tok_own + t);
}

// tokens past the end act as identity: gate 1, everything else 0
template <typename IOE> __device__ __forceinline__ void raw_patch_tail(RawSet &r, int tok_own, int tok_oth, int T) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        if (tok_oth + t >= T) r.goth[t] = IOE::ONE_BITS;
        if (tok_own + t >= T) {
            r.gown[t] = IOE::ONE_BITS;
            r.val[t] = 0;
        }
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

__device__ __forceinline__ void write_tm8(unsigned char *stage, int tile, int c, int t0, const Packed8 &v) {
    u16 *tm = reinterpret_cast<u16 *>(stage + OFF_TM + tile * TM_TILE) + t0 * TS + tm_pos(c);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        tm[(2 * i) * TS] = (u16)(v.p[i] & 0xffffu);
        tm[(2 * i + 1) * TS] = (u16)(v.p[i] >> 16);
    }
}

__device__ __forceinline__ void write_cm8(unsigned char *stage, int tile, int c, int t0, const Packed8 &v) {
    uint2 *cm = reinterpret_cast<uint2 *>(stage + OFF_CM + tile * CM_TILE + (c * CC + t0) * 2);
    cm[0] = make_uint2(v.p[0], v.p[1]);
    cm[1] = make_uint2(v.p[2], v.p[3]);
}

__device__ __forceinline__ void write_cf8(unsigned char *stage, int tile, int c, int t0, const float (&v)[8]) {
    float4 *cf = reinterpret_cast<float4 *>(stage + OFF_CF + tile * CF_TILE + (c * CC + t0) * 4);
    cf[0] = make_float4(v[0], v[1], v[2], v[3]);
    cf[1] = make_float4(v[4], v[5], v[6], v[7]);
}

template <typename IOE> __device__ __forceinline__ float product8(const u16 (&g)[8]) {
    float p = IOE::mul2(g[0], g[1]);
#pragma unroll
    for (int t = 2; t < 8; ++t) p = IOE::mul(g[t], p);
    return p;
}

// Gate-suffix scalings of one half block: hat = v * prod_{r>t} gate_r, til = hat / total,
// inv = 1 / prod_{r<=t} gate_r; returns the 16-step product.
template <typename IOE, typename OPE>
__device__ __forceinline__ float suffix_scale(const RawSet &r, int h, bool check, float (&hat)[8], float (&til)[8],
                                              float (&inv)[8], u32 &bad) {
    const float poth = product8<IOE>(r.goth);
    const float tot = product8<IOE>(r.gown) * poth;
    if (check) bad |= gate_check8<IOE>(r.gown);
    bad |= (tot >= OPE::MIN_PRODUCT) ? 0u : 1u;
    const float itot = __builtin_amdgcn_rcpf(tot);
    float sfx = h ? 1.0f : poth;
#pragma unroll
    for (int t = 7; t >= 0; --t) {
        inv[t] = sfx * itot;
        hat[t] = IOE::mul(r.val[t], sfx);
        til[t] = hat[t] * itot;
        sfx = IOE::mul(r.gown[t], sfx);
    }
    return tot;
}

// B stage, one prep wave: one role, tokens 8h..8h+7 of the block, channel c.
//   role 0: other gate prefix -> AOS (token- and channel-major)
//   role 1: other gate suffix -> VOH (both layouts), VOT (token-major), L_other
//   role 2: own gate prefix   -> AS, 1/gate, prefix (side 1)
//   role 3: own gate suffix   -> VH, VT, 1/prefix, L_own
template <typename IOE, typename OPE>
__device__ __forceinline__ void prep_b(const RawSet &r, unsigned char *stage, int role, int h, int c, bool want_pp,
                                       u32 &bad) {
    const bool other = role < 2;
    const int t0 = 8 * h;
    if ((role & 1) == 0) {
        const float base = h ? product8<IOE>(r.goth) : 1.0f;
        float run = base;
        float pre[8], v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            run = IOE::mul(r.gown[t], run);
            pre[t] = run;
            v[t] = IOE::mul(r.val[t], run);
        }
        const Packed8 vp = pack8<OPE>(v);
        if (other) {
            write_tm8(stage, TM_AOS, c, t0, vp);
            write_cm8(stage, CM_AOS, c, t0, vp);
        } else {
            // 1/gate_t = prefix_{t-1} / prefix_t from one reciprocal and the running products
            float ipre = __builtin_amdgcn_rcpf(pre[7]);
            float rg[8];
#pragma unroll
            for (int t = 7; t >= 1; --t) {
                rg[t] = pre[t - 1] * ipre;
                ipre = IOE::mul(r.gown[t], ipre);
            }
            rg[0] = base * ipre;
            write_cm8(stage, CM_AS, c, t0, vp);
            write_cf8(stage, F_RG, c, t0, rg);
            if (want_pp) write_cf8(stage, F_PP, c, t0, pre);
        }
    } else {
        float hat[8], til[8], inv[8];
        const float tot = suffix_scale<IOE, OPE>(r, h, true, hat, til, inv, bad);
        if (h == 0) lv_vec(stage, 0, other ? 0 : 1)[c] = tot;
        const Packed8 hp = pack8<OPE>(hat), tp = pack8<OPE>(til);
        if (other) {
            write_cm8(stage, CM_VOH, c, t0, hp);
            write_tm8(stage, TM_VOH, c, t0, hp);
            write_tm8(stage, TM_VOT, c, t0, tp);
        } else {
            write_cm8(stage, CM_VH, c, t0, hp);
            write_cm8(stage, CM_VT, c, t0, tp);
            write_cf8(stage, F_IP, c, t0, inv);
        }
    }
}

// R stage, one prep wave: block j of the pair, own or other side, tokens 8h..8h+7, channel c:
// the suffix-scaled values (channel-major) and the 16-step gate product.  (Every block's gates
// are range-checked in its B stage.)
template <typename IOE, typename OPE>
__device__ __forceinline__ void prep_r(const RawSet &r, unsigned char *stage, int j, int own, int h, int c, u32 &bad) {
    float hat[8], til[8], inv[8];
    const float tot = suffix_scale<IOE, OPE>(r, h, false, hat, til, inv, bad);
    if (h == 0) lv_vec(stage, j, own)[c] = tot;
    write_cm8(stage, 2 * j + own, c, 8 * h, pack8<OPE>(hat));
}

template <typename IOE, typename OPE, int NB, bool HEADS>
__device__ __forceinline__ void split_prep_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b,
                                                 int side) {
    const int pw = __builtin_amdgcn_readfirstlane(tid >> 6), c = tid & 63;
    // B stages: SIMD-balanced assignment of (role, token half); roles 1 and 3 are the heavier ones
    const int h = pw >> 2;
    const int role = (h ? (pw ^ 1) : pw) & 3;
    // R stages: (block of the pair, side, token half)
    const int rj = (pw >> 1) & 1, rown = pw & 1;
    const int T = (int)p.T;                              // the launcher admits T * heads < 2^24 only
    const int64_t row_off = row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N;
    // this batch row of: other gate, other value, own gate, own value, other adjoint, own adjoint
    const u16 *const x = reinterpret_cast<const u16 *>(p.x) + row_off, *const f = reinterpret_cast<const u16 *>(p.f) + row_off;
    const u16 *const g = reinterpret_cast<const u16 *>(p.g_out) + row_off, *const k = reinterpret_cast<const u16 *>(p.k) + row_off;
    const u16 *const fk = reinterpret_cast<const u16 *>(p.f_key) + row_off, *const q = reinterpret_cast<const u16 *>(p.q) + row_off;
    const u16 *const GO = side == 0 ? fk : f, *const VO = side == 0 ? k : x, *const GW = side == 0 ? f : fk;
    const u16 *const VW = side == 0 ? x : k, *const AO = side == 0 ? q : g, *const AW = side == 0 ? g : q;
    // the two arrays this wave reads in B stages and in R stages
    const u16 *const b_gate = role < 2 ? GO : GW;
    const u16 *const b_val = role == 0 ? AO : role == 1 ? VO : role == 2 ? AW : VW;
    const u16 *const r_gate = rown ? GW : GO;
    const u16 *const r_val = rown ? VW : VO;
    const SplitSchedule<NB> sched(p.T, p.NC, p.C);
    u32 bad = 0;

    TokenMap<HEADS> tmap(HEADS ? (u32)p.heads * CH_N : (u32)CH_N, h, c);
    const u32 ts = tmap.ts;                              // elements between consecutive tokens
    // first token of the block this wave works on in stage st (R stages cover a pair of blocks)
    auto block_tok = [&](int st) -> int { return (st >> 1) + ((st & 1) ? 0 : rj * CH_L); };
    auto issue = [&](RawSet &r, int st) {          // raw inputs of stage st (wave-uniform) -> registers
        const bool bmode = st & 1;
        const int tok = block_tok(st);
        const u16 *const gate = bmode ? b_gate : r_gate, *const val = bmode ? b_val : r_val;
        if (tok + CH_L <= T)
            raw_issue<HEADS>(r, gate + (u32)tok * ts, val + (u32)tok * ts, tmap);
        else        // the block reaches past the end (or, second block of the last R pair, lies past it)
            raw_issue_tail(r, gate, val, tok + 8 * h, tok + 8 * (1 - h), T, c, ts);
    };
    // Three register sets rotate: the tiles of stage s are built from `cur`, which was loaded two
    // stages ago, while `refill` (used up in the stage before) takes the raw inputs of stage s + 2.
    // The loads are unconditional (past the end: the last stage again), so that the number of loads
    // in flight is the same on every path and the waits for them can be exact.
    StageIter<NB> it_load(sched);
    int st_cur = 0, st_next = 0;                   // descriptors of stages s and s + 1
    PHASE_BEGIN();
    auto prepare = [&](const RawSet &cur, RawSet &refill, int s) {
        const int st = st_cur;
        it_load.advance();
        const int st_new = it_load.cur();
        issue(refill, st_new);
        st_cur = st_next;
        st_next = st_new;
        // the loads complete in order: one wait for the last of `cur` covers the whole set
        asm volatile("" ::"v"(cur.val[7]));
        RawSet raw = cur;
        const int tok = block_tok(st);
        if (tok + CH_L > T) raw_patch_tail<IOE>(raw, tok + 8 * h, tok + 8 * (1 - h), T);
        unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
        if (st & 1)
            prep_b<IOE, OPE>(raw, stage, role, h, c, side == 1, bad);
        else
            prep_r<IOE, OPE>(raw, stage, rj, rown, h, c, bad);
        PHASE_MARK(2);
        __syncthreads();
        PHASE_MARK(3);
    };

    // Stages are done in triples (sets A, B, C in turn) with no exit inside a triple, so that the
    // order of the loads in flight is the same on every path.  First the stages of the last chunk of
    // the sequence (it may be short), with the general iterator; its first (count % 3) stages are
    // peeled off, with the sets assigned so that the triples start on A.
    RawSet setA, setB, setC;
    int s = 0;
    // (with a checkpoint per block, also as many of the following blocks as make the rest a multiple of three)
    const int n_last = sched.st_last + (NB == 1 ? (sched.NC - 1) % 3 : 0);
    const int rem = n_last % 3;
    st_cur = it_load.cur();
    it_load.advance();
    st_next = it_load.cur();
    if (rem == 0) {
        issue(setA, st_cur);
        issue(setB, st_next);
    } else if (rem == 1) {
        issue(setC, st_cur);
        issue(setA, st_next);
        prepare(setC, setB, 0);
        s = 1;
    } else {
        issue(setB, st_cur);
        issue(setC, st_next);
        prepare(setB, setA, 0);
        prepare(setC, setB, 1);
        s = 2;
    }
    for (; s < n_last; s += 3) {
        prepare(setA, setC, s);
        prepare(setB, setA, s + 1);
        prepare(setC, setB, s + 2);
    }

    if constexpr (NB != 1) {
        // Then the full chunks, last to first.  Inside a chunk the kind of every stage and its block are
        // compile-time constants (position POS of PER), which leaves a pointer bump per stage for the
        // scalar unit; PER is a multiple of three, so every chunk starts on set A.  The refill of
        // position POS + 2 reaches into the chunk below for the last two positions (below the first
        // chunk: that chunk again, never used).
        constexpr int PER = (int)SplitSchedule<NB>::PER_CHUNK, NR = NB / 2;
        static_assert(PER % 3 == 0, "a chunk must take a whole number of register-set triples");
        const u16 *const r_gate_w = r_gate + (u32)(rj * CH_L) * ts, *const r_val_w = r_val + (u32)(rj * CH_L) * ts;
        auto issue_at = [&](RawSet &r, int chunk_tok, auto pos_c) {
            constexpr int POS = decltype(pos_c)::value;
            if constexpr (POS < NR) {
                const u32 e = (u32)(chunk_tok + 2 * POS * CH_L) * ts;
                raw_issue<HEADS>(r, r_gate_w + e, r_val_w + e, tmap);
            } else {
                const u32 e = (u32)(chunk_tok + (NB - 1 - (POS - NR)) * CH_L) * ts;
                raw_issue<HEADS>(r, b_gate + e, b_val + e, tmap);
            }
        };
        auto prepare_at = [&](const RawSet &cur, RawSet &refill, int chunk_tok, int below_tok, auto pos_c) {
            constexpr int POS = decltype(pos_c)::value;
            if constexpr (POS + 2 < PER)
                issue_at(refill, chunk_tok, std::integral_constant<int, (POS + 2) % PER>{});
            else
                issue_at(refill, below_tok, std::integral_constant<int, (POS + 2) % PER>{});
            // the loads complete in order: one wait for the last of `cur` covers the whole set
            asm volatile("" ::"v"(cur.val[7]));
            unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
            if constexpr (POS >= NR)
                prep_b<IOE, OPE>(cur, stage, role, h, c, side == 1, bad);
            else
                prep_r<IOE, OPE>(cur, stage, rj, rown, h, c, bad);
            ++s;
            PHASE_MARK(POS >= NR ? 2 : 0);
            __syncthreads();
            PHASE_MARK(POS >= NR ? 3 : 1);
        };
        for (int chunk_tok = (sched.NC - 2) * p.C; chunk_tok >= 0; chunk_tok -= p.C) {
            const int below_tok = max(chunk_tok - p.C, 0);
            prepare_at(setA, setC, chunk_tok, below_tok, std::integral_constant<int, 0>{});
            prepare_at(setB, setA, chunk_tok, below_tok, std::integral_constant<int, 1>{});
            prepare_at(setC, setB, chunk_tok, below_tok, std::integral_constant<int, 2>{});
            if constexpr (PER == 6) {
                prepare_at(setA, setC, chunk_tok, below_tok, std::integral_constant<int, 3>{});
                prepare_at(setB, setA, chunk_tok, below_tok, std::integral_constant<int, 4>{});
                prepare_at(setC, setB, chunk_tok, below_tok, std::integral_constant<int, 5>{});
            }
        }
    } else {
        // A checkpoint per block: what is left are B stages of full blocks, a multiple of three of
        // them, last to first; set A holds the highest one, set B the one below it.
        auto prepare_block = [&](const RawSet &cur, RawSet &refill, int refill_tok) {
            const u32 e = (u32)max(refill_tok, 0) * ts;      // below the first block: that block again, never used
            raw_issue<HEADS>(refill, b_gate + e, b_val + e, tmap);
            // the loads complete in order: one wait for the last of `cur` covers the whole set
            asm volatile("" ::"v"(cur.val[7]));
            prep_b<IOE, OPE>(cur, smem + (s & 1) * STAGE_BYTES, role, h, c, side == 1, bad);
            ++s;
            PHASE_MARK(2);
            __syncthreads();
            PHASE_MARK(3);
        };
        const int nblocks = (sched.NC - 1) / 3 * 3;
        for (int tok = (nblocks - 1) * CH_L; tok >= 0; tok -= 3 * CH_L) {
            prepare_block(setA, setC, tok - 2 * CH_L);
            prepare_block(setB, setA, tok - 3 * CH_L);
            prepare_block(setC, setB, tok - 4 * CH_L);
        }
    }
    // Both workgroups of a row see all four gates' blocks and reach the same verdict, so either
    // order of their writes leaves the same flag.
    if (bad) p.row_flags[b] = 1;
    PHASE_END(4 + (tid >> 6));
}

// SIDE is a template parameter here: the stores at the end of a stage (and the state loads) then
// carry no branches on it.
template <typename IOE, typename OPE, int NB, bool HEADS, int SIDE>
__device__ __forceinline__ void split_matrix_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b) {
    constexpr int side = SIDE;
    const int w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int ch = 16 * w + r;       // this lane's own-side channel
    const int T = (int)p.T;                              // the launcher admits T < 2^24 only
    const int64_t NC = p.NC;
    const int C = p.C;
    const u16 *ckpt = reinterpret_cast<const u16 *>(p.ckpt) + b * NC * (CH_N * CH_N);
    const int nb_last = (int)((p.T - (NC - 1) * C + CH_L - 1) / CH_L);
    // this batch row of the gradients this side writes
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
    // A checkpoint per block (NB = 1): the block-start state of every block but the last comes
    // straight from memory: raw loads (side 0: four 8-byte loads, side 1: sixteen 2-byte loads of a
    // column) issued at the start of the stage above and put together at its end; `top` keeps the raw
    // state of the latest block whose start is a multiple of four blocks (for the anchor).
    u32 ahead[NB == 1 ? 16 : 1];
    uint2 below[4] = {};             // raw start state of the block below the current one
    uint2 top[4] = {pf[0], pf[1], pf[2], pf[3]};
    auto fetch_ahead = [&](const u16 *m) {
        if (side == 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint2 v = ld2(m + ch * CH_N + 16 * j + 4 * g);
                ahead[(2 * j) % (NB == 1 ? 16 : 1)] = v.x;
                ahead[(2 * j + 1) % (NB == 1 ? 16 : 1)] = v.y;
            }
#pragma unroll
            for (int j = 8; j < (NB == 1 ? 16 : 1); ++j) ahead[j] = 0;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) ahead[(4 * j + i) % (NB == 1 ? 16 : 1)] = m[(16 * j + 4 * g + i) * CH_N + ch];
        }
    };
    auto take_ahead = [&](uint2 (&dst)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            constexpr int M = NB == 1 ? 16 : 1;
            if (side == 0)
                dst[j] = make_uint2(ahead[(2 * j) % M], ahead[(2 * j + 1) % M]);
            else
                dst[j] = make_uint2(ahead[(4 * j) % M] | (ahead[(4 * j + 1) % M] << 16),
                                    ahead[(4 * j + 2) % M] | (ahead[(4 * j + 3) % M] << 16));
        }
    };
    // raw state (I/O type, four values per 32-bit pair) -> the two MFMA operands
    auto to_operands = [&](const uint2 (&raw)[4], uint4 &lo, uint4 &hi) {
        if constexpr (std::is_same<IOE, OPE>::value) {
            lo = cat(raw[0], raw[1]);
            hi = cat(raw[2], raw[3]);
        } else {
            uint2 o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float t[4];
                unpack4<IOE>(raw[j], t);
                const floatx4 v = {t[0], t[1], t[2], t[3]};
                o[j] = pack4v<OPE>(v);
            }
            lo = cat(o[0], o[1]);
            hi = cat(o[2], o[3]);
        }
    };
    float carry = 0.f;
    int s = 0;
    if (tid == 0) {      // both flag slots of the row (the backward kernels report in the first)
        p.row_flags[b] = 0;
        p.row_flags[chunk_rows_padded(p.B) + b] = 0;
    }
    PHASE_BEGIN();

    // every stage starts with the workgroup barrier that publishes its operand tiles
    for (int64_t chunk = NC - 1; chunk >= 0; --chunk) {
        const bool last = chunk == NC - 1;
        const int nb = last ? nb_last : NB;
        const bool recompute = NB != 1 || last;              // this chunk has R stages
        if (recompute) {
            take_state(pf, S);
            if (NB != 1 && chunk > 0) load_state(ckpt + (chunk - 1) * (CH_N * CH_N), pf);
        }
        // ---- R stages: block-start states, forward in time, two blocks per stage
#pragma unroll
        for (int i2 = 0; i2 < NB; i2 += 2) {
            if (i2 < nb && recompute) {
                __syncthreads();
                PHASE_MARK(3);
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) {
                    const int i = (i2 + jb) % NB;           // (i2 + jb < NB wherever the branch below is taken)
                    if (i2 + jb < nb) {
                        const u16 *VOHc = reinterpret_cast<const u16 *>(stage + OFF_CM + (2 * jb) * CM_TILE);
                        const u16 *VHc = reinterpret_cast<const u16 *>(stage + OFF_CM + (2 * jb + 1) * CM_TILE);
                        const float *LX = lv_vec(stage, jb, 0), *LO = lv_vec(stage, jb, 1);
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
        // (with a checkpoint per block: every fourth block, S_end = the start state of the block above)
        if (NB == 1 && !last && (chunk & 3) == 3) take_state(top, S);
        if (recompute || (chunk & 3) == 3) {
            float us = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) us += G[j][i] * S[j][i];
            carry = row_sums(us).all;
        }
        // ---- B stages: blocks last to first
#pragma unroll
        for (int i = NB - 1; i >= 0; --i) {
            if (i < nb) {
                __syncthreads();
                PHASE_MARK(2);
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
                const u16 *AOS = reinterpret_cast<const u16 *>(stage + OFF_TM + TM_AOS * TM_TILE);
                const u16 *VOT = reinterpret_cast<const u16 *>(stage + OFF_TM + TM_VOT * TM_TILE);
                const u16 *VOH = reinterpret_cast<const u16 *>(stage + OFF_TM + TM_VOH * TM_TILE);
                const u16 *AOSc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_AOS * CM_TILE);
                const u16 *ASc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_AS * CM_TILE);
                const u16 *VTc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_VT * CM_TILE);
                const float *LX = lv_vec(stage, 0, 0), *LO = lv_vec(stage, 0, 1);
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                // the state at the start of this block, as MFMA operands
                uint4 sb0 = sv[i][0], sb1 = sv[i][1];
                if constexpr (NB == 1) {
                    if (!last) {
                        to_operands(below, sb0, sb1);
                        if ((chunk & 3) == 0) {
#pragma unroll
                            for (int j = 0; j < 4; ++j) top[j] = below[j];
                        }
                    }
                    if (chunk > 0) fetch_ahead(ckpt + (chunk - 1) * (CH_N * CH_N));
                }
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
                    const float *cf = reinterpret_cast<const float *>(stage + OFF_CF) + ch * CC + 4 * g;
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
                    // The state of the block below has had this stage's arithmetic to arrive; it is taken
                    // before the stores are issued, so that the wait for it never includes them.
                    if constexpr (NB == 1) {
                        if (chunk > 0) take_ahead(below);
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
__global__ __launch_bounds__(SP_THREADS) void lfw_bwd_chunk_kernel(ChunkBwdArgs p, int rows_padded) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    // blockIdx = side * rows_padded + row with rows_padded a multiple of 8: the two workgroups of a
    // row land on the same XCD and share its L2 for the inputs both of them read
    const int side = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - side * rows_padded;
    if (b >= p.B) return;
    // both branches execute exactly 2 + (number of stages) workgroup barriers
    if (tid < 256) {
        if (side == 0)
            split_matrix_waves<IOE, OPE, NB, HEADS, 0>(p, smem, tid, b);
        else
            split_matrix_waves<IOE, OPE, NB, HEADS, 1>(p, smem, tid, b);
    }
    else
        split_prep_waves<IOE, OPE, NB, HEADS>(p, smem, tid - 256, b, side);
}

template <typename IOE, typename OPE, int NB, bool HEADS> int launch(const ChunkBwdArgs &a, hipStream_t stream) {
    auto kern = lfw_bwd_chunk_kernel<IOE, OPE, NB, HEADS>;
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, SP_SMEM),
                       "hipFuncSetAttribute(backward chunk kernel)");
    if (rc) return rc;
    if (a.B > 0x1fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    if (a.heads < 1 || a.T * a.heads >= CHUNK_MAX_T)
        return fail(T2FW_ERR_UNSUPPORTED, "T=%lld with %d heads is too long for 32-bit row offsets", (long long)a.T, a.heads);
    const int rows_padded = (int)((a.B + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(2u * (unsigned)rows_padded), dim3(SP_THREADS), SP_SMEM, stream, a, rows_padded);
    return check_hip(hipGetLastError(), "lfw_bwd_chunk_kernel launch");
}

template <typename IOE, typename OPE> int by_nb(const ChunkBwdArgs &a, hipStream_t stream) {
    if (a.C == 16) return a.heads == 1 ? launch<IOE, OPE, 1, false>(a, stream) : launch<IOE, OPE, 1, true>(a, stream);
    if (a.C == 64) return a.heads == 1 ? launch<IOE, OPE, 4, false>(a, stream) : launch<IOE, OPE, 4, true>(a, stream);
    if (a.C == 32) return a.heads == 1 ? launch<IOE, OPE, 2, false>(a, stream) : launch<IOE, OPE, 2, true>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked backward kernel takes checkpoint intervals 16, 32 or 64");
}

}  // namespace

int chunk_backward(const ChunkBwdArgs &a, int dtype, int op, hipStream_t stream) {
    if (dtype == T2FW_F16) return op == 1 ? by_nb<Fp16, Fp16>(a, stream) : by_nb<Fp16, Bf16>(a, stream);
    if (dtype == T2FW_BF16) return by_nb<Bf16, Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
