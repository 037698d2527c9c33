// Backward pass of the decay rule, chunked matrix-core form, split by side: two workgroups
// per batch row (algebra: lfw_chunk.hpp and lfw_chunk_bwd.hip).
//
// The recurrence is symmetric under (x, f, g_out, D) <-> (k, f_key, q, K) with the state
// transposed.  The whole-row kernel exploits this by keeping two copies of S and of its
// adjoint; here each copy gets a workgroup (and a CU) of its own and nothing is exchanged:
//   side 0 ("value side"): own = (x, f, g_out), other = (k, f_key, q); writes d_x, d_f, d_s0
//   side 1 ("key side")  : own = (k, f_key, q), other = (x, f, g_out); writes d_k, d_f_key, d_q
// In the names below V = own value (x | k), A = own adjoint (g_out | q), VO / AO the other
// side's, a suffix S / T / H = scaled by the gate prefix / divided by it / scaled by the
// gate suffix (qs, kt, kh ... of lfw_chunk.hpp).  With own channel c, other channel e:
//   P[t,s]  = AOS_t . VOT_s                                         (contraction over e)
//   o'_t[c] = sum_e S0[c,e] AOS_t[e] + sum_{s<t} P[t,s] VT_s[c]
//   v'_t[c] = sum_e (L_own[c] Gb[c,e]) VOH_t[e] + sum_{r>t} P[r,t] AS_r[c]
//   d_own_gate_t = RG_t * (carry + sum_{r>=t} o'_r AS_r - v'_r VT_r)
//   d_V_t = IP_t * (v'_t + AS_t P[t,t])        d_A_t = PP_t * (o'_t + VT_t P[t,t])   (side 1 only)
//   Gb <- L_own[c] L_other[e] Gb[c,e] + sum_t AS_t[c] AOS_t[e]
// Used when twice the batch fits the CUs of the device: the 12-wave workgroups (4 matrix
// waves + 8 prep waves, two per role, each taking 8 of a block's 16 tokens) halve the
// instructions on every wave's critical path compared with the whole-row kernel.
//
// Replaces lfw_cuda_bwd_kernel and the six einsums of the reference
// (t2fw/csrc/lfw_kernel.cu:61-102, t2fw/csrc/lfw.cpp:84-93).
#include "lfw_chunk_bwd_dev.hpp"

namespace t2fw {
namespace {

using namespace bwd;

constexpr int SP_THREADS = 768;
constexpr int SP_PREP = 512;
constexpr int CC = 20;   // channel-major 16-token tiles: row stride in elements

// ---- LDS layout of one stage buffer (bytes) ----------------------------------------------
constexpr int TM_TILE = CH_L * TS * 2;       // token-major 16-bit tile [16][TS], channels permuted (tm_pos)
constexpr int CM_TILE = CH_N * CC * 2;       // channel-major 16-bit tile [64][CC]
constexpr int CF_TILE = CH_N * CC * 4;       // channel-major fp32 tile [64][CC]
enum { TM_AOS = 0, TM_VOT, TM_VOH, TM_NUM };
enum { CM_AOS = 0, CM_VOH, CM_AS, CM_VT, CM_VH, CM_NUM };
enum { F_RG = 0, F_IP, F_PP, F_NUM };        // 1/own gate, 1/own prefix, own prefix
constexpr int OFF_TM = 0;
constexpr int OFF_CM = OFF_TM + TM_NUM * TM_TILE;
constexpr int OFF_CF = OFF_CM + CM_NUM * CM_TILE;
constexpr int OFF_LX = OFF_CF + F_NUM * CF_TILE;           // 16-step product of the other side's gate [64] f32
constexpr int OFF_LO = OFF_LX + CH_N * 4;                  // 16-step product of the own gate [64] f32
constexpr int STAGE_BYTES = OFF_LO + CH_N * 4;
constexpr int RAW_ARRAY = CH_L * CH_N * 2;                 // [16][64] u16
enum { R_GO = 0, R_VO, R_GW, R_VW, R_AO, R_AW, R_NUM };   // R stages need the first four only
constexpr int RAW_BYTES = R_NUM * RAW_ARRAY;
constexpr int SOFF_RAW = 2 * STAGE_BYTES;
constexpr int SP_SMEM = SOFF_RAW + 2 * RAW_BYTES;
static_assert(SP_SMEM <= 160 * 1024, "backward stage buffers exceed the LDS of one CU");
static_assert(STAGE_BYTES % 16 == 0, "stage buffers must keep 16-byte alignment");

// Position of channel c = 16j + 4g + e inside a token-major row: 16g + 4j + e.  The 16 values a
// lane contracts against its own accumulators (channels 16j + 4g + e, j = 0..3) are then
// contiguous.  Products between two token-major tiles are indifferent to the order.
__device__ __forceinline__ int tm_pos(int c) { return 16 * ((c >> 2) & 3) + 4 * (c >> 4) + (c & 3); }

struct Side {
    const u16 *src[R_NUM];      // raw arrays in the order of R_*
};

__device__ __forceinline__ Side make_side(const ChunkBwdArgs &p, int side) {
    Side s;
    const u16 *x = reinterpret_cast<const u16 *>(p.x), *f = reinterpret_cast<const u16 *>(p.f);
    const u16 *g = reinterpret_cast<const u16 *>(p.g_out), *k = reinterpret_cast<const u16 *>(p.k);
    const u16 *fk = reinterpret_cast<const u16 *>(p.f_key), *q = reinterpret_cast<const u16 *>(p.q);
    if (side == 0) {
        s.src[R_GO] = fk; s.src[R_VO] = k; s.src[R_GW] = f; s.src[R_VW] = x; s.src[R_AO] = q; s.src[R_AW] = g;
    } else {
        s.src[R_GO] = f; s.src[R_VO] = x; s.src[R_GW] = fk; s.src[R_VW] = k; s.src[R_AO] = g; s.src[R_AW] = q;
    }
    return s;
}

// ---- raw staging -------------------------------------------------------------------------
// A stage's raw inputs are R_NUM arrays of [16 tokens][64 channels]: 768 pieces of 16 bytes;
// prep thread i moves pieces i and (for i < 256, B stages only) i + 512.  R stages need pieces
// 0..511 only.  A wave's pieces come from one array, so the array base stays in scalar
// registers and a piece is addressed by a 32-bit element offset inside the batch row.  Loads
// are issued at the top of an iteration and parked in LDS at its end, so the wait for them
// overlaps the tile building in between; they are unconditional (clamped token, identity fill
// selected afterwards), which keeps the hardware memory counters exact.
constexpr int NPIECE = 2;
struct RawRegs {
    uint4 v[NPIECE];
    bool valid;
};

// element a of a small pointer table, a wave-uniform: scalar selects that keep the pointers' provenance
template <typename P> __device__ __forceinline__ P pick(int a, P p0, P p1, P p2, P p3, P p4, P p5) {
    return a == 0 ? p0 : a == 1 ? p1 : a == 2 ? p2 : a == 3 ? p3 : a == 4 ? p4 : p5;
}

struct PieceMap {
    const u16 *ld[NPIECE];   // this batch row of the array raw piece m comes from (wave-uniform)
    int tok;                 // token inside the block (the same for both pieces)
    u32 col;                 // element offset of the piece inside a token's 64 channels
    u32 fill;                // identity fill of piece 0 for steps past the end of the sequence (piece 1: zero)
    bool second;             // this thread also moves piece i + 512 (wave-uniform)
};

__device__ __forceinline__ void raw_load(RawRegs &st, const PieceMap &pm, int T, int t0, bool bmode) {
    const int t = t0 + pm.tok;
    st.valid = t < T;
    const u32 off = (u32)(st.valid ? t : T - 1) * CH_N + pm.col;
    st.v[0] = *reinterpret_cast<const uint4 *>(pm.ld[0] + off);
    if (pm.second && bmode) st.v[1] = *reinterpret_cast<const uint4 *>(pm.ld[1] + off);
}

__device__ __forceinline__ void raw_store(const RawRegs &st, const PieceMap &pm, unsigned char *raw, bool bmode, int tid) {
    const u32 fl = pm.fill;
    *reinterpret_cast<uint4 *>(raw + tid * 16) = st.valid ? st.v[0] : make_uint4(fl, fl, fl, fl);
    if (pm.second && bmode)
        *reinterpret_cast<uint4 *>(raw + (tid + SP_PREP) * 16) = st.valid ? st.v[1] : make_uint4(0u, 0u, 0u, 0u);
}

// eight consecutive tokens (from t0) of channel c of one raw array
__device__ __forceinline__ void raw_col8(u16 (&dst)[8], const unsigned char *raw, int array, int c, int t0) {
    const u16 *base = reinterpret_cast<const u16 *>(raw + array * RAW_ARRAY) + t0 * CH_N + c;
#pragma unroll
    for (int t = 0; t < 8; ++t) dst[t] = base[t * CH_N];
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

template <typename OPE>
__device__ __forceinline__ void write_tm8(unsigned char *stage, int tile, int c, int t0, const float (&v)[8]) {
    u16 *tm = reinterpret_cast<u16 *>(stage + OFF_TM + tile * TM_TILE) + t0 * TS + tm_pos(c);
#pragma unroll
    for (int t = 0; t < 8; ++t) tm[t * TS] = cvt1<OPE>(v[t]);
}

template <typename OPE>
__device__ __forceinline__ void write_cm8(unsigned char *stage, int tile, int c, int t0, const float (&v)[8]) {
    uint2 *cm = reinterpret_cast<uint2 *>(stage + OFF_CM + tile * CM_TILE + (c * CC + t0) * 2);
    cm[0] = packq<OPE>(v[0], v[1], v[2], v[3]);
    cm[1] = packq<OPE>(v[4], v[5], v[6], v[7]);
}

__device__ __forceinline__ void write_cf8(unsigned char *stage, int tile, int c, int t0, const float (&v)[8]) {
    float4 *cf = reinterpret_cast<float4 *>(stage + OFF_CF + tile * CF_TILE + (c * CC + t0) * 4);
    cf[0] = make_float4(v[0], v[1], v[2], v[3]);
    cf[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// One prep wave: one role, tokens 8h..8h+7 of the block, channel c.
//   role 0: other gate prefix -> AOS (token- and channel-major)
//   role 1: other gate suffix -> VOH (both layouts), VOT (token-major), L_other
//   role 2: own gate prefix   -> AS, 1/gate, prefix (side 1)
//   role 3: own gate suffix   -> VH, VT, 1/prefix, L_own
// R stages need VOH and VH channel-major and the two 16-step products only.
template <typename IOE, typename OPE>
__device__ __forceinline__ void split_prep(const unsigned char *raw, unsigned char *stage, int role, int h, int c,
                                           bool bmode, bool want_pp, u32 &bad) {
    const bool other = role < 2;
    const bool prefix_role = (role & 1) == 0;
    if (!bmode && prefix_role) return;
    const int t0 = 8 * h;
    const int garr = other ? R_GO : R_GW;
    u16 gown[8], goth[8], ar[8];
    raw_col8(gown, raw, garr, c, t0);
    raw_col8(ar, raw, prefix_role ? (other ? R_AO : R_AW) : (other ? R_VO : R_VW), c, t0);
    if (prefix_role) {
        float run = 1.0f;
        if (h) {
            raw_col8(goth, raw, garr, c, 0);
#pragma unroll
            for (int t = 0; t < 8; ++t) run *= IOE::to_f32(goth[t]);
        }
        float pre[8], v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            run *= IOE::to_f32(gown[t]);
            pre[t] = run;
            v[t] = IOE::to_f32(ar[t]) * run;
        }
        if (other) {
            write_tm8<OPE>(stage, TM_AOS, c, t0, v);
            write_cm8<OPE>(stage, CM_AOS, c, t0, v);
        } else {
            float rg[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) rg[t] = __builtin_amdgcn_rcpf(IOE::to_f32(gown[t]));
            write_cm8<OPE>(stage, CM_AS, c, t0, v);
            write_cf8(stage, F_RG, c, t0, rg);
            if (want_pp) write_cf8(stage, F_PP, c, t0, pre);
        }
    } else {
        raw_col8(goth, raw, garr, c, 8 - t0);
        bad |= gate_check8<IOE>(gown);
        float gate[8];
        float pown = 1.0f, poth = 1.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            gate[t] = IOE::to_f32(gown[t]);
            pown *= gate[t];
            poth *= IOE::to_f32(goth[t]);
        }
        const float tot = pown * poth;
        bad |= (tot >= OPE::MIN_PRODUCT) ? 0u : 1u;
        const float itot = __builtin_amdgcn_rcpf(tot);
        float hat[8], til[8], inv[8];
        float sfx = h ? 1.0f : poth;
#pragma unroll
        for (int t = 7; t >= 0; --t) {
            inv[t] = sfx * itot;                            // 1 / prefix_t
            hat[t] = IOE::to_f32(ar[t]) * sfx;
            til[t] = hat[t] * itot;
            sfx *= gate[t];
        }
        write_cm8<OPE>(stage, other ? CM_VOH : CM_VH, c, t0, hat);
        if (h == 0) reinterpret_cast<float *>(stage + (other ? OFF_LX : OFF_LO))[c] = tot;
        if (bmode) {
            if (other) {
                write_tm8<OPE>(stage, TM_VOH, c, t0, hat);
                write_tm8<OPE>(stage, TM_VOT, c, t0, til);
            } else {
                write_cm8<OPE>(stage, CM_VT, c, t0, til);
                write_cf8(stage, F_IP, c, t0, inv);
            }
        }
    }
}

template <typename IOE, typename OPE, int NB>
__device__ __forceinline__ void split_prep_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b,
                                                 int side) {
    // wave pw: SIMD-balanced assignment of (role, token half); roles 1 and 3 are the heavier ones
    const int pw = tid >> 6, c = tid & 63;
    const int h = pw >> 2;
    const int role = (h ? (pw ^ 1) : pw) & 3;
    const int T = (int)p.T;                              // the launcher admits T < 2^24 only
    const int64_t row_base = b * p.T;
    const Side sd = make_side(p, side);
    const Schedule<NB> sched(p.T, p.NC, p.C);
    const int total = sched.total;
    u32 bad = 0;
    // a stage as one int: first token of its block * 2 + (1 for a B stage)
    auto stage_at = [&](int s) -> int {
        const StageInfo si = sched.at(s);
        return ((si.chunk * p.C + si.block * CH_L) << 1) | (si.bmode ? 1 : 0);
    };

    PieceMap pm;
    {
        const int a0 = __builtin_amdgcn_readfirstlane(pw >> 1);   // pieces are ordered [array][token][8 pieces]
        pm.tok = (tid >> 3) & 15;
        pm.col = 8u * (tid & 7);
        pm.second = a0 < 2;
        pm.ld[0] = pick(a0, sd.src[0], sd.src[1], sd.src[2], sd.src[3], sd.src[4], sd.src[5]) + row_base * CH_N;
        pm.ld[1] = (a0 == 0 ? sd.src[4] : sd.src[5]) + row_base * CH_N;
        pm.fill = (a0 == R_GO || a0 == R_GW) ? (u32)IOE::ONE_BITS * 0x10001u : 0u;
    }

    // raw inputs of stage m live in RAW[m & 1]; stA / stB carry the even / odd stages, loaded two
    // iterations before they are parked in LDS (HBM latency is of the order of one iteration)
    RawRegs stA, stB;
    int cur = stage_at(0), nxt = cur;                  // stages s and s+1 of the loop below
    {
        raw_load(stA, pm, T, cur >> 1, cur & 1);
        raw_store(stA, pm, smem + SOFF_RAW, cur & 1, tid);
        if (total > 1) {
            nxt = stage_at(1);
            raw_load(stB, pm, T, nxt >> 1, nxt & 1);
            raw_store(stB, pm, smem + SOFF_RAW + RAW_BYTES, nxt & 1, tid);
        }
        __syncthreads();
        split_prep<IOE, OPE>(smem + SOFF_RAW, smem, role, h, c, cur & 1, side == 1, bad);
        __syncthreads();
    }
    int inA = cur, inB = cur;                          // the stages whose raw inputs stA / stB hold
    if (total > 2) {
        inA = stage_at(2);
        raw_load(stA, pm, T, inA >> 1, inA & 1);
    }
    if (total > 3) {
        inB = stage_at(3);
        raw_load(stB, pm, T, inB >> 1, inB & 1);
    }

    PHASE_BEGIN();
#define T2FW_SPLIT_ITERATION(s_, st, in)                                                                              \
    {                                                                                                                  \
        const int s = (s_);             /* st holds stage s+2 (= in), then takes stage s+4 */                          \
        PHASE_SELECT((cur & 1) ? 0 : 4);                                                                               \
        PHASE_MARK(0);                                                                                                 \
        if (s + 1 < total)                                                                                             \
            split_prep<IOE, OPE>(smem + SOFF_RAW + ((s + 1) & 1) * RAW_BYTES, smem + ((s + 1) & 1) * STAGE_BYTES,      \
                                 role, h, c, nxt & 1, side == 1, bad);                                                 \
        PHASE_MARK(2);                                                                                                 \
        cur = nxt;                                                                                                     \
        if (s + 2 < total) {                                                                                           \
            raw_store(st, pm, smem + SOFF_RAW + (s & 1) * RAW_BYTES, in & 1, tid);                                     \
            nxt = in;                                                                                                  \
        }                                                                                                              \
        if (s + 4 < total) {                                                                                           \
            in = stage_at(s + 4);                                                                                      \
            raw_load(st, pm, T, in >> 1, in & 1);                                                                      \
        }                                                                                                              \
        PHASE_MARK(1);                                                                                                 \
        __syncthreads();                                                                                               \
        PHASE_MARK(3);                                                                                                 \
    }
    for (int s2 = 0; s2 < total; s2 += 2) {
        T2FW_SPLIT_ITERATION(s2, stA, inA)
        if (s2 + 1 < total) T2FW_SPLIT_ITERATION(s2 + 1, stB, inB)
    }
#undef T2FW_SPLIT_ITERATION
    // Both workgroups of a row see all four gates' blocks and reach the same verdict, so either
    // order of their writes leaves the same flag.
    if (bad) p.row_flags[b] = 1;
    PHASE_END(4 + (tid >> 6));
}

template <typename IOE, typename OPE, int NB>
__device__ __forceinline__ void split_matrix_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b,
                                                   int side) {
    const int w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int ch = 16 * w + r;       // this lane's own-side channel
    const int T = (int)p.T;                              // the launcher admits T < 2^24 only
    const int64_t NC = p.NC;
    const int C = p.C;
    const u16 *ckpt = reinterpret_cast<const u16 *>(p.ckpt) + b * NC * (CH_N * CH_N);
    const int nb_last = (int)((p.T - (NC - 1) * C + CH_L - 1) / CH_L);
    // this batch row of the gradients this side writes
    u16 *const d_val = reinterpret_cast<u16 *>(side == 0 ? p.d_x : p.d_k) + b * p.T * CH_N;
    u16 *const d_gate = reinterpret_cast<u16 *>(side == 0 ? p.d_f : p.d_f_key) + b * p.T * CH_N;
    u16 *const d_adj = reinterpret_cast<u16 *>(p.d_q) + b * p.T * CH_N;

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
    if (tid == 0) p.row_flags[b] = 0;
    __syncthreads();      // raw inputs of the first stages are in LDS
    __syncthreads();      // operand tiles of stage 0 are in LDS
    PHASE_BEGIN();

    for (int64_t chunk = NC - 1; chunk >= 0; --chunk) {
        const int nb = chunk == NC - 1 ? nb_last : NB;
        take_state(pf, S);
        if (chunk > 0) load_state(ckpt + (chunk - 1) * (CH_N * CH_N), pf);
        // ---- R stages: block-start states, forward in time
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (i < nb) {
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
                const u16 *VOHc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_VOH * CM_TILE);
                const u16 *VHc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_VH * CM_TILE);
                const float *LX = reinterpret_cast<const float *>(stage + OFF_LX);
                const float *LO = reinterpret_cast<const float *>(stage + OFF_LO);
                {
                    const uint2 a0 = pack4v<OPE>(S[0]), a1 = pack4v<OPE>(S[1]), a2 = pack4v<OPE>(S[2]), a3 = pack4v<OPE>(S[3]);
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
                PHASE_MARK(0);
                __syncthreads();
                PHASE_MARK(3);
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
            us += __shfl_xor(us, 16, 64);
            us += __shfl_xor(us, 32, 64);
            carry = us;
        }
        // ---- B stages: blocks last to first
#pragma unroll
        for (int i = NB - 1; i >= 0; --i) {
            if (i < nb) {
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
                const u16 *AOS = reinterpret_cast<const u16 *>(stage + OFF_TM + TM_AOS * TM_TILE);
                const u16 *VOT = reinterpret_cast<const u16 *>(stage + OFF_TM + TM_VOT * TM_TILE);
                const u16 *VOH = reinterpret_cast<const u16 *>(stage + OFF_TM + TM_VOH * TM_TILE);
                const u16 *AOSc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_AOS * CM_TILE);
                const u16 *ASc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_AS * CM_TILE);
                const u16 *VTc = reinterpret_cast<const u16 *>(stage + OFF_CM + CM_VT * CM_TILE);
                const float *LX = reinterpret_cast<const float *>(stage + OFF_LX);
                const float *LO = reinterpret_cast<const float *>(stage + OFF_LO);
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
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
                floatx4 oa = OPE::mfma32(ld4(AOS + po + 8), sv[i][1], OPE::mfma32(ld4(AOS + po), sv[i][0], zero));
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
                    reverse_running_sum(du, carry, g, r);
                    const float *cf = reinterpret_cast<const float *>(stage + OFF_CF) + ch * CC + 4 * g;
                    const float4 rg = *reinterpret_cast<const float4 *>(cf + F_RG * (CF_TILE / 4));
                    const float4 ip = *reinterpret_cast<const float4 *>(cf + F_IP * (CF_TILE / 4));
                    const float rgv[4] = {rg.x, rg.y, rg.z, rg.w}, ipv[4] = {ip.x, ip.y, ip.z, ip.w};
                    // 16 lanes write 32 contiguous bytes of a token row; the four waves complete the row
                    const int tg = (int)chunk * C + i * CH_L + 4 * g;         // this lane's first token
                    const u32 go = (u32)tg * CH_N + (u32)ch;
#pragma unroll
                    for (int ii = 0; ii < 4; ++ii) {
                        if (tg + ii < T) {
                            d_val[go + ii * CH_N] = cvt1<IOE>(ipv[ii] * (va[ii] + asv[ii] * pd[ii]));
                            d_gate[go + ii * CH_N] = cvt1<IOE>(du[ii] * rgv[ii]);
                        }
                    }
                    if (side == 1) {
                        const float4 pp = *reinterpret_cast<const float4 *>(cf + F_PP * (CF_TILE / 4));
                        const float ppv[4] = {pp.x, pp.y, pp.z, pp.w};
#pragma unroll
                        for (int ii = 0; ii < 4; ++ii)
                            if (tg + ii < T) d_adj[go + ii * CH_N] = cvt1<IOE>(ppv[ii] * (oa[ii] + vtv[ii] * pd[ii]));
                    }
                }
                PHASE_MARK(1);
                __syncthreads();
                PHASE_MARK(2);
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

template <typename IOE, typename OPE, int NB>
__global__ __launch_bounds__(SP_THREADS) void lfw_bwd_split_kernel(ChunkBwdArgs p, int rows_padded) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    // blockIdx = side * rows_padded + row with rows_padded a multiple of 8: the two workgroups of a
    // row land on the same XCD and share its L2 for the inputs both of them read
    const int side = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - side * rows_padded;
    if (b >= p.B) return;
    // both branches execute exactly 2 + (number of stages) workgroup barriers
    if (tid < 256)
        split_matrix_waves<IOE, OPE, NB>(p, smem, tid, b, side);
    else
        split_prep_waves<IOE, OPE, NB>(p, smem, tid - 256, b, side);
}

template <typename IOE, typename OPE, int NB> int launch(const ChunkBwdArgs &a, hipStream_t stream) {
    auto kern = lfw_bwd_split_kernel<IOE, OPE, NB>;
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, SP_SMEM),
                       "hipFuncSetAttribute(split backward chunk kernel)");
    if (rc) return rc;
    if (a.B > 0x1fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    if (a.T >= CHUNK_SPLIT_MAX_T) return fail(T2FW_ERR_UNSUPPORTED, "T=%lld is too long for 32-bit row offsets", (long long)a.T);
    const int rows_padded = (int)((a.B + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(2u * (unsigned)rows_padded), dim3(SP_THREADS), SP_SMEM, stream, a, rows_padded);
    return check_hip(hipGetLastError(), "lfw_bwd_split_kernel launch");
}

template <typename IOE, typename OPE> int by_nb(const ChunkBwdArgs &a, hipStream_t stream) {
    if (a.C == 64) return launch<IOE, OPE, 4>(a, stream);
    if (a.C == 32) return launch<IOE, OPE, 2>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked backward kernel takes checkpoint intervals 32 or 64");
}

}  // namespace

int chunk_backward_split(const ChunkBwdArgs &a, int dtype, int op, hipStream_t stream) {
    if (dtype == T2FW_F16) return op == 1 ? by_nb<Fp16, Fp16>(a, stream) : by_nb<Fp16, Bf16>(a, stream);
    if (dtype == T2FW_BF16) return by_nb<Bf16, Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
