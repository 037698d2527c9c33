// Backward pass of the decay rule in chunked matrix-core form (algebra: lfw_chunk.hpp).
//
// With G = dL/dS flowing backwards in time, Gb the adjoint entering a 16-step block from
// the future, S0 the state at the block start and the block-local scalings of
// lfw_chunk.hpp (qs, kt, kh, xt, xh, gs = g*a_t):
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
// One workgroup (8 waves) per batch row.  Matrix wave w holds, in fp32 accumulators, the
// slabs S[16w.., :] / Gb[16w.., :] ("D copy", indexed [k][d]) and S[:, 16w..] / Gb[:, 16w..]
// ("K copy", indexed [d][k]) so that every contraction is local to a wave.  Chunks are
// visited last to first; inside a chunk a forward sweep ("R" stages) recomputes the
// block-start states from the checkpoint and keeps them as 16-bit operands in registers,
// then the blocks are visited last to first ("B" stages).  Four prep waves build the
// operand tiles of the next stage, prefetch raw inputs and write the previous stage's
// gradients; one barrier per stage.
//
// Replaces lfw_cuda_bwd_kernel and the six einsums of the reference
// (t2fw/csrc/lfw_kernel.cu:61-102, t2fw/csrc/lfw.cpp:84-93).
#include "lfw_chunk_bwd_dev.hpp"

namespace t2fw {
namespace {

using namespace bwd;

constexpr int BWD_THREADS = 512;
constexpr int CC = 20;   // channel-major 16-token tiles: row stride in elements

// ---- LDS layout of one stage buffer (bytes) ----------------------------------------------
constexpr int TM_TILE = CH_L * TS * 2;       // token-major 16-bit tile [16][TS]
constexpr int CM_TILE = CH_N * CC * 2;       // channel-major 16-bit tile [64][CC]
constexpr int CF_TILE = CH_N * CC * 4;       // channel-major fp32 tile [64][CC]
enum { T_QT = 0, T_KT, T_GT, T_XT, T_KH, T_XH, T_NUM };   // same order in both layouts
constexpr int OFF_TM = 0;
constexpr int OFF_CM = OFF_TM + T_NUM * TM_TILE;
enum { F_BT = 0, F_RFK, F_IA, F_RF, F_NUM };              // b_t, 1/fk_t, 1/a_t, 1/f_t
constexpr int OFF_CF = OFF_CM + T_NUM * CM_TILE;
constexpr int OFF_BLV = OFF_CF + F_NUM * CF_TILE;          // b_L [64] f32
constexpr int OFF_ALV = OFF_BLV + CH_N * 4;                // a_L [64] f32
constexpr int STAGE_BYTES = OFF_ALV + CH_N * 4;
constexpr int BOUT_TILE = CH_L * OS * 2;                   // one gradient tile [16][OS] u16
enum { O_DX = 0, O_DF, O_DQ, O_DK, O_DFK, O_NUM };
constexpr int BOUT_BYTES = O_NUM * BOUT_TILE;
constexpr int BRAW_ARRAY = CH_L * CH_N * 2;                // [16][64] u16
enum { R_FK = 0, R_K, R_F, R_X, R_Q, R_G, R_NUM };         // R stages need the first four only
constexpr int BRAW_BYTES = R_NUM * BRAW_ARRAY;
constexpr int BOFF_OUT = 2 * STAGE_BYTES;
constexpr int BOFF_RAW = BOFF_OUT + 2 * BOUT_BYTES;
constexpr int BWD_SMEM = BOFF_RAW + 2 * BRAW_BYTES;
static_assert(BWD_SMEM <= 160 * 1024, "backward stage buffers exceed the LDS of one CU");

// ---- raw staging -------------------------------------------------------------------------
// A stage's raw inputs are R_NUM arrays of [16 tokens][64 channels]: 768 pieces of 16 bytes,
// three per prep thread.  Everything that does not depend on the stage is worked out once per
// thread (PieceMap), so that issuing a stage's loads costs a handful of instructions.
struct BStage {
    uint4 v[3];
};

struct PieceMap {
    const u16 *ld[3];     // source of raw piece m at token offset 0 of this batch row
    u16 *st[3];           // destination of gradient piece m at token offset 0 (null: no such piece)
    int arr[3];           // raw array index of piece m
    int tok[3];           // token inside the block
    u32 fill[3];          // identity fill for steps past the end of the sequence
    int out_off[3];       // byte offset of gradient piece m inside one OUT buffer
};

__device__ __forceinline__ void bstage_load(BStage &st, const PieceMap &pm, int64_t T, int64_t t0, bool bmode) {
    const int narr = bmode ? R_NUM : 4;
#pragma unroll
    for (int m = 0; m < 3; ++m) {
        if (pm.arr[m] < narr) {
            if (t0 + pm.tok[m] < T)
                st.v[m] = *reinterpret_cast<const uint4 *>(pm.ld[m] + t0 * CH_N);
            else
                st.v[m] = make_uint4(pm.fill[m], pm.fill[m], pm.fill[m], pm.fill[m]);
        }
    }
}

__device__ __forceinline__ void bstage_store(const BStage &st, const PieceMap &pm, unsigned char *raw, bool bmode,
                                             int tid) {
    const int narr = bmode ? R_NUM : 4;
#pragma unroll
    for (int m = 0; m < 3; ++m)
        if (pm.arr[m] < narr) *reinterpret_cast<uint4 *>(raw + (tid + 256 * m) * 16) = st.v[m];
}

// column of one raw array for channel c
__device__ __forceinline__ void raw_col(u16 (&dst)[CH_L], const unsigned char *raw, int array, int c) {
    const u16 *base = reinterpret_cast<const u16 *>(raw + array * BRAW_ARRAY) + c;
#pragma unroll
    for (int t = 0; t < CH_L; ++t) dst[t] = base[t * CH_N];
}

template <typename OPE>
__device__ __forceinline__ void write_tm(unsigned char *stage, int tile, int c, const float (&v)[CH_L]) {
    u16 *tm = reinterpret_cast<u16 *>(stage + OFF_TM + tile * TM_TILE);
#pragma unroll
    for (int t = 0; t < CH_L; ++t) tm[t * TS + c] = cvt1<OPE>(v[t]);
}

template <typename OPE>
__device__ __forceinline__ void write_cm(unsigned char *stage, int tile, int c, const float (&v)[CH_L]) {
    uint2 *cm = reinterpret_cast<uint2 *>(stage + OFF_CM + tile * CM_TILE + c * CC * 2);
#pragma unroll
    for (int t = 0; t < CH_L; t += 4) cm[t / 4] = packq<OPE>(v[t], v[t + 1], v[t + 2], v[t + 3]);
}

__device__ __forceinline__ void write_cf(unsigned char *stage, int tile, int c, const float (&v)[CH_L]) {
    float4 *cf = reinterpret_cast<float4 *>(stage + OFF_CF + tile * CF_TILE + c * CC * 4);
#pragma unroll
    for (int t = 0; t < CH_L; t += 4) cf[t / 4] = make_float4(v[t], v[t + 1], v[t + 2], v[t + 3]);
}

// One prep wave, one role (role = prep wave index 0..3), channel c:
//   role 0: key gate prefix -> qs tiles, b_t, 1/fk_t            role 1: key gate suffix -> kh, kt tiles, b_L
//   role 2: value gate prefix -> gs tiles, 1/f_t                role 3: value gate suffix -> xh, xt tiles, 1/a_t, a_L
// In R stages only roles 1 and 3 work and only the channel-major kh / xh tiles and a_L, b_L are made.
template <typename IOE, typename OPE>
__device__ __forceinline__ void bwd_prep(const unsigned char *raw, unsigned char *stage, int role, int c, bool bmode,
                                         u32 &bad) {
    const bool kside = role < 2;
    const bool prefix_role = (role & 1) == 0;
    if (!bmode && prefix_role) return;
    u16 gr[CH_L], ar[CH_L];
    raw_col(gr, raw, kside ? R_FK : R_F, c);
    raw_col(ar, raw, prefix_role ? (kside ? R_Q : R_G) : (kside ? R_K : R_X), c);
    float gate[CH_L];
#pragma unroll
    for (int t = 0; t < CH_L; ++t) gate[t] = IOE::to_f32(gr[t]);
    if (prefix_role) {
        float pre[CH_L], v[CH_L], rg[CH_L];
        pre[0] = gate[0];
#pragma unroll
        for (int t = 1; t < CH_L; ++t) pre[t] = pre[t - 1] * gate[t];
#pragma unroll
        for (int t = 0; t < CH_L; ++t) {
            v[t] = IOE::to_f32(ar[t]) * pre[t];            // qs or gs
            rg[t] = __builtin_amdgcn_rcpf(gate[t]);        // 1/fk_t or 1/f_t
        }
        write_tm<OPE>(stage, kside ? T_QT : T_GT, c, v);
        write_cm<OPE>(stage, kside ? T_QT : T_GT, c, v);
        write_cf(stage, kside ? F_RFK : F_RF, c, rg);
        if (kside) write_cf(stage, F_BT, c, pre);
    } else {
        bad |= gate_check<IOE>(gr);
        float tot = gate[0];
#pragma unroll
        for (int t = 1; t < CH_L; ++t) tot *= gate[t];
        bad |= (tot >= OPE::MIN_PRODUCT) ? 0u : 1u;
        const float itot = __builtin_amdgcn_rcpf(tot);
        float hat[CH_L], til[CH_L], inv[CH_L];
        float sfx = 1.0f;
#pragma unroll
        for (int t = CH_L - 1; t >= 0; --t) {
            inv[t] = sfx * itot;                            // 1 / prefix_t
            hat[t] = IOE::to_f32(ar[t]) * sfx;              // kh or xh
            til[t] = hat[t] * itot;                         // kt or xt
            sfx *= gate[t];
        }
        write_cm<OPE>(stage, kside ? T_KH : T_XH, c, hat);
        reinterpret_cast<float *>(stage + (kside ? OFF_BLV : OFF_ALV))[c] = tot;
        if (bmode) {
            write_tm<OPE>(stage, kside ? T_KH : T_XH, c, hat);
            write_tm<OPE>(stage, kside ? T_KT : T_XT, c, til);
            write_cm<OPE>(stage, kside ? T_KT : T_XT, c, til);
            if (!kside) write_cf(stage, F_IA, c, inv);
        }
    }
}

template <typename IOE, typename OPE, int NB>
__device__ __forceinline__ void bwd_prep_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b) {
    const int role = tid >> 6, c = tid & 63;
    const int64_t T = p.T;
    const int64_t row_base = b * T;
    const u16 *const src[R_NUM] = {reinterpret_cast<const u16 *>(p.f_key), reinterpret_cast<const u16 *>(p.k),
                                   reinterpret_cast<const u16 *>(p.f),     reinterpret_cast<const u16 *>(p.x),
                                   reinterpret_cast<const u16 *>(p.q),     reinterpret_cast<const u16 *>(p.g_out)};
    u16 *const dst[O_NUM] = {reinterpret_cast<u16 *>(p.d_x), reinterpret_cast<u16 *>(p.d_f),
                             reinterpret_cast<u16 *>(p.d_q), reinterpret_cast<u16 *>(p.d_k),
                             reinterpret_cast<u16 *>(p.d_f_key)};
    const Schedule<NB> sched(T, p.NC, p.C);
    const int total = sched.total;
    u32 bad = 0;
    if (tid == 0) {      // both flag slots of the row (the backward kernels report in the first)
        p.row_flags[b] = 0;
        p.row_flags[chunk_rows_padded(p.B) + b] = 0;
    }
    auto tok0_of = [&](const StageInfo &si) -> int64_t { return (int64_t)si.chunk * p.C + si.block * CH_L; };

    PieceMap pm;
#pragma unroll
    for (int m = 0; m < 3; ++m) {
        const int pi = tid + 256 * m;              // [array or gradient][token][8 pieces]
        const int a = pi >> 7, tok = (pi >> 3) & 15, piece = pi & 7;
        const int64_t off = (row_base + tok) * CH_N + 8 * piece;
        pm.arr[m] = a;
        pm.tok[m] = tok;
        pm.ld[m] = src[a] + off;                   // a <= 5 for every piece
        pm.fill[m] = (a == R_FK || a == R_F) ? (u32)IOE::ONE_BITS * 0x10001u : 0u;
        pm.st[m] = a < O_NUM ? dst[a] + off : nullptr;
        pm.out_off[m] = a * BOUT_TILE + (tok * OS + 8 * piece) * 2;
    }

    // raw inputs of stage m live in RAW[m & 1]; stA / stB carry the even / odd stages two ahead
    BStage stA, stB;
    {
        const StageInfo s0 = sched.at(0);
        bstage_load(stA, pm, T, tok0_of(s0), s0.bmode);
        bstage_store(stA, pm, smem + BOFF_RAW, s0.bmode, tid);
        if (total > 1) {
            const StageInfo s1 = sched.at(1);
            bstage_load(stB, pm, T, tok0_of(s1), s1.bmode);
            bstage_store(stB, pm, smem + BOFF_RAW + BRAW_BYTES, s1.bmode, tid);
        }
        if (total > 2) {
            const StageInfo s2 = sched.at(2);
            bstage_load(stA, pm, T, tok0_of(s2), s2.bmode);
        }
        if (total > 3) {
            const StageInfo s3 = sched.at(3);
            bstage_load(stB, pm, T, tok0_of(s3), s3.bmode);
        }
        __syncthreads();
        bwd_prep<IOE, OPE>(smem + BOFF_RAW, smem, role, c, s0.bmode, bad);
        __syncthreads();
    }

    auto store_out = [&](int s) {       // gradients of B stage s: LDS tiles -> global, 16 B pieces
        const StageInfo si = sched.at(s);
        if (!si.bmode) return;
        const unsigned char *outp = smem + BOFF_OUT + (s & 1) * BOUT_BYTES;
        const int64_t t0 = tok0_of(si);
#pragma unroll
        for (int m = 0; m < 3; ++m) {
            if (pm.st[m] != nullptr && t0 + pm.tok[m] < T) {
                const u16 *tile = reinterpret_cast<const u16 *>(outp + pm.out_off[m]);
                const uint2 lo = *reinterpret_cast<const uint2 *>(tile);
                const uint2 hi = *reinterpret_cast<const uint2 *>(tile + 4);
                *reinterpret_cast<uint4 *>(pm.st[m] + t0 * CH_N) = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        }
    };

    PHASE_BEGIN();
    auto iteration = [&](int s, BStage &st) {       // st holds stage s+2, then takes stage s+4
        PHASE_SELECT(sched.at(s).bmode ? 0 : 4);
        if (s + 2 < total) bstage_store(st, pm, smem + BOFF_RAW + (s & 1) * BRAW_BYTES, sched.at(s + 2).bmode, tid);
        PHASE_MARK(1);
        if (s > 0) store_out(s - 1);
        if (s + 4 < total) {
            const StageInfo s4 = sched.at(s + 4);
            bstage_load(st, pm, T, tok0_of(s4), s4.bmode);
        }
        PHASE_MARK(0);
        if (s + 1 < total)
            bwd_prep<IOE, OPE>(smem + BOFF_RAW + ((s + 1) & 1) * BRAW_BYTES, smem + ((s + 1) & 1) * STAGE_BYTES, role, c,
                               sched.at(s + 1).bmode, bad);
        PHASE_MARK(2);
        __syncthreads();
        PHASE_MARK(3);
    };
    for (int s = 0; s < total; s += 2) {
        iteration(s, stA);
        if (s + 1 < total) iteration(s + 1, stB);
    }
    store_out(total - 1);
    if (bad) p.row_flags[b] = 1;
    PHASE_END(4 + (tid >> 6));
}

// helpers of the matrix waves ----------------------------------------------------------------
__device__ __forceinline__ const u16 *tm_tile(const unsigned char *stage, int tile) {
    return reinterpret_cast<const u16 *>(stage + OFF_TM + tile * TM_TILE);
}
__device__ __forceinline__ const u16 *cm_tile(const unsigned char *stage, int tile) {
    return reinterpret_cast<const u16 *>(stage + OFF_CM + tile * CM_TILE);
}
__device__ __forceinline__ const float *cf_tile(const unsigned char *stage, int tile) {
    return reinterpret_cast<const float *>(stage + OFF_CF + tile * CF_TILE);
}
template <typename IOE, typename OPE, int NB>
__device__ __forceinline__ void bwd_matrix_waves(const ChunkBwdArgs &p, unsigned char *smem, int tid, int64_t b) {
    const int w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int ch = 16 * w + r;       // this lane's d in the D copies and its k in the K copies
    const int64_t T = p.T, NC = p.NC;
    const int C = p.C;
    const u16 *ckpt = reinterpret_cast<const u16 *>(p.ckpt) + b * NC * (CH_N * CH_N);
    const int nb_last = (int)((T - (NC - 1) * C + CH_L - 1) / CH_L);

    floatx4 Sd[4], Sk[4], Gd[4], Gk[4];
    uint2 svd[NB][4], svk[NB][4];     // block-start states as 16-bit MFMA operands
    uint2 pfd[4];                     // checkpoint prefetch: D copy rows (4 values each)
    u16 pfk[16];                      //                      K copy column
    auto ckpt_issue = [&](int64_t chunk) {
        const u16 *ck = ckpt + chunk * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            pfd[j] = ld2(ck + ch * CH_N + 16 * j + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; ++i) pfk[4 * j + i] = ck[(16 * j + 4 * g + i) * CH_N + ch];
        }
    };
    auto ckpt_take = [&]() {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float t[4];
            unpack4<IOE>(pfd[j], t);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                Sd[j][i] = t[i];
                Sk[j][i] = IOE::to_f32(pfk[4 * j + i]);
            }
        }
    };
    {   // incoming state gradient
        const u16 *gs = reinterpret_cast<const u16 *>(p.g_state) + b * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float t[4];
            unpack4<IOE>(ld2(gs + ch * CH_N + 16 * j + 4 * g), t);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                Gd[j][i] = t[i];
                Gk[j][i] = IOE::to_f32(gs[(16 * j + 4 * g + i) * CH_N + ch]);
            }
        }
    }
    ckpt_issue(NC - 1);
    float u_carry = 0.f, v_carry = 0.f;
    int64_t s = 0;
    __syncthreads();      // raw inputs of the first stages are in LDS
    __syncthreads();      // operand tiles of stage 0 are in LDS
    PHASE_BEGIN();

    for (int64_t chunk = NC - 1; chunk >= 0; --chunk) {
        const int nb = chunk == NC - 1 ? nb_last : NB;
        ckpt_take();
        if (chunk > 0) ckpt_issue(chunk - 1);
        // ---- R stages: block-start states, forward in time
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (i < nb) {
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
                const u16 *KHc = cm_tile(stage, T_KH), *XHc = cm_tile(stage, T_XH);
                const float *BLV = reinterpret_cast<const float *>(stage + OFF_BLV);
                const float *ALV = reinterpret_cast<const float *>(stage + OFF_ALV);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    svd[i][j] = pack4v<OPE>(Sd[j]);
                    svk[i][j] = pack4v<OPE>(Sk[j]);
                }
                const float aL = ALV[ch], bL = BLV[ch];
                const uint2 xh_d = ld2(XHc + ch * CC + 4 * g), kh_k = ld2(KHc + ch * CC + 4 * g);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float4 bl = *reinterpret_cast<const float4 *>(BLV + 16 * j + 4 * g);
                    const float4 al = *reinterpret_cast<const float4 *>(ALV + 16 * j + 4 * g);
                    Sd[j][0] *= aL * bl.x; Sd[j][1] *= aL * bl.y; Sd[j][2] *= aL * bl.z; Sd[j][3] *= aL * bl.w;
                    Sk[j][0] *= al.x * bL; Sk[j][1] *= al.y * bL; Sk[j][2] *= al.z * bL; Sk[j][3] *= al.w * bL;
                    Sd[j] = OPE::mfma16(ld2(KHc + (16 * j + r) * CC + 4 * g), xh_d, Sd[j]);
                    Sk[j] = OPE::mfma16(ld2(XHc + (16 * j + r) * CC + 4 * g), kh_k, Sk[j]);
                }
                PHASE_MARK(0);
                __syncthreads();
                PHASE_MARK(3);
                ++s;
            }
        }
        // ---- re-anchor the running sums: u = rowsum(Gb * S_end), v = colsum(Gb * S_end)
        {
            float us = 0.f, vs = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    us += Gd[j][i] * Sd[j][i];
                    vs += Gk[j][i] * Sk[j][i];
                }
            us += __shfl_xor(us, 16, 64);
            us += __shfl_xor(us, 32, 64);
            vs += __shfl_xor(vs, 16, 64);
            vs += __shfl_xor(vs, 32, 64);
            u_carry = us;
            v_carry = vs;
        }
        // ---- B stages: blocks last to first
#pragma unroll
        for (int i = NB - 1; i >= 0; --i) {
            if (i < nb) {
                const unsigned char *stage = smem + (s & 1) * STAGE_BYTES;
                unsigned char *outp = smem + BOFF_OUT + (s & 1) * BOUT_BYTES;
                const u16 *QT = tm_tile(stage, T_QT), *KT = tm_tile(stage, T_KT), *GT = tm_tile(stage, T_GT);
                const u16 *XT = tm_tile(stage, T_XT), *KH = tm_tile(stage, T_KH), *XH = tm_tile(stage, T_XH);
                const u16 *QTc = cm_tile(stage, T_QT), *KTc = cm_tile(stage, T_KT), *GTc = cm_tile(stage, T_GT);
                const u16 *XTc = cm_tile(stage, T_XT);
                const float *BLV = reinterpret_cast<const float *>(stage + OFF_BLV);
                const float *ALV = reinterpret_cast<const float *>(stage + OFF_ALV);
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                // the four 16x16 token-token products (full contraction over 64 channels each)
                const int ro = r * TS + 8 * g;
                const uint4 kt_lo = ld4(KT + ro), kt_hi = ld4(KT + ro + 32), qt_lo = ld4(QT + ro), qt_hi = ld4(QT + ro + 32);
                const uint4 gt_lo = ld4(GT + ro), gt_hi = ld4(GT + ro + 32), xt_lo = ld4(XT + ro), xt_hi = ld4(XT + ro + 32);
                floatx4 pt1 = OPE::mfma32(kt_hi, qt_hi, OPE::mfma32(kt_lo, qt_lo, zero));   // P[t=r][s=4g+i]
                floatx4 pt2 = OPE::mfma32(qt_hi, kt_hi, OPE::mfma32(qt_lo, kt_lo, zero));   // P[r'=4g+i][t=r]
                floatx4 wt1 = OPE::mfma32(xt_hi, gt_hi, OPE::mfma32(xt_lo, gt_lo, zero));   // W[t=r][s=4g+i]
                floatx4 wt2 = OPE::mfma32(gt_hi, xt_hi, OPE::mfma32(gt_lo, xt_lo, zero));   // W[r'=4g+i][t=r]
                float pd[4], wd[4];     // diagonals for this lane's tokens 4g+i
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    pd[ii] = __shfl(pt1[ii], 20 * g + ii, 64);
                    wd[ii] = __shfl(wt1[ii], 20 * g + ii, 64);
                }
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    const bool lower = 4 * g + ii < r, upper = 4 * g + ii > r;
                    pt1[ii] = lower ? pt1[ii] : 0.f;
                    wt1[ii] = lower ? wt1[ii] : 0.f;
                    pt2[ii] = upper ? pt2[ii] : 0.f;
                    wt2[ii] = upper ? wt2[ii] : 0.f;
                }
                const uint2 pa_o = pack4v<OPE>(pt1), pa_x = pack4v<OPE>(pt2), pa_q = pack4v<OPE>(wt1), pa_k = pack4v<OPE>(wt2);
                const uint2 xtc = ld2(XTc + ch * CC + 4 * g), gtc = ld2(GTc + ch * CC + 4 * g);
                const uint2 ktc = ld2(KTc + ch * CC + 4 * g), qtc = ld2(QTc + ch * CC + 4 * g);
                const float aL = ALV[ch], bL = BLV[ch];
                const int po = r * TS + 4 * g;
                // o' and dq' use the block-start state
                floatx4 oa = OPE::mfma32(cat(ld2(QT + po), ld2(QT + po + 16)), cat(svd[i][0], svd[i][1]), zero);
                oa = OPE::mfma32(cat(ld2(QT + po + 32), ld2(QT + po + 48)), cat(svd[i][2], svd[i][3]), oa);
                oa += OPE::mfma16(pa_o, xtc, zero);
                floatx4 dqa = OPE::mfma32(cat(ld2(GT + po), ld2(GT + po + 16)), cat(svk[i][0], svk[i][1]), zero);
                dqa = OPE::mfma32(cat(ld2(GT + po + 32), ld2(GT + po + 48)), cat(svk[i][2], svk[i][3]), dqa);
                dqa += OPE::mfma16(pa_q, ktc, zero);
                // dx' and dk' use the adjoint entering the block, scaled to the block end on one side
                floatx4 ga[4], gb[4];
                uint2 gap[4], gbp[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    ga[j] = Gd[j] * aL;
                    gb[j] = Gk[j] * bL;
                    gap[j] = pack4v<OPE>(ga[j]);
                    gbp[j] = pack4v<OPE>(gb[j]);
                }
                floatx4 dxa = OPE::mfma32(cat(ld2(KH + po), ld2(KH + po + 16)), cat(gap[0], gap[1]), zero);
                dxa = OPE::mfma32(cat(ld2(KH + po + 32), ld2(KH + po + 48)), cat(gap[2], gap[3]), dxa);
                dxa += OPE::mfma16(pa_x, gtc, zero);
                floatx4 dka = OPE::mfma32(cat(ld2(XH + po), ld2(XH + po + 16)), cat(gbp[0], gbp[1]), zero);
                dka = OPE::mfma32(cat(ld2(XH + po + 32), ld2(XH + po + 48)), cat(gbp[2], gbp[3]), dka);
                dka += OPE::mfma16(pa_k, qtc, zero);
                // adjoint of the previous block: Gb <- (a_L (x) b_L) * Gb + sum_t gs_t (x) qs_t
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float4 bl = *reinterpret_cast<const float4 *>(BLV + 16 * j + 4 * g);
                    const float4 al = *reinterpret_cast<const float4 *>(ALV + 16 * j + 4 * g);
                    ga[j][0] *= bl.x; ga[j][1] *= bl.y; ga[j][2] *= bl.z; ga[j][3] *= bl.w;
                    gb[j][0] *= al.x; gb[j][1] *= al.y; gb[j][2] *= al.z; gb[j][3] *= al.w;
                    Gd[j] = OPE::mfma16(ld2(QTc + (16 * j + r) * CC + 4 * g), gtc, ga[j]);
                    Gk[j] = OPE::mfma16(ld2(GTc + (16 * j + r) * CC + 4 * g), qtc, gb[j]);
                }
                // ---- value side: d_x, d_f for tokens 4g+i, channel ch
                {
                    float gsv[4], xtv[4], du[4];
                    unpack4<OPE>(gtc, gsv);
                    unpack4<OPE>(xtc, xtv);
#pragma unroll
                    for (int ii = 0; ii < 4; ++ii) du[ii] = oa[ii] * gsv[ii] - dxa[ii] * xtv[ii];
                    reverse_running_sum(du, u_carry, g, r);
                    const float4 rf = *reinterpret_cast<const float4 *>(cf_tile(stage, F_RF) + ch * CC + 4 * g);
                    const float4 ia = *reinterpret_cast<const float4 *>(cf_tile(stage, F_IA) + ch * CC + 4 * g);
                    const float rfv[4] = {rf.x, rf.y, rf.z, rf.w}, iav[4] = {ia.x, ia.y, ia.z, ia.w};
                    u16 *DX = reinterpret_cast<u16 *>(outp + O_DX * BOUT_TILE), *DF = reinterpret_cast<u16 *>(outp + O_DF * BOUT_TILE);
#pragma unroll
                    for (int ii = 0; ii < 4; ++ii) {
                        DX[(4 * g + ii) * OS + ch] = cvt1<IOE>(iav[ii] * (dxa[ii] + gsv[ii] * pd[ii]));
                        DF[(4 * g + ii) * OS + ch] = cvt1<IOE>(du[ii] * rfv[ii]);
                    }
                }
                // ---- key side: d_q, d_k, d_f_key for tokens 4g+i, channel ch
                {
                    float qsv[4], ktv[4], dv[4];
                    unpack4<OPE>(qtc, qsv);
                    unpack4<OPE>(ktc, ktv);
#pragma unroll
                    for (int ii = 0; ii < 4; ++ii) dv[ii] = dqa[ii] * qsv[ii] - dka[ii] * ktv[ii];
                    reverse_running_sum(dv, v_carry, g, r);
                    const float4 bt = *reinterpret_cast<const float4 *>(cf_tile(stage, F_BT) + ch * CC + 4 * g);
                    const float4 rk = *reinterpret_cast<const float4 *>(cf_tile(stage, F_RFK) + ch * CC + 4 * g);
                    const float btv[4] = {bt.x, bt.y, bt.z, bt.w}, rkv[4] = {rk.x, rk.y, rk.z, rk.w};
                    u16 *DQ = reinterpret_cast<u16 *>(outp + O_DQ * BOUT_TILE), *DK = reinterpret_cast<u16 *>(outp + O_DK * BOUT_TILE);
                    u16 *DFK = reinterpret_cast<u16 *>(outp + O_DFK * BOUT_TILE);
#pragma unroll
                    for (int ii = 0; ii < 4; ++ii) {
                        DQ[(4 * g + ii) * OS + ch] = cvt1<IOE>(btv[ii] * (dqa[ii] + ktv[ii] * wd[ii]));
                        DK[(4 * g + ii) * OS + ch] =
                            cvt1<IOE>(__builtin_amdgcn_rcpf(btv[ii]) * (dka[ii] + qsv[ii] * wd[ii]));
                        DFK[(4 * g + ii) * OS + ch] = cvt1<IOE>(dv[ii] * rkv[ii]);
                    }
                }
                PHASE_MARK(1);
                __syncthreads();
                PHASE_MARK(2);
                ++s;
            }
        }
    }
    // d_s0 = adjoint after the first block
    {
        u16 *ds = reinterpret_cast<u16 *>(p.d_s0) + b * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint2 *>(ds + ch * CH_N + 16 * j + 4 * g) = pack4v<IOE>(Gd[j]);
    }
    PHASE_END(tid >> 6);
}

template <typename IOE, typename OPE, int NB>
__global__ __launch_bounds__(BWD_THREADS) void lfw_bwd_chunk_kernel(ChunkBwdArgs p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int64_t b = blockIdx.x;
    // both branches execute exactly 2 + (number of stages) workgroup barriers
    if (tid < 256)
        bwd_matrix_waves<IOE, OPE, NB>(p, smem, tid, b);
    else
        bwd_prep_waves<IOE, OPE, NB>(p, smem, tid - 256, b);
}

template <typename IOE, typename OPE, int NB> int launch(const ChunkBwdArgs &a, hipStream_t stream) {
    auto kern = lfw_bwd_chunk_kernel<IOE, OPE, NB>;
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, BWD_SMEM),
                       "hipFuncSetAttribute(backward chunk kernel)");
    if (rc) return rc;
    if (a.B > 0x7fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    hipLaunchKernelGGL(kern, dim3((unsigned)a.B), dim3(BWD_THREADS), BWD_SMEM, stream, a);
    return check_hip(hipGetLastError(), "lfw_bwd_chunk_kernel launch");
}

template <typename IOE, typename OPE> int by_nb(const ChunkBwdArgs &a, hipStream_t stream) {
    if (a.C == 64) return launch<IOE, OPE, 4>(a, stream);
    if (a.C == 32) return launch<IOE, OPE, 2>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked backward kernel takes checkpoint intervals 32 or 64");
}

}  // namespace

int chunk_backward(const ChunkBwdArgs &a, int dtype, int op, hipStream_t stream) {
    if (dtype == T2FW_F16) return op == 1 ? by_nb<Fp16, Fp16>(a, stream) : by_nb<Fp16, Bf16>(a, stream);
    if (dtype == T2FW_BF16) return by_nb<Bf16, Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
