// Backward pass of the delta rule on the matrix cores, D = M = 64, fp32 / fp16 / bf16 tensors (block algebra,
// precision, element types and staging: dfw_chunk.hpp).  Blocks of 16 steps are visited last to first.  With g = dL/dO of the block,
// G_end the adjoint of the state after it, Delta the block's saved deltas and Tm = (I + A)^-1:
//   dDelta = Bq^T g + K G_end^T            dU = Tm^T dDelta  (= d_value)
//   G_start = G_end + g^T Q - dU^T K       (d_state = G before the first block)
//   S0 = S_end - Delta^T K                 (the state walked backwards from final_state, as the reference does)
//   d_query = g S0 + X1 K                  X1[t][s] = g_t . delta_s   (s < t)
//   d_key   = X1^T Q + Delta G_end - dU S0 + (X2 + X2^T) K            X2[t][s] = -dU_t . delta_s  (s < t)
// Two launches, as in the reference (t2fw/csrc/dfw_kernel.cu:203-283 and :290-384):
//   value side  one workgroup per (row, half of the value channels): G rows in fp32 accumulators; writes d_value
//               and d_state.  Its chain per block is  G_end -> dU = Tm^T Bq^T g + (Tm^T K) G_end^T -> G_start,
//               with Tm, Bq and K'' = Tm^T K prepared ahead by the matrix waves.
//   key side    one workgroup per (row, half of the key channels): columns of S and of G in fp32 accumulators,
//               both plain running sums (it reads d_value from the first launch); writes d_query and d_key.
#include <type_traits>
#include "common.hpp"
#include "dfw_chunk.hpp"
#include "dfw_scan.hpp"

namespace t2fw {
namespace {

using namespace dfwc;

constexpr int BW_THREADS = 512;

// ---- value side -----------------------------------------------------------------------------------------
constexpr int VS_KT = 0, VS_QT = VS_KT + 2 * TM_TILE, VS_KC = VS_QT + 2 * TM_TILE, VS_QC = VS_KC + 2 * CM_TILE,
              VS_RAW_BLOCK = VS_QC + 2 * CM_TILE;
constexpr int VS_KPP = 0, VS_TM = VS_KPP + 2 * TM_TILE, VS_BQ = VS_TM + 2 * ST_TILE, VS_ST_BLOCK = VS_BQ + 2 * ST_TILE;
using VsRing = Ring<VS_RAW_BLOCK, VS_ST_BLOCK, DNB>;
static_assert(VsRing::SMEM <= 160 * 1024, "value-side tiles exceed the LDS of one CU");

// first token of block `bb` of a stage when the blocks are visited last to first
__device__ __forceinline__ int reverse_tok0(int nblocks, int nblk_per_stage, int stage, int bb) {
    return (nblocks - 1 - (stage * nblk_per_stage + bb)) * DL;
}

template <bool SP> __device__ __forceinline__ void vs_structure_wave(unsigned char *smem, int nstages, int bb, int lane) {
    const int r = lane & 15, g = lane >> 4;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    for (int tick = 0; tick < nstages + 2; ++tick) {
        const int stage = tick - 1;
        if (stage >= 0 && stage < nstages) {
            const unsigned char *raw = VsRing::raw(smem, stage, bb);
            const TmTile<SP> KT(raw + VS_KT), QT(raw + VS_QT);
            const CmTile<SP> KC(raw + VS_KC);
            const Sp4<SP> k0 = KT.any_order(r, g, 0), k1 = KT.any_order(r, g, 1);
            const Sp4<SP> q0 = QT.any_order(r, g, 0), q1 = QT.any_order(r, g, 1);
            const floatx4 kk = mma32(k1, k1, mma32(k0, k0, zero));
            const floatx4 qk = mma32(q1, k1, mma32(q0, k0, zero));      // [t = 4g+e][s = r] = q_t . k_s
            floatx4 bq;
#pragma unroll
            for (int e = 0; e < 4; ++e) bq[e] = r < 4 * g + e ? qk[e] : 0.f;       // Bq[t][s] for s < t
            const BlockInverse<SP> inv(kk, r, g);
            const Sp2<SP> tm = split4<SP>(inv.acc_tm());
            unsigned char *st = VsRing::st(smem, stage, bb);
            st_store<SP>(st + VS_TM, lane, tm);
            st_store<SP>(st + VS_BQ, lane, split4<SP>(bq));
            // K''^T tile j: [m = 16 j + 4 g + e][t = r] = sum_s K[s][m] Tm[s][t]   (K'' = Tm^T K)
            floatx4 kpp[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) kpp[j] = mma16(KC.tokens(16 * j + r, g), tm, zero);
            store_tm_from_acc<SP>(st + VS_KPP, r, g, kpp);
        }
        __syncthreads();
    }
}

template <bool SP, typename E> __device__ __forceinline__ void vs_slab_wave(const DfwBwdArgs &p, unsigned char *smem, int64_t b, int d0, int nstages, int lane) {
    typedef typename E::elem elem;
    const int r = lane & 15, g = lane >> 4, d = d0 + r, T = (int)p.T, nblocks = nstages * DNB;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    const elem *const go = reinterpret_cast<const elem *>(p.g_out) + b * p.T * CH_N;
    elem *const d_v = reinterpret_cast<elem *>(p.d_v) + b * p.T * CH_N;
    const u32 lane_off = (u32)(4 * g * CH_N + d);
    // G[j][e] = G[d][16 j + 4 g + e]
    floatx4 G[4];
    {
        const elem *gs = reinterpret_cast<const elem *>(p.g_state) + (b * CH_N + d) * CH_N + 4 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) G[j] = E::load4(gs + 16 * j);
    }
    // g of a stage as loaded, one stage ahead (converted where the stage uses it)
    struct GRaw {
        elem x[DNB][4];
    };
    auto load_g = [&](GRaw &x, int stage) {
#pragma unroll
        for (int bb = 0; bb < DNB; ++bb)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                x.x[bb][e] = go[(size_t)min(reverse_tok0(nblocks, DNB, stage, bb) + 4 * g + e, T - 1) * CH_N + d];
    };
    // One stage.  FULL: every token of the stage is below T and the body has no branch.  (The waits that the
    // compiler places count outstanding memory operations along every path: a path that skips stores, or loads
    // still pending where the loop is entered, would make each stage wait for the stores of the stage before.)
    auto stage_body = [&](auto full, int stage, GRaw &graw, GRaw &gnxt) {
        constexpr bool FULL = decltype(full)::value;
        load_g(gnxt, min(stage + 1, nstages - 1));
#pragma unroll
        for (int bb = 0; bb < DNB; ++bb) {
            const int tok0 = reverse_tok0(nblocks, DNB, stage, bb);
            floatx4 gcur;
#pragma unroll
            for (int e = 0; e < 4; ++e) gcur[e] = (FULL || tok0 + 4 * g + e < T) ? E::f(graw.x[bb][e]) : 0.f;
            const unsigned char *raw = VsRing::raw(smem, stage, bb);
            const unsigned char *st = VsRing::st(smem, stage, bb);
            const TmTile<SP> KPP(st + VS_KPP);
            const CmTile<SP> KC(raw + VS_KC), QC(raw + VS_QC);
            // dU[tok 4g+e][d] = Tm^T (Bq^T g) + K'' G_end^T: only the second term waits for the adjoint
            const Sp2<SP> gs = split4<SP>(gcur);
            const floatx4 bg = mma16(st_load<SP>(st + VS_BQ, lane), gs, zero);
            const floatx4 tbg = mma16(st_load<SP>(st + VS_TM, lane), split4<SP>(bg), zero);
            const Sp4<SP> gb0 = cat(split4<SP>(G[0]), split4<SP>(G[1])), gb1 = cat(split4<SP>(G[2]), split4<SP>(G[3]));
            const floatx4 kg = mma32(KPP.acc_order(r, g, 1), gb1, mma32(KPP.acc_order(r, g, 0), gb0, zero));
            const floatx4 du = tbg + kg;
            elem *const vb = d_v + (size_t)tok0 * CH_N;        // wave-uniform
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (FULL || tok0 + 4 * g + e < T) vb[lane_off + e * CH_N] = E::e(du[e]);
            // G += g^T Q - dU^T K
            const Sp2<SP> ndu = split4<SP>(-du);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                G[j] = mma16(QC.tokens(16 * j + r, g), gs, G[j]);
                G[j] = mma16(KC.tokens(16 * j + r, g), ndu, G[j]);
            }
        }
        __syncthreads();
    };
    GRaw g_a, g_b;
    load_g(g_a, 0);
    __syncthreads();        // ticks 0 and 1: the prep and matrix waves fill the pipeline
    __syncthreads();
    // the blocks are visited last to first: only stage 0 can hold tokens at or past T
    stage_body(std::false_type{}, 0, g_a, g_b);
    wait_vmem_all();
    int stage = 1;
    for (; stage + 2 <= nstages; stage += 2) {
        stage_body(std::true_type{}, stage, g_b, g_a);
        stage_body(std::true_type{}, stage + 1, g_a, g_b);
    }
    if (stage < nstages) stage_body(std::true_type{}, stage, g_b, g_a);
    elem *ds0 = reinterpret_cast<elem *>(p.d_s0) + (b * CH_N + d) * CH_N + 4 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) E::store4(ds0 + 16 * j, G[j]);
}

// blockIdx = half * rows_padded + row (rows_padded a multiple of 8: both halves of a row on one XCD).  Waves 0, 1:
// slab waves, alone on SIMDs 0 and 1; waves 2, 3: matrix waves; waves 6, 7: prep waves; waves 4, 5 leave at once.
template <bool SP, typename E> __global__ __launch_bounds__(BW_THREADS) void dfw_chunk_bwd_value_kernel(DfwBwdArgs p, int rows_padded) {
    typedef typename E::elem elem;
    extern __shared__ __align__(16) unsigned char smem[];
    const int half = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - half * rows_padded;
    if (b >= p.B) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int T = (int)p.T, nstages = (T + DL * DNB - 1) / (DL * DNB), nblocks = nstages * DNB;
    const elem *const k = reinterpret_cast<const elem *>(p.k) + b * p.T * CH_N;
    const elem *const q = reinterpret_cast<const elem *>(p.q) + b * p.T * CH_N;
    auto tok0_of = [=](int stage, int bb) { return reverse_tok0(nblocks, DNB, stage, bb); };
    static_assert(DNB == 2, "one matrix wave per block of a stage");
    if (wave < 2) {
        vs_slab_wave<SP, E>(p, smem, b, 32 * half + 16 * wave, nstages, lane);
    } else if (wave < 4) {
        vs_structure_wave<SP>(smem, nstages, wave - 2, lane);
    } else if (wave == 6) {
        const PrepJob<E> jobs[1] = {{k, VS_KT, VS_KC, 1.f, false}};
        prep_wave_jobs<VsRing, DNB, 1, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, nullptr);
    } else if (wave == 7) {
        const PrepJob<E> jobs[1] = {{q, VS_QT, VS_QC, 1.f, false}};
        prep_wave_jobs<VsRing, DNB, 1, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, nullptr);
    }
}

// ---- key side -------------------------------------------------------------------------------------------
// one block per stage; raw tiles per block: Delta, g, -dU token-major, -Delta, K, Q channel-major
constexpr int KS_DT = 0, KS_GT = KS_DT + 2 * TM_TILE, KS_NUT = KS_GT + 2 * TM_TILE, KS_NDC = KS_NUT + 2 * TM_TILE,
              KS_KC = KS_NDC + 2 * CM_TILE, KS_QC = KS_KC + 2 * CM_TILE, KS_RAW_BLOCK = KS_QC + 2 * CM_TILE;
constexpr int KS_X1 = 0, KS_X1T = KS_X1 + 2 * ST_TILE, KS_X2S = KS_X1T + 2 * ST_TILE, KS_ST_BLOCK = KS_X2S + 2 * ST_TILE;
using KsRing = Ring<KS_RAW_BLOCK, KS_ST_BLOCK, 1>;
// The adjoint waves hand G_end of a block to the state waves as a ready B operand: per (stage parity, wave,
// half of the value channels, head / remainder) 16 bytes per lane.
constexpr int KS_XG = KsRing::SMEM, KS_XG_PIECE = 64 * 16, KS_SCRATCH = KS_XG + 2 * 2 * 2 * 2 * KS_XG_PIECE;
// ... and two prep waves keep a token-major tile of their own (K, Q: wanted channel-major only)
constexpr int KS_SMEM = KS_SCRATCH + 2 * 2 * TM_TILE;
static_assert(KS_SMEM <= 160 * 1024, "key-side tiles exceed the LDS of one CU");
__device__ __forceinline__ uint4 *xg_piece(unsigned char *smem, int stage, int wave, int which, int part, int lane) {
    return reinterpret_cast<uint4 *>(smem + KS_XG + ((((stage & 1) * 2 + wave) * 2 + which) * 2 + part) * KS_XG_PIECE) + lane;
}

template <bool SP> __device__ __forceinline__ void ks_structure_wave(unsigned char *smem, int nstages, int lane) {
    const int r = lane & 15, g = lane >> 4;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    for (int tick = 0; tick < nstages + 2; ++tick) {
        const int stage = tick - 1;
        if (stage >= 0 && stage < nstages) {
            const unsigned char *raw = KsRing::raw(smem, stage, 0);
            const TmTile<SP> DT(raw + KS_DT), GT(raw + KS_GT), NUT(raw + KS_NUT);
            const Sp4<SP> d0 = DT.any_order(r, g, 0), d1 = DT.any_order(r, g, 1);
            const Sp4<SP> g0 = GT.any_order(r, g, 0), g1 = GT.any_order(r, g, 1);
            const Sp4<SP> u0 = NUT.any_order(r, g, 0), u1 = NUT.any_order(r, g, 1);
            const floatx4 z = mma32(g1, d1, mma32(g0, d0, zero));       // [t = 4g+e][s = r] =  g_t . delta_s
            const floatx4 zt = mma32(d1, g1, mma32(d0, g0, zero));      // [s = 4g+e][t = r] =  delta_s . g_t
            const floatx4 y = mma32(u1, d1, mma32(u0, d0, zero));       // [t = 4g+e][s = r] = -dU_t . delta_s
            const floatx4 yt = mma32(d1, u1, mma32(d0, u0, zero));      // [s = 4g+e][t = r] = -delta_s . dU_t
            floatx4 x1, x1t, x2s;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 4 * g + e;
                x1[e] = r < row ? z[e] : 0.f;                 // X1[t][s], s < t
                x1t[e] = row < r ? zt[e] : 0.f;               // X1^T[s][t], s < t
                x2s[e] = r < row ? y[e] : (row < r ? yt[e] : 0.f);      // X2 + X2^T
            }
            unsigned char *st = KsRing::st(smem, stage, 0);
            st_store<SP>(st + KS_X1, lane, split4<SP>(x1));
            st_store<SP>(st + KS_X1T, lane, split4<SP>(x1t));
            st_store<SP>(st + KS_X2S, lane, split4<SP>(x2s));
        }
        __syncthreads();
    }
}

// The adjoint chain of 16 key channels: G_start = G_end + g^T Q - dU^T K, one stage ahead of the state waves, to
// which it hands G_end of every block as a split B operand.  It shares a SIMD with the state wave of the same
// channels: two independent chains whose instruction streams interleave.
template <bool SP, typename E> __device__ __forceinline__ void ks_adjoint_wave(const DfwBwdArgs &p, unsigned char *smem, int64_t b, int m0, int w, int nstages, int lane) {
    typedef typename E::elem elem;
    const int r = lane & 15, g = lane >> 4, m = m0 + r;
    // G[j][e] = G[d = 16 j + 4 g + e][m]: columns of the state's adjoint
    floatx4 G[4];
    {
        const elem *gs = reinterpret_cast<const elem *>(p.g_state) + b * CH_N * CH_N + m;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) G[j][e] = E::f(gs[(16 * j + 4 * g + e) * CH_N]);
    }
    for (int tick = 0; tick < nstages + 2; ++tick) {
        const int stage = tick - 1;
        if (stage >= 0 && stage < nstages) {
            const unsigned char *raw = KsRing::raw(smem, stage, 0);
            // g and -dU along the tokens of a value channel come out of the token-major tiles through the transposing
            // read: this wave has the time for it, the prep waves do not have it for two more derived tiles
            const TmTile<SP> GT(raw + KS_GT), NUT(raw + KS_NUT);
            const CmTile<SP> KC(raw + KS_KC), QC(raw + KS_QC);
            const Sp2<SP> kb = KC.tokens(m, g), qb = QC.tokens(m, g);          // K[t = 4g+e][m], Q[t][m]
            const Sp4<SP> gb0 = cat(split4<SP>(G[0]), split4<SP>(G[1])), gb1 = cat(split4<SP>(G[2]), split4<SP>(G[3]));
            *xg_piece(smem, stage, w, 0, 0, lane) = gb0.hi;
            *xg_piece(smem, stage, w, 1, 0, lane) = gb1.hi;
            if constexpr (SP) {
                *xg_piece(smem, stage, w, 0, 1, lane) = gb0.lo;
                *xg_piece(smem, stage, w, 1, 1, lane) = gb1.lo;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                G[j] = mma16(GT.column(j, r, g), qb, G[j]);
                G[j] = mma16(NUT.column(j, r, g), kb, G[j]);
            }
        }
        __syncthreads();
    }
}

// The state chain of 16 key channels, walked backwards (S0 = S_end - Delta^T K), and the block's d_query, d_key.
template <bool SP, typename E> __device__ __forceinline__ void ks_slab_wave(const DfwBwdArgs &p, unsigned char *smem, int64_t b, int m0, int w, int nstages, int lane) {
    typedef typename E::elem elem;
    const int r = lane & 15, g = lane >> 4, m = m0 + r, T = (int)p.T, nblocks = nstages;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    elem *const d_q = reinterpret_cast<elem *>(p.d_q) + b * p.T * CH_N;
    elem *const d_k = reinterpret_cast<elem *>(p.d_k) + b * p.T * CH_N;
    const u32 lane_off = (u32)(4 * g * CH_N + m);
    // S[j][e] = S[d = 16 j + 4 g + e][m]: columns of the state
    floatx4 S[4];
    {
        const elem *fs = reinterpret_cast<const elem *>(p.final_state) + b * CH_N * CH_N + m;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) S[j][e] = E::f(fs[(16 * j + 4 * g + e) * CH_N]);
    }
    // one stage (= one block).  FULL: every token of the stage is below T and the body has no branch (see the
    // value side)
    auto stage_body = [&](auto full, int stage) {
        constexpr bool FULL = decltype(full)::value;
        const int tok0 = reverse_tok0(nblocks, 1, stage, 0);
        const unsigned char *raw = KsRing::raw(smem, stage, 0);
        const unsigned char *st = KsRing::st(smem, stage, 0);
        const TmTile<SP> DT(raw + KS_DT), GT(raw + KS_GT), NUT(raw + KS_NUT);
        const CmTile<SP> NDC(raw + KS_NDC), KC(raw + KS_KC), QC(raw + KS_QC);
        const Sp2<SP> kb = KC.tokens(m, g), qb = QC.tokens(m, g);          // K[t = 4g+e][m], Q[t][m]
        // the adjoint after the block, as the adjoint wave left it one stage ago
        Sp4<SP> gb0, gb1;
        gb0.hi = *xg_piece(smem, stage, w, 0, 0, lane);
        gb1.hi = *xg_piece(smem, stage, w, 1, 0, lane);
        gb0.lo = SP ? *xg_piece(smem, stage, w, 0, 1, lane) : make_uint4(0u, 0u, 0u, 0u);
        gb1.lo = SP ? *xg_piece(smem, stage, w, 1, 1, lane) : make_uint4(0u, 0u, 0u, 0u);
        // S0 = S_end - Delta^T K
#pragma unroll
        for (int j = 0; j < 4; ++j) S[j] = mma16(NDC.tokens(16 * j + r, g), kb, S[j]);
        const Sp4<SP> sb0 = cat(split4<SP>(S[0]), split4<SP>(S[1])), sb1 = cat(split4<SP>(S[2]), split4<SP>(S[3]));
        // d_query[t][m] = g S0 + X1 K
        const floatx4 dq = mma32(GT.acc_order(r, g, 1), sb1, mma32(GT.acc_order(r, g, 0), sb0, zero)) +
                           mma16(st_load<SP>(st + KS_X1T, lane), kb, zero);
        // d_key[s][m] = Delta G_end - dU S0 + X1^T Q + (X2 + X2^T) K
        const floatx4 dk = mma32(NUT.acc_order(r, g, 1), sb1,
                                 mma32(NUT.acc_order(r, g, 0), sb0,
                                       mma32(DT.acc_order(r, g, 1), gb1, mma32(DT.acc_order(r, g, 0), gb0, zero)))) +
                           mma16(st_load<SP>(st + KS_X2S, lane), kb, mma16(st_load<SP>(st + KS_X1, lane), qb, zero));
        elem *const qo = d_q + (size_t)tok0 * CH_N, *const ko = d_k + (size_t)tok0 * CH_N;      // wave-uniform
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (FULL || tok0 + 4 * g + e < T) {
                qo[lane_off + e * CH_N] = E::e(dq[e]);
                ko[lane_off + e * CH_N] = E::e(dk[e]);
            }
        __syncthreads();
    };
    __syncthreads();        // ticks 0 and 1: the prep, matrix and adjoint waves fill the pipeline
    __syncthreads();
    // the blocks are visited last to first: only stage 0 can hold tokens at or past T
    stage_body(std::false_type{}, 0);
    wait_vmem_all();
    for (int stage = 1; stage < nstages; ++stage) stage_body(std::true_type{}, stage);
}

// Waves 0, 1: state waves (16 key channels each) and waves 4, 5: the adjoint waves of the same channels, on SIMDs 0
// and 1; wave 2: matrix wave; waves 3, 6, 7: prep waves.
template <bool SP, typename E> __global__ __launch_bounds__(BW_THREADS) void dfw_chunk_bwd_key_kernel(DfwBwdArgs p, int rows_padded) {
    typedef typename E::elem elem;
    extern __shared__ __align__(16) unsigned char smem[];
    const int half = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - half * rows_padded;
    if (b >= p.B) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int T = (int)p.T, nstages = (T + DL - 1) / DL;
    const int64_t row = b * p.T * CH_N;
    const elem *const k = reinterpret_cast<const elem *>(p.k) + row;
    const elem *const q = reinterpret_cast<const elem *>(p.q) + row;
    const elem *const dl = reinterpret_cast<const elem *>(p.delta) + row;
    const elem *const go = reinterpret_cast<const elem *>(p.g_out) + row;
    const elem *const dv = reinterpret_cast<const elem *>(p.d_v) + row;
    auto tok0_of = [=](int stage, int bb) { return reverse_tok0(nstages, 1, stage, bb); };
    if (wave < 2) {
        ks_slab_wave<SP, E>(p, smem, b, 32 * half + 16 * wave, wave, nstages, lane);
    } else if (wave == 4 || wave == 5) {
        ks_adjoint_wave<SP, E>(p, smem, b, 32 * half + 16 * (wave - 4), wave - 4, nstages, lane);
    } else if (wave == 2) {
        ks_structure_wave<SP>(smem, nstages, lane);
    } else if (wave == 3) {
        const PrepJob<E> jobs[1] = {{dl, KS_DT, KS_NDC, 1.f, true}};
        prep_wave_jobs<KsRing, 1, 1, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, nullptr);
    } else if (wave == 6) {
        const PrepJob<E> jobs[2] = {{go, KS_GT, -1, 1.f, false}, {k, -1, KS_KC, 1.f, false}};
        prep_wave_jobs<KsRing, 1, 2, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, smem + KS_SCRATCH);
    } else if (wave == 7) {
        const PrepJob<E> jobs[2] = {{dv, KS_NUT, -1, -1.f, false}, {q, -1, KS_QC, 1.f, false}};
        prep_wave_jobs<KsRing, 1, 2, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, smem + KS_SCRATCH + 2 * TM_TILE);
    }
}

}  // namespace

template <bool SP, typename E> static int launch_backward(const DfwBwdArgs &a, hipStream_t stream) {
    auto value_side = dfw_chunk_bwd_value_kernel<SP, E>;
    auto key_side = dfw_chunk_bwd_key_kernel<SP, E>;
    int rc = enable_lds(reinterpret_cast<const void *>(value_side), VsRing::SMEM, "hipFuncSetAttribute(delta-rule backward kernel, value side)");
    if (rc) return rc;
    if ((rc = enable_lds(reinterpret_cast<const void *>(key_side), KS_SMEM, "hipFuncSetAttribute(delta-rule backward kernel, key side)"))) return rc;
    const int rows_padded = (int)((a.B + 7) / 8 * 8);
    hipLaunchKernelGGL(value_side, dim3(2u * (unsigned)rows_padded), dim3(BW_THREADS), VsRing::SMEM, stream, a, rows_padded);
    if ((rc = check_hip(hipGetLastError(), "dfw_chunk_bwd_value_kernel launch"))) return rc;
    hipLaunchKernelGGL(key_side, dim3(2u * (unsigned)rows_padded), dim3(BW_THREADS), KS_SMEM, stream, a, rows_padded);
    return check_hip(hipGetLastError(), "dfw_chunk_bwd_key_kernel launch");
}

template <typename E> static int backward_of(const DfwBwdArgs &a, bool split_operands, hipStream_t stream) {
    return split_operands ? launch_backward<true, E>(a, stream) : launch_backward<false, E>(a, stream);
}

int dfw_chunk_backward(const DfwBwdArgs &a, int dtype, bool split_operands, hipStream_t stream) {
    if (a.D != CH_N || a.M != CH_N) return fail(T2FW_ERR_UNSUPPORTED, "the block-wise delta-rule kernels take D = M = 64");
    if (a.T * CH_N >= 0x7fffffffLL || a.B > 0x1fffffffLL)
        return fail(T2FW_ERR_UNSUPPORTED, "B=%lld T=%lld is too large for the block-wise delta-rule kernels", (long long)a.B, (long long)a.T);
    switch (dtype) {
    case T2FW_F32: return backward_of<ElF32>(a, split_operands, stream);
    case T2FW_F16: return backward_of<El16<Fp16>>(a, split_operands, stream);
    case T2FW_BF16: return backward_of<El16<Bf16>>(a, split_operands, stream);
    default: return fail(T2FW_ERR_UNSUPPORTED, "the block-wise delta-rule kernels take fp32, fp16 and bf16 tensors");
    }
}

}  // namespace t2fw
