// Forward pass of the delta rule on the matrix cores, D = M = 64, fp32 / fp16 / bf16 tensors (algebra, precision
// and element types: dfw_chunk.hpp).  Two workgroups per batch row, one per half of the value channels: the rows S[d, :] of the
// state, and with them the columns of V, Delta and O, never interact.  A workgroup has six waves (eight are launched; two leave at once):
//   two slab waves    each keeps 16 rows of the state in fp32 accumulators for the whole sequence; per block:
//                     Delta = Tm V - K' S0^T, O = Q S0^T + Bq Delta, S += Delta^T K; they load V and store O
//                     and Delta themselves (64 contiguous bytes per token)
//   two matrix waves  everything that does not depend on the state, one stage ahead of the slab waves, one
//                     block of the stage each: K K^T and K Q^T, the triangular masks, Tm = (I + A)^-1 by
//                     squarings, K' = Tm K; they leave Tm^T and Bq^T as ready operands and K' as a tile in LDS
//   two prep waves    K (token-major, and channel-major derived from that tile) and Q (token-major) as bf16
//                     head / remainder tiles, two stages ahead
// One workgroup barrier per stage of two blocks.
//
// Replaces lfw_cuda_fwd_kernel of the reference's delta rule (t2fw/csrc/dfw_kernel.cu:105-196), semantics
// t2fw/torch.py:44-53; `delta` is the tensor that kernel emits for its backward (dfw_kernel.cu:176-183).
#include <type_traits>
#include "common.hpp"
#include "dfw_chunk.hpp"
#include "dfw_scan.hpp"

namespace t2fw {
namespace {

using namespace dfwc;

constexpr int FW_THREADS = 512;
// per block: raw tiles K token-major, Q token-major, K channel-major (head + remainder each) ...
constexpr int FW_KT = 0, FW_QT = FW_KT + 2 * TM_TILE, FW_KC = FW_QT + 2 * TM_TILE, FW_RAW_BLOCK = FW_KC + 2 * CM_TILE;
// ... and what the matrix waves make of them: K' token-major, Tm^T and Bq^T as operands
constexpr int FW_KP = 0, FW_TT = FW_KP + 2 * TM_TILE, FW_BQT = FW_TT + 2 * ST_TILE, FW_ST_BLOCK = FW_BQT + 2 * ST_TILE;
constexpr int FW_RAW = 0;                                        // three stages of raw tiles
constexpr int FW_ST = FW_RAW + 3 * DNB * FW_RAW_BLOCK;           // two stages of the matrix waves' results
constexpr int FW_SMEM = FW_ST + 2 * DNB * FW_ST_BLOCK;
static_assert(FW_SMEM <= 160 * 1024, "forward tiles exceed the LDS of one CU");
using FwRing = Ring<FW_RAW_BLOCK, FW_ST_BLOCK, DNB>;         // the same layout, for the shared prep-wave routine
static_assert(FwRing::SMEM == FW_SMEM && FwRing::ST == FW_ST, "ring layout");

__device__ __forceinline__ unsigned char *raw_block(unsigned char *smem, int stage, int bb) {
    return smem + FW_RAW + ((stage % 3) * DNB + bb) * FW_RAW_BLOCK;
}
__device__ __forceinline__ unsigned char *st_block(unsigned char *smem, int stage, int bb) {
    return smem + FW_ST + ((stage & 1) * DNB + bb) * FW_ST_BLOCK;
}

// The state-independent part of block `bb` of every stage, one stage ahead of the slab waves.
template <bool SP> __device__ __forceinline__ void structure_wave(unsigned char *smem, int nstages, int bb, int lane) {
    const int r = lane & 15, g = lane >> 4;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    for (int tick = 0; tick < nstages + 2; ++tick) {
        const int stage = tick - 1;
        if (stage >= 0 && stage < nstages) {
            const unsigned char *raw = raw_block(smem, stage, bb);
            const TmTile<SP> KT(raw + FW_KT), QT(raw + FW_QT);
            const CmTile<SP> KC(raw + FW_KC);
            const Sp4<SP> k0 = KT.any_order(r, g, 0), k1 = KT.any_order(r, g, 1);
            const Sp4<SP> q0 = QT.any_order(r, g, 0), q1 = QT.any_order(r, g, 1);
            const floatx4 kk = mma32(k1, k1, mma32(k0, k0, zero));      // [s = 4g+e][t = r] = k_s . k_t
            const floatx4 kq = mma32(k1, q1, mma32(k0, q0, zero));      // [s = 4g+e][t = r] = k_s . q_t
            floatx4 bqt;
#pragma unroll
            for (int e = 0; e < 4; ++e) bqt[e] = 4 * g + e < r ? kq[e] : 0.f;      // Bq^T[s][t] = k_s . q_t for s < t
            const BlockInverse<SP> inv(kk, r, g);
            const Sp2<SP> tt = split4<SP>(inv.acc_tm_transposed());
            unsigned char *st = st_block(smem, stage, bb);
            st_store<SP>(st + FW_TT, lane, tt);
            st_store<SP>(st + FW_BQT, lane, split4<SP>(bqt));
            // K'^T tile j: [m = 16 j + 4 g + e][t = r] = sum_s K[s][m] Tm[t][s]
            floatx4 kp[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) kp[j] = mma16(KC.tokens(16 * j + r, g), tt, zero);
            store_tm_from_acc<SP>(st + FW_KP, r, g, kp);
        }
        __syncthreads();
    }
}

template <bool SP, typename E> __device__ __forceinline__ void slab_wave(const DfwFwdArgs &p, unsigned char *smem, int64_t b, int d0, int nstages, int lane) {
    typedef typename E::elem elem;
    const int r = lane & 15, g = lane >> 4, d = d0 + r, T = (int)p.T;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    // token addresses: a wave-uniform base per block plus the lane's fixed offset (first token 4 g, channel d)
    const elem *const v = reinterpret_cast<const elem *>(p.v) + b * p.T * CH_N;
    elem *const out = reinterpret_cast<elem *>(p.out) + b * p.T * CH_N;
    elem *const delta = reinterpret_cast<elem *>(p.delta) + b * p.T * CH_N;
    const u32 lane_off = (u32)(4 * g * CH_N + d);
    // S[j][e] = S[d][16 j + 4 g + e]
    floatx4 S[4];
    {
        const elem *s0 = reinterpret_cast<const elem *>(p.s0) + (b * CH_N + d) * CH_N + 4 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) S[j] = E::load4(s0 + 16 * j);
    }
    // V of a stage: element [bb][e] is token (stage * DNB + bb) * 16 + 4 g + e; loaded one stage ahead into the
    // register set the stage before has left, as loaded (converted where the stage uses it)
    // (unconditional loads: tokens at or past T are read from token T - 1 and zeroed where they are used)
    struct VRaw {
        elem x[DNB][4];
    };
    auto load_v = [&](VRaw &x, int stage) {
#pragma unroll
        for (int bb = 0; bb < DNB; ++bb)
#pragma unroll
            for (int e = 0; e < 4; ++e) x.x[bb][e] = v[(size_t)min((stage * DNB + bb) * DL + 4 * g + e, T - 1) * CH_N + d];
    };
    // One stage.  FULL: every token of the stage is below T, and the body is free of branches: the waits that
    // the compiler places count outstanding memory operations along every path, so a path that skips stores
    // would make the loads of the next stage wait for the stores of this one.
    auto stage_body = [&](auto full, int stage, VRaw &vraw, VRaw &vnxt) {
        constexpr bool FULL = decltype(full)::value;
        load_v(vnxt, min(stage + 1, nstages - 1));
#pragma unroll
        for (int bb = 0; bb < DNB; ++bb) {
            const int tok0 = (stage * DNB + bb) * DL;
            floatx4 vcur;
#pragma unroll
            for (int e = 0; e < 4; ++e) vcur[e] = (FULL || tok0 + 4 * g + e < T) ? E::f(vraw.x[bb][e]) : 0.f;
            const unsigned char *raw = raw_block(smem, stage, bb);
            const unsigned char *st = st_block(smem, stage, bb);
            const TmTile<SP> QT(raw + FW_QT), KP(st + FW_KP);
            const CmTile<SP> KC(raw + FW_KC);
            // Delta[tok 4g+e][d] = Tm V - K' S0^T: only the second term waits for the state
            const floatx4 tv = mma16(st_load<SP>(st + FW_TT, lane), split4<SP>(vcur), zero);
            const Sp4<SP> sb0 = cat(split4<SP>(S[0]), split4<SP>(S[1])), sb1 = cat(split4<SP>(S[2]), split4<SP>(S[3]));
            const floatx4 ks = mma32(KP.acc_order(r, g, 1), sb1, mma32(KP.acc_order(r, g, 0), sb0, zero));
            const floatx4 dl = tv - ks;
            const Sp2<SP> dls = split4<SP>(dl);
            // O = Q S0^T + Bq Delta
            const floatx4 qs = mma32(QT.acc_order(r, g, 1), sb1, mma32(QT.acc_order(r, g, 0), sb0, zero));
            const floatx4 o = qs + mma16(st_load<SP>(st + FW_BQT, lane), dls, zero);
            elem *const ob = out + (size_t)tok0 * CH_N, *const db = delta + (size_t)tok0 * CH_N;      // wave-uniform
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (FULL || tok0 + 4 * g + e < T) {
                    ob[lane_off + e * CH_N] = E::e(o[e]);
                    db[lane_off + e * CH_N] = E::e(dl[e]);
                }
            // S += Delta^T K
#pragma unroll
            for (int j = 0; j < 4; ++j) S[j] = mma16(KC.tokens(16 * j + r, g), dls, S[j]);
        }
        __syncthreads();
    };
    VRaw v_a, v_b;
    load_v(v_a, 0);
    __syncthreads();        // ticks 0 and 1: the prep and matrix waves fill the pipeline
    __syncthreads();
    // Nothing of this wave's is in flight when the loop is entered: the compiler merges what may be outstanding at
    // the loop head over both ways in, and loads still pending on entry would turn every iteration's waits into
    // waits for the stores of the iteration before.
    wait_vmem_all();
    const int nfull = T / (DL * DNB);       // stages without a token at or past T; at most one more follows
    int stage = 0;
    for (; stage + 2 <= nfull; stage += 2) {
        stage_body(std::true_type{}, stage, v_a, v_b);
        stage_body(std::true_type{}, stage + 1, v_b, v_a);
    }
    if (stage < nfull) {
        stage_body(std::true_type{}, stage, v_a, v_b);
        if (stage + 1 < nstages) stage_body(std::false_type{}, stage + 1, v_b, v_a);
    } else if (stage < nstages) {
        stage_body(std::false_type{}, stage, v_a, v_b);
    }
    elem *fin = reinterpret_cast<elem *>(p.final_state) + (b * CH_N + d) * CH_N + 4 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) E::store4(fin + 16 * j, S[j]);
}

// blockIdx = half * rows_padded + row with rows_padded a multiple of 8: the two halves of a row land on the
// same XCD and share its L2 for K and Q, which both read
template <bool SP, typename E> __global__ __launch_bounds__(FW_THREADS) void dfw_chunk_fwd_kernel(DfwFwdArgs p, int rows_padded) {
    typedef typename E::elem elem;
    extern __shared__ __align__(16) unsigned char smem[];
    const int half = (int)blockIdx.x >= rows_padded ? 1 : 0;
    const int64_t b = (int)blockIdx.x - half * rows_padded;
    if (b >= p.B) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int T = (int)p.T, nstages = (T + DL * DNB - 1) / (DL * DNB);
    const elem *const k = reinterpret_cast<const elem *>(p.k) + b * p.T * CH_N;
    const elem *const q = reinterpret_cast<const elem *>(p.q) + b * p.T * CH_N;
    // Every wave that stays executes nstages + 2 workgroup barriers.  Wave i runs on SIMD i % 4: the slab waves,
    // whose chain of dependent steps sets the kernel's duration, get SIMDs 0 and 1 to themselves (waves 4 and 5
    // leave at once; a workgroup barrier waits only for the waves that are left), the matrix waves and the
    // prep waves share SIMDs 2 and 3.
    static_assert(DNB == 2, "one matrix wave per block of a stage");
    auto tok0_of = [](int stage, int bb) { return (stage * DNB + bb) * DL; };
    if (wave < 2)
        slab_wave<SP, E>(p, smem, b, 32 * half + 16 * wave, nstages, lane);
    else if (wave < 4)
        structure_wave<SP>(smem, nstages, wave - 2, lane);
    else if (wave == 6) {          // K: token-major, and channel-major derived from it
        const PrepJob<E> jobs[1] = {{k, FW_KT, FW_KC, 1.f, false}};
        prep_wave_jobs<FwRing, DNB, 1, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, nullptr);
    } else if (wave == 7) {        // Q: token-major
        const PrepJob<E> jobs[1] = {{q, FW_QT, -1, 1.f, false}};
        prep_wave_jobs<FwRing, DNB, 1, SP, 3, E>(smem, jobs, T, nstages, lane, tok0_of, nullptr);
    }
}

}  // namespace

template <bool SP, typename E> static int launch_forward(const DfwFwdArgs &a, hipStream_t stream) {
    auto kern = dfw_chunk_fwd_kernel<SP, E>;
    int rc = enable_lds(reinterpret_cast<const void *>(kern), FW_SMEM, "hipFuncSetAttribute(delta-rule forward kernel)");
    if (rc) return rc;
    const int rows_padded = (int)((a.B + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(2u * (unsigned)rows_padded), dim3(FW_THREADS), FW_SMEM, stream, a, rows_padded);
    return check_hip(hipGetLastError(), "dfw_chunk_fwd_kernel launch");
}

template <typename E> static int forward_of(const DfwFwdArgs &a, bool split_operands, hipStream_t stream) {
    return split_operands ? launch_forward<true, E>(a, stream) : launch_forward<false, E>(a, stream);
}

int dfw_chunk_forward(const DfwFwdArgs &a, int dtype, bool split_operands, hipStream_t stream) {
    if (a.D != CH_N || a.M != CH_N) return fail(T2FW_ERR_UNSUPPORTED, "the block-wise delta-rule kernels take D = M = 64");
    if (a.T * CH_N >= 0x7fffffffLL || a.B > 0x1fffffffLL)
        return fail(T2FW_ERR_UNSUPPORTED, "B=%lld T=%lld is too large for the block-wise delta-rule kernels", (long long)a.B, (long long)a.T);
    switch (dtype) {
    case T2FW_F32: return forward_of<ElF32>(a, split_operands, stream);
    case T2FW_F16: return forward_of<El16<Fp16>>(a, split_operands, stream);
    case T2FW_BF16: return forward_of<El16<Bf16>>(a, split_operands, stream);
    default: return fail(T2FW_ERR_UNSUPPORTED, "the block-wise delta-rule kernels take fp32, fp16 and bf16 tensors");
    }
}

}  // namespace t2fw
