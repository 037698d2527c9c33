// Backward pass of the decay rule, chunk-parallel matrix-core form (layout and scalings: lfw_par.hpp).
//
// With G = dL/dS flowing backwards in time, S0 the state at a chunk's start (the checkpoint), Ge the
// adjoint of the state at the chunk's end coming from the future, A = a_CL, B = b_CL the chunk's gate
// products and Gh = (A (x) B) * Ge:
//   P[t,s] = qs_t.kt_s       W[t,s] = gs_t.xt_s
//   o'_t  = S0 qs_t    + sum_{s<t} P[t,s] xt_s          (output without its own write, / a_t)
//   q'_t  = S0^T gs_t  + sum_{s<t} W[t,s] kt_s          (d_q without its own term, / b_t)
//   x'_t  = Gh kt_t    + sum_{r>t} P[r,t] gs_r          (d_x without its own term, * a_t)
//   k'_t  = Gh^T xt_t  + sum_{r>t} W[r,t] qs_r          (d_k without its own term, * b_t)
//   d_x_t = (x'_t + gs_t P[t,t]) / a_t    d_k_t = (k'_t + qs_t W[t,t]) / b_t    d_q_t = (q'_t + kt_t W[t,t]) * b_t
//   f_t * d_f_t   = u_t,  u_t = beta - sum_{r<t} (gs_r * o'_r - xt_r * x'_r)     (elementwise)
//   fk_t * d_fk_t = v_t,  v_t = gamma - sum_{r<t} (qs_r * q'_r - kt_r * k'_r)
//   beta  = rowsum((Gh + sum_t gs_t (x) qs_t) * S0) = rowsum(Gh * S0) + sum_t gs_t * (S0 qs_t)
//   gamma = colsum(...)                             = colsum(Gh * S0) + sum_t qs_t * (S0^T gs_t)
//   adjoint leaving the chunk towards the past:  Gh + sum_t gs_t (x) qs_t
// The recurrence is symmetric under (x, f, g_out, D) <-> (k, f_key, q, K) with the state transposed;
// the value-side waves compute o', x', u and the key-side waves q', k', v with the same code.
//
// All scalings are relative to the middle of the chunk (lfw_par.hpp): a_t, b_t above stand for
// a_t / a_mid, b_t / b_mid, S0 for (a_mid (x) b_mid) * S0 and Gh for (A/a_mid (x) B/b_mid) * Ge; the
// formulas are unchanged by that.
//
// Launch 1 (lfw_par_incr_kernel, one workgroup per (row, chunk)): the chunk's increment of the adjoint,
// sum_t gs_t (x) qs_t with prefixes from the chunk START (factors <= 1), as bf16, and the chunk's
// gate products.  Launch 2 (lfw_par_scan_kernel, elementwise, eight workgroups per row): the
// adjoint chain over the chunks of a row, last to first, in fp32; it overwrites every increment
// with the Gh of its chunk (bf16, the type the third launch feeds to the matrix cores) and writes
// d_s0.  Launch 3 (lfw_par_grads_kernel, one workgroup per (row, chunk)) computes everything else.
// No workgroup waits for another one inside a launch.
//
// Replaces lfw_cuda_bwd_kernel and the six einsums of the reference
// (t2fw/csrc/lfw_kernel.cu:61-102, t2fw/csrc/lfw.cpp:84-93).
#include <type_traits>

#include "lfw_par.hpp"

namespace t2fw {
namespace {

using namespace par;

// ---- launch 1: per-chunk adjoint increments and gate products -------------------------------------
constexpr int INCR_SMEM = 2 * CM_BYTES;        // gs tile, qs tile

template <typename IOE, int NT, bool HEADS>
__global__ __launch_bounds__(PAR_THREADS) void lfw_par_incr_kernel(ParBwdArgs p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int CL = 16 * NT;
    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63;
    const int side = w >> 2, cb = w & 3, i = l & 15, kg = l >> 4, c = 16 * cb + i;
    const int NC = (int)p.NC, T = (int)p.T;
    const int item = (int)blockIdx.x;
    const int64_t b = item / NC;
    const int chunk = item - (int)b * NC;
    const u32 ts = HEADS ? (u32)p.heads * CH_N : (u32)CH_N;
    const int tok0 = chunk * CL + 4 * kg, n_left = T - tok0;
    // the chunk's first token (wave-uniform) and the lane's offset from there
    const int64_t chunk_off = wave_uniform(row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N + (int64_t)(chunk * CL) * ts);
    const u32 lane_off = (u32)(4 * kg) * ts + (u32)c;
    const u16 *const gate = reinterpret_cast<const u16 *>(side ? p.f_key : p.f) + chunk_off;
    const u16 *const adj = reinterpret_cast<const u16 *>(side ? p.q : p.g_out) + chunk_off;
    u32 bad;
    {
        RawTokens<NT> rg, ra;
        LaneChunk<NT> lc;
        float gt[NT][4], av[NT][4];
        if (chunk * CL + CL <= T) {
            load_tokens<NT, true>(rg, gate, lane_off, ts, n_left);
            load_tokens<NT, true>(ra, adj, lane_off, ts, n_left);
            gate_scan<IOE, NT, true, false>(lc, gt, rg, kg, n_left);
            to_floats<IOE, NT, true>(av, ra, n_left);
        } else {
            load_tokens<NT, false>(rg, gate, lane_off, ts, n_left);
            load_tokens<NT, false>(ra, adj, lane_off, ts, n_left);
            gate_scan<IOE, NT, false, false>(lc, gt, rg, kg, n_left);
            to_floats<IOE, NT, false>(av, ra, n_left);
        }
        bad = lc.bad;
        uint2 as[NT];
        scale_pack<NT>(as, av, lc.pre);
        store_cm<NT>(reinterpret_cast<u16 *>(smem + side * CM_BYTES), c, kg, as);
        if (kg == 0) {
            float *v = p.vecs + (int64_t)item * (PAR_NVEC * CH_N) + side * CH_N + c;
            v[0] = lc.tot;
            v[2 * CH_N] = lc.ref;
            v[4 * CH_N] = lc.sfx;
        }
    }
    const int any_bad = __syncthreads_or((int)bad);
    if (tid == 0) p.chunk_flags[item] = any_bad ? 1 : 0;
    // this wave's two tiles of the increment: rows d = 16 db + 4 kg + j, column k = 16 kb + i
    const u16 *const GS = reinterpret_cast<const u16 *>(smem), *const QS = reinterpret_cast<const u16 *>(smem + CM_BYTES);
    const int db = w & 3, kb0 = 2 * (w >> 2);
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    uint4 ga[NT / 2];
#pragma unroll
    for (int h = 0; h < NT / 2; ++h) ga[h] = mat_rows_op(GS, 16 * db, h, i, kg);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int kb = kb0 + t;
        floatx4 m = zero;
#pragma unroll
        for (int h = 0; h < NT / 2; ++h) m = Bf16::mfma32(ga[h], mat_rows_op(QS, 16 * kb, h, i, kg), m);
        u16 *const dst = reinterpret_cast<u16 *>(p.gh) + (int64_t)item * (CH_N * CH_N) + (16 * db + 4 * kg) * CH_N + 16 * kb + i;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j * CH_N] = cvt1<Bf16>(m[j]);
    }
}

// ---- launch 2: the adjoint chain over the chunks of a row -------------------------------------------
// G enters the row's last chunk as g_state; per chunk, last to first:
//   Gh'[chunk] = (sfxA (x) sfxB) * G       (overwrites the chunk's increment)
//   G          = (totA (x) totB) * G + increment[chunk]
// and d_s0 = G after chunk 0.  A workgroup owns eight rows of the 64 x 64 matrix of one batch row, a
// thread two adjacent elements.  Chunks are taken sixteen at a time: the gate products of the
// sixteen go through LDS, and a thread's sixteen loads of the increments are all in flight before
// the chain starts (they do not depend on it).
constexpr int SCAN_TPB = 256, SCAN_BATCH = 16, SCAN_VEC = 2 * 8 + 2 * CH_N;      // per chunk: totA, sfxA of 8 rows; totB, sfxB

template <typename IOE> __global__ __launch_bounds__(SCAN_TPB) void lfw_par_scan_kernel(ParBwdArgs p) {
    __shared__ float vl[SCAN_BATCH * SCAN_VEC];
    // Consecutive workgroups go to the eight XCDs in turn: the eight slabs of a batch row, which all read
    // the row's gate-product vectors, get ids that are 8 apart and share one XCD's L2.
    const int64_t b = (int64_t)(blockIdx.x >> 6) * 8 + (blockIdx.x & 7);
    if (b >= p.B) return;
    const int slab = (int)((blockIdx.x >> 3) & 7), tid = threadIdx.x;
    const int dl = tid >> 5, d = slab * 8 + dl, k = (tid & 31) * 2;
    const int NC = (int)p.NC;
    float G0, G1;
    {
        const u32 g = *reinterpret_cast<const u32 *>(reinterpret_cast<const u16 *>(p.g_state) + b * (CH_N * CH_N) + d * CH_N + k);
        G0 = IOE::to_f32((u16)(g & 0xffffu));
        G1 = IOE::to_f32((u16)(g >> 16));
    }
    u16 *const gh = reinterpret_cast<u16 *>(p.gh) + b * NC * (int64_t)(CH_N * CH_N) + d * CH_N + k;
    const float *const vecs = p.vecs + b * NC * (int64_t)(PAR_NVEC * CH_N);
    for (int c_top = NC - 1; c_top >= 0; c_top -= SCAN_BATCH) {
        u32 m[SCAN_BATCH];
#pragma unroll
        for (int u = 0; u < SCAN_BATCH; ++u) {
            const int c = c_top - u > 0 ? c_top - u : 0;
            m[u] = *reinterpret_cast<const u32 *>(gh + (int64_t)c * (CH_N * CH_N));
        }
        __syncthreads();                                   // the previous batch's vectors are no longer read
        static_assert(SCAN_BATCH * SCAN_VEC % SCAN_TPB == 0, "vector staging assumes whole passes");
        float tmp[SCAN_BATCH * SCAN_VEC / SCAN_TPB];
#pragma unroll
        for (int it = 0; it < SCAN_BATCH * SCAN_VEC / SCAN_TPB; ++it) {
            const int idx = tid + it * SCAN_TPB;
            const int u = idx / SCAN_VEC, wv = idx - u * SCAN_VEC;
            const int c = c_top - u > 0 ? c_top - u : 0;
            const float *v = vecs + (int64_t)c * (PAR_NVEC * CH_N);
            const int src = wv < 8 ? slab * 8 + wv                                 // totA
                          : wv < 16 ? 4 * CH_N + slab * 8 + wv - 8                 // sfxA
                          : wv < 16 + CH_N ? CH_N + wv - 16                        // totB
                          : 5 * CH_N + wv - 16 - CH_N;                             // sfxB
            tmp[it] = v[src];
        }
#pragma unroll
        for (int it = 0; it < SCAN_BATCH * SCAN_VEC / SCAN_TPB; ++it) vl[tid + it * SCAN_TPB] = tmp[it];
        __syncthreads();
        // the factors of all sixteen steps first (they do not depend on the chain), then the chain
        float tau0[SCAN_BATCH], tau1[SCAN_BATCH], sig0[SCAN_BATCH], sig1[SCAN_BATCH];
#pragma unroll
        for (int u = 0; u < SCAN_BATCH; ++u) {
            const float *v = vl + u * SCAN_VEC;
            const float ta = v[dl], sa = v[8 + dl] * PAR_STATE_SHIFT;      // Gh' is stored shifted
            const float2 tb = *reinterpret_cast<const float2 *>(v + 16 + k), sb = *reinterpret_cast<const float2 *>(v + 16 + CH_N + k);
            tau0[u] = ta * tb.x; tau1[u] = ta * tb.y;
            sig0[u] = sa * sb.x; sig1[u] = sa * sb.y;
        }
#pragma unroll
        for (int u = 0; u < SCAN_BATCH; ++u) {
            const int c = c_top - u;
            if (c >= 0) {
                *reinterpret_cast<u32 *>(gh + (int64_t)c * (CH_N * CH_N)) = Bf16::pack2(G0 * sig0[u], G1 * sig1[u]);
                G0 = G0 * tau0[u] + Bf16::to_f32((u16)(m[u] & 0xffffu));
                G1 = G1 * tau1[u] + Bf16::to_f32((u16)(m[u] >> 16));
            }
        }
    }
    *reinterpret_cast<u32 *>(reinterpret_cast<u16 *>(p.d_s0) + b * (CH_N * CH_N) + d * CH_N + k) = IOE::pack2(G0, G1);
    if (slab == 0) {                  // the row's verdict: any chunk the form cannot take (workgroup-uniform branch)
        int mine = 0;
        for (int cc = tid; cc < NC; cc += SCAN_TPB) mine |= p.chunk_flags[b * NC + cc];
        const int any = __syncthreads_or(mine);
        if (tid == 0) p.row_flags[b] = any ? 1 : 0;
    }
}

// ---- launch 3: gradients --------------------------------------------------------------------------
// One workgroup of 8 waves per (row, chunk) item; wave (side, cb) owns channel block cb of its side:
// lane (i, kg) owns channel 16 cb + i and the tokens 16 m + 4 kg + j (m < NT, j < 4) of the chunk.
// Two such workgroups fit a compute unit (LDS; 128 registers per lane, four waves per SIMD) and run
// independently of each other, so the memory latency and the barrier waits of one are filled with
// the other's work.
//   A  raw inputs (2-byte loads, a token row of a channel block = 32 contiguous bytes) -> gate products
//      relative to the middle of the chunk -> scaled operands -> channel-major tiles; the
//      chunk-start state (scaled, as bf16) and Gh' go to LDS                              | barrier
//   P  the token x token products of a side (P for the value side, W for the key side) are the same
//      for all channel blocks: the side's four waves share its ten 16 x 16 tiles (s <= t), mask
//      them and leave them in LDS as ready 16-bit A operands of the forward-like sweep, plus the
//      diagonal; the backward-like sweep reads the same tiles transposed                  | barrier
//   S  per side: forward-like sweep (o' / q'), backward-like sweep (x' / k'), gate gradient; the
//      results go to global memory from the accumulator layout
constexpr int GR_THREADS = 512;
constexpr int PT_TILE = 64 * 8;                  // one 16 x 16 product tile as 16-bit operand: 8 bytes per lane
constexpr int GR_ADJ = 0;                        // adjoint-scaled tile of each side
constexpr int GR_VAL = GR_ADJ + 2 * CM_BYTES;    // value-scaled tile of each side
constexpr int GR_S0 = GR_VAL + 2 * CM_BYTES, GR_GH = GR_S0 + CM_BYTES;
constexpr int GR_PT = GR_GH + CM_BYTES;          // per side: the 10 product tiles (m, n <= m)
constexpr int GR_PD = GR_PT + 2 * 10 * PT_TILE;  // per side: diagonal of the product, 64 floats
constexpr int GR_SMEM = GR_PD + 2 * CH_N * 4;
static_assert(2 * GR_SMEM <= 160 * 1024, "two workgroups of the gradient kernel must fit the LDS of one CU");

template <int NT> struct SideState {
    LaneChunk<NT> lc;
};

template <typename IOE, int NT, bool HEADS, bool FULL> struct GradsItem {
    static constexpr int CL = 16 * NT;
    const ParBwdArgs &p;
    unsigned char *smem;
    int tid, T, NC, cb, side, i, kg, c, lane, n_left;
    u32 ts, lane_off;
    int64_t item, chunk_off;

    __device__ __forceinline__ GradsItem(const ParBwdArgs &p_, unsigned char *smem_, int64_t item_) : p(p_), smem(smem_), item(item_) {
        tid = threadIdx.x;
        T = (int)p.T; NC = (int)p.NC;
        ts = HEADS ? (u32)p.heads * CH_N : (u32)CH_N;
        cb = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);
        side = __builtin_amdgcn_readfirstlane(tid >> 8);
        lane = tid & 63;
        i = lane & 15; kg = lane >> 4; c = 16 * cb + i;
        const int64_t b = item / NC;
        const int chunk = (int)(item - b * NC);
        n_left = T - (chunk * CL + 4 * kg);
        // element offsets in the [.., T, .., 64] arrays: the chunk's first token (wave-uniform: token addresses
        // are a scalar base plus the lane's fixed offset, whatever the token stride) and the lane's
        // (first token, channel) from there
        chunk_off = wave_uniform(row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N + (int64_t)(chunk * CL) * ts);
        lane_off = (u32)(4 * kg) * ts + (u32)c;
    }
    template <int SIDE> __device__ __forceinline__ u16 *tile_adj() const { return reinterpret_cast<u16 *>(smem + GR_ADJ + SIDE * CM_BYTES); }
    template <int SIDE> __device__ __forceinline__ u16 *tile_val() const { return reinterpret_cast<u16 *>(smem + GR_VAL + SIDE * CM_BYTES); }

    struct Raw {
        RawTokens<NT> g, v, a;
    };
    template <int SIDE> __device__ __forceinline__ void issue_raw(Raw &r) const {
        load_tokens<NT, FULL>(r.g, reinterpret_cast<const u16 *>(SIDE ? p.f_key : p.f) + chunk_off, lane_off, ts, n_left);
        load_tokens<NT, FULL>(r.v, reinterpret_cast<const u16 *>(SIDE ? p.k : p.x) + chunk_off, lane_off, ts, n_left);
        load_tokens<NT, FULL>(r.a, reinterpret_cast<const u16 *>(SIDE ? p.q : p.g_out) + chunk_off, lane_off, ts, n_left);
    }
    // phase A of one side: gate products relative to the middle of the chunk, scaled operands -> tiles
    template <int SIDE> __device__ __forceinline__ void prep(SideState<NT> &st, const Raw &r) const {
        float gt[NT][4], fv[NT][4], fa[NT][4];
        gate_scan<IOE, NT, FULL, true>(st.lc, gt, r.g, kg, n_left);      // products relative to the middle of the chunk
        to_floats<IOE, NT, FULL>(fv, r.v, n_left);
        to_floats<IOE, NT, FULL>(fa, r.a, n_left);
        // 1 / pre lives only here: the sweeps take the reciprocals again where they use them, which costs four
        // instructions per token tile and frees sixteen registers for the whole kernel
        float inv[NT][4];
        inverse_products<NT>(inv, st.lc, gt);
        uint2 valT[NT], adjS[NT];
        scale_pack<NT>(valT, fv, inv);
        scale_pack<NT>(adjS, fa, st.lc.pre);
        store_cm<NT>(tile_val<SIDE>(), c, kg, valT);
        store_cm<NT>(tile_adj<SIDE>(), c, kg, adjS);
    }
    // the chunk-start state scaled to the middle of the chunk, as bf16, and Gh': one 16-byte piece of each
    // per thread (eight columns (tid & 7) of row tid >> 3); the loads are issued with the raw inputs
    struct MatRegs {
        uint4 s0, gh;
        float ra;
        float4 rb[2];
    };
    __device__ __forceinline__ void issue_mats(MatRegs &r) const {
        const float *const vref = p.vecs + item * (PAR_NVEC * CH_N);
        r.s0 = *reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.ckpt) + item * (CH_N * CH_N) + tid * 8);
        r.gh = *reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.gh) + item * (CH_N * CH_N) + tid * 8);
        r.ra = vref[2 * CH_N + (tid >> 3)];
        r.rb[0] = *reinterpret_cast<const float4 *>(vref + 3 * CH_N + (tid & 7) * 8);
        r.rb[1] = *reinterpret_cast<const float4 *>(vref + 3 * CH_N + (tid & 7) * 8 + 4);
    }
    __device__ __forceinline__ void stage_mats(const MatRegs &r) const {
        const float rbv[8] = {r.rb[0].x, r.rb[0].y, r.rb[0].z, r.rb[0].w, r.rb[1].x, r.rb[1].y, r.rb[1].z, r.rb[1].w};
        const u32 sw[4] = {r.s0.x, r.s0.y, r.s0.z, r.s0.w};
        const float ras = r.ra * PAR_STATE_SHIFT;                 // S0' is stored shifted
        float v[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[2 * e] = IOE::to_f32((u16)(sw[e] & 0xffffu)) * (ras * rbv[2 * e]);
            v[2 * e + 1] = IOE::to_f32((u16)(sw[e] >> 16)) * (ras * rbv[2 * e + 1]);
        }
        const int o = (tid >> 3) * CMS + (tid & 7) * 8;
        *reinterpret_cast<uint4 *>(reinterpret_cast<u16 *>(smem + GR_S0) + o) =
            make_uint4(Bf16::pack2(v[0], v[1]), Bf16::pack2(v[2], v[3]), Bf16::pack2(v[4], v[5]), Bf16::pack2(v[6], v[7]));
        *reinterpret_cast<uint4 *>(reinterpret_cast<u16 *>(smem + GR_GH) + o) = r.gh;
    }
    // Product tile (m, n), n <= m, of a side: element [t = 16 m + i][s = 16 n + 4 kg + j] in lane (i, kg),
    // kept for s < t; that is the A operand of the forward-like sweep.  The backward-like sweep contracts
    // over t and reads the same tile transposed.
    template <int SIDE> __device__ __forceinline__ u16 *pt_tile(int m, int n) const {
        return reinterpret_cast<u16 *>(smem + GR_PT + SIDE * 10 * PT_TILE + (m * (m + 1) / 2 + n) * PT_TILE);
    }
    template <int SIDE> __device__ __forceinline__ uint2 fw_read(int m, int n) const {
        return reinterpret_cast<const uint2 *>(pt_tile<SIDE>(m, n))[lane];
    }
    // lane (i, kg) receives [t = 16 m + 4 kg + j][s = 16 n + i]: row j of that 4 x 16 block lies in the four
    // 8-byte pieces of lanes (4 kg + j, 0 .. 3)
    template <int SIDE> __device__ __forceinline__ uint2 bw_read(int m, int n) const {
        const u16 *q = pt_tile<SIDE>(m, n) + 4 * (16 * (i & 3) + 4 * kg + (i >> 2));
        return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(q)));
    }
    template <int SIDE> __device__ __forceinline__ float *diag() const { return reinterpret_cast<float *>(smem + GR_PD) + SIDE * CH_N; }

    // phase P of one side: the ten (NT = 4) or three (NT = 2) product tiles, spread over the side's four waves
    template <int SIDE> __device__ __forceinline__ void product_tile(int m, int n, const uint4 &w0, const uint4 &w1) const {
        const u16 *const oth_adj = tile_adj<1 - SIDE>();
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
        const uint4 a0 = tok_rows_op(oth_adj, 16 * m, 0, i, kg), a1 = tok_rows_op(oth_adj, 16 * m, 1, i, kg);
        const floatx4 pt = Bf16::mfma32(w1, a1, Bf16::mfma32(w0, a0, zero));             // [s][t]
        if (m == n) {
            float dg[4];
            tile_diagonal(dg, pt, kg);
            if (i == 0) *reinterpret_cast<float4 *>(diag<SIDE>() + 16 * m + 4 * kg) = make_float4(dg[0], dg[1], dg[2], dg[3]);
            reinterpret_cast<uint2 *>(pt_tile<SIDE>(m, n))[lane] = mask_pack<KEEP_ROW_LT_COL>(pt, i, kg);
        } else {
            reinterpret_cast<uint2 *>(pt_tile<SIDE>(m, n))[lane] = mask_pack<KEEP_ALL>(pt, i, kg);
        }
    }
    template <int SIDE> __device__ __forceinline__ void products() const {
        const u16 *const oth_val = tile_val<1 - SIDE>();
        // wave cb: the diagonal tile (cb, cb) and, of the others, those of token column n = cb; the last
        // wave has only its diagonal tile in that column and takes (1, 0) over from the first
        if (cb < NT) {
            const uint4 w0 = tok_rows_op(oth_val, 16 * cb, 0, i, kg), w1 = tok_rows_op(oth_val, 16 * cb, 1, i, kg);
            product_tile<SIDE>(cb, cb, w0, w1);
#pragma unroll
            for (int m = NT - 1; m > 1; --m)
                if (m > cb) product_tile<SIDE>(m, cb, w0, w1);
            if (NT == 2 && cb == 0) product_tile<SIDE>(1, 0, w0, w1);
        }
        if (NT == 4 && cb == 3) {
            const uint4 w0 = tok_rows_op(oth_val, 0, 0, i, kg), w1 = tok_rows_op(oth_val, 0, 1, i, kg);
            product_tile<SIDE>(1, 0, w0, w1);
        }
    }

    // phase S of one side, in pieces per token tile
    template <int SIDE> struct Sweep {
        const GradsItem &g;
        const SideState<NT> &st;
        const u16 *own_adj, *own_val, *oth_adj, *oth_val;
        const float *pd;
        u16 *d_val, *d_gate, *d_adj;
        float du[NT][4];
        float anchor_acc;                        // sum_t adjS_t * (S0' adj-op_t)
        float anchor, carry;                     // gate gradient: see begin_gate_gradient
        float chk;                               // 0 until a stored result is inf or NaN, then NaN

        __device__ __forceinline__ Sweep(const GradsItem &g_, const SideState<NT> &st_) : g(g_), st(st_) {
            own_adj = g.template tile_adj<SIDE>(); own_val = g.template tile_val<SIDE>();
            oth_adj = g.template tile_adj<1 - SIDE>(); oth_val = g.template tile_val<1 - SIDE>();
            pd = g.template diag<SIDE>();
            // at the chunk's first token (wave-uniform); a store adds the token's scalar offset and the
            // lane's fixed one
            d_val = reinterpret_cast<u16 *>(SIDE ? g.p.d_k : g.p.d_x) + g.chunk_off;
            d_gate = reinterpret_cast<u16 *>(SIDE ? g.p.d_f_key : g.p.d_f) + g.chunk_off;
            d_adj = reinterpret_cast<u16 *>(g.p.d_q) + g.chunk_off;          // key side only
            anchor_acc = 0.f;
            chk = 0.f;
        }
        // operands of the own side (this lane's channel, tokens 16 m + 4 kg + j), re-read from the own tiles
        __device__ __forceinline__ uint2 b_val(int m) const { return ld2(own_val + g.c * CMS + 16 * m + 4 * g.kg); }
        __device__ __forceinline__ uint2 b_adj(int m) const { return ld2(own_adj + g.c * CMS + 16 * m + 4 * g.kg); }
        // state operands: own channel in the lane, the other side's channels contracted
        __device__ __forceinline__ uint4 state_op(int region, int h) const {
            const u16 *mt = reinterpret_cast<const u16 *>(g.smem + region);
            return SIDE ? mat_cols_op(mt, 16 * g.cb, h, g.i, g.kg) : mat_rows_op(mt, 16 * g.cb, h, g.i, g.kg);
        }
        __device__ __forceinline__ void store4(u16 *dst, int mm, const float (&v)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (IOE::CHECK_RESULTS) chk = __builtin_fmaf(v[j], 0.0f, chk);
                if (FULL || 16 * mm + j < g.n_left) (dst + (size_t)(16 * mm + j) * g.ts)[g.lane_off] = cvt1<IOE>(v[j]);
            }
        }
        // forward-like sweep, token tile m: o' (value side) / q' (key side)
        __device__ __forceinline__ void forward_tile(int m, const uint4 &s0a, const uint4 &s0b) {
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            const uint2 none = make_uint2(0u, 0u);
            const uint4 a0 = tok_rows_op(oth_adj, 16 * m, 0, g.i, g.kg), a1 = tok_rows_op(oth_adj, 16 * m, 1, g.i, g.kg);
            floatx4 acc = Bf16::mfma32(a1, s0b, Bf16::mfma32(a0, s0a, zero));
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] *= PAR_STATE_UNSHIFT;
            float af[4];
            unpack4<Bf16>(b_adj(m), af);
#pragma unroll
            for (int j = 0; j < 4; ++j) anchor_acc += af[j] * acc[j];
#pragma unroll
            for (int n0 = 0; n0 <= m; n0 += 2)
                acc = Bf16::mfma32(cat(g.template fw_read<SIDE>(m, n0), n0 + 1 <= m ? g.template fw_read<SIDE>(m, n0 + 1) : none),
                                   cat(b_val(n0), n0 + 1 <= m ? b_val(n0 + 1) : none), acc);
            if (SIDE == 1) {
                const float4 dgv = *reinterpret_cast<const float4 *>(pd + 16 * m + 4 * g.kg);
                const float dg[4] = {dgv.x, dgv.y, dgv.z, dgv.w};
                float vf[4], dq[4];
                unpack4<Bf16>(b_val(m), vf);
#pragma unroll
                for (int j = 0; j < 4; ++j) dq[j] = st.lc.pre[m][j] * (acc[j] + vf[j] * dg[j]);
                store4(d_adj, m, dq);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) du[m][j] = af[j] * acc[j];
        }
        // gate gradient = (anchor - sum over the earlier tokens of du) / gate; diag = rowsum / colsum of Gh' * S0'
        __device__ __forceinline__ void begin_gate_gradient(float diag_part) {
            anchor = diag_part + row_scan_add(anchor_acc, g.kg).all;
            carry = 0.f;
        }
        // backward-like sweep, token tile n: x' (value side) / k' (key side); then the tile's gate gradient (du of
        // this tile and of the earlier ones is final by now)
        __device__ __forceinline__ void backward_tile(int n, const uint4 &gha, const uint4 &ghb) {
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            const uint2 none = make_uint2(0u, 0u);
            const uint4 v0 = tok_rows_op(oth_val, 16 * n, 0, g.i, g.kg), v1 = tok_rows_op(oth_val, 16 * n, 1, g.i, g.kg);
            floatx4 acc = Bf16::mfma32(v1, ghb, Bf16::mfma32(v0, gha, zero));
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] *= PAR_STATE_UNSHIFT;
#pragma unroll
            for (int m0 = n; m0 < NT; m0 += 2)
                acc = Bf16::mfma32(cat(g.template bw_read<SIDE>(m0, n), m0 + 1 < NT ? g.template bw_read<SIDE>(m0 + 1, n) : none),
                                   cat(b_adj(m0), m0 + 1 < NT ? b_adj(m0 + 1) : none), acc);
            const float4 dgv = *reinterpret_cast<const float4 *>(pd + 16 * n + 4 * g.kg);
            const float dg[4] = {dgv.x, dgv.y, dgv.z, dgv.w};
            float af[4], vf[4], dv[4], inv[4];
            unpack4<Bf16>(b_adj(n), af);
            unpack4<Bf16>(b_val(n), vf);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                inv[j] = __builtin_amdgcn_rcpf(st.lc.pre[n][j]);
                dv[j] = inv[j] * (acc[j] + af[j] * dg[j]);
                du[n][j] -= vf[j] * acc[j];
            }
            store4(d_val, n, dv);
            float e[4];
            e[0] = 0.f;
#pragma unroll
            for (int j = 1; j < 4; ++j) e[j] = e[j - 1] + du[n][j - 1];
            const RowScan sc = row_scan_add(e[3] + du[n][3], g.kg);
            const float base = anchor - (carry + sc.lower);
            carry += sc.all;
            float dgt[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float rgate = (j == 0 ? st.lc.off[n] : st.lc.pre[n][j > 0 ? j - 1 : 0]) * inv[j];      // 1 / gate
                dgt[j] = (base - e[j]) * rgate;
            }
            store4(d_gate, n, dgt);
        }
        // rowsum / colsum of Gh' * S0' = diagonal of Gh' S0'^T
        __device__ __forceinline__ float state_diagonal(const uint4 &s0a, const uint4 &s0b, const uint4 &gha, const uint4 &ghb) const {
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            const floatx4 d = Bf16::mfma32(ghb, s0b, Bf16::mfma32(gha, s0a, zero));
            const int jj = g.i & 3;
            const float sel = jj == 0 ? d[0] : (jj == 1 ? d[1] : (jj == 2 ? d[2] : d[3]));      // element (i, i), held by row i / 4
            return __shfl(sel, 16 * (g.i >> 2) + g.i, 64) * (PAR_STATE_UNSHIFT * PAR_STATE_UNSHIFT);
        }
    };

    template <int SIDE> __device__ __forceinline__ void sweeps(const SideState<NT> &st) const {
        Sweep<SIDE> w(*this, st);
        float diag_part;
        {
            const uint4 s0a = w.state_op(GR_S0, 0), s0b = w.state_op(GR_S0, 1);
            diag_part = w.state_diagonal(s0a, s0b, w.state_op(GR_GH, 0), w.state_op(GR_GH, 1));
#pragma unroll
            for (int m = 0; m < NT; ++m) {
                lds_fence();
                w.forward_tile(m, s0a, s0b);
            }
        }
        {
            lds_fence();
            const uint4 gha = w.state_op(GR_GH, 0), ghb = w.state_op(GR_GH, 1);
            w.begin_gate_gradient(diag_part);
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                lds_fence();
                w.backward_tile(n, gha, ghb);
            }
        }
        // A result that is not finite (a scaled operand or a product of scaled operands left the range of its
        // type) declines the row after the fact: the launch that follows redoes it.
        if (!(w.chk == 0.0f)) p.row_flags[item / NC] = 1;
    }

    template <int SIDE> __device__ __forceinline__ void run_side() const {
        SideState<NT> st;
        {
            // The row's verdict (second launch) is fetched with the inputs and looked at once they are in (a branch
            // before that would have the compiler move the input loads behind it).  A row that the form cannot take
            // is left alone from there on: the launch that follows redoes it whole, and under T2FW_FLAG_NO_FIXUP
            // its results are declared invalid anyway.  The branch is uniform over the workgroup.
            const int declined = p.row_flags[item / NC];
            Raw r;
            MatRegs mr;
            issue_raw<SIDE>(r);
            issue_mats(mr);
            prep<SIDE>(st, r);
            stage_mats(mr);
            if (__builtin_amdgcn_readfirstlane(declined)) return;
        }
        __syncthreads();                         // tiles, S0', Gh' complete
        products<SIDE>();
        __syncthreads();                         // product tiles complete
        sweeps<SIDE>(st);
    }
    __device__ __forceinline__ void run() const {
        if (side == 0)                           // wave-uniform; both branches meet the same two barriers
            run_side<0>();
        else
            run_side<1>();
    }
};

template <typename IOE, int NT, bool HEADS>
__global__ __launch_bounds__(GR_THREADS, 4) void lfw_par_grads_kernel(ParBwdArgs p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int64_t item = blockIdx.x;
    if ((int)(item % p.NC) * 16 * NT + 16 * NT <= (int)p.T)
        GradsItem<IOE, NT, HEADS, true>(p, smem, item).run();
    else
        GradsItem<IOE, NT, HEADS, false>(p, smem, item).run();
}

template <typename IOE, int NT, bool HEADS> int launch(const ParBwdArgs &a, hipStream_t stream) {
    auto incr = lfw_par_incr_kernel<IOE, NT, HEADS>;
    auto scan = lfw_par_scan_kernel<IOE>;
    auto grads = lfw_par_grads_kernel<IOE, NT, HEADS>;
    int rc = enable_lds(reinterpret_cast<const void *>(grads), GR_SMEM, "hipFuncSetAttribute(gradient kernel)");
    if (rc) return rc;
    const int64_t items = a.B * a.NC;
    if (items > 0x3fffffffLL || a.B > 0x0fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B * chunks = %lld is too large", (long long)items);
    if (a.heads < 1 || a.T * a.heads >= CHUNK_MAX_T || a.B * a.T * CH_N >= 0x7fffffffLL)
        return fail(T2FW_ERR_UNSUPPORTED, "B=%lld T=%lld with %d heads is too large for 32-bit element offsets", (long long)a.B, (long long)a.T, a.heads);
    hipLaunchKernelGGL(incr, dim3((unsigned)items), dim3(PAR_THREADS), INCR_SMEM, stream, a);
    if ((rc = check_hip(hipGetLastError(), "lfw_par_incr_kernel launch"))) return rc;
    hipLaunchKernelGGL(scan, dim3((unsigned)(64 * ((a.B + 7) / 8))), dim3(SCAN_TPB), 0, stream, a);
    if ((rc = check_hip(hipGetLastError(), "lfw_par_scan_kernel launch"))) return rc;
    hipLaunchKernelGGL(grads, dim3((unsigned)items), dim3(GR_THREADS), GR_SMEM, stream, a);
    return check_hip(hipGetLastError(), "lfw_par_grads_kernel launch");
}

template <typename IOE> int by_chunk(const ParBwdArgs &a, hipStream_t stream) {
    if (a.C == 64) return a.heads == 1 ? launch<IOE, 4, false>(a, stream) : launch<IOE, 4, true>(a, stream);
    if (a.C == 32) return a.heads == 1 ? launch<IOE, 2, false>(a, stream) : launch<IOE, 2, true>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunk-parallel backward takes checkpoint intervals 32 or 64");
}

}  // namespace

int par_backward(const ParBwdArgs &a, int dtype, hipStream_t stream) {
    if (dtype == T2FW_F16) return by_chunk<Fp16>(a, stream);
    if (dtype == T2FW_BF16) return by_chunk<Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunk-parallel kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
