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
// gate products.  Launch 2 (lfw_par_scan_kernel, elementwise, 32 workgroups per row): the
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
    const int64_t off = row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N + (int64_t)tok0 * ts + c;
    const u16 *const gate = reinterpret_cast<const u16 *>(side ? p.f_key : p.f) + off;
    const u16 *const adj = reinterpret_cast<const u16 *>(side ? p.q : p.g_out) + off;
    u32 bad;
    {
        RawTokens<NT> rg, ra;
        LaneChunk<NT> lc;
        float gt[NT][4], av[NT][4];
        if (chunk * CL + CL <= T) {
            load_tokens<NT, true>(rg, gate, ts, n_left);
            load_tokens<NT, true>(ra, adj, ts, n_left);
            gate_scan<IOE, NT, true>(lc, gt, rg, kg, n_left);
            to_floats<IOE, NT, true>(av, ra, n_left);
        } else {
            load_tokens<NT, false>(rg, gate, ts, n_left);
            load_tokens<NT, false>(ra, adj, ts, n_left);
            gate_scan<IOE, NT, false>(lc, gt, rg, kg, n_left);
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
    const int64_t b = blockIdx.x >> 3;
    const int slab = (int)(blockIdx.x & 7), tid = threadIdx.x;
    const int dl = tid >> 5, d = slab * 8 + dl, k = (tid & 31) * 2;
    const int NC = (int)p.NC;
    PT_DECL;
    PT_MARK();
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
        PT_MARK();
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
        PT_MARK();
        __syncthreads();
        PT_MARK();
        // the factors of all sixteen steps first (they do not depend on the chain), then the chain
        float tau0[SCAN_BATCH], tau1[SCAN_BATCH], sig0[SCAN_BATCH], sig1[SCAN_BATCH];
#pragma unroll
        for (int u = 0; u < SCAN_BATCH; ++u) {
            const float *v = vl + u * SCAN_VEC;
            const float ta = v[dl], sa = v[8 + dl];
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
    PT_MARK();
    *reinterpret_cast<u32 *>(reinterpret_cast<u16 *>(p.d_s0) + b * (CH_N * CH_N) + d * CH_N + k) = IOE::pack2(G0, G1);
    if (slab == 0) {                  // the row's verdict: any chunk the form cannot take (workgroup-uniform branch)
        int mine = 0;
        for (int cc = tid; cc < NC; cc += SCAN_TPB) mine |= p.chunk_flags[b * NC + cc];
        const int any = __syncthreads_or(mine);
        if (tid == 0) p.row_flags[b] = any ? 1 : 0;
    }
    PT_MARK();
#ifdef T2FW_PAR_TIMERS
    if (p.dbg != nullptr) p.dbg += 16 * 32;      // after the gradient kernel's slots
#endif
    PT_FLUSH(p);
}

// ---- launch 3: gradients --------------------------------------------------------------------------
// Workgroups of 8 waves = (side, channel block cb), persistent (one per compute unit), walking over
// (row, chunk) items.  Lane (i, kg) of a wave owns channel 16 cb + i of its side and the tokens
// 16 m + 4 kg + j (m < NT, j < 4) of the chunk.  Per item:
//   A  every lane picks its channel's tokens out of the staged inputs, builds the gate products
//      relative to the middle of the chunk and the scaled operands, and writes the latter to the
//      channel-major tiles; the chunk-start state (scaled, as bf16) and Gh' go to LDS     | barrier
//   P  the token x token products of a side (P for the value side, W for the key side) are the same
//      for its four waves: wave cb computes the tiles of token column cb (forward-like orientation)
//      and of token row cb (backward-like orientation), 5 of the 20 tiles, masks them and leaves
//      them in LDS as ready 16-bit A operands, plus the diagonal                          | barrier
//   S  forward-like sweep (o' / q'), backward-like sweep (x' / k'), gate gradient; the results go
//      to global memory from the accumulator layout                                       | barrier
// The six input arrays of an item (64 token rows of 128 bytes each) come in with 16-byte loads that
// write straight into LDS (no registers), issued for the NEXT item at the start of phase P of the
// current one, so that they travel while it computes.
constexpr int RAW_BYTES = CH_N * CH_N * 2;       // one staged input array: 64 token rows of 128 bytes
constexpr int PT_TILE = 64 * 8;                  // one 16 x 16 product tile as 16-bit operand: 8 bytes per lane
constexpr int GR_RAW = 0;                        // six arrays: f, x, g_out, f_key, k, q
constexpr int GR_ADJ = GR_RAW + 6 * RAW_BYTES;   // adjoint-scaled tile of each side
constexpr int GR_VAL = GR_ADJ + 2 * CM_BYTES;    // value-scaled tile of each side
constexpr int GR_S0 = GR_VAL + 2 * CM_BYTES, GR_GH = GR_S0 + CM_BYTES;
constexpr int GR_PT = GR_GH + CM_BYTES;          // per side: 16 forward-like tiles [m][n], 16 backward-like tiles [n][m]
constexpr int GR_PD = GR_PT + 2 * 32 * PT_TILE;  // per side: diagonal of the product, 64 floats
constexpr int GR_SMEM = GR_PD + 2 * CH_N * 4;
static_assert(GR_SMEM <= 160 * 1024, "gradient kernel tiles exceed the LDS of one CU");

// Row slot of token t in a staged array: rows are 128 bytes, i.e. two rows span all LDS banks, and the
// four row groups of a wave read tokens four apart; swapping each odd group's neighbouring rows
// leaves two groups per bank half instead of four.
__device__ __forceinline__ int raw_slot(int t) { return t ^ ((t >> 2) & 1); }

typedef __attribute__((address_space(3))) void *lds_void_ptr;

// the lane's tokens of one staged input array: [m][j] = token 4 kg + 16 m + j, channel c
template <int NT> __device__ __forceinline__ void raw_from_lds(RawTokens<NT> &r, const unsigned char *arr, int c, int kg) {
    const unsigned char *a = arr + 4 * kg * 128 + c * 2;
    const int flip = (kg & 1) * 128;             // raw_slot: odd row groups swap neighbouring rows
#pragma unroll
    for (int m = 0; m < NT; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u16 v = *reinterpret_cast<const u16 *>(a + 16 * m * 128 + ((j * 128) ^ flip));
            if (j & 1)
                r.p[m][j >> 1].y = v;
            else
                r.p[m][j >> 1].x = v;
        }
}

struct GradsMats {
    uint4 s0, gh;      // eight columns of one row of the chunk-start state and of Gh'
};

template <typename IOE, int NT, bool HEADS, int SIDE> struct GradsWave {
    static constexpr int CL = 16 * NT;
    const ParBwdArgs &p;
    unsigned char *smem;
    int tid, T, NC, cb, i, kg, c, lane;
    u32 ts;

    __device__ __forceinline__ GradsWave(const ParBwdArgs &p_, unsigned char *smem_) : p(p_), smem(smem_) {
        tid = threadIdx.x;
        T = (int)p.T; NC = (int)p.NC;
        ts = HEADS ? (u32)p.heads * CH_N : (u32)CH_N;
        const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
        lane = tid & 63;
        cb = w & 3; i = lane & 15; kg = lane >> 4; c = 16 * cb + i;
    }

    // The six input arrays of an item: global -> LDS staging area, asynchronously, 1 KB per
    // instruction.  NWAVES waves (w = 0 .. NWAVES - 1) share the 48 instructions.  LDS instructions
    // of a wave queue behind its own outstanding loads of this kind, so they are issued by waves that
    // have no LDS work ahead of them (the value-side waves, before their gate-gradient phase).
    template <int NWAVES> __device__ __forceinline__ void issue_inputs(int item, int w) const {
        const int64_t b = item / NC;
        const int chunk = item - (int)b * NC;
        const int64_t row = row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N;
#pragma unroll
        for (int u = 0; u < 48 / NWAVES; ++u) {
            const int q = w + NWAVES * u, arr = q >> 3, r = q & 7;   // array, group of eight row slots
            const void *base = arr == 0 ? p.f : arr == 1 ? p.x : arr == 2 ? p.g_out : arr == 3 ? p.f_key : arr == 4 ? p.k : p.q;
            const int tok = min(chunk * CL + raw_slot(8 * r + (lane >> 3)), T - 1);
            const u16 *src = reinterpret_cast<const u16 *>(base) + row + (int64_t)tok * ts + (lane & 7) * 8;
            // 64 lanes x 16 bytes -> 1 KB of LDS starting at the wave-uniform address in M0.  Issued as
            // inline assembly: through the builtin the compiler makes every later LDS read wait for
            // these loads (it cannot tell that the staging area and the operand tiles are disjoint);
            // body() waits for them itself before the barrier that publishes the staging area.
            const u32 dst = (u32)(uintptr_t)(lds_void_ptr)(smem + GR_RAW + arr * RAW_BYTES + r * 1024);
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(dst) : "m0", "memory");
        }
    }
    __device__ __forceinline__ void issue_mats(GradsMats &mt, int item) const {
        const int64_t mat = (int64_t)item * (CH_N * CH_N) + tid * 8;
        mt.s0 = *reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.ckpt) + mat);
        mt.gh = *reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.gh) + mat);
    }

    // One item.  On entry the staged inputs of the item are in LDS and mats holds the thread's pieces of
    // its state and Gh'; on return the same holds for item `next` (if >= 0).
    template <bool FULL, typename PT> __device__ __forceinline__ void body(int item, int next, GradsMats &mats, PT &pt_t, int &pt_n) const {
        constexpr int side = SIDE;
        const int64_t b = item / NC;
        const int chunk = item - (int)b * NC;
        const int n_left = T - (chunk * CL + 4 * kg);
        // element offset of (the lane's first token, its channel) in the [.., T, .., 64] arrays (the launcher
        // admits arrays of less than 2^31 elements only)
        const u32 off = (u32)(row_first_token(b, p.T, HEADS ? p.heads : 1) * CH_N) + (u32)(chunk * CL + 4 * kg) * ts + (u32)c;
        u16 *const own_adj = reinterpret_cast<u16 *>(smem + GR_ADJ + side * CM_BYTES);
        u16 *const own_val = reinterpret_cast<u16 *>(smem + GR_VAL + side * CM_BYTES);

        // ---- phase A
        PT_MARK();
        const float *const vref = p.vecs + (int64_t)item * (PAR_NVEC * CH_N);
        const float ref_a = vref[2 * CH_N + (tid >> 3)];
        const float4 ref_b0 = *reinterpret_cast<const float4 *>(vref + 3 * CH_N + (tid & 7) * 8);
        const float4 ref_b1 = *reinterpret_cast<const float4 *>(vref + 3 * CH_N + (tid & 7) * 8 + 4);
        LaneChunk<NT> lc;
        float inv[NT][4];
        {
            uint2 valT[NT], adjS[NT];
            RawTokens<NT> rg, rv, ra;
            raw_from_lds(rg, smem + GR_RAW + (3 * side + 0) * RAW_BYTES, c, kg);
            raw_from_lds(rv, smem + GR_RAW + (3 * side + 1) * RAW_BYTES, c, kg);
            raw_from_lds(ra, smem + GR_RAW + (3 * side + 2) * RAW_BYTES, c, kg);
            float gt[NT][4], fv[NT][4], fa[NT][4];
            gate_scan<IOE, NT, FULL>(lc, gt, rg, kg, n_left);
            lc.scale_by(__builtin_amdgcn_rcpf(lc.ref));      // the products up to the middle of the chunk divide out
            to_floats<IOE, NT, FULL>(fv, rv, n_left);
            to_floats<IOE, NT, FULL>(fa, ra, n_left);
            inverse_products<NT>(inv, lc, gt);
            scale_pack<NT>(valT, fv, inv);
            scale_pack<NT>(adjS, fa, lc.pre);
            store_cm<NT>(own_val, c, kg, valT);
            store_cm<NT>(own_adj, c, kg, adjS);
        }
        {
            // the state scaled to the middle of the chunk, as bf16, and Gh'
            float v[8];
            const u32 sw[4] = {mats.s0.x, mats.s0.y, mats.s0.z, mats.s0.w};
            const float rb[8] = {ref_b0.x, ref_b0.y, ref_b0.z, ref_b0.w, ref_b1.x, ref_b1.y, ref_b1.z, ref_b1.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[2 * e] = IOE::to_f32((u16)(sw[e] & 0xffffu)) * (ref_a * rb[2 * e]);
                v[2 * e + 1] = IOE::to_f32((u16)(sw[e] >> 16)) * (ref_a * rb[2 * e + 1]);
            }
            const int o = (tid >> 3) * CMS + (tid & 7) * 8;
            *reinterpret_cast<uint4 *>(reinterpret_cast<u16 *>(smem + GR_S0) + o) =
                make_uint4(Bf16::pack2(v[0], v[1]), Bf16::pack2(v[2], v[3]), Bf16::pack2(v[4], v[5]), Bf16::pack2(v[6], v[7]));
            *reinterpret_cast<uint4 *>(reinterpret_cast<u16 *>(smem + GR_GH) + o) = mats.gh;
        }
        PT_MARK();
        __syncthreads();                         // tiles, S0', Gh' complete; the staged inputs are consumed
        PT_MARK();

        // ---- phase P: the next item's inputs start travelling; product tiles of this side
        if (next >= 0) issue_mats(mats, next);
        const u16 *const oth_adj = reinterpret_cast<const u16 *>(smem + GR_ADJ + (1 - side) * CM_BYTES);
        const u16 *const oth_val = reinterpret_cast<const u16 *>(smem + GR_VAL + (1 - side) * CM_BYTES);
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
        const uint2 none = make_uint2(0u, 0u);
        unsigned char *const pt_side = smem + GR_PT + side * 32 * PT_TILE;
        // forward-like tile (m, n), n <= m: rows s = 16 n + 4 kg + j, column t = 16 m + i, kept for s < t;
        // backward-like tile (n, m), m >= n: rows t = 16 m + 4 kg + j, column s = 16 n + i, kept for t > s
        auto fw_tile = [&](int m, int n) { return reinterpret_cast<uint2 *>(pt_side + (m * 4 + n) * PT_TILE) + lane; };
        auto bw_tile = [&](int n, int m) { return reinterpret_cast<uint2 *>(pt_side + (16 + n * 4 + m) * PT_TILE) + lane; };
        float *const pd = reinterpret_cast<float *>(smem + GR_PD) + side * CH_N;
        if (cb < NT) {                           // wave-uniform; token column / row cb of the product
            // branch-free in cb: tiles with n > cb (m < cb) are computed and dropped
            const uint4 a0 = tok_rows_op(oth_adj, 16 * cb, 0, i, kg), a1 = tok_rows_op(oth_adj, 16 * cb, 1, i, kg);
            const uint4 v0 = tok_rows_op(oth_val, 16 * cb, 0, i, kg), v1 = tok_rows_op(oth_val, 16 * cb, 1, i, kg);
            {
                const floatx4 pt = Bf16::mfma32(v1, a1, Bf16::mfma32(v0, a0, zero));             // [s][t], diagonal tile
                float dg[4];
                tile_diagonal(dg, pt, kg);
                if (i == 0) *reinterpret_cast<float4 *>(pd + 16 * cb + 4 * kg) = make_float4(dg[0], dg[1], dg[2], dg[3]);
                *fw_tile(cb, cb) = mask_pack<KEEP_ROW_LT_COL>(pt, i, kg);
                const floatx4 pb = Bf16::mfma32(a1, v1, Bf16::mfma32(a0, v0, zero));             // [t][s], diagonal tile
                *bw_tile(cb, cb) = mask_pack<KEEP_ROW_GT_COL>(pb, i, kg);
            }
#pragma unroll
            for (int o = 0; o < NT; ++o) {
                if (o < cb) {                    // forward-like tiles of column cb: n = o < m = cb
                    const uint4 w0 = tok_rows_op(oth_val, 16 * o, 0, i, kg), w1 = tok_rows_op(oth_val, 16 * o, 1, i, kg);
                    *fw_tile(cb, o) = mask_pack<KEEP_ALL>(Bf16::mfma32(w1, a1, Bf16::mfma32(w0, a0, zero)), i, kg);
                } else if (o > cb) {             // backward-like tiles of row cb: m = o > n = cb
                    const uint4 w0 = tok_rows_op(oth_adj, 16 * o, 0, i, kg), w1 = tok_rows_op(oth_adj, 16 * o, 1, i, kg);
                    *bw_tile(cb, o) = mask_pack<KEEP_ALL>(Bf16::mfma32(w1, v1, Bf16::mfma32(w0, v0, zero)), i, kg);
                }
            }
        }
        PT_MARK();
        __syncthreads();                         // product tiles complete
        PT_MARK();

        // ---- phase S
        // operands of the own side (this lane's channel, tokens 16 m + 4 kg + j), re-read from the own tiles
        auto b_val = [&](int m) { return ld2(own_val + c * CMS + 16 * m + 4 * kg); };
        auto b_adj = [&](int m) { return ld2(own_adj + c * CMS + 16 * m + 4 * kg); };
        const u16 *const S0 = reinterpret_cast<const u16 *>(smem + GR_S0), *const GH = reinterpret_cast<const u16 *>(smem + GR_GH);
        // state operands: own channel in the lane, the other side's channels contracted
        auto state_op = [&](const u16 *mt, int h) { return side ? mat_cols_op(mt, 16 * cb, h, i, kg) : mat_rows_op(mt, 16 * cb, h, i, kg); };
        u16 *const d_val = reinterpret_cast<u16 *>(side ? p.d_k : p.d_x);
        u16 *const d_gate = reinterpret_cast<u16 *>(side ? p.d_f_key : p.d_f);
        u16 *const d_adj = reinterpret_cast<u16 *>(p.d_q);             // key side only
        auto store4 = [&](u16 *dst, int mm, const float (&v)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (FULL || 16 * mm + j < n_left) dst[off + (u32)(16 * mm + j) * ts] = cvt1<IOE>(v[j]);
        };
        const uint4 s0a = state_op(S0, 0), s0b = state_op(S0, 1);
        const uint4 gha = state_op(GH, 0), ghb = state_op(GH, 1);
        // anchor of the gate-gradient sums: rowsum / colsum of Gh' * S0' = diagonal of Gh' S0'^T ...
        float anchor;
        {
            const floatx4 d = Bf16::mfma32(ghb, s0b, Bf16::mfma32(gha, s0a, zero));
            const int jj = i & 3;
            const float sel = jj == 0 ? d[0] : (jj == 1 ? d[1] : (jj == 2 ? d[2] : d[3]));      // element (i, i), held by row i / 4
            anchor = __shfl(sel, 16 * (i >> 2) + i, 64);
        }
        // forward-like sweep: o' (value side) / q' (key side), token tile m
        float du[NT][4];
        float anchor_acc = 0.f;                  // ... plus sum_t adjS_t * (S0' adj-op_t)
#pragma unroll
        for (int m = 0; m < NT; ++m) {
            lds_fence();
            const uint4 a0 = tok_rows_op(oth_adj, 16 * m, 0, i, kg), a1 = tok_rows_op(oth_adj, 16 * m, 1, i, kg);
            floatx4 acc = Bf16::mfma32(a1, s0b, Bf16::mfma32(a0, s0a, zero));
            float af[4];
            unpack4<Bf16>(b_adj(m), af);
#pragma unroll
            for (int j = 0; j < 4; ++j) anchor_acc += af[j] * acc[j];
#pragma unroll
            for (int n0 = 0; n0 <= m; n0 += 2)
                acc = Bf16::mfma32(cat(*fw_tile(m, n0), n0 + 1 <= m ? *fw_tile(m, n0 + 1) : none),
                                   cat(b_val(n0), n0 + 1 <= m ? b_val(n0 + 1) : none), acc);
            if (side == 1) {
                const float4 dgv = *reinterpret_cast<const float4 *>(pd + 16 * m + 4 * kg);
                const float dg[4] = {dgv.x, dgv.y, dgv.z, dgv.w};
                float vf[4], dq[4];
                unpack4<Bf16>(b_val(m), vf);
#pragma unroll
                for (int j = 0; j < 4; ++j) dq[j] = lc.pre[m][j] * (acc[j] + vf[j] * dg[j]);
                store4(d_adj, m, dq);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) du[m][j] = af[j] * acc[j];
        }
        PT_MARK();
        // backward-like sweep: x' (value side) / k' (key side), token tile n
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            lds_fence();
            const uint4 v0 = tok_rows_op(oth_val, 16 * n, 0, i, kg), v1 = tok_rows_op(oth_val, 16 * n, 1, i, kg);
            floatx4 acc = Bf16::mfma32(v1, ghb, Bf16::mfma32(v0, gha, zero));
#pragma unroll
            for (int m0 = n; m0 < NT; m0 += 2)
                acc = Bf16::mfma32(cat(*bw_tile(n, m0), m0 + 1 < NT ? *bw_tile(n, m0 + 1) : none),
                                   cat(b_adj(m0), m0 + 1 < NT ? b_adj(m0 + 1) : none), acc);
            const float4 dgv = *reinterpret_cast<const float4 *>(pd + 16 * n + 4 * kg);
            const float dg[4] = {dgv.x, dgv.y, dgv.z, dgv.w};
            float af[4], vf[4], dv[4];
            unpack4<Bf16>(b_adj(n), af);
            unpack4<Bf16>(b_val(n), vf);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                dv[j] = inv[n][j] * (acc[j] + af[j] * dg[j]);
                du[n][j] -= vf[j] * acc[j];
            }
            store4(d_val, n, dv);
        }
        PT_MARK();
        if (side == 0 && next >= 0) issue_inputs<4>(next, cb);
        // gate gradient = (anchor - sum over the earlier tokens of du) / gate
        anchor += row_scan_add(anchor_acc, kg).all;
        float carry = 0.f;
#pragma unroll
        for (int m = 0; m < NT; ++m) {
            float e[4];
            e[0] = 0.f;
#pragma unroll
            for (int j = 1; j < 4; ++j) e[j] = e[j - 1] + du[m][j - 1];
            const RowScan sc = row_scan_add(e[3] + du[m][3], kg);
            const float base = anchor - (carry + sc.lower);
            carry += sc.all;
            float dgt[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float rgate = (j == 0 ? lc.off[m] : lc.pre[m][j > 0 ? j - 1 : 0]) * inv[m][j];      // 1 / gate
                dgt[j] = (base - e[j]) * rgate;
            }
            store4(d_gate, m, dgt);
        }
        // this wave's share of the next item's inputs has arrived in the staging area
        PT_MARK();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PT_MARK();
        __syncthreads();                         // staged inputs complete; this item's tiles are no longer read
    }

    __device__ __forceinline__ void run() const {
        const int n_items = (int)p.B * NC, stride = (int)gridDim.x;
        int item = (int)blockIdx.x;
        issue_inputs<8>(item, __builtin_amdgcn_readfirstlane(tid >> 6));
        GradsMats mats;
        issue_mats(mats, item);
#ifdef T2FW_PAR_TIMERS
        PT_DECL;
#else
        int pt_t = 0, pt_n = 0;
#endif
        PT_MARK();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        for (; item < n_items; item += stride) {
            const int next = item + stride < n_items ? item + stride : -1;
            if ((item % NC) * CL + CL <= T)
                body<true>(item, next, mats, pt_t, pt_n);
            else
                body<false>(item, next, mats, pt_t, pt_n);
        }
        PT_MARK();
        PT_FLUSH(p);
    }
};

template <typename IOE, int NT, bool HEADS>
__global__ __launch_bounds__(PAR_THREADS) void lfw_par_grads_kernel(ParBwdArgs p) {
    extern __shared__ __align__(16) unsigned char smem[];
    // waves 0-3: value side, 4-7: key side; both execute the same workgroup barriers
    if (threadIdx.x < PAR_THREADS / 2)
        GradsWave<IOE, NT, HEADS, 0>(p, smem).run();
    else
        GradsWave<IOE, NT, HEADS, 1>(p, smem).run();
}

template <typename IOE, int NT, bool HEADS> int launch(const ParBwdArgs &a, hipStream_t stream) {
    auto incr = lfw_par_incr_kernel<IOE, NT, HEADS>;
    auto scan = lfw_par_scan_kernel<IOE>;
    auto grads = lfw_par_grads_kernel<IOE, NT, HEADS>;
    int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(grads), hipFuncAttributeMaxDynamicSharedMemorySize, GR_SMEM),
                       "hipFuncSetAttribute(gradient kernel)");
    if (rc) return rc;
    const int64_t items = a.B * a.NC;
    if (items > 0x3fffffffLL || a.B > 0x0fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B * chunks = %lld is too large", (long long)items);
    if (a.heads < 1 || a.T * a.heads >= CHUNK_MAX_T || a.B * a.T * CH_N >= 0x7fffffffLL)
        return fail(T2FW_ERR_UNSUPPORTED, "B=%lld T=%lld with %d heads is too large for 32-bit element offsets", (long long)a.B, (long long)a.T, a.heads);
    hipLaunchKernelGGL(incr, dim3((unsigned)items), dim3(PAR_THREADS), INCR_SMEM, stream, a);
    if ((rc = check_hip(hipGetLastError(), "lfw_par_incr_kernel launch"))) return rc;
    hipLaunchKernelGGL(scan, dim3((unsigned)(8 * a.B)), dim3(SCAN_TPB), 0, stream, a);
    if ((rc = check_hip(hipGetLastError(), "lfw_par_scan_kernel launch"))) return rc;
    // persistent workgroups, one per compute unit (or one per item when there are fewer items)
    int dev = 0, cus = 0;
    if ((rc = check_hip(hipGetDevice(&dev), "hipGetDevice"))) return rc;
    if ((rc = check_hip(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev), "hipDeviceGetAttribute"))) return rc;
    hipLaunchKernelGGL(grads, dim3((unsigned)(items < cus ? items : cus)), dim3(PAR_THREADS), GR_SMEM, stream, a);
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
