// Delta-rule ("DFW") recurrence kernels: any D, M, dtype.
//
//   out_t = S_{t-1} q_t ;  delta_t = v_t - S_{t-1} k_t ;  S_t = S_{t-1} + delta_t (x) k_t
// (t2fw/torch.py:44-53; note the output uses the state BEFORE the update, unlike the decay
// rule).  Backward, with G = dL/dS flowing backwards (t2fw/torch.py:82-143,
// t2fw/csrc/dfw_kernel.cu:250-276,345-383):
//   dv_t = G_t k_t ;  G_{t-1} = G_t - dv_t (x) k_t + g_t (x) q_t ;  d_state = G_{-1}
//   S_{t-1} = S_t - delta_t (x) k_t ;  dq_t = S_{t-1}^T g_t ;  dk_t = G_t^T delta_t - S_{t-1}^T dv_t
//
// One lane owns KPL adjacent elements of one state row, KG lanes share a row and reduce
// with DPP (replacing the reference's shared-memory sumReduc, dfw_kernel.cu:58-100); the
// state stays in registers for the whole sequence and inputs are staged through LDS one time
// block ahead.  The backward pass is two launches: rows along D give d_v and d_state, rows
// along M give d_q and d_k (and consume d_v), so every reduction is along the lane-shared row.
#include <type_traits>

#include "common.hpp"
#include "dfw_scan.hpp"
#include "scan_tile.hpp"

namespace t2fw {
namespace {

using namespace scan;

// ---- forward: rows = D, columns = M ------------------------------------------------------
template <typename IO, int KPL>
__global__ __launch_bounds__(SCAN_THREADS) void dfw_fwd_kernel(DfwFwdArgs p) {
    using Acc = typename AccOf<IO>::type;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const Tile g(p.kg, KPL);
    const int tb = p.tb;
    Acc *colL = reinterpret_cast<Acc *>(smem_raw);        // [tb][2][KP]   k, q
    Acc *rowL = colL + (size_t)tb * 2 * g.KP;            // [tb][1][rows] v
    Acc *outL = rowL + (size_t)tb * g.rows;              // [tb][2][rows] out, delta
    const int64_t b = blockIdx.x / p.ntiles;
    const int64_t T = p.T, D = p.D, M = p.M;
    const int64_t d0 = (int64_t)(blockIdx.x % p.ntiles) * g.rows;
    const int64_t d = d0 + g.r;
    const bool row_ok = d < D;
    const IO *const colp[2] = {(const IO *)p.k, (const IO *)p.q};
    const IO *const rowp[1] = {(const IO *)p.v};
    IO *out = (IO *)p.out, *delta = (IO *)p.delta;

    Acc S[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j)
        S[j] = (row_ok && g.k0 + j < M) ? to_acc(((const IO *)p.s0)[(b * D + d) * M + g.k0 + j]) : Acc(0);

    Prefetch<IO, 2, 1> pf;
    block_load(pf, g, colp, rowp, b, T, 0, (int)(T < tb ? T : tb), M, D, d0);
    int n_prev = 0;
    int64_t t_prev = 0;
    auto flush = [&]() {
        for (int idx = threadIdx.x; idx < n_prev * g.rows; idx += SCAN_THREADS) {
            const int tt = idx / g.rows, rr = idx % g.rows;
            if (d0 + rr < D) {
                const int64_t o = (b * T + t_prev + tt) * D + d0 + rr;
                out[o] = from_acc<IO>(outL[(tt * 2 + 0) * g.rows + rr]);
                delta[o] = from_acc<IO>(outL[(tt * 2 + 1) * g.rows + rr]);
            }
        }
    };
    // The steps of one staged block.  kgv: lanes per state row, as a compile-time constant for the
    // common geometry (which leaves the cross-lane sums without branches and the LDS strides as
    // immediates) or as a run-time value.
    auto steps = [&](int n, auto kgv) {
        const int kg = kgv, rows = SCAN_THREADS / kg, KP = kg * KPL;
#pragma unroll 4
        for (int tt = 0; tt < n; ++tt) {
            const Acc vd = rowL[tt * rows + g.r];
            const Acc *ck = colL + (tt * 2 + 0) * KP + g.k0;
            const Acc *cq = colL + (tt * 2 + 1) * KP + g.k0;
            Acc so = 0, sq = 0;
#pragma unroll
            for (int j = 0; j < KPL; ++j) {
                so += S[j] * ck[j];       // old = S k
                sq += S[j] * cq[j];       // out = S q (state before the update)
            }
            so = group_sum(so, kg);
            sq = group_sum(sq, kg);
            const Acc dl = vd - so;
#pragma unroll
            for (int j = 0; j < KPL; ++j) S[j] += dl * ck[j];
            if (g.kgi == 0) {
                outL[(tt * 2 + 0) * rows + g.r] = sq;
                outL[(tt * 2 + 1) * rows + g.r] = dl;
            }
        }
    };
    for (int64_t t0 = 0; t0 < T; t0 += tb) {
        const int n = (int)(T - t0 < tb ? T - t0 : tb);
        __syncthreads();
        flush();
        block_store<IO, Acc, 2, 1>(pf, g, colL, rowL, tb);
        __syncthreads();
        if (t0 + tb < T) {
            const int64_t tn = t0 + tb;
            block_load(pf, g, colp, rowp, b, T, tn, (int)(T - tn < tb ? T - tn : tb), M, D, d0);
        }
        if (g.kg == 16)
            steps(n, std::integral_constant<int, 16>{});
        else
            steps(n, g.kg);
        n_prev = n;
        t_prev = t0;
    }
    __syncthreads();
    flush();
    if (row_ok) {
#pragma unroll
        for (int j = 0; j < KPL; ++j)
            if (g.k0 + j < M) ((IO *)p.final_state)[(b * D + d) * M + g.k0 + j] = from_acc<IO>(S[j]);
    }
}

// ---- backward ----------------------------------------------------------------------------
// SIDE 0: rows = D, cols = M.  row input g_out; col inputs k, q.       Outputs d_v (per row), d_s0.
// SIDE 1: rows = M, cols = D.  row inputs k, q; col inputs delta, g_out, d_v.  Outputs d_k, d_q.
// Time runs backwards; blocks of tb steps are staged in reverse order.
template <typename IO, int KPL, int SIDE>
__global__ __launch_bounds__(SCAN_THREADS) void dfw_bwd_kernel(DfwBwdArgs p) {
    using Acc = typename AccOf<IO>::type;
    constexpr int NCA = SIDE == 0 ? 2 : 3, NRA = SIDE == 0 ? 1 : 2, NOUT = SIDE == 0 ? 1 : 2;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const Tile g(p.kg, KPL);
    const int tb = p.tb;
    Acc *colL = reinterpret_cast<Acc *>(smem_raw);              // [tb][NCA][KP]
    Acc *rowL = colL + (size_t)tb * NCA * g.KP;                // [tb][NRA][rows]
    Acc *outL = rowL + (size_t)tb * NRA * g.rows;              // [tb][NOUT][rows]
    const int64_t b = blockIdx.x / p.ntiles;
    const int64_t T = p.T;
    const int64_t nrows = SIDE == 0 ? p.D : p.M, ncols = SIDE == 0 ? p.M : p.D;
    const int64_t row0 = (int64_t)(blockIdx.x % p.ntiles) * g.rows;
    const int64_t row = row0 + g.r;
    const bool row_ok = row < nrows;
    const int64_t DM = p.D * p.M;

    const IO *colp[NCA];
    const IO *rowp[NRA];
    if (SIDE == 0) {
        colp[0] = (const IO *)p.k; colp[1] = (const IO *)p.q;
        rowp[0] = (const IO *)p.g_out;
    } else {
        colp[0] = (const IO *)p.delta; colp[1] = (const IO *)p.g_out; colp[NCA - 1] = (const IO *)p.d_v;
        rowp[0] = (const IO *)p.k; rowp[NRA - 1] = (const IO *)p.q;
    }
    const IO *const(&colr)[NCA] = reinterpret_cast<const IO *const(&)[NCA]>(colp);
    const IO *const(&rowr)[NRA] = reinterpret_cast<const IO *const(&)[NRA]>(rowp);
    IO *o0 = (IO *)(SIDE == 0 ? p.d_v : p.d_k);
    IO *o1 = (IO *)p.d_q;

    auto st_off = [&](int j) -> int64_t {   // element (row, col0 + j) of a [D, M] state
        return SIDE == 0 ? row * p.M + (g.k0 + j) : (int64_t)(g.k0 + j) * p.M + row;
    };
    auto el_ok = [&](int j) -> bool { return row_ok && g.k0 + j < ncols; };

    Acc G[KPL], S[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j) {
        G[j] = el_ok(j) ? to_acc(((const IO *)p.g_state)[b * DM + st_off(j)]) : Acc(0);
        S[j] = (SIDE == 1 && el_ok(j)) ? to_acc(((const IO *)p.final_state)[b * DM + st_off(j)]) : Acc(0);
    }

    const int64_t nblk = (T + tb - 1) / tb;
    Prefetch<IO, NCA, NRA> pf;
    {
        const int64_t t0 = (nblk - 1) * tb;
        block_load(pf, g, colr, rowr, b, T, t0, (int)(T - t0), ncols, nrows, row0);
    }
    int n_prev = 0;
    int64_t t_prev = 0;
    auto flush = [&]() {
        for (int idx = threadIdx.x; idx < n_prev * g.rows; idx += SCAN_THREADS) {
            const int tt = idx / g.rows, rr = idx % g.rows;
            if (row0 + rr < nrows) {
                const int64_t o = (b * T + t_prev + tt) * nrows + row0 + rr;
                o0[o] = from_acc<IO>(outL[(tt * NOUT + 0) * g.rows + rr]);
                if (SIDE == 1) o1[o] = from_acc<IO>(outL[(tt * NOUT + NOUT - 1) * g.rows + rr]);
            }
        }
    };
    // The steps of one staged block, last to first; kgv as in the forward kernel.
    auto steps = [&](int n, auto kgv) {
        const int kg = kgv, rows = SCAN_THREADS / kg, KP = kg * KPL;
#pragma unroll 4
        for (int tt = n - 1; tt >= 0; --tt) {
            if (SIDE == 0) {
                const Acc gr = rowL[tt * rows + g.r];
                const Acc *ck = colL + (tt * 2 + 0) * KP + g.k0;
                const Acc *cq = colL + (tt * 2 + 1) * KP + g.k0;
                Acc dv = 0;
#pragma unroll
                for (int j = 0; j < KPL; ++j) dv += G[j] * ck[j];          // dv_t = G_t k_t
                dv = group_sum(dv, kg);
#pragma unroll
                for (int j = 0; j < KPL; ++j) G[j] += gr * cq[j] - dv * ck[j];
                if (g.kgi == 0) outL[tt * rows + g.r] = dv;
            } else {
                const Acc kr = rowL[(tt * 2 + 0) * rows + g.r];
                const Acc qr = rowL[(tt * 2 + 1) * rows + g.r];
                const Acc *cd = colL + (tt * 3 + 0) * KP + g.k0;   // delta
                const Acc *cg = colL + (tt * 3 + 1) * KP + g.k0;   // g_out
                const Acc *cv = colL + (tt * 3 + 2) * KP + g.k0;   // d_v
                Acc sk = 0, sq = 0;
#pragma unroll
                for (int j = 0; j < KPL; ++j) {
                    S[j] -= cd[j] * kr;                               // S_{t-1}
                    sq += S[j] * cg[j];                               // dq = S_{t-1}^T g
                    sk += G[j] * cd[j] - S[j] * cv[j];                // dk = G_t^T delta - S_{t-1}^T dv
                    G[j] += cg[j] * qr - cv[j] * kr;
                }
                sk = group_sum(sk, kg);
                sq = group_sum(sq, kg);
                if (g.kgi == 0) {
                    outL[(tt * 2 + 0) * rows + g.r] = sk;
                    outL[(tt * 2 + 1) * rows + g.r] = sq;
                }
            }
        }
    };
    for (int64_t blk = nblk - 1; blk >= 0; --blk) {
        const int64_t t0 = blk * tb;
        const int n = (int)(T - t0 < tb ? T - t0 : tb);
        __syncthreads();
        flush();
        block_store<IO, Acc, NCA, NRA>(pf, g, colL, rowL, tb);
        __syncthreads();
        if (blk > 0) block_load(pf, g, colr, rowr, b, T, t0 - tb, tb, ncols, nrows, row0);
        if (g.kg == 16)
            steps(n, std::integral_constant<int, 16>{});
        else
            steps(n, g.kg);
        n_prev = n;
        t_prev = t0;
    }
    __syncthreads();
    flush();
    if (SIDE == 0) {
#pragma unroll
        for (int j = 0; j < KPL; ++j)
            if (el_ok(j)) ((IO *)p.d_s0)[b * DM + st_off(j)] = from_acc<IO>(G[j]);
    }
}

// ---- host dispatch -----------------------------------------------------------------------
int block_steps(const ScanGeom &g) {
    int tb = 32;
    const int by_cols = PFC * SCAN_THREADS / (g.kg * g.kpl);
    const int by_rows = PFR * SCAN_THREADS / g.rows;
    if (by_cols < tb) tb = by_cols;
    if (by_rows < tb) tb = by_rows;
    return tb < 1 ? 1 : tb;
}

template <typename IO, int KPL> int launch_fwd(DfwFwdArgs a, const ScanGeom &g, hipStream_t stream) {
    using Acc = typename AccOf<IO>::type;
    a.kg = g.kg;
    a.tb = block_steps(g);
    a.ntiles = (int)((a.D + g.rows - 1) / g.rows);
    const size_t smem = ((size_t)a.tb * 2 * g.kg * g.kpl + (size_t)a.tb * 3 * g.rows) * sizeof(Acc);
    const int64_t nblocks = a.B * a.ntiles;
    if (nblocks > 0x7fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "grid of %lld workgroups is too large", (long long)nblocks);
    hipLaunchKernelGGL((dfw_fwd_kernel<IO, KPL>), dim3((unsigned)nblocks), dim3(SCAN_THREADS), smem, stream, a);
    return check_hip(hipGetLastError(), "dfw_fwd_kernel launch");
}

template <typename IO, int KPL, int SIDE> int launch_bwd(DfwBwdArgs a, const ScanGeom &g, hipStream_t stream) {
    using Acc = typename AccOf<IO>::type;
    constexpr int NCA = SIDE == 0 ? 2 : 3, NRA = SIDE == 0 ? 1 : 2, NOUT = SIDE == 0 ? 1 : 2;
    const int64_t nrows = SIDE == 0 ? a.D : a.M;
    a.kg = g.kg;
    a.tb = block_steps(g);
    a.ntiles = (int)((nrows + g.rows - 1) / g.rows);
    const size_t smem = ((size_t)a.tb * NCA * g.kg * g.kpl + (size_t)a.tb * (NRA + NOUT) * g.rows) * sizeof(Acc);
    const int64_t nblocks = a.B * a.ntiles;
    if (nblocks > 0x7fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "grid of %lld workgroups is too large", (long long)nblocks);
    hipLaunchKernelGGL((dfw_bwd_kernel<IO, KPL, SIDE>), dim3((unsigned)nblocks), dim3(SCAN_THREADS), smem, stream, a);
    return check_hip(hipGetLastError(), "dfw_bwd_kernel launch");
}

#define T2FW_KPL_SWITCH(kpl, CALL)                                               \
    switch (kpl) {                                                               \
        case 1: return CALL(1);                                                  \
        case 2: return CALL(2);                                                  \
        case 4: return CALL(4);                                                  \
        case 8: return CALL(8);                                                  \
        case 16: return CALL(16);                                                \
        case 32: return CALL(32);                                                \
    }                                                                            \
    return fail(T2FW_ERR_UNSUPPORTED, "unsupported columns-per-lane %d", kpl)

template <typename IO> int fwd_t(const DfwFwdArgs &a, hipStream_t stream) {
    if (a.M > SCAN_MAX_COLS) return fail(T2FW_ERR_UNSUPPORTED, "M=%lld exceeds the supported maximum %d", (long long)a.M, SCAN_MAX_COLS);
    const ScanGeom g = scan_geometry(a.M);
#define CALL(N) launch_fwd<IO, N>(a, g, stream)
    T2FW_KPL_SWITCH(g.kpl, CALL);
#undef CALL
}

template <typename IO, int SIDE> int bwd_side(const DfwBwdArgs &a, hipStream_t stream) {
    const int64_t ncols = SIDE == 0 ? a.M : a.D;
    if (ncols > SCAN_MAX_COLS)
        return fail(T2FW_ERR_UNSUPPORTED, "%s=%lld exceeds the supported maximum %d", SIDE == 0 ? "M" : "D", (long long)ncols, SCAN_MAX_COLS);
    const ScanGeom g = scan_geometry(ncols);
#define CALL(N) launch_bwd<IO, N, SIDE>(a, g, stream)
    T2FW_KPL_SWITCH(g.kpl, CALL);
#undef CALL
}

template <typename IO> int bwd_t(const DfwBwdArgs &a, hipStream_t stream) {
    int rc = bwd_side<IO, 0>(a, stream);      // d_v, d_s0
    if (rc != T2FW_OK) return rc;
    return bwd_side<IO, 1>(a, stream);        // d_k, d_q (reads d_v)
}

}  // namespace

int dfw_forward(const DfwFwdArgs &a, int dtype, hipStream_t stream) {
    switch (dtype) {
        case T2FW_F32: return fwd_t<float>(a, stream);
        case T2FW_F16: return fwd_t<__half>(a, stream);
        case T2FW_BF16: return fwd_t<__hip_bfloat16>(a, stream);
        case T2FW_F64: return fwd_t<double>(a, stream);
    }
    return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
}

int dfw_backward(const DfwBwdArgs &a, int dtype, hipStream_t stream) {
    switch (dtype) {
        case T2FW_F32: return bwd_t<float>(a, stream);
        case T2FW_F16: return bwd_t<__half>(a, stream);
        case T2FW_BF16: return bwd_t<__hip_bfloat16>(a, stream);
        case T2FW_F64: return bwd_t<double>(a, stream);
    }
    return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
}

}  // namespace t2fw
