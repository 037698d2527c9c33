// Device bodies of the exact per-step scan (one workgroup of SCAN_THREADS threads works on one
// batch row and one tile of state rows): used by the scan kernels of lfw_scan.hip and, for rows
// that the chunked matrix-core kernels cannot take, by those kernels themselves.
//
// Reference semantics: t2fw/torch.py:21-31 (forward), t2fw/csrc/lfw_kernel.cu:85-100
// and t2fw/csrc/lfw.cpp:84-93 (backward).
#pragma once

#include "common.hpp"
#include "lfw_scan.hpp"
#include "scan_tile.hpp"

namespace t2fw {
namespace scan {

// ------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------
// batch row b, tile of g.rows value channels.  KG: lanes per state row as a compile-time constant
// (p.kg must equal it), which leaves the cross-lane sums without branches and the LDS strides as
// immediates; 0 = take p.kg at run time.
template <typename IO, int KPL, int KG>
__device__ __forceinline__ void fwd_scan_body_kg(const ScanFwdArgs &p, int64_t b, int tile) {
    using Acc = typename AccOf<IO>::type;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const Tile g(KG > 0 ? KG : p.kg, KPL);
    const int tb = p.tb;
    Acc *colL = reinterpret_cast<Acc *>(smem_raw);        // [tb][3][KP]   k, f_key, q
    Acc *rowL = colL + (size_t)tb * 3 * g.KP;            // [tb][2][rows] x, f
    Acc *outL = rowL + (size_t)tb * 2 * g.rows;          // [tb][rows]

    const int64_t T = p.T, D = p.D, K = p.K;
    const int64_t col0 = p.col0, KW = p.colw > 0 ? p.colw : K;      // this pass's window of key channels
    const bool accumulate = p.accumulate != 0;
    const int64_t line0 = row_first_token(b, T, p.heads);      // [.., D] line of this row's step 0
    const int64_t d0 = (int64_t)tile * g.rows;
    const int64_t d = d0 + g.r;
    const bool row_ok = d < D;

    const IO *const colp[3] = {(const IO *)p.k, (const IO *)p.f_key, (const IO *)p.q};
    const IO *const rowp[2] = {(const IO *)p.x, (const IO *)p.f};
    const IO *s0 = (const IO *)p.s0;
    IO *out = (IO *)p.out, *next_state = (IO *)p.next_state, *ckpt = (IO *)p.ckpt;

    Acc S[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j)
        S[j] = (row_ok && g.k0 + j < KW) ? to_acc(s0[(b * D + d) * K + col0 + g.k0 + j]) : Acc(0);

    // outputs of a block of steps: written, or added to what the passes over other key channels left
    auto flush = [&](int n_blk, int64_t t_blk) {
        for (int idx = threadIdx.x; idx < n_blk * g.rows; idx += SCAN_THREADS) {
            const int tt = idx / g.rows, rr = idx % g.rows;
            if (d0 + rr < D) {
                IO *const o = out + (line0 + (t_blk + tt) * p.heads) * D + d0 + rr;
                *o = from_acc<IO>(accumulate ? to_acc(*o) + outL[idx] : outL[idx]);
            }
        }
    };

    Prefetch<IO, 3, 2> pf;
    block_load(pf, g, colp, rowp, b, T, 0, (int)(T < tb ? T : tb), K, D, d0, p.heads, col0, p.colw);

    int until_ckpt = 0;          // steps until the next checkpoint is due
    int64_t chunk = 0;
    int n_prev = 0;
    int64_t t_prev = 0;
    for (int64_t t0 = 0; t0 < T; t0 += tb) {
        const int n = (int)(T - t0 < tb ? T - t0 : tb);
        __syncthreads();                                   // previous block fully consumed
        // flush the previous block's outputs, then publish this block's inputs
        flush(n_prev, t_prev);
        block_store<IO, Acc, 3, 2>(pf, g, colL, rowL, tb);
        __syncthreads();
        if (t0 + tb < T) {
            const int64_t tn = t0 + tb;
            block_load(pf, g, colp, rowp, b, T, tn, (int)(T - tn < tb ? T - tn : tb), K, D, d0, p.heads, col0, p.colw);
        }
#pragma unroll 4
        for (int tt = 0; tt < n; ++tt) {
            if (ckpt != nullptr) {
                if (until_ckpt == 0) {
                    if (row_ok) {
#pragma unroll
                        for (int j = 0; j < KPL; ++j)
                            if (g.k0 + j < KW)
                                ckpt[((b * p.NC + chunk) * D + d) * K + col0 + g.k0 + j] = from_acc<IO>(S[j]);
                    }
                    until_ckpt = p.C;
                    ++chunk;
                }
                --until_ckpt;
            }
            const Acc xd = rowL[(tt * 2 + 0) * g.rows + g.r];
            const Acc fd = rowL[(tt * 2 + 1) * g.rows + g.r];
            const Acc *ck = colL + (tt * 3 + 0) * g.KP + g.k0;
            const Acc *cf = colL + (tt * 3 + 1) * g.KP + g.k0;
            const Acc *cq = colL + (tt * 3 + 2) * g.KP + g.k0;
            Acc acc = 0;
#pragma unroll
            for (int j = 0; j < KPL; ++j) {
                S[j] = S[j] * (fd * cf[j]) + xd * ck[j];
                acc += S[j] * cq[j];
            }
            acc = group_sum(acc, g.kg);
            if (g.kgi == 0) outL[tt * g.rows + g.r] = acc;
        }
        n_prev = n;
        t_prev = t0;
    }
    __syncthreads();
    flush(n_prev, t_prev);
    if (row_ok) {
#pragma unroll
        for (int j = 0; j < KPL; ++j)
            if (g.k0 + j < KW) next_state[(b * D + d) * K + col0 + g.k0 + j] = from_acc<IO>(S[j]);
    }
}

// The common geometry (16 lanes per state row: 16 to 64 columns) runs with constant strides.
template <typename IO, int KPL>
__device__ __forceinline__ void fwd_scan_body(const ScanFwdArgs &p, int64_t b, int tile) {
    if constexpr (KPL <= 4) {          // wider rows are spread over more than 16 lanes
        if (p.kg == 16) {
            fwd_scan_body_kg<IO, KPL, 16>(p, b, tile);
            return;
        }
    }
    fwd_scan_body_kg<IO, KPL, 0>(p, b, tile);
}

// ------------------------------------------------------------------------------------
// backward, one side.  "rows" are the dimension this launch keeps per lane-group,
// "cols" the dimension it reduces over:
//   side 0: rows = D, cols = K : a_r = x,  gate_r = f,     u_r = g_out ; a_c = k, gate_c = f_key, u_c = q
//           outputs d_a = d_x, d_gate = d_f, plus d_s0
//   side 1: rows = K, cols = D : a_r = k,  gate_r = f_key, u_r = q     ; a_c = x, gate_c = f,     u_c = g_out
//           outputs d_a = d_k, d_gate = d_f_key, d_u = d_q
// State element (row, col) lives at [b, row, col] (side 0) or [b, col, row] (side 1).
//
// Per chunk: the states at segment starts are recomputed from the checkpoint and kept
// in LDS (lane-private slots); then segments are visited last to first, each segment's
// SEG states are recomputed into registers and the adjoint runs backwards over them.
// ------------------------------------------------------------------------------------
template <int KPL> struct SegLen { static constexpr int value = (32 / KPL) < 1 ? 1 : (KPL <= 4 ? 8 : 32 / KPL); };

// KG as for the forward body; SUB: 1 / 0 = p.use_sub is known to be set / clear, -1 = read it.
template <typename IO, int KPL, int SIDE, int KG, int SUB = -1>
__device__ __forceinline__ void bwd_scan_body_kg(const ScanBwdArgs &p, int64_t b, int tile) {
    using Acc = typename AccOf<IO>::type;
    constexpr int SEG = SegLen<KPL>::value;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const Tile g(KG > 0 ? KG : p.kg, KPL);
    Acc *colL = reinterpret_cast<Acc *>(smem_raw);        // [SEG][3][KP]   a_c, gate_c, u_c
    Acc *rowL = colL + (size_t)SEG * 3 * g.KP;           // [SEG][3][rows] a_r, gate_r, u_r
    Acc *outL = rowL + (size_t)SEG * 3 * g.rows;         // [SEG][3][rows] d_a, d_gate, d_u
    Acc *subL = outL + (size_t)SEG * 3 * g.rows;         // [nseg_max][KPL][SCAN_THREADS]

    const int64_t T = p.T;
    const int64_t line0 = row_first_token(b, T, p.heads);      // [.., D|K] line of this row's step 0
    const int64_t nrows = SIDE == 0 ? p.D : p.K, ncols = SIDE == 0 ? p.K : p.D;
    const int64_t col0 = p.col0, colw = p.colw > 0 ? p.colw : ncols;      // this pass's window of the reduced channels
    const bool accumulate = p.accumulate != 0;
    const int64_t row0 = (int64_t)tile * g.rows;
    const int64_t row = row0 + g.r;
    const bool row_ok = row < nrows;
    const int64_t DK = p.D * p.K;

    const IO *const colp[3] = {(const IO *)(SIDE == 0 ? p.k : p.x), (const IO *)(SIDE == 0 ? p.f_key : p.f),
                               (const IO *)(SIDE == 0 ? p.q : p.g_out)};
    const IO *const rowp[3] = {(const IO *)(SIDE == 0 ? p.x : p.k), (const IO *)(SIDE == 0 ? p.f : p.f_key),
                               (const IO *)(SIDE == 0 ? p.g_out : p.q)};
    IO *d_a = (IO *)(SIDE == 0 ? p.d_x : p.d_k);
    IO *d_gate = (IO *)(SIDE == 0 ? p.d_f : p.d_f_key);
    IO *d_u = (IO *)p.d_q;   // side 1 only
    const IO *ckpt = (const IO *)p.ckpt;

    // element offset of (row, col0 + j) inside one [D,K] state
    auto st_off = [&](int j) -> int64_t {
        return SIDE == 0 ? row * p.K + (col0 + g.k0 + j) : (col0 + g.k0 + j) * p.K + row;
    };
    auto el_ok = [&](int j) -> bool { return row_ok && g.k0 + j < colw; };

    Acc G[KPL];
    {
        const IO *gs = (const IO *)p.g_state + b * DK;
#pragma unroll
        for (int j = 0; j < KPL; ++j) G[j] = el_ok(j) ? to_acc(gs[st_off(j)]) : Acc(0);
    }

    const int C = p.C;
    const bool use_sub = SUB < 0 ? p.use_sub != 0 : SUB != 0;
    Prefetch<IO, 3, 3> pf;

    auto load_ckpt = [&](Acc (&S)[KPL], int64_t c) {
        const IO *ck = ckpt + (b * p.NC + c) * DK;
#pragma unroll
        for (int j = 0; j < KPL; ++j) S[j] = el_ok(j) ? to_acc(ck[st_off(j)]) : Acc(0);
    };
    // prefetched inputs -> LDS, between two barriers (the LDS of the step before is no longer read)
    auto stage = [&]() {
        __syncthreads();
        block_store<IO, Acc, 3, 3, SEG>(pf, g, colL, rowL, SEG);
        __syncthreads();
    };
    // S over the SEG staged steps
    auto advance = [&](Acc (&S)[KPL]) {
#pragma unroll
        for (int tt = 0; tt < SEG; ++tt) {
            const Acc ar = rowL[(tt * 3 + 0) * g.rows + g.r];
            const Acc fr = rowL[(tt * 3 + 1) * g.rows + g.r];
            const Acc *ca = colL + (tt * 3 + 0) * g.KP + g.k0;
            const Acc *cf = colL + (tt * 3 + 1) * g.KP + g.k0;
#pragma unroll
            for (int j = 0; j < KPL; ++j) S[j] = S[j] * (fr * cf[j]) + ar * ca[j];
        }
    };
    // The staged segment [t0, t0 + n): its states recomputed into registers from st[0], the adjoint
    // backwards over them, the outputs written.
    auto reverse_segment = [&](Acc (&st)[SEG + 1][KPL], int n, int64_t t0) {
#pragma unroll
        for (int tt = 0; tt < SEG; ++tt) {
            const Acc ar = rowL[(tt * 3 + 0) * g.rows + g.r];
            const Acc fr = rowL[(tt * 3 + 1) * g.rows + g.r];
            const Acc *ca = colL + (tt * 3 + 0) * g.KP + g.k0;
            const Acc *cf = colL + (tt * 3 + 1) * g.KP + g.k0;
#pragma unroll
            for (int j = 0; j < KPL; ++j) st[tt + 1][j] = st[tt][j] * (fr * cf[j]) + ar * ca[j];
        }
        // adjoint, last step of the segment first
#pragma unroll
        for (int tt = SEG - 1; tt >= 0; --tt) {
            if (tt < n) {
                const Acc fr = rowL[(tt * 3 + 1) * g.rows + g.r];
                const Acc ur = rowL[(tt * 3 + 2) * g.rows + g.r];
                const Acc *ca = colL + (tt * 3 + 0) * g.KP + g.k0;
                const Acc *cf = colL + (tt * 3 + 1) * g.KP + g.k0;
                const Acc *cu = colL + (tt * 3 + 2) * g.KP + g.k0;
                Acc sa = 0, sg = 0, su = 0;
#pragma unroll
                for (int j = 0; j < KPL; ++j) {
                    G[j] += ur * cu[j];                       // G_t = g_t (x) q_t + ...
                    sa += G[j] * ca[j];                       // d_x / d_k
                    sg += (G[j] * st[tt][j]) * cf[j];         // d_f / d_f_key   (uses S_{t-1})
                    if (SIDE == 1) su += st[tt + 1][j] * cu[j];   // d_q = S_t^T g_t
                    G[j] *= fr * cf[j];
                }
                sa = group_sum(sa, g.kg);
                sg = group_sum(sg, g.kg);
                if (SIDE == 1) su = group_sum(su, g.kg);
                if (g.kgi == 0) {
                    outL[(tt * 3 + 0) * g.rows + g.r] = sa;
                    outL[(tt * 3 + 1) * g.rows + g.r] = sg;
                    if (SIDE == 1) outL[(tt * 3 + 2) * g.rows + g.r] = su;
                }
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n * g.rows; idx += SCAN_THREADS) {
            const int tt = idx / g.rows, rr = idx % g.rows;
            if (row0 + rr < nrows) {
                const int64_t o = (line0 + (t0 + tt) * p.heads) * nrows + row0 + rr;
                Acc va = outL[(tt * 3 + 0) * g.rows + rr], vg = outL[(tt * 3 + 1) * g.rows + rr];
                Acc vu = SIDE == 1 ? outL[(tt * 3 + 2) * g.rows + rr] : Acc(0);
                if (accumulate) {            // the passes over other reduced channels came first
                    va += to_acc(d_a[o]);
                    vg += to_acc(d_gate[o]);
                    if (SIDE == 1) vu += to_acc(d_u[o]);
                }
                d_a[o] = from_acc<IO>(va);
                d_gate[o] = from_acc<IO>(vg);
                if (SIDE == 1) d_u[o] = from_acc<IO>(vu);
            }
        }
    };
    auto chunk_len = [&](int64_t c) -> int { return (int)(T - c * C < C ? T - c * C : C); };

    if (use_sub) {
        // A chunk with nseg segments is 2 * nseg - 1 staged jobs: nseg - 1 that advance S to the
        // segment starts (kept in subL), then the segments last to first.  The global loads of a
        // job are issued while the job before it computes.
        auto issue = [&](int64_t c, int q) {
            const int len = chunk_len(c), nseg = (len + SEG - 1) / SEG;
            const int sg = q < nseg - 1 ? q : 2 * nseg - 2 - q;
            const int n = q < nseg - 1 ? SEG : (len - sg * SEG < SEG ? len - sg * SEG : SEG);
            block_load<SEG>(pf, g, colp, rowp, b, T, c * C + (int64_t)sg * SEG, n, ncols, nrows, row0, p.heads, col0, p.colw);
        };
        Acc Snext[KPL];                      // checkpoint of the chunk that comes next
        load_ckpt(Snext, p.NC - 1);
        issue(p.NC - 1, 0);
        for (int64_t c = p.NC - 1; c >= 0; --c) {
            const int64_t tc0 = c * C;
            const int len = chunk_len(c), nseg = (len + SEG - 1) / SEG, njobs = 2 * nseg - 1;
            Acc S[KPL];
#pragma unroll
            for (int j = 0; j < KPL; ++j) S[j] = Snext[j];
            if (c > 0) load_ckpt(Snext, c - 1);
#pragma unroll
            for (int j = 0; j < KPL; ++j) subL[(size_t)j * SCAN_THREADS + threadIdx.x] = S[j];
            for (int q = 0; q < njobs; ++q) {
                stage();
                if (q + 1 < njobs)
                    issue(c, q + 1);
                else if (c > 0)
                    issue(c - 1, 0);
                if (q < nseg - 1) {
                    advance(S);
#pragma unroll
                    for (int j = 0; j < KPL; ++j) subL[((size_t)(q + 1) * KPL + j) * SCAN_THREADS + threadIdx.x] = S[j];
                } else {
                    const int sg = 2 * nseg - 2 - q;
                    Acc st[SEG + 1][KPL];
#pragma unroll
                    for (int j = 0; j < KPL; ++j) st[0][j] = subL[((size_t)sg * KPL + j) * SCAN_THREADS + threadIdx.x];
                    reverse_segment(st, len - sg * SEG < SEG ? len - sg * SEG : SEG, tc0 + (int64_t)sg * SEG);
                }
            }
        }
    } else {
        // no room for the segment-start states: every segment is replayed from the checkpoint
        for (int64_t c = p.NC - 1; c >= 0; --c) {
            const int64_t tc0 = c * C;
            const int len = chunk_len(c), nseg = (len + SEG - 1) / SEG;
            for (int s = nseg - 1; s >= 0; --s) {
                Acc st[SEG + 1][KPL];
                load_ckpt(st[0], c);
                for (int s2 = 0; s2 < s; ++s2) {
                    block_load<SEG>(pf, g, colp, rowp, b, T, tc0 + (int64_t)s2 * SEG, SEG, ncols, nrows, row0, p.heads, col0, p.colw);
                    stage();
                    advance(st[0]);
                }
                const int n = len - s * SEG < SEG ? len - s * SEG : SEG;
                block_load<SEG>(pf, g, colp, rowp, b, T, tc0 + (int64_t)s * SEG, n, ncols, nrows, row0, p.heads, col0, p.colw);
                stage();
                reverse_segment(st, n, tc0 + (int64_t)s * SEG);
            }
        }
    }
    if (SIDE == 0) {
        IO *ds = (IO *)p.d_s0 + b * DK;
#pragma unroll
        for (int j = 0; j < KPL; ++j)
            if (el_ok(j)) ds[st_off(j)] = from_acc<IO>(G[j]);
    }
}

}  // namespace scan
}  // namespace t2fw
