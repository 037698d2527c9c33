// Device-side staging helpers shared by the exact scan kernels (lfw_scan.hip, dfw_scan.hip):
// per-workgroup tile geometry, register prefetch of one time block of inputs, LDS layout.
#pragma once

#include "common.hpp"

namespace t2fw {
namespace scan {

constexpr int PFC = 8;   // prefetch slots per thread per column-side array
constexpr int PFR = 4;   // prefetch slots per thread per row-side array

__device__ __forceinline__ int ilog2(int v) { return 31 - __clz(v); }

// Geometry derived on the device from (kg, kpl): all powers of two.
struct Tile {
    int kg, rows, KP;        // lanes per row, rows per workgroup, padded columns
    int CW, SP, lncc;        // column staging: lanes across columns, steps per pass, log2(KP/CW)
    int SPR;                 // row staging: steps per pass
    int r, kgi, k0;          // this lane's row, position in the row, first column
    __device__ Tile(int kg_, int kpl) {
        kg = kg_;
        rows = SCAN_THREADS / kg;
        KP = kg * kpl;
        CW = KP < SCAN_THREADS ? KP : SCAN_THREADS;
        SP = SCAN_THREADS / CW;
        lncc = ilog2(KP / CW);
        SPR = SCAN_THREADS / rows;
        r = threadIdx.x / kg;
        kgi = threadIdx.x % kg;
        k0 = kgi * kpl;
    }
};

// Prefetch registers for one time block: NCA column-side and NRA row-side arrays.
template <typename IO, int NCA, int NRA> struct Prefetch {
    IO c[NCA][PFC];
    IO r[NRA][PFR];
};

// Issue the global loads of a block of n steps starting at step t0 of batch row b.
// colp[a] are [B,T,ncols] arrays, rowp[a] are [B,T,nrows] arrays (heads = 1), or
// [B/heads,T,heads,ncols] and [B/heads,T,heads,nrows] with row b = (batch, head); this
// workgroup needs all columns and rows [row0, row0 + rows).
// TMAX: an upper bound of n known at compile time; slots that can only hold later steps are
// skipped (which removes their loads when the geometry is a compile-time constant too).
template <int TMAX = 1 << 30, typename IO, int NCA, int NRA>
__device__ __forceinline__ void block_load(Prefetch<IO, NCA, NRA> &pf, const Tile &g,
                                           const IO *const (&colp)[NCA],
                                           const IO *const (&rowp)[NRA],
                                           int64_t b, int64_t T, int64_t t0, int n,
                                           int64_t ncols, int64_t nrows, int64_t row0, int64_t heads = 1,
                                           int64_t col0 = 0, int64_t colw = 0) {
    // col0, colw: the window of the column arrays this pass works on (colw = 0: all ncols columns)
    const int csub = threadIdx.x % g.CW, tsub = threadIdx.x / g.CW;
    const int64_t line0 = row_first_token(b, T, heads) + t0 * heads;      // [.., width] line of step t0
    const int64_t cstep = heads * ncols, rstep = heads * nrows;           // elements between consecutive steps
    const int64_t cbase = line0 * ncols + col0;
    if (colw > 0) ncols = colw;
#pragma unroll
    for (int m = 0; m < PFC; ++m) {
        if (g.SP * (m >> g.lncc) >= TMAX) continue;
        const int tt = tsub + g.SP * (m >> g.lncc);
        const int c = csub + g.CW * (m & ((1 << g.lncc) - 1));
        const bool ok = tt < n && c < ncols;
#pragma unroll
        for (int a = 0; a < NCA; ++a)
            pf.c[a][m] = ok ? colp[a][cbase + (int64_t)tt * cstep + c] : IO(0);
    }
    const int rsub = threadIdx.x % g.rows, tsr = threadIdx.x / g.rows;
    const int64_t rbase = line0 * nrows + row0;
#pragma unroll
    for (int m = 0; m < PFR; ++m) {
        if (g.SPR * m >= TMAX) continue;
        const int tt = tsr + g.SPR * m;
        const bool ok = tt < n && row0 + rsub < nrows;
#pragma unroll
        for (int a = 0; a < NRA; ++a)
            pf.r[a][m] = ok ? rowp[a][rbase + (int64_t)tt * rstep + rsub] : IO(0);
    }
}

// Write the prefetched block into LDS: colL[(tt*NCA + a)*KP + c], rowL[(tt*NRA + a)*rows + r]
template <typename IO, typename Acc, int NCA, int NRA, int TMAX = 1 << 30>
__device__ __forceinline__ void block_store(const Prefetch<IO, NCA, NRA> &pf, const Tile &g,
                                            Acc *colL, Acc *rowL, int tb) {
    const int csub = threadIdx.x % g.CW, tsub = threadIdx.x / g.CW;
#pragma unroll
    for (int m = 0; m < PFC; ++m) {
        if (g.SP * (m >> g.lncc) >= TMAX) continue;
        const int tt = tsub + g.SP * (m >> g.lncc);
        const int c = csub + g.CW * (m & ((1 << g.lncc) - 1));
        if (tt < tb) {
#pragma unroll
            for (int a = 0; a < NCA; ++a) colL[(tt * NCA + a) * g.KP + c] = to_acc(pf.c[a][m]);
        }
    }
    const int rsub = threadIdx.x % g.rows, tsr = threadIdx.x / g.rows;
#pragma unroll
    for (int m = 0; m < PFR; ++m) {
        if (g.SPR * m >= TMAX) continue;
        const int tt = tsr + g.SPR * m;
        if (tt < tb) {
#pragma unroll
            for (int a = 0; a < NRA; ++a) rowL[(tt * NRA + a) * g.rows + rsub] = to_acc(pf.r[a][m]);
        }
    }
}

}  // namespace scan
}  // namespace t2fw
