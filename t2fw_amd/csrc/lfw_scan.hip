// Exact per-step scan kernels for the decay-rule recurrence: any D, K, dtype.
//
// These are the general-shape path (odd sizes, fp32/fp64, tiny gates) and the
// row-level fallback of the chunked MFMA kernels.  One lane owns KPL adjacent
// elements of one state row; KG lanes share a row and reduce with DPP.  The state
// stays in VGPRs for the whole sequence; inputs are staged through LDS one time
// block ahead (global loads for block n+1 are in flight while block n is computed).
//
// The backward pass is run as two launches of one kernel template, once with the
// state rows along D (gives d_x, d_f, d_s0) and once along K (gives d_k, d_f_key,
// d_q): the recurrence is symmetric under swapping (x,f,g_out) with (k,f_key,q) and
// transposing the state, so every reduction is along the lane-shared row and no
// atomics or cross-workgroup reductions are needed.
//
// Reference semantics: t2fw/torch.py:21-31 (forward), t2fw/csrc/lfw_kernel.cu:85-100
// and t2fw/csrc/lfw.cpp:84-93 (backward).
#include "lfw_scan_body.hpp"

namespace t2fw {

namespace {

using namespace scan;

// One workgroup per (batch row, tile).
template <typename IO, int KPL>
__global__ __launch_bounds__(SCAN_THREADS) void lfw_fwd_scan_kernel(ScanFwdArgs p) {
    fwd_scan_body<IO, KPL>(p, blockIdx.x / p.ntiles, (int)(blockIdx.x % p.ntiles));
}

// One workgroup per (batch row, tile); a kernel per geometry (KG lanes per state row, 0 = any) and
// per use of the segment-start buffer, so that each is register-allocated on its own: a spill
// in the loop would wait for the prefetched global loads, which return in order with it.
template <typename IO, int KPL, int SIDE, int KG, int SUB>
__global__ __launch_bounds__(SCAN_THREADS) void lfw_bwd_scan_kernel(ScanBwdArgs p) {
    bwd_scan_body_kg<IO, KPL, SIDE, KG, SUB>(p, blockIdx.x / p.ntiles, (int)(blockIdx.x % p.ntiles));
}

// ------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------
template <typename IO, int KPL>
int launch_fwd(const ScanFwdArgs &a, const ScanGeom &g, hipStream_t stream) {
    using Acc = typename AccOf<IO>::type;
    const size_t smem = scan_fwd_lds_bytes(a.tb, g.kg, g.kpl, g.rows) * sizeof(Acc) / 4;
    ScanFwdArgs a2 = a;
    a2.ntiles = (int)((a.D + g.rows - 1) / g.rows);
    const int64_t nblocks = a.B * a2.ntiles;
    if (nblocks > 0x7fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "grid of %lld workgroups is too large", (long long)nblocks);
    dim3 grid((unsigned)nblocks, 1, 1);
    hipLaunchKernelGGL((lfw_fwd_scan_kernel<IO, KPL>), grid, dim3(SCAN_THREADS), smem, stream, a2);
    return check_hip(hipGetLastError(), "lfw_fwd_scan_kernel launch");
}

template <typename IO, int KPL, int SIDE>
int launch_bwd(ScanBwdArgs a, const ScanGeom &g, hipStream_t stream) {
    using Acc = typename AccOf<IO>::type;
    constexpr int SEG = SegLen<KPL>::value;
    const int64_t nrows = SIDE == 0 ? a.D : a.K;
    const size_t base = scan_bwd_lds_bytes(SEG, g.kg, g.kpl, g.rows, a.C, false) * sizeof(Acc) / 4;
    const size_t with_sub = scan_bwd_lds_bytes(SEG, g.kg, g.kpl, g.rows, a.C, true) * sizeof(Acc) / 4;
    a.use_sub = (with_sub <= 64 * 1024) ? 1 : 0;
    const size_t smem = a.use_sub ? with_sub : base;
    a.kg = g.kg;
    a.ntiles = (int)((nrows + g.rows - 1) / g.rows);
    const int64_t nblocks = a.B * a.ntiles;
    if (nblocks > 0x7fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "grid of %lld workgroups is too large", (long long)nblocks);
    dim3 grid((unsigned)nblocks, 1, 1);
    if (KPL <= 4 && g.kg == 16 && a.use_sub)
        hipLaunchKernelGGL((lfw_bwd_scan_kernel<IO, KPL, SIDE, (KPL <= 4 ? 16 : 0), 1>), grid, dim3(SCAN_THREADS), smem, stream, a);
    else if (a.use_sub)
        hipLaunchKernelGGL((lfw_bwd_scan_kernel<IO, KPL, SIDE, 0, 1>), grid, dim3(SCAN_THREADS), smem, stream, a);
    else
        hipLaunchKernelGGL((lfw_bwd_scan_kernel<IO, KPL, SIDE, 0, 0>), grid, dim3(SCAN_THREADS), smem, stream, a);
    return check_hip(hipGetLastError(), "lfw_bwd_scan_kernel launch");
}

// One pass: the key channels [a.col0, a.col0 + width) of the state.
template <typename IO> int fwd_pass(ScanFwdArgs a, int64_t width, hipStream_t stream) {
    const ScanGeom g = scan_geometry(width);
    a.kg = g.kg;
    int tb = 32;
    const int by_cols = PFC * SCAN_THREADS / (g.kg * g.kpl);
    const int by_rows = PFR * SCAN_THREADS / g.rows;
    if (by_cols < tb) tb = by_cols;
    if (by_rows < tb) tb = by_rows;
    a.tb = tb < 1 ? 1 : tb;
    switch (g.kpl) {
        case 1: return launch_fwd<IO, 1>(a, g, stream);
        case 2: return launch_fwd<IO, 2>(a, g, stream);
        case 4: return launch_fwd<IO, 4>(a, g, stream);
        case 8: return launch_fwd<IO, 8>(a, g, stream);
        case 16: return launch_fwd<IO, 16>(a, g, stream);
        case 32: return launch_fwd<IO, 32>(a, g, stream);
    }
    return fail(T2FW_ERR_UNSUPPORTED, "unsupported columns-per-lane %d", g.kpl);
}

// A lane group holds up to SCAN_MAX_COLS columns of a state row.  Wider states run as several
// launches, one per window of columns: the columns of the state never interact (each has its own
// gate and its own input), and the outputs are sums over them, which the later launches add to
// (the reference tiles K over blocks, t2fw/csrc/lfw_kernel.cu:146-155).  With 16-bit tensors the
// sum is rounded to the tensor type once per launch.
template <typename IO> int fwd_by_kpl(ScanFwdArgs a, hipStream_t stream) {
    if (a.K <= SCAN_MAX_COLS) return fwd_pass<IO>(a, a.K, stream);
    for (int64_t c0 = 0; c0 < a.K; c0 += SCAN_MAX_COLS) {
        a.col0 = c0;
        a.colw = a.K - c0 < SCAN_MAX_COLS ? a.K - c0 : SCAN_MAX_COLS;
        a.accumulate = c0 > 0 ? 1 : 0;
        const int rc = fwd_pass<IO>(a, a.colw, stream);
        if (rc != T2FW_OK) return rc;
    }
    return T2FW_OK;
}

template <typename IO, int SIDE> int bwd_pass(const ScanBwdArgs &a, int64_t width, hipStream_t stream) {
    const ScanGeom g = scan_geometry(width);
    switch (g.kpl) {
        case 1: return launch_bwd<IO, 1, SIDE>(a, g, stream);
        case 2: return launch_bwd<IO, 2, SIDE>(a, g, stream);
        case 4: return launch_bwd<IO, 4, SIDE>(a, g, stream);
        case 8: return launch_bwd<IO, 8, SIDE>(a, g, stream);
        case 16: return launch_bwd<IO, 16, SIDE>(a, g, stream);
        case 32: return launch_bwd<IO, 32, SIDE>(a, g, stream);
    }
    return fail(T2FW_ERR_UNSUPPORTED, "unsupported columns-per-lane %d", g.kpl);
}

// The reduced dimension (K on side 0, D on side 1) in windows, as for the forward.
template <typename IO, int SIDE> int bwd_by_kpl(ScanBwdArgs a, hipStream_t stream) {
    const int64_t ncols = SIDE == 0 ? a.K : a.D;
    if (ncols <= SCAN_MAX_COLS) return bwd_pass<IO, SIDE>(a, ncols, stream);
    for (int64_t c0 = 0; c0 < ncols; c0 += SCAN_MAX_COLS) {
        a.col0 = c0;
        a.colw = ncols - c0 < SCAN_MAX_COLS ? ncols - c0 : SCAN_MAX_COLS;
        a.accumulate = c0 > 0 ? 1 : 0;
        const int rc = bwd_pass<IO, SIDE>(a, a.colw, stream);
        if (rc != T2FW_OK) return rc;
    }
    return T2FW_OK;
}

template <typename IO> int bwd_both(const ScanBwdArgs &a, hipStream_t stream) {
    int rc = bwd_by_kpl<IO, 0>(a, stream);
    if (rc != T2FW_OK) return rc;
    return bwd_by_kpl<IO, 1>(a, stream);
}

}  // namespace

int scan_forward(const ScanFwdArgs &a, int dtype, hipStream_t stream) {
    switch (dtype) {
        case T2FW_F32: return fwd_by_kpl<float>(a, stream);
        case T2FW_F16: return fwd_by_kpl<__half>(a, stream);
        case T2FW_BF16: return fwd_by_kpl<__hip_bfloat16>(a, stream);
        case T2FW_F64: return fwd_by_kpl<double>(a, stream);
    }
    return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
}

int scan_backward(const ScanBwdArgs &a, int dtype, hipStream_t stream) {
    switch (dtype) {
        case T2FW_F32: return bwd_both<float>(a, stream);
        case T2FW_F16: return bwd_both<__half>(a, stream);
        case T2FW_BF16: return bwd_both<__hip_bfloat16>(a, stream);
        case T2FW_F64: return bwd_both<double>(a, stream);
    }
    return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
}

}  // namespace t2fw
