// Argument blocks and host entry points of the exact scan kernels (lfw_scan.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace t2fw {

struct ScanFwdArgs {
    const void *x, *f, *q, *k, *f_key, *s0;
    void *out, *next_state, *ckpt;      // ckpt may be null
    int64_t B, T, D, K, NC;
    int32_t C, kg, tb, ntiles;
    int32_t heads;                      // 1, or H: row b is head b % H of [B/H, T, H, D|K] tensors (x, f, q, k, f_key, out)
    // One pass over the key channels [col0, col0 + colw) of a state wider than a lane group holds
    // (colw = 0: all of them).  The state's columns never interact, and the outputs are sums over
    // them: a pass with accumulate set adds its share to what the passes before it left in out.
    int64_t col0, colw;
    int32_t accumulate;
};

struct ScanBwdArgs {
    const void *g_out, *g_state, *x, *f, *q, *k, *f_key, *ckpt;
    void *d_x, *d_f, *d_q, *d_k, *d_f_key, *d_s0;
    int64_t B, T, D, K, NC;
    int32_t C, kg, use_sub, ntiles;
    int32_t heads;                      // as for the forward (inputs, g_out and the five [.., T, .., D|K] gradients)
    // One pass over the reduced channels [col0, col0 + colw) (key channels on side 0, value channels on
    // side 1; colw = 0: all of them); with accumulate set the pass adds to the [.., T, .., D|K] gradients.
    int64_t col0, colw;
    int32_t accumulate;
};

// Dynamic LDS, in bytes, that the scan bodies use for a 32-bit accumulator (lfw_scan_body.hpp): the kernels
// that run a scan body inside another kernel's allocation check their own size against these.
//   forward: tb staged steps of the column inputs (kg * kpl columns) and the row inputs (rows per workgroup)
inline size_t scan_fwd_lds_bytes(int tb, int kg, int kpl, int rows) {
    return ((size_t)tb * 3 * kg * kpl + (size_t)tb * 3 * rows) * 4;
}
//   backward: seg staged steps of column inputs, row inputs and row outputs, plus (use_sub) the segment-start
//   states of one chunk, kpl values per thread of the 256
inline size_t scan_bwd_lds_bytes(int seg, int kg, int kpl, int rows, int C, bool use_sub) {
    const size_t base = ((size_t)seg * 3 * kg * kpl + (size_t)seg * 6 * rows) * 4;
    return base + (use_sub ? (size_t)((C + seg - 1) / seg) * kpl * 256 * 4 : 0);
}

int scan_forward(const ScanFwdArgs &a, int dtype, hipStream_t stream);
int scan_backward(const ScanBwdArgs &a, int dtype, hipStream_t stream);

}  // namespace t2fw
