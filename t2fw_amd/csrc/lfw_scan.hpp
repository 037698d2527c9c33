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

int scan_forward(const ScanFwdArgs &a, int dtype, hipStream_t stream);
int scan_backward(const ScanBwdArgs &a, int dtype, hipStream_t stream);

}  // namespace t2fw
