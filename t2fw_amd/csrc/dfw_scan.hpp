// Argument blocks and host entry points of the delta-rule kernels (dfw_scan.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace t2fw {

struct DfwFwdArgs {
    const void *q, *k, *v, *s0;
    void *out, *final_state, *delta;
    int64_t B, T, D, M;
    int32_t kg, tb, ntiles;
};

struct DfwBwdArgs {
    const void *g_out, *g_state, *q, *k, *delta, *final_state;
    void *d_q, *d_k, *d_v, *d_s0;
    int64_t B, T, D, M;
    int32_t kg, tb, ntiles;
};

int dfw_forward(const DfwFwdArgs &a, int dtype, hipStream_t stream);
int dfw_backward(const DfwBwdArgs &a, int dtype, hipStream_t stream);
// block-wise matrix-core kernels: D = M = 64, fp32 / fp16 / bf16 tensors, 16-byte aligned pointers (dfw_chunk_fwd.hip,
// dfw_chunk_bwd.hip)
int dfw_chunk_forward(const DfwFwdArgs &a, int dtype, bool split_operands, hipStream_t stream);
int dfw_chunk_backward(const DfwBwdArgs &a, int dtype, bool split_operands, hipStream_t stream);

}  // namespace t2fw
