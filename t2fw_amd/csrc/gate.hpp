// Argument blocks and host entry points of the sigmoid gating kernels (gate.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace t2fw {

struct GateFwdArgs {
    const void *f_logit, *fk_logit;     // [n_f], [n_fk]
    void *f, *f_key;                    // may alias the logits
    int64_t n_f, n_fk;
};

struct GateBwdArgs {
    const void *d_f, *d_f_key, *f, *f_key;
    void *d_f_logit, *d_fk_logit;       // may alias d_f, d_f_key
    int64_t n_f, n_fk;
};

int gate_forward(const GateFwdArgs &a, int dtype, hipStream_t stream);
int gate_backward(const GateBwdArgs &a, int dtype, hipStream_t stream);

}  // namespace t2fw
