// Argument block and host entry point of the T = 1 generation-step kernel (lfw_step.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace t2fw {

struct StepArgs {
    const void *x, *f, *q, *k, *f_key, *s0;   // x,f [B,64]; q,k,f_key [B,64]; s0 [B,64,64]
    void *out, *next_state;                   // next_state may alias s0
    int64_t B;
};

int step_forward(const StepArgs &a, int dtype, hipStream_t stream);

}  // namespace t2fw
