// Argument block and host entry point of the multi-tensor conversion kernel (cast.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace t2fw {

constexpr int CAST_MAX_TENSORS = 8;

struct CastArgs {
    const void *src[CAST_MAX_TENSORS];
    void *dst[CAST_MAX_TENSORS];
    int64_t n[CAST_MAX_TENSORS];      // elements
    int32_t count;
};

// float32 <-> float16 / bfloat16, every tensor of the list in one launch
int cast_tensors(const CastArgs &a, int src_dtype, int dst_dtype, hipStream_t stream);

}  // namespace t2fw
