// Shared device/host helpers for the gfx950 kernels: I/O element types, conversions,
// wave64 cross-lane reductions (DPP), error plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/t2fw_hip.h"

namespace t2fw {

// ----------------------------------------------------------------------------------
// error plumbing (host)
// ----------------------------------------------------------------------------------
int fail(int code, const char *fmt, ...);   // records the message, returns code
int check_hip(hipError_t e, const char *what);
// Allows `kernel` to be launched with up to `bytes` of dynamic LDS (more than 64 KB has to be enabled per
// function and device); the runtime is asked once per (kernel, device).
int enable_lds(const void *kernel, int bytes, const char *what);

// ----------------------------------------------------------------------------------
// layout of the [.., T, .., width] tensors: batch rows are either contiguous [T, width] slabs
// (heads = 1) or the heads of a [B / heads, T, heads, width] tensor.  Token t of row b sits at
// element (row_first_token(b, T, heads) + t * heads) * width.
// ----------------------------------------------------------------------------------
__host__ __device__ inline int64_t row_first_token(int64_t b, int64_t T, int64_t heads) {
    return heads == 1 ? b * T : (b / heads) * T * heads + b % heads;
}

// ----------------------------------------------------------------------------------
// element types: IO is what lives in HBM, Acc is what the recurrence is carried in
// ----------------------------------------------------------------------------------
template <typename IO> struct AccOf { using type = float; };
template <> struct AccOf<double> { using type = double; };

__device__ __forceinline__ float to_acc(float v) { return v; }
__device__ __forceinline__ double to_acc(double v) { return v; }
__device__ __forceinline__ float to_acc(__half v) { return __half2float(v); }
__device__ __forceinline__ float to_acc(__hip_bfloat16 v) { return __bfloat162float(v); }

template <typename IO> __device__ __forceinline__ IO from_acc(typename AccOf<IO>::type v);
template <> __device__ __forceinline__ float from_acc<float>(float v) { return v; }
template <> __device__ __forceinline__ double from_acc<double>(double v) { return v; }
template <> __device__ __forceinline__ __half from_acc<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 from_acc<__hip_bfloat16>(float v) {
    return __float2bfloat16(v);
}

// ----------------------------------------------------------------------------------
// DPP cross-lane moves inside a row of 16 lanes (no LDS traffic).
// ----------------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

constexpr int DPP_QUAD_XOR1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// Sum over groups of `group` adjacent lanes (group = power of two, 1..64); every lane
// of a group ends with the group's total.  Groups up to 16 use DPP only.
__device__ __forceinline__ float group_sum(float v, int group) {
    if (group >= 2) v += dpp_move<DPP_QUAD_XOR1>(v);
    if (group >= 4) v += dpp_move<DPP_QUAD_XOR2>(v);
    if (group >= 8) v += dpp_move<DPP_ROW_HALF_MIRROR>(v);   // quads already uniform
    if (group >= 16) v += dpp_move<DPP_ROW_MIRROR>(v);       // half rows already uniform
    if (group >= 32) v += __shfl_xor(v, 16, 64);
    if (group >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ double group_sum(double v, int group) {
    for (int m = 1; m < group; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Wait until none of this wave's global loads and stores is outstanding (s_waitcnt vmcnt(0); the other
// counters of the immediate left at their maxima, i.e. not waited for).
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0f70); }

// ----------------------------------------------------------------------------------
// launch geometry of the exact scan kernels (shared by host dispatch and kernels)
// ----------------------------------------------------------------------------------
constexpr int SCAN_THREADS = 256;
constexpr int SCAN_MAX_KPL = 32;     // columns held per lane
constexpr int SCAN_MAX_COLS = 64 * SCAN_MAX_KPL;

struct ScanGeom {
    int kg;      // lanes cooperating on one state row (power of two, <= 64)
    int kpl;     // columns per lane (power of two, <= SCAN_MAX_KPL)
    int rows;    // state rows per workgroup = SCAN_THREADS / kg
};

inline int next_pow2(int64_t n) {
    int p = 1;
    while (p < n) p <<= 1;
    return p;
}

// cols = length of the reduced dimension (K for the value-side kernels)
inline ScanGeom scan_geometry(int64_t cols) {
    ScanGeom g;
    int p = next_pow2(cols);
    if (p < 2) p = 2;                 // at least two lanes per row (bounds rows per workgroup)
    g.kg = p < 16 ? p : 16;
    g.kpl = p / g.kg;
    while (g.kpl > SCAN_MAX_KPL / 8 && g.kg < 64) {   // wide rows: spread over more lanes
        g.kg <<= 1;
        g.kpl >>= 1;
    }
    if (g.kpl < 1) g.kpl = 1;
    g.rows = SCAN_THREADS / g.kg;
    return g;
}

}  // namespace t2fw
