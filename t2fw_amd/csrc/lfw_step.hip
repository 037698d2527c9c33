// One generation step (T = 1) of the decay rule for D = K = 64, 16-bit tensors:
//   S' = S * (f (x) f_key) + x (x) k ;  out = S' q
// Pure state streaming: 8 KB of state in and out per batch row against ~1.4 flop per byte,
// so the kernel is HBM bound.  One wave owns one row; lane (dr, kq) holds the
// 8 x 8 block S[8dr..8dr+8, 8kq..8kq+8] as eight 16-byte pieces (each load instruction
// covers eight full 128-byte state rows), and out_d is reduced over the eight lanes of a row group
// with DPP.
// The state may be updated in place.  Serves the T = 1 calls the reference makes in
// generation (tests/benchmark.py:86-88,104-105).
#include "lfw_chunk.hpp"
#include "lfw_step.hpp"

namespace t2fw {
namespace {

constexpr int STEP_THREADS = 128;

template <typename E> __device__ __forceinline__ void unpack8(const uint4 &v, float (&o)[8]) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        o[2 * i] = E::to_f32((u16)(w[i] & 0xffff));
        o[2 * i + 1] = E::to_f32((u16)(w[i] >> 16));
    }
}

template <typename E>
__global__ __launch_bounds__(STEP_THREADS) void lfw_step_kernel(StepArgs p) {
    const int lane = threadIdx.x & 63;
    const int kq = lane & 7, dr = lane >> 3;
    const int64_t wave = (int64_t)blockIdx.x * (STEP_THREADS / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (STEP_THREADS / 64);
    const u16 *s0 = reinterpret_cast<const u16 *>(p.s0);
    u16 *s1 = reinterpret_cast<u16 *>(p.next_state);
    // element offset of this lane's piece i inside a [64][64] state: row 8dr+i, columns 8kq..
    const int soff = (8 * dr) * CH_N + 8 * kq;

    // one row per wave; the loop only serves batches beyond the largest grid
    for (int64_t row = wave; row < p.B; row += nwaves) {
        uint4 cur[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) cur[i] = *reinterpret_cast<const uint4 *>(s0 + row * (CH_N * CH_N) + soff + i * CH_N);
        const int64_t vo = row * CH_N;
        float xv[8], fv[8], kv[8], gv[8], qv[8];
        unpack8<E>(*reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.x) + vo + 8 * dr), xv);
        unpack8<E>(*reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.f) + vo + 8 * dr), fv);
        unpack8<E>(*reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.k) + vo + 8 * kq), kv);
        unpack8<E>(*reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.f_key) + vo + 8 * kq), gv);
        unpack8<E>(*reinterpret_cast<const uint4 *>(reinterpret_cast<const u16 *>(p.q) + vo + 8 * kq), qv);
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float sv[8];
            unpack8<E>(cur[i], sv);
            float a = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sv[e] = sv[e] * (fv[i] * gv[e]) + xv[i] * kv[e];
                a += sv[e] * qv[e];
            }
            acc[i] = a;
            *reinterpret_cast<uint4 *>(s1 + row * (CH_N * CH_N) + soff + i * CH_N) =
                make_uint4(E::pack2(sv[0], sv[1]), E::pack2(sv[2], sv[3]), E::pack2(sv[4], sv[5]), E::pack2(sv[6], sv[7]));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = group_sum(acc[i], 8);
        if (kq == 0)
            *reinterpret_cast<uint4 *>(reinterpret_cast<u16 *>(p.out) + vo + 8 * dr) =
                make_uint4(E::pack2(acc[0], acc[1]), E::pack2(acc[2], acc[3]), E::pack2(acc[4], acc[5]), E::pack2(acc[6], acc[7]));
    }
}

template <typename E> int launch(const StepArgs &a, hipStream_t stream) {
    const int64_t waves_per_wg = STEP_THREADS / 64;
    int64_t wgs = (a.B + waves_per_wg - 1) / waves_per_wg;
    // One wave per row, as many workgroups as rows need: measured 7 % faster than a grid of
    // resident waves that loop over rows with a register prefetch (5.5 against 5.2 TB/s).
    if (wgs > 0x7fffffffLL) wgs = 0x7fffffffLL;
    hipLaunchKernelGGL(lfw_step_kernel<E>, dim3((unsigned)wgs), dim3(STEP_THREADS), 0, stream, a);
    return check_hip(hipGetLastError(), "lfw_step_kernel launch");
}

}  // namespace

int step_forward(const StepArgs &a, int dtype, hipStream_t stream) {
    if (dtype == T2FW_F16) return launch<Fp16>(a, stream);
    if (dtype == T2FW_BF16) return launch<Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the step kernel takes fp16 or bf16 tensors");
}

}  // namespace t2fw
