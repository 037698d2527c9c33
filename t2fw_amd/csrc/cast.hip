// Conversion of up to eight arrays between float32 and a 16-bit type in one launch: what a caller with float32
// tensors pays to run the 16-bit matrix-core kernels (the six inputs of the recurrence in one launch, its two
// outputs in another, likewise for the gradients).  Pure streaming: a lane converts eight elements per step
// (32 bytes of float32, 16 bytes of the 16-bit type); blockIdx.y is the array.  The reference has one kernel
// for every dtype (t2fw/csrc/lfw_kernel.cu:157-168) and no counterpart of this.
#include "common.hpp"
#include "cast.hpp"
#include "lfw_chunk.hpp"

namespace t2fw {
namespace {

constexpr int CAST_THREADS = 256;
constexpr int CAST_PIECE = 8;         // elements per lane and step

// H: Fp16 or Bf16 (bit-level conversions of lfw_chunk.hpp); NARROW: float32 -> H, else H -> float32
template <typename H, bool NARROW> __global__ __launch_bounds__(CAST_THREADS) void cast_kernel(CastArgs p) {
    const int a = blockIdx.y;
    const int64_t n = p.n[a];
    const int64_t npieces = (n + CAST_PIECE - 1) / CAST_PIECE;
    const float *const wide = NARROW ? static_cast<const float *>(p.src[a]) : static_cast<float *>(p.dst[a]);
    const u16 *const narrow = NARROW ? static_cast<u16 *>(p.dst[a]) : static_cast<const u16 *>(p.src[a]);
    for (int64_t piece = (int64_t)blockIdx.x * CAST_THREADS + threadIdx.x; piece < npieces; piece += (int64_t)gridDim.x * CAST_THREADS) {
        const int64_t e0 = piece * CAST_PIECE;
        if (e0 + CAST_PIECE <= n) {
            if (NARROW) {
                const float4 lo = *reinterpret_cast<const float4 *>(wide + e0), hi = *reinterpret_cast<const float4 *>(wide + e0 + 4);
                *reinterpret_cast<uint4 *>(const_cast<u16 *>(narrow) + e0) =
                    make_uint4(H::pack2(lo.x, lo.y), H::pack2(lo.z, lo.w), H::pack2(hi.x, hi.y), H::pack2(hi.z, hi.w));
            } else {
                const uint4 v = *reinterpret_cast<const uint4 *>(narrow + e0);
                float *const d = const_cast<float *>(wide) + e0;
                *reinterpret_cast<float4 *>(d) = make_float4(H::to_f32((u16)(v.x & 0xffffu)), H::to_f32((u16)(v.x >> 16)),
                                                             H::to_f32((u16)(v.y & 0xffffu)), H::to_f32((u16)(v.y >> 16)));
                *reinterpret_cast<float4 *>(d + 4) = make_float4(H::to_f32((u16)(v.z & 0xffffu)), H::to_f32((u16)(v.z >> 16)),
                                                                 H::to_f32((u16)(v.w & 0xffffu)), H::to_f32((u16)(v.w >> 16)));
            }
        } else {
            for (int64_t e = e0; e < n; ++e) {
                if (NARROW)
                    const_cast<u16 *>(narrow)[e] = (u16)(H::pack2(wide[e], 0.f) & 0xffffu);
                else
                    const_cast<float *>(wide)[e] = H::to_f32(narrow[e]);
            }
        }
    }
}

template <typename H, bool NARROW> int launch(const CastArgs &a, hipStream_t stream) {
    int64_t most = 0;
    for (int i = 0; i < a.count; ++i) most = a.n[i] > most ? a.n[i] : most;
    if (most == 0) return T2FW_OK;
    const int64_t blocks = (most + (int64_t)CAST_THREADS * CAST_PIECE - 1) / ((int64_t)CAST_THREADS * CAST_PIECE);
    const unsigned gx = (unsigned)(blocks < 8192 ? blocks : 8192);
    hipLaunchKernelGGL((cast_kernel<H, NARROW>), dim3(gx, (unsigned)a.count), dim3(CAST_THREADS), 0, stream, a);
    return check_hip(hipGetLastError(), "cast_kernel launch");
}

}  // namespace

int cast_tensors(const CastArgs &a, int src_dtype, int dst_dtype, hipStream_t stream) {
    if (src_dtype == T2FW_F32 && dst_dtype == T2FW_F16) return launch<Fp16, true>(a, stream);
    if (src_dtype == T2FW_F32 && dst_dtype == T2FW_BF16) return launch<Bf16, true>(a, stream);
    if (src_dtype == T2FW_F16 && dst_dtype == T2FW_F32) return launch<Fp16, false>(a, stream);
    if (src_dtype == T2FW_BF16 && dst_dtype == T2FW_F32) return launch<Bf16, false>(a, stream);
    return fail(T2FW_ERR_BAD_DTYPE, "t2fw_cast converts between float32 and float16 / bfloat16 only (got %d -> %d)", src_dtype, dst_dtype);
}

}  // namespace t2fw
