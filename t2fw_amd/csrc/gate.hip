// Sigmoid gating of the two forget gates in one launch, and its backward.
//   forward : f = sigmoid(f_logit), f_key = sigmoid(fk_logit)
//   backward: d_logit = d_gate * gate * (1 - gate)          (may run in place over d_gate)
// The recurrence kernels take gates that are already in (0, 1]; the reference leaves the
// non-linearity to the caller ("does not perform the non-linear sigmoid gating",
// t2fw/functional_lfw.py:25-30), which costs separate elementwise passes per gate and
// direction.  These kernels are pure streaming: 16 bytes per lane per access, both arrays
// covered by one grid, arithmetic in fp32.
#include "common.hpp"
#include "gate.hpp"

namespace t2fw {
namespace {

constexpr int GATE_THREADS = 256;
constexpr int GATE_UNROLL = 4;

template <typename IO> struct Vec16 { static constexpr int N = 16 / sizeof(IO); };

// 16-bit results: hardware exp2 and reciprocal (about 2^-21 relative, far below the rounding of the
// result); fp32 results: the accurate library exponential and an IEEE division
template <typename IO> __device__ __forceinline__ float sigmoid_of(IO z) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-(float)to_acc(z)));
}
template <> __device__ __forceinline__ float sigmoid_of<float>(float z) { return 1.0f / (1.0f + expf(-z)); }

// Work is cut into pieces of N elements (16 bytes); pieces [0, np_f) belong to the first array,
// the rest to the second.  A workgroup covers GATE_UNROLL * GATE_THREADS consecutive pieces and a
// lane takes GATE_UNROLL of them, GATE_THREADS apart, with all loads issued before the arithmetic.
template <typename IO> struct Piece {
    const IO *a, *b;   // sources (b only for backward)
    IO *dst;
    int64_t e0, n;
    bool live, full;
};

template <typename IO, bool BWD>
__device__ __forceinline__ Piece<IO> locate(const void *a_f, const void *a_k, const void *b_f, const void *b_k, void *o_f,
                                            void *o_k, int64_t n_f, int64_t n_fk, int64_t i) {
    constexpr int N = Vec16<IO>::N;
    const int64_t np_f = (n_f + N - 1) / N, np = np_f + (n_fk + N - 1) / N;
    const bool first = i < np_f;
    Piece<IO> pc;
    pc.a = static_cast<const IO *>(first ? a_f : a_k);
    pc.b = BWD ? static_cast<const IO *>(first ? b_f : b_k) : nullptr;
    pc.dst = static_cast<IO *>(first ? o_f : o_k);
    pc.n = first ? n_f : n_fk;
    pc.e0 = (first ? i : i - np_f) * N;
    pc.live = i < np;
    pc.full = pc.live && pc.e0 + N <= pc.n;
    return pc;
}

template <typename IO>
__global__ __launch_bounds__(GATE_THREADS) void gate_fwd_kernel(GateFwdArgs p) {
    constexpr int N = Vec16<IO>::N;
    const int64_t base = (int64_t)blockIdx.x * (GATE_UNROLL * GATE_THREADS) + threadIdx.x;
    Piece<IO> pc[GATE_UNROLL];
    uint4 raw[GATE_UNROLL];
#pragma unroll
    for (int u = 0; u < GATE_UNROLL; ++u) {
        pc[u] = locate<IO, false>(p.f_logit, p.fk_logit, nullptr, nullptr, p.f, p.f_key, p.n_f, p.n_fk,
                                  base + (int64_t)u * GATE_THREADS);
        if (pc[u].full) raw[u] = *reinterpret_cast<const uint4 *>(pc[u].a + pc[u].e0);
    }
#pragma unroll
    for (int u = 0; u < GATE_UNROLL; ++u) {
        if (pc[u].full) {
            IO v[N];
            *reinterpret_cast<uint4 *>(v) = raw[u];
#pragma unroll
            for (int j = 0; j < N; ++j) v[j] = from_acc<IO>(sigmoid_of(v[j]));
            *reinterpret_cast<uint4 *>(pc[u].dst + pc[u].e0) = *reinterpret_cast<const uint4 *>(v);
        } else if (pc[u].live) {
            for (int64_t e = pc[u].e0; e < pc[u].n; ++e) pc[u].dst[e] = from_acc<IO>(sigmoid_of(pc[u].a[e]));
        }
    }
}

template <typename IO>
__global__ __launch_bounds__(GATE_THREADS) void gate_bwd_kernel(GateBwdArgs p) {
    constexpr int N = Vec16<IO>::N;
    const int64_t base = (int64_t)blockIdx.x * (GATE_UNROLL * GATE_THREADS) + threadIdx.x;
    Piece<IO> pc[GATE_UNROLL];
    uint4 ra[GATE_UNROLL], rb[GATE_UNROLL];
#pragma unroll
    for (int u = 0; u < GATE_UNROLL; ++u) {
        pc[u] = locate<IO, true>(p.d_f, p.d_f_key, p.f, p.f_key, p.d_f_logit, p.d_fk_logit, p.n_f, p.n_fk,
                                 base + (int64_t)u * GATE_THREADS);
        if (pc[u].full) {
            ra[u] = *reinterpret_cast<const uint4 *>(pc[u].a + pc[u].e0);
            rb[u] = *reinterpret_cast<const uint4 *>(pc[u].b + pc[u].e0);
        }
    }
#pragma unroll
    for (int u = 0; u < GATE_UNROLL; ++u) {
        if (pc[u].full) {
            IO a[N], b[N];
            *reinterpret_cast<uint4 *>(a) = ra[u];
            *reinterpret_cast<uint4 *>(b) = rb[u];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const float g = (float)to_acc(b[j]);
                a[j] = from_acc<IO>((float)to_acc(a[j]) * g * (1.0f - g));
            }
            *reinterpret_cast<uint4 *>(pc[u].dst + pc[u].e0) = *reinterpret_cast<const uint4 *>(a);
        } else if (pc[u].live) {
            for (int64_t e = pc[u].e0; e < pc[u].n; ++e) {
                const float g = (float)to_acc(pc[u].b[e]);
                pc[u].dst[e] = from_acc<IO>((float)to_acc(pc[u].a[e]) * g * (1.0f - g));
            }
        }
    }
}

// one workgroup per GATE_UNROLL * GATE_THREADS pieces
int64_t blocks_for(int64_t pieces) {
    return (pieces + GATE_UNROLL * GATE_THREADS - 1) / (GATE_UNROLL * GATE_THREADS);
}

template <typename IO> int launch_fwd(const GateFwdArgs &a, hipStream_t stream) {
    constexpr int N = Vec16<IO>::N;
    const int64_t pieces = (a.n_f + N - 1) / N + (a.n_fk + N - 1) / N;
    if (pieces == 0) return T2FW_OK;
    if (blocks_for(pieces) > 0x7fffffff) return fail(T2FW_ERR_BAD_SHAPE, "gate arrays too large for one launch");
    hipLaunchKernelGGL(gate_fwd_kernel<IO>, dim3((unsigned)blocks_for(pieces)), dim3(GATE_THREADS), 0, stream, a);
    return check_hip(hipGetLastError(), "gate_fwd_kernel launch");
}

template <typename IO> int launch_bwd(const GateBwdArgs &a, hipStream_t stream) {
    constexpr int N = Vec16<IO>::N;
    const int64_t pieces = (a.n_f + N - 1) / N + (a.n_fk + N - 1) / N;
    if (pieces == 0) return T2FW_OK;
    if (blocks_for(pieces) > 0x7fffffff) return fail(T2FW_ERR_BAD_SHAPE, "gate arrays too large for one launch");
    hipLaunchKernelGGL(gate_bwd_kernel<IO>, dim3((unsigned)blocks_for(pieces)), dim3(GATE_THREADS), 0, stream, a);
    return check_hip(hipGetLastError(), "gate_bwd_kernel launch");
}

}  // namespace

int gate_forward(const GateFwdArgs &a, int dtype, hipStream_t stream) {
    switch (dtype) {
        case T2FW_F32: return launch_fwd<float>(a, stream);
        case T2FW_F16: return launch_fwd<__half>(a, stream);
        case T2FW_BF16: return launch_fwd<__hip_bfloat16>(a, stream);
    }
    return fail(T2FW_ERR_BAD_DTYPE, "the gating kernels take fp32, fp16 or bf16 (dtype code %d)", dtype);
}

int gate_backward(const GateBwdArgs &a, int dtype, hipStream_t stream) {
    switch (dtype) {
        case T2FW_F32: return launch_bwd<float>(a, stream);
        case T2FW_F16: return launch_bwd<__half>(a, stream);
        case T2FW_BF16: return launch_bwd<__hip_bfloat16>(a, stream);
    }
    return fail(T2FW_ERR_BAD_DTYPE, "the gating kernels take fp32, fp16 or bf16 (dtype code %d)", dtype);
}

}  // namespace t2fw
