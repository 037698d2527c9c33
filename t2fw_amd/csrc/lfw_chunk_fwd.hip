// Forward scan of the decay rule in chunked matrix-core form (see lfw_chunk.hpp for the
// algebra).  One workgroup owns one batch row; matrix wave w keeps the 64 x 16
// slab S[:, 16w:16w+16] of the state in fp32 accumulator registers for the whole
// sequence.  Four more waves turn raw inputs into scaled 16-bit operand tiles in LDS, one
// (channel, 16-token block) per thread and one 32-token step ahead of the MFMA phase;
// raw inputs travel HBM -> registers (16-byte loads, two steps ahead) -> LDS -> per-channel columns.
//
// Replaces lfw_cuda_fwd_kernel + the output einsum of the reference
// (t2fw/csrc/lfw_kernel.cu:18-59, t2fw/csrc/lfw.cpp:45); semantics t2fw/torch.py:21-31.
#include "lfw_chunk.hpp"

// Build-time diagnostic (-DT2FW_PHASE_TIMERS): workgroup 0 accumulates shader-clock ticks
// per phase into row_flags[64..]; off in the shipped library.
#ifdef T2FW_PHASE_TIMERS
#define PHASE_BEGIN() unsigned long long ph_t = __builtin_amdgcn_s_memtime(); unsigned long long ph_acc[4] = {0, 0, 0, 0}
#define PHASE_MARK(i) { const unsigned long long ph_n = __builtin_amdgcn_s_memtime(); ph_acc[i] += ph_n - ph_t; ph_t = ph_n; }
#define PHASE_END(slot) if (b == 0 && (tid & 63) == 0) { for (int ph_i = 0; ph_i < 4; ++ph_i) p.row_flags[64 + (slot) * 8 + ph_i * 2] = (int)(ph_acc[ph_i] & 0x7fffffff); }
#else
#define PHASE_BEGIN()
#define PHASE_MARK(i)
#define PHASE_END(slot)
#endif

namespace t2fw {
namespace {

// ---- LDS layout of one operand buffer (bytes) -------------------------------------------
constexpr int OFF_QT = 0;                                  // qs  token-major  [32][TS] u16
constexpr int OFF_KT = OFF_QT + CH_STEP * TS * 2;          // kt  token-major  [32][TS] u16
constexpr int OFF_KH = OFF_KT + CH_STEP * TS * 2;          // kh  channel-major [64][CS] u16
constexpr int OFF_XT = OFF_KH + CH_N * CS * 2;             // xt  channel-major
constexpr int OFF_XH = OFF_XT + CH_N * CS * 2;             // xh  channel-major
constexpr int OFF_AS = OFF_XH + CH_N * CS * 2;             // a_t channel-major [64][CS] f32
constexpr int OFF_BL = OFF_AS + CH_N * CS * 4;             // b_L [2][64] f32
constexpr int OFF_AL = OFF_BL + 2 * CH_N * 4;              // a_L [2][64] f32
constexpr int OPS_BYTES = OFF_AL + 2 * CH_N * 4;
constexpr int OUT_BYTES = CH_STEP * OS * 2;
constexpr int OFF_OUT = 2 * OPS_BYTES;
// raw inputs of one step as they lie in HBM: 5 arrays [32 tokens][64 ch] u16 (f_key,k,q,f,x)
constexpr int RAW_ARRAY = CH_STEP * CH_N * 2;
constexpr int RAW_BYTES = 5 * RAW_ARRAY;
constexpr int OFF_RAW = OFF_OUT + 2 * OUT_BYTES;
constexpr int FWD_SMEM = OFF_RAW + 2 * RAW_BYTES;

struct Raw {
    u16 g[CH_L];   // gate  (f_key or f)
    u16 a[CH_L];   // k or x
    u16 u[CH_L];   // q (key side only)
};

// One step of raw inputs in flight: thread (token = tid/8, piece = tid%8) carries the
// 16-byte piece [token][8*piece .. 8*piece+8) of each of the five arrays.
struct Stage {
    uint4 v[5];
};

template <typename IOE>
__device__ __forceinline__ void stage_load(Stage &st, const u16 *const (&src)[5], int64_t row_base, int64_t T,
                                           int64_t step, int tid) {
    const int tok = tid >> 3, piece = tid & 7;
    const int64_t t = step * CH_STEP + tok;
    if (t < T) {
        const int64_t o = (row_base + t) * CH_N + 8 * piece;
#pragma unroll
        for (int a = 0; a < 5; ++a) st.v[a] = *reinterpret_cast<const uint4 *>(src[a] + o);
    } else {
        // steps past the end act as identity: gates 1, everything else 0
        const u32 one2 = (u32)IOE::ONE_BITS * 0x10001u;
#pragma unroll
        for (int a = 0; a < 5; ++a) st.v[a] = make_uint4(0, 0, 0, 0);
        st.v[0] = make_uint4(one2, one2, one2, one2);
        st.v[3] = make_uint4(one2, one2, one2, one2);
    }
}

__device__ __forceinline__ void stage_store(const Stage &st, unsigned char *raw, int tid) {
#pragma unroll
    for (int a = 0; a < 5; ++a) *reinterpret_cast<uint4 *>(raw + a * RAW_ARRAY + tid * 16) = st.v[a];
}

// channel c, block h: this thread's column of the raw tiles
__device__ __forceinline__ void raw_read(Raw &r, const unsigned char *raw, bool kside, int h, int c) {
    const u16 *base = reinterpret_cast<const u16 *>(raw + (kside ? 0 : 3) * RAW_ARRAY) + (CH_L * h) * CH_N + c;
#pragma unroll
    for (int t = 0; t < CH_L; ++t) {
        r.g[t] = base[t * CH_N];
        r.a[t] = base[RAW_ARRAY / 2 + t * CH_N];
        if (kside) r.u[t] = base[RAW_ARRAY + t * CH_N];
    }
}

// One thread: channel c of one side, block h of the step -> operand tiles.
template <typename IOE, typename OPE>
__device__ __forceinline__ void prep_block(const Raw &r, bool kside, int h, int c, unsigned char *ops, u32 &bad) {
    float gate[CH_L], pre[CH_L];
    u16 mx = 0;
#pragma unroll
    for (int t = 0; t < CH_L; ++t) {
        gate[t] = IOE::to_f32(r.g[t]);
        const u16 m1 = (u16)(r.g[t] - 1);     // gates must lie in (0, 1]: 0 < bits <= bits(1.0)
        mx = m1 > mx ? m1 : mx;
    }
    bad |= (mx >= IOE::ONE_BITS) ? 1u : 0u;
    pre[0] = gate[0];
#pragma unroll
    for (int t = 1; t < CH_L; ++t) pre[t] = pre[t - 1] * gate[t];
    const float pL = pre[CH_L - 1];
    bad |= (pL >= OPE::MIN_PRODUCT) ? 0u : 1u;
    const float ipL = __builtin_amdgcn_rcpf(pL);
    float hat[CH_L], til[CH_L];
    float sfx = 1.0f;
#pragma unroll
    for (int t = CH_L - 1; t >= 0; --t) {
        hat[t] = IOE::to_f32(r.a[t]) * sfx;      // scaled to the block end   (<= |a|)
        til[t] = hat[t] * ipL;                   // scaled to the block start (a / prefix)
        sfx *= gate[t];
    }
    const int tok0 = CH_L * h;
    if (kside) {
        u16 *QT = reinterpret_cast<u16 *>(ops + OFF_QT);
        u16 *KT = reinterpret_cast<u16 *>(ops + OFF_KT);
#pragma unroll
        for (int t = 0; t < CH_L; ++t) {
            QT[(tok0 + t) * TS + c] = cvt1<OPE>(IOE::to_f32(r.u[t]) * pre[t]);
            KT[(tok0 + t) * TS + c] = cvt1<OPE>(til[t]);
        }
        uint2 *KH = reinterpret_cast<uint2 *>(ops + OFF_KH + (c * CS + tok0) * 2);
#pragma unroll
        for (int t = 0; t < CH_L; t += 4)
            KH[t / 4] = make_uint2(OPE::pack2(hat[t], hat[t + 1]), OPE::pack2(hat[t + 2], hat[t + 3]));
        reinterpret_cast<float *>(ops + OFF_BL)[h * CH_N + c] = pL;
    } else {
        uint2 *XT = reinterpret_cast<uint2 *>(ops + OFF_XT + (c * CS + tok0) * 2);
        uint2 *XH = reinterpret_cast<uint2 *>(ops + OFF_XH + (c * CS + tok0) * 2);
        float4 *AS = reinterpret_cast<float4 *>(ops + OFF_AS + (c * CS + tok0) * 4);
#pragma unroll
        for (int t = 0; t < CH_L; t += 4) {
            XT[t / 4] = make_uint2(OPE::pack2(til[t], til[t + 1]), OPE::pack2(til[t + 2], til[t + 3]));
            XH[t / 4] = make_uint2(OPE::pack2(hat[t], hat[t + 1]), OPE::pack2(hat[t + 2], hat[t + 3]));
            AS[t / 4] = make_float4(pre[t], pre[t + 1], pre[t + 2], pre[t + 3]);
        }
        reinterpret_cast<float *>(ops + OFF_AL)[h * CH_N + c] = pL;
    }
}

template <typename E>
__device__ __forceinline__ uint2 pack4(const floatx4 &v) {
    return make_uint2(E::pack2(v[0], v[1]), E::pack2(v[2], v[3]));
}

// state slab of one wave <-> global [64][64] state of one row (16-bit I/O)
template <typename IOE>
__device__ __forceinline__ void store_state(const floatx4 (&S)[4], u16 *dst, int d, int g) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uint2 *>(dst + d * CH_N + 16 * j + 4 * g) = pack4<IOE>(S[j]);
}

// Workgroup = 8 waves.  Waves 0-3 ("matrix waves") own the state slabs and run the MFMA
// phase of step n; waves 4-7 ("prep waves") build the operand tiles of step n+1, prefetch
// raw inputs and write the previous step's outputs.  One barrier per step hands the
// double-buffered tiles over.
constexpr int FWD_THREADS = 512;

template <typename IOE, typename OPE>
__device__ __forceinline__ void fwd_prep_waves(const ChunkFwdArgs &p, unsigned char *smem, int tid, int64_t b) {
    const int h = tid >> 7, c = tid & 63;      // block of the step, channel
    const bool kside = ((tid >> 6) & 1) == 0;
    const int64_t T = p.T;
    const int64_t row_base = b * T;
    const u16 *const src[5] = {reinterpret_cast<const u16 *>(p.f_key), reinterpret_cast<const u16 *>(p.k),
                               reinterpret_cast<const u16 *>(p.q), reinterpret_cast<const u16 *>(p.f),
                               reinterpret_cast<const u16 *>(p.x)};
    u16 *out = reinterpret_cast<u16 *>(p.out);
    const int64_t nsteps = (T + CH_STEP - 1) / CH_STEP;
    u32 bad = 0;
    if (tid == 0) p.row_flags[b] = 0;

    // step m of the raw inputs lives in RAW[m & 1]; `st` carries the next step to be written
    Stage st;
    stage_load<IOE>(st, src, row_base, T, 0, tid);
    stage_store(st, smem + OFF_RAW, tid);
    if (nsteps > 1) {
        stage_load<IOE>(st, src, row_base, T, 1, tid);
        stage_store(st, smem + OFF_RAW + RAW_BYTES, tid);
    }
    if (nsteps > 2) stage_load<IOE>(st, src, row_base, T, 2, tid);
    __syncthreads();
    {
        Raw r;
        raw_read(r, smem + OFF_RAW, kside, h, c);
        prep_block<IOE, OPE>(r, kside, h, c, smem, bad);
    }
    __syncthreads();

    auto store_out = [&](int64_t step) {      // outputs of `step`: LDS tile -> global, 16 B per thread
        const u16 *OUTP = reinterpret_cast<const u16 *>(smem + OFF_OUT + (step & 1) * OUT_BYTES);
        const int tok = tid >> 3, piece = tid & 7;
        const int64_t t = step * CH_STEP + tok;
        if (t < T) {
            const uint2 lo = *reinterpret_cast<const uint2 *>(OUTP + tok * OS + 8 * piece);
            const uint2 hi = *reinterpret_cast<const uint2 *>(OUTP + tok * OS + 8 * piece + 4);
            *reinterpret_cast<uint4 *>(out + (row_base + t) * CH_N + 8 * piece) = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
    };
    PHASE_BEGIN();
    for (int64_t n = 0; n < nsteps; ++n) {
        Raw r;
        if (n + 1 < nsteps) raw_read(r, smem + OFF_RAW + ((n + 1) & 1) * RAW_BYTES, kside, h, c);
        if (n > 0) store_out(n - 1);
        PHASE_MARK(2);
        if (n + 2 < nsteps) stage_store(st, smem + OFF_RAW + (n & 1) * RAW_BYTES, tid);   // step n+2
        if (n + 3 < nsteps) stage_load<IOE>(st, src, row_base, T, n + 3, tid);
        PHASE_MARK(1);
        if (n + 1 < nsteps) prep_block<IOE, OPE>(r, kside, h, c, smem + ((n + 1) & 1) * OPS_BYTES, bad);
        PHASE_MARK(0);
        __syncthreads();
        PHASE_MARK(3);
    }
    store_out(nsteps - 1);
    if (bad) p.row_flags[b] = 1;
    PHASE_END(4 + (tid >> 6));
}

template <typename IOE, typename OPE>
__device__ __forceinline__ void fwd_matrix_waves(const ChunkFwdArgs &p, unsigned char *smem, int tid, int64_t b) {
    const int w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int d = 16 * w + r;                  // this lane's state column
    const int64_t T = p.T;
    u16 *ckpt = reinterpret_cast<u16 *>(p.ckpt);
    floatx4 S[4];
    {
        const u16 *s0 = reinterpret_cast<const u16 *>(p.s0) + b * (CH_N * CH_N);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint2 v = *reinterpret_cast<const uint2 *>(s0 + d * CH_N + 16 * j + 4 * g);
            S[j][0] = IOE::to_f32((u16)(v.x & 0xffff));
            S[j][1] = IOE::to_f32((u16)(v.x >> 16));
            S[j][2] = IOE::to_f32((u16)(v.y & 0xffff));
            S[j][3] = IOE::to_f32((u16)(v.y >> 16));
        }
    }
    const int64_t nsteps = (T + CH_STEP - 1) / CH_STEP;
    int until_ckpt = 0;
    int64_t chunk = 0;
    __syncthreads();      // raw inputs of the first steps are in LDS
    __syncthreads();      // operand tiles of step 0 are in LDS
    PHASE_BEGIN();
    for (int64_t n = 0; n < nsteps; ++n) {
        const unsigned char *ops = smem + (n & 1) * OPS_BYTES;
        u16 *OUT = reinterpret_cast<u16 *>(smem + OFF_OUT + (n & 1) * OUT_BYTES);
        const u16 *QT = reinterpret_cast<const u16 *>(ops + OFF_QT);
        const u16 *KT = reinterpret_cast<const u16 *>(ops + OFF_KT);
        const u16 *KH = reinterpret_cast<const u16 *>(ops + OFF_KH);
        const u16 *XT = reinterpret_cast<const u16 *>(ops + OFF_XT);
        const u16 *XH = reinterpret_cast<const u16 *>(ops + OFF_XH);
        const float *AS = reinterpret_cast<const float *>(ops + OFF_AS);
        const float *BL = reinterpret_cast<const float *>(ops + OFF_BL);
        const float *AL = reinterpret_cast<const float *>(ops + OFF_AL);
        if (ckpt != nullptr) {          // checkpoint interval is a multiple of the step
            if (until_ckpt == 0) {
                store_state<IOE>(S, ckpt + (b * p.NC + chunk) * (CH_N * CH_N), d, g);
                until_ckpt = p.C;
                ++chunk;
            }
            until_ckpt -= CH_STEP;
        }
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int tok0 = CH_L * hh;
            // P^T[s,t] = kt_s . qs_t, kept for s <= t, as the A operand of the intra product
            const u16 *krow = KT + (tok0 + r) * TS + 8 * g;
            const u16 *qrow = QT + (tok0 + r) * TS + 8 * g;
            floatx4 pt = {0.f, 0.f, 0.f, 0.f};
            pt = OPE::mfma32(*reinterpret_cast<const uint4 *>(krow), *reinterpret_cast<const uint4 *>(qrow), pt);
            pt = OPE::mfma32(*reinterpret_cast<const uint4 *>(krow + 32), *reinterpret_cast<const uint4 *>(qrow + 32), pt);
#pragma unroll
            for (int i = 0; i < 4; ++i) pt[i] = (4 * g + i <= r) ? pt[i] : 0.f;
            const uint2 pa = pack4<OPE>(pt);
            // o[t,d] = a_t[d] * ( sum_k qs_t[k] S0[d,k] + sum_{s<=t} P[t,s] xt_s[d] )
            const u16 *qperm = QT + (tok0 + r) * TS + 4 * g;
            const uint2 q0 = *reinterpret_cast<const uint2 *>(qperm);
            const uint2 q1 = *reinterpret_cast<const uint2 *>(qperm + 16);
            const uint2 q2 = *reinterpret_cast<const uint2 *>(qperm + 32);
            const uint2 q3 = *reinterpret_cast<const uint2 *>(qperm + 48);
            const uint2 s0p = pack4<OPE>(S[0]), s1p = pack4<OPE>(S[1]), s2p = pack4<OPE>(S[2]), s3p = pack4<OPE>(S[3]);
            floatx4 o = {0.f, 0.f, 0.f, 0.f};
            o = OPE::mfma32(make_uint4(q0.x, q0.y, q1.x, q1.y), make_uint4(s0p.x, s0p.y, s1p.x, s1p.y), o);
            o = OPE::mfma32(make_uint4(q2.x, q2.y, q3.x, q3.y), make_uint4(s2p.x, s2p.y, s3p.x, s3p.y), o);
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            const floatx4 oi = OPE::mfma16(pa, *reinterpret_cast<const uint2 *>(XT + d * CS + tok0 + 4 * g), zero);
            const float4 as = *reinterpret_cast<const float4 *>(AS + d * CS + tok0 + 4 * g);
            OUT[(tok0 + 4 * g + 0) * OS + d] = cvt1<IOE>((o[0] + oi[0]) * as.x);
            OUT[(tok0 + 4 * g + 1) * OS + d] = cvt1<IOE>((o[1] + oi[1]) * as.y);
            OUT[(tok0 + 4 * g + 2) * OS + d] = cvt1<IOE>((o[2] + oi[2]) * as.z);
            OUT[(tok0 + 4 * g + 3) * OS + d] = cvt1<IOE>((o[3] + oi[3]) * as.w);
            // S_L = (a_L (x) b_L) * S0 + sum_s xh_s (x) kh_s
            const float aL = AL[hh * CH_N + d];
            const uint2 xh = *reinterpret_cast<const uint2 *>(XH + d * CS + tok0 + 4 * g);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 bl = *reinterpret_cast<const float4 *>(BL + hh * CH_N + 16 * j + 4 * g);
                S[j][0] *= aL * bl.x;
                S[j][1] *= aL * bl.y;
                S[j][2] *= aL * bl.z;
                S[j][3] *= aL * bl.w;
                S[j] = OPE::mfma16(*reinterpret_cast<const uint2 *>(KH + (16 * j + r) * CS + tok0 + 4 * g), xh, S[j]);
            }
            PHASE_MARK(hh);
        }
        __syncthreads();
        PHASE_MARK(3);
    }
    store_state<IOE>(S, reinterpret_cast<u16 *>(p.next_state) + b * (CH_N * CH_N), d, g);
    PHASE_END(tid >> 6);
}

template <typename IOE, typename OPE>
__global__ __launch_bounds__(FWD_THREADS) void lfw_fwd_chunk_kernel(ChunkFwdArgs p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int64_t b = blockIdx.x;
    // both branches execute exactly 2 + nsteps workgroup barriers
    if (tid < 256)
        fwd_matrix_waves<IOE, OPE>(p, smem, tid, b);
    else
        fwd_prep_waves<IOE, OPE>(p, smem, tid - 256, b);
}

template <typename IOE, typename OPE> int launch(const ChunkFwdArgs &a, hipStream_t stream) {
    auto kern = lfw_fwd_chunk_kernel<IOE, OPE>;
    // more than 64 KB of dynamic LDS has to be enabled per function (and per device)
    int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, FWD_SMEM),
                       "hipFuncSetAttribute(forward chunk kernel)");
    if (rc) return rc;
    if (a.B > 0x7fffffffLL) return fail(T2FW_ERR_UNSUPPORTED, "B=%lld is too large", (long long)a.B);
    hipLaunchKernelGGL(kern, dim3((unsigned)a.B), dim3(FWD_THREADS), FWD_SMEM, stream, a);
    return check_hip(hipGetLastError(), "lfw_fwd_chunk_kernel launch");
}

}  // namespace

int chunk_forward(const ChunkFwdArgs &a, int dtype, int op, hipStream_t stream) {
    if (dtype == T2FW_F16) return op == 1 ? launch<Fp16, Fp16>(a, stream) : launch<Fp16, Bf16>(a, stream);
    if (dtype == T2FW_BF16) return launch<Bf16, Bf16>(a, stream);
    return fail(T2FW_ERR_UNSUPPORTED, "the chunked kernels take fp16 or bf16 tensors");
}

}  // namespace t2fw
