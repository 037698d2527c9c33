// C ABI of libt2fw_hip.so: argument validation and kernel-path selection.
// Declarations and the reference interfaces they replace: include/t2fw_hip.h.
#include "common.hpp"
#include "lfw_scan.hpp"
#include "lfw_chunk.hpp"
#include "lfw_par.hpp"
#include "dfw_scan.hpp"
#include "cast.hpp"
#include "gate.hpp"
#include "lfw_step.hpp"

#include <cstring>
#include <initializer_list>
#include <mutex>
#include <set>
#include <utility>

namespace t2fw {

namespace {
thread_local char g_err[512] = "";
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return T2FW_OK;
    return fail(T2FW_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int enable_lds(const void *kernel, int bytes, const char *what) {
    static std::mutex mu;
    static std::set<std::pair<const void *, int>> done;
    int dev = 0;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    std::lock_guard<std::mutex> lock(mu);
    if (done.count({kernel, dev})) return T2FW_OK;
    if ((rc = check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes), what))) return rc;
    done.insert({kernel, dev});
    return T2FW_OK;
}

namespace {

size_t elem_size(int dtype) {
    switch (dtype) {
        case T2FW_F32: return 4;
        case T2FW_F16: return 2;
        case T2FW_BF16: return 2;
        case T2FW_F64: return 8;
    }
    return 0;
}

struct NamedPtr {
    const char *name;
    const void *ptr;
};

int check_ptrs(const NamedPtr *v, int n, size_t es) {
    for (int i = 0; i < n; ++i) {
        if (v[i].ptr == nullptr) return fail(T2FW_ERR_NULL_POINTER, "%s is a null pointer", v[i].name);
        if (reinterpret_cast<uintptr_t>(v[i].ptr) % es != 0)
            return fail(T2FW_ERR_MISALIGNED, "%s is not aligned to the %zu-byte element size", v[i].name, es);
    }
    return T2FW_OK;
}

bool aligned16(std::initializer_list<const void *> ps) {
    for (const void *p : ps)
        if (p != nullptr && reinterpret_cast<uintptr_t>(p) % 16 != 0) return false;
    return true;
}

// The chunked matrix-core kernels cover D = K = 64 with 16-bit tensors.
bool chunk_shape_ok(int64_t D, int64_t K, int32_t dtype, int32_t flags) {
    return (flags & T2FW_FLAG_FORCE_SCAN) == 0 && D == 64 && K == 64 && (dtype == T2FW_F16 || dtype == T2FW_BF16);
}

// compute units of the current device (-1 on error)
int compute_units() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
    return n;
}

// Workspace of the matrix-core kernels:
//   [0, row_flag_bytes)                 flags of the block-wise kernels, two slots per batch row (kernels
//                                       that split a row over two workgroups use both)
//   [row_flag_bytes, 2 * row_flag_bytes)  flags of the chunk-parallel kernels, one slot per row
//   then, backward only (ParScratch): per-chunk flags [B * NC] int32, per-chunk gate products
//   [B, NC, PAR_NVEC, 64] fp32, adjoint entering every chunk [B, NC, 64, 64] bf16
size_t row_flag_bytes(int64_t B) { return (size_t)((2 * chunk_rows_padded(B) * 4 + 255) / 256 * 256); }

// The chunk-parallel kernels take checkpoint intervals 32 and 64, bf16 matrix-core operands and
// [B, T, 64] arrays of fewer than 2^31 elements (32-bit element offsets); anything else that the
// matrix cores can take runs block-wise.
bool par_ok(int64_t B, int64_t T, int32_t C, int32_t flags) {
    if ((C != 32 && C != 64) || (flags & (T2FW_FLAG_BLOCKWISE | T2FW_FLAG_FP16_OPERANDS)) != 0) return false;
    const long double elems = (long double)B * (long double)T * CH_N;
    return elems < 2147483647.0L && (long double)B * (long double)((T + C - 1) / C) <= (long double)0x3fffffff;
}

struct ParScratch {
    size_t chunk_flags, vecs, gh, total;       // byte offsets from the start of the workspace
};
ParScratch par_scratch(int64_t B, int64_t T, int32_t C) {
    const int64_t nc = (C < 1 || T <= 0) ? 1 : (T + C - 1) / C;
    const size_t items = (size_t)(B * nc);
    ParScratch s;
    s.chunk_flags = 2 * row_flag_bytes(B);
    s.vecs = s.chunk_flags + (items * 4 + 255) / 256 * 256;
    s.gh = s.vecs + items * (size_t)(PAR_NVEC * CH_N * 4);
    s.total = s.gh + items * (size_t)(CH_N * CH_N * 2);
    return s;
}

size_t forward_workspace_bytes(int64_t B, int64_t D, int64_t K, int32_t dtype, int32_t flags) {
    if (B > 0 && chunk_shape_ok(D, K, dtype, flags)) return 2 * row_flag_bytes(B);
    return 0;
}

// Checkpoint intervals that are a multiple of 32 other than 32 and 64 (the forward takes them, the backward
// kernels do not): the backward call first runs the forward kernel once more at an interval the backward takes,
// into checkpoints of its own in the workspace, and then proceeds as for that interval.
int32_t backward_interval(int32_t C) {
    if (C == 32 || C == 64 || C < 32 || C % 32 != 0) return C;
    return C % 64 == 0 ? 64 : 32;
}
size_t align256(size_t n) { return (n + 255) / 256 * 256; }

struct DenseScratch {
    size_t ckpt, out, next, total;      // byte offsets from the start of the workspace
};
DenseScratch dense_scratch(size_t inner, int64_t B, int64_t T, int32_t Cd, size_t es) {
    const int64_t nc = T <= 0 ? 1 : (T + Cd - 1) / Cd;
    DenseScratch d;
    d.ckpt = align256(inner);
    d.out = d.ckpt + align256((size_t)(B * nc) * CH_N * CH_N * es);
    d.next = d.out + align256((size_t)(B * (T > 0 ? T : 1)) * CH_N * es);
    d.total = d.next + align256((size_t)B * CH_N * CH_N * es);
    return d;
}

size_t backward_workspace_bytes(int64_t B, int64_t T, int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags) {
    if (B > 0 && chunk_shape_ok(D, K, dtype, flags)) {
        const int32_t Cd = backward_interval(C);
        const size_t inner = par_ok(B, T, Cd, flags) ? par_scratch(B, T, Cd).total : 2 * row_flag_bytes(B);
        return Cd == C ? inner : dense_scratch(inner, B, T, Cd, elem_size(dtype)).total;
    }
    return 0;
}

int check_dims(int64_t B, int64_t T, int64_t D, int64_t K) {
    if (B < 0 || T < 0) return fail(T2FW_ERR_BAD_SHAPE, "B=%lld and T=%lld must be non-negative", (long long)B, (long long)T);
    if (D < 1 || K < 1) return fail(T2FW_ERR_BAD_SHAPE, "D=%lld and K=%lld must be positive", (long long)D, (long long)K);
    // every tensor must be addressable with 63-bit element offsets
    const long double big = (long double)B * (long double)(T > 0 ? T : 1) * (long double)D * (long double)K;
    if (big > 4.0e18L) return fail(T2FW_ERR_BAD_SHAPE, "B*T*D*K is too large");
    return T2FW_OK;
}

}  // namespace
}  // namespace t2fw

using namespace t2fw;

// ---- forward scan for callers that cannot allocate -------------------------------------------
// The scratch of t2fw_lfw_forward (the row flags of the matrix-core kernels) lives in a file-scope
// device array instead of a caller's workspace.  Every GPU holds its own copy of the array at its
// own address; the array's name is only a host-side handle, so the address is looked up once per
// device with hipGetSymbolAddress and only that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[T2FW_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[MAX_DEVICES] = {};

// device address of `scratch` on the current device (looked up on the first call per device)
int static_scratch(void **out) {
    int dev = -1;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    if (dev < 0 || dev >= MAX_DEVICES) return fail(T2FW_ERR_UNSUPPORTED, "device ordinal %d is out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
        if (rc) return rc;
        if (ptr == nullptr) return fail(T2FW_ERR_HIP, "hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return T2FW_OK;
}
}  // namespace

extern "C" {

int t2fw_abi_version(void) { return T2FW_ABI_VERSION; }

const char *t2fw_last_error(void) { return g_err; }

int64_t t2fw_lfw_num_ckpt(int64_t T, int32_t C) {
    if (C < 1 || T <= 0) return 1;
    return (T + C - 1) / C;
}

size_t t2fw_lfw_workspace_bytes(int64_t B, int64_t T, int64_t D, int64_t K, int32_t C, int32_t dtype,
                                int32_t flags) {
    const size_t fwd = forward_workspace_bytes(B, D, K, dtype, flags);
    const size_t bwd = backward_workspace_bytes(B, T, D, K, C, dtype, flags);
    return fwd > bwd ? fwd : bwd;
}

size_t t2fw_lfw_forward_workspace_bytes(int64_t B, int64_t T, int64_t D, int64_t K, int32_t C, int32_t dtype,
                                        int32_t flags) {
    (void)T; (void)C;
    return forward_workspace_bytes(B, D, K, dtype, flags);
}

int t2fw_host_workspace_device_pointer(void *host_workspace, void **device_pointer) {
    if (host_workspace == nullptr || device_pointer == nullptr) return fail(T2FW_ERR_NULL_POINTER, "null pointer");
    *device_pointer = nullptr;
    return check_hip(hipHostGetDevicePointer(device_pointer, host_workspace, 0), "hipHostGetDevicePointer");
}

int t2fw_lfw_flag_regions(int64_t B, int64_t T, int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags,
                          int64_t *regions) {
    if (regions == nullptr) return fail(T2FW_ERR_NULL_POINTER, "regions is a null pointer");
    for (int i = 0; i < 6; ++i) regions[i] = 0;
    if (elem_size(dtype) == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    const int rc = check_dims(B, T, D, K);
    if (rc) return rc;
    if (B == 0 || !chunk_shape_ok(D, K, dtype, flags)) return T2FW_OK;       // exact kernels: no flags
    const int64_t slots = 2 * chunk_rows_padded(B), region = (int64_t)row_flag_bytes(B);
    regions[0] = 0; regions[1] = slots;                  // forward verdicts
    regions[2] = region; regions[3] = slots;             // forward hints for the backward
    const int32_t Cd = backward_interval(C);
    if (Cd == 32 || Cd == 64) {                          // else the backward runs on the exact kernels
        if (par_ok(B, T, Cd, flags)) {
            regions[4] = region; regions[5] = B;
        } else {
            regions[4] = 0; regions[5] = slots;
        }
    }
    return T2FW_OK;
}

// B batch rows; heads = 1: rows are contiguous [T, D|K] slabs, heads = H > 1: row b is head b % H of
// [B / H, T, H, D|K] tensors (x, f, q, k, f_key, out); states and checkpoints are per row either way
static int lfw_forward_rows(const void *x, const void *f, const void *q, const void *k, const void *f_key,
                            const void *s0, void *out, void *next_state, void *ckpt, int64_t B, int64_t T,
                            int64_t heads, int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags,
                            void *workspace, size_t workspace_bytes, void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    int rc = check_dims(B, T, D, K);
    if (rc) return rc;
    if (ckpt != nullptr && C < 1) return fail(T2FW_ERR_BAD_SHAPE, "checkpoint interval C=%d must be >= 1", C);
    if (B == 0) return T2FW_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    {
        const NamedPtr sp[] = {{"s0", s0}, {"next_state", next_state}};
        if ((rc = check_ptrs(sp, 2, es))) return rc;
        if (ckpt != nullptr && reinterpret_cast<uintptr_t>(ckpt) % es != 0)
            return fail(T2FW_ERR_MISALIGNED, "ckpt is not aligned to the %zu-byte element size", es);
    }
    if (T == 0) {   // no steps: the state passes through
        const size_t bytes = (size_t)(B * D * K) * es;
        if (next_state != s0 &&
            (rc = check_hip(hipMemcpyAsync(next_state, s0, bytes, hipMemcpyDeviceToDevice, st), "state copy")))
            return rc;
        if (ckpt != nullptr &&
            (rc = check_hip(hipMemcpyAsync(ckpt, s0, bytes, hipMemcpyDeviceToDevice, st), "checkpoint copy")))
            return rc;
        return T2FW_OK;
    }
    const NamedPtr ptrs[] = {{"x", x}, {"f", f}, {"q", q}, {"k", k}, {"f_key", f_key}, {"out", out}};
    if ((rc = check_ptrs(ptrs, 6, es))) return rc;

    ScanFwdArgs a{};
    a.x = x; a.f = f; a.q = q; a.k = k; a.f_key = f_key; a.s0 = s0;
    a.out = out; a.next_state = next_state; a.ckpt = ckpt;
    a.B = B; a.T = T; a.D = D; a.K = K;
    a.heads = (int32_t)heads;
    a.C = ckpt ? C : 1;
    a.NC = ckpt ? t2fw_lfw_num_ckpt(T, C) : 1;

    if (chunk_shape_ok(D, K, dtype, flags) && (ckpt == nullptr || C % 32 == 0) && T * heads < CHUNK_MAX_T &&
        aligned16({x, f, q, k, f_key, s0, out, next_state, ckpt})) {
        const size_t need = forward_workspace_bytes(B, D, K, dtype, flags);
        if (workspace == nullptr || workspace_bytes < need)
            return fail(T2FW_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        if (!aligned16({workspace})) return fail(T2FW_ERR_MISALIGNED, "the workspace must be 16-byte aligned");
        ChunkFwdArgs c{};
        c.x = x; c.f = f; c.q = q; c.k = k; c.f_key = f_key; c.s0 = s0;
        c.out = out; c.next_state = next_state; c.ckpt = ckpt;
        c.row_flags = static_cast<int32_t *>(workspace);
        c.par_hint = reinterpret_cast<int32_t *>(static_cast<unsigned char *>(workspace) + row_flag_bytes(B));
        c.B = B; c.T = T; c.NC = a.NC; c.C = a.C;
        c.heads = (int32_t)heads;
        c.redo = (flags & T2FW_FLAG_NO_FIXUP) ? 0 : 1;       // flagged rows are redone inside the kernel
        const int op = (dtype == T2FW_F16 && (flags & T2FW_FLAG_FP16_OPERANDS)) ? 1 : 0;
        // two workgroups per batch row while that still fits the device in one wave of workgroups
        const int cus = compute_units();
        if (cus < 0) return fail(T2FW_ERR_HIP, "could not read the device's compute-unit count");
        const bool split = 2 * chunk_rows_padded(B) <= cus;
        return chunk_forward(c, dtype, op, split, st);
    }
    return scan_forward(a, dtype, st);
}

static int check_heads(int64_t B, int64_t H) {
    if (B < 0 || H < 1 || H > 65536) return fail(T2FW_ERR_BAD_SHAPE, "B=%lld must be non-negative and H=%lld in [1, 65536]", (long long)B, (long long)H);
    if ((long double)B * (long double)H > 4.0e18L) return fail(T2FW_ERR_BAD_SHAPE, "B*H is too large");
    return T2FW_OK;
}

int t2fw_lfw_forward(const void *x, const void *f, const void *q, const void *k, const void *f_key,
                     const void *s0, void *out, void *next_state, void *ckpt, int64_t B, int64_t T,
                     int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags, void *workspace,
                     size_t workspace_bytes, void *stream) {
    return lfw_forward_rows(x, f, q, k, f_key, s0, out, next_state, ckpt, B, T, 1, D, K, C, dtype, flags, workspace,
                            workspace_bytes, stream);
}

int t2fw_static_init(void) {
    void *ws = nullptr;
    return static_scratch(&ws);
}

int t2fw_lfw_forward_static(const void *x, const void *f, const void *q, const void *k, const void *f_key,
                            const void *s0, void *out, void *next_state, void *ckpt, int64_t B, int64_t T,
                            int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags, void *stream) {
    const size_t need = t2fw_lfw_forward_workspace_bytes(B, T, D, K, C, dtype, flags);
    if (need > (size_t)T2FW_STATIC_SCRATCH_BYTES)
        return fail(T2FW_ERR_WORKSPACE,
                    "t2fw_lfw_forward_static: this shape needs %zu bytes of scratch, the built-in buffer holds %d "
                    "(use t2fw_lfw_forward with a workspace)", need, T2FW_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (need > 0) {
        const int rc = static_scratch(&ws);
        if (rc) return rc;
    }
    // the kernels clear the flags of the rows they work on themselves, so what an earlier call left
    // in the buffer does not matter
    return lfw_forward_rows(x, f, q, k, f_key, s0, out, next_state, ckpt, B, T, 1, D, K, C, dtype, flags, ws, need, stream);
}

int t2fw_lfw_forward_heads(const void *x, const void *f, const void *q, const void *k, const void *f_key,
                           const void *s0, void *out, void *next_state, void *ckpt, int64_t B, int64_t T,
                           int64_t H, int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags,
                           void *workspace, size_t workspace_bytes, void *stream) {
    const int rc = check_heads(B, H);
    if (rc) return rc;
    return lfw_forward_rows(x, f, q, k, f_key, s0, out, next_state, ckpt, B * H, T, H, D, K, C, dtype, flags, workspace,
                            workspace_bytes, stream);
}

static int lfw_backward_rows(const void *g_out, const void *g_state, const void *x, const void *f, const void *q,
                             const void *k, const void *f_key, const void *s0, const void *ckpt, void *d_x, void *d_f,
                             void *d_q, void *d_k, void *d_f_key, void *d_s0, int64_t B, int64_t T, int64_t heads,
                             int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags, void *workspace,
                             size_t workspace_bytes, void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    int rc = check_dims(B, T, D, K);
    if (rc) return rc;
    if (C < 1) return fail(T2FW_ERR_BAD_SHAPE, "checkpoint interval C=%d must be >= 1", C);
    if (B == 0) return T2FW_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    {
        const NamedPtr sp[] = {{"g_state", g_state}, {"d_s0", d_s0}};
        if ((rc = check_ptrs(sp, 2, es))) return rc;
    }
    if (T == 0) {
        if (d_s0 != g_state)
            return check_hip(hipMemcpyAsync(d_s0, g_state, (size_t)(B * D * K) * es, hipMemcpyDeviceToDevice, st),
                             "state-gradient copy");
        return T2FW_OK;
    }
    const NamedPtr ptrs[] = {{"g_out", g_out}, {"x", x}, {"f", f}, {"q", q}, {"k", k}, {"f_key", f_key},
                             {"ckpt", ckpt}, {"d_x", d_x}, {"d_f", d_f}, {"d_q", d_q}, {"d_k", d_k},
                             {"d_f_key", d_f_key}};
    if ((rc = check_ptrs(ptrs, 12, es))) return rc;

    ScanBwdArgs a{};
    a.g_out = g_out; a.g_state = g_state; a.x = x; a.f = f; a.q = q; a.k = k; a.f_key = f_key; a.ckpt = ckpt;
    a.d_x = d_x; a.d_f = d_f; a.d_q = d_q; a.d_k = d_k; a.d_f_key = d_f_key; a.d_s0 = d_s0;
    a.B = B; a.T = T; a.D = D; a.K = K; a.C = C;
    a.heads = (int32_t)heads;
    a.NC = t2fw_lfw_num_ckpt(T, C);

    const int32_t C_given = C;
    C = backward_interval(C);
    if (chunk_shape_ok(D, K, dtype, flags) && (C == 32 || C == 64) && T * heads < CHUNK_MAX_T &&
        aligned16({g_out, g_state, x, f, q, k, f_key, ckpt, d_x, d_f, d_q, d_k, d_f_key, d_s0}) &&
        (C == C_given || (s0 != nullptr && aligned16({s0})))) {
        const size_t need = backward_workspace_bytes(B, T, D, K, C_given, dtype, flags);
        if (workspace == nullptr || workspace_bytes < need)
            return fail(T2FW_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        if (!aligned16({workspace})) return fail(T2FW_ERR_MISALIGNED, "the workspace must be 16-byte aligned");
        a.C = C;
        a.NC = t2fw_lfw_num_ckpt(T, C);
        if (C != C_given) {
            // checkpoints at the interval the backward kernels take: the forward kernel once more, from s0
            const size_t inner = par_ok(B, T, C, flags) ? par_scratch(B, T, C).total : 2 * row_flag_bytes(B);
            const DenseScratch ds = dense_scratch(inner, B, T, C, es);
            unsigned char *const ws = static_cast<unsigned char *>(workspace);
            rc = lfw_forward_rows(x, f, q, k, f_key, s0, ws + ds.out, ws + ds.next, ws + ds.ckpt, B, T, heads, D, K, C,
                                  dtype, flags & T2FW_FLAG_FP16_OPERANDS, workspace, inner, stream);
            if (rc) return rc;
            ckpt = ws + ds.ckpt;
        }
        ChunkBwdArgs c{};
        c.g_out = g_out; c.g_state = g_state; c.x = x; c.f = f; c.q = q; c.k = k; c.f_key = f_key; c.ckpt = ckpt;
        c.d_x = d_x; c.d_f = d_f; c.d_q = d_q; c.d_k = d_k; c.d_f_key = d_f_key; c.d_s0 = d_s0;
        c.row_flags = static_cast<int32_t *>(workspace);
        c.row_select = nullptr;
        c.B = B; c.T = T; c.NC = a.NC; c.C = C;
        c.heads = (int32_t)heads;
        if (par_ok(B, T, C, flags)) {
            // chunk-parallel kernels
            ParBwdArgs pa{};
            pa.g_out = g_out; pa.g_state = g_state; pa.x = x; pa.f = f; pa.q = q; pa.k = k; pa.f_key = f_key; pa.ckpt = ckpt;
            pa.d_x = d_x; pa.d_f = d_f; pa.d_q = d_q; pa.d_k = d_k; pa.d_f_key = d_f_key; pa.d_s0 = d_s0;
            unsigned char *const ws = static_cast<unsigned char *>(workspace);
            const ParScratch sc = par_scratch(B, T, C);
            pa.row_flags = reinterpret_cast<int32_t *>(ws + row_flag_bytes(B));
            pa.chunk_flags = reinterpret_cast<int32_t *>(ws + sc.chunk_flags);
            pa.vecs = reinterpret_cast<float *>(ws + sc.vecs);
            pa.gh = ws + sc.gh;
            pa.B = B; pa.T = T; pa.NC = a.NC; pa.C = C;
            pa.heads = (int32_t)heads;
            if ((rc = par_backward(pa, dtype, st))) return rc;
            if (flags & T2FW_FLAG_NO_FIXUP) return T2FW_OK;
            // The rows it declined go to the block-wise kernel (16-step products instead of products over
            // half a chunk), which redoes with the exact scan, inside the kernel, what it cannot take
            // either.  Every other workgroup of that launch reads its row's flag and leaves.
            c.row_select = pa.row_flags;
            c.redo = 1;
            return chunk_backward(c, dtype, 0, st);
        }
        const int op = (dtype == T2FW_F16 && (flags & T2FW_FLAG_FP16_OPERANDS)) ? 1 : 0;
        c.redo = (flags & T2FW_FLAG_NO_FIXUP) ? 0 : 1;
        return chunk_backward(c, dtype, op, st);
    }
    a.C = C_given;
    a.NC = t2fw_lfw_num_ckpt(T, C_given);
    return scan_backward(a, dtype, st);
}

int t2fw_lfw_backward(const void *g_out, const void *g_state, const void *x, const void *f, const void *q,
                      const void *k, const void *f_key, const void *s0, const void *ckpt, void *d_x,
                      void *d_f, void *d_q, void *d_k, void *d_f_key, void *d_s0, int64_t B, int64_t T,
                      int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags, void *workspace,
                      size_t workspace_bytes, void *stream) {
    return lfw_backward_rows(g_out, g_state, x, f, q, k, f_key, s0, ckpt, d_x, d_f, d_q, d_k, d_f_key, d_s0, B, T, 1, D, K, C,
                             dtype, flags, workspace, workspace_bytes, stream);
}

int t2fw_lfw_backward_heads(const void *g_out, const void *g_state, const void *x, const void *f, const void *q,
                            const void *k, const void *f_key, const void *s0, const void *ckpt, void *d_x, void *d_f,
                            void *d_q, void *d_k, void *d_f_key, void *d_s0, int64_t B, int64_t T, int64_t H,
                            int64_t D, int64_t K, int32_t C, int32_t dtype, int32_t flags, void *workspace,
                            size_t workspace_bytes, void *stream) {
    const int rc = check_heads(B, H);
    if (rc) return rc;
    return lfw_backward_rows(g_out, g_state, x, f, q, k, f_key, s0, ckpt, d_x, d_f, d_q, d_k, d_f_key, d_s0, B * H, T, H, D, K,
                             C, dtype, flags, workspace, workspace_bytes, stream);
}

int t2fw_lfw_step(const void *x, const void *f, const void *q, const void *k, const void *f_key, const void *s0,
                  void *out, void *next_state, int64_t B, int64_t D, int64_t K, int32_t dtype, void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    int rc = check_dims(B, 1, D, K);
    if (rc) return rc;
    if (B == 0) return T2FW_OK;
    const NamedPtr ptrs[] = {{"x", x}, {"f", f}, {"q", q}, {"k", k}, {"f_key", f_key}, {"s0", s0}, {"out", out},
                             {"next_state", next_state}};
    if ((rc = check_ptrs(ptrs, 8, es))) return rc;
    if (D == 64 && K == 64 && (dtype == T2FW_F16 || dtype == T2FW_BF16) &&
        aligned16({x, f, q, k, f_key, s0, out, next_state})) {
        StepArgs a{};
        a.x = x; a.f = f; a.q = q; a.k = k; a.f_key = f_key; a.s0 = s0; a.out = out; a.next_state = next_state;
        a.B = B;
        return step_forward(a, dtype, static_cast<hipStream_t>(stream));
    }
    // general shapes: the exact scan kernel with T = 1 (each lane reads its state elements before
    // it writes them, so updating in place is safe there too)
    return t2fw_lfw_forward(x, f, q, k, f_key, s0, out, next_state, nullptr, B, 1, D, K, 1, dtype,
                            T2FW_FLAG_FORCE_SCAN, nullptr, 0, stream);
}

// The block-wise matrix-core kernels of the delta rule cover D = M = 64 with fp32, fp16 and bf16 tensors.
static bool dfw_chunk_ok(int64_t D, int64_t M, int32_t dtype, int32_t flags) {
    return (flags & T2FW_FLAG_FORCE_SCAN) == 0 && D == 64 && M == 64 &&
           (dtype == T2FW_F32 || dtype == T2FW_F16 || dtype == T2FW_BF16);
}

int t2fw_dfw_forward(const void *q, const void *k, const void *v, const void *s0, void *out, void *final_state,
                     void *delta, int64_t B, int64_t T, int64_t D, int64_t M, int32_t dtype, int32_t flags,
                     void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    int rc = check_dims(B, T, D, M);
    if (rc) return rc;
    if (B == 0) return T2FW_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    {
        const NamedPtr sp[] = {{"s0", s0}, {"final_state", final_state}};
        if ((rc = check_ptrs(sp, 2, es))) return rc;
    }
    if (T == 0) {
        if (final_state != s0)
            return check_hip(hipMemcpyAsync(final_state, s0, (size_t)(B * D * M) * es, hipMemcpyDeviceToDevice, st),
                             "state copy");
        return T2FW_OK;
    }
    const NamedPtr ptrs[] = {{"q", q}, {"k", k}, {"v", v}, {"out", out}, {"delta", delta}};
    if ((rc = check_ptrs(ptrs, 5, es))) return rc;
    DfwFwdArgs a{};
    a.q = q; a.k = k; a.v = v; a.s0 = s0; a.out = out; a.final_state = final_state; a.delta = delta;
    a.B = B; a.T = T; a.D = D; a.M = M;
    if (dfw_chunk_ok(D, M, dtype, flags) && T * CH_N < 0x7fffffffLL && aligned16({q, k, v, s0, out, final_state, delta}))
        return dfw_chunk_forward(a, dtype, (flags & T2FW_FLAG_BF16_OPERANDS) == 0, st);
    return dfw_forward(a, dtype, st);
}

int t2fw_dfw_backward(const void *g_out, const void *g_state, const void *q, const void *k, const void *delta,
                      const void *final_state, void *d_q, void *d_k, void *d_v, void *d_s0, int64_t B, int64_t T,
                      int64_t D, int64_t M, int32_t dtype, int32_t flags, void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    int rc = check_dims(B, T, D, M);
    if (rc) return rc;
    if (B == 0) return T2FW_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    {
        const NamedPtr sp[] = {{"g_state", g_state}, {"d_s0", d_s0}};
        if ((rc = check_ptrs(sp, 2, es))) return rc;
    }
    if (T == 0) {
        if (d_s0 != g_state)
            return check_hip(hipMemcpyAsync(d_s0, g_state, (size_t)(B * D * M) * es, hipMemcpyDeviceToDevice, st),
                             "state-gradient copy");
        return T2FW_OK;
    }
    const NamedPtr ptrs[] = {{"g_out", g_out}, {"q", q}, {"k", k}, {"delta", delta}, {"final_state", final_state},
                             {"d_q", d_q}, {"d_k", d_k}, {"d_v", d_v}};
    if ((rc = check_ptrs(ptrs, 8, es))) return rc;
    DfwBwdArgs a{};
    a.g_out = g_out; a.g_state = g_state; a.q = q; a.k = k; a.delta = delta; a.final_state = final_state;
    a.d_q = d_q; a.d_k = d_k; a.d_v = d_v; a.d_s0 = d_s0;
    a.B = B; a.T = T; a.D = D; a.M = M;
    if (dfw_chunk_ok(D, M, dtype, flags) && T * CH_N < 0x7fffffffLL &&
        aligned16({g_out, g_state, q, k, delta, final_state, d_q, d_k, d_v, d_s0}))
        return dfw_chunk_backward(a, dtype, (flags & T2FW_FLAG_BF16_OPERANDS) == 0, st);
    return dfw_backward(a, dtype, st);
}

int t2fw_cast(const void *const *src, void *const *dst, const int64_t *n, int32_t count, int32_t src_dtype,
              int32_t dst_dtype, void *stream) {
    if (count < 0 || count > CAST_MAX_TENSORS) return fail(T2FW_ERR_BAD_SHAPE, "t2fw_cast takes 0 to %d arrays, got %d", CAST_MAX_TENSORS, count);
    if (count > 0 && (src == nullptr || dst == nullptr || n == nullptr)) return fail(T2FW_ERR_NULL_POINTER, "null pointer list");
    CastArgs a{};
    a.count = count;
    for (int i = 0; i < count; ++i) {
        if (n[i] < 0) return fail(T2FW_ERR_BAD_SHAPE, "element counts must be non-negative");
        if (n[i] > 0 && (src[i] == nullptr || dst[i] == nullptr)) return fail(T2FW_ERR_NULL_POINTER, "null array pointer");
        if (!aligned16({src[i], dst[i]})) return fail(T2FW_ERR_MISALIGNED, "arrays must be 16-byte aligned");
        a.src[i] = src[i]; a.dst[i] = dst[i]; a.n[i] = n[i];
    }
    return cast_tensors(a, src_dtype, dst_dtype, static_cast<hipStream_t>(stream));
}

int t2fw_gate_forward(const void *f_logit, const void *fk_logit, void *f, void *f_key, int64_t n_f, int64_t n_fk,
                      int32_t dtype, void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    if (n_f < 0 || n_fk < 0) return fail(T2FW_ERR_BAD_SHAPE, "element counts must be non-negative");
    if ((n_f > 0 && (f_logit == nullptr || f == nullptr)) || (n_fk > 0 && (fk_logit == nullptr || f_key == nullptr)))
        return fail(T2FW_ERR_NULL_POINTER, "null gate pointer");
    if (!aligned16({f_logit, fk_logit, f, f_key})) return fail(T2FW_ERR_MISALIGNED, "gate arrays must be 16-byte aligned");
    GateFwdArgs a{};
    a.f_logit = f_logit; a.fk_logit = fk_logit; a.f = f; a.f_key = f_key; a.n_f = n_f; a.n_fk = n_fk;
    return gate_forward(a, dtype, static_cast<hipStream_t>(stream));
}

int t2fw_gate_backward(const void *d_f, const void *d_f_key, const void *f, const void *f_key, void *d_f_logit,
                       void *d_fk_logit, int64_t n_f, int64_t n_fk, int32_t dtype, void *stream) {
    const size_t es = elem_size(dtype);
    if (es == 0) return fail(T2FW_ERR_BAD_DTYPE, "unknown dtype code %d", dtype);
    if (n_f < 0 || n_fk < 0) return fail(T2FW_ERR_BAD_SHAPE, "element counts must be non-negative");
    if ((n_f > 0 && (d_f == nullptr || f == nullptr || d_f_logit == nullptr)) ||
        (n_fk > 0 && (d_f_key == nullptr || f_key == nullptr || d_fk_logit == nullptr)))
        return fail(T2FW_ERR_NULL_POINTER, "null gate pointer");
    if (!aligned16({d_f, d_f_key, f, f_key, d_f_logit, d_fk_logit}))
        return fail(T2FW_ERR_MISALIGNED, "gate arrays must be 16-byte aligned");
    GateBwdArgs a{};
    a.d_f = d_f; a.d_f_key = d_f_key; a.f = f; a.f_key = f_key; a.d_f_logit = d_f_logit; a.d_fk_logit = d_fk_logit;
    a.n_f = n_f; a.n_fk = n_fk;
    return gate_backward(a, dtype, static_cast<hipStream_t>(stream));
}

}  // extern "C"
