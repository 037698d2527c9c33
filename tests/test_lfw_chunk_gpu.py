"""GPU parity of the chunked matrix-core LFW kernels (D = K = 64, fp16 / bf16 tensors)
against the CPU oracle, through the C ABI: headline shapes, ragged lengths, both checkpoint
intervals, gate regimes that stress the 16-step products, rows that must fall back to the
exact scan kernels, and size-independent properties at the benchmark's full size."""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs, make_reference_test_inputs
from tests.test_lfw_gpu import TOL, TOL_CHUNK, TOL_CHUNK_GATE, assert_close, gate_grad_floor

pytestmark = pytest.mark.gpu
NAMES = ("d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state")


def flagged_rows(ws, B, chunk_parallel=False):
    """Rows the matrix-core kernels handed to the exact kernels.  The block-wise kernels keep two
    flag slots per row at the start of the workspace (kernels that split a row over two workgroups
    report per workgroup), the second at the batch padded to 8; the chunk-parallel backward keeps
    one slot per row in the 256-byte-aligned region after them."""
    f = ws.view(torch.int32)
    pad = (B + 7) // 8 * 8
    if chunk_parallel:
        base = (2 * pad * 4 + 255) // 256 * 256 // 4
        return int((f[base:base + B] != 0).sum())
    return int(((f[:B] != 0) | (f[pad:pad + B] != 0)).sum())


class Flagged(tuple):
    """(rows flagged by the forward, rows flagged by the backward's first kernel); ``exact`` = rows the
    backward handed on to the exact scan (for the chunk-parallel backward: rows that the block-wise kernel,
    which takes what it declines, declined as well)"""
    def __new__(cls, fwd, bwd, exact):
        obj = super().__new__(cls, (fwd, bwd))
        obj.exact = exact
        return obj


def chunk_parallel_backward(C, flags):
    """the backward runs the chunk-parallel kernels unless a flag asks for the block-wise ones"""
    from t2fw_amd import _lib
    return C >= 32 and C % 32 == 0 and not flags & (_lib.FLAG_BLOCKWISE | 2 | 1)


def run_abi(inputs, go, gs, C, flags=0, with_backward=True):
    """forward (+ backward) through the C ABI; returns out, next_state, ckpt, grads, flagged rows"""
    from t2fw_amd import _lib
    lib = _lib.load()
    ins = [t.cuda() for t in inputs]
    x = ins[0]
    B, T, D = x.shape
    K = ins[2].shape[2]
    code = _lib.DTYPE_CODE[x.dtype]
    out, nxt = torch.empty_like(x), torch.empty_like(ins[5])
    nc = lib.t2fw_lfw_num_ckpt(T, C)
    ckpt = torch.empty(B, nc, D, K, dtype=x.dtype, device="cuda")
    wsb = lib.t2fw_lfw_workspace_bytes(B, T, D, K, C, code, flags)
    ws = torch.zeros(max(wsb, 256), dtype=torch.uint8, device="cuda")
    st = _lib.current_stream_handle(x.device)
    _lib.check(lib.t2fw_lfw_forward(*[_lib.ptr(t) for t in ins], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt),
                                    B, T, D, K, C, code, flags, _lib.ptr(ws), wsb, st))
    torch.cuda.synchronize()
    flagged_fwd = flagged_rows(ws, B) if wsb else 0
    grads, flagged_bwd, exact_bwd = None, 0, 0
    if with_backward:
        grads = [torch.empty_like(t) for t in ins]
        go_d, gs_d = go.cuda(), gs.cuda()      # keep the device copies alive across the launch
        _lib.check(lib.t2fw_lfw_backward(_lib.ptr(go_d), _lib.ptr(gs_d), *[_lib.ptr(t) for t in ins],
                                         _lib.ptr(ckpt), *[_lib.ptr(t) for t in grads], B, T, D, K, C, code, flags,
                                         _lib.ptr(ws), wsb, st))
        torch.cuda.synchronize()
        flagged_bwd = flagged_rows(ws, B, chunk_parallel_backward(C, flags)) if wsb else 0
        exact_bwd = flagged_rows(ws, B) if wsb else 0
    return out, nxt, ckpt, grads, Flagged(flagged_fwd, flagged_bwd, exact_bwd)


def assert_within_reference_bounds(out, r_out, grads, r_grads):
    """The tolerances of the reference's own fp16 test (tests/test_lfw.py:65,92), the outer bound.
    The reference computes in fp32 and asserts these on its own shape grid (no 64 x 64 state, at
    most 64 steps).  The matrix-core kernels round the contraction operands to bf16: their error is
    a fraction of max|ref| (the chunk tolerance), which passes atol = 1e-2 on near-zero elements only
    while max|ref| stays below about 3; tests whose outputs grow larger opt out and say so."""
    assert torch.allclose(out.double().cpu(), torch.as_tensor(r_out).double(), atol=1e-2, rtol=1e-1)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert torch.allclose(g.double().cpu(), torch.as_tensor(r).double(), atol=0.1, rtol=1e-1), n


def check_against_oracle(inputs, go, gs, C, dtype, flags=0, expect_flagged=None, tol=None, gate_tol=None,
                         reference_bounds=True, expect_flagged_parallel=None):
    """Forward and backward against the fp64 oracle.  Where the chunk-parallel backward applies, the
    block-wise backward (flag 8) is checked on the same inputs as well."""
    from t2fw_amd import _lib
    r_out, r_nxt = c_oracle.lfw_forward(*inputs)
    r_grads = c_oracle.lfw_backward(go, gs, *inputs)
    tol = tol or TOL_CHUNK
    gate_tol = gate_tol or TOL_CHUNK_GATE
    floors = gate_grad_floor(inputs, go, r_out, r_grads)
    variants = [flags] + ([flags | _lib.FLAG_BLOCKWISE] if chunk_parallel_backward(C, flags) else [])
    first = None
    for fl in variants:
        tag = " (flags %d)" % fl
        out, nxt, ckpt, grads, flagged = run_abi(inputs, go, gs, C, fl)
        if expect_flagged is not None:
            want = (expect_flagged, expect_flagged)
            if expect_flagged_parallel is not None and chunk_parallel_backward(C, fl):
                want = (expect_flagged, expect_flagged_parallel)     # the two backward forms accept different gate ranges
            assert flagged == want, (flagged, fl)
        assert_close(out, r_out, dtype, "outputs" + tag, tol=tol)
        assert_close(nxt, r_nxt, dtype, "next_state" + tag, tol=tol)
        for n, g, r in zip(NAMES, grads, r_grads):
            assert_close(g, r, dtype, n + tag, tol=gate_tol if n in ("d_f", "d_f_key") else tol,
                         floor=floors.get(n, 0.0))
        if dtype == torch.float16 and reference_bounds:
            assert_within_reference_bounds(out, r_out, grads, r_grads)
        first = first or (out, nxt, ckpt, grads)
    return first


@pytest.mark.parametrize("dtype,gate_mean,state_std", [(torch.float16, 2.0, 0.0), (torch.bfloat16, 3.0, 0.1)])
@pytest.mark.parametrize("B,T,C", [(4, 1024, 64), (3, 1000, 64), (2, 77, 32), (5, 1, 64), (2, 16, 64),
                                   (2, 33, 64), (1, 130, 32), (2, 96, 32)])
def test_config_like_inputs(dtype, gate_mean, state_std, B, T, C):
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, dtype, seed=T, gate_mean=gate_mean,
                                                    state_std=state_std)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, dtype, expect_flagged=0)


@pytest.mark.parametrize("dtype,B,T,C", [(torch.bfloat16, 3, 112, 64), (torch.float16, 2, 48, 32),
                                         (torch.float16, 3, 16, 64), (torch.bfloat16, 2, 80, 64),
                                         (torch.float16, 2, 77, 32), (torch.float16, 3, 15, 64),
                                         (torch.bfloat16, 2, 65, 64), (torch.float16, 2, 113, 64),
                                         (torch.float16, 2, 64, 64), (torch.bfloat16, 2, 32, 32),
                                         (torch.float16, 1, 128, 64), (torch.float16, 2, 64, 32),
                                         (torch.float16, 2, 192, 64), (torch.bfloat16, 1, 160, 64),
                                         (torch.float16, 2, 161, 64), (torch.float16, 1, 31, 32)])
def test_short_and_ragged_last_chunks(dtype, B, T, C):
    """Last chunks of 1..4 blocks, with and without a partial last block, one chunk only, and
    sequences of whole chunks (the backward reads the last chunk of a sequence through a general
    loader unless it is full, and pairs the work of neighbouring chunks in its stages)."""
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, dtype, seed=100 + T, gate_mean=2.5, state_std=0.3)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, dtype, expect_flagged=0)


def test_batch_larger_than_half_the_device():
    """With more than 128 rows the forward runs one workgroup per row (below that, two); the
    backward's grid exceeds the number of CUs."""
    B, T = 136, 80
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=31, state_std=0.2)
    f = f.clone()
    f[135, 70, 50] = 1.25               # rows for the exact recurrence: one in the last workgroup,
    f[64, 3, 7] = -0.0                  # one with a sign bit (a plain zero gate stays on the matrix cores)
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 64)
    assert flagged == (2, 2), flagged
    rows = [0, 63, 64, 127, 128, 135]
    sub = [t[rows] for t in (x, f, q, k, fk, s)]
    r_out, r_nxt = c_oracle.lfw_forward(*sub)
    r_grads = c_oracle.lfw_backward(go[rows], gs[rows], *sub)
    assert_close(out[rows], r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt[rows], r_nxt, torch.float16, "next_state", tol=TOL_CHUNK)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[rows], r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)
    # one workgroup per row: a flagged row is redone whole, in both directions
    for i in (2, 5):
        assert_close(out[rows[i]], r_out[i], torch.float16, "outputs[flagged row %d]" % rows[i])
        assert_close(nxt[rows[i]], r_nxt[i], torch.float16, "next_state[flagged row %d]" % rows[i])
        for n, g, r in zip(NAMES, grads, r_grads):
            assert_close(g[rows[i]], r[i], torch.float16, "%s[flagged row %d]" % (n, rows[i]))


def test_flagged_rows_with_a_partial_last_block():
    B, T = 3, 90
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=11, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[0, 40, 9] = -0.0
    fk[2, 89, 63] = 2.0                 # in the partial last block
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 32)
    assert flagged == (2, 2), flagged
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[0:1], r[0:1], torch.float16, n + "[flagged row 0]")
        assert_close(g[2:3], r[2:3], torch.float16, n + "[flagged row 2]")
        assert_close(g, r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)


def test_no_fixup_flag_reports_but_does_not_repair():
    from t2fw_amd import _lib
    B, T = 2, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=12, state_std=0.3)
    f = f.clone()
    f[1, 5, 2] = -0.0
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 64, flags=_lib.FLAG_NO_FIXUP)
    assert flagged == (1, 1), flagged
    # the unflagged row is valid without the exact kernels having run
    r_out, _ = c_oracle.lfw_forward(x[:1], f[:1], q[:1], k[:1], fk[:1], s[:1])
    assert_close(out[:1], r_out, torch.float16, "outputs[row 0]", tol=TOL_CHUNK)


def test_wide_gate_distribution_stays_on_the_chunked_path():
    # gates = sigmoid(N(0,1)): 16-step products down to ~1e-10, far below what fp16 operands could carry
    x, f, q, k, fk, s, go, gs = make_config_inputs(3, 256, 64, 64, torch.float16, seed=5, gate_mean=0.0,
                                                    state_std=0.5)
    check_against_oracle((x, f, q, k, fk, s), go, gs, 64, torch.float16, expect_flagged=0,
                         gate_tol=(2e-1, 4e-2))


def test_reference_test_gates_stay_on_the_matrix_cores_via_the_block_wise_backward():
    # per-channel constant gates in (1/64, 1-1/64) as the reference's tests build them
    # (16-step products down to 2^-96).  The forward takes them.  The chunk-parallel backward scales by
    # products over half a chunk, which these gates take below its range in every row: it declines both rows
    # and the block-wise kernel that follows computes them (nothing reaches the exact scan; a caller that
    # reads the forward's hints goes to the block-wise kernel directly, tests/test_zero_gates_gpu.py).
    # Unit-variance inputs over 256 steps give outputs up to 6, so atol = 1e-2 of the reference's test
    # is below the bf16 rounding of the forward's operands: chunk tolerance only.
    x, f, q, k, fk, s, go, gs = make_reference_test_inputs(2, 256, 64, 64, torch.float16, seed=1)
    check_against_oracle((x, f, q, k, fk, s), go, gs, 64, torch.float16, expect_flagged=0,
                         expect_flagged_parallel=2, gate_tol=(2e-1, 4e-2), reference_bounds=False)


@pytest.mark.parametrize("kind", ["negative_zero_gate", "negative_zero_gate_upper_channels", "gate_above_one", "negative_gate",
                                  "tiny_product", "nan_free_inf_gate"])
def test_rows_outside_the_gate_range_fall_back_to_the_exact_kernels(kind):
    B, T = 4, 160
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=3, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    if kind == "negative_zero_gate":            # the range check is on the bits: a sign bit is outside [0, 1]
        f[1, 70, 5] = -0.0
    elif kind == "negative_zero_gate_upper_channels":
        f[1, 70, 40] = -0.0             # seen only by the workgroup that owns value channels 32..63
    elif kind == "gate_above_one":
        fk[1, 3, 60] = 1.5
    elif kind == "negative_gate":
        f[1, 100, 0] = -0.5
    elif kind == "tiny_product":
        fk[1, 32:48, 7] = 1e-3          # 16-step product 1e-48 < 2^-100
    else:
        f[1, 10, 3] = 6e-8              # smallest positive fp16: product underflows the accepted range
        f[1, 11:26, 3] = 6e-8
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 64)
    assert flagged == (1, 1), flagged
    # The forward at this batch size runs one workgroup per (row, 32 value channels), and each
    # redoes its own channels with the exact recurrence when their gates (or the key-side gates,
    # which both see) are outside the range: tight tolerance on those channels, chunk tolerance on
    # the others.  The backward redoes the whole row from the checkpoints the forward left, so its
    # value-side results are tight on the same channels and its key-side results (sums over all
    # value channels) are tight when the whole row was redone.
    exact = {"negative_zero_gate": slice(0, 32), "negative_zero_gate_upper_channels": slice(32, 64), "negative_gate": slice(0, 32),
             "nan_free_inf_gate": slice(0, 32)}.get(kind, slice(0, 64))
    whole = exact == slice(0, 64)
    r_out, r_nxt = c_oracle.lfw_forward(x, f, q, k, fk, s)
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    assert_close(out[1:2, :, exact], r_out[1:2, :, exact], torch.float16, "outputs[flagged row]")
    assert_close(nxt[1:2, exact], r_nxt[1:2, exact], torch.float16, "next_state[flagged row]")
    for n, g, r in zip(NAMES, grads, r_grads):
        if n in ("d_x", "d_f"):
            assert_close(g[1:2, :, exact], r[1:2, :, exact], torch.float16, n + "[flagged row]")
        elif n == "d_state":
            assert_close(g[1:2, exact], r[1:2, exact], torch.float16, n + "[flagged row]")
        elif whole:
            assert_close(g[1:2], r[1:2], torch.float16, n + "[flagged row]")
        assert_close(g, r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)
    assert_close(out, r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt, r_nxt, torch.float16, "next_state", tol=TOL_CHUNK)


def test_fp16_operand_flag():
    # gates close to one: fp16 operands apply and give fp16-level accuracy
    x, f, q, k, fk, s, go, gs = make_config_inputs(2, 256, 64, 64, torch.float16, seed=8, gate_mean=4.5,
                                                    state_std=0.3)
    check_against_oracle((x, f, q, k, fk, s), go, gs, 64, torch.float16, flags=2, expect_flagged=0,
                         tol=(4e-3, 2e-3), gate_tol=(1e-2, 8e-3))


def test_full_size_headline_properties():
    """B=96, T=1024 (the benchmark's configuration): oracle parity on a slice of rows (rows are
    independent), plus linearity and segment composition over the whole batch."""
    B, T = 96, 1024
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=0, state_std=0.0)
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 64)
    assert flagged == (0, 0)
    rows = [0, 17, 95]
    sub = [t[rows] for t in (x, f, q, k, fk, s)]
    r_out, r_nxt = c_oracle.lfw_forward(*sub)
    r_grads = c_oracle.lfw_backward(go[rows], gs[rows], *sub)
    assert_close(out[rows], r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt[rows], r_nxt, torch.float16, "next_state", tol=TOL_CHUNK)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[rows], r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)
    # batch-row permutation: every row is an independent recurrence, bit for bit
    perm = torch.randperm(B, generator=torch.Generator().manual_seed(1))
    out_p, nxt_p, _, grads_p, _ = run_abi([t[perm] for t in (x, f, q, k, fk, s)], go[perm], gs[perm], 64)
    assert torch.equal(out_p.cpu(), out.cpu()[perm]) and torch.equal(nxt_p.cpu(), nxt.cpu()[perm])
    for a, b2 in zip(grads_p, grads):
        assert torch.equal(a.cpu(), b2.cpu()[perm])
    # segment composition: [0,512) then [512,1024) carrying the state == the whole sequence
    h = T // 2
    o1, m, _, _, _ = run_abi([t[:, :h].contiguous() for t in (x, f, q, k, fk)] + [s], go, gs, 64, with_backward=False)
    o2, n2, _, _, _ = run_abi([t[:, h:].contiguous() for t in (x, f, q, k, fk)] + [m.cpu()], go, gs, 64,
                              with_backward=False)
    whole = out.float().cpu()
    assert_close(torch.cat([o1, o2], 1), whole, torch.float16, "segment composition", tol=TOL_CHUNK)
    assert_close(n2, nxt.float().cpu(), torch.float16, "segment composition state", tol=TOL_CHUNK)
    # checkpoints: ckpt[:, c] is the state after c*64 steps == next_state of the first c*64 steps
    assert torch.equal(ckpt[:, 0].cpu(), s)
    o8, n8, _, _, _ = run_abi([t[:, :512].contiguous() for t in (x, f, q, k, fk)] + [s], go, gs, 64,
                              with_backward=False)
    assert torch.equal(ckpt[:, 8].cpu(), n8.cpu())


def test_long_context_bf16_slice():
    """cfg4 shape per row (T=8192, bf16, gates sigmoid(N(3,1)), nonzero initial state) on a few rows."""
    B, T = 2, 8192
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.bfloat16, seed=4, gate_mean=3.0,
                                                    state_std=0.1)
    check_against_oracle((x, f, q, k, fk, s), go, gs, 64, torch.bfloat16, expect_flagged=0)


@pytest.mark.parametrize("seed", range(24))
def test_random_lengths_and_intervals(seed):
    """seeded random (T, C, B, dtype): every combination of chunk count, pairs in the last chunk and
    tokens in the last block that the stage schedule of the backward distinguishes"""
    g = torch.Generator().manual_seed(1000 + seed)
    C = (32, 64)[int(torch.randint(0, 2, (1,), generator=g))]
    T = int(torch.randint(1, 5 * C + 1, (1,), generator=g))
    B = int(torch.randint(1, 4, (1,), generator=g))
    dtype = (torch.float16, torch.bfloat16)[int(torch.randint(0, 2, (1,), generator=g))]
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, dtype, seed=seed, gate_mean=2.5, state_std=0.3)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, dtype, expect_flagged=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("C,T", [(96, 300), (128, 1024), (128, 130), (256, 700), (1024, 1000), (160, 161)])
def test_checkpoint_intervals_that_are_other_multiples_of_32(C, T, dtype):
    """The forward takes any multiple of 32; the backward kernels take 32 and 64 and get there by running the
    forward kernel once more into checkpoints of their own (in the workspace), from s0."""
    x, f, q, k, fk, s, go, gs = make_config_inputs(3, T, 64, 64, dtype, seed=C + T, gate_mean=2.5, state_std=0.3)
    out, nxt, ckpt, grads = check_against_oracle((x, f, q, k, fk, s), go, gs, C, dtype, expect_flagged=0)
    # the caller's checkpoints are at the interval it asked for
    from t2fw_amd import _lib
    assert ckpt.shape[1] == _lib.load().t2fw_lfw_num_ckpt(T, C)


def test_sparse_checkpoints_with_rows_that_fall_back():
    B, T, C = 4, 400, 128
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=77, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[1, 200, 5] = -0.5                 # the exact recurrence, forward and backward
    fk[2, 64:96, 9] = 0.15              # declined by the chunk-parallel backward only
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (1, 2) and flagged.exact == 1, (flagged, flagged.exact)
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g, r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)
        assert_close(g[1:2], r[1:2], torch.float16, n + "[row on the exact scan]")


def test_float32_tensors_through_the_16_bit_kernels_by_explicit_cast():
    """lfw_apply_16bit: float32 in and out, the float16 matrix-core kernels in between; against the float64
    oracle on the float32 inputs, every tensor within 1e-2 of max|ref| (the gates' rounding to float16
    included), and the plain float32 call on the same inputs within the exact kernels' tolerance"""
    from oracle.lfw_ref import lfw_reference_grads
    from t2fw_amd import LFWFunction, lfw_apply_16bit
    x, f, q, k, fk, s, go, gs = make_config_inputs(4, 200, 64, 64, torch.float32, seed=77, state_std=0.2)
    r_out, r_nxt, r_grads = lfw_reference_grads(x, f, q, k, fk, s, go, gs)
    refs = [r_out, r_nxt] + list(r_grads)
    names = ["outputs", "next_state", "d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state"]
    for fn, bound in ((lfw_apply_16bit, 1e-2), (LFWFunction.apply, 1e-4)):
        ins = [t.cuda().requires_grad_(True) for t in (x, f, q, k, fk, s)]
        o, n = fn(*ins)
        assert o.dtype == torch.float32 and n.dtype == torch.float32
        torch.autograd.backward([o, n], [go.cuda(), gs.cuda()])
        got = [o, n] + [t.grad for t in ins]
        for name, g, r in zip(names, got, refs):
            assert g.dtype == torch.float32
            err = (g.detach().double().cpu() - r.double()).abs().max().item()
            scale = r.double().abs().max().item()
            assert err <= bound * scale, "%s (bound %g of max|ref|): max error %.3e against max|ref| %.3e" % (name, bound, err, scale)
