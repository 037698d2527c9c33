"""GPU parity of the chunk-parallel LFW backward (D = K = 64, fp16 / bf16 tensors, checkpoint
interval 32 or 64) against the CPU oracle, through the C ABI: which gate sequences it accepts,
that the rows it declines are redone exactly, and launch shapes (chunk counts on either side of the
chunk-scan's batches, more rows x chunks than the device has compute units)."""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs
from tests.test_lfw_chunk_gpu import NAMES, check_against_oracle, run_abi
from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close

pytestmark = pytest.mark.gpu


def oracle(inputs, go, gs):
    return c_oracle.lfw_forward(*inputs), c_oracle.lfw_backward(go, gs, *inputs)


def assert_rows_exact(grads, r_grads, rows, dtype):
    """rows redone by the exact scan meet the exact kernels' tolerance"""
    for n, g, r in zip(NAMES, grads, r_grads):
        for b in rows:
            assert_close(g[b:b + 1], r[b:b + 1], dtype, "%s[flagged row %d]" % (n, b))


def assert_all_chunk(grads, r_grads, dtype):
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g, r, dtype, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)


@pytest.mark.parametrize("C", [32, 64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 31, 32, 33, 64, 65, 127, 128, 1023, 1040, 1100, 2100])
def test_chunk_counts_and_ragged_last_chunks(C, dtype, T):
    """one chunk, whole chunks, a last chunk of every fill, and chunk counts on either side of 16
    and 32 (the chunk scan walks the chunks of a row in batches of 16)"""
    B = 2 if T > 128 else 3
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, dtype, seed=7 * T + C, gate_mean=2.5,
                                                    state_std=0.3)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, dtype, expect_flagged=0)


def test_more_items_than_compute_units():
    B, T = 300, 130
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=41, state_std=0.2)
    f = f.clone()
    f[299, 129, 63] = -0.0              # the last token of the last row, in a chunk of two tokens
    f[150, 64, 0] = 1.5
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 64)
    assert flagged == (2, 2), flagged
    rows = [0, 1, 149, 150, 151, 255, 256, 298, 299]
    sub = [t[rows] for t in (x, f, q, k, fk, s)]
    r_grads = c_oracle.lfw_backward(go[rows], gs[rows], *sub)
    assert_all_chunk([g[rows] for g in grads], r_grads, torch.float16)
    assert_rows_exact([g[rows] for g in grads], r_grads, [3, 8], torch.float16)


@pytest.mark.parametrize("C", [32, 64])
def test_gate_products_down_to_the_accepted_range_stay_on_the_matrix_cores(C):
    """Half a chunk of gates whose product is 2^-67 (C = 64) or 2^-34 (C = 32): inside the range, so no
    row is flagged, and the results still meet the chunk tolerance."""
    B, T = 3, 4 * C
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=17, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[1, C:C + C // 2, 11] = 0.2344         # 2^-2.09 per step
    fk[2, 2 * C + C // 2:3 * C, 40] = 0.2344
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, torch.float16, expect_flagged=0, gate_tol=(2e-1, 4e-2))


@pytest.mark.parametrize("where", ["first_half", "second_half", "key_side", "last_partial_chunk"])
def test_half_chunk_products_below_the_range_are_flagged_in_the_backward_only(where):
    """32 gates of 0.15 (product 2^-87.6) in one half of a chunk: the forward's 16-step blocks take
    them (2^-43.8 each); the chunk-parallel backward declines the row, and the block-wise kernel that
    follows it takes it (nothing reaches the exact scan)."""
    B, T, C = 3, 230, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=19, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    if where == "first_half":
        f[1, 64:96, 3] = 0.15
    elif where == "second_half":
        f[1, 96:128, 63] = 0.15
    elif where == "key_side":
        fk[1, 128:160, 32] = 0.15
    else:
        fk[1, 192:224, 0] = 0.15            # the last chunk holds 38 tokens
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (0, 1) and flagged.exact == 0, (flagged, flagged.exact)
    (r_out, r_nxt), r_grads = oracle((x, f, q, k, fk, s), go, gs)
    assert_all_chunk(grads, r_grads, torch.float16)


def test_rows_that_neither_matrix_core_form_takes_reach_the_exact_scan():
    """a row with small gates over half a chunk (declined by the chunk-parallel form only) next to a row
    with a 16-step product below the block-wise form's limit and a row with a gate that has a sign bit"""
    B, T, C = 4, 256, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=21, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[0, 64:96, 3] = 0.15               # 2^-87.6 over half a chunk, 2^-43.8 per block
    fk[1, 128:144, 9] = 0.01            # 2^-106 in one block
    f[3, 200, 60] = -0.0
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged[1] == 3 and flagged.exact == 2, (flagged, flagged.exact)
    (r_out, r_nxt), r_grads = oracle((x, f, q, k, fk, s), go, gs)
    assert_all_chunk(grads, r_grads, torch.float16)
    assert_rows_exact(grads, r_grads, [1, 3], torch.float16)


def test_small_gates_across_a_half_chunk_boundary_are_accepted():
    """the same 32 gates of 0.15, 16 on either side of the middle of a chunk: each half's product is
    2^-43.8, nothing is flagged"""
    B, T, C = 2, 192, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=23, state_std=0.3)
    f = f.clone()
    f[0, 80:112, 5] = 0.15
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, torch.float16, expect_flagged=0, gate_tol=(2e-1, 4e-2))


@pytest.mark.parametrize("C", [32, 64])
@pytest.mark.parametrize("where", ["first_half", "second_half", "both_halves"])
def test_small_gate_products_on_both_sides_at_once(where, C):
    """Every channel of BOTH gates decays by 2^-76 over half a chunk: inside the accepted range on
    either side, while the state entering the chunk and the adjoint entering it from the future are
    scaled by the product of the two sides, 2^-152, which no 32-bit exponent holds unshifted.  The
    half's first token keeps gates of one, so that d_q, d_f and d_f_key there see the whole entering
    state; the chunk's last token always sees the whole adjoint from beyond the chunk (d_x, d_k)."""
    B, T, h = 3, 3 * C, C // 2
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=53 + C, gate_mean=3.0,
                                                    state_std=0.5)
    f, fk = f.clone(), fk.clone()
    small_first = 2.0 ** (-76.0 / (h - 1))       # h - 1 steps after a first step of one
    small_second = 2.0 ** (-76.0 / h)
    for b, c0 in ((0, 0), (1, C), (2, 2 * C)):       # row b: chunk b
        if where != "second_half":
            for g in (f, fk):
                g[b, c0] = 1.0
                g[b, c0 + 1:c0 + h] = small_first
        if where != "first_half":
            for g in (f, fk):
                g[b, c0 + h:c0 + C] = small_second
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, torch.float16, expect_flagged=0, gate_tol=(2e-1, 4e-2),
                         reference_bounds=False)
    # the tokens named above, on their own scale
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    for b, c0 in ((0, 0), (1, C), (2, 2 * C)):
        checks = []
        if where != "second_half":
            checks += [("d_q", c0)]
        if where != "first_half":
            checks += [("d_x", c0 + C - 1), ("d_k", c0 + C - 1)]
        for n, t in checks:
            got = grads[NAMES.index(n)][b, t].double().cpu()
            ref = torch.as_tensor(r_grads[NAMES.index(n)])[b, t].double()
            assert (got - ref).abs().max() <= 2e-2 * ref.abs().max(), (n, b, t)


@pytest.mark.parametrize("chunk", [0, 15, 16, 17, 36])
@pytest.mark.parametrize("bad", [-0.0, -0.25, 1.0625])
def test_a_gate_outside_the_range_in_any_chunk_flags_the_row(chunk, bad):
    B, C = 3, 32
    T = 37 * C - 5
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.bfloat16, seed=29 + chunk, gate_mean=3.0,
                                                    state_std=0.2)
    fk = fk.clone()
    fk[2, chunk * C + 7, 9] = bad
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged[1] == 1, flagged
    (r_out, r_nxt), r_grads = oracle((x, f, q, k, fk, s), go, gs)
    assert_all_chunk(grads, r_grads, torch.bfloat16)
    assert_rows_exact(grads, r_grads, [2], torch.bfloat16)


def test_no_fixup_reports_the_rows_and_leaves_them():
    from t2fw_amd import _lib
    B, T = 3, 200
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=31, state_std=0.3)
    f = f.clone()
    f[1, 160:192, 2] = 0.15             # the second half of the third chunk
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, 64, flags=_lib.FLAG_NO_FIXUP)
    assert flagged == (0, 1), flagged
    keep = [0, 2]
    r_grads = c_oracle.lfw_backward(go[keep], gs[keep], *[t[keep] for t in (x, f, q, k, fk, s)])
    assert_all_chunk([g[keep] for g in grads], r_grads, torch.float16)


def test_flags_are_forgotten_between_calls_on_one_workspace():
    """a second backward on the same workspace, with inputs that need no exact rows, reports none"""
    from t2fw_amd import _lib
    lib = _lib.load()
    B, T, C = 2, 128, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=37, state_std=0.3)
    bad_f = f.clone()
    bad_f[0, 3, 3] = -0.0
    code = _lib.DTYPE_CODE[x.dtype]
    wsb = lib.t2fw_lfw_workspace_bytes(B, T, 64, 64, C, code, 0)
    ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
    st = _lib.current_stream_handle(ws.device)
    counts, results = [], []
    for gates in (bad_f, f):
        ins = [t.cuda() for t in (x, gates, q, k, fk, s)]
        out, nxt = torch.empty_like(ins[0]), torch.empty_like(ins[5])
        ckpt = torch.empty(B, lib.t2fw_lfw_num_ckpt(T, C), 64, 64, dtype=x.dtype, device="cuda")
        grads = [torch.empty_like(t) for t in ins]
        go_d, gs_d = go.cuda(), gs.cuda()
        _lib.check(lib.t2fw_lfw_forward(*[_lib.ptr(t) for t in ins], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt),
                                        B, T, 64, 64, C, code, 0, _lib.ptr(ws), wsb, st))
        _lib.check(lib.t2fw_lfw_backward(_lib.ptr(go_d), _lib.ptr(gs_d), *[_lib.ptr(t) for t in ins], _lib.ptr(ckpt),
                                         *[_lib.ptr(t) for t in grads], B, T, 64, 64, C, code, 0, _lib.ptr(ws), wsb, st))
        torch.cuda.synchronize()
        from tests.test_lfw_chunk_gpu import flagged_rows
        counts.append(flagged_rows(ws, B, True))
        results.append(grads)
    assert counts == [1, 0], counts
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    assert_all_chunk(results[1], r_grads, torch.float16)


def test_workspace_too_small_is_refused_before_any_launch():
    from t2fw_amd import _lib
    lib = _lib.load()
    B, T, C = 2, 128, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=43)
    code = _lib.DTYPE_CODE[x.dtype]
    need = lib.t2fw_lfw_workspace_bytes(B, T, 64, 64, C, code, 0)
    fwd_need = lib.t2fw_lfw_forward_workspace_bytes(B, T, 64, 64, C, code, 0)
    assert need > fwd_need > 0
    assert lib.t2fw_lfw_workspace_bytes(B, T, 64, 64, C, code, _lib.FLAG_BLOCKWISE) == fwd_need
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    ckpt = torch.zeros(B, lib.t2fw_lfw_num_ckpt(T, C), 64, 64, dtype=x.dtype, device="cuda")
    grads = [torch.full_like(t, 7.0) for t in ins]
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    go_d, gs_d = go.cuda(), gs.cuda()
    rc = lib.t2fw_lfw_backward(_lib.ptr(go_d), _lib.ptr(gs_d), *[_lib.ptr(t) for t in ins], _lib.ptr(ckpt),
                               *[_lib.ptr(t) for t in grads], B, T, 64, 64, C, code, 0, _lib.ptr(ws), need - 1,
                               _lib.current_stream_handle(ws.device))
    torch.cuda.synchronize()
    assert rc == 6, rc
    assert all(bool((g == 7.0).all()) for g in grads)
