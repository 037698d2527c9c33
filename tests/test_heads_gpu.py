"""GPU parity of the head-strided entry points (tensors [B,T,H,D] / [B,T,H,K], states [B,H,D,K]).

Two checks per case: against the CPU oracle run on the folded [B*H,T,D] rows (the layout the
reference requires, t2fw/csrc/lfw.cpp:24-26), and against this library's folded entry points on
the same rows.  The strided kernels do the same arithmetic in the same order and only the
addresses differ, so the results agree to the last bit except where the compiler contracted a
multiply-add or a multiply-convert differently in the two instantiations (one unit in the last
place, seen on about one element in a million); anything larger is an addressing mistake."""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs, make_reference_test_inputs
from tests.test_lfw_chunk_gpu import NAMES, chunk_parallel_backward, flagged_rows, run_abi
from tests.test_lfw_gpu import TOL, TOL_CHUNK, TOL_CHUNK_GATE, assert_close, gate_grad_floor, on_chunk_path

pytestmark = pytest.mark.gpu


def to_heads(t, B, H):
    """[B*H, T, W] -> [B, T, H, W] (contiguous)"""
    return t.view(B, H, t.shape[1], t.shape[2]).transpose(1, 2).contiguous()


def from_heads(t):
    """[B, T, H, W] -> [B*H, T, W]"""
    B, T, H, W = t.shape
    return t.transpose(1, 2).reshape(B * H, T, W)


ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2.0 ** -22, torch.float64: 2.0 ** -50}


def assert_same(a, b, what):
    """equal up to one unit in the last place on at most 0.1 % of the elements"""
    if torch.equal(a, b):
        return
    assert a.shape == b.shape, what
    x, y = a.double(), b.double()
    diff = (x - y).abs()
    assert not torch.isnan(diff).any(), what + ": NaN"
    differing = int((diff > 0).sum())
    assert differing <= max(1, a.numel() // 1000), "%s: %d of %d elements differ" % (what, differing, a.numel())
    bound = ULP[a.dtype] * torch.maximum(x.abs(), y.abs())
    assert (diff <= bound).all(), "%s: differs from the folded layout's by up to %.3e" % (what, float(diff.max()))


def run_heads_abi(inputs, go, gs, B, H, C, flags=0):
    """forward + backward through the head-strided C ABI; inputs are folded [B*H, ...] CPU tensors.
    Returns everything folded again, plus the flagged-row counts."""
    from t2fw_amd import _lib
    lib = _lib.load()
    x, f, q, k, fk, s = inputs
    T, D, K = x.shape[1], x.shape[2], q.shape[2]
    ins = [to_heads(t, B, H).cuda() for t in (x, f, q, k, fk)] + [s.cuda()]      # state [B,H,D,K] == [B*H,D,K]
    code = _lib.DTYPE_CODE[x.dtype]
    # canaries: nothing outside the tensors may be written, so poison the outputs and compare all of them
    out = torch.full_like(ins[0], float("nan"))
    nxt = torch.full_like(ins[5], float("nan"))
    nc = lib.t2fw_lfw_num_ckpt(T, C)
    ckpt = torch.empty(B * H, nc, D, K, dtype=x.dtype, device="cuda")
    wsb = lib.t2fw_lfw_workspace_bytes(B * H, T, D, K, C, code, flags)
    ws = torch.zeros(max(wsb, 256), dtype=torch.uint8, device="cuda")
    st = _lib.current_stream_handle(out.device)
    _lib.check(lib.t2fw_lfw_forward_heads(*[_lib.ptr(t) for t in ins], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt),
                                          B, T, H, D, K, C, code, flags, _lib.ptr(ws), wsb, st))
    torch.cuda.synchronize()
    flagged_fwd = flagged_rows(ws, B * H) if wsb else 0
    grads = [torch.full_like(t, float("nan")) for t in ins]
    go_d, gs_d = to_heads(go, B, H).cuda(), gs.cuda()
    _lib.check(lib.t2fw_lfw_backward_heads(_lib.ptr(go_d), _lib.ptr(gs_d), *[_lib.ptr(t) for t in ins], _lib.ptr(ckpt),
                                           *[_lib.ptr(t) for t in grads], B, T, H, D, K, C, code, flags,
                                           _lib.ptr(ws), wsb, st))
    torch.cuda.synchronize()
    flagged_bwd = flagged_rows(ws, B * H, chunk_parallel_backward(C, flags)) if wsb else 0
    folded = [from_heads(g) for g in grads[:5]] + [grads[5]]
    return from_heads(out), nxt, ckpt, folded, (flagged_fwd, flagged_bwd)


def check_heads(inputs, go, gs, B, H, C, dtype, expect_flagged=None, oracle_rows=None):
    out, nxt, ckpt, grads, flagged = run_heads_abi(inputs, go, gs, B, H, C)
    if expect_flagged is not None:
        assert flagged == (expect_flagged, expect_flagged), flagged
    # (1) against the folded entry points
    f_out, f_nxt, f_ckpt, f_grads, f_flagged = run_abi(inputs, go, gs, C)
    assert f_flagged == flagged
    assert_same(out, f_out, "outputs")
    assert_same(nxt, f_nxt, "next_state")
    assert_same(ckpt, f_ckpt, "checkpoints")
    for n, a, b in zip(NAMES, grads, f_grads):
        assert_same(a, b, n)
    # (2) against the oracle (on a subset of rows where the case is large)
    rows = list(range(B * H)) if oracle_rows is None else oracle_rows
    sub = [t[rows] for t in inputs]
    r_out, r_nxt = c_oracle.lfw_forward(*sub)
    r_grads = c_oracle.lfw_backward(go[rows], gs[rows], *sub)
    D, K = inputs[0].shape[2], inputs[2].shape[2]
    chunk = on_chunk_path(dtype, D, K)
    tol = TOL_CHUNK if chunk else TOL[dtype]
    gate_tol = TOL_CHUNK_GATE if chunk else TOL[dtype]
    floors = gate_grad_floor(sub, go[rows], r_out, r_grads) if chunk else {}
    assert_close(out[rows], r_out, dtype, "outputs", tol=tol)
    assert_close(nxt[rows], r_nxt, dtype, "next_state", tol=tol)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[rows], r, dtype, n, tol=gate_tol if n in ("d_f", "d_f_key") else tol, floor=floors.get(n, 0.0))


@pytest.mark.parametrize("dtype,gate_mean", [(torch.float16, 2.0), (torch.bfloat16, 3.0)])
@pytest.mark.parametrize("B,H,T,C", [(2, 3, 256, 64), (1, 12, 200, 64), (3, 2, 77, 32), (2, 4, 1, 64), (1, 5, 16, 64),
                                     (2, 2, 33, 64), (1, 3, 130, 32), (4, 1, 96, 64)])
def test_matrix_core_path(dtype, gate_mean, B, H, T, C):
    x, f, q, k, fk, s, go, gs = make_config_inputs(B * H, T, 64, 64, dtype, seed=7 * T + H, gate_mean=gate_mean,
                                                    state_std=0.1)
    check_heads((x, f, q, k, fk, s), go, gs, B, H, C, dtype, expect_flagged=0)


def test_more_rows_than_half_the_device_takes_the_one_workgroup_per_row_forward():
    B, H, T = 9, 16, 150           # 144 rows
    x, f, q, k, fk, s, go, gs = make_config_inputs(B * H, T, 64, 64, torch.float16, seed=3, state_std=0.2)
    check_heads((x, f, q, k, fk, s), go, gs, B, H, 64, torch.float16, expect_flagged=0,
                oracle_rows=[0, 1, 15, 16, 77, 143])


def test_flagged_rows_are_redone_by_the_exact_kernels_in_place():
    B, H, T = 2, 3, 90
    x, f, q, k, fk, s, go, gs = make_config_inputs(B * H, T, 64, 64, torch.float16, seed=11, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[1, 40, 9] = -0.0                 # batch 0, head 1
    fk[5, 89, 63] = 2.0                # batch 1, head 2, in the partial last block
    check_heads((x, f, q, k, fk, s), go, gs, B, H, 32, torch.float16, expect_flagged=2)


def test_flagged_rows_with_one_workgroup_per_row():
    B, H, T = 23, 6, 70                # 138 rows: the forward runs one workgroup per row
    x, f, q, k, fk, s, go, gs = make_config_inputs(B * H, T, 64, 64, torch.bfloat16, seed=19, gate_mean=3.0,
                                                    state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[137, 69, 33] = -0.0              # last row, last token
    fk[6, 0, 0] = -1.0                 # batch 1, head 0, first token
    check_heads((x, f, q, k, fk, s), go, gs, B, H, 64, torch.bfloat16, expect_flagged=2,
                oracle_rows=[0, 5, 6, 7, 136, 137])


@pytest.mark.parametrize("dtype,B,H,T,D,K", [(torch.float32, 2, 3, 77, 33, 17), (torch.float16, 1, 4, 50, 32, 16),
                                             (torch.float64, 2, 2, 40, 5, 9), (torch.bfloat16, 2, 2, 300, 64, 32),
                                             (torch.float32, 1, 2, 70, 64, 64)])
def test_exact_kernels(dtype, B, H, T, D, K):
    x, f, q, k, fk, s, go, gs = make_reference_test_inputs(B * H, T, D, K, dtype, seed=T)
    check_heads((x, f, q, k, fk, s), go, gs, B, H, 64, dtype)


def test_entry_points_reject_bad_head_counts():
    from t2fw_amd import _lib
    lib = _lib.load()
    z = torch.zeros(2 * 8 * 2 * 64, dtype=torch.float16, device="cuda")
    s = torch.zeros(4 * 64 * 64, dtype=torch.float16, device="cuda")
    p, st = _lib.ptr, _lib.current_stream_handle(z.device)
    ws = torch.zeros(256, dtype=torch.uint8, device="cuda")
    args = lambda H: (p(z), p(z), p(z), p(z), p(z), p(s), p(z), p(s), None, 2, 8, H, 64, 64, 64, 1, 0, p(ws), 256, st)
    assert lib.t2fw_lfw_forward_heads(*args(0)) != 0
    assert lib.t2fw_lfw_forward_heads(*args(-3)) != 0
    assert b"H=" in lib.t2fw_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("logits", [False, True])
def test_autograd_function(logits):
    """LFWHeadsFunction against LFWFunction / LFWGatedFunction on the folded rows."""
    from t2fw_amd import LFWFunction, LFWGatedFunction, LFWHeadsFunction
    B, H, T, dtype = 2, 6, 260, torch.float16
    g = torch.Generator().manual_seed(17)
    mk = lambda *sh: torch.randn(*sh, generator=g)
    x, q, k = [(mk(B * H, T, 64) / 8).to(dtype) for _ in range(3)]
    zf, zk = [(mk(B * H, T, 64) + 2).to(dtype) for _ in range(2)]
    if not logits:
        zf, zk = torch.sigmoid(zf.float()).to(dtype), torch.sigmoid(zk.float()).to(dtype)
    s = (mk(B * H, 64, 64) * 0.1).to(dtype)
    go, gs = mk(B * H, T, 64).to(dtype), (mk(B * H, 64, 64) * 0.1).to(dtype)

    folded = [t.cuda().requires_grad_(True) for t in (x, zf, q, k, zk, s)]
    out_f, nxt_f = (LFWGatedFunction if logits else LFWFunction).apply(*folded)
    out_f.backward(go.cuda(), retain_graph=True)
    nxt_f.backward(gs.cuda())

    heads = [to_heads(t, B, H).cuda().requires_grad_(True) for t in (x, zf, q, k, zk)]
    heads.append(s.view(B, H, 64, 64).cuda().requires_grad_(True))
    out_h, nxt_h = LFWHeadsFunction.apply(*heads, logits)
    assert out_h.shape == (B, T, H, 64) and nxt_h.shape == (B, H, 64, 64)
    out_h.backward(to_heads(go, B, H).cuda(), retain_graph=True)
    nxt_h.backward(gs.view(B, H, 64, 64).cuda())
    torch.cuda.synchronize()

    assert_same(from_heads(out_h), out_f, "outputs")
    assert_same(nxt_h.view(B * H, 64, 64), nxt_f, "next_state")
    for i in range(5):
        assert_same(from_heads(heads[i].grad), folded[i].grad, "gradient %d" % i)
    assert_same(heads[5].grad.view(B * H, 64, 64), folded[5].grad, "d_state")


def test_shape_checks_of_the_autograd_function():
    from t2fw_amd import LFWHeadsFunction
    z = torch.zeros(2, 8, 3, 64, dtype=torch.float16, device="cuda")
    s = torch.zeros(2, 3, 64, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        LFWHeadsFunction.apply(z, z, z, z, z, s.view(6, 64, 64))
    with pytest.raises(RuntimeError):
        LFWHeadsFunction.apply(z, z, z[:, :, :2].contiguous(), z[:, :, :2].contiguous(), z[:, :, :2].contiguous(), s)
    wide = torch.zeros(2, 8, 3, 128, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        LFWHeadsFunction.apply(wide[..., :64], z, z, z, z, s)             # not contiguous
