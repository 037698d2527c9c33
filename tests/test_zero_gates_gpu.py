"""Exactly zero gates (what an fp16 sigmoid returns below a logit of about -17) on the matrix-core
kernels: the reference multiplies by any gate value (t2fw/csrc/lfw_kernel.cu:46-50), so a zero is
an ordinary input there; here the forward and the chunk-parallel backward take it without handing the
row to the exact recurrence, within the matrix-core tolerance, and at the speed of any other row.
Also the forward's hints that steer the backward call from the host (t2fw_amd/path_hint.py)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs, make_reference_test_inputs
from tests.test_lfw_chunk_gpu import NAMES, run_abi
from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close, gate_grad_floor

pytestmark = pytest.mark.gpu


def check(inputs, go, gs, out, nxt, grads, dtype, rows=None):
    sel = (lambda t: t[rows]) if rows is not None else (lambda t: t)
    sub = [sel(t) for t in inputs]
    r_out, r_nxt = c_oracle.lfw_forward(*sub)
    r_grads = c_oracle.lfw_backward(sel(go), sel(gs), *sub)
    floors = gate_grad_floor(sub, sel(go), r_out, r_grads)
    assert_close(sel(out), r_out, dtype, "outputs", tol=TOL_CHUNK)
    assert_close(sel(nxt), r_nxt, dtype, "next_state", tol=TOL_CHUNK)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(sel(g), r, dtype, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK,
                     floor=floors.get(n, 0.0))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("C", [32, 64])
def test_zero_gates_stay_on_the_matrix_cores(dtype, C):
    B, T = 5, 4 * C + 9
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, dtype, seed=51 + C, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[0, 0, 0] = 0.0                    # the first token of a row
    f[0, C, 17] = 0.0                   # the first token of a chunk
    f[1, C - 1, 63] = 0.0               # the last token of a chunk
    fk[1, C + C // 2, 31] = 0.0         # the first token of a second half chunk, key side
    fk[2, T - 1, 5] = 0.0               # the last token of a ragged last chunk
    f[3, 2 * C + 3, 40] = 0.0           # two zeros in one channel of one half chunk
    f[3, 2 * C + 9, 40] = 0.0
    fk[3, 70:73, 8] = 0.0               # three in a row
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (0, 0) and flagged.exact == 0, (flagged, flagged.exact)
    check((x, f, q, k, fk, s), go, gs, out, nxt, grads, dtype)


def test_tiny_positive_gates_are_taken_like_zeros():
    """gates between zero and the kernels' floors (2^-24 forward, 2^-12 backward)"""
    B, T, C = 3, 200, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.bfloat16, seed=57, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[0, 50, 3] = 1e-30
    fk[1, 130, 60] = 3e-6
    f[2, 10, 9] = 1e-4
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (0, 0), flagged
    check((x, f, q, k, fk, s), go, gs, out, nxt, grads, torch.bfloat16)


def _time_backward(inputs, go, gs, C, flags, reps=30):
    from t2fw_amd import _lib
    lib = _lib.load()
    ins = [t.cuda() for t in inputs]
    B, T, D = ins[0].shape
    code = _lib.DTYPE_CODE[ins[0].dtype]
    out, nxt = torch.empty_like(ins[0]), torch.empty_like(ins[5])
    ckpt = torch.empty(B, lib.t2fw_lfw_num_ckpt(T, C), D, D, dtype=ins[0].dtype, device="cuda")
    wsb = lib.t2fw_lfw_workspace_bytes(B, T, D, D, C, code, flags)
    ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
    st = _lib.current_stream_handle(ins[0].device)
    grads = [torch.empty_like(t) for t in ins]
    go_d, gs_d = go.cuda(), gs.cuda()
    _lib.check(lib.t2fw_lfw_forward(*[_lib.ptr(t) for t in ins], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt),
                                    B, T, D, D, C, code, flags, _lib.ptr(ws), wsb, st))

    def bwd():
        _lib.check(lib.t2fw_lfw_backward(_lib.ptr(go_d), _lib.ptr(gs_d), *[_lib.ptr(t) for t in ins], _lib.ptr(ckpt),
                                         *[_lib.ptr(t) for t in grads], B, T, D, D, C, code, flags, _lib.ptr(ws), wsb, st))
    for _ in range(5):
        bwd()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        bwd()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps, out, nxt, grads


def test_headline_shape_with_zero_gates_runs_at_the_speed_of_any_other_input():
    B, T, C = 96, 1024, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=0)
    base_ms, _, _, _ = _time_backward((x, f, q, k, fk, s), go, gs, C, 0)
    f, fk = f.clone(), fk.clone()
    rows = [3, 17, 30, 44, 58, 71, 85, 95]
    for i, b in enumerate(rows):
        (f if i % 2 == 0 else fk)[b, 100 * i + 37, 8 * i + 1] = 0.0
    ms, out, nxt, grads = _time_backward((x, f, q, k, fk, s), go, gs, C, 0)
    print("backward %.4f ms with a zero gate in each of %d rows, %.4f ms without" % (ms, len(rows), base_ms))
    assert ms <= 2.0 * base_ms, (ms, base_ms)
    check((x, f, q, k, fk, s), go, gs, out, nxt, grads, torch.float16, rows=rows)


def test_gated_function_with_saturated_logits():
    """logits of -20 and below: the fp16 sigmoid is exactly zero there"""
    from t2fw_amd import LFWGatedFunction, sigmoid_gates
    dtype = torch.float16
    g = torch.Generator().manual_seed(77)
    B, T, D, K = 3, 256, 64, 64
    x, q, k = [(torch.randn(B, T, n, generator=g) / 8).to(dtype) for n in (D, K, K)]
    zf, zk = [(torch.randn(B, T, n, generator=g) + 2).to(dtype) for n in (D, K)]
    s = (torch.randn(B, D, K, generator=g) * 0.1).to(dtype)
    go = torch.randn(B, T, D, generator=g).to(dtype)
    gs = (torch.randn(B, D, K, generator=g) * 0.1).to(dtype)
    zf[0, 33, 4] = -20.0
    zf[1, 128, 60] = -30.0
    zk[1, 200, 9] = -25.0
    zk[2, 0, 0] = -60000.0
    ins = [t.cuda().requires_grad_(True) for t in (x, zf, q, k, zk, s)]
    out, nxt = LFWGatedFunction.apply(*ins)
    out.backward(go.cuda(), retain_graph=True)
    nxt.backward(gs.cuda())
    torch.cuda.synchronize()
    f, fk = [t.cpu() for t in sigmoid_gates(ins[1].detach(), ins[4].detach())]
    assert float(f[0, 33, 4]) == 0.0 and float(fk[2, 0, 0]) == 0.0
    inputs = (x, f, q, k, fk, s)
    r_out, r_nxt = c_oracle.lfw_forward(*inputs)
    r_grads = [torch.as_tensor(t).double() for t in c_oracle.lfw_backward(go, gs, *inputs)]
    floors = gate_grad_floor(inputs, go, r_out, r_grads)
    assert_close(out, r_out, dtype, "outputs", tol=TOL_CHUNK)
    assert_close(nxt, r_nxt, dtype, "next_state", tol=TOL_CHUNK)
    slope_f, slope_k = f.double() * (1 - f.double()), fk.double() * (1 - fk.double())
    refs = [r_grads[0], r_grads[1] * slope_f, r_grads[2], r_grads[3], r_grads[4] * slope_k, r_grads[5]]
    for n, t, r in zip(("d_x", "d_f_logit", "d_q", "d_k", "d_fk_logit", "d_state"), ins, refs):
        if n == "d_f_logit":
            assert_close(t.grad, r, dtype, n, tol=TOL_CHUNK_GATE, floor=0.25 * floors["d_f"])
        elif n == "d_fk_logit":
            assert_close(t.grad, r, dtype, n, tol=TOL_CHUNK_GATE, floor=0.25 * floors["d_f_key"])
        else:
            assert_close(t.grad, r, dtype, n, tol=TOL_CHUNK)
    assert float(ins[1].grad[0, 33, 4]) == 0.0          # a saturated gate passes no gradient to its logit


# ---- the forward's hints and the host's choice of the backward path -------------------------------

def _forward_hints(inputs, C, pinned):
    """forward through the C ABI with the workspace in device or pinned host memory; returns the number of
    rows hinted"""
    from t2fw_amd import _lib
    from t2fw_amd.path_hint import count_hinted_rows
    lib = _lib.load()
    ins = [t.cuda() for t in inputs]
    B, T, D = ins[0].shape
    code = _lib.DTYPE_CODE[ins[0].dtype]
    out, nxt = torch.empty_like(ins[0]), torch.empty_like(ins[5])
    ckpt = torch.empty(B, lib.t2fw_lfw_num_ckpt(T, C), D, D, dtype=ins[0].dtype, device="cuda")
    wsb = lib.t2fw_lfw_forward_workspace_bytes(B, T, D, D, C, code, 0)
    regions = (ctypes.c_int64 * 6)()
    _lib.check(lib.t2fw_lfw_flag_regions(B, T, D, D, C, code, 0, regions))
    if pinned:
        ws = torch.empty(wsb, dtype=torch.uint8, pin_memory=True).fill_(255)
        dptr = ctypes.c_void_p()
        _lib.check(lib.t2fw_host_workspace_device_pointer(ctypes.c_void_p(ws.data_ptr()), ctypes.byref(dptr)))
    else:
        ws = torch.full((wsb,), 255, dtype=torch.uint8, device="cuda")
        dptr = _lib.ptr(ws)
    _lib.check(lib.t2fw_lfw_forward(*[_lib.ptr(t) for t in ins], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt),
                                    B, T, D, D, C, code, 0, dptr, wsb, _lib.current_stream_handle(ins[0].device)))
    torch.cuda.synchronize()
    host = ws.cpu().numpy()
    hints = host[regions[2]:regions[2] + 4 * regions[3]].view(np.int32)
    return count_hinted_rows(hints, B)


@pytest.mark.parametrize("pinned", [False, True])
@pytest.mark.parametrize("B", [5, 136])         # two workgroups per row, one workgroup per row
def test_forward_hints_cover_what_the_chunk_parallel_backward_declines(pinned, B):
    T, C = 200, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=61, state_std=0.2)
    assert _forward_hints((x, f, q, k, fk, s), C, pinned) == 0
    f, fk = f.clone(), fk.clone()
    f[1, 64:96, 3] = 0.15               # 2^-43.8 per block: hinted, and declined by the backward
    fk[2, 128:144, 40] = 0.2            # 2^-37 in one block: neither
    f[3, 7, 7] = 0.0                    # a single zero: neither
    f[4, 150, 50] = -0.5                # outside [0, 1]: both
    assert _forward_hints((x, f, q, k, fk, s), C, pinned) == 2
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (1, 2), flagged


def test_autograd_wrapper_picks_the_backward_path_from_the_hints(monkeypatch):
    """LFWFunction: no row hinted -> the backward call carries NO_FIXUP; every row hinted (the reference
    test's gates) -> BLOCKWISE; results match the oracle either way"""
    from t2fw.functional_lfw import LFWFunction
    from t2fw_amd import _lib
    lib = _lib.load()
    seen = []
    real = lib.t2fw_lfw_backward

    class Spy:
        def __call__(self, *a):
            seen.append(a[21])          # the flags argument
            return real(*a)
    monkeypatch.setattr(lib, "t2fw_lfw_backward", Spy())

    def run(inputs, go, gs):
        ins = [t.cuda().requires_grad_(True) for t in inputs]
        out, nxt = LFWFunction.apply(*ins)
        torch.cuda.synchronize()        # the forward has completed: its hints are readable
        torch.autograd.backward([out, nxt], [go.cuda(), gs.cuda()])
        torch.cuda.synchronize()
        return out, nxt, [t.grad for t in ins]

    x, f, q, k, fk, s, go, gs = make_config_inputs(4, 300, 64, 64, torch.float16, seed=71, state_std=0.2)
    out, nxt, grads = run((x, f, q, k, fk, s), go, gs)
    assert seen[-1] == _lib.FLAG_NO_FIXUP, seen
    check((x, f, q, k, fk, s), go, gs, out, nxt, grads, torch.float16)

    x, f, q, k, fk, s, go, gs = make_reference_test_inputs(4, 200, 64, 64, torch.float16, seed=3)
    x, q, k = x / 8, q / 8, k / 8
    out, nxt, grads = run((x, f, q, k, fk, s), go, gs)
    assert seen[-1] == _lib.FLAG_BLOCKWISE, seen
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    floors = gate_grad_floor((x, f, q, k, fk, s), go, c_oracle.lfw_forward(x, f, q, k, fk, s)[0], r_grads)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g, r, torch.float16, n, tol=(2e-1, 4e-2) if n in ("d_f", "d_f_key") else TOL_CHUNK,
                     floor=floors.get(n, 0.0))


def test_backward_before_the_hints_arrive_takes_the_default_path(monkeypatch):
    """a backward issued while the forward may still be running must not wait: it runs the default call"""
    from t2fw.functional_lfw import LFWFunction
    from t2fw_amd import path_hint
    monkeypatch.setattr(path_hint.ForwardHints, "hinted_rows", lambda self: None)
    x, f, q, k, fk, s, go, gs = make_config_inputs(3, 130, 64, 64, torch.float16, seed=73, state_std=0.2)
    f = f.clone()
    f[1, 64:96, 3] = 0.15
    ins = [t.cuda().requires_grad_(True) for t in (x, f, q, k, fk, s)]
    out, nxt = LFWFunction.apply(*ins)
    torch.autograd.backward([out, nxt], [go.cuda(), gs.cuda()])
    torch.cuda.synchronize()
    check((x, f, q, k, fk, s), go, gs, out, nxt, [t.grad for t in ins], torch.float16)
