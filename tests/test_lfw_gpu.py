"""GPU parity of the LFW kernels against the CPU oracle (fp64, same quantised inputs).

Mirrors the reference's own test (tests/test_lfw.py:28-103): same shape grid, gate
construction, two-call backward protocol; the reference's tolerances are the outer
bound and a tighter stated tolerance is enforced on top.  All calls go through the
C ABI (directly or via the autograd wrapper that binds it)."""
import math

import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import (err_stats, make_config_inputs, make_reference_test_inputs,
                             reference_shape_grid)

pytestmark = pytest.mark.gpu

# Stated tolerances: |got-ref| <= rtol*|ref| + afrac*max|ref|.
# Exact scan kernels (fp32 state, result rounded once to the I/O dtype):
TOL = {
    torch.float16: (2e-3, 1e-3),
    torch.bfloat16: (1.6e-2, 8e-3),
    torch.float32: (2e-5, 2e-5),
    torch.float64: (1e-12, 1e-12),
}
# Chunked matrix-core kernels (D = K = 64, 16-bit tensors): operands of the contractions are
# rounded to bf16 (2^-9 relative), accumulation is fp32.  The gate gradients are differences
# of products of such quantities and carry a wider bound.
TOL_CHUNK = (2e-2, 1e-2)
TOL_CHUNK_GATE = (2e-2, 2e-2)


def on_chunk_path(dtype, D, K):
    import os
    return D == 64 and K == 64 and dtype in (torch.float16, torch.bfloat16) and \
        not (int(os.environ.get("T2FW_FLAGS", "0")) & 1)


def gate_grad_floor(inputs, go, r_out, r_grads):
    """Natural magnitude of the terms whose difference forms f*d_f and fkey*d_fkey
    (g.o - x.dx and q.dq - k.dk): the absolute error of the chunked kernels scales with
    these, also where the exact gradient happens to vanish (e.g. a zero initial state)."""
    x, f, q, k, fk, s = [t.double() for t in inputs]
    d_x, d_f, d_q, d_k, d_fk, d_s = [torch.as_tensor(t).double() for t in r_grads]
    fl_f = float(((go.double() * torch.as_tensor(r_out).double()).abs() + (x * d_x).abs()).max()) if x.numel() else 0.0
    fl_k = float(((q * d_q).abs() + (k * d_k).abs()).max()) if q.numel() else 0.0
    return {"d_f": fl_f, "d_f_key": fl_k}


# (rtol, afrac, tensor) -> largest |err| / bound seen in this session; printed after the run so the
# stated tolerances can be compared with what the kernels actually use of them
TOLERANCE_USE = {}


def assert_close(got, ref, dtype, what, scale=1.0, tol=None, floor=0.0):
    rtol, afrac = tol if tol is not None else TOL[dtype]
    got = got.detach().double().cpu()
    ref = torch.as_tensor(ref).double()
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    if ref.numel() == 0:
        return
    assert torch.isfinite(got).all(), what + " has non-finite values"
    bound = scale * (rtol * ref.abs() + afrac * max(float(ref.abs().max()), floor))
    bad = (got - ref).abs() > bound
    key = (rtol, afrac, what.split("[")[0].split(" (")[0])
    TOLERANCE_USE[key] = max(TOLERANCE_USE.get(key, 0.0), float(((got - ref).abs() / bound.clamp_min(1e-300)).max()))
    assert not bad.any(), "%s: %d/%d outside tolerance, max-abs err %.3e (max|ref| %.3e)" % (
        what, int(bad.sum()), ref.numel(), float((got - ref).abs().max()), float(ref.abs().max()))


def run_autograd(inputs, go, gs):
    """two-call backward protocol of tests/test_lfw.py:59-62 through LFWFunction"""
    from t2fw.functional_lfw import LFWFunction
    ins = [t.cuda().requires_grad_(True) for t in inputs]
    out, nxt = LFWFunction.apply(*ins)
    out.backward(go.cuda(), retain_graph=True)
    nxt.backward(gs.cuda())
    torch.cuda.synchronize()
    return out, nxt, [t.grad for t in ins]


def oracle_all(inputs, go, gs):
    out, nxt = c_oracle.lfw_forward(*inputs)
    grads = c_oracle.lfw_backward(go, gs, *inputs)
    return out, nxt, grads


NAMES = ("d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state")


def check_all(inputs, go, gs, dtype, scale=1.0):
    out, nxt, grads = run_autograd(inputs, go, gs)
    r_out, r_nxt, r_grads = oracle_all(inputs, go, gs)
    assert out.dtype == dtype and nxt.dtype == dtype
    chunk = on_chunk_path(dtype, inputs[0].shape[2], inputs[2].shape[2])
    tol = TOL_CHUNK if chunk else None
    floors = gate_grad_floor(inputs, go, r_out, r_grads) if chunk else {}
    assert_close(out, r_out, dtype, "outputs", scale, tol)
    assert_close(nxt, r_nxt, dtype, "next_state", scale, tol)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert g.dtype == dtype
        assert_close(g, r, dtype, n, scale, (TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK) if chunk else None,
                     floors.get(n, 0.0))
    # outer bound: the reference's own tolerances (tests/test_lfw.py:65,92)
    if dtype == torch.float16:
        assert torch.allclose(out.double().cpu(), torch.as_tensor(r_out), atol=1e-2, rtol=1e-1)
        for g, r in zip(grads, r_grads):
            assert torch.allclose(g.double().cpu(), torch.as_tensor(r), atol=0.1, rtol=1e-1)


@pytest.mark.parametrize("bsz,seqlen,dim", list(reference_shape_grid()))
def test_reference_shape_grid_fp16(bsz, seqlen, dim):
    kdim = math.ceil(dim / 2)
    x, f, q, k, fk, s, go, gs = make_reference_test_inputs(bsz, seqlen, dim, kdim, torch.float16,
                                                           seed=1000 + bsz * 7 + seqlen + dim)
    check_all((x, f, q, k, fk, s), go, gs, torch.float16)


def test_cfg1_readme_shape_fp32():
    x, f, q, k, fk, s, go, gs = make_config_inputs(1, 4, 4, 4, torch.float32, seed=0, in_scale=1.0,
                                                    gate_mean=0.0, state_std=1.0, gstate_std=1.0)
    check_all((x, f, q, k, fk, s), go, gs, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64, torch.float16])
@pytest.mark.parametrize("shape", [(3, 70, 64, 64), (2, 33, 5, 130), (2, 40, 130, 3), (1, 9, 1, 1),
                                   (2, 17, 24, 300)])
def test_general_shapes_all_dtypes(dtype, shape):
    B, T, D, K = shape
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, D, K, dtype, seed=5, in_scale=0.5,
                                                    gate_mean=1.0, state_std=0.5, gstate_std=0.5)
    check_all((x, f, q, k, fk, s), go, gs, dtype)


WIDE_SHAPES = [(1, 6, 3, 100), (1, 6, 100, 3), (1, 5, 2, 600), (1, 5, 600, 2), (1, 4, 2, 2048), (1, 4, 2048, 2)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", WIDE_SHAPES)
def test_wide_states_every_lane_geometry(dtype, shape):
    """State rows of 65..128, 513..1024 and 2048 columns on either side: 32 lanes per row and 16 / 32
    columns per lane, which no narrower shape reaches."""
    B, T, D, K = shape
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, D, K, dtype, seed=6, in_scale=0.5,
                                                    gate_mean=1.0, state_std=0.5, gstate_std=0.5)
    check_all((x, f, q, k, fk, s), go, gs, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(1, 5, 3, 5000), (1, 5, 5000, 3), (2, 9, 2, 2049), (1, 4, 2100, 2500)])
def test_states_wider_than_a_lane_group_run_in_column_passes(dtype, shape):
    """More than 2048 columns on either side (the reference tiles K over blocks,
    t2fw/csrc/lfw_kernel.cu:146-155): several launches, each over a window of columns, the later ones
    adding to the outputs.  16-bit outputs are rounded once per launch, hence the scale."""
    B, T, D, K = shape
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, D, K, dtype, seed=13, in_scale=0.5,
                                                    gate_mean=1.0, state_std=0.5, gstate_std=0.5)
    check_all((x, f, q, k, fk, s), go, gs, dtype, scale=1.0 if dtype == torch.float32 else 3.0)


@pytest.mark.parametrize("C", [1, 7, 16, 64, 100, 1000])
def test_checkpoint_interval_any_value(C, monkeypatch):
    # C need not divide T; C > T keeps a single checkpoint
    monkeypatch.setenv("T2FW_CKPT_INTERVAL", str(C))
    x, f, q, k, fk, s, go, gs = make_config_inputs(2, 150, 64, 64, torch.float16, seed=9,
                                                    gate_mean=2.0, state_std=0.3)
    check_all((x, f, q, k, fk, s), go, gs, torch.float16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_scan_kernels_at_the_matrix_core_shape(dtype, monkeypatch):
    # D = K = 64 through the exact scan kernels only (the row-level fallback of the chunked path)
    monkeypatch.setenv("T2FW_FLAGS", "1")
    x, f, q, k, fk, s, go, gs = make_config_inputs(3, 200, 64, 64, dtype, seed=12, state_std=0.3)
    check_all((x, f, q, k, fk, s), go, gs, dtype)


def test_checkpoints_hold_chunk_start_states():
    from t2fw_amd import _lib
    lib = _lib.load()
    B, T, D, K, C = 2, 100, 64, 64, 32
    x, f, q, k, fk, s, _, _ = make_config_inputs(B, T, D, K, torch.float32, seed=3, state_std=0.5)
    dev = [t.cuda() for t in (x, f, q, k, fk, s)]
    out, nxt = torch.empty_like(dev[0]), torch.empty_like(dev[5])
    nc = lib.t2fw_lfw_num_ckpt(T, C)
    assert nc == 4
    ckpt = torch.empty(B, nc, D, K, device="cuda")
    _lib.check(lib.t2fw_lfw_forward(*[_lib.ptr(t) for t in dev], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt),
                                    B, T, D, K, C, _lib.F32, 0, None, 0, _lib.current_stream_handle(out.device)))
    torch.cuda.synchronize()
    for c in range(nc):
        if c == 0:
            ref = s.double().numpy()
        else:
            _, ref = c_oracle.lfw_forward(x[:, :c * C], f[:, :c * C], q[:, :c * C], k[:, :c * C], fk[:, :c * C], s)
        assert_close(ckpt[:, c], ref, torch.float32, "ckpt[%d]" % c)


def test_segment_composition_on_device():
    # running [0,T1) then [T1,T) carrying next_state == running [0,T)
    from t2fw.functional_lfw import LFWFunction
    x, f, q, k, fk, s, _, _ = make_config_inputs(4, 200, 64, 64, torch.float32, seed=4, state_std=0.3)
    d = [t.cuda() for t in (x, f, q, k, fk, s)]
    with torch.no_grad():
        o, n = LFWFunction.apply(*d)
        o1, m = LFWFunction.apply(*[t[:, :77].contiguous() for t in d[:5]], d[5])
        o2, n2 = LFWFunction.apply(*[t[:, 77:].contiguous() for t in d[:5]], m)
    assert torch.allclose(torch.cat([o1, o2], 1), o, atol=1e-5, rtol=1e-5)
    assert torch.allclose(n2, n, atol=1e-5, rtol=1e-5)


def test_empty_and_degenerate_inputs():
    from t2fw.functional_lfw import LFWFunction
    s = torch.randn(2, 4, 3, device="cuda")
    e = lambda w: torch.empty(2, 0, w, device="cuda")
    o, n = LFWFunction.apply(e(4), e(4), e(3), e(3), e(3), s)
    assert o.shape == (2, 0, 4) and torch.equal(n, s)
    z = torch.empty(0, 5, 4, device="cuda")
    zk = torch.empty(0, 5, 3, device="cuda")
    o, n = LFWFunction.apply(z, z, zk, zk, zk, torch.empty(0, 4, 3, device="cuda"))
    assert o.shape == (0, 5, 4) and n.shape == (0, 4, 3)


def test_wrapper_errors_match_reference_behaviour():
    from t2fw.functional_lfw import LFWFunction
    x = torch.randn(2, 5, 4, device="cuda")
    k = torch.randn(2, 5, 3, device="cuda")
    s = torch.randn(2, 4, 3, device="cuda")
    with pytest.raises(AssertionError):                       # functional_lfw.py:42
        LFWFunction.apply(x, x[:, :4].contiguous(), k, k, k, s)
    with pytest.raises(AssertionError):                       # functional_lfw.py:46-49
        LFWFunction.apply(x, x, k.half(), k, k, s)
    with pytest.raises(RuntimeError):                         # lfw.cpp:25 contiguity
        LFWFunction.apply(x.transpose(0, 1).contiguous().transpose(0, 1), x, k, k, k, s)
    with pytest.raises(RuntimeError):                         # lfw.cpp:24 device
        LFWFunction.apply(x.cpu(), x.cpu(), k.cpu(), k.cpu(), k.cpu(), s.cpu())
