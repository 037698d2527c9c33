"""GPU parity of the fused sigmoid gating (gate kernels + LFWGatedFunction).

The gates are checked against the library's sigmoid evaluated in float64 on the CPU, to two
units in the last place of the tensor dtype; the recurrence is then checked against the CPU
oracle run on the gates the kernel produced, and the logit gradients against the oracle's gate
gradients times f(1-f) in float64."""
import pytest
import torch

from oracle import c_oracle
from tests.test_lfw_gpu import TOL, TOL_CHUNK, TOL_CHUNK_GATE, assert_close, gate_grad_floor, on_chunk_path

pytestmark = pytest.mark.gpu

ULP = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -22}


def sigmoid64(z):
    return torch.sigmoid(z.double().cpu())


def assert_gate(got, logits, dtype):
    ref = sigmoid64(logits.cpu())
    got = got.double().cpu()
    # two units in the last place of the result, plus fp16's smallest normal for results that
    # round towards zero there
    bound = 2 * ULP[dtype] * ref + (6.2e-5 if dtype == torch.float16 else 1e-30)
    bad = (got - ref).abs() > bound
    assert not bad.any(), "sigmoid: %d outside, worst %.3e" % (int(bad.sum()), float((got - ref).abs().max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n_f,n_fk", [(0, 0), (1, 0), (0, 7), (8, 8), (1000, 333), (64 * 1024 + 5, 3 * 64 * 1024 + 1),
                                      (5 * 1024 * 1024, 5 * 1024 * 1024)])
def test_gate_forward_and_backward_kernels(dtype, n_f, n_fk):
    from t2fw_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(n_f + 3 * n_fk)
    zf = (torch.randn(n_f, generator=g) * 4).to(dtype).cuda()
    zk = (torch.randn(n_fk, generator=g) * 4).to(dtype).cuda()
    if n_f > 4:
        zf[:4] = torch.tensor([-30.0, 30.0, 0.0, -11.0], dtype=dtype)
    f, fk = torch.full_like(zf, -1), torch.full_like(zk, -1)
    code = _lib.DTYPE_CODE[dtype]
    st = _lib.current_stream_handle(zf.device)
    _lib.check(lib.t2fw_gate_forward(_lib.ptr(zf), _lib.ptr(zk), _lib.ptr(f), _lib.ptr(fk), n_f, n_fk, code, st))
    torch.cuda.synchronize()
    assert_gate(f, zf, dtype)
    assert_gate(fk, zk, dtype)
    assert (f >= 0).all() and (f <= 1).all() and (fk >= 0).all() and (fk <= 1).all()

    df = torch.randn(n_f, generator=g).to(dtype).cuda()
    dk = torch.randn(n_fk, generator=g).to(dtype).cuda()
    ref_f = df.double() * f.double() * (1 - f.double())
    ref_k = dk.double() * fk.double() * (1 - fk.double())
    of, ok = torch.full_like(df, 7), torch.full_like(dk, 7)
    _lib.check(lib.t2fw_gate_backward(_lib.ptr(df), _lib.ptr(dk), _lib.ptr(f), _lib.ptr(fk), _lib.ptr(of), _lib.ptr(ok),
                                      n_f, n_fk, code, st))
    # in place over the gate gradients
    df2, dk2 = df.clone(), dk.clone()
    _lib.check(lib.t2fw_gate_backward(_lib.ptr(df2), _lib.ptr(dk2), _lib.ptr(f), _lib.ptr(fk), _lib.ptr(df2),
                                      _lib.ptr(dk2), n_f, n_fk, code, st))
    torch.cuda.synchronize()
    for got, ref in ((of, ref_f), (ok, ref_k), (df2, ref_f), (dk2, ref_k)):
        err = (got.double() - ref).abs()
        assert (err <= 2 * ULP[dtype] * ref.abs() + 1e-7).all(), float(err.max())
    assert torch.equal(of, df2) and torch.equal(ok, dk2)


def test_gate_entry_points_reject_bad_arguments():
    from t2fw_amd import _lib
    lib = _lib.load()
    z = torch.zeros(64, dtype=torch.float16, device="cuda")
    o = torch.zeros(64, dtype=torch.float16, device="cuda")
    st = _lib.current_stream_handle(z.device)
    code = _lib.DTYPE_CODE[torch.float16]
    assert lib.t2fw_gate_forward(_lib.ptr(z), _lib.ptr(z), _lib.ptr(o), _lib.ptr(o), -1, 0, code, st) != 0
    assert lib.t2fw_gate_forward(_lib.ptr(z), _lib.ptr(z), _lib.ptr(o), _lib.ptr(o), 8, 8, 99, st) != 0
    assert lib.t2fw_gate_forward(None, _lib.ptr(z), _lib.ptr(o), _lib.ptr(o), 8, 8, code, st) != 0
    assert lib.t2fw_gate_forward(z.data_ptr() + 2, _lib.ptr(z), _lib.ptr(o), _lib.ptr(o), 8, 8, code, st) != 0
    assert lib.t2fw_gate_backward(_lib.ptr(z), _lib.ptr(z), None, _lib.ptr(z), _lib.ptr(o), _lib.ptr(o), 8, 8, code, st) != 0
    # an empty array may come with a null pointer
    assert lib.t2fw_gate_forward(None, _lib.ptr(z), None, _lib.ptr(o), 0, 8, code, st) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,B,T,D,K", [(torch.float16, 3, 200, 64, 64), (torch.bfloat16, 2, 130, 64, 64),
                                           (torch.float32, 2, 77, 33, 17), (torch.float16, 2, 50, 32, 16)])
def test_gated_function_matches_oracle(dtype, B, T, D, K):
    from t2fw_amd import LFWGatedFunction, sigmoid_gates
    g = torch.Generator().manual_seed(T)
    scale = 0.125 if on_chunk_path(dtype, D, K) else 1.0
    x = (torch.randn(B, T, D, generator=g) * scale).to(dtype)
    zf = (torch.randn(B, T, D, generator=g) + 2).to(dtype)
    q = (torch.randn(B, T, K, generator=g) * scale).to(dtype)
    k = (torch.randn(B, T, K, generator=g) * scale).to(dtype)
    zk = (torch.randn(B, T, K, generator=g) + 2).to(dtype)
    s = (torch.randn(B, D, K, generator=g) * 0.1).to(dtype)
    go = torch.randn(B, T, D, generator=g).to(dtype)
    gs = (torch.randn(B, D, K, generator=g) * 0.1).to(dtype)

    ins = [t.cuda().requires_grad_(True) for t in (x, zf, q, k, zk, s)]
    out, nxt = LFWGatedFunction.apply(*ins)
    out.backward(go.cuda(), retain_graph=True)
    nxt.backward(gs.cuda())
    torch.cuda.synchronize()

    f, fk = sigmoid_gates(ins[1].detach(), ins[4].detach())
    assert_gate(f, zf, dtype)
    assert_gate(fk, zk, dtype)
    f, fk = f.cpu(), fk.cpu()
    inputs = (x, f, q, k, fk, s)
    r_out, r_nxt = c_oracle.lfw_forward(*inputs)
    r_grads = [torch.as_tensor(t).double() for t in c_oracle.lfw_backward(go, gs, *inputs)]
    chunk = on_chunk_path(dtype, D, K)
    tol = TOL_CHUNK if chunk else TOL[dtype]
    gate_tol = TOL_CHUNK_GATE if chunk else TOL[dtype]
    floors = gate_grad_floor(inputs, go, r_out, r_grads) if chunk else {}
    assert_close(out, r_out, dtype, "outputs", tol=tol)
    assert_close(nxt, r_nxt, dtype, "next_state", tol=tol)
    # d_logit = d_gate * gate * (1 - gate); the bound of d_gate carries over scaled by max gate(1-gate) = 1/4
    slope_f, slope_k = f.double() * (1 - f.double()), fk.double() * (1 - fk.double())
    refs = [r_grads[0], r_grads[1] * slope_f, r_grads[2], r_grads[3], r_grads[4] * slope_k, r_grads[5]]
    names = ("d_x", "d_f_logit", "d_q", "d_k", "d_fk_logit", "d_state")
    for n, t, r in zip(names, ins, refs):
        if n == "d_f_logit":
            assert_close(t.grad, r, dtype, n, tol=gate_tol, floor=0.25 * floors.get("d_f", 0.0))
        elif n == "d_fk_logit":
            assert_close(t.grad, r, dtype, n, tol=gate_tol, floor=0.25 * floors.get("d_f_key", 0.0))
        else:
            assert_close(t.grad, r, dtype, n, tol=tol)


@pytest.mark.parametrize("logit_mean,bound", [(-2.0, 8e-2), (-1.0, 4e-2), (0.0, 2e-2)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_logit_gradients_at_fast_decay(dtype, logit_mean, bound):
    """Gates from sigmoid(N(m, 1)) for m down to -2 (gates down to 1e-3; the chunk-parallel backward
    declines most rows at m = -2 and the block-wise kernel takes them).  d_gate at a step with a small
    gate is (gate * d_gate) / gate, with an absolute error set by the bf16 rounding of the terms that
    cancel in gate * d_gate; the logit gradient multiplies the gate back in.  Bounds: the worst of a
    randomized sweep was 4.9e-2 / 1.8e-2 / 1.1e-2 of max|ref| for m = -2 / -1 / 0."""
    from t2fw_amd import LFWGatedFunction, sigmoid_gates
    B, T = 6, 200
    g = torch.Generator().manual_seed(11)
    x, q, k = [(torch.randn(B, T, 64, generator=g) * 0.125).to(dtype) for _ in range(3)]
    zf, zk = [(torch.randn(B, T, 64, generator=g) + logit_mean).to(dtype) for _ in range(2)]
    s = (torch.randn(B, 64, 64, generator=g) * 0.3).to(dtype)
    go = torch.randn(B, T, 64, generator=g).to(dtype)
    gs = (torch.randn(B, 64, 64, generator=g) * 0.1).to(dtype)
    ins = [t.cuda().requires_grad_(True) for t in (x, zf, q, k, zk, s)]
    out, nxt = LFWGatedFunction.apply(*ins)
    torch.autograd.backward([out, nxt], [go.cuda(), gs.cuda()])
    torch.cuda.synchronize()
    f, fk = [t.cpu() for t in sigmoid_gates(ins[1].detach(), ins[4].detach())]
    inputs = (x, f, q, k, fk, s)
    r_out, _ = c_oracle.lfw_forward(*inputs)
    r_grads = [torch.as_tensor(t).double() for t in c_oracle.lfw_backward(go, gs, *inputs)]
    assert_close(out, r_out, dtype, "outputs", tol=TOL_CHUNK)
    for i, n in ((0, "d_x"), (2, "d_q"), (3, "d_k"), (5, "d_state")):
        assert_close(ins[i].grad, r_grads[i], dtype, n, tol=TOL_CHUNK)
    for i, gate, n in ((1, f, "d_f_logit"), (4, fk, "d_fk_logit")):
        ref = r_grads[i] * gate.double() * (1 - gate.double())
        err = (ins[i].grad.double().cpu() - ref).abs().max() / ref.abs().max()
        assert err <= bound, (n, float(err))


def test_gated_function_equals_ungated_on_its_own_gates():
    """same kernels underneath: outputs and non-gate gradients are bit-identical to LFWFunction on
    sigmoid_gates' output, and the logit gradients are the gate gradients times f(1-f)"""
    from t2fw_amd import LFWFunction, LFWGatedFunction, sigmoid_gates
    dtype = torch.float16
    g = torch.Generator().manual_seed(5)
    B, T, D, K = 4, 300, 64, 64
    mk = lambda *sh: torch.randn(*sh, generator=g)
    x, q, k = [(mk(B, T, n) / 8).to(dtype).cuda() for n in (D, K, K)]
    zf, zk = [(mk(B, T, n) + 2).to(dtype).cuda() for n in (D, K)]
    s = (mk(B, D, K) * 0.1).to(dtype).cuda()
    go = mk(B, T, D).to(dtype).cuda()
    a = [t.clone().requires_grad_(True) for t in (x, zf, q, k, zk, s)]
    out_a, nxt_a = LFWGatedFunction.apply(*a)
    out_a.backward(go)
    f, fk = sigmoid_gates(zf, zk)
    b = [t.clone().requires_grad_(True) for t in (x, f, q, k, fk, s)]
    out_b, nxt_b = LFWFunction.apply(*b)
    out_b.backward(go)
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b) and torch.equal(nxt_a, nxt_b)
    for i in (0, 2, 3, 5):
        assert torch.equal(a[i].grad, b[i].grad), i
    for i, gate in ((1, f), (4, fk)):
        ref = b[i].grad.double() * gate.double() * (1 - gate.double())
        err = (a[i].grad.double() - ref).abs()
        assert (err <= 2 * ULP[dtype] * ref.abs() + 1e-7).all(), (i, float(err.max()))
