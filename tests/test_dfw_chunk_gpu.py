"""GPU parity of the block-wise matrix-core kernels of the delta rule (D = M = 64; fp32 tensors, and fp16 / bf16
ones in the tests at the end) against the CPU oracle (fp64, same inputs), through the C ABI.  The operands of every contraction are split into a
bf16 head and remainder, so the results are held to the tolerance of the exact per-step kernels
(tests/test_dfw_gpu.py), not to a 16-bit one; the exact kernels (flag 1) are run on the same inputs."""
import pytest
import torch

from oracle.dfw_ref import dfw_deltas, dfw_reference_grads
from tests.test_dfw_gpu import NAMES, TOL_DFW, make_inputs
from tests.test_lfw_gpu import assert_close

pytestmark = pytest.mark.gpu
TOL = TOL_DFW[torch.float32]


def run_abi(q, k, v, s, go, gs, flags=0, backward=True):
    from t2fw_amd import _lib
    lib = _lib.load()
    q, k, v, s = [t.cuda() for t in (q, k, v, s)]
    B, T, D = v.shape
    M = q.shape[2]
    code = _lib.DTYPE_CODE[v.dtype]
    st = _lib.current_stream_handle(v.device)
    out, delta, fin = torch.empty_like(v), torch.empty_like(v), torch.empty_like(s)
    P = _lib.ptr
    _lib.check(lib.t2fw_dfw_forward(P(q), P(k), P(v), P(s), P(out), P(fin), P(delta), B, T, D, M, code, flags, st))
    grads = None
    if backward:
        go_d, gs_d = go.cuda(), gs.cuda()
        grads = [torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(s)]
        _lib.check(lib.t2fw_dfw_backward(P(go_d), P(gs_d), P(q), P(k), P(delta), P(fin), *[P(t) for t in grads],
                                         B, T, D, M, code, flags, st))
    torch.cuda.synchronize()
    return out, fin, delta, grads


def check(B, T, seed, key_scale=None, backward=True):
    q, k, v, s, go, gs = make_inputs(B, T, 64, 64, torch.float32, seed)
    if key_scale is not None:          # unnormalised keys of a chosen size instead of the reference test's
        g = torch.Generator().manual_seed(seed + 1)
        k = torch.randn(B, T, 64, generator=g) * key_scale
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    r_delta = dfw_deltas(q.double(), k.double(), v.double(), s.double())
    for flags in (0, 1):
        tag = " (flags %d)" % flags
        out, fin, delta, grads = run_abi(q, k, v, s, go, gs, flags, backward)
        assert_close(out, r_out, torch.float32, "outputs" + tag, tol=TOL)
        assert_close(fin, r_fin, torch.float32, "final_state" + tag, tol=TOL)
        assert_close(delta, r_delta, torch.float32, "delta" + tag, tol=TOL)
        if backward:
            for n, g, r in zip(NAMES, grads, r_grads):
                assert_close(g, r, torch.float32, n + tag, tol=TOL)


@pytest.mark.parametrize("T", [1, 15, 16, 17, 31, 32, 33, 47, 48, 64, 65, 100, 257, 1024])
def test_sequence_lengths_around_block_and_stage_boundaries(T):
    check(3, T, seed=100 + T)


@pytest.mark.parametrize("B", [1, 8, 9, 130, 300])
def test_batch_sizes_around_the_grid_padding(B):
    check(B, 70, seed=200 + B)


@pytest.mark.parametrize("scale", [0.05, 0.125, 0.2])
def test_unnormalised_keys(scale):
    """|k|^2 up to about 2.5: the triangular factors are far from the identity"""
    check(2, 200, seed=300, key_scale=scale)


def test_long_sequence():
    """T = 2050: 65 stages of the forward, 129 of the key side, a partial last block"""
    check(2, 2050, seed=77)


def test_large_values_and_states():
    """values of size 100 and a state of size 50: the relative accuracy of the split operands does not depend on scale"""
    q, k, v, s, go, gs = make_inputs(3, 130, 64, 64, torch.float32, seed=31)
    v, s = v * 100.0, s * 50.0
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    out, fin, delta, grads = run_abi(q, k, v, s, go, gs)
    assert_close(out, r_out, torch.float32, "outputs", tol=TOL)
    assert_close(fin, r_fin, torch.float32, "final_state", tol=TOL)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g, r, torch.float32, n, tol=TOL)


def test_headline_shape_rows_against_the_oracle():
    """B = 96, T = 1024 as the benchmark runs it; the oracle on three rows"""
    q, k, v, s, go, gs = make_inputs(96, 1024, 64, 64, torch.float32, seed=5)
    out, fin, delta, grads = run_abi(q, k, v, s, go, gs)
    rows = [0, 47, 95]
    r_out, r_fin, r_grads = dfw_reference_grads(q[rows], k[rows], v[rows], s[rows], go[rows], gs[rows])
    assert_close(out[rows], r_out, torch.float32, "outputs", tol=TOL)
    assert_close(fin[rows], r_fin, torch.float32, "final_state", tol=TOL)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[rows], r, torch.float32, n, tol=TOL)


@pytest.mark.parametrize("B,T", [(3, 100), (9, 257), (2, 1024)])
def test_single_bf16_operand_mode(B, T):
    """flag 16: one bf16 operand per product instead of head + remainder.  Held to 1e-2 of max|ref| per result,
    the bound of the other 16-bit-operand kernels of this library; different from the default's results (so the
    flag is seen to select other kernels), and the default's stay inside the fp32 tolerance."""
    q, k, v, s, go, gs = make_inputs(B, T, 64, 64, torch.float32, seed=400 + T)
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    out, fin, delta, grads = run_abi(q, k, v, s, go, gs, flags=16)
    out0 = run_abi(q, k, v, s, go, gs, flags=0)[0]
    assert not torch.equal(out, out0)
    for n, got, ref in [("outputs", out, r_out), ("final_state", fin, r_fin)] + [(n, g, r) for n, g, r in zip(NAMES, grads, r_grads)]:
        err = (got.double().cpu() - ref.double()).abs().max().item()
        scale = ref.double().abs().max().item()
        assert err <= 1e-2 * scale, "%s: max error %.3e against max|ref| %.3e" % (n, err, scale)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,T", [(3, 1), (3, 17), (2, 100), (9, 257), (2, 1024)])
def test_16_bit_tensors(dtype, B, T):
    """fp16 / bf16 tensors run the same block-wise kernels (loads and stores convert; all arithmetic as for fp32
    tensors).  Against the fp64 oracle on the same 16-bit inputs, to the tolerance of the exact per-step kernels
    for the type; the saved deltas and the final state that the backward starts from are 16-bit there as here.
    The error of the block-wise kernels stays within twice that of the exact kernels on the same inputs (both are
    dominated by the rounding of what is stored), and flag 16 selects other kernels."""
    q, k, v, s, go, gs = make_inputs(B, T, 64, 64, dtype, seed=600 + T)
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    r_delta = dfw_deltas(q.double(), k.double(), v.double(), s.double())
    tol = TOL_DFW[dtype]
    refs = [("outputs", r_out), ("final_state", r_fin), ("delta", r_delta)] + list(zip(NAMES, r_grads))
    worst = {}
    for flags in (1, 0, 16):
        out, fin, delta, grads = run_abi(q, k, v, s, go, gs, flags)
        got = [out, fin, delta] + grads
        for (n, r), t in zip(refs, got):
            assert t.dtype == dtype
            assert_close(t, r, dtype, "%s (flags %d)" % (n, flags), tol=tol)
            worst[(flags, n)] = ((t.double().cpu() - r.double()).abs().max() / r.double().abs().max()).item()
    for n, _ in refs:
        floor = 2.0 ** (-11 if dtype == torch.float16 else -8)          # one rounding of the largest element
        assert worst[(0, n)] <= 2.0 * max(worst[(1, n)], floor), (n, worst[(0, n)], worst[(1, n)])
    if T > 1:
        assert not torch.equal(run_abi(q, k, v, s, go, gs, 0)[0], run_abi(q, k, v, s, go, gs, 16)[0])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_16_bit_tensors_through_the_autograd_function(dtype):
    """DFWFunction on 16-bit tensors: fp16 with the default (split) operands, bf16 with single bf16 operands
    (flag 16; the wrapper's choice for that type) -- bit-identical to the C-ABI call with those flags, and inside
    the type's tolerance against the oracle."""
    from t2fw.functional_dfw import DFWFunction
    q, k, v, s, go, gs = make_inputs(5, 200, 64, 64, dtype, seed=19)
    ins = [t.cuda().requires_grad_(True) for t in (q, k, v, s)]
    out, fin = DFWFunction.apply(*ins)
    torch.autograd.backward([out, fin], [go.cuda(), gs.cuda()])
    torch.cuda.synchronize()
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    assert out.dtype == dtype and fin.dtype == dtype
    assert_close(out, r_out, dtype, "outputs", tol=TOL_DFW[dtype])
    assert_close(fin, r_fin, dtype, "final_state", tol=TOL_DFW[dtype])
    for n, t, r in zip(NAMES, ins, r_grads):
        assert t.grad.dtype == dtype
        assert_close(t.grad, r, dtype, n, tol=TOL_DFW[dtype])
    a_out, a_fin, _, a_grads = run_abi(q, k, v, s, go, gs, flags=16 if dtype == torch.bfloat16 else 0)
    assert torch.equal(out, a_out) and torch.equal(fin, a_fin)
    for t, g in zip(ins, a_grads):
        assert torch.equal(t.grad, g)


def test_the_wrapper_s_flag_choice_yields_to_the_environment(monkeypatch):
    from t2fw_amd import _lib
    from t2fw_amd.functional_dfw import _dfw_flags
    monkeypatch.delenv("T2FW_FLAGS", raising=False)
    assert _dfw_flags(torch.bfloat16) == _lib.FLAG_BF16_OPERANDS
    assert _dfw_flags(torch.float16) == 0 and _dfw_flags(torch.float32) == 0
    monkeypatch.setenv("T2FW_FLAGS", "1")
    assert _dfw_flags(torch.bfloat16) == 1


def test_autograd_function_uses_the_block_wise_kernels():
    from t2fw.functional_dfw import DFWFunction
    q, k, v, s, go, gs = make_inputs(4, 130, 64, 64, torch.float32, seed=9)
    ins = [t.cuda().requires_grad_(True) for t in (q, k, v, s)]
    out, fin = DFWFunction.apply(*ins)
    out.backward(go.cuda(), retain_graph=True)
    fin.backward(gs.cuda())
    torch.cuda.synchronize()
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    assert_close(out, r_out, torch.float32, "outputs", tol=TOL)
    for n, t, r in zip(NAMES, ins, r_grads):
        assert_close(t.grad, r, torch.float32, n, tol=TOL)
