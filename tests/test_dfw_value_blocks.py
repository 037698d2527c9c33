"""Delta rule with a value width that is a multiple of 64 other than 64 (key width 64): independent [64, 64] blocks
that share q and k, run as extra batch rows on the matrix-core kernels.

CPU: the decomposition itself in float64 with the oracle in place of the two kernel calls, against the oracle on
the undivided tensors.  GPU: DFWFunction.apply against the oracle."""
import pytest
import torch

from oracle.dfw_ref import dfw_backward_two_pass, dfw_deltas, dfw_reference, dfw_reference_grads
from tests.test_dfw_gpu import NAMES, TOL_DFW, make_inputs


def _forward_by_oracle(q, k, v, s):
    assert all(t.is_contiguous() for t in (q, k, v, s))
    out, fin = dfw_reference(q, k, v, s)
    return out, fin, dfw_deltas(q, k, v, s)


def _backward_by_oracle(go, gs, q, k, delta, fin):
    assert go.is_contiguous() and gs.is_contiguous()
    return dfw_backward_two_pass(go, gs, q, k, delta, fin)


@pytest.mark.parametrize("D", [128, 192, 256])
def test_decomposition_is_the_same_recurrence(monkeypatch, D):
    from t2fw_amd import functional_dfw as F
    monkeypatch.setattr(F, "_dfw_forward", _forward_by_oracle)
    monkeypatch.setattr(F, "_dfw_backward", _backward_by_oracle)
    q, k, v, s, go, gs = [t.double() for t in make_inputs(2, 11, D, 64, torch.float32, seed=D)]
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    nd = D // 64
    out, fin, kept = F._dfw_forward_blocked(q, k, v, s, nd)
    grads = F._dfw_backward_blocked(go, gs, *kept, nd)
    for a, b in zip([out, fin] + list(grads), [r_out, r_fin] + list(r_grads)):
        assert a.shape == b.shape
        assert torch.allclose(a, b, rtol=1e-11, atol=1e-11)


def test_which_tensors_run_as_value_blocks(monkeypatch):
    from t2fw_amd.functional_dfw import _value_block_count
    monkeypatch.delenv("T2FW_FLAGS", raising=False)
    t = lambda w, dtype=torch.float32: torch.empty(2, 3, w, dtype=dtype)
    assert _value_block_count(t(128), t(64)) == 2 and _value_block_count(t(256, torch.bfloat16), t(64, torch.bfloat16)) == 4
    assert _value_block_count(t(64), t(64)) == 0            # the kernels' own shape
    assert _value_block_count(t(128), t(128)) == 0          # the key side cannot be cut
    assert _value_block_count(t(100), t(64)) == 0 and _value_block_count(t(128, torch.float64), t(64, torch.float64)) == 0
    monkeypatch.setenv("T2FW_FLAGS", "1")
    assert _value_block_count(t(128), t(64)) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,T,D", [(3, 100, 128), (2, 257, 192), (1, 17, 256)])
def test_value_blocks_through_the_autograd_function(dtype, B, T, D):
    from t2fw.functional_dfw import DFWFunction
    q, k, v, s, go, gs = make_inputs(B, T, D, 64, dtype, seed=900 + D + T)
    ins = [t.cuda().requires_grad_(True) for t in (q, k, v, s)]
    out, fin = DFWFunction.apply(*ins)
    torch.autograd.backward([out, fin], [go.cuda(), gs.cuda()])
    torch.cuda.synchronize()
    from tests.test_lfw_gpu import assert_close
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    assert out.shape == (B, T, D) and fin.shape == (B, D, 64) and out.dtype == dtype
    assert_close(out, r_out, dtype, "outputs", tol=TOL_DFW[dtype])
    assert_close(fin, r_fin, dtype, "final_state", tol=TOL_DFW[dtype])
    for n, t, r in zip(NAMES, ins, r_grads):
        assert t.grad.shape == t.shape
        assert_close(t.grad, r, dtype, n, tol=TOL_DFW[dtype])


@pytest.mark.gpu
def test_value_blocks_run_the_matrix_core_kernels(monkeypatch):
    """D = 128: not the exact kernels' bits (T2FW_FLAGS=1), and within the fp32 tolerance of them"""
    from t2fw.functional_dfw import DFWFunction
    q, k, v, s, go, gs = make_inputs(2, 300, 128, 64, torch.float32, seed=5)
    ins = [t.cuda() for t in (q, k, v, s)]
    a, _ = DFWFunction.apply(*ins)
    monkeypatch.setenv("T2FW_FLAGS", "1")
    b, _ = DFWFunction.apply(*ins)
    torch.cuda.synchronize()
    assert not torch.equal(a, b)
    assert (a.double() - b.double()).abs().max() <= 2e-4 * b.double().abs().max()
