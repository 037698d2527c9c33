"""``lfw_apply_blocked``: value / key widths other than 64 as independent 64 x 64 blocks.

CPU: the decomposition itself (which channels go to which block, how outputs, states and gradients come back),
with the two autograd functions it calls replaced by the oracle's plain-torch recurrence, in float64 against the
same recurrence on the undivided tensors.  GPU: the real kernels against the C oracle."""
import pytest
import torch

from oracle.lfw_ref import lfw_reference
from tests.lfw_cases import make_config_inputs

SHAPES = [(128, 64), (64, 128), (128, 128), (192, 64), (64, 64), (32, 32), (100, 70), (1, 1), (65, 64)]


class _HeadsByOracle:
    @staticmethod
    def apply(x, f, q, k, fk, s):
        B, T, H, _ = x.shape
        fold = lambda t: t.transpose(1, 2).reshape(B * H, T, 64)
        out, nxt = lfw_reference(fold(x), fold(f), fold(q), fold(k), fold(fk), s.reshape(B * H, 64, 64))
        return out.view(B, H, T, 64).transpose(1, 2), nxt.view(B, H, 64, 64)


class _RowsByOracle:
    @staticmethod
    def apply(x, f, q, k, fk, s):
        return lfw_reference(x, f, q, k, fk, s)


@pytest.mark.parametrize("D,K", SHAPES)
def test_decomposition_is_the_same_recurrence(monkeypatch, D, K):
    from t2fw_amd import functional_lfw as F
    monkeypatch.setattr(F, "LFWHeadsFunction", _HeadsByOracle)
    monkeypatch.setattr(F, "LFWFunction", _RowsByOracle)
    B, T = 2, 9
    x, f, q, k, fk, s, go, gs = [t.double() for t in make_config_inputs(B, T, D, K, torch.float32, seed=D + K, state_std=0.5)]
    results = []
    for fn in (lfw_reference, None):          # None: the decomposition, whatever the tensor type
        leaves = [t.clone().requires_grad_(True) for t in (x, f, q, k, fk, s)]
        out, nxt = (fn or F._blocked)(*leaves)
        torch.autograd.backward([out, nxt], [go, gs])
        results.append([out.detach(), nxt.detach()] + [t.grad for t in leaves])
    for a, b in zip(*results):
        assert a.shape == b.shape
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_16_bit_tensors_only():
    from t2fw_amd import lfw_apply_blocked
    x, f, q, k, fk, s, go, gs = make_config_inputs(1, 3, 128, 64, torch.float32, seed=1)
    with pytest.raises(AssertionError):
        lfw_apply_blocked(x, f, q, k, fk, s)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,K", [(128, 64), (64, 128), (128, 128), (192, 64), (32, 32), (100, 70), (65, 64)])
def test_blocked_widths_on_the_matrix_cores(D, K, dtype):
    """against the fp64 C oracle at the matrix-core kernels' tolerance (the gate gradients at theirs)"""
    from oracle import c_oracle
    from t2fw_amd import lfw_apply_blocked
    from tests.test_lfw_chunk_gpu import NAMES
    from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close
    B, T = 3, 200
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, D, K, dtype, seed=3 * D + K, gate_mean=2.5, state_std=0.3)
    leaves = [t.cuda().requires_grad_(True) for t in (x, f, q, k, fk, s)]
    out, nxt = lfw_apply_blocked(*leaves)
    torch.autograd.backward([out, nxt], [go.cuda(), gs.cuda()])
    torch.cuda.synchronize()
    assert out.shape == (B, T, D) and nxt.shape == (B, D, K) and out.dtype == dtype and out.is_contiguous()
    r_out, r_nxt = c_oracle.lfw_forward(x, f, q, k, fk, s)
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    assert_close(out, r_out, dtype, "outputs", tol=TOL_CHUNK)
    assert_close(nxt, r_nxt, dtype, "next_state", tol=TOL_CHUNK)
    for n, t, r in zip(NAMES, leaves, r_grads):
        assert t.grad.shape == t.shape
        assert_close(t.grad, r, dtype, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)


@pytest.mark.gpu
def test_blocked_path_runs_the_matrix_core_kernels_not_the_exact_ones():
    """128 x 128: different from LFWFunction.apply on the same tensors (exact kernels), by no more than the
    matrix-core tolerance"""
    from t2fw_amd import LFWFunction, lfw_apply_blocked
    x, f, q, k, fk, s, go, gs = make_config_inputs(2, 300, 128, 128, torch.float16, seed=77, gate_mean=2.5, state_std=0.3)
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    a, _ = lfw_apply_blocked(*ins)
    b, _ = LFWFunction.apply(*ins)
    torch.cuda.synchronize()
    assert not torch.equal(a, b)
    assert (a.double() - b.double()).abs().max() <= 2e-2 * b.double().abs().max()
