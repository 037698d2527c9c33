"""Pins the DFW oracle (oracle/dfw_ref.py) without the reference: closed forms, the delta
rule's retrieval property, autograd vs the two-pass backward, finite differences, invariants."""
import pytest
import torch

from oracle.dfw_ref import (dfw_backward_two_pass, dfw_deltas, dfw_reference, dfw_reference_grads)

DT = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=DT)


def small(B=2, T=5, D=3, M=4, seed=0):
    return rnd(B, T, M, seed=seed), rnd(B, T, M, seed=seed + 1) * 0.5, rnd(B, T, D, seed=seed + 2), rnd(B, D, M, seed=seed + 3)


def test_zero_keys_leave_the_state_untouched():
    q, k, v, s = small()
    out, fin = dfw_reference(q, torch.zeros_like(k), v, s)
    assert torch.equal(fin, s)
    assert torch.allclose(out, torch.einsum("bdm,btm->btd", s, q), atol=1e-13)


def test_single_step_formula_and_output_uses_state_before_update():
    q, k, v, s = small(T=1)
    out, fin = dfw_reference(q, k, v, s)
    assert torch.allclose(out[:, 0], torch.einsum("bdm,bm->bd", s, q[:, 0]), atol=1e-14)
    old = torch.einsum("bdm,bm->bd", s, k[:, 0])
    assert torch.allclose(fin, s + (v[:, 0] - old)[:, :, None] * k[:, 0, None, :], atol=1e-14)


def test_unit_norm_key_retrieves_the_written_value():
    # with |k_t| = 1 the delta rule stores v_t exactly: S_t k_t = v_t
    q, k, v, s = small(T=4)
    k = k / k.norm(dim=-1, keepdim=True)
    for t in range(1, 5):
        _, fin = dfw_reference(q[:, :t], k[:, :t], v[:, :t], s)
        assert torch.allclose(torch.einsum("bdm,bm->bd", fin, k[:, t - 1]), v[:, t - 1], atol=1e-12)


def test_orthonormal_keys_store_all_values():
    B, D, M = 2, 3, 4
    v, s = rnd(B, M, D, seed=5), torch.zeros(B, D, M, dtype=DT)
    k = torch.eye(M, dtype=DT).expand(B, M, M).contiguous()
    _, fin = dfw_reference(torch.zeros_like(k), k, v, s)
    assert torch.allclose(fin, v.transpose(1, 2), atol=1e-14)


@pytest.mark.parametrize("split", [1, 3])
def test_segment_composition(split):
    q, k, v, s = small(T=6)
    out, fin = dfw_reference(q, k, v, s)
    o1, mid = dfw_reference(q[:, :split], k[:, :split], v[:, :split], s)
    o2, end = dfw_reference(q[:, split:], k[:, split:], v[:, split:], mid)
    assert torch.allclose(torch.cat([o1, o2], 1), out, atol=1e-13) and torch.allclose(end, fin, atol=1e-13)


def test_linearity_in_values_and_state():
    q, k, v, s = small(seed=4)
    v2, s2 = rnd(*v.shape, seed=40), rnd(*s.shape, seed=41)
    o1, f1 = dfw_reference(q, k, v, s)
    o2, f2 = dfw_reference(q, k, v2, s2)
    o3, f3 = dfw_reference(q, k, 2 * v - 3 * v2, 2 * s - 3 * s2)
    assert torch.allclose(o3, 2 * o1 - 3 * o2, atol=1e-12) and torch.allclose(f3, 2 * f1 - 3 * f2, atol=1e-12)


@pytest.mark.parametrize("shape", [(2, 5, 3, 4), (1, 1, 1, 1), (3, 7, 4, 2), (2, 6, 1, 5)])
def test_two_pass_backward_matches_autograd(shape):
    B, T, D, M = shape
    q, k, v, s = small(B, T, D, M, seed=9)
    go, gs = rnd(B, T, D, seed=70), rnd(B, D, M, seed=71)
    out, fin, auto = dfw_reference_grads(q, k, v, s, go, gs)
    delta = dfw_deltas(q, k, v, s)
    manual = dfw_backward_two_pass(go, gs, q, k, delta, fin)
    for a, m in zip(auto, manual):
        assert torch.allclose(a, m, atol=1e-11)


@pytest.mark.parametrize("shape", [(2, 5, 3, 4), (1, 1, 1, 1), (3, 7, 4, 2), (2, 6, 1, 5)])
def test_one_pass_backward_matches_autograd_and_the_two_pass_form(shape):
    """the reference's second derivation (t2fw/torch.py:148-242): a dropped term or a state that is not
    walked back before use shows against either of the other two"""
    from oracle.dfw_ref import dfw_backward_one_pass
    B, T, D, M = shape
    q, k, v, s = small(B, T, D, M, seed=11)
    go, gs = rnd(B, T, D, seed=72), rnd(B, D, M, seed=73)
    out, fin, auto = dfw_reference_grads(q, k, v, s, go, gs)
    one = dfw_backward_one_pass(go, gs, q, k, v, s, fin)
    two = dfw_backward_two_pass(go, gs, q, k, dfw_deltas(q, k, v, s), fin)
    for a, m, w in zip(auto, one, two):
        assert torch.allclose(a, m, atol=1e-11)
        assert torch.allclose(m, w, atol=1e-11)


def test_gradcheck_finite_differences():
    ins = [t.clone().requires_grad_(True) for t in small(B=1, T=3, D=2, M=3, seed=21)]
    assert torch.autograd.gradcheck(dfw_reference, ins, eps=1e-6, atol=1e-6)
