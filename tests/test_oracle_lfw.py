"""Pins the LFW oracle (oracle/lfw_ref.py, oracle/lfw_oracle.c) WITHOUT the reference:
closed forms, brute force, invariants, autograd and finite differences.  Each check is
chosen so that a plausible slip (output taken before the update, a dropped gate, a
transposed outer product, an off-by-one in the reverse scan) fails at least one."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle.lfw_ref import (lfw_backward_closed_form, lfw_bruteforce, lfw_reference,
                            lfw_reference_grads, lfw_reference_script)
from tests.lfw_cases import make_config_inputs, make_reference_test_inputs

DT = torch.float64


def rnd(*shape, seed=0, gate=False):
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(*shape, generator=g, dtype=DT)
    return torch.sigmoid(t) if gate else t


def small_inputs(B=2, T=5, D=3, K=4, seed=0):
    return (rnd(B, T, D, seed=seed), rnd(B, T, D, seed=seed + 1, gate=True),
            rnd(B, T, K, seed=seed + 2), rnd(B, T, K, seed=seed + 3),
            rnd(B, T, K, seed=seed + 4, gate=True), rnd(B, D, K, seed=seed + 5))


def test_readme_shape_cfg1():
    # BASELINE config 1: bsz=1, seqlen=4, dim=kdim=4, fp32, seed 0
    x, f, q, k, fk, s, go, gs = make_config_inputs(1, 4, 4, 4, torch.float32, seed=0,
                                                    in_scale=1.0, gate_mean=0.0, state_std=1.0,
                                                    gstate_std=1.0)
    out, nxt = lfw_reference(x, f, q, k, fk, s)
    assert out.shape == (1, 4, 4) and nxt.shape == (1, 4, 4)
    bo, bn = lfw_bruteforce(x.double(), f.double(), q.double(), k.double(), fk.double(), s.double())
    assert torch.allclose(out.double(), bo, atol=1e-5)
    assert torch.allclose(nxt.double(), bn, atol=1e-5)


def test_bruteforce_unrolled_sum():
    ins = small_inputs(B=2, T=4, D=3, K=2)
    out, nxt = lfw_reference(*ins)
    bo, bn = lfw_bruteforce(*ins)
    assert torch.allclose(out, bo, atol=1e-12)
    assert torch.allclose(nxt, bn, atol=1e-12)


def test_gates_one_is_masked_cumulative_matmul():
    x, _, q, k, _, s = small_inputs(T=7)
    one_d, one_k = torch.ones_like(x), torch.ones_like(q)
    out, nxt = lfw_reference(x, one_d, q, k, one_k, s)
    # o_t = (S0 + sum_{s<=t} x_s k_s^T) q_t = S0 q_t + sum_s tril(q k^T)[t,s] x_s
    P = torch.tril(q @ k.transpose(1, 2))
    expect = torch.einsum("bdk,btk->btd", s, q) + P @ x
    assert torch.allclose(out, expect, atol=1e-12)
    assert torch.allclose(nxt, s + torch.einsum("btd,btk->bdk", x, k), atol=1e-12)


def test_gates_zero_is_single_step():
    x, _, q, k, _, s = small_inputs()
    z_d, z_k = torch.zeros_like(x), torch.zeros_like(q)
    out, nxt = lfw_reference(x, z_d, q, k, z_k, s)
    assert torch.allclose(out, x * (k * q).sum(-1, keepdim=True), atol=1e-12)
    assert torch.allclose(nxt, x[:, -1, :, None] * k[:, -1, None, :], atol=1e-12)


def test_constant_scalar_gates_geometric():
    x, _, q, k, _, s = small_inputs(T=6)
    a, b = 0.7, 0.9
    out, nxt = lfw_reference(x, torch.full_like(x, a), q, k, torch.full_like(q, b), s)
    T = x.shape[1]
    t = torch.arange(T, dtype=DT)
    W = torch.tril((a * b) ** (t[:, None] - t[None, :]).clamp_min(0))     # (ab)^(t-s)
    P = (q @ k.transpose(1, 2)) * W
    decay0 = (a * b) ** (t + 1)
    expect = torch.einsum("bdk,btk->btd", s, q) * decay0[None, :, None] + P @ x
    assert torch.allclose(out, expect, atol=1e-12)


def test_single_step_and_zero_query():
    x, f, q, k, fk, s = small_inputs(T=1)
    out, nxt = lfw_reference(x, f, q, k, fk, s)
    s1 = s * (f[:, 0, :, None] * fk[:, 0, None, :]) + x[:, 0, :, None] * k[:, 0, None, :]
    assert torch.allclose(nxt, s1, atol=1e-14)
    assert torch.allclose(out[:, 0], torch.einsum("bdk,bk->bd", s1, q[:, 0]), atol=1e-14)
    x, f, q, k, fk, s = small_inputs(T=5)
    out0, nxt0 = lfw_reference(x, f, torch.zeros_like(q), k, fk, s)
    _, nxt1 = lfw_reference(x, f, q, k, fk, s)
    assert out0.abs().max() == 0 and torch.equal(nxt0, nxt1)


@pytest.mark.parametrize("split", [1, 3, 6])
def test_segment_composition(split):
    ins = small_inputs(T=7)
    x, f, q, k, fk, s = ins
    out, nxt = lfw_reference(*ins)
    o1, mid = lfw_reference(x[:, :split], f[:, :split], q[:, :split], k[:, :split], fk[:, :split], s)
    o2, end = lfw_reference(x[:, split:], f[:, split:], q[:, split:], k[:, split:], fk[:, split:], mid)
    assert torch.allclose(torch.cat([o1, o2], 1), out, atol=1e-13)
    assert torch.allclose(end, nxt, atol=1e-13)


def test_linearity_in_x_and_state():
    x, f, q, k, fk, s = small_inputs(seed=3)
    x2, s2 = rnd(*x.shape, seed=50), rnd(*s.shape, seed=51)
    o1, n1 = lfw_reference(x, f, q, k, fk, s)
    o2, n2 = lfw_reference(x2, f, q, k, fk, s2)
    o3, n3 = lfw_reference(2 * x - 3 * x2, f, q, k, fk, 2 * s - 3 * s2)
    assert torch.allclose(o3, 2 * o1 - 3 * o2, atol=1e-12)
    assert torch.allclose(n3, 2 * n1 - 3 * n2, atol=1e-12)


def test_batch_rows_independent():
    ins = small_inputs(B=3)
    out, nxt = lfw_reference(*ins)
    perm = torch.tensor([2, 0, 1])
    o2, n2 = lfw_reference(*[t[perm] for t in ins])
    assert torch.equal(o2, out[perm]) and torch.equal(n2, nxt[perm])


def test_transpose_symmetry_of_state():
    # swapping the roles of (x,f) and (k,fkey) transposes the state
    x, f, q, k, fk, s = small_inputs(D=3, K=4)
    _, n1 = lfw_reference(x, f, q, k, fk, s)
    _, n2 = lfw_reference(k, fk, torch.zeros_like(x), x, f, s.transpose(1, 2).contiguous())
    assert torch.allclose(n1, n2.transpose(1, 2), atol=1e-14)


def test_script_variant_matches_loop():
    ins = small_inputs(B=3, T=9, D=5, K=2)
    o1, n1 = lfw_reference(*ins)
    o2, n2 = lfw_reference_script(*ins)
    assert torch.allclose(o1, o2, atol=1e-13) and torch.allclose(n1, n2, atol=1e-13)


def test_c_oracle_forward_matches_torch():
    ins = small_inputs(B=3, T=11, D=5, K=7, seed=9)
    o1, n1 = lfw_reference(*ins)
    o2, n2 = c_oracle.lfw_forward(*ins)
    assert np.allclose(o1.numpy(), o2, atol=1e-13) and np.allclose(n1.numpy(), n2, atol=1e-13)


@pytest.mark.parametrize("shape", [(2, 5, 3, 4), (1, 1, 1, 1), (3, 9, 4, 2), (2, 6, 1, 5)])
def test_closed_form_backward_matches_autograd(shape):
    B, T, D, K = shape
    ins = small_inputs(B, T, D, K, seed=11)
    go, gs = rnd(B, T, D, seed=70), rnd(B, D, K, seed=71)
    _, _, auto = lfw_reference_grads(*ins, go, gs)
    manual = lfw_backward_closed_form(go, gs, *ins)
    cgrads = c_oracle.lfw_backward(go, gs, *ins)
    for a, m, c in zip(auto, manual, cgrads):
        assert torch.allclose(a, m, atol=1e-12)
        assert np.allclose(a.numpy(), c, atol=1e-12)


def test_gradcheck_finite_differences():
    ins = [t.clone().requires_grad_(True) for t in small_inputs(B=1, T=3, D=2, K=3, seed=21)]
    assert torch.autograd.gradcheck(lfw_reference, ins, eps=1e-6, atol=1e-6)


def test_backward_state_gradient_only_path():
    # grad_output = 0: d_state = grad_state * prod_t F_t, d_q = 0
    ins = small_inputs(T=4)
    x, f, q, k, fk, s = ins
    gs = rnd(*s.shape, seed=5)
    d_x, d_f, d_q, d_k, d_fk, d_s = lfw_backward_closed_form(torch.zeros_like(x), gs, *ins)
    F = torch.ones_like(s)
    for t in range(4):
        F = F * (f[:, t, :, None] * fk[:, t, None, :])
    assert torch.allclose(d_s, gs * F, atol=1e-14) and d_q.abs().max() == 0


def test_reference_test_grid_inputs_are_well_formed():
    x, f, q, k, fk, s, go, gs = make_reference_test_inputs(5, 129, 33, 17, torch.float16, seed=1)
    assert x.shape == (5, 129, 33) and fk.shape == (5, 129, 17) and s.shape == (5, 33, 17)
    assert float(f.min()) > 0 and float(f.max()) < 1
    # gates are constant over batch and time, per channel (tests/test_lfw.py:10-16)
    assert torch.equal(f[0, 0], f[4, 128]) and torch.equal(fk[0, 0], fk[2, 77])
