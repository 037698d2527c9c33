"""The reference's three import paths resolve here (tests/test_lfw.py:4-7, tests/test_dfw.py:4-7,
tests/benchmark.py:5 of the reference), and ``t2fw.torch`` states the same recurrences as the
oracle.  CPU only.  ``t2fw.torch`` is independent of the oracle (it imports nothing but torch, and
nothing in the kernel package imports it), so agreement between the two is a check of both."""
import ast
import os

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_reference_tests_import_lines_resolve():
    from t2fw.functional_lfw import LFWFunction                    # tests/test_lfw.py:6
    from t2fw.functional_dfw import DFWFunction                    # tests/test_dfw.py:6
    from t2fw.torch import t2fw_torch                              # tests/test_lfw.py:7
    from t2fw.torch import t2dfw_torch, t2dfw_torch_bw             # tests/test_dfw.py:7
    from t2fw.torch import t2dfw_torch_bw_simple                   # t2fw/torch.py:148
    assert issubclass(LFWFunction, torch.autograd.Function)
    assert issubclass(DFWFunction, torch.autograd.Function)
    for fn in (t2fw_torch, t2dfw_torch, t2dfw_torch_bw, t2dfw_torch_bw_simple):
        assert callable(fn)


def _imports_of(path):
    tree = ast.parse(open(path).read())
    names = set()
    for node in ast.walk(tree):
        if isinstance(node, ast.Import):
            names.update(a.name.split(".")[0] for a in node.names)
        elif isinstance(node, ast.ImportFrom):
            names.add((node.module or "").split(".")[0] if node.level == 0 else ".")
    return names


def test_torch_module_is_independent_of_oracle_and_kernels():
    assert _imports_of(os.path.join(ROOT, "t2fw", "torch.py")) <= {"torch", "typing"}
    # ... and the kernel package never reaches for it or for the oracle
    pkg = os.path.join(ROOT, "t2fw_amd")
    for name in os.listdir(pkg):
        if name.endswith(".py"):
            text = open(os.path.join(pkg, name)).read()
            assert "oracle" not in _imports_of(os.path.join(pkg, name)), name
            assert "t2fw.torch" not in text, name


def _lfw_inputs(B, T, D, K, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    return (r(B, T, D), torch.sigmoid(r(B, T, D)), r(B, T, K), r(B, T, K), torch.sigmoid(r(B, T, K)), r(B, D, K))


@pytest.mark.parametrize("shape", [(1, 4, 4, 4), (3, 17, 5, 2), (2, 1, 1, 1), (2, 40, 33, 17)])
def test_decay_rule_matches_the_oracle(shape):
    from oracle import lfw_ref
    from t2fw.torch import t2fw_torch
    ins = _lfw_inputs(*shape, seed=3)
    out, nxt = t2fw_torch(*ins)
    r_out, r_nxt = lfw_ref.lfw_reference(*ins)
    assert torch.allclose(out, r_out, rtol=1e-12, atol=1e-12)
    assert torch.allclose(nxt, r_nxt, rtol=1e-12, atol=1e-12)
    # gradients by autograd through it = the oracle's closed-form backward
    leaves = [t.clone().requires_grad_(True) for t in ins]
    out, nxt = t2fw_torch(*leaves)
    g = torch.Generator().manual_seed(5)
    go = torch.randn(out.shape, generator=g, dtype=torch.float64)
    gs = torch.randn(nxt.shape, generator=g, dtype=torch.float64)
    out.backward(go, retain_graph=True)        # the two-call protocol of tests/test_lfw.py:49-53
    nxt.backward(gs)
    ref = lfw_ref.lfw_backward_closed_form(go, gs, *ins)
    for got, want in zip(leaves, ref):
        assert torch.allclose(got.grad, want, rtol=1e-10, atol=1e-10)


def _dfw_inputs(B, T, D, M, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    k = r(B, T, M)
    k = torch.softmax(k, dim=-1) * torch.sigmoid(k.mean(dim=-1, keepdim=True))      # tests/test_dfw.py:45-46
    return r(B, T, M), k, r(B, T, D), r(B, D, M)


@pytest.mark.parametrize("shape", [(1, 4, 4, 4), (3, 19, 6, 3), (2, 1, 1, 1), (2, 33, 9, 17)])
def test_delta_rule_and_both_backward_forms_match_the_oracle(shape):
    from oracle import dfw_ref
    from t2fw.torch import t2dfw_torch, t2dfw_torch_bw, t2dfw_torch_bw_simple
    q, k, v, s = _dfw_inputs(*shape, seed=7)
    out, fin = t2dfw_torch(q, k, v, s)
    r_out, r_fin = dfw_ref.dfw_reference(q, k, v, s)
    assert torch.allclose(out, r_out, rtol=1e-12, atol=1e-12)
    assert torch.allclose(fin, r_fin, rtol=1e-12, atol=1e-12)
    g = torch.Generator().manual_seed(9)
    go = torch.randn(out.shape, generator=g, dtype=torch.float64)
    gs = torch.randn(fin.shape, generator=g, dtype=torch.float64)
    _, _, want = dfw_ref.dfw_reference_grads(q, k, v, s, go, gs)
    for fn in (t2dfw_torch_bw, t2dfw_torch_bw_simple):
        got = fn(go, gs, q, k, v, s, fin)                    # (d_query, d_key, d_value, d_state)
        for a, b in zip(got, want):
            assert torch.allclose(a, b, rtol=1e-10, atol=1e-10), fn.__name__


def test_output_reads_the_state_after_the_write_for_decay_and_before_it_for_delta():
    """The one-step closed forms that tell the two rules apart (t2fw/torch.py:27 against :47)."""
    from t2fw.torch import t2fw_torch, t2dfw_torch
    x, f, q, k, fk, s = _lfw_inputs(2, 1, 3, 4, seed=11)
    out, nxt = t2fw_torch(x, f, q, k, fk, s)
    want_state = s * (f[:, 0, :, None] * fk[:, 0, None, :]) + x[:, 0, :, None] * k[:, 0, None, :]
    assert torch.allclose(nxt, want_state, rtol=1e-13, atol=1e-13)
    assert torch.allclose(out[:, 0], (want_state * q[:, 0, None, :]).sum(-1), rtol=1e-13, atol=1e-13)
    out, fin = t2dfw_torch(q, k, x, s)
    assert torch.allclose(out[:, 0], (s * q[:, 0, None, :]).sum(-1), rtol=1e-13, atol=1e-13)
    delta = x[:, 0] - (s * k[:, 0, None, :]).sum(-1)
    assert torch.allclose(fin, s + delta[:, :, None] * k[:, 0, None, :], rtol=1e-13, atol=1e-13)
