"""The committed fixtures of tests/golden (made by tests/golden/make_vectors.py from the oracle; the reference holds
no vectors of its own): the Python oracle and the C oracle still reproduce them, a recurrence written out element by
element in numpy agrees with them, and on the GPU the exact float64 kernels do."""
import json
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with open(os.path.join(GOLDEN, name)) as fh:
        return {k: torch.tensor(v, dtype=torch.float64) for k, v in json.load(fh).items()}


LFW_IN = ["x", "f", "q", "k", "f_key", "s0"]
LFW_GRADS = ["d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state"]
DFW_IN = ["q", "k", "v", "s0"]
DFW_GRADS = ["d_q", "d_k", "d_v", "d_state"]


def close(a, b, tol=1e-12):
    a, b = torch.as_tensor(a, dtype=torch.float64), torch.as_tensor(b, dtype=torch.float64)
    assert a.shape == b.shape
    assert (a - b).abs().max().item() <= tol * max(1.0, b.abs().max().item())


def test_python_oracle_reproduces_the_fixtures():
    from oracle.dfw_ref import dfw_reference_grads
    from oracle.lfw_ref import lfw_reference_grads
    d = load("lfw_small.json")
    out, nxt, grads = lfw_reference_grads(*[d[n] for n in LFW_IN], d["g_out"], d["g_state"])
    close(out, d["outputs"]); close(nxt, d["next_state"])
    for n, g in zip(LFW_GRADS, grads):
        close(g, d[n])
    d = load("dfw_small.json")
    out, fin, grads = dfw_reference_grads(*[d[n] for n in DFW_IN], d["g_out"], d["g_state"])
    close(out, d["outputs"]); close(fin, d["final_state"])
    for n, g in zip(DFW_GRADS, grads):
        close(g, d[n])


def test_c_oracle_reproduces_the_decay_rule_fixture():
    from oracle import c_oracle
    d = load("lfw_small.json")
    ins = [d[n] for n in LFW_IN]
    out, nxt = c_oracle.lfw_forward(*ins)
    close(out, d["outputs"]); close(nxt, d["next_state"])
    grads = c_oracle.lfw_backward(d["g_out"], d["g_state"], *ins)
    for n, g in zip(LFW_GRADS, grads):
        close(g, d[n])


def test_fixtures_against_the_recurrences_written_out_per_element():
    """S[d][k] <- S[d][k] * f[d] * fk[k] + x[d] * k[k], o[d] = sum_k S[d][k] q[k]   (t2fw/torch.py:21-29)
    o[d] = sum_m S[d][m] q[m], delta[d] = v[d] - sum_m S[d][m] k[m], S[d][m] += delta[d] k[m]   (t2fw/torch.py:44-53)"""
    d = {k: v.numpy() for k, v in load("lfw_small.json").items()}
    B, T, D = d["x"].shape
    K = d["q"].shape[2]
    for b in range(B):
        S = d["s0"][b].copy()
        for t in range(T):
            for i in range(D):
                for j in range(K):
                    S[i][j] = S[i][j] * d["f"][b, t, i] * d["f_key"][b, t, j] + d["x"][b, t, i] * d["k"][b, t, j]
            for i in range(D):
                assert abs(sum(S[i][j] * d["q"][b, t, j] for j in range(K)) - d["outputs"][b, t, i]) < 1e-12
        assert np.abs(S - d["next_state"][b]).max() < 1e-12
    d = {k: v.numpy() for k, v in load("dfw_small.json").items()}
    B, T, D = d["v"].shape
    M = d["q"].shape[2]
    for b in range(B):
        S = d["s0"][b].copy()
        for t in range(T):
            for i in range(D):
                assert abs(sum(S[i][m] * d["q"][b, t, m] for m in range(M)) - d["outputs"][b, t, i]) < 1e-12
            delta = [d["v"][b, t, i] - sum(S[i][m] * d["k"][b, t, m] for m in range(M)) for i in range(D)]
            for i in range(D):
                for m in range(M):
                    S[i][m] += delta[i] * d["k"][b, t, m]
        assert np.abs(S - d["final_state"][b]).max() < 1e-12


def test_decay_rule_gradients_of_the_fixture_by_finite_differences():
    """central differences of L = <g_out, outputs> + <g_state, next_state> in float64 on a few coordinates of every input"""
    from oracle.lfw_ref import lfw_reference
    d = load("lfw_small.json")

    def loss(ins):
        o, n = lfw_reference(*ins)
        return (o * d["g_out"]).sum().item() + (n * d["g_state"]).sum().item()
    ins = [d[n].clone() for n in LFW_IN]
    h = 1e-6
    for which, gname in enumerate(LFW_GRADS):
        flat = ins[which].view(-1)
        for idx in (0, flat.numel() // 2, flat.numel() - 1):
            keep = flat[idx].item()
            flat[idx] = keep + h
            up = loss(ins)
            flat[idx] = keep - h
            down = loss(ins)
            flat[idx] = keep
            assert abs((up - down) / (2 * h) - d[gname].view(-1)[idx].item()) < 1e-7


@pytest.mark.gpu
def test_exact_float64_kernels_reproduce_the_fixtures():
    from t2fw.functional_dfw import DFWFunction
    from t2fw.functional_lfw import LFWFunction
    d = load("lfw_small.json")
    ins = [d[n].cuda().requires_grad_(True) for n in LFW_IN]
    out, nxt = LFWFunction.apply(*ins)
    torch.autograd.backward([out, nxt], [d["g_out"].cuda(), d["g_state"].cuda()])
    close(out.detach().cpu(), d["outputs"]); close(nxt.detach().cpu(), d["next_state"])
    for n, t in zip(LFW_GRADS, ins):
        close(t.grad.cpu(), d[n])
    d = load("dfw_small.json")
    ins = [d[n].cuda().requires_grad_(True) for n in DFW_IN]
    out, fin = DFWFunction.apply(*ins)
    torch.autograd.backward([out, fin], [d["g_out"].cuda(), d["g_state"].cuda()])
    close(out.detach().cpu(), d["outputs"], 1e-10); close(fin.detach().cpu(), d["final_state"], 1e-10)
    for n, t in zip(DFW_GRADS, ins):
        close(t.grad.cpu(), d[n], 1e-10)
