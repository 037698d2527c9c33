"""Synthetic inputs of the benchmark configurations and of the reference's test procedure
(CPU tensors; callers move them), shared by bench.py, the benchmark harness and the tests."""
import math

import torch


def uniform_gate_logits(shape, gen, dtype=torch.float32):
    """Per-channel gate bias logit(u), u ~ U(1/n, 1-1/n), constant over batch and time:
    the gate construction of the reference's tests (tests/test_lfw.py:10-16)."""
    n = shape[-1]
    u = torch.rand(n, generator=gen, dtype=dtype) * (1 - 2.0 / n) + 1.0 / n
    return (-torch.log(1 / u - 1)).expand(shape).contiguous()


def reference_shape_grid():
    """(bsz, seqlen, dim) grid of tests/test_lfw.py:19-24; kdim = ceil(dim/2) (:34)."""
    for bsz in range(1, 16, 4):
        for dim in range(1, 64, 32):
            for seqlen in range(1, 512, 128):
                yield bsz, seqlen, dim
    yield 2, 1024, 32


def make_reference_test_inputs(bsz, seqlen, dim, kdim, dtype, seed):
    """Inputs as tests/test_lfw.py:37-42 builds them: x,q,k,s ~ N(0,1); gates =
    sigmoid(per-channel uniform-gate bias).  Generated in fp32 on CPU, then quantised
    to ``dtype`` so the oracle and the kernel see bit-identical values."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(bsz, seqlen, dim, generator=g)
    f = torch.sigmoid(uniform_gate_logits((bsz, seqlen, dim), g))
    q = torch.randn(bsz, seqlen, kdim, generator=g)
    k = torch.randn(bsz, seqlen, kdim, generator=g)
    fk = torch.sigmoid(uniform_gate_logits((bsz, seqlen, kdim), g))
    s = torch.randn(bsz, dim, kdim, generator=g)
    go = torch.randn(bsz, seqlen, dim, generator=g)
    gs = torch.randn(bsz, dim, kdim, generator=g)
    return tuple(t.to(dtype) for t in (x, f, q, k, fk, s, go, gs))


def make_config_inputs(B, T, D, K, dtype, seed=0, in_scale=0.125, gate_mean=2.0,
                       state_std=0.0, gout_std=1.0, gstate_std=0.1):
    """Benchmark-config inputs: x,q,k ~ N(0,1)*in_scale, gates = sigmoid(N(gate_mean,1)),
    s ~ N(0,state_std), grad_output ~ N(0,gout_std), grad_state ~ N(0,gstate_std)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, D, generator=g) * in_scale
    f = torch.sigmoid(torch.randn(B, T, D, generator=g) + gate_mean)
    q = torch.randn(B, T, K, generator=g) * in_scale
    k = torch.randn(B, T, K, generator=g) * in_scale
    fk = torch.sigmoid(torch.randn(B, T, K, generator=g) + gate_mean)
    s = torch.randn(B, D, K, generator=g) * state_std
    go = torch.randn(B, T, D, generator=g) * gout_std
    gs = torch.randn(B, D, K, generator=g) * gstate_std
    return tuple(t.to(dtype) for t in (x, f, q, k, fk, s, go, gs))


def err_stats(got, ref):
    """(max-abs error, max-abs / max|ref|, mean relative error) in float64."""
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    diff = (got - ref).abs()
    denom = ref.abs().max().clamp_min(1e-30)
    mean_rel = (diff / ref.abs().clamp_min(1e-6 * float(denom))).mean()
    return float(diff.max()) if diff.numel() else 0.0, \
        float(diff.max() / denom) if diff.numel() else 0.0, \
        float(mean_rel) if diff.numel() else 0.0
