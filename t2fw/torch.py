"""Plain-PyTorch statements of the two fast-weight rules, on the reference's import path
(``from t2fw.torch import t2fw_torch, t2dfw_torch, t2dfw_torch_bw``, as the reference's tests
do: tests/test_lfw.py:7, tests/test_dfw.py:7, tests/benchmark.py:5).

Same names, positional arguments and return values as t2fw/torch.py:9-31 (decay rule),
:34-55 (delta rule), :59-145 and :148-242 (the delta rule's two hand-derived backward passes).
They run on any device and dtype torch supports and are differentiable by autograd; they are
what a user compares the kernels against, not a fallback of the kernels: nothing in the
kernel package imports this module, and this module imports nothing but torch.

Shapes: ``x, f, value: [B, T, D]``; ``query, key, f_key: [B, T, M]``; states ``[B, D, M]``.
"""
from typing import List, Tuple

import torch


@torch.jit.script
def t2fw_torch(x: torch.Tensor, f: torch.Tensor, query: torch.Tensor, key: torch.Tensor, f_key: torch.Tensor,
               state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Decay rule: ``S_t = S_{t-1} * (f_t (x) f_key_t) + x_t (x) key_t``, ``out_t = S_t query_t``
    (the output reads the state after the step's write).  Returns ``(outputs [B, T, D], S_{T-1})``."""
    rows = torch.jit.annotate(List[torch.Tensor], [])
    for t in range(x.size(1)):
        decay = torch.einsum("bd,bm->bdm", f[:, t], f_key[:, t])
        state = state * decay + torch.einsum("bd,bm->bdm", x[:, t], key[:, t])
        rows.append(torch.einsum("bdm,bm->bd", state, query[:, t]))
    return torch.stack(rows, dim=1), state


@torch.jit.script
def t2dfw_torch(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Delta rule: ``out_t = S_{t-1} query_t`` (the output reads the state before the step's write),
    ``S_t = S_{t-1} + (value_t - S_{t-1} key_t) (x) key_t``.  Returns ``(outputs [B, T, D], S_{T-1})``."""
    rows = torch.jit.annotate(List[torch.Tensor], [])
    for t in range(value.size(1)):
        k = key[:, t]
        rows.append(torch.einsum("bdm,bm->bd", state, query[:, t]))
        correction = value[:, t] - torch.einsum("bdm,bm->bd", state, k)
        state = state + torch.einsum("bd,bm->bdm", correction, k)
    return torch.stack(rows, dim=1), state


def _stack_reversed(rows: List[torch.Tensor], like: torch.Tensor) -> torch.Tensor:
    if not rows:
        return like.new_zeros(like.shape)
    return torch.stack(rows[::-1], dim=1)


def t2dfw_torch_bw(grad_output: torch.Tensor, grad_state: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                   value: torch.Tensor, state: torch.Tensor,
                   final_state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Backward of the delta rule as two reverse sweeps, the decomposition the kernels use
    (t2fw/torch.py:59-145): the corrections ``delta_t = value_t - S_{t-1} key_t`` are recomputed by a
    forward sweep; sweep one carries the state adjoint ``G`` and yields ``d_value_t = G_t key_t`` and
    ``d_state``; sweep two walks the state back from ``final_state`` (``S_{t-1} = S_t - delta_t (x)
    key_t``) next to the same adjoint and yields ``d_query_t = S_{t-1}^T g_t`` and
    ``d_key_t = G_t^T delta_t - S_{t-1}^T d_value_t``.  Returns ``(d_query, d_key, d_value, d_state)``."""
    T = value.size(1)
    deltas = []
    s = state
    for t in range(T):
        delta = value[:, t] - torch.einsum("bdm,bm->bd", s, key[:, t])
        s = s + torch.einsum("bd,bm->bdm", delta, key[:, t])
        deltas.append(delta)

    d_value_rev = []
    adj = grad_state.clone()
    for t in range(T - 1, -1, -1):
        dv = torch.einsum("bdm,bm->bd", adj, key[:, t])
        d_value_rev.append(dv)
        adj = adj - torch.einsum("bd,bm->bdm", dv, key[:, t]) + torch.einsum("bd,bm->bdm", grad_output[:, t], query[:, t])
    d_state = adj
    d_value = _stack_reversed(d_value_rev, value)

    d_query_rev, d_key_rev = [], []
    adj = grad_state.clone()
    s = final_state.clone()
    for t in range(T - 1, -1, -1):
        k, g, dv = key[:, t], grad_output[:, t], d_value[:, t]
        s = s - torch.einsum("bd,bm->bdm", deltas[t], k)
        d_key_rev.append(torch.einsum("bd,bdm->bm", deltas[t], adj) - torch.einsum("bd,bdm->bm", dv, s))
        d_query_rev.append(torch.einsum("bd,bdm->bm", g, s))
        adj = adj - torch.einsum("bd,bm->bdm", dv, k) + torch.einsum("bd,bm->bdm", g, query[:, t])
    return _stack_reversed(d_query_rev, query), _stack_reversed(d_key_rev, key), d_value, d_state


def t2dfw_torch_bw_simple(grad_output: torch.Tensor, grad_state: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                          value: torch.Tensor, state: torch.Tensor,
                          final_state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """The same backward as one reverse sweep (t2fw/torch.py:148-242): a forward sweep keeps what each
    step overwrote, ``old_t = S_{t-1} key_t``; the reverse sweep then has ``d_key_t = G_t^T value_t -
    (S_{t-1}^T (G_t key_t) + G_t^T old_t)``.  Returns ``(d_query, d_key, d_value, d_state)``."""
    T = value.size(1)
    olds = []
    s = state
    for t in range(T):
        old = torch.einsum("bdm,bm->bd", s, key[:, t])
        s = s + torch.einsum("bd,bm->bdm", value[:, t] - old, key[:, t])
        olds.append(old)

    d_query_rev, d_key_rev, d_value_rev = [], [], []
    adj = grad_state.clone()
    s = final_state.clone()
    for t in range(T - 1, -1, -1):
        k, v, g = key[:, t], value[:, t], grad_output[:, t]
        adj_k = torch.einsum("bdm,bm->bd", adj, k)
        d_value_rev.append(adj_k)
        s = s - torch.einsum("bd,bm->bdm", v - olds[t], k)
        d_key_rev.append(torch.einsum("bd,bdm->bm", v - olds[t], adj) - torch.einsum("bd,bdm->bm", adj_k, s))
        d_query_rev.append(torch.einsum("bd,bdm->bm", g, s))
        adj = adj - torch.einsum("bd,bm->bdm", adj_k, k) + torch.einsum("bd,bm->bdm", g, query[:, t])
    return (_stack_reversed(d_query_rev, query), _stack_reversed(d_key_rev, key), _stack_reversed(d_value_rev, value),
            adj)
