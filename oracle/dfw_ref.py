"""CPU restatement of the reference's delta-rule ("DFW") recurrence.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

What it follows in the reference (paths relative to the reference tree):

* ``dfw_reference``          -> t2fw/torch.py:34-55 (``t2dfw_torch``: out_t from the state
                                BEFORE the update, delta write, final state returned)
* ``dfw_backward_two_pass``  -> t2fw/torch.py:59-145 (``t2dfw_torch_bw``) = the two reverse
                                passes of t2fw/csrc/dfw_kernel.cu:250-276 (d_value, d_state)
                                and :345-383 (d_query, d_key with the state walked backwards)
* ``dfw_backward_one_pass``  -> t2fw/torch.py:148-242 (``t2dfw_torch_bw_simple``): the overwritten values
                                S_{t-1} k_t recomputed by a forward sweep, then all four gradients
                                in one reverse sweep from the final state
* ``dfw_deltas``             -> the ``delta_value`` tensor the forward kernel emits
                                (t2fw/csrc/dfw_kernel.cu:176-183), which the backward consumes

Pinning (tests/test_oracle_dfw.py): closed forms (zero keys, single step, unit-norm key
retrieval S_t k_t = v_t, orthonormal keys), ``torch.autograd`` through the restated forward
vs the two-pass and the one-pass backward, ``gradcheck``, segment composition, linearity in (v, S_0).
The reference holds no stored vectors for this path (tests/test_dfw.py:30-60 draws random
tensors at run time).
"""
from typing import Tuple

import torch


def dfw_reference(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                  state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """query,key [B,T,M]; value [B,T,D]; state [B,D,M] -> (outputs [B,T,D], final state)."""
    B, T, D = value.shape
    outs = []
    s = state
    for t in range(T):
        old = (s * key[:, t, None, :]).sum(-1)                   # torch.py:45
        outs.append((s * query[:, t, None, :]).sum(-1))           # torch.py:47 (before update)
        s = s + (value[:, t] - old)[:, :, None] * key[:, t, None, :]   # torch.py:50
    if T == 0:
        return value.new_zeros((B, 0, D)), s
    return torch.stack(outs, dim=1), s


def dfw_deltas(query, key, value, state):
    """delta_t = v_t - S_{t-1} k_t for every step, [B,T,D]."""
    T = value.shape[1]
    ds = []
    s = state
    for t in range(T):
        d = value[:, t] - (s * key[:, t, None, :]).sum(-1)
        s = s + d[:, :, None] * key[:, t, None, :]
        ds.append(d)
    return torch.stack(ds, dim=1) if T else value.new_zeros(value.shape)


def dfw_reference_grads(query, key, value, state, grad_output, grad_state, dtype=torch.float64):
    """Forward + autograd backward with the two-call protocol of tests/test_dfw.py:55-60."""
    ins = [t.detach().to("cpu", dtype).clone().requires_grad_(True) for t in (query, key, value, state)]
    out, fin = dfw_reference(*ins)
    out.backward(grad_output.detach().to("cpu", dtype), retain_graph=True)
    fin.backward(grad_state.detach().to("cpu", dtype))
    return out.detach(), fin.detach(), tuple(t.grad for t in ins)


def dfw_backward_two_pass(grad_output, grad_state, query, key, delta, final_state):
    """The kernels' formulation: consumes delta and the FINAL state (as saved by the reference's
    autograd function, t2fw/functional_dfw.py:46-51).  Returns (d_q, d_k, d_v, d_state)."""
    B, T, D = delta.shape
    d_v = torch.zeros_like(delta)
    G = grad_state.clone()
    for t in range(T - 1, -1, -1):                                   # dfw_kernel.cu:250-276
        dv = (G * key[:, t, None, :]).sum(-1)
        d_v[:, t] = dv
        G = G - dv[:, :, None] * key[:, t, None, :] + grad_output[:, t, :, None] * query[:, t, None, :]
    d_state = G
    d_q = torch.zeros_like(query)
    d_k = torch.zeros_like(key)
    G = grad_state.clone()
    S = final_state.clone()
    for t in range(T - 1, -1, -1):                                   # dfw_kernel.cu:345-383
        S = S - delta[:, t, :, None] * key[:, t, None, :]            # S_{t-1}
        d_q[:, t] = (S * grad_output[:, t, :, None]).sum(1)
        d_k[:, t] = (G * delta[:, t, :, None]).sum(1) - (S * d_v[:, t, :, None]).sum(1)
        G = G - d_v[:, t, :, None] * key[:, t, None, :] + grad_output[:, t, :, None] * query[:, t, None, :]
    return d_q, d_k, d_v, d_state


def dfw_backward_one_pass(grad_output, grad_state, query, key, value, state, final_state):
    """The reference's second derivation (t2fw/torch.py:148-242): a forward sweep recomputes the
    value each step overwrote, old_t = S_{t-1} k_t (torch.py:159-168); one reverse sweep then walks
    the state back from ``final_state`` and carries the adjoint G.  Returns (d_q, d_k, d_v, d_state)."""
    B, T, D = value.shape
    olds = []
    s = state
    for t in range(T):                                               # torch.py:159-168
        old = (s * key[:, t, None, :]).sum(-1)
        s = s + (value[:, t] - old)[:, :, None] * key[:, t, None, :]
        olds.append(old)
    d_q, d_k, d_v = torch.zeros_like(query), torch.zeros_like(key), torch.zeros_like(value)
    G = grad_state.clone()
    S = final_state.clone()
    for t in range(T - 1, -1, -1):                                   # torch.py:178-233
        k, v, g = key[:, t], value[:, t], grad_output[:, t]
        Gk = (G * k[:, None, :]).sum(-1)                             # [B, D]
        d_v[:, t] = Gk                                               # torch.py:186
        S = S - (v - olds[t])[:, :, None] * k[:, None, :]            # S_{t-1}, torch.py:190
        a = (G * v[:, :, None]).sum(1)                               # G^T v       torch.py:217
        c = (G * olds[t][:, :, None]).sum(1)                         # G^T old     torch.py:219
        b = (S * Gk[:, :, None]).sum(1)                              # S_{t-1}^T G k   torch.py:221
        d_k[:, t] = a - (b + c)
        G = G - Gk[:, :, None] * k[:, None, :] + g[:, :, None] * query[:, t, None, :]   # torch.py:227-230
        d_q[:, t] = (S * g[:, :, None]).sum(1)                       # torch.py:234
    return d_q, d_k, d_v, G
