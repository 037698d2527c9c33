"""CPU restatement of the reference's decay-rule ("LFW") recurrence.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

What it follows in the reference (paths relative to the reference tree):

* ``lfw_reference``      -> t2fw/torch.py:9-31   (``t2fw_torch``: the recurrence, the
                            output taken from the state AFTER the update, the final
                            state returned as second value)
* ``lfw_reference_script`` -> the same loop under ``torch.jit.script`` (the reference
                            decorates its function with it, t2fw/torch.py:8); this is
                            the "TorchScript CPU path" timed as the CPU baseline
* ``lfw_backward_closed_form`` -> t2fw/csrc/lfw_kernel.cu:85-100 (reverse scan of the
                            state gradient) + t2fw/csrc/lfw.cpp:84-93 (the six
                            contractions that turn it into input gradients)
* ``lfw_bruteforce``     -> no counterpart; the O(T^2) unrolled sum the recurrence
                            solves to, used to pin ``lfw_reference`` on tiny inputs

Pinning status (tests/test_oracle_lfw.py): every function here is checked against
closed forms (gates == 1 -> masked cumulative matmul, gates == 0 -> single-step
outer product, constant scalar gates -> geometric weights), the brute-force
unrolled sum, segment composition, linearity, the D<->K transpose symmetry,
``torch.autograd`` through the restated forward and ``torch.autograd.gradcheck``.
The reference holds no stored golden vectors for this path
(tests/test_lfw.py:29-42 draws random tensors at run time).
"""
from typing import List, Tuple

import torch


def lfw_reference(x: torch.Tensor, f: torch.Tensor, query: torch.Tensor,
                  key: torch.Tensor, f_key: torch.Tensor,
                  state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """S_t = S_{t-1} * (f_t (x) fkey_t) + x_t (x) k_t ;  o_t = S_t q_t.

    x, f: [B,T,D]; query, key, f_key: [B,T,K]; state: [B,D,K].
    Returns (outputs [B,T,D], final state [B,D,K]).  t2fw/torch.py:21-31.
    """
    B, T, D = x.shape
    outs = []
    s = state
    for t in range(T):
        gate = f[:, t, :, None] * f_key[:, t, None, :]          # torch.py:22
        write = x[:, t, :, None] * key[:, t, None, :]           # torch.py:23
        s = s * gate + write                                    # torch.py:25
        outs.append((s * query[:, t, None, :]).sum(dim=-1))      # torch.py:27
    if T == 0:
        return x.new_zeros((B, 0, D)), s
    return torch.stack(outs, dim=1), s                          # torch.py:29-31


@torch.jit.script
def lfw_reference_script(x: torch.Tensor, f: torch.Tensor, query: torch.Tensor,
                         key: torch.Tensor, f_key: torch.Tensor,
                         state: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """The same loop compiled by TorchScript with batched mat-vec products, the op
    mix t2fw/torch.py:21-29 executes (two outer products, one multiply-add, one
    mat-vec per step).  Used as the timed CPU baseline."""
    outs = torch.jit.annotate(List[torch.Tensor], [])
    for t in range(x.size(1)):
        gate = torch.bmm(f[:, t].unsqueeze(2), f_key[:, t].unsqueeze(1))
        write = torch.bmm(x[:, t].unsqueeze(2), key[:, t].unsqueeze(1))
        state = torch.addcmul(write, state, gate)
        outs.append(torch.bmm(state, query[:, t].unsqueeze(2)).squeeze(2))
    return torch.stack(outs, dim=1), state


def lfw_reference_grads(x, f, query, key, f_key, state, grad_output, grad_state,
                        dtype=torch.float64):
    """Forward + autograd backward of ``lfw_reference`` in ``dtype`` on CPU, using the
    two-call backward protocol of tests/test_lfw.py:49-53 (outputs first with
    retain_graph, then the state).  Returns (outputs, next_state, 6-tuple of grads in
    forward-argument order)."""
    ins = [t.detach().to("cpu", dtype).clone().requires_grad_(True)
           for t in (x, f, query, key, f_key, state)]
    out, nxt = lfw_reference(*ins)
    out.backward(grad_output.detach().to("cpu", dtype), retain_graph=True)
    nxt.backward(grad_state.detach().to("cpu", dtype))
    return out.detach(), nxt.detach(), tuple(t.grad for t in ins)


def lfw_backward_closed_form(grad_output, grad_state, x, f, query, key, f_key, state):
    """Manual backward in the reference's own formulation.

    Reverse scan (t2fw/csrc/lfw_kernel.cu:85-100):
        G <- g_t (x) q_t + G ; s_grad[t] = G ; G <- G * (f_t (x) fkey_t)
    then the contractions of t2fw/csrc/lfw.cpp:84-93.
    Returns (d_x, d_f, d_q, d_k, d_f_key, d_state) (lfw.cpp:95).
    """
    B, T, D = x.shape
    K = key.shape[-1]
    states = []
    s = state
    for t in range(T):
        s = s * (f[:, t, :, None] * f_key[:, t, None, :]) + x[:, t, :, None] * key[:, t, None, :]
        states.append(s)
    d_x = torch.zeros_like(x)
    d_f = torch.zeros_like(f)
    d_q = torch.zeros_like(query)
    d_k = torch.zeros_like(key)
    d_fk = torch.zeros_like(f_key)
    G = grad_state.clone()
    for t in range(T - 1, -1, -1):
        G = grad_output[:, t, :, None] * query[:, t, None, :] + G      # lfw_kernel.cu:89
        d_q[:, t] = (grad_output[:, t, :, None] * states[t]).sum(1)     # lfw.cpp:84
        d_x[:, t] = (G * key[:, t, None, :]).sum(2)                     # lfw.cpp:85
        d_k[:, t] = (G * x[:, t, :, None]).sum(1)                       # lfw.cpp:86
        prev = states[t - 1] if t > 0 else state                       # lfw.cpp:89-90
        H = G * prev
        d_f[:, t] = (H * f_key[:, t, None, :]).sum(2)                   # lfw.cpp:92
        d_fk[:, t] = (H * f[:, t, :, None]).sum(1)                      # lfw.cpp:93
        G = G * (f[:, t, :, None] * f_key[:, t, None, :])               # lfw_kernel.cu:93
    return d_x, d_f, d_q, d_k, d_fk, G                                  # lfw_kernel.cu:100


def lfw_bruteforce(x, f, query, key, f_key, state):
    """O(T^2) unrolled solution of the recurrence, python loops, tiny inputs only:
    S_t[d,k] = S_0[d,k] prod_{r<=t} f_r[d] fk_r[k]
             + sum_{s<=t} x_s[d] k_s[k] prod_{s<r<=t} f_r[d] fk_r[k]."""
    B, T, D = x.shape
    K = key.shape[-1]
    out = torch.zeros(B, T, D, dtype=x.dtype)
    last = state.clone()
    for b in range(B):
        for t in range(T):
            for d in range(D):
                acc_o = 0.0
                for k in range(K):
                    w = 1.0
                    for r in range(t + 1):
                        w = w * float(f[b, r, d]) * float(f_key[b, r, k])
                    sdk = float(state[b, d, k]) * w
                    for s in range(t + 1):
                        w = 1.0
                        for r in range(s + 1, t + 1):
                            w = w * float(f[b, r, d]) * float(f_key[b, r, k])
                        sdk += float(x[b, s, d]) * float(key[b, s, k]) * w
                    acc_o += sdk * float(query[b, t, k])
                    if t == T - 1:
                        last[b, d, k] = sdk
                out[b, t, d] = acc_o
    return out, last
