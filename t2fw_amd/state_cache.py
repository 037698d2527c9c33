"""Per-layer fast-weight state for generation: an ``nn.Module`` around the decay rule that owns
the ``[B, D, K]`` state between calls.

The reference stops at the autograd function (README.md:32); its benchmark drives generation
by calling the T = 1 forward per token and rebinding ``state`` (tests/benchmark.py:104-105),
which allocates a fresh ``[B, T, D, K]`` checkpoint tensor and a new state every step.  Here

  * a sequence (training, or the prompt at inference) goes through ``LFWFunction`` and the
    returned final state is kept;
  * single tokens under ``torch.no_grad()`` go through the T = 1 kernel, which streams the
    state through HBM once and updates it in place (no allocation per step).

Inputs are already gated, as for ``LFWFunction`` (t2fw/functional_lfw.py:25-30).
"""
import torch

from .functional_lfw import LFWFunction, lfw_step


class FastWeightState(torch.nn.Module):
    """Holds the fast-weight memory of one layer for a folded batch of ``B = batch * heads`` rows.

    ``forward(x, f, q, k, f_key)`` takes ``x, f: [B, T, D]`` and ``q, k, f_key: [B, T, K]`` (or the
    same without the T axis for one token) and returns the outputs ``[B, T, D]`` (``[B, D]``).
    The state starts at zero on first use, or at what ``reset(state)`` was given.
    """

    def __init__(self, value_dim, key_dim):
        super().__init__()
        self.value_dim = int(value_dim)
        self.key_dim = int(key_dim)
        self.state = None              # [B, D, K]; not a parameter and not a buffer: it is per-sequence data

    def reset(self, state=None):
        """Forget the memory (``None``) or install a given ``[B, D, K]`` state (copied)."""
        self.state = None if state is None else state.detach().clone().contiguous()
        return self

    def _state_for(self, x, rows):
        st = self.state
        if st is None:
            st = torch.zeros(rows, self.value_dim, self.key_dim, dtype=x.dtype, device=x.device)
        if st.shape[0] != rows or st.dtype != x.dtype or st.device != x.device:
            raise RuntimeError("FastWeightState: state %s %s on %s does not match inputs (%d rows, %s on %s); "
                               "call reset() between sequences" % (tuple(st.shape), st.dtype, st.device, rows,
                                                                   x.dtype, x.device))
        return st

    def forward(self, x, f, q, k, f_key):
        single = x.dim() == 2
        if x.shape[-1] != self.value_dim or q.shape[-1] != self.key_dim:
            raise RuntimeError("FastWeightState: expected value dim %d and key dim %d, got %d and %d"
                               % (self.value_dim, self.key_dim, x.shape[-1], q.shape[-1]))
        state = self._state_for(x, x.shape[0])
        needs_grad = torch.is_grad_enabled() and any(t.requires_grad for t in (x, f, q, k, f_key, state))
        if single and not needs_grad:
            # generation step: the state is read and written once, in place
            if self.state is None:
                self.state = state
            elif self.state.grad_fn is not None or self.state.requires_grad:
                # the state is still part of a recorded graph (a training call came before): step on a
                # private copy, so that nothing the graph may read is overwritten behind autograd's back
                self.state = self.state.detach().clone()
            out, _ = lfw_step(x, f, q, k, f_key, self.state, inplace=True)
            # the kernel wrote through a raw pointer: tell autograd's version counter
            torch.autograd.graph.increment_version(self.state)
            return out
        if single:
            x, f, q, k, f_key = (t.unsqueeze(1) for t in (x, f, q, k, f_key))
        out, new_state = LFWFunction.apply(x, f, q, k, f_key, state)
        # keep the graph only while gradients are being recorded (truncated BPTT is the caller's
        # choice: detach_state() cuts it)
        self.state = new_state if needs_grad else new_state.detach()
        return out.squeeze(1) if single else out

    def _apply(self, fn, *args, **kwargs):
        """``.to()``, ``.half()``, ``.cuda()`` move the carried state with the module (it is neither a
        parameter nor a buffer, so that it never lands in a state_dict)."""
        super()._apply(fn, *args, **kwargs)
        if self.state is not None:
            self.state = fn(self.state.detach())
        return self

    def detach_state(self):
        if self.state is not None:
            self.state = self.state.detach()
        return self
