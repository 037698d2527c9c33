"""Autograd boundary of the delta rule: same call as the reference's
``DFWFunction.apply(query, key, value, state)`` (t2fw/functional_dfw.py:29-65), backed by the
HIP kernels in libt2fw_hip.so.  As in the reference, backward consumes the per-step deltas
and the final state saved by forward (t2fw/functional_dfw.py:46-51)."""
import os

import torch

from . import _lib
from .functional_lfw import _check_input, _dtype_code, _flags, _on_device


def _dfw_flags(dtype):
    """Kernel-path flags of a call.  bfloat16 tensors take the matrix-core kernels' single-bf16-operand mode
    (include/t2fw_hip.h, T2FW_FLAG_BF16_OPERANDS): their inputs are bf16 numbers already, and rounding the
    intermediates to bf16 as well leaves the results at the accuracy that storing them in bf16 has anyway
    (measured against the fp64 oracle: 4e-3 .. 6e-3 of max|ref| per tensor, against 2e-3 .. 3.5e-3 for the exact
    per-step kernels), at 1.7 times the speed.  float32 and float16 tensors keep the split operands (results at
    the accuracy of the exact kernels for the type).  T2FW_FLAGS overrides this as everywhere."""
    if os.environ.get("T2FW_FLAGS"):
        return _flags()
    return _lib.FLAG_BF16_OPERANDS if dtype == torch.bfloat16 else _lib.FLAG_AUTO


class DFWFunction(torch.autograd.Function):
    """Delta rule: out_t = S_{t-1} q_t, S_t = S_{t-1} + (v_t - S_{t-1} k_t) (x) k_t.
    Any scalar write strength is assumed to be absorbed into the key."""

    @staticmethod
    def forward(ctx, query, key, value, state):
        """Return: (outputs [B,T,D], final state [B,D,M])"""
        # same asserts as t2fw/functional_dfw.py:38-40
        assert query.shape == key.shape
        assert query.dtype == value.dtype
        assert state.dtype == value.dtype
        assert key.dtype == value.dtype
        for t, n in ((query, "query"), (key, "key"), (value, "value"), (state, "state")):
            _check_input(t, n)
        if value.dim() != 3 or query.dim() != 3 or state.dim() != 3:
            raise RuntimeError("t2fw: expected query,key [B,T,M]; value [B,T,D]; state [B,D,M]")
        B, T, D = value.shape
        M = query.shape[2]
        if query.shape[0] != B or query.shape[1] != T or tuple(state.shape) != (B, D, M):
            raise RuntimeError("t2fw: inconsistent shapes query %s, value %s, state %s"
                               % (tuple(query.shape), tuple(value.shape), tuple(state.shape)))
        code = _dtype_code(value.dtype)
        lib = _lib.load()
        dev = value.device
        with _on_device(dev):
            outputs = torch.empty_like(value)
            final_state = torch.empty_like(state)
            delta = torch.empty_like(value)
            _lib.check(lib.t2fw_dfw_forward(
                _lib.ptr(query), _lib.ptr(key), _lib.ptr(value), _lib.ptr(state), _lib.ptr(outputs),
                _lib.ptr(final_state), _lib.ptr(delta), B, T, D, M, code, _dfw_flags(value.dtype), _lib.current_stream_handle(dev)))
        ctx.save_for_backward(query, key, delta, final_state)
        return outputs, final_state

    @staticmethod
    def backward(ctx, grad_output, grad_state):
        query, key, delta, final_state = ctx.saved_tensors
        # t2fw/functional_dfw.py:58-59
        assert grad_state.dtype == delta.dtype
        assert grad_output.dtype == delta.dtype
        grad_output = grad_output.contiguous()
        grad_state = grad_state.contiguous()
        B, T, D = delta.shape
        M = query.shape[2]
        lib = _lib.load()
        dev = delta.device
        with _on_device(dev):
            d_q, d_k = torch.empty_like(query), torch.empty_like(key)
            d_v, d_s = torch.empty_like(delta), torch.empty_like(final_state)
            _lib.check(lib.t2fw_dfw_backward(
                _lib.ptr(grad_output), _lib.ptr(grad_state), _lib.ptr(query), _lib.ptr(key), _lib.ptr(delta),
                _lib.ptr(final_state), _lib.ptr(d_q), _lib.ptr(d_k), _lib.ptr(d_v), _lib.ptr(d_s),
                B, T, D, M, _dtype_code(delta.dtype), _dfw_flags(delta.dtype), _lib.current_stream_handle(dev)))
        # order of t2fw/csrc/dfw_kernel.cu:557
        return d_q, d_k, d_v, d_s
