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


def _dfw_forward(query, key, value, state):
    """The forward kernels on [B,T,M], [B,T,M], [B,T,D], [B,D,M]: (outputs, final_state, delta)"""
    B, T, D = value.shape
    M = query.shape[2]
    lib = _lib.load()
    dev = value.device
    with _on_device(dev):
        outputs = torch.empty_like(value)
        final_state = torch.empty_like(state)
        delta = torch.empty_like(value)
        _lib.check(lib.t2fw_dfw_forward(
            _lib.ptr(query), _lib.ptr(key), _lib.ptr(value), _lib.ptr(state), _lib.ptr(outputs),
            _lib.ptr(final_state), _lib.ptr(delta), B, T, D, M, _dtype_code(value.dtype), _dfw_flags(value.dtype),
            _lib.current_stream_handle(dev)))
    return outputs, final_state, delta


def _dfw_backward(grad_output, grad_state, query, key, delta, final_state):
    """The backward kernels: (d_q, d_k, d_v, d_s), the order of t2fw/csrc/dfw_kernel.cu:557"""
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
    return d_q, d_k, d_v, d_s


# ---- value widths that are multiples of 64 (key width 64) as independent blocks -----------------------------
# The rows of the state do not interact in the delta rule either: S[d, :] sees v[d], q, k only (the key side is
# coupled through delta_t = v_t - S_{t-1} k_t, a sum over all of M, so only the value side can be cut).  A
# [D, 64] state with D a multiple of 64 is D / 64 independent [64, 64] recurrences that share q and k; they run as
# extra batch rows on the matrix-core kernels, which take D = M = 64 only.  d_query and d_key add up over the blocks.
def _value_block_count(value, query):
    D, M = value.shape[-1], query.shape[-1]
    if M != 64 or D % 64 or D <= 64 or value.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        return 0
    if _dfw_flags(value.dtype) & _lib.FLAG_FORCE_SCAN:
        return 0
    return D // 64


def _rows_of_value_blocks(t, nd):          # [B,T,64 nd] -> [B nd,T,64]
    B, T = t.shape[:2]
    return t.view(B, T, nd, 64).permute(0, 2, 1, 3).reshape(B * nd, T, 64).contiguous()


def _rows_repeated(t, nd):                 # [B,T,M] -> [B nd,T,M]
    B, T, M = t.shape
    return t.unsqueeze(1).expand(B, nd, T, M).reshape(B * nd, T, M).contiguous()


def _value_blocks_from_rows(t, nd):        # [B nd,T,64] -> [B,T,64 nd]
    Bn, T = t.shape[:2]
    return t.view(Bn // nd, nd, T, 64).permute(0, 2, 1, 3).reshape(Bn // nd, T, 64 * nd)


def _dfw_forward_blocked(query, key, value, state, nd):
    """(outputs, final_state, what the backward needs: q and k repeated per block, delta and final state of the blocks)"""
    B, D, M = state.shape
    qb, kb = _rows_repeated(query, nd), _rows_repeated(key, nd)
    out_b, fin_b, delta_b = _dfw_forward(qb, kb, _rows_of_value_blocks(value, nd), state.view(B * nd, 64, M))
    return _value_blocks_from_rows(out_b, nd), fin_b.view(B, D, M), (qb, kb, delta_b, fin_b)


def _dfw_backward_blocked(grad_output, grad_state, qb, kb, delta_b, fin_b, nd):
    Bn, T, M = qb.shape
    B = Bn // nd
    d_qb, d_kb, d_vb, d_sb = _dfw_backward(_rows_of_value_blocks(grad_output, nd), grad_state.reshape(Bn, 64, M), qb, kb,
                                           delta_b, fin_b)
    return (d_qb.view(B, nd, T, M).sum(dim=1), d_kb.view(B, nd, T, M).sum(dim=1), _value_blocks_from_rows(d_vb, nd),
            d_sb.view(B, 64 * nd, M))


class DFWFunction(torch.autograd.Function):
    """Delta rule: out_t = S_{t-1} q_t, S_t = S_{t-1} + (v_t - S_{t-1} k_t) (x) k_t.
    Any scalar write strength is assumed to be absorbed into the key.
    D = M = 64 (fp32, fp16, bf16) runs on the matrix-core kernels, a value width that is another multiple of 64
    (with M = 64) as independent blocks on the same kernels, everything else on the exact per-step kernels."""

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
        _dtype_code(value.dtype)
        ctx.value_blocks = _value_block_count(value, query)
        if ctx.value_blocks:
            outputs, final_state, kept = _dfw_forward_blocked(query, key, value, state, ctx.value_blocks)
            ctx.save_for_backward(*kept)
        else:
            outputs, final_state, delta = _dfw_forward(query, key, value, state)
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
        if ctx.value_blocks:
            return _dfw_backward_blocked(grad_output, grad_state, query, key, delta, final_state, ctx.value_blocks)
        return _dfw_backward(grad_output, grad_state, query, key, delta, final_state)
