"""Autograd boundary of the decay rule: same call as the reference's
``LFWFunction.apply(value, forget, query, key, f_key, state)``
(t2fw/functional_lfw.py:31-78), backed by the HIP kernels in libt2fw_hip.so.

Differences from the reference that a caller can observe:
  * the state is stored only every ``C`` steps (``[B, ceil(T/C), D, K]``) instead of
    every step (``[B, T, D, K]``, t2fw/csrc/lfw_kernel.cu:140-144); backward recomputes
    inside each chunk.  ``next_state`` is its own ``[B, D, K]`` tensor, not a view.
  * bf16 is accepted in addition to fp64/fp32/fp16.
  * kernels run on the current torch stream and on the inputs' device.
"""
import contextlib
import ctypes
import functools
import os

import torch

from . import _lib
from .path_hint import ForwardHints, choose_backward_flags

DEFAULT_CKPT_INTERVAL = 64


def _ckpt_interval():
    v = os.environ.get("T2FW_CKPT_INTERVAL")
    return int(v) if v else DEFAULT_CKPT_INTERVAL


def _flags():
    """Kernel-path flags (include/t2fw_hip.h): 0 = automatic, 1 = exact scan kernels only,
    2 = fp16 matrix-core operands for fp16 tensors, 8 = block-wise matrix-core kernels.
    Overridable with T2FW_FLAGS."""
    v = os.environ.get("T2FW_FLAGS")
    return int(v) if v else _lib.FLAG_AUTO


@functools.lru_cache(maxsize=256)
def _sizes(rows, T, D, K, C, code, flags):
    """(checkpoints per row, forward workspace bytes, forward + backward workspace bytes, flag regions)
    of a shape: calls into the library that a training loop would otherwise repeat every step"""
    lib = _lib.load()
    regions = (ctypes.c_int64 * 6)()
    _lib.check(lib.t2fw_lfw_flag_regions(rows, T, D, K, C, code, flags, regions))
    return (lib.t2fw_lfw_num_ckpt(T, C), lib.t2fw_lfw_forward_workspace_bytes(rows, T, D, K, C, code, flags),
            lib.t2fw_lfw_workspace_bytes(rows, T, D, K, C, code, flags), tuple(regions))


def _host_hints_enabled():
    """T2FW_HOST_HINTS=0 keeps every workspace in device memory (the backward then decides on the device)."""
    return os.environ.get("T2FW_HOST_HINTS", "1") != "0"


def _on_device(dev):
    """Make ``dev`` current for the allocations and the launch, without the cost of switching when it already is."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return contextlib.nullcontext()
    return torch.cuda.device(dev)


def _check_input(t, name):
    # mirrors CHECK_INPUT of t2fw/csrc/lfw.cpp:24-26 (TORCH_CHECK -> RuntimeError)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def _dtype_code(dtype):
    try:
        return _lib.DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError("t2fw: unsupported dtype %s" % dtype)


# ---- widths that are multiples of 64 (other than 64 x 64) as independent 64 x 64 blocks -------------------
# The recurrence couples neither the rows of the state nor its columns: S[d, k] sees x[d], f[d], k[k], f_key[k]
# only, and o[d] is a sum over k.  A D x K state is (D / 64) (K / 64) independent 64 x 64 recurrences -- value
# channels 64 i .. 64 i + 63 with key channels 64 j .. 64 j + 63 -- whose outputs add up over j.  For fp16 / bf16
# tensors the blocks run as heads through the head-strided entry points, i.e. on the matrix-core
# kernels, which take 64 x 64 states only; the exact per-step kernels that would otherwise serve such widths take
# 4.1 ms for a forward + backward at B=24, T=1024, D=K=128 where the blocks take 0.24 ms.  The reference has one
# kernel for every shape (t2fw/csrc/lfw_kernel.cu:105-121).
def _block_counts(value, query, flags):
    """(D / 64, K / 64) if tensors of these widths run as blocks, else None"""
    D, K = value.shape[-1], query.shape[-1]
    if value.dim() not in (3, 4) or value.dtype not in (torch.float16, torch.bfloat16) or (flags & _lib.FLAG_FORCE_SCAN):
        return None
    if D % 64 or K % 64 or D == 0 or K == 0 or (D == 64 and K == 64):
        return None
    return D // 64, K // 64


# Tensors are [B,T,W] or, with a head axis, [B,T,H,W]; states [B,D,K] or [B,H,D,K].  Block (i, j) of head h becomes
# head (h * nd + i) * nk + j of the 64-wide call.
def _value_blocks(t, nd, nk):
    lead = t.shape[:-1]
    return t.view(*lead, nd, 1, 64).expand(*lead, nd, nk, 64).reshape(lead[0], lead[1], -1, 64).contiguous()


def _key_blocks(t, nd, nk):
    lead = t.shape[:-1]
    return t.view(*lead, 1, nk, 64).expand(*lead, nd, nk, 64).reshape(lead[0], lead[1], -1, 64).contiguous()


def _state_blocks(s, nd, nk):
    B = s.shape[0]
    return s.view(B, -1, nd, 64, nk, 64).permute(0, 1, 2, 4, 3, 5).reshape(B, -1, 64, 64).contiguous()


def _state_from_blocks(sb, nd, nk, like):
    """back to the shape of ``like`` ([B,D,K] or [B,H,D,K])"""
    B = sb.shape[0]
    return sb.view(B, -1, nd, nk, 64, 64).permute(0, 1, 2, 4, 3, 5).reshape(like.shape)


def _sum_key_blocks(tb, nd, nk, like):
    """[B,T,heads of blocks,64] -> the shape of ``like`` ([B,T,D] or [B,T,H,D]): what the blocks of one row of
    blocks hold adds up (fp32 accumulation)"""
    B, T = tb.shape[:2]
    return tb.view(B, T, -1, nd, nk, 64).sum(dim=4).reshape(like.shape)


def _sum_value_blocks(tb, nd, nk, like):
    B, T = tb.shape[:2]
    return tb.view(B, T, -1, nd, nk, 64).sum(dim=3).reshape(like.shape)


class _BlockedCall:
    """What a forward call on blocks leaves for its backward call: the block copies of the six inputs (made once,
    not again in the backward) and the hints of the call underneath.  Travels in the ``hints`` slot."""
    __slots__ = ("tensors", "hints")

    def __init__(self, tensors, hints):
        self.tensors = tensors
        self.hints = hints


def _lfw_forward_blocked(value, forget, query, key, f_key, state, need_grad, blocks):
    nd, nk = blocks
    tensors = (_value_blocks(value, nd, nk), _value_blocks(forget, nd, nk), _key_blocks(query, nd, nk),
               _key_blocks(key, nd, nk), _key_blocks(f_key, nd, nk), _state_blocks(state, nd, nk))
    out_b, nxt_b, ckpt, C, flags, hints = _lfw_forward(*tensors, need_grad, heads=True)
    kept = _BlockedCall(tensors, hints) if need_grad else None
    return _sum_key_blocks(out_b, nd, nk, value), _state_from_blocks(nxt_b, nd, nk, state), ckpt, C, flags, kept


def _lfw_backward_blocked(grad_output, grad_state, value, forget, query, key, f_key, state, ckpt, C, flags, kept, blocks):
    """The adjoint of the copies is the sum over the blocks that share a channel."""
    nd, nk = blocks
    if isinstance(kept, _BlockedCall):
        tensors, hints = kept.tensors, kept.hints
    else:
        tensors = (_value_blocks(value, nd, nk), _value_blocks(forget, nd, nk), _key_blocks(query, nd, nk),
                   _key_blocks(key, nd, nk), _key_blocks(f_key, nd, nk), _state_blocks(state, nd, nk))
        hints = None
    d_xb, d_fb, d_qb, d_kb, d_fkb, d_sb = _lfw_backward(
        _value_blocks(grad_output, nd, nk), _state_blocks(grad_state, nd, nk), *tensors, ckpt, C, flags, heads=True,
        hints=hints)
    return (_sum_key_blocks(d_xb, nd, nk, value), _sum_key_blocks(d_fb, nd, nk, value),
            _sum_value_blocks(d_qb, nd, nk, query), _sum_value_blocks(d_kb, nd, nk, query),
            _sum_value_blocks(d_fkb, nd, nk, query), _state_from_blocks(d_sb, nd, nk, state))


def _lfw_forward(value, forget, query, key, f_key, state, need_grad, heads=False):
    """Checks as in t2fw/functional_lfw.py:42-49 and t2fw/csrc/lfw.cpp:24-26,36-41, then the forward
    kernels.  heads=False: x,f [B,T,D]; q,k,f_key [B,T,K]; state [B,D,K].  heads=True: x,f [B,T,H,D];
    q,k,f_key [B,T,H,K]; state [B,H,D,K].  Returns (outputs, next_state, ckpt or None, checkpoint
    interval, flags, hints): ``hints`` is None, or the forward's verdict on which backward path the
    gates allow, readable from the host once the forward has run (path_hint.py)."""
    assert value.shape == forget.shape
    assert query.shape == key.shape
    assert query.shape == f_key.shape
    assert forget.dtype == value.dtype
    assert query.dtype == value.dtype
    assert f_key.dtype == value.dtype
    assert state.dtype == value.dtype
    assert key.dtype == value.dtype
    for t, n in ((value, "x"), (forget, "f"), (query, "query"), (key, "key"),
                 (f_key, "f_key"), (state, "state")):
        _check_input(t, n)
    nd = 4 if heads else 3
    if value.dim() != nd or query.dim() != nd or state.dim() != nd:
        raise RuntimeError("t2fw: expected x,f [B,T,H,D]; q,k,f_key [B,T,H,K]; state [B,H,D,K]" if heads else
                           "t2fw: expected x,f [B,T,D]; q,k,f_key [B,T,K]; state [B,D,K]")
    B, T = value.shape[:2]
    H = value.shape[2] if heads else 1
    D, K = value.shape[-1], query.shape[-1]
    if tuple(query.shape[:-1]) != tuple(value.shape[:-1]) or \
            tuple(state.shape) != ((B, H, D, K) if heads else (B, D, K)):
        raise RuntimeError("t2fw: inconsistent shapes x %s, query %s, state %s"
                           % (tuple(value.shape), tuple(query.shape), tuple(state.shape)))
    code = _dtype_code(value.dtype)
    flags = _flags()
    blocks = _block_counts(value, query, flags)
    if blocks is not None:
        return _lfw_forward_blocked(value, forget, query, key, f_key, state, need_grad, blocks)
    lib = _lib.load()
    C = _ckpt_interval()
    dev = value.device
    nc, ws_bytes, _, regions = _sizes(B * H, T, D, K, C, code, flags)
    with _on_device(dev):
        outputs = torch.empty_like(value)
        next_state = torch.empty_like(state)
        ckpt = None
        if need_grad:
            ckpt = torch.empty((B * H, nc, D, K), dtype=value.dtype, device=dev)
        hints = None
        if need_grad and ws_bytes and regions[3] and regions[5] and _host_hints_enabled() and ForwardHints.usable(dev):
            # a backward on the matrix cores will follow: the workspace goes to pinned host memory
            hints = ForwardHints(dev, ws_bytes, regions[2], regions[3], B * H)
            ws_ptr = hints.workspace()[0]
        else:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
            ws_ptr = _lib.ptr(ws)
        ptrs = (_lib.ptr(value), _lib.ptr(forget), _lib.ptr(query), _lib.ptr(key), _lib.ptr(f_key),
                _lib.ptr(state), _lib.ptr(outputs), _lib.ptr(next_state), _lib.ptr(ckpt))
        tail = (D, K, C, code, flags, ws_ptr, ws_bytes, _lib.current_stream_handle(dev))
        if heads:
            _lib.check(lib.t2fw_lfw_forward_heads(*ptrs, B, T, H, *tail))
        else:
            _lib.check(lib.t2fw_lfw_forward(*ptrs, B, T, *tail))
        if hints is not None:
            hints.launched()
    return outputs, next_state, ckpt, C, flags, hints


def _lfw_backward(grad_output, grad_state, value, forget, query, key, f_key, state, ckpt, C, flags, heads=False,
                  hints=None):
    """The backward kernels; gradients in the order of t2fw/csrc/lfw.cpp:95, laid out as their inputs.
    ``hints``: what the forward call on the same gates left for this call (path_hint.py), or None."""
    # t2fw/functional_lfw.py:71-72
    assert grad_state.dtype == value.dtype
    assert grad_output.dtype == value.dtype
    grad_output = grad_output.contiguous()
    grad_state = grad_state.contiguous()
    blocks = _block_counts(value, query, flags)
    if blocks is not None:
        return _lfw_backward_blocked(grad_output, grad_state, value, forget, query, key, f_key, state, ckpt, C,
                                     flags, hints, blocks)
    B, T = value.shape[:2]
    H = value.shape[2] if heads else 1
    D, K = value.shape[-1], query.shape[-1]
    code = _dtype_code(value.dtype)
    lib = _lib.load()
    dev = value.device
    if hints is not None:
        flags = choose_backward_flags(flags, hints.hinted_rows(), B * H)
    ws_bytes = _sizes(B * H, T, D, K, C, code, flags)[2]
    with _on_device(dev):
        d_x = torch.empty_like(value)
        d_f = torch.empty_like(forget)
        d_q = torch.empty_like(query)
        d_k = torch.empty_like(key)
        d_fk = torch.empty_like(f_key)
        d_s = torch.empty_like(state)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
        ptrs = (_lib.ptr(grad_output), _lib.ptr(grad_state), _lib.ptr(value), _lib.ptr(forget),
                _lib.ptr(query), _lib.ptr(key), _lib.ptr(f_key), _lib.ptr(state), _lib.ptr(ckpt),
                _lib.ptr(d_x), _lib.ptr(d_f), _lib.ptr(d_q), _lib.ptr(d_k), _lib.ptr(d_fk), _lib.ptr(d_s))
        tail = (D, K, C, code, flags, _lib.ptr(ws), ws_bytes, _lib.current_stream_handle(dev))
        if heads:
            _lib.check(lib.t2fw_lfw_backward_heads(*ptrs, B, T, H, *tail))
        else:
            _lib.check(lib.t2fw_lfw_backward(*ptrs, B, T, *tail))
    return d_x, d_f, d_q, d_k, d_fk, d_s


class LFWFunction(torch.autograd.Function):
    """Decay update rule S_t = S_{t-1} * (f_t (x) f_key_t) + x_t (x) k_t, o_t = S_t q_t.
    Inputs are already gated (no sigmoid is applied here), as in the reference.
    fp16 / bf16 tensors with D = K = 64 run on the matrix-core kernels, those whose widths are other multiples
    of 64 as independent 64 x 64 blocks on the same kernels (``_block_counts`` above), everything else on the
    exact per-step kernels; T2FW_FLAGS=1 keeps the exact kernels for every shape."""

    @staticmethod
    def forward(ctx, value, forget, query, key, f_key, state):
        """Return: (outputs [B,T,D], final state [B,D,K])"""
        need_grad = any(ctx.needs_input_grad)
        outputs, next_state, ckpt, C, flags, hints = _lfw_forward(value, forget, query, key, f_key, state, need_grad)
        if need_grad:
            ctx.save_for_backward(value, forget, query, key, f_key, state, ckpt)
            ctx.ckpt_interval = C
            ctx.flags = flags
            ctx.hints = hints
        return outputs, next_state

    @staticmethod
    def backward(ctx, grad_output, grad_state):
        value, forget, query, key, f_key, state, ckpt = ctx.saved_tensors
        return _lfw_backward(grad_output, grad_state, value, forget, query, key, f_key, state, ckpt,
                             ctx.ckpt_interval, ctx.flags, hints=ctx.hints)


def sigmoid_gates(f_logit, fk_logit, out_f=None, out_fk=None):
    """f = sigmoid(f_logit), f_key = sigmoid(fk_logit) in one launch (no autograd)."""
    for t, n in ((f_logit, "f_logit"), (fk_logit, "fk_logit")):
        _check_input(t, n)
    assert f_logit.dtype == fk_logit.dtype
    lib = _lib.load()
    dev = f_logit.device
    with _on_device(dev):
        f = torch.empty_like(f_logit) if out_f is None else out_f
        fk = torch.empty_like(fk_logit) if out_fk is None else out_fk
        _lib.check(lib.t2fw_gate_forward(_lib.ptr(f_logit), _lib.ptr(fk_logit), _lib.ptr(f), _lib.ptr(fk),
                                         f_logit.numel(), fk_logit.numel(), _dtype_code(f_logit.dtype),
                                         _lib.current_stream_handle(dev)))
    return f, fk


def _gate_backward_inplace(d_f, d_fk, forget, f_key):
    """d_f, d_fk: gate gradients on entry, logit gradients d_gate * gate * (1 - gate) on return."""
    lib = _lib.load()
    dev = d_f.device
    with _on_device(dev):
        _lib.check(lib.t2fw_gate_backward(_lib.ptr(d_f), _lib.ptr(d_fk), _lib.ptr(forget), _lib.ptr(f_key),
                                          _lib.ptr(d_f), _lib.ptr(d_fk), d_f.numel(), d_fk.numel(),
                                          _dtype_code(d_f.dtype), _lib.current_stream_handle(dev)))


class LFWGatedFunction(torch.autograd.Function):
    """``LFWFunction`` on gate *logits*: f = sigmoid(f_logit), f_key = sigmoid(fk_logit) are computed
    by one streaming kernel for both gates, the gates (not the logits) are kept for backward, and
    the gate gradients are turned into logit gradients in place by one more kernel.  The reference
    leaves the non-linearity to the caller (t2fw/functional_lfw.py:25-30), where it costs two
    elementwise passes forward and several backward, plus a second saved tensor per gate."""

    @staticmethod
    def forward(ctx, value, f_logit, query, key, fk_logit, state):
        assert value.shape == f_logit.shape and query.shape == fk_logit.shape
        assert f_logit.dtype == value.dtype and fk_logit.dtype == value.dtype
        forget, f_key = sigmoid_gates(f_logit, fk_logit)
        need_grad = any(ctx.needs_input_grad)
        outputs, next_state, ckpt, C, flags, hints = _lfw_forward(value, forget, query, key, f_key, state, need_grad)
        if need_grad:
            ctx.save_for_backward(value, forget, query, key, f_key, state, ckpt)
            ctx.ckpt_interval = C
            ctx.flags = flags
            ctx.hints = hints
        return outputs, next_state

    @staticmethod
    def backward(ctx, grad_output, grad_state):
        value, forget, query, key, f_key, state, ckpt = ctx.saved_tensors
        d_x, d_f, d_q, d_k, d_fk, d_s = _lfw_backward(grad_output, grad_state, value, forget, query, key, f_key,
                                                      state, ckpt, ctx.ckpt_interval, ctx.flags, hints=ctx.hints)
        _gate_backward_inplace(d_f, d_fk, forget, f_key)
        return d_x, d_f, d_q, d_k, d_fk, d_s


class LFWHeadsFunction(torch.autograd.Function):
    """The decay rule on tensors that keep the head axis next to the channels: x, f ``[B,T,H,D]``;
    q, k, f_key ``[B,T,H,K]``; state ``[B,H,D,K]``; returns outputs ``[B,T,H,D]`` and the final state
    ``[B,H,D,K]``.  Every (batch, head) pair is one recurrence.  The reference needs the folded,
    contiguous ``[B*H,T,D]`` layout (t2fw/csrc/lfw.cpp:24-26), i.e. ``transpose(1, 2).contiguous()``
    on five inputs and the inverse on the outputs and on six gradients; here the kernels stride
    over the head axis and those copies disappear.

    ``logits=True``: ``f`` and ``f_key`` are gate logits and the sigmoid is applied here (as in
    ``LFWGatedFunction``); the gradients returned for them are then logit gradients."""

    @staticmethod
    def forward(ctx, value, forget, query, key, f_key, state, logits=False):
        if logits:
            assert value.shape == forget.shape and query.shape == f_key.shape
            assert forget.dtype == value.dtype and f_key.dtype == value.dtype
            forget, f_key = sigmoid_gates(forget, f_key)
        need_grad = any(ctx.needs_input_grad)
        outputs, next_state, ckpt, C, flags, hints = _lfw_forward(value, forget, query, key, f_key, state, need_grad,
                                                                  heads=True)
        if need_grad:
            ctx.save_for_backward(value, forget, query, key, f_key, state, ckpt)
            ctx.ckpt_interval = C
            ctx.flags = flags
            ctx.hints = hints
            ctx.logits = bool(logits)
        return outputs, next_state

    @staticmethod
    def backward(ctx, grad_output, grad_state):
        value, forget, query, key, f_key, state, ckpt = ctx.saved_tensors
        d_x, d_f, d_q, d_k, d_fk, d_s = _lfw_backward(grad_output, grad_state, value, forget, query, key, f_key,
                                                      state, ckpt, ctx.ckpt_interval, ctx.flags, heads=True,
                                                      hints=ctx.hints)
        if ctx.logits:
            _gate_backward_inplace(d_f, d_fk, forget, f_key)
        return d_x, d_f, d_q, d_k, d_fk, d_s, None


def _narrow_copies(tensors, dtype, stream):
    """``dtype`` copies of float32 tensors: one allocation, one launch."""
    dev = tensors[0].device
    offs, total = [], 0
    for t in tensors:
        offs.append(total)
        total += (t.numel() + 127) // 128 * 128          # every copy starts 256 bytes aligned
    buf = torch.empty(total, dtype=dtype, device=dev)
    outs = [buf[o:o + t.numel()].view(t.shape) for o, t in zip(offs, tensors)]
    _lib.cast_tensors(list(tensors), outs, stream)
    return outs


class LFW16Function(torch.autograd.Function):
    """The recurrence on float32 tensors through the 16-bit matrix-core kernels (see lfw_apply_16bit).  The
    16-bit copies of the inputs, not the float32 tensors, are what is kept for the backward."""

    @staticmethod
    def forward(ctx, value, forget, query, key, f_key, state, dtype):
        ins = (value, forget, query, key, f_key, state)
        for t, n in zip(ins, ("x", "f", "query", "key", "f_key", "state")):
            _check_input(t, n)
            if t.dtype != torch.float32:
                raise RuntimeError("t2fw: lfw_apply_16bit takes float32 tensors, %s is %s" % (n, t.dtype))
        need_grad = any(ctx.needs_input_grad)
        dev = value.device
        with _on_device(dev):
            stream = _lib.current_stream_handle(dev)
            narrow = _narrow_copies(ins, dtype, stream)
            out16, nxt16, ckpt, C, flags, hints = _lfw_forward(*narrow, need_grad)
            outputs, next_state = torch.empty_like(value), torch.empty_like(state)
            _lib.cast_tensors([out16, nxt16], [outputs, next_state], stream)
        if need_grad:
            ctx.save_for_backward(*narrow, ckpt)
            ctx.ckpt_interval, ctx.flags, ctx.hints, ctx.narrow = C, flags, hints, dtype
        return outputs, next_state

    @staticmethod
    def backward(ctx, grad_output, grad_state):
        *narrow, ckpt = ctx.saved_tensors
        dev = grad_output.device
        with _on_device(dev):
            stream = _lib.current_stream_handle(dev)
            go16, gs16 = _narrow_copies((grad_output.contiguous().float(), grad_state.contiguous().float()), ctx.narrow, stream)
            grads16 = _lfw_backward(go16, gs16, *narrow, ckpt, ctx.ckpt_interval, ctx.flags, hints=ctx.hints)
            grads = [torch.empty(g.shape, dtype=torch.float32, device=dev) for g in grads16]
            _lib.cast_tensors(list(grads16), grads, stream)
        return (*grads, None)


def lfw_apply_16bit(value, forget, query, key, f_key, state, dtype=torch.float16):
    """``LFWFunction.apply`` for float32 tensors at the speed of the 16-bit matrix-core kernels: the six
    inputs are converted to ``dtype`` (float16 or bfloat16) in one launch, the recurrence and its backward
    run in that type, outputs and gradients come back as float32.  An explicit choice of the caller: the
    results carry the 16-bit kernels' accuracy (within 1e-2 of max|ref| per tensor; gates are rounded to
    ``dtype`` before they are multiplied up, 2^-11 relative per step in float16, so bfloat16 is for short
    memories only), where ``LFWFunction.apply`` on float32 tensors runs the exact kernels.  The reference
    has one kernel for every dtype (t2fw/csrc/lfw_kernel.cu:157-168) and no counterpart of this."""
    assert dtype in (torch.float16, torch.bfloat16)
    return LFW16Function.apply(value, forget, query, key, f_key, state, dtype)


def lfw_apply_padded(value, forget, query, key, f_key, state):
    """``LFWFunction.apply`` for fp16 / bf16 tensors whose value or key width is not a multiple of 64, on the
    matrix-core kernels: the widths are padded up to the next multiple of 64 (values, keys, queries and the state
    with zeros, gates with ones -- the padded channels stay zero and add nothing), the padded tensors run as
    64 x 64 blocks (``LFWFunction.apply`` does that by itself for multiples of 64), and the results are cut back.
    Correct for any width, and as expensive as the padded width: a 32 x 32 state costs what a 64 x 64 one costs,
    which is still a quarter of the exact per-step kernels' time at B=96, T=1024.  An explicit choice of the
    caller, because the results carry the matrix-core kernels' accuracy where ``LFWFunction.apply`` runs the exact
    kernels for such widths.  Padding, cutting and their gradients are plain tensor operations."""
    assert value.dtype in (torch.float16, torch.bfloat16), "the matrix-core kernels take fp16 / bf16 tensors"
    assert value.shape == forget.shape and query.shape == key.shape and query.shape == f_key.shape
    B, T, D = value.shape
    K = query.shape[2]
    assert tuple(state.shape) == (B, D, K)
    Dp, Kp = 64 * -(-D // 64), 64 * -(-K // 64)
    if Dp == D and Kp == K:
        return LFWFunction.apply(value, forget, query, key, f_key, state)
    pad = torch.nn.functional.pad
    out, nxt = LFWFunction.apply(pad(value, (0, Dp - D)), pad(forget, (0, Dp - D), value=1.0), pad(query, (0, Kp - K)),
                                 pad(key, (0, Kp - K)), pad(f_key, (0, Kp - K), value=1.0),
                                 pad(state, (0, Kp - K, 0, Dp - D)))
    return out[..., :D].contiguous(), nxt[:, :D, :K].contiguous()


def lfw_step(x, f, query, key, f_key, state, out=None, inplace=True):
    """One generation step (T = 1) without autograd: x,f [B,D]; query,key,f_key [B,K];
    state [B,D,K] updated in place when ``inplace``.  Returns (out [B,D], state).
    The reference does this through the T=1 forward (tests/benchmark.py:104-105), which
    allocates a new state tensor per step."""
    for t, n in ((x, "x"), (f, "f"), (query, "query"), (key, "key"), (f_key, "f_key"), (state, "state")):
        _check_input(t, n)
        assert t.dtype == x.dtype
    B, D = x.shape
    K = query.shape[1]
    assert tuple(state.shape) == (B, D, K) and f.shape == x.shape
    assert key.shape == query.shape and f_key.shape == query.shape
    lib = _lib.load()
    dev = x.device
    with _on_device(dev):
        if out is None:
            out = torch.empty_like(x)
        nxt = state if inplace else torch.empty_like(state)
        _lib.check(lib.t2fw_lfw_step(
            _lib.ptr(x), _lib.ptr(f), _lib.ptr(query), _lib.ptr(key), _lib.ptr(f_key), _lib.ptr(state),
            _lib.ptr(out), _lib.ptr(nxt), B, D, K, _dtype_code(x.dtype), _lib.current_stream_handle(dev)))
    return out, nxt
