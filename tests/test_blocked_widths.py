"""Value / key widths other than 64 on the matrix-core kernels: multiples of 64 as independent 64 x 64 blocks
(what ``LFWFunction.apply`` does by itself for fp16 / bf16 tensors), other widths padded (``lfw_apply_padded``).

CPU: the decomposition itself -- which channels go to which block, how outputs, states and gradients come back --
with the two kernel calls replaced by the oracle's plain-torch recurrence on the blocks, in float64, against the
same recurrence on the undivided tensors.  GPU: the real kernels against the C oracle."""
import pytest
import torch

from oracle.lfw_ref import lfw_reference
from tests.lfw_cases import make_config_inputs


def _fold(t):
    B, T, H, W = t.shape
    return t.transpose(1, 2).reshape(B * H, T, W)


def _heads_forward_by_oracle(x, f, q, k, fk, s, need_grad, heads=False):
    assert heads and x.is_contiguous() and k.is_contiguous() and s.is_contiguous()
    B, T, H, _ = x.shape
    out, nxt = lfw_reference(_fold(x), _fold(f), _fold(q), _fold(k), _fold(fk), s.reshape(B * H, 64, 64))
    return out.view(B, H, T, 64).transpose(1, 2).contiguous(), nxt.view(B, H, 64, 64), "ckpt", 64, 0, None


def _heads_backward_by_oracle(go, gs, x, f, q, k, fk, s, ckpt, C, flags, heads=False, hints=None):
    assert heads and ckpt == "ckpt" and go.is_contiguous() and gs.is_contiguous()
    B, T, H, _ = x.shape
    leaves = [_fold(t).clone().requires_grad_(True) for t in (x, f, q, k, fk)] + [s.reshape(B * H, 64, 64).clone().requires_grad_(True)]
    with torch.enable_grad():
        out, nxt = lfw_reference(*leaves)
        grads = torch.autograd.grad([out, nxt], leaves, [_fold(go), gs.reshape(B * H, 64, 64)])
    unfold = lambda t: t.view(B, H, T, 64).transpose(1, 2).contiguous()
    return tuple(unfold(g) for g in grads[:5]) + (grads[5].view(B, H, 64, 64),)


@pytest.mark.parametrize("H", [0, 3])
@pytest.mark.parametrize("D,K", [(128, 64), (64, 128), (128, 128), (192, 64), (64, 192), (256, 128)])
def test_decomposition_is_the_same_recurrence(monkeypatch, D, K, H):
    """H = 0: [B,T,W] tensors; H = 3: a head axis, [B,T,H,W] tensors and [B,H,D,K] states"""
    from t2fw_amd import functional_lfw as F
    monkeypatch.setattr(F, "_lfw_forward", _heads_forward_by_oracle)
    monkeypatch.setattr(F, "_lfw_backward", _heads_backward_by_oracle)
    B, T = 2, 9
    rows = B * max(H, 1)
    x, f, q, k, fk, s, go, gs = [t.double() for t in make_config_inputs(rows, T, D, K, torch.float32, seed=D + K, state_std=0.5)]
    leaves = [t.clone().requires_grad_(True) for t in (x, f, q, k, fk, s)]
    r_out, r_nxt = lfw_reference(*leaves)
    torch.autograd.backward([r_out, r_nxt], [go, gs])
    refs = [r_out.detach(), r_nxt.detach()] + [t.grad for t in leaves]
    if H:       # rows are (batch, head) pairs: the same data with the head axis next to the channels
        to_heads = lambda t: t.view(B, H, T, -1).transpose(1, 2).contiguous() if t.shape[1] == T and t.dim() == 3 else t.view(B, H, *t.shape[1:])
        x, f, q, k, fk, go = [t.view(B, H, T, -1).transpose(1, 2).contiguous() for t in (x, f, q, k, fk, go)]
        s, gs = s.view(B, H, D, K), gs.view(B, H, D, K)
        refs = [refs[0].view(B, H, T, D).transpose(1, 2), refs[1].view(B, H, D, K)] + \
               [r.view(B, H, T, -1).transpose(1, 2) for r in refs[2:7]] + [refs[7].view(B, H, D, K)]
    blocks = (D // 64, K // 64)
    out, nxt, ckpt, C, flags, kept = F._lfw_forward_blocked(x, f, q, k, fk, s, True, blocks)
    grads = F._lfw_backward_blocked(go, gs, x, f, q, k, fk, s, ckpt, C, flags, kept, blocks)
    for a, b in zip([out, nxt] + list(grads), refs):
        assert a.shape == b.shape
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_which_tensors_run_as_blocks():
    from t2fw_amd import _lib
    from t2fw_amd.functional_lfw import _block_counts
    t = lambda w, dtype=torch.float16: torch.empty(2, 3, w, dtype=dtype)
    assert _block_counts(t(128), t(64), 0) == (2, 1)
    assert _block_counts(t(64), t(192), 0) == (1, 3)
    assert _block_counts(t(256, torch.bfloat16), t(128, torch.bfloat16), 0) == (4, 2)
    assert _block_counts(t(64), t(64), 0) is None                       # the kernels' own shape
    assert _block_counts(t(128), t(100), 0) is None and _block_counts(t(32), t(64), 0) is None
    assert _block_counts(t(128, torch.float32), t(128, torch.float32), 0) is None     # exact kernels
    assert _block_counts(t(128), t(128), _lib.FLAG_FORCE_SCAN) is None
    heads = lambda w: torch.empty(2, 3, 5, w, dtype=torch.float16)
    assert _block_counts(heads(128), heads(64), 0) == (2, 1) and _block_counts(heads(64), heads(64), 0) is None


def test_padding_takes_16_bit_tensors_only():
    from t2fw_amd import lfw_apply_padded
    x, f, q, k, fk, s, go, gs = make_config_inputs(1, 3, 100, 64, torch.float32, seed=1)
    with pytest.raises(AssertionError):
        lfw_apply_padded(x, f, q, k, fk, s)


def _check_on_gpu(fn, D, K, dtype, B=3, T=200):
    from oracle import c_oracle
    from tests.test_lfw_chunk_gpu import NAMES
    from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, D, K, dtype, seed=3 * D + K, gate_mean=2.5, state_std=0.3)
    leaves = [t.cuda().requires_grad_(True) for t in (x, f, q, k, fk, s)]
    out, nxt = fn(*leaves)
    torch.autograd.backward([out, nxt], [go.cuda(), gs.cuda()])
    torch.cuda.synchronize()
    assert out.shape == (B, T, D) and nxt.shape == (B, D, K) and out.dtype == dtype and out.is_contiguous()
    r_out, r_nxt = c_oracle.lfw_forward(x, f, q, k, fk, s)
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    assert_close(out, r_out, dtype, "outputs", tol=TOL_CHUNK)
    assert_close(nxt, r_nxt, dtype, "next_state", tol=TOL_CHUNK)
    for n, t, r in zip(NAMES, leaves, r_grads):
        assert t.grad.shape == t.shape
        assert_close(t.grad, r, dtype, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,K", [(128, 64), (64, 128), (128, 128), (192, 64), (256, 128)])
def test_multiples_of_64_through_the_autograd_function(D, K, dtype):
    """LFWFunction.apply itself, against the fp64 C oracle at the matrix-core kernels' tolerance"""
    from t2fw_amd import LFWFunction
    _check_on_gpu(LFWFunction.apply, D, K, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,K", [(32, 32), (100, 70), (65, 64), (1, 1), (128, 130)])
def test_other_widths_padded(D, K, dtype):
    from t2fw_amd import lfw_apply_padded
    _check_on_gpu(lfw_apply_padded, D, K, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("D,K", [(128, 64), (128, 128)])
def test_head_strided_tensors_with_wide_heads(D, K):
    """LFWHeadsFunction on [B,T,H,D] tensors with D, K multiples of 64: against the oracle on the folded rows"""
    from oracle import c_oracle
    from t2fw_amd import LFWHeadsFunction
    from tests.test_lfw_chunk_gpu import NAMES
    from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close
    B, H, T, dtype = 2, 3, 130, torch.float16
    x, f, q, k, fk, s, go, gs = make_config_inputs(B * H, T, D, K, dtype, seed=D + 7 * K, gate_mean=2.5, state_std=0.3)
    r_out, r_nxt = c_oracle.lfw_forward(x, f, q, k, fk, s)
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    heads = lambda t: t.view(B, H, T, -1).transpose(1, 2).contiguous()
    fold = lambda t: t.transpose(1, 2).reshape(B * H, T, -1)
    leaves = [heads(t).cuda().requires_grad_(True) for t in (x, f, q, k, fk)] + [s.view(B, H, D, K).cuda().requires_grad_(True)]
    out, nxt = LFWHeadsFunction.apply(*leaves)
    torch.autograd.backward([out, nxt], [heads(go).cuda(), gs.view(B, H, D, K).cuda()])
    torch.cuda.synchronize()
    assert out.shape == (B, T, H, D) and nxt.shape == (B, H, D, K)
    assert_close(fold(out), r_out, dtype, "outputs", tol=TOL_CHUNK)
    assert_close(nxt.reshape(B * H, D, K), r_nxt, dtype, "next_state", tol=TOL_CHUNK)
    for n, t, r in zip(NAMES, leaves, r_grads):
        g = t.grad.reshape(B * H, D, K) if n == "d_state" else fold(t.grad)
        assert_close(g, r, dtype, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)


@pytest.mark.gpu
def test_blocks_run_the_matrix_core_kernels_and_force_scan_the_exact_ones(monkeypatch):
    """128 x 128: different from the exact kernels' results (T2FW_FLAGS=1) by no more than the matrix-core
    tolerance, and not equal to them"""
    from t2fw_amd import LFWFunction
    x, f, q, k, fk, s, go, gs = make_config_inputs(2, 300, 128, 128, torch.float16, seed=77, gate_mean=2.5, state_std=0.3)
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    a, _ = LFWFunction.apply(*ins)
    monkeypatch.setenv("T2FW_FLAGS", "1")
    b, _ = LFWFunction.apply(*ins)
    torch.cuda.synchronize()
    assert not torch.equal(a, b)
    assert (a.double() - b.double()).abs().max() <= 2e-2 * b.double().abs().max()


@pytest.mark.gpu
def test_gated_and_float32_routes_inherit_the_blocks():
    """LFWGatedFunction and lfw_apply_16bit go through the same calls: 128 x 64 on logits, and float32 tensors
    narrowed to fp16, against the oracle"""
    from oracle import c_oracle
    from t2fw_amd import LFWGatedFunction, lfw_apply_16bit, sigmoid_gates
    from tests.test_lfw_gpu import TOL_CHUNK, assert_close
    B, T, D, K = 2, 150, 128, 64
    g = torch.Generator().manual_seed(4)
    x, q, k = [(torch.randn(B, T, w, generator=g) * 0.125).half() for w in (D, K, K)]
    zf, zk = [(torch.randn(B, T, w, generator=g) + 2.5).half() for w in (D, K)]
    s = (torch.randn(B, D, K, generator=g) * 0.3).half()
    out, nxt = LFWGatedFunction.apply(x.cuda(), zf.cuda(), q.cuda(), k.cuda(), zk.cuda(), s.cuda())
    f, fk = [t.cpu() for t in sigmoid_gates(zf.cuda(), zk.cuda())]
    r_out, r_nxt = c_oracle.lfw_forward(x, f, q, k, fk, s)
    assert_close(out, r_out, torch.float16, "outputs (logits)", tol=TOL_CHUNK)
    assert_close(nxt, r_nxt, torch.float16, "next_state (logits)", tol=TOL_CHUNK)
    x32, f32, q32, k32, fk32, s32, _, _ = make_config_inputs(B, T, D, K, torch.float32, seed=8, gate_mean=2.5, state_std=0.3)
    out, nxt = lfw_apply_16bit(*[t.cuda() for t in (x32, f32, q32, k32, fk32, s32)])
    r_out, r_nxt = c_oracle.lfw_forward(x32, f32, q32, k32, fk32, s32)
    assert out.dtype == torch.float32
    assert (out.double().cpu() - torch.as_tensor(r_out).double()).abs().max() <= 1e-2 * torch.as_tensor(r_out).double().abs().max()
    assert (nxt.double().cpu() - torch.as_tensor(r_nxt).double()).abs().max() <= 1e-2 * torch.as_tensor(r_nxt).double().abs().max()
