"""GPU parity of the delta-rule kernels against the CPU oracle (fp64, same inputs), through
DFWFunction.  Mirrors the reference's test (tests/test_dfw.py:30-115): same shape grid
(incl. dim=96), fp32, keys = softmax(k) * sigmoid(mean k), two-call backward protocol; its
tolerances (:77, :104) are the outer bound and a tighter stated tolerance is enforced."""
import math

import pytest
import torch

from oracle.dfw_ref import dfw_reference_grads
from tests.test_lfw_gpu import assert_close

pytestmark = pytest.mark.gpu
NAMES = ("d_q", "d_k", "d_v", "d_state")
# delta-rule errors compound through the state (each step re-reads what it wrote), so the
# bound is wider than one rounding: |err| <= rtol*|ref| + afrac*max|ref|
TOL_DFW = {torch.float32: (2e-4, 2e-4), torch.float64: (1e-10, 1e-10),
           torch.float16: (1e-2, 8e-3), torch.bfloat16: (1e-2, 6e-3)}


def shape_grid():
    """tests/test_dfw.py:20-26"""
    for bsz in range(1, 16, 4):
        for dim in range(1, 64, 32):
            for seqlen in range(1, 512, 128):
                yield bsz, seqlen, dim
    yield 2, 1024, 32
    yield 2, 1024, 96


def make_inputs(bsz, seqlen, dim, mdim, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    v = torch.randn(bsz, seqlen, dim, generator=g)
    q = torch.randn(bsz, seqlen, mdim, generator=g)
    k = torch.randn(bsz, seqlen, mdim, generator=g)
    k = torch.softmax(k, dim=-1) * torch.sigmoid(k.mean(dim=-1, keepdim=True))     # test_dfw.py:45-46
    s = torch.randn(bsz, dim, mdim, generator=g)
    go = torch.randn(bsz, seqlen, dim, generator=g)
    gs = torch.randn(bsz, dim, mdim, generator=g)
    return tuple(t.to(dtype) for t in (q, k, v, s, go, gs))


def check(q, k, v, s, go, gs, dtype):
    from t2fw.functional_dfw import DFWFunction
    ins = [t.cuda().requires_grad_(True) for t in (q, k, v, s)]
    out, fin = DFWFunction.apply(*ins)
    out.backward(go.cuda(), retain_graph=True)
    fin.backward(gs.cuda())
    torch.cuda.synchronize()
    r_out, r_fin, r_grads = dfw_reference_grads(q, k, v, s, go, gs)
    tol = TOL_DFW[dtype]
    assert out.dtype == dtype and fin.dtype == dtype
    assert_close(out, r_out, dtype, "outputs", tol=tol)
    assert_close(fin, r_fin, dtype, "final_state", tol=tol)
    for n, t, r in zip(NAMES, ins, r_grads):
        assert_close(t.grad, r, dtype, n, tol=tol)
    if dtype == torch.float32:      # the reference's own tolerances
        assert torch.allclose(out.double().cpu(), r_out, atol=1e-2, rtol=1e-1)
        for t, r in zip(ins, r_grads):
            assert torch.allclose(t.grad.double().cpu(), r, atol=0.1, rtol=1e-1)


@pytest.mark.parametrize("bsz,seqlen,dim", list(shape_grid()))
def test_reference_shape_grid_fp32(bsz, seqlen, dim):
    mdim = math.ceil(dim / 2)
    check(*make_inputs(bsz, seqlen, dim, mdim, torch.float32, seed=2000 + bsz + seqlen + dim), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 70, 64, 64), (2, 33, 5, 130), (2, 40, 130, 3), (1, 9, 1, 1)])
def test_other_dtypes_and_shapes(dtype, shape):
    B, T, D, M = shape
    check(*make_inputs(B, T, D, M, dtype, seed=7), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", [(1, 6, 3, 100), (1, 6, 100, 3), (1, 5, 2, 600), (1, 5, 600, 2), (1, 4, 2, 2048),
                                   (1, 4, 2048, 2)])
def test_wide_states_every_lane_geometry(dtype, shape):
    """state rows of 65..128, 513..1024 and 2048 columns on either side (32 lanes per row, 16 / 32
    columns per lane)"""
    B, T, D, M = shape
    check(*make_inputs(B, T, D, M, dtype, seed=8), dtype)


def test_value_dim_larger_than_key_dim():
    # D > M, the case where the reference's backward kernel overruns its shared memory
    # (dfw_kernel.cu:227 vs :523); nothing of the kind exists here
    check(*make_inputs(2, 64, 96, 8, torch.float32, seed=3), torch.float32)


def test_empty_sequence_and_errors():
    from t2fw.functional_dfw import DFWFunction
    s = torch.randn(2, 4, 3, device="cuda")
    e = lambda w: torch.empty(2, 0, w, device="cuda")
    o, n = DFWFunction.apply(e(3), e(3), e(4), s)
    assert o.shape == (2, 0, 4) and torch.equal(n, s)
    q = torch.randn(2, 5, 3, device="cuda")
    v = torch.randn(2, 5, 4, device="cuda")
    with pytest.raises(AssertionError):                       # functional_dfw.py:38
        DFWFunction.apply(q, q[:, :4].contiguous(), v, s)
    with pytest.raises(AssertionError):                       # functional_dfw.py:39
        DFWFunction.apply(q.half(), q.half(), v, s)
    with pytest.raises(RuntimeError):
        DFWFunction.apply(q.cpu(), q.cpu(), v.cpu(), s.cpu())
