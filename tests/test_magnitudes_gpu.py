"""bfloat16 tensors whose values are large enough for an intermediate of the matrix-core forms (a result times
up to 1 / product of the gates) to leave the range of its type, while every gate is inside the accepted range
and the true results are representable: the kernels look at what they store, decline such rows after the fact
and the exact recurrence redoes them.  Through the C ABI, against the fp64 oracle.  (With float16 tensors no
operand can overflow and an overflowing product means a result beyond float16: nothing to check there.)"""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs
from tests.test_lfw_chunk_gpu import NAMES, run_abi

pytestmark = pytest.mark.gpu


def rel_err(got, ref):
    ref = torch.as_tensor(ref).double()
    return (got.double().cpu() - ref).abs().max().item() / ref.abs().max().item()


def large_inputs(kind, seed):
    x, f, q, k, fk, s, go, gs = make_config_inputs(3, 128, 64, 64, torch.bfloat16, seed=seed, gate_mean=3.0, state_std=0.1)
    row = 1
    if kind == "product_of_scaled_operands":
        # value channel 0 of row 1: gates of 1/64 (16-step products of 2^-96, inside the forward's and the
        # block-wise backward's range), x of size 2^20 there and coherent q, k of size 16: (q.k) x / product > 2^128
        f[row, :, 0] = 1.0 / 64
        x[row, :, 0] = 2.0 ** 20
        q[row], k[row] = 16.0, 16.0
    elif kind == "scaled_operand":
        # x beyond 2^27 with the same gates: x / product is not a bfloat16 any more
        f[row, :, 0] = 1.0 / 64
        x[row, :, 0] = 2.0 ** 31
    elif kind == "inside_the_chunk_parallel_range":
        # gates of 0.25 on one value channel (products over half a chunk of 2^-64: the chunk-parallel backward
        # takes the row) and an incoming gradient of size 2^60 on it: its scaled copies leave fp32 in the sweeps
        f[row, :, 0] = 0.25
        go[row, :, 0] = 2.0 ** 60
        q[row], k[row] = 8.0, 8.0
    return [t.contiguous() for t in (x, f, q, k, fk, s)], go, gs, row


@pytest.mark.parametrize("kind", ["product_of_scaled_operands", "scaled_operand", "inside_the_chunk_parallel_range"])
@pytest.mark.parametrize("flags", [0, 8])
def test_rows_with_overflowing_intermediates_are_redone_exactly(kind, flags):
    """the row with the large values agrees with what the exact kernels compute (flag 1 on the same inputs; at such
    magnitudes the bfloat16 checkpoints set their accuracy, not the redo), the other rows with the oracle, both
    within the matrix-core bounds; everything finite, as the oracle's results are"""
    inputs, go, gs, row = large_inputs(kind, seed=40)
    r_out, r_nxt = c_oracle.lfw_forward(*inputs)
    r_grads = c_oracle.lfw_backward(go, gs, *inputs)
    for t in [r_out, r_nxt] + list(r_grads):
        assert torch.isfinite(torch.as_tensor(t)).all() and float(torch.as_tensor(t).abs().max()) < 3e38
    out, nxt, ckpt, grads, flagged = run_abi(inputs, go, gs, 64, flags)
    e_out, e_nxt, _, e_grads, _ = run_abi(inputs, go, gs, 64, 1)
    others = [r for r in range(inputs[0].shape[0]) if r != row]
    triples = [("outputs", out, e_out, r_out), ("next_state", nxt, e_nxt, r_nxt)]
    triples += [(n, g, e, r) for n, g, e, r in zip(NAMES, grads, e_grads, r_grads)]
    for name, got, exact, ref in triples:
        assert torch.isfinite(got).all(), "%s has non-finite values (%s, flags %d)" % (name, kind, flags)
        # (the gate gradients of the block-wise backward are differences of terms that carry the large channel: with
        # one channel 2^30 above the others their bf16 operand rounding shows, up to 5e-2 here, overflow or not)
        bound = 6e-2 if name in ("d_f", "d_f_key") else 1e-2
        err = rel_err(got[row], exact[row].cpu())
        assert err <= bound, "%s of the row with the large values: %.3e of max|exact kernels' result| (%s, flags %d)" % (name, err, kind, flags)
        bound = 2e-2 if name in ("d_f", "d_f_key") else 1e-2
        err = rel_err(got[others], torch.as_tensor(ref)[others])
        assert err <= bound, "%s: %.3e of max|ref| on the other rows (%s, flags %d)" % (name, err, kind, flags)


def test_the_fast_path_alone_reports_such_rows():
    """T2FW_FLAG_NO_FIXUP: nothing is redone, the flags say which rows are not valid"""
    inputs, go, gs, row = large_inputs("product_of_scaled_operands", seed=41)
    out, nxt, ckpt, grads, flagged = run_abi(inputs, go, gs, 64, 4)
    assert flagged[0] >= 1            # the forward declined the row after the fact
    assert not torch.isfinite(out[row]).all()
    assert torch.isfinite(out[0]).all() and torch.isfinite(out[2]).all()
    # the backward's turn: the forward is fine here, the chunk-parallel backward's sweeps are not
    inputs, go, gs, row = large_inputs("inside_the_chunk_parallel_range", seed=41)
    out, nxt, ckpt, grads, flagged = run_abi(inputs, go, gs, 64, 4)
    assert flagged[0] == 0 and flagged[1] >= 1
    assert torch.isfinite(out).all()
    assert any(not torch.isfinite(g[row]).all() for g in grads)
    assert all(torch.isfinite(g[0]).all() and torch.isfinite(g[2]).all() for g in grads)
