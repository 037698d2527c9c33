"""GPU parity of the matrix-core kernels with a checkpoint per 16-step block (C = 16): the
backward then reads every block-start state from memory instead of recomputing it, and only
the last block of a sequence keeps a recompute stage.  Same oracle, tolerances and cases as for
the longer intervals, plus the checkpoints themselves."""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs
from tests.test_heads_gpu import check_heads
from tests.test_lfw_chunk_gpu import NAMES, check_against_oracle, run_abi
from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close

pytestmark = pytest.mark.gpu
C = 16


@pytest.mark.parametrize("dtype,gate_mean,state_std", [(torch.float16, 2.0, 0.0), (torch.bfloat16, 3.0, 0.1)])
@pytest.mark.parametrize("B,T", [(4, 1024), (3, 1000), (2, 77), (5, 1), (2, 16), (2, 17), (2, 32), (2, 33), (1, 48),
                                 (2, 49), (1, 64), (3, 65), (2, 80), (2, 96), (1, 112), (1, 130), (2, 15)])
def test_config_like_inputs(dtype, gate_mean, state_std, B, T):
    """every count of blocks modulo three (the backward peels that many stages) and modulo four (the
    gate-gradient sum is re-anchored every fourth block), with and without a partial last block"""
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, dtype, seed=T, gate_mean=gate_mean,
                                                    state_std=max(state_std, 0.2 if T < 100 else 0.0))
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, dtype, expect_flagged=0)


def test_checkpoints_are_the_block_start_states():
    B, T = 3, 200
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=9, state_std=0.3)
    out, nxt, ckpt, _, _ = run_abi((x, f, q, k, fk, s), go, gs, C, with_backward=False)
    assert ckpt.shape[1] == 13
    assert torch.equal(ckpt[:, 0].cpu(), s)
    for c in (1, 2, 5, 12):
        _, n, _, _, _ = run_abi([t[:, :16 * c].contiguous() for t in (x, f, q, k, fk)] + [s], go, gs, C,
                                with_backward=False)
        assert torch.equal(ckpt[:, c].cpu(), n.cpu()), c
    # and the same outputs as with the default interval
    out64, nxt64, _, _, _ = run_abi((x, f, q, k, fk, s), go, gs, 64, with_backward=False)
    assert torch.equal(out, out64) and torch.equal(nxt, nxt64)


def test_batch_larger_than_half_the_device_with_a_flagged_row():
    B, T = 136, 80
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=31, state_std=0.2)
    f = f.clone()
    f[135, 70, 50] = 1.25
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (1, 1), flagged
    rows = [0, 63, 64, 127, 128, 135]
    sub = [t[rows] for t in (x, f, q, k, fk, s)]
    r_out, r_nxt = c_oracle.lfw_forward(*sub)
    r_grads = c_oracle.lfw_backward(go[rows], gs[rows], *sub)
    assert_close(out[rows], r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt[rows], r_nxt, torch.float16, "next_state", tol=TOL_CHUNK)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[rows], r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)


def test_flagged_rows_with_a_partial_last_block():
    B, T = 3, 90
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=11, state_std=0.3)
    f, fk = f.clone(), fk.clone()
    f[0, 40, 9] = 0.0
    fk[2, 89, 63] = 2.0
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (2, 2), flagged
    r_grads = c_oracle.lfw_backward(go, gs, x, f, q, k, fk, s)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[0:1], r[0:1], torch.float16, n + "[flagged row 0]")
        assert_close(g[2:3], r[2:3], torch.float16, n + "[flagged row 2]")
        assert_close(g, r, torch.float16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)


def test_wide_gate_distribution():
    x, f, q, k, fk, s, go, gs = make_config_inputs(3, 256, 64, 64, torch.float16, seed=5, gate_mean=0.0, state_std=0.5)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, torch.float16, expect_flagged=0, gate_tol=(2e-1, 4e-2))


def test_fp16_operands():
    x, f, q, k, fk, s, go, gs = make_config_inputs(2, 256, 64, 64, torch.float16, seed=8, gate_mean=4.5, state_std=0.3)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, torch.float16, flags=2, expect_flagged=0,
                         tol=(4e-3, 2e-3), gate_tol=(1e-2, 8e-3))


@pytest.mark.parametrize("B,H,T", [(2, 3, 200), (1, 12, 77), (9, 16, 150)])
def test_head_strided_layout(B, H, T):
    x, f, q, k, fk, s, go, gs = make_config_inputs(B * H, T, 64, 64, torch.float16, seed=T + H, state_std=0.2)
    check_heads((x, f, q, k, fk, s), go, gs, B, H, C, torch.float16, expect_flagged=0,
                oracle_rows=None if B * H < 20 else [0, 1, 15, 16, 77, 143])


def test_long_context_bf16_slice():
    B, T = 2, 8192
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.bfloat16, seed=4, gate_mean=3.0, state_std=0.1)
    check_against_oracle((x, f, q, k, fk, s), go, gs, C, torch.bfloat16, expect_flagged=0)
