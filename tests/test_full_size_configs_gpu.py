"""The benchmark configurations at their full sizes, nothing reduced: the forward-only call
(no checkpoints) at B = 96, T = 1024 fp16; the long-context training shape B = 128, T = 8192 bf16;
the serving step at B = 49152 carried in place for 256 steps.  Rows are independent recurrences,
so the oracle checks a slice of rows and size-independent properties cover the rest."""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs
from tests.test_lfw_chunk_gpu import NAMES, run_abi
from tests.test_lfw_gpu import TOL_CHUNK, TOL_CHUNK_GATE, assert_close

pytestmark = pytest.mark.gpu


def test_forward_only_call_at_full_size():
    """t2fw_lfw_forward with ckpt = NULL (inference): same kernels, no checkpoint stores; the results
    equal those of the checkpointing call bit for bit."""
    from t2fw_amd import _lib
    lib = _lib.load()
    B, T, C = 96, 1024, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.float16, seed=2, state_std=0.0)
    out_c, nxt_c, ckpt, _, flagged = run_abi((x, f, q, k, fk, s), go, gs, C, with_backward=False)
    assert flagged == (0, 0)
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    code = _lib.DTYPE_CODE[x.dtype]
    out, nxt = torch.empty_like(ins[0]), torch.empty_like(ins[5])
    wsb = lib.t2fw_lfw_forward_workspace_bytes(B, T, 64, 64, C, code, 0)
    ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
    _lib.check(lib.t2fw_lfw_forward(*[_lib.ptr(t) for t in ins], _lib.ptr(out), _lib.ptr(nxt), _lib.ptr(None),
                                    B, T, 64, 64, C, code, 0, _lib.ptr(ws), wsb, _lib.current_stream_handle(ws.device)))
    torch.cuda.synchronize()
    assert torch.equal(out, out_c) and torch.equal(nxt, nxt_c)
    rows = [0, 50, 95]
    r_out, r_nxt = c_oracle.lfw_forward(*[t[rows] for t in (x, f, q, k, fk, s)])
    assert_close(out[rows], r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt[rows], r_nxt, torch.float16, "next_state", tol=TOL_CHUNK)


def test_long_context_training_shape_at_full_size():
    """B = 128, T = 8192, bf16, gates sigmoid(N(3,1)), initial state N(0, 0.1): oracle on three rows,
    every row bit-equal under a permutation of the batch."""
    B, T, C = 128, 8192, 64
    x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, 64, 64, torch.bfloat16, seed=4, gate_mean=3.0, state_std=0.1)
    out, nxt, ckpt, grads, flagged = run_abi((x, f, q, k, fk, s), go, gs, C)
    assert flagged == (0, 0)
    rows = [0, 77, 127]
    sub = [t[rows] for t in (x, f, q, k, fk, s)]
    r_out, r_nxt = c_oracle.lfw_forward(*sub)
    r_grads = c_oracle.lfw_backward(go[rows], gs[rows], *sub)
    assert_close(out[rows], r_out, torch.bfloat16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt[rows], r_nxt, torch.bfloat16, "next_state", tol=TOL_CHUNK)
    for n, g, r in zip(NAMES, grads, r_grads):
        assert_close(g[rows], r, torch.bfloat16, n, tol=TOL_CHUNK_GATE if n in ("d_f", "d_f_key") else TOL_CHUNK)
    out, nxt, grads = out.cpu(), nxt.cpu(), [g.cpu() for g in grads]
    perm = torch.randperm(B, generator=torch.Generator().manual_seed(3))
    out_p, nxt_p, _, grads_p, _ = run_abi([t[perm] for t in (x, f, q, k, fk, s)], go[perm], gs[perm], C)
    assert torch.equal(out_p.cpu(), out[perm]) and torch.equal(nxt_p.cpu(), nxt[perm])
    for n, a, b2 in zip(NAMES, grads_p, grads):
        assert torch.equal(a.cpu(), b2[perm]), n
    # the checkpoints are the states every 64 steps: the last one continues to next_state
    tail = [t[rows, T - C:].contiguous() for t in (x, f, q, k, fk)]
    r_out2, r_nxt2 = c_oracle.lfw_forward(*tail, ckpt[rows, T // C - 1].cpu())
    assert_close(nxt[rows], r_nxt2, torch.bfloat16, "next_state from the last checkpoint")


def test_serving_step_at_full_batch_for_256_steps(capsys):
    """B = 49152 (4096 x 12 heads), fp16, 256 steps carrying the state in place.  Inputs are drawn on
    the device per step; four rows are followed on the CPU: by the oracle stepped the same way (the
    carried state rounded to fp16 after every step, as the device stores it) and by the oracle run
    over the whole sequence in fp64, which gives the drift that 256 roundings cost."""
    from t2fw_amd import lfw_step
    B, T, D = 49152, 256, 64
    rows = torch.tensor([0, 1, 24575, 49151])
    gen = torch.Generator(device="cuda").manual_seed(11)
    state = torch.zeros(B, D, D, dtype=torch.float16, device="cuda")
    kept = {n: [] for n in ("x", "f", "q", "k", "fk")}
    outs = []
    for t in range(T):
        step = {}
        for n in ("x", "q", "k"):
            step[n] = (torch.randn(B, D, generator=gen, device="cuda") / 8).half()
        for n in ("f", "fk"):
            step[n] = torch.sigmoid(torch.randn(B, D, generator=gen, device="cuda") + 2.0).half()
        out, state = lfw_step(step["x"], step["f"], step["q"], step["k"], step["fk"], state)
        outs.append(out[rows.cuda()].cpu())
        for n in kept:
            kept[n].append(step[n][rows.cuda()].cpu())
    torch.cuda.synchronize()
    seq = {n: torch.stack(v, 1) for n, v in kept.items()}          # [4, T, 64]
    got_out = torch.stack(outs, 1)
    got_state = state[rows.cuda()].cpu()
    s0 = torch.zeros(len(rows), D, D, dtype=torch.float16)
    # stepped like the device
    ref_state, ref_outs = s0, []
    for t in range(T):
        o, n = c_oracle.lfw_forward(*[seq[m][:, t:t + 1] for m in ("x", "f", "q", "k", "fk")], ref_state)
        ref_outs.append(torch.as_tensor(o[:, 0]))
        ref_state = torch.as_tensor(n).half()
    assert_close(got_out, torch.stack(ref_outs, 1), torch.float16, "out", scale=2.0)
    assert_close(got_state, ref_state.double(), torch.float16, "state", scale=2.0)
    # never rounded
    r_out, r_state = c_oracle.lfw_forward(*[seq[m] for m in ("x", "f", "q", "k", "fk")], s0)
    r_out, r_state = torch.as_tensor(r_out), torch.as_tensor(r_state)
    drift_out = float((got_out.double() - r_out).abs().max() / r_out.abs().max())
    drift_state = float((got_state.double() - r_state).abs().max() / r_state.abs().max())
    with capsys.disabled():
        print("\n  serving step, 256 carried fp16 states: max |err| / max |ref| vs the unrounded fp64 oracle: "
              "out %.2e, state %.2e" % (drift_out, drift_state))
    # 256 roundings of 2^-11 relative, shrunk by the gates (mean 0.87 per side): a few fp16 ulps
    assert drift_out < 4e-3 and drift_state < 4e-3
    # the other rows took the same code path: every output finite, every state bounded like the checked ones
    assert torch.isfinite(state).all()
    assert float(state.abs().max()) < 4 * float(r_state.abs().max()) + 1.0
