"""GPU tests of the per-layer state cache (prompt through the sequence kernels, then single-token
steps through the T = 1 kernel) against the CPU oracle run on the whole sequence."""
import pytest
import torch

from oracle import c_oracle
from tests.lfw_cases import make_config_inputs
from tests.test_lfw_gpu import TOL_CHUNK, assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,D,K", [(torch.float16, 64, 64), (torch.bfloat16, 64, 64), (torch.float32, 33, 17)])
def test_prompt_then_single_steps_match_the_whole_sequence(dtype, D, K):
    from t2fw_amd.state_cache import FastWeightState
    B, T, P = 3, 48, 32                     # P prompt tokens, then T - P generation steps
    x, f, q, k, fk, s, _, _ = make_config_inputs(B, T, D, K, dtype, seed=21, state_std=0.3)
    r_out, r_nxt = c_oracle.lfw_forward(x, f, q, k, fk, s)
    xd, fd, qd, kd, fkd = (t.cuda() for t in (x, f, q, k, fk))
    layer = FastWeightState(D, K).reset(s.cuda())
    with torch.no_grad():
        outs = [layer(xd[:, :P].contiguous(), fd[:, :P].contiguous(), qd[:, :P].contiguous(), kd[:, :P].contiguous(),
                      fkd[:, :P].contiguous())]
        state_ptr = None
        for t in range(P, T):
            o = layer(xd[:, t].contiguous(), fd[:, t].contiguous(), qd[:, t].contiguous(), kd[:, t].contiguous(),
                      fkd[:, t].contiguous())
            outs.append(o.unsqueeze(1))
            if state_ptr is None:
                state_ptr = layer.state.data_ptr()
            assert layer.state.data_ptr() == state_ptr, "generation steps must update the state in place"
    out = torch.cat(outs, 1)
    tol = TOL_CHUNK if dtype != torch.float32 else None
    assert_close(out, r_out, dtype, "outputs", tol=tol)
    assert_close(layer.state, r_nxt, dtype, "state", tol=tol)


def test_zero_state_on_first_use_and_reset():
    from t2fw_amd.state_cache import FastWeightState
    B, T = 2, 16
    x, f, q, k, fk, s, _, _ = make_config_inputs(B, T, 64, 64, torch.float16, seed=22, state_std=0.0)
    r_out, _ = c_oracle.lfw_forward(x, f, q, k, fk, torch.zeros_like(s))
    layer = FastWeightState(64, 64)
    args = [t.cuda() for t in (x, f, q, k, fk)]
    with torch.no_grad():
        o1 = layer(*args)
        layer.reset()
        o2 = layer(*args)
    assert_close(o1, r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert torch.equal(o1, o2)
    with pytest.raises(RuntimeError):
        layer(*[t[:1].contiguous() for t in args])          # batch changed without reset()


def test_training_keeps_the_graph_through_the_state():
    from t2fw_amd.state_cache import FastWeightState
    B, T = 2, 32
    x, f, q, k, fk, s, go, _ = make_config_inputs(B, 2 * T, 64, 64, torch.float32, seed=23, state_std=0.2)
    leaves = [t.cuda().requires_grad_(True) for t in (x, f, q, k, fk)]
    layer = FastWeightState(64, 64).reset(s.cuda())
    o1 = layer(*[t[:, :T].contiguous() for t in leaves])
    o2 = layer(*[t[:, T:].contiguous() for t in leaves])         # depends on the first half through the state
    (torch.cat([o1, o2], 1) * go.cuda()).sum().backward()
    r = c_oracle.lfw_backward(go, torch.zeros_like(s), x, f, q, k, fk, s)
    for name, leaf, ref in zip(("d_x", "d_f", "d_q", "d_k", "d_f_key"), leaves, r):
        assert_close(leaf.grad, ref, torch.float32, name)


def test_generation_after_a_training_call_does_not_touch_the_recorded_state():
    """A training call leaves a state that belongs to its graph; the in-place generation step that
    follows works on a copy, and tensors derived from the old state keep their values."""
    from t2fw_amd.state_cache import FastWeightState
    B, T = 2, 16
    x, f, q, k, fk, s, go, _ = make_config_inputs(B, T + 1, 64, 64, torch.float16, seed=24, state_std=0.2)
    leaves = [t.cuda().requires_grad_(True) for t in (x, f, q, k, fk)]
    layer = FastWeightState(64, 64).reset(s.cuda())
    o1 = layer(*[t[:, :T].contiguous() for t in leaves])
    recorded = layer.state
    assert recorded.grad_fn is not None
    before = recorded.detach().clone()
    with torch.no_grad():
        layer(*[t[:, T].contiguous() for t in leaves])
    assert layer.state.data_ptr() != recorded.data_ptr() and layer.state.grad_fn is None
    assert torch.equal(recorded.detach(), before)
    version = layer.state._version
    with torch.no_grad():
        layer(*[t[:, T].contiguous() for t in leaves])
    assert layer.state._version > version            # the raw in-place write is visible to autograd
    (o1 * go[:, :T].cuda()).sum().backward()          # the graph of the training call is intact
    assert all(t.grad is not None for t in leaves)


def test_state_follows_the_module_across_dtype_changes():
    from t2fw_amd.state_cache import FastWeightState
    B = 2
    x, f, q, k, fk, s, _, _ = make_config_inputs(B, 2, 64, 64, torch.float32, seed=25, state_std=0.2)
    layer = FastWeightState(64, 64).reset(s.cuda())
    layer.half()
    assert layer.state.dtype == torch.float16
    with torch.no_grad():
        out = layer(*[t[:, 0].cuda().half().contiguous() for t in (x, f, q, k, fk)])
    r_out, _ = c_oracle.lfw_forward(*[t[:, :1].half() for t in (x, f, q, k, fk)], s.half())
    assert_close(out, r_out[:, 0], torch.float16, "out")
