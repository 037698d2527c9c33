"""The forward entry point that allocates nothing (t2fw_lfw_forward_static: its scratch is a buffer
built into the library) against t2fw_lfw_forward with a caller's workspace, through the C ABI:
the same kernels run, so outputs, final state and checkpoints must be equal bit for bit.  Two calls
in a row, the second on a smaller input (the buffer keeps what the first call left in it), then a
case whose rows are flagged and redone, then a shape the buffer cannot hold."""
import pytest
import torch

from tests.lfw_cases import make_config_inputs

pytestmark = pytest.mark.gpu


def _forward(lib, _lib, ins, C, static, with_ckpt=True):
    x = ins[0]
    B, T, D = x.shape
    K = ins[2].shape[2]
    code = _lib.DTYPE_CODE[x.dtype]
    out, nxt = torch.empty_like(x), torch.empty_like(ins[5])
    ckpt = torch.empty(B, lib.t2fw_lfw_num_ckpt(T, C), D, K, dtype=x.dtype, device="cuda") if with_ckpt else None
    st = _lib.current_stream_handle(x.device)
    ptrs = [_lib.ptr(t) for t in ins] + [_lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt)]
    if static:
        rc = lib.t2fw_lfw_forward_static(*ptrs, B, T, D, K, C, code, 0, st)
    else:
        wsb = lib.t2fw_lfw_workspace_bytes(B, T, D, K, C, code, 0)
        ws = torch.zeros(max(wsb, 256), dtype=torch.uint8, device="cuda")
        rc = lib.t2fw_lfw_forward(*ptrs, B, T, D, K, C, code, 0, _lib.ptr(ws), wsb, st)
    _lib.check(rc)
    torch.cuda.synchronize()
    return out, nxt, ckpt


def _same(a, b):
    assert len(a) == len(b)
    for u, v in zip(a, b):
        if u is None:
            assert v is None
        else:
            assert torch.equal(u, v)


def test_static_forward_equals_workspace_forward_on_two_calls_in_a_row():
    from t2fw_amd import _lib
    lib = _lib.load()
    # first call: 12 rows; second call: 3 rows of another length (smaller in every dimension the
    # scratch depends on), right after it
    for (B, T, dtype, seed) in ((12, 300, torch.float16, 1), (3, 130, torch.float16, 2)):
        x, f, q, k, fk, s, _, _ = make_config_inputs(B, T, 64, 64, dtype, seed=seed, state_std=0.2)
        ins = [t.cuda() for t in (x, f, q, k, fk, s)]
        _same(_forward(lib, _lib, ins, 64, static=True), _forward(lib, _lib, ins, 64, static=False))
    # inference mode (no checkpoints) and bf16
    x, f, q, k, fk, s, _, _ = make_config_inputs(2, 96, 64, 64, torch.bfloat16, seed=3, gate_mean=3.0, state_std=0.1)
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    _same(_forward(lib, _lib, ins, 64, static=True, with_ckpt=False),
          _forward(lib, _lib, ins, 64, static=False, with_ckpt=False))


def test_static_forward_redoes_flagged_rows_and_forgets_them():
    from t2fw_amd import _lib
    lib = _lib.load()
    x, f, q, k, fk, s, _, _ = make_config_inputs(4, 128, 64, 64, torch.float16, seed=5)
    f[1, 40:60, 7] = 0.0          # a zero gate: row 1 must be redone with the exact recurrence
    fk[2, :, 3] = 1.0 / 64        # 16-step products far below what the matrix-core form takes
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    _same(_forward(lib, _lib, ins, 64, static=True), _forward(lib, _lib, ins, 64, static=False))
    # the flags the call above left in the buffer must not leak into a call with clean rows
    x, f, q, k, fk, s, _, _ = make_config_inputs(4, 128, 64, 64, torch.float16, seed=6)
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    _same(_forward(lib, _lib, ins, 64, static=True), _forward(lib, _lib, ins, 64, static=False))


def test_static_forward_general_shapes_need_no_scratch():
    from t2fw_amd import _lib
    lib = _lib.load()
    x, f, q, k, fk, s, _, _ = make_config_inputs(2, 9, 5, 3, torch.float32, seed=7, state_std=1.0)
    ins = [t.cuda() for t in (x, f, q, k, fk, s)]
    _same(_forward(lib, _lib, ins, 4, static=True), _forward(lib, _lib, ins, 4, static=False))


def test_static_forward_rejects_what_the_buffer_cannot_hold():
    from t2fw_amd import _lib
    lib = _lib.load()
    B = 1 << 20                    # the flags of so many rows exceed the built-in buffer
    code = _lib.DTYPE_CODE[torch.float16]
    assert lib.t2fw_lfw_workspace_bytes(B, 1, 64, 64, 64, code, 0) > (1 << 20)
    dummy = torch.zeros(16, dtype=torch.float16, device="cuda")
    p = _lib.ptr(dummy)
    rc = lib.t2fw_lfw_forward_static(p, p, p, p, p, p, p, p, None, B, 1, 64, 64, 64, code, 0, None)
    assert rc == 6                 # T2FW_ERR_WORKSPACE, before anything is launched
    assert b"built-in buffer" in lib.t2fw_last_error()


def test_static_forward_under_graph_capture_allocates_nothing():
    """after t2fw_static_init the call can be recorded into a HIP graph; replays on new inputs equal the
    workspace call, and the device's free memory does not move across capture and replays"""
    from t2fw_amd import _lib
    lib = _lib.load()
    _lib.check(lib.t2fw_static_init())
    B, T, C = 6, 200, 64
    code = _lib.DTYPE_CODE[torch.float16]
    mk = lambda seed: [t.cuda() for t in make_config_inputs(B, T, 64, 64, torch.float16, seed=seed, state_std=0.2)[:6]]
    static_ins = mk(11)
    out, nxt = torch.empty_like(static_ins[0]), torch.empty_like(static_ins[5])
    ckpt = torch.empty(B, lib.t2fw_lfw_num_ckpt(T, C), 64, 64, dtype=torch.float16, device="cuda")
    ptrs = [_lib.ptr(t) for t in static_ins] + [_lib.ptr(out), _lib.ptr(nxt), _lib.ptr(ckpt)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # one eager call on the capture stream first
        _lib.check(lib.t2fw_lfw_forward_static(*ptrs, B, T, 64, 64, C, code, 0, _lib.current_stream_handle(out.device)))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.t2fw_lfw_forward_static(*ptrs, B, T, 64, 64, C, code, 0, _lib.current_stream_handle(out.device)))
    graph.replay()
    torch.cuda.synchronize()
    # nothing but the graph object itself may have taken device memory (no torch allocation happened in between)
    assert torch.cuda.mem_get_info()[0] >= free_before - (8 << 20), "capture or replay allocated device memory"
    for seed in (12, 13, 14):
        fresh = mk(seed)
        want = _forward(lib, _lib, fresh, C, static=False)      # eager work between the replays
        for dst, src in zip(static_ins, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        _same((out, nxt, ckpt), want)
