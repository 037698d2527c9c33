"""The autograd functions under HIP graph capture: a forward + backward step recorded once with
torch.cuda.graph and replayed on new input contents must reproduce the eager results every time.
(At the benchmark's shape one step is ~0.13 ms of GPU work, less than the host needs to issue it
through autograd; a replayed graph removes that host cost.)  Every replay is checked, with eager
work and synchronisations in between, not only the first."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def make(B, T, seed, dtype=torch.float16, heads=None):
    g = torch.Generator().manual_seed(seed)
    shape = (B, T, 64) if heads is None else (B // heads, T, heads, 64)
    mk = lambda *s: torch.randn(*s, generator=g)
    x, q, k = [(mk(*shape) / 8).to(dtype).cuda() for _ in range(3)]
    f, fk = [torch.sigmoid(mk(*shape) + 2).to(dtype).cuda() for _ in range(2)]
    s = (mk(B, 64, 64) * 0.1).to(dtype).cuda()
    if heads is not None:
        s = s.view(B // heads, heads, 64, 64)
    go = mk(*shape).to(dtype).cuda()
    gs = (mk(*s.shape) * 0.1).to(dtype).cuda()
    return [x, f, q, k, fk, s], go, gs


@pytest.mark.parametrize("kind", ["folded", "heads", "flagged"])
def test_replays_match_eager(kind):
    from t2fw_amd import LFWFunction, LFWHeadsFunction
    B, T = 6, 200
    heads = 3 if kind == "heads" else None
    fn = LFWHeadsFunction if heads else LFWFunction

    def eager(ins, go, gs):
        leaves = [t.clone().requires_grad_(True) for t in ins]
        o, n = fn.apply(*leaves)
        torch.autograd.backward([o, n], [go, gs])
        return [o.detach().clone(), n.detach().clone()] + [t.grad.clone() for t in leaves]

    static_ins, static_go, static_gs = make(B, T, 0, heads=heads)
    static_ins = [t.requires_grad_(True) for t in static_ins]

    def step():
        o, n = fn.apply(*static_ins)
        torch.autograd.backward([o, n], [static_go, static_gs])
        return o, n

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
            for t in static_ins:
                t.grad = None
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, nxt = step()
    static_grads = [t.grad for t in static_ins]

    for seed in (1, 2, 3, 4):
        ins, go, gs = make(B, T, seed, heads=heads)
        if kind == "flagged" and seed % 2 == 0:
            ins[1][seed, 7, 5] = -0.0           # a row for the exact kernels, on some replays only
        want = eager(ins, go, gs)               # eager work between the replays
        torch.cuda.synchronize()
        with torch.no_grad():
            for dst, src in zip(static_ins, ins):
                dst.copy_(src)
            static_go.copy_(go)
            static_gs.copy_(gs)
        graph.replay()
        torch.cuda.synchronize()
        got = [out, nxt] + static_grads
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), "replay with seed %d: result %d differs from eager" % (seed, i)
