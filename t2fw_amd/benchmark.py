"""Sequence-length sweep of the fast-weight rules against softmax attention: run time and peak
memory per variant, in the shape of the reference's harness (tests/benchmark.py: variants
`:82`, sweep `range(0, 2048, 128)` `:84`, backward / inference toggles `:85-88`, `bsz=32`,
`dim=kdim=64`, fp16 `:90-94`, timing protocol `:10-71`, peak memory `:134,149-151`).

    python -m t2fw_amd.benchmark                      # forward, sequence mode
    python -m t2fw_amd.benchmark --backward           # forward + backward
    python -m t2fw_amd.benchmark --inference          # one generated token with the state carried
                                                      # (attention: one query over the whole context)

Timing: warm-up, then `--reps` timed calls, a cache-flush buffer zeroed before each (512 MB,
twice MI355X's 256 MB last-level cache), HIP events around the call, median and the 20th /
80th percentile; gradients are dropped between calls.  Prints two tables (ms, peak MB).
"""
import argparse

import torch

from .functional_dfw import DFWFunction
from .functional_lfw import LFWFunction, lfw_step

FLUSH_BYTES = 512 * 1024 * 1024


_flush = None


def flush_buffer():
    """The cache-flush buffer, allocated once (so that peak-memory figures can leave it out)."""
    global _flush
    if _flush is None:
        _flush = torch.empty(FLUSH_BYTES, dtype=torch.int8, device="cuda")
    return _flush


def timed(fn, warmup_ms=25.0, reps=100, drop_grads=()):
    """(median, p20, p80) milliseconds of fn() on the current stream."""
    fn()
    torch.cuda.synchronize()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    for _ in range(5):
        fn()
    t1.record()
    torch.cuda.synchronize()
    estimate = max(t0.elapsed_time(t1) / 5, 1e-3)
    flush = flush_buffer()
    for _ in range(int(warmup_ms / estimate)):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        for t in drop_grads:
            t.grad = None
        flush.zero_()
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([a.elapsed_time(b) for a, b in zip(starts, stops)])
    p20, p80 = torch.quantile(times, torch.tensor([0.2, 0.8])).tolist()
    return times.median().item(), p20, p80


def softmax_attention(q, k, v):
    return torch.softmax(q @ k.transpose(-1, -2), dim=-1) @ v


def make_inputs(bsz, seqlen, dim, kdim, dtype, single_query):
    g = torch.Generator(device="cuda").manual_seed(seqlen)
    rnd = lambda *shape: torch.randn(*shape, dtype=dtype, device="cuda", generator=g)
    value = rnd(bsz, seqlen, dim)
    # gates in (0, 1): the rules take pre-gated inputs (t2fw/functional_lfw.py:25-30)
    f = torch.sigmoid(rnd(bsz, seqlen, dim) + 2)
    k = rnd(bsz, seqlen, kdim) / 8
    f_key = torch.sigmoid(rnd(bsz, seqlen, kdim) + 2)
    q = rnd(bsz, 1 if single_query else seqlen, kdim) / 8
    s = torch.zeros(bsz, dim, kdim, dtype=dtype, device="cuda")
    return value, f, q, k, f_key, s


def run(args):
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    seqlens = [n for n in range(0, args.max_seqlen, args.seqlen_step) if n > 0]
    variants = args.variants.split(",")
    ms, mem = {v: [] for v in variants}, {v: [] for v in variants}
    for variant in variants:
        for seqlen in seqlens:
            recurrent = variant != "attention"
            # inference: a recurrent rule generates one token from its state whatever the context
            # length; attention answers one query over the whole context (tests/benchmark.py:107-119)
            n = 1 if (recurrent and args.inference) else seqlen
            value, f, q, k, f_key, s = make_inputs(args.bsz, n, args.dim, args.kdim, dtype,
                                                   single_query=(not recurrent and args.inference))
            leaves = (value, f, q, k, f_key, s)
            if args.backward:
                for t in leaves:
                    t.requires_grad_()
            grad = torch.randn_like(value[:, : q.shape[1]] if variant == "attention" else value)
            if variant == "attention":
                fwd = lambda: softmax_attention(q, k, value)
            elif variant == "LFWFunction":
                fwd = lambda: LFWFunction.apply(value, f, q, k, f_key, s)[0]
            elif variant == "DFWFunction":
                fwd = lambda: DFWFunction.apply(q, k, value, s)[0]
            elif variant == "lfw_step":
                if not args.inference or args.backward:
                    raise SystemExit("variant lfw_step needs --inference and no --backward")
                sq = [t[:, 0].contiguous() for t in (value, f, q, k, f_key)]
                fwd = lambda: lfw_step(*sq, s, inplace=True)[0]
            else:
                raise SystemExit("unknown variant %r" % variant)
            call = (lambda: fwd().backward(grad)) if args.backward else fwd
            flush_buffer()
            torch.cuda.reset_peak_memory_stats()
            with torch.set_grad_enabled(args.backward):
                med, _, _ = timed(call, reps=args.reps, drop_grads=leaves if args.backward else ())
            ms[variant].append(med)
            mem[variant].append((torch.cuda.max_memory_allocated() - FLUSH_BYTES) * 1e-6)
    return seqlens, variants, ms, mem


def table(title, seqlens, variants, cols):
    rows = [[n] + [cols[v][i] for v in variants] for i, n in enumerate(seqlens)]
    try:
        from tabulate import tabulate
        body = tabulate(rows, headers=["seqlen"] + variants, floatfmt=".4f")
    except ImportError:
        body = "\n".join("\t".join(str(c) for c in r) for r in [["seqlen"] + variants] + rows)
    return "%s\n%s\n" % (title, body)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--variants", default="attention,LFWFunction,DFWFunction")
    ap.add_argument("--backward", action="store_true")
    ap.add_argument("--inference", action="store_true")
    ap.add_argument("--bsz", type=int, default=32)
    ap.add_argument("--dim", type=int, default=64)
    ap.add_argument("--kdim", type=int, default=64)
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16", "fp32"])
    ap.add_argument("--max-seqlen", type=int, default=2048)
    ap.add_argument("--seqlen-step", type=int, default=128)
    ap.add_argument("--reps", type=int, default=100)
    args = ap.parse_args(argv)
    seqlens, variants, ms, mem = run(args)
    mode = ("inference (one token)" if args.inference else "sequence") + (", forward + backward" if args.backward else ", forward")
    print(table("Run time, ms (median) - %s, bsz=%d dim=%d kdim=%d %s" % (mode, args.bsz, args.dim, args.kdim, args.dtype),
                seqlens, variants, ms))
    print(table("Peak memory, MB (inputs, outputs and saved tensors; without the cache-flush buffer)", seqlens, variants, mem))


if __name__ == "__main__":
    main()
