#!/usr/bin/env python3
"""Benchmark of the LFW hot path on one MI355X.

A "step" is one forward + backward pass of the decay-rule recurrence over one batch of
synthetic input already resident in HBM, at the headline configuration
(B*H=96, T=1024, D=K=64, fp16 I/O, checkpoint interval 64).  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg3_heads|cfg3_refgates|cfg2|cfg4|cfg5|dfw|copy256|copy64]
                    [--no-cpu-baseline] [--no-other-configs] [--force-scan] [--dfw-bf16-operands]
                    [--dfw-dtype float32|float16|bfloat16]

value      = B*T*steps / wall time of the timed region, in Mtokens/s (token = one
             (batch row, time step) pair), driving the C ABI directly with preallocated
             outputs; `autograd_api` repeats it through LFWFunction.apply + backward.
roofline   = algorithmic bytes of the dominant call (the backward: four launches, named in
             `launches`) / its mean duration as shipped (flags 0), measured with events on the launch
             stream; `launch_ms` gives the median and the 20th / 80th percentile of the same calls;
             `backward_no_fixup_ms` / `frac_no_fixup` are the call a caller makes that holds the
             forward's all-zero hints (it leaves the fourth launch out).  `traffic` = HBM bytes of the
             same launches from profiles/traffic_<workload>.json (rocprofv3 counters, not measured in
             this run: `traffic_source` says so).  Against 8 TB/s.
other_configs = after the headline's timed region (cfg3 only): cfg2, cfg4, cfg3 with the gates of the
             reference's tests, cfg5, the delta rule (default and single-operand mode) and cfg3's shape
             with float32 tensors, and a 128 x 128 state (run as 64 x 64 blocks), each briefly.
dfw        = the delta-rule kernels (forward + backward) at cfg3's shape in fp32, the dtype the
             reference tests them in (--dfw-bf16-operands: their opt-in single-operand mode;
             --dfw-dtype: 16-bit tensors through the same kernels).
copy256    = calibration workload for those counters: a 256 MiB device-to-device copy.
copy64     = the same copy at 64 MiB: source and destination together stay inside the 256 MB of last-level cache.
cpu_baseline = the TorchScript restatement of the reference loop (oracle/), fp32,
             forward + autograd backward, timed on this host's cores on a bounded sample.
parity     = computed in the same CPU leg: per tensor, the GPU results of the first three rows of
             input set 0 against the float64 oracle on the same quantised inputs (max-abs error,
             max-abs error / max|reference|, mean relative error), and beside each the error of the
             reference's own arithmetic (its recurrence evaluated in the tensors' dtype on the CPU).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (B, T, D, K, dtype, gate_mean, state_std, backward)
    "cfg2": dict(B=96, T=1024, D=64, K=64, dtype="float16", gate_mean=2.0, state_std=0.0, backward=False),
    "cfg3": dict(B=96, T=1024, D=64, K=64, dtype="float16", gate_mean=2.0, state_std=0.0, backward=True),
    # cfg3 with the head axis kept next to the channels: tensors [8, 1024, 12, 64], head-strided entry points
    "cfg3_heads": dict(B=96, H=12, T=1024, D=64, K=64, dtype="float16", gate_mean=2.0, state_std=0.0, backward=True),
    "cfg4": dict(B=128, T=8192, D=64, K=64, dtype="bfloat16", gate_mean=3.0, state_std=0.1, backward=True),
    "cfg5": dict(B=49152, T=1, D=64, K=64, dtype="float16", gate_mean=2.0, state_std=0.0, backward=False),
}


def algorithmic_bytes(B, T, D, K, es, C, backward):
    """Bytes one pass must move: forward reads x,f,q,k,f_key + s0, writes out +
    next_state (+ checkpoints when a backward follows); backward reads the five inputs,
    g_out, checkpoints and g_state, writes five gradients and d_s0."""
    tok = B * T
    nc = (T + C - 1) // C
    fwd = tok * (3 * D + 3 * K) * es + 2 * B * D * K * es
    if not backward:
        return fwd, 0
    fwd += B * nc * D * K * es
    bwd = tok * (3 * D + 3 * K) * es + B * nc * D * K * es + tok * (2 * D + 3 * K) * es + 2 * B * D * K * es
    return fwd, bwd


def percentiles(v):
    """median, 20th and 80th percentile (the three figures the reference's do_bench returns,
    tests/benchmark.py:66-71)"""
    import numpy as np
    a = np.asarray(v, dtype=np.float64)
    return {"p50": round(float(np.percentile(a, 50)), 5), "p20": round(float(np.percentile(a, 20)), 5),
            "p80": round(float(np.percentile(a, 80)), 5)}


def bench_lfw(args, name, steps, warmup, extras, max_sets=16, gates="config"):
    """Forward (+ backward) of the decay rule through the C ABI on workload `name`; returns the JSON line
    as a dict.  extras: also the autograd leg, the CPU baseline and the parity report."""
    import torch
    from t2fw_amd import _lib
    from t2fw_amd.synthetic import make_config_inputs, make_reference_test_inputs

    lib = _lib.load()
    w = WORKLOADS[name]
    B, T, D, K = w["B"], w["T"], w["D"], w["K"]
    H = w.get("H")                     # None: folded rows [B, T, D]; else rows are the heads of [B / H, T, H, D] tensors
    dtype = getattr(torch, w["dtype"])
    es = torch.empty((), dtype=dtype).element_size()
    C = args.ckpt_interval
    backward = w["backward"]
    flags = _lib.FLAG_FORCE_SCAN if args.force_scan else _lib.FLAG_AUTO
    code = _lib.DTYPE_CODE[dtype]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # several independent input sets so that consecutive steps do not re-read the same
    # lines out of the 256 MB last-level cache
    per_set = (5 * B * T * D + (B * T * D if backward else 0)) * es * (2 if backward else 1) + 2 * B * T * D * es
    nsets = max(2, min(max_sets, int(1.2e9 // max(per_set, 1)) + 1))
    sets = []
    nc = lib.t2fw_lfw_num_ckpt(T, C)
    ws_bytes = lib.t2fw_lfw_workspace_bytes(B, T, D, K, C, code, flags)
    for i in range(nsets):
        if gates == "reference_test":      # per-channel constant gates in (1/64, 63/64), tests/test_lfw.py:10-16
            x, f, q, k, fk, s, go, gs = make_reference_test_inputs(B, T, D, K, dtype, seed=i)
            x, q, k = x / 8, q / 8, k / 8
        else:
            x, f, q, k, fk, s, go, gs = make_config_inputs(B, T, D, K, dtype, seed=i, gate_mean=w["gate_mean"],
                                                            state_std=w["state_std"])
        if H:
            heads = lambda t: t.view(B // H, H, T, t.shape[2]).transpose(1, 2).contiguous()
            x, f, q, k, fk, go = (heads(t) for t in (x, f, q, k, fk, go))
        ins = [t.to(dev) for t in (x, f, q, k, fk, s)]
        d = dict(ins=ins, out=torch.empty_like(ins[0]), nxt=torch.empty_like(ins[5]),
                 ws=torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev))
        if backward:
            d["ckpt"] = torch.empty(B, nc, D, K, dtype=dtype, device=dev)
            d["go"], d["gs"] = go.to(dev), gs.to(dev)
            d["grads"] = [torch.empty_like(t) for t in ins]
        sets.append(d)
    stream = _lib.current_stream_handle(dev)

    dims = (B // H, T, H, D, K) if H else (B, T, D, K)
    lfw_forward = lib.t2fw_lfw_forward_heads if H else lib.t2fw_lfw_forward
    lfw_backward = lib.t2fw_lfw_backward_heads if H else lib.t2fw_lfw_backward

    def fwd(d, fl=None):
        _lib.check(lfw_forward(*[_lib.ptr(t) for t in d["ins"]], _lib.ptr(d["out"]), _lib.ptr(d["nxt"]),
                               _lib.ptr(d.get("ckpt")), *dims, C, code, flags if fl is None else fl,
                               _lib.ptr(d["ws"]), ws_bytes, stream))

    def bwd(d, fl=None):
        i = d["ins"]
        g = d["grads"]
        _lib.check(lfw_backward(_lib.ptr(d["go"]), _lib.ptr(d["gs"]), *[_lib.ptr(t) for t in i],
                                _lib.ptr(d["ckpt"]), *[_lib.ptr(t) for t in g], *dims, C, code,
                                flags if fl is None else fl, _lib.ptr(d["ws"]), ws_bytes, stream))

    def step(i):
        d = sets[i % nsets]
        fwd(d)
        if backward:
            bwd(d)

    # The timed region: the calls as the library ships them by default (flags 0: every decision about
    # flagged rows is taken on the device, which for the backward includes its launch for flagged rows).
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / steps * 1e3
    mtok = B * T * steps / wall / 1e6

    # per-call durations with events on the launch stream (same stream torch uses)
    nrep = min(steps, 100)

    def timed_calls(call_flags):
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(nrep)]
        for i in range(nrep):
            d = sets[i % nsets]
            ev[i][0].record()
            fwd(d, call_flags)
            ev[i][1].record()
            if backward:
                bwd(d, call_flags)
            ev[i][2].record()
        torch.cuda.synchronize()
        return [e[0].elapsed_time(e[1]) for e in ev], [e[1].elapsed_time(e[2]) for e in ev]

    fwd_ms, bwd_ms = timed_calls(flags)
    fwd_avg, bwd_avg = sum(fwd_ms) / nrep, sum(bwd_ms) / nrep
    fwd_bytes, bwd_bytes = algorithmic_bytes(B, T, D, K, es, C, backward)
    if backward and bwd_avg >= fwd_avg:
        dom, dom_bytes, dom_ms, dom_all = "backward", bwd_bytes, bwd_avg, bwd_ms
    else:
        dom, dom_bytes, dom_ms, dom_all = "forward", fwd_bytes, fwd_avg, fwd_ms
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "traffic_%s.json" % name)
    if os.path.exists(tpath) and gates == "config":
        try:
            traffic = json.load(open(tpath)).get(dom)
            traffic_source = "profiles/traffic_%s.json (rocprofv3 FETCH_SIZE / WRITE_SIZE of the same launches, static: not measured in this run)" % name
        except Exception:
            traffic = None
    chunk_parallel = C in (32, 64) and not flags & (_lib.FLAG_BLOCKWISE | _lib.FLAG_FP16_OPERANDS)
    if dom == "forward":
        launches = ["lfw_fwd_scan_kernel"] if args.force_scan else ["lfw_fwd_chunk_half_kernel" if 2 * ((B + 7) // 8 * 8) <= 256
                                                                    else "lfw_fwd_chunk_kernel"]
    elif args.force_scan:
        launches = ["lfw_bwd_scan_kernel (value side)", "lfw_bwd_scan_kernel (key side)"]
    elif chunk_parallel:
        launches = ["lfw_par_incr_kernel", "lfw_par_scan_kernel", "lfw_par_grads_kernel",
                    "lfw_bwd_chunk_kernel (rows the first three flagged)"]
    else:
        launches = ["lfw_bwd_chunk_kernel"]
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "kernel": dom, "launches": launches, "call": "as shipped (flags 0)",
                "algorithmic_bytes": dom_bytes, "avg_launch_ms": round(dom_ms, 5), "launch_ms": percentiles(dom_all)}
    if backward and not args.force_scan:
        # the same calls when the caller knows that no row will be flagged (what LFWFunction passes once the
        # forward's hints have reached the host): the backward's launch for flagged rows is left out
        _, nf = timed_calls(flags | _lib.FLAG_NO_FIXUP)
        roofline["backward_no_fixup_ms"] = round(sum(nf) / nrep, 5)
        roofline["frac_no_fixup"] = round(bwd_bytes / (sum(nf) / nrep * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    whole = (fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9

    line = {
        "metric": "fwd+bwd Mtokens/s + % HBM roofline, B*H=96 T=1024 d=kdim=64 fp16" if name == "cfg3" and gates == "config"
                  else "Mtokens/s (%s)" % name,
        "value": round(mtok, 1), "unit": "Mtokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float16": "fp16", "bfloat16": "bf16"}[w["dtype"]] + (
            " I/O, fp32 state" if args.force_scan else " I/O, bf16 MFMA operands, fp32 accumulate"),
        "data": "synthetic",
        "config": {"workload": "%s: B=%d T=%d D=%d K=%d %s %s, checkpoint interval %d%s" % (
            name, B, T, D, K, w["dtype"], "fwd+bwd" if backward else "fwd", C,
            ", gates as the reference's tests build them" if gates == "reference_test" else ""),
            "input_sets_rotated": nsets, "path": "scan" if args.force_scan else "auto"},
        "whole_step_algorithmic_GBs": round(whole, 1),
        "whole_step_roofline_frac": round(whole / HBM_PEAK_GBS, 4),
        "forward_avg_ms": round(fwd_avg, 5), "backward_avg_ms": round(bwd_avg, 5) if backward else None,
        "forward_ms": percentiles(fwd_ms), "backward_ms": percentiles(bwd_ms) if backward else None,
        "roofline": roofline,
    }
    if gates == "reference_test" and backward:
        _, bw = timed_calls(flags | _lib.FLAG_BLOCKWISE)
        line["backward_blockwise_ms"] = round(sum(bw) / nrep, 5)      # what the forward's hints make LFWFunction choose
    if not extras:
        return line

    # the same step through the autograd API (allocations and Python dispatch included)
    autograd = None
    if backward and not H:
        from t2fw.functional_lfw import LFWFunction
        os.environ["T2FW_CKPT_INTERVAL"] = str(C)
        os.environ["T2FW_FLAGS"] = str(flags)          # the same kernel path as the C-ABI legs above
        leaves = [[t.detach().clone().requires_grad_(True) for t in d["ins"]] for d in sets[:2]]

        def astep(i):
            ins = leaves[i % 2]
            o, n = LFWFunction.apply(*ins)
            torch.autograd.backward([o, n], [sets[i % 2]["go"], sets[i % 2]["gs"]])
            for t in ins:
                t.grad = None
        for i in range(5):
            astep(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n_a = min(steps, 50)
        for i in range(n_a):
            astep(i)
        torch.cuda.synchronize()
        autograd = {"ms_per_step": round((time.perf_counter() - t0) / n_a * 1e3, 4)}
        autograd["value"] = round(B * T / autograd["ms_per_step"] / 1e3, 1)
        # ... and recorded once into a HIP graph and replayed: the host cost of issuing the step
        # through autograd (which exceeds the GPU time at small shapes) disappears
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            astep(0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            o, n = LFWFunction.apply(*leaves[0])
            torch.autograd.backward([o, n], [sets[0]["go"], sets[0]["gs"]])
        for i in range(5):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_a):
            graph.replay()
        torch.cuda.synchronize()
        autograd["graph_replay_ms_per_step"] = round((time.perf_counter() - t0) / n_a * 1e3, 4)
        autograd["graph_replay_value"] = round(B * T / autograd["graph_replay_ms_per_step"] / 1e3, 1)
    line["autograd_api"] = autograd

    cpu = None
    parity = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(w, backward)
        if not H:
            parity = parity_report(sets[0], fwd, bwd if backward else None)
    line["cpu_baseline"] = cpu
    line["parity"] = parity
    if cpu:
        line["speedup_vs_cpu"] = round(mtok / cpu["value"], 1) if cpu["value"] else None
    return line


def brief(line):
    """what `other_configs` keeps of a workload's line"""
    r = line.get("roofline") or {}
    out = {"value": line["value"], "unit": line["unit"], "ms_per_step": line["ms_per_step"], "steps": line["steps"],
           "workload": line["config"]["workload"],
           "whole_step_roofline_frac": line.get("whole_step_roofline_frac"),
           "roofline": {k: r.get(k) for k in ("kernel", "frac", "achieved", "avg_launch_ms", "algorithmic_bytes")}}
    for k in ("forward_avg_ms", "backward_avg_ms", "backward_blockwise_ms", "state_GBs"):
        if line.get(k) is not None:
            out[k] = line[k]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg3", choices=sorted(WORKLOADS) + ["dfw", "copy256", "copy64", "cfg3_refgates"])
    ap.add_argument("--ckpt-interval", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="headline workload only (default: cfg2, cfg4, cfg5 and the delta rule are run briefly afterwards)")
    ap.add_argument("--force-scan", action="store_true", help="exact scan kernels only")
    ap.add_argument("--dfw-bf16-operands", action="store_true",
                    help="--workload dfw: the opt-in single-bf16 operand mode (flag 16)")
    ap.add_argument("--dfw-dtype", default="float32", choices=["float32", "float16", "bfloat16"],
                    help="--workload dfw: tensor dtype")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards over the batch with no "
              "exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.workload == "cfg5":
        line = bench_generation(args, args.steps, args.warmup)
    elif args.workload in ("copy256", "copy64"):
        line = bench_copy(args)
    elif args.workload == "dfw":
        line = bench_dfw(args, args.steps, args.warmup, args.dfw_bf16_operands, args.dfw_dtype)
    elif args.workload == "cfg3_refgates":
        line = bench_lfw(args, "cfg3", args.steps, args.warmup, extras=False, gates="reference_test")
    else:
        line = bench_lfw(args, args.workload, args.steps, args.warmup, extras=True)
        if args.workload == "cfg3" and not args.no_other_configs and not args.force_scan:
            # the other configurations of the baseline, briefly, outside the headline's timed region
            torch.cuda.empty_cache()
            others = {}
            for name, kw in (("cfg2", {}), ("cfg4", {"max_sets": 2}), ("cfg3_reference_test_gates", {"gates": "reference_test", "max_sets": 4})):
                wl = "cfg3" if name.startswith("cfg3") else name
                others[name] = brief(bench_lfw(args, wl, 20, 5, extras=False, **kw))
                torch.cuda.empty_cache()
            others["cfg5"] = brief(bench_generation(args, 50, 10))
            torch.cuda.empty_cache()
            others["dfw"] = brief(bench_dfw(args, 20, 5))
            others["dfw_bf16_operands"] = brief(bench_dfw(args, 20, 5, bf16_operands=True))
            others["dfw_float16"] = brief(bench_dfw(args, 20, 5, dtype_name="float16"))
            others["dfw_bfloat16_bf16_operands"] = brief(bench_dfw(args, 20, 5, bf16_operands=True, dtype_name="bfloat16"))
            torch.cuda.empty_cache()
            others["cfg3_float32"] = bench_float32(args, 20, 3)
            torch.cuda.empty_cache()
            others["width_128x128"] = bench_blocked_widths(args, 20, 3)
            line["other_configs"] = others
    print(json.dumps(line))


def parity_report(d, fwd, bwd, rows=3):
    """Part of the CPU leg: the GPU results of input set `d` (recomputed here, outside any timed
    region) against the float64 oracle on the first `rows` batch rows (rows are independent).
    Next to each tensor's error stands the error of the reference's own arithmetic on the same
    inputs: the recurrence of t2fw/torch.py:21-29 evaluated in the tensors' dtype on the CPU, with
    gradients by autograd, which is what the reference's test compares its kernels against
    (tests/test_lfw.py:30,48-53) and about what its kernels do (state and products in the tensor
    dtype, t2fw/csrc/lfw_kernel.cu:38,46-50)."""
    import torch
    from oracle import c_oracle, lfw_ref
    from t2fw_amd.synthetic import err_stats
    fwd(d)
    if bwd is not None:
        bwd(d)
    torch.cuda.synchronize()
    ins = [t[:rows].cpu() for t in d["ins"]]
    r_out, r_nxt = c_oracle.lfw_forward(*ins)
    names = ["outputs", "next_state"]
    got = [d["out"][:rows], d["nxt"][:rows]]
    ref = [r_out, r_nxt]
    own = None
    if bwd is not None:
        go, gs = d["go"][:rows].cpu(), d["gs"][:rows].cpu()
        names += ["d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state"]
        got += [g[:rows] for g in d["grads"]]
        ref += list(c_oracle.lfw_backward(go, gs, *ins))
        try:
            o, n, g = lfw_ref.lfw_reference_grads(*ins, go, gs, dtype=ins[0].dtype)
            own = [o, n] + list(g)
        except Exception:                 # an op this torch build lacks for the dtype on the CPU
            own = None
    else:
        try:
            with torch.no_grad():
                own = list(lfw_ref.lfw_reference(*ins))
        except Exception:
            own = None
    rep = {"reference": "float64 oracle (oracle/lfw_oracle.c) on the same quantised inputs", "rows": rows,
           "reference_arithmetic": "the recurrence of the reference evaluated in %s on the CPU (oracle/lfw_ref.py), "
                                   "same inputs, against the same float64 oracle" % str(ins[0].dtype).replace("torch.", ""),
           "tensors": {}}
    for i, name in enumerate(names):
        mx, rel, mean_rel = err_stats(got[i], torch.as_tensor(ref[i]))
        rep["tensors"][name] = {"max_abs": float("%.3e" % mx), "max_abs_over_max_ref": float("%.3e" % rel),
                                "mean_rel": float("%.3e" % mean_rel)}
        if own is not None:
            omx, orel, _ = err_stats(own[i], torch.as_tensor(ref[i]))
            rep["tensors"][name]["reference_arithmetic_max_abs_over_max_ref"] = float("%.3e" % orel)
    return rep


def bench_copy(args):
    """Calibration of the HBM traffic counters: a 256 MiB (or 64 MiB) device-to-device copy per step."""
    import torch
    mib = int(args.workload[4:])
    n = mib * 1024 * 1024
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    for _ in range(args.warmup):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gbs = 2 * n * args.steps / wall / 1e9
    return {"metric": "device copy GB/s (read + write), %d MiB" % mib, "value": round(gbs, 1), "unit": "GB/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(wall / args.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "%s: torch copy_ of %d bytes, device to device" % (args.workload, n)}}


def bench_dfw(args, steps, warmup, bf16_operands=False, dtype_name="float32"):
    """Delta rule (t2fw/functional_dfw.py:29-65) forward + backward through the C ABI: B=96, T=1024,
    D=M=64, fp32 (dtype_name: or float16 / bfloat16 tensors), keys built as the reference's test builds them
    (tests/test_dfw.py:45-46).  A step
    is one forward and one backward call; the backward call is two launches (value side, then
    query/key side).  bf16_operands: the opt-in single-bf16 mode of the matrix-core kernels (flag 16)
    instead of their default split operands.  Bytes: forward reads q,k,v,s0 and writes out,delta,final_state; backward
    reads g_out,g_state,q,k,delta,final_state and writes d_q,d_k,d_v,d_s0."""
    import torch
    from t2fw_amd import _lib
    lib = _lib.load()
    B, T, D, M = 96, 1024, 64, 64
    dtype = getattr(torch, dtype_name)
    es = torch.empty(0, dtype=dtype).element_size()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    code = _lib.DTYPE_CODE[dtype]
    flags = _lib.FLAG_FORCE_SCAN if args.force_scan else (_lib.FLAG_BF16_OPERANDS if bf16_operands else _lib.FLAG_AUTO)
    stream = _lib.current_stream_handle(dev)
    per_set = (B * T * (3 * D + 2 * M) + B * T * (2 * D + 2 * M)) * es
    nsets = max(2, min(16, int(1.2e9 // per_set) + 1))
    sets = []
    for i in range(nsets):
        g = torch.Generator().manual_seed(i)
        v = torch.randn(B, T, D, generator=g)
        q = torch.randn(B, T, M, generator=g)
        k = torch.randn(B, T, M, generator=g)
        k = torch.softmax(k, dim=-1) * torch.sigmoid(k.mean(dim=-1, keepdim=True))
        s0 = torch.randn(B, D, M, generator=g)
        go = torch.randn(B, T, D, generator=g)
        gs = torch.randn(B, D, M, generator=g)
        d = {n: t.to(dtype).to(dev) for n, t in (("q", q), ("k", k), ("v", v), ("s0", s0), ("go", go), ("gs", gs))}
        for n, like in (("out", "v"), ("delta", "v"), ("fin", "s0"), ("d_q", "q"), ("d_k", "k"), ("d_v", "v"), ("d_s0", "s0")):
            d[n] = torch.empty_like(d[like])
        sets.append(d)
    P = _lib.ptr

    def fwd(d):
        _lib.check(lib.t2fw_dfw_forward(P(d["q"]), P(d["k"]), P(d["v"]), P(d["s0"]), P(d["out"]), P(d["fin"]),
                                        P(d["delta"]), B, T, D, M, code, flags, stream))

    def bwd(d):
        _lib.check(lib.t2fw_dfw_backward(P(d["go"]), P(d["gs"]), P(d["q"]), P(d["k"]), P(d["delta"]), P(d["fin"]),
                                         P(d["d_q"]), P(d["d_k"]), P(d["d_v"]), P(d["d_s0"]), B, T, D, M, code, flags, stream))

    for i in range(warmup):
        fwd(sets[i % nsets]); bwd(sets[i % nsets])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fwd(sets[i % nsets]); bwd(sets[i % nsets])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    nrep = min(steps, 100)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(nrep)]
    for i in range(nrep):
        d = sets[i % nsets]
        ev[i][0].record(); fwd(d); ev[i][1].record(); bwd(d); ev[i][2].record()
    torch.cuda.synchronize()
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / nrep
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / nrep
    tok = B * T
    fwd_bytes = (tok * (2 * M + 3 * D) + 2 * B * D * M) * es
    bwd_bytes = (tok * (2 * D + 2 * M + 2 * M + D) + 3 * B * D * M) * es
    ms_per_step = wall / steps * 1e3
    achieved = bwd_bytes / (bwd_ms * 1e-3) / 1e9
    line = {
        "metric": "delta rule fwd+bwd Mtokens/s, B=96 T=1024 D=M=64 %s" % {"float32": "fp32", "float16": "fp16", "bfloat16": "bf16"}[dtype_name],
        "value": round(tok * steps / wall / 1e6, 1),
        "unit": "Mtokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float32": "f32", "float16": "f16 I/O, fp32 accumulate", "bfloat16": "bf16 I/O, fp32 accumulate"}[dtype_name], "data": "synthetic",
        "config": {"workload": "dfw: B=%d T=%d D=%d M=%d %s fwd+bwd" % (B, T, D, M, dtype_name), "input_sets_rotated": nsets,
                   "operands": "exact per-step kernels" if args.force_scan else
                               ("single bf16 (flag 16)" if bf16_operands else "bf16 head + remainder (default)")},
        "forward_avg_ms": round(fwd_ms, 5), "backward_avg_ms": round(bwd_ms, 5),
        "whole_step_algorithmic_GBs": round((fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "backward (two launches)",
                     "algorithmic_bytes": bwd_bytes, "avg_launch_ms": round(bwd_ms, 5)},
        "cpu_baseline": None,
    }
    return line


def bench_float32(args, steps, warmup):
    """cfg3's shape with float32 tensors through the autograd API: LFWFunction.apply (exact kernels: the
    matrix-core kernels take 16-bit tensors) against lfw_apply_16bit (casts to float16 around the matrix-core
    kernels, the caller's explicit choice), and the second one's error against the first's results."""
    import torch
    from t2fw_amd import LFWFunction, lfw_apply_16bit
    from t2fw_amd.synthetic import make_config_inputs
    w = WORKLOADS["cfg3"]
    B, T, D, K = w["B"], w["T"], w["D"], w["K"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    os.environ["T2FW_CKPT_INTERVAL"] = str(args.ckpt_interval)
    os.environ["T2FW_FLAGS"] = "0"
    x, f, q, k, fk, s0, go, gs = make_config_inputs(B, T, D, K, torch.float32, seed=0, gate_mean=w["gate_mean"])
    leaves = [t.to(dev).requires_grad_(True) for t in (x, f, q, k, fk, s0)]
    go, gs = go.to(dev), gs.to(dev)

    def run(fn, n):
        res = None
        for _ in range(n):
            for t in leaves:
                t.grad = None
            o, nx = fn(*leaves)
            torch.autograd.backward([o, nx], [go, gs])
            res = [o.detach(), nx.detach()] + [t.grad for t in leaves]
        return res
    out = {}
    results = {}
    for name, fn, n in (("exact_float32", LFWFunction.apply, max(2, steps // 4)), ("cast_to_float16", lfw_apply_16bit, steps)):
        run(fn, warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        results[name] = run(fn, n)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / n * 1e3
        out[name] = {"value": round(B * T / ms / 1e3, 1), "unit": "Mtokens/s", "ms_per_step": round(ms, 5), "steps": n}
    # the cast path recorded once into a HIP graph and replayed: its GPU time without the host's share
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(lfw_apply_16bit, 1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for t in leaves:
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o, nx = lfw_apply_16bit(*leaves)
        torch.autograd.backward([o, nx], [go, gs])
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    out["cast_to_float16"]["graph_replay_ms_per_step"] = round(ms, 5)
    out["cast_to_float16"]["graph_replay_value"] = round(B * T / ms / 1e3, 1)
    names = ["outputs", "next_state", "d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state"]
    worst = max(((a - b).abs().max() / b.abs().max()).item() for a, b in zip(results["cast_to_float16"], results["exact_float32"]))
    out["cast_to_float16"]["max_abs_over_max_ref_vs_exact_float32"] = round(worst, 6)
    out["cast_to_float16"]["tensors"] = names
    out["workload"] = "cfg3 shape, float32 tensors, LFWFunction.apply + autograd backward (host and allocations included)"
    return out


def bench_blocked_widths(args, steps, warmup):
    """A 128 x 128 state (B=24, T=1024, fp16: the state bytes of cfg3) through LFWFunction.apply + autograd:
    as the library runs it (four independent 64 x 64 blocks per row on the matrix-core kernels) against the exact
    per-step kernels (T2FW_FLAGS=1), and the first one's error against the second's results."""
    import torch
    from t2fw_amd import LFWFunction
    from t2fw_amd.synthetic import make_config_inputs
    B, T, D, K = 24, 1024, 128, 128
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    os.environ["T2FW_CKPT_INTERVAL"] = str(args.ckpt_interval)
    x, f, q, k, fk, s0, go, gs = make_config_inputs(B, T, D, K, torch.float16, seed=0, gate_mean=2.0)
    leaves = [t.to(dev).requires_grad_(True) for t in (x, f, q, k, fk, s0)]
    go, gs = go.to(dev), gs.to(dev)

    def run(n):
        res = None
        for _ in range(n):
            for t in leaves:
                t.grad = None
            o, nx = LFWFunction.apply(*leaves)
            torch.autograd.backward([o, nx], [go, gs])
            res = [o.detach(), nx.detach()] + [t.grad for t in leaves]
        return res
    out, results = {}, {}
    for name, flags, n in (("exact_kernels", "1", max(2, steps // 4)), ("blocks", "0", steps)):
        os.environ["T2FW_FLAGS"] = flags
        run(warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        results[name] = run(n)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / n * 1e3
        out[name] = {"value": round(B * T / ms / 1e3, 1), "unit": "Mtokens/s", "ms_per_step": round(ms, 5), "steps": n}
    # recorded once into a HIP graph and replayed: the GPU time without the host's share
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for t in leaves:
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o, nx = LFWFunction.apply(*leaves)
        torch.autograd.backward([o, nx], [go, gs])
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    out["blocks"]["graph_replay_ms_per_step"] = round(ms, 5)
    out["blocks"]["graph_replay_value"] = round(B * T / ms / 1e3, 1)
    worst = max(((a.double() - b.double()).abs().max() / b.double().abs().max()).item()
                for a, b in zip(results["blocks"], results["exact_kernels"]))
    out["blocks"]["max_abs_over_max_ref_vs_exact_kernels"] = round(worst, 6)
    out["blocks"]["tensors"] = ["outputs", "next_state", "d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state"]
    out["workload"] = ("B=24 T=1024 D=K=128 float16, LFWFunction.apply + autograd backward (host and allocations "
                       "included): 64 x 64 blocks on the matrix-core kernels / exact per-step kernels")
    return out


def bench_generation(args, steps, warmup):
    """cfg5: O(1) generation steps at serving batch, the state carried in place.  A "step" is
    one call of t2fw_lfw_step over the whole batch; bytes = state read + write + six vectors."""
    import torch
    from t2fw_amd import _lib
    from t2fw_amd.synthetic import make_config_inputs
    lib = _lib.load()
    w = WORKLOADS["cfg5"]
    B, D, K = w["B"], w["D"], w["K"]
    dtype = getattr(torch, w["dtype"])
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    nvec = 8
    x, f, q, k, fk, s, _, _ = make_config_inputs(B, nvec, D, K, dtype, seed=0, gate_mean=w["gate_mean"])
    vec = [[a[:, i].contiguous().to(dev) for a in (x, f, q, k, fk)] for i in range(nvec)]
    state = s.to(dev)
    out = torch.empty(B, D, dtype=dtype, device=dev)
    stream = _lib.current_stream_handle(dev)
    code = _lib.DTYPE_CODE[dtype]

    def step(i):
        v = vec[i % nvec]
        _lib.check(lib.t2fw_lfw_step(*[_lib.ptr(t) for t in v], _lib.ptr(state), _lib.ptr(out), _lib.ptr(state),
                                     B, D, K, code, stream))
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    nrep = min(steps, 100)
    ev[0].record()
    for i in range(nrep):
        step(i)
    ev[1].record()
    torch.cuda.synchronize()
    kern_ms = ev[0].elapsed_time(ev[1]) / nrep
    es = 2
    nbytes = B * (2 * D * K * es + (3 * D + 3 * K) * es)
    achieved = nbytes / (kern_ms * 1e-3) / 1e9
    line = {
        "metric": "generation steps: Mtokens/s and state GB/s (cfg5)", "value": round(B * steps / wall / 1e6, 1),
        "unit": "Mtokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(wall / steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp16 I/O, fp32 arithmetic", "data": "synthetic",
        "config": {"workload": "cfg5: B=%d T=1 D=%d K=%d float16, state carried in place over consecutive calls" % (B, D, K)},
        "state_GBs": round(2 * B * D * K * es / (kern_ms * 1e-3) / 1e9, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "lfw_step_kernel",
                     "algorithmic_bytes": nbytes, "avg_launch_ms": round(kern_ms, 5)},
        "cpu_baseline": None,
    }
    return line


def cpu_baseline(w, backward):
    """TorchScript restatement of the reference loop, fp32, on this host's cores.
    Bounded sample: a slice of the batch (rows are independent, so cost is linear in B)."""
    import torch
    from oracle.lfw_ref import lfw_reference_script
    from t2fw_amd.synthetic import make_config_inputs
    B, T, D, K = w["B"], w["T"], w["D"], w["K"]
    Bs = min(B, 24)
    Ts = min(T, 1024)
    x, f, q, k, fk, s, go, gs = make_config_inputs(Bs, Ts, D, K, torch.float32, seed=0, gate_mean=w["gate_mean"],
                                                    state_std=w["state_std"])
    ins = [t.clone().requires_grad_(backward) for t in (x, f, q, k, fk, s)]

    def run():
        o, n = lfw_reference_script(*ins)
        if backward:
            torch.autograd.backward([o, n], [go, gs])
            for t in ins:
                t.grad = None
    run()   # warm-up (TorchScript profiling runs)
    run()
    t0 = time.perf_counter()
    reps = 0
    while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 20):
        run()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(Bs * Ts / dt / 1e6, 4), "unit": "Mtokens/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "TorchScript loop (oracle/lfw_ref.py), fp32, %s, B=%d of %d rows, T=%d of %d, "
                      "%d reps, %.2f s each; host reports %d cpus" % (
                          "fwd+autograd bwd" if backward else "fwd", Bs, B, Ts, T, reps, dt, os.cpu_count())}


if __name__ == "__main__":
    main()
