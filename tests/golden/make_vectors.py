"""Writes the two small fixtures of this folder from the oracle (float64).  Run from the repository root:
    python tests/golden/make_vectors.py
The reference is not involved: inputs are seeded here, outputs come from oracle/lfw_ref.py and oracle/dfw_ref.py."""
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.dfw_ref import dfw_reference_grads  # noqa: E402
from oracle.lfw_ref import lfw_reference_grads  # noqa: E402


def tolist(t):
    return t.detach().to(torch.float64).tolist()


def lfw_case():
    g = torch.Generator().manual_seed(20240611)
    B, T, D, K = 2, 5, 3, 2
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x, q, k = r(B, T, D), r(B, T, K), r(B, T, K)
    f, fk = torch.sigmoid(r(B, T, D)), torch.sigmoid(r(B, T, K))
    s0, go, gs = r(B, D, K), r(B, T, D), r(B, D, K)
    out, nxt, grads = lfw_reference_grads(x, f, q, k, fk, s0, go, gs)
    names = ["x", "f", "q", "k", "f_key", "s0", "g_out", "g_state"]
    d = {n: tolist(t) for n, t in zip(names, (x, f, q, k, fk, s0, go, gs))}
    d.update(outputs=tolist(out), next_state=tolist(nxt))
    d.update({n: tolist(t) for n, t in zip(["d_x", "d_f", "d_q", "d_k", "d_f_key", "d_state"], grads)})
    return d


def dfw_case():
    g = torch.Generator().manual_seed(20240612)
    B, T, D, M = 2, 5, 3, 2
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    q, k, v = r(B, T, M), 0.5 * r(B, T, M), r(B, T, D)
    s0, go, gs = r(B, D, M), r(B, T, D), r(B, D, M)
    out, fin, grads = dfw_reference_grads(q, k, v, s0, go, gs)
    d = {n: tolist(t) for n, t in zip(["q", "k", "v", "s0", "g_out", "g_state"], (q, k, v, s0, go, gs))}
    d.update(outputs=tolist(out), final_state=tolist(fin))
    d.update({n: tolist(t) for n, t in zip(["d_q", "d_k", "d_v", "d_state"], grads)})
    return d


if __name__ == "__main__":
    for name, case in (("lfw_small.json", lfw_case()), ("dfw_small.json", dfw_case())):
        with open(os.path.join(HERE, name), "w") as fh:
            json.dump(case, fh, indent=0)
        print("wrote", name)
