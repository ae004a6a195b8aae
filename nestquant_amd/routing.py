"""Synthetic routing for tests and benches (reference sm120/routing.py:4-20, sm120/common.py:3-8).

'distinct': no expert shared between tokens (worst case, 8 B runs). 'recency': token t reuses each of token t-1's
experts with probability p. `routings` makes consecutive calls avoid the previous call's experts so weights are cold.
`softmax_topk` is the seeded router of the full-layer configuration: softmax over N(0,1) logits, top-k, fp16 weights."""
import random

import torch


def make_sel(B, pool, mode="recency", p=0.4, rng=None, avoid=(), topk=8):
    rng = rng or random.Random(0)
    avoid = set(avoid)
    pool = [e for e in pool if e not in avoid]
    rows, used = [], set()
    for t in range(B):
        row = []
        if t and mode == "recency":
            row = [e for e in rows[-1] if rng.random() < p]
        cand = [e for e in pool if e not in row and (mode != "distinct" or e not in used)]
        rng.shuffle(cand)
        row += cand[: topk - len(row)]
        rng.shuffle(row)
        rows.append(row)
        used |= set(row)
    return rows


def routing_tensors(rows, device="cuda", seed=0):
    g = torch.Generator().manual_seed(seed)
    sel = torch.tensor(rows, dtype=torch.long)
    w = torch.rand(sel.shape, generator=g) + 0.1
    w = w / w.sum(1, keepdim=True)
    return sel.to(device), w.half().to(device)


def routings(B, NP, R, mode="recency", seed=0, device="cuda", topk=8):
    """R routings, each avoiding the previous call's experts (cold caches for weights between consecutive calls)"""
    rng = random.Random(seed * 100 + B)
    out, prev = [], ()
    for i in range(R):
        rows = make_sel(B, range(NP), mode, rng=rng, avoid=prev, topk=topk)
        prev = [e for r in rows for e in r]
        out.append(routing_tensors(rows, device=device, seed=i))
    return out


def softmax_topk(B, E, topk=8, seed=0, device="cuda"):
    """seeded router: logits ~ N(0,1) [B, E] -> softmax -> top-k ids (distinct per token) and fp16 weights"""
    g = torch.Generator().manual_seed(seed)
    p = torch.softmax(torch.randn(B, E, generator=g), -1)
    w, ids = torch.topk(p, topk, dim=-1)
    return ids.to(device), w.half().to(device)
