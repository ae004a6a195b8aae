"""Synthetic routing for tests and benches (reference sm120/routing.py:4-20, sm120/common.py:3-8).

'distinct': no expert shared between tokens (worst case, 8 B runs). 'recency': token t reuses each of token t-1's
experts with probability p. `routings` makes consecutive calls avoid the previous call's experts so weights are cold.
`softmax_topk` is the seeded router of the full-layer configuration: softmax over N(0,1) logits, top-k, fp16 weights."""
import random

import torch


def make_sel(B, pool, mode="recency", p=0.4, rng=None, avoid=(), topk=8):
    """B rows of topk distinct expert ids drawn from `pool` minus `avoid`. 'recency': a token keeps each id of the token before it
    with probability p and fills up with fresh ones; 'distinct': no id serves two tokens; anything else: rows independent."""
    rng = rng or random.Random(0)
    banned = set(avoid)
    allowed = [e for e in pool if e not in banned]
    rows, taken = [], set()
    for t in range(B):
        kept = [e for e in rows[t - 1] if rng.random() < p] if (t > 0 and mode == "recency") else []
        blocked = set(kept) | (taken if mode == "distinct" else set())
        fresh = [e for e in allowed if e not in blocked]
        rng.shuffle(fresh)
        row = kept + fresh[: topk - len(kept)]
        rng.shuffle(row)
        taken.update(row)
        rows.append(row)
    return rows


def routing_tensors(rows, device="cuda", seed=0):
    """(sel int64 [B, topk], rw fp16 [B, topk]) for id rows: weights uniform in [0.1, 1.1), normalised per token"""
    sel = torch.as_tensor(rows, dtype=torch.int64)
    raw = 0.1 + torch.rand(sel.shape, generator=torch.Generator().manual_seed(seed))
    rw = raw / raw.sum(dim=1, keepdim=True)
    return sel.to(device), rw.to(torch.float16).to(device)


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
