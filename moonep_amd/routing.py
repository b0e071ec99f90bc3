"""Synthetic top-k routing workloads for tests and benchmarks.

Everything is generated on the CPU from seeded ``torch.Generator``s so that
the same seed gives the same routing on every machine; callers move the
tensors to the GPU themselves.

Patterns follow the ones the reference exercises
(reference tests/generate_topk_routing.py:6-44 and
tests/kernel_test_utils.py:80-113): round-robin balanced, popularity-biased
sampling without replacement, all_local, all_remote, single_expert and
duplicate_topk; plus the logit model of the headline benchmark
(per-expert bias N(0, sigma) shared by all ranks added to N(0,1) logits,
top-k, softmax over the selected logits) with sigma bisected to a target
``maxvio = max_e T_e / mean_e T_e - 1`` (reference README.md:15,
benchmarks/bench_vs_deepep.py:83-113).
"""

from __future__ import annotations

import torch


def tokens_per_expert(topk: torch.Tensor, E: int) -> torch.Tensor:
    """[..., S, K] int expert ids -> [..., E] int32 counts."""
    lead = topk.shape[:-2]
    flat = topk.reshape(-1, topk.shape[-2] * topk.shape[-1]).long()
    out = torch.zeros(flat.shape[0], E, dtype=torch.int64)
    out.scatter_add_(1, flat, torch.ones_like(flat))
    return out.reshape(*lead, E).to(torch.int32)


def maxvio(tpe_RE: torch.Tensor) -> float:
    """Load-imbalance figure of the whole EP group."""
    tot = tpe_RE.reshape(-1, tpe_RE.shape[-1]).sum(0).double()
    return float(tot.max() / tot.mean() - 1.0)


def round_robin(S: int, K: int, E: int, R: int, rank: int, seed: int = 0) -> torch.Tensor:
    """Perfectly balanced routing: token s, choice k goes to rank (s+k)%R and
    to a permuted local expert ((s//R)+k)%epn."""
    epn = E // R
    g = torch.Generator().manual_seed(seed * 1000 + rank)
    s = torch.arange(S)[:, None]
    k = torch.arange(K)[None, :]
    perm = torch.randperm(epn, generator=g)
    return (((s + k) % R) * epn + perm[((s // R) + k) % epn]).to(torch.int32)


def popularity_biased(S: int, K: int, E: int, R: int, rank: int, sigma: float,
                      seed: int = 0) -> torch.Tensor:
    """exp(N(0, sigma)) expert popularity shared by all ranks, K draws without
    replacement per token from a per-rank stream."""
    if sigma == 0.0:
        return round_robin(S, K, E, R, rank, seed)
    gs = torch.Generator().manual_seed(seed)
    gl = torch.Generator().manual_seed(seed * 7919 + 1 + rank)
    pop = torch.exp(torch.normal(0.0, sigma, (E,), generator=gs))
    return torch.multinomial(pop[None, :].expand(S, E), K, replacement=False,
                             generator=gl).to(torch.int32)


def pattern(name: str, S: int, K: int, E: int, R: int, rank: int) -> torch.Tensor:
    """Deterministic corner-case routings."""
    epn = E // R
    s = torch.arange(S)[:, None]
    k = torch.arange(K)[None, :]
    if name == "all_local":
        t = rank * epn + ((s + k) % epn)
    elif name == "all_remote":
        t = ((rank + 1) % R) * epn + ((s + k) % epn)
    elif name == "single_expert":
        t = torch.zeros(S, K, dtype=torch.long)
    elif name == "duplicate_topk":
        t = torch.full((S, K), ((rank + 1) % R) * epn, dtype=torch.long)
    else:
        raise ValueError(f"unknown routing pattern: {name}")
    return t.to(torch.int32).contiguous()


def _logit_topk(S, K, E, R, sigma, seed, want_weights):
    g0 = torch.Generator().manual_seed(seed)
    bias = torch.normal(0.0, 1.0, (E,), generator=g0) * sigma
    topk, w = [], []
    for r in range(R):
        gr = torch.Generator().manual_seed(seed + 1 + r)
        logits = torch.randn(S, E, generator=gr) + bias
        v, i = torch.topk(logits, K, dim=1)
        topk.append(i.to(torch.int32))
        if want_weights:
            w.append(torch.softmax(v, dim=1))
    return torch.stack(topk), (torch.stack(w) if want_weights else None)


def logit_routing(S: int, K: int, E: int, R: int, target_maxvio: float, seed: int = 0,
                  tol: float = 0.03, want_weights: bool = True):
    """Routing of all R ranks at a target maxvio.

    Returns (topk[R,S,K] int32, weights[R,S,K] fp32 | None, tpe[R,E] int32,
    realised maxvio, sigma).  ``target_maxvio <= 0`` gives the round-robin
    closed form with uniform weights.
    """
    if target_maxvio <= 0.0:
        topk = torch.stack([round_robin(S, K, E, R, r, seed) for r in range(R)])
        w = torch.full((R, S, K), 1.0 / K) if want_weights else None
        tpe = tokens_per_expert(topk, E)
        return topk, w, tpe, maxvio(tpe), 0.0
    lo, hi = 0.0, 4.0
    while True:  # grow the bracket until it contains the target
        topk, _ = _logit_topk(S, K, E, R, hi, seed, False)
        if maxvio(tokens_per_expert(topk, E)) >= target_maxvio or hi > 64:
            break
        lo, hi = hi, hi * 2
    sigma = hi
    for _ in range(30):
        sigma = 0.5 * (lo + hi)
        topk, _ = _logit_topk(S, K, E, R, sigma, seed, False)
        mv = maxvio(tokens_per_expert(topk, E))
        if abs(mv - target_maxvio) <= tol * max(target_maxvio, 1e-9):
            break
        if mv < target_maxvio:
            lo = sigma
        else:
            hi = sigma
    topk, w = _logit_topk(S, K, E, R, sigma, seed, want_weights)
    tpe = tokens_per_expert(topk, E)
    return topk, w, tpe, maxvio(tpe), sigma
