"""CPU restatement of the MoonEP planner -- TEST INFRASTRUCTURE ONLY.

This module is a checker.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it; the product (moonep_amd) never
does and fails loudly when its HIP library is missing.

It restates, in plain numpy + short Python loops, the algorithm of the
reference's torch oracle ``launch_planning_torch_reference``
(reference tests/planning_reference.py:25-311), which is what the reference's
own device planner (reference moonep/planning.py:495-1101) is tested against.

Pinned by: tests/golden/planner_*.npz (vectors written by running the
reference oracle itself, tests/golden/make_planner_golden.py), an independent
C restatement (oracle/planner_oracle.c) cross-checked on random tiny inputs,
and closed-form cases (balanced round-robin, all_local, single_expert).

All arithmetic is int32-valued; numpy int64 is used for the intermediate
values, which never exceed 2**31 for supported shapes.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np


def align_up(x: int, a: int) -> int:
    return ((x + a - 1) // a) * a


def nvs_for(S: int, K: int, E: int, R: int, token_padding: int) -> int:
    """Dispatched slots per rank (reference moonep/api.py:265-279)."""
    epn = E // R
    return align_up(S * K + (token_padding - 1) * 2 * epn, token_padding)


@dataclass
class GlobalPlan:
    """Rank-independent planner tables ("Part 1" of the reference oracle)."""

    R: int
    E: int
    S: int
    K: int
    NvS: int
    token_padding: int
    tpe_cumsum: np.ndarray       # [R, E]  prefix over source ranks
    z: np.ndarray                # [R, R]  tokens home group h ships to dest d
    alloc: np.ndarray            # [E, R]  tokens of expert e landing on dest d
    alloc_cumsum: np.ndarray     # [E, R]
    expert_off: np.ndarray       # [R, E]  first slot of expert e on dest d
    cu_seqlens: np.ndarray       # [R, 2*epn]
    experts_to_copy: np.ndarray  # [R, epn]
    remote_stats: np.ndarray     # [R, 2]
    zero_fill: np.ndarray        # [R, 2*epn, 2]


def _first_argmax(a: np.ndarray) -> int:
    # numpy argmax/argmin return the first extremal index, like torch.argmax
    # on CPU and like the device kernel's "min index on ties" reductions
    # (reference moonep/planning.py:200-210).
    return int(np.argmax(a))


def _first_argmin(a: np.ndarray) -> int:
    return int(np.argmin(a))


def plan_global(tpe: np.ndarray, S: int, K: int, token_padding: int,
                NvS: int | None = None) -> GlobalPlan:
    """Balanced allocation + per-destination layout.

    Follows reference tests/planning_reference.py:56-204.
    ``tpe`` is [R, E]: tokens each source rank routes to each expert.
    """
    tpe = np.asarray(tpe, dtype=np.int64)
    R, E = tpe.shape
    assert E % R == 0
    epn = E // R
    CAP = S * K
    if NvS is None:
        NvS = nvs_for(S, K, E, R, token_padding)

    tpe_cumsum = np.cumsum(tpe, axis=0)                    # :60
    expert_count = tpe_cumsum[R - 1].copy()                # :61
    group_tokens = expert_count.reshape(R, epn).sum(axis=1)  # :63-65
    balance = group_tokens - CAP                           # :70

    alloc = np.zeros((E, R), dtype=np.int64)               # :77-79
    for e in range(E):
        alloc[e, e // epn] = expert_count[e]

    # Receivers and their quotas (:85-96).  Every chosen receiver is filled
    # to exactly CAP; the donor may overshoot and become a receiver later.
    z = np.zeros((R, R), dtype=np.int64)
    while True:
        h = _first_argmax(balance)
        u = _first_argmin(balance)
        if balance[h] <= 0:
            break
        move = -balance[u]
        z[h, u] = move            # assignment, not accumulation
        balance[h] -= move
        balance[u] = 0

    # Which tokens of which expert migrate (:100-121).  The device kernel
    # also stops when nothing remains (reference moonep/planning.py:728-729);
    # with consistent inputs that guard never fires.
    for h in range(R):
        es = h * epn
        remaining = expert_count[es:es + epn].copy()
        quotas = z[h].copy()
        while True:
            d = _first_argmax(quotas)
            quota = quotas[d]
            if quota <= 0:
                break
            le = _first_argmax(remaining)
            rem = remaining[le]
            if rem <= 0:
                break
            take = min(rem, quota)
            alloc[es + le, d] += take
            alloc[es + le, h] -= take
            remaining[le] -= take
            quotas[d] -= take

    assert np.array_equal(alloc.sum(axis=1), expert_count), "token conservation"
    assert not (alloc.sum(axis=0) > CAP).any(), "rank capacity exceeded"

    alloc_cumsum = np.cumsum(alloc, axis=1)                # :134
    expert_off = np.zeros((R, E), dtype=np.int64)
    cu_seqlens = np.zeros((R, 2 * epn), dtype=np.int64)
    experts_to_copy = np.full((R, epn), -1, dtype=np.int64)
    remote_stats = np.zeros((R, 2), dtype=np.int64)
    zero_fill = np.zeros((R, 2 * epn, 2), dtype=np.int64)

    for d in range(R):                                      # :148-204
        lo, hi = d * epn, (d + 1) * epn
        remote = [e for e in range(E) if alloc[e, d] > 0 and not (lo <= e < hi)]
        assert len(remote) <= epn, "remote experts exceed epn"
        remote_stats[d, 0] = len(remote)
        for b, e in enumerate(remote):
            experts_to_copy[d, b] = e
            remote_stats[e // epn, 1] += 1
        start = 0
        for g in range(2 * epn):
            cnt, eid = 0, -1
            if g < epn:
                eid = lo + g
                cnt = int(alloc[eid, d])
            elif experts_to_copy[d, g - epn] >= 0:
                eid = int(experts_to_copy[d, g - epn])
                cnt = int(alloc[eid, d])
            padded = align_up(cnt, token_padding) if cnt > 0 else 0
            cu_seqlens[d, g] = start + padded
            if cnt > 0:
                expert_off[d, eid] = start
                if padded > cnt:
                    zero_fill[d, g, 0] = start + cnt
                    zero_fill[d, g, 1] = padded - cnt
            start += padded
        assert cu_seqlens[d].max() <= NvS, "padded layout exceeds NvS"

    return GlobalPlan(R, E, S, K, NvS, token_padding, tpe_cumsum, z, alloc,
                      alloc_cumsum, expert_off, cu_seqlens, experts_to_copy,
                      remote_stats, zero_fill)


def raw_dst_for_rank(gp: GlobalPlan, topk_flat: np.ndarray, rank: int) -> np.ndarray:
    """Per-entry slot before duplicate canonicalisation ("Part 2").

    Follows reference tests/planning_reference.py:206-236: entries of one
    expert are numbered globally in (source rank, flat index) order and cut
    into the destinations' allocations in rank order.
    """
    topk_flat = np.asarray(topk_flat, dtype=np.int64).reshape(-1)
    N = topk_flat.size
    # local_cnt[i] = number of earlier flat entries of this rank with the
    # same expert (:207-212), computed with a stable sort instead of a loop.
    order = np.argsort(topk_flat, kind="stable")
    sorted_e = topk_flat[order]
    first = np.searchsorted(sorted_e, sorted_e, side="left")
    local_cnt = np.empty(N, dtype=np.int64)
    local_cnt[order] = np.arange(N) - first
    prev = np.zeros(gp.E, dtype=np.int64) if rank == 0 else gp.tpe_cumsum[rank - 1]
    g = prev[topk_flat] + local_cnt                          # :214-218
    ac = gp.alloc_cumsum[topk_flat]                          # [N, R]
    dest = (ac <= g[:, None]).sum(axis=1)                    # searchsorted right (:227)
    assert (dest < gp.R).all(), "no destination rank found"
    prev_alloc = np.where(dest > 0, ac[np.arange(N), np.maximum(dest - 1, 0)], 0)
    base = gp.expert_off[dest, topk_flat]
    return dest * gp.NvS + base + (g - prev_alloc)           # :231-236


def canonicalize_dst(raw: np.ndarray, K: int, NvS: int) -> np.ndarray:
    """Within each token keep the first entry per destination rank; later
    ones become ``-raw - 1`` (reference tests/planning_reference.py:262-294,
    device: moonep/planning.py:1051-1081)."""
    raw = np.asarray(raw, dtype=np.int64).reshape(-1, K)
    dest = raw // NvS
    out = raw.copy()
    for k in range(1, K):
        dup = (dest[:, :k] == dest[:, k:k + 1]).any(axis=1)
        out[dup, k] = -raw[dup, k] - 1
    return out.reshape(-1)


def decode_dst(dst: np.ndarray, NvS: int):
    """(raw, dest_rank, local_offset, is_primary) of encoded entries
    (reference moonep/dispatch.py:406-415)."""
    dst = np.asarray(dst, dtype=np.int64)
    raw = np.where(dst < 0, -dst - 1, dst)
    return raw, raw // NvS, raw % NvS, dst >= 0


def dedup_structs(dst_all: np.ndarray, rank: int, S: int, K: int, NvS: int):
    """Destination-side duplicate groups of ``rank`` from every source rank's
    (raw or canonical) dst, in the reference oracle's deterministic order
    (reference tests/planning_reference.py:251-289): source rank major, token
    minor, destination in order of first appearance.

    Returns (dup_groups[NvS,3], dup_loffs[NvS], dup_counts[2]).
    """
    dst_all = np.asarray(dst_all, dtype=np.int64)
    R = dst_all.shape[0]
    raw, drank, loff, _ = decode_dst(dst_all.reshape(R, S, K), NvS)
    dup_groups = np.zeros((NvS, 3), dtype=np.int64)
    dup_loffs = np.zeros(NvS, dtype=np.int64)
    ng = nd = 0
    for src in range(R):
        mine = drank[src] == rank                     # [S, K]
        toks = np.nonzero(mine.sum(axis=1) > 1)[0]
        for s in toks:
            ks = np.nonzero(mine[s])[0]
            lo = loff[src, s, ks]
            dup_groups[ng] = (lo[0], nd, len(ks) - 1)
            dup_loffs[nd:nd + len(ks) - 1] = lo[1:]
            ng += 1
            nd += len(ks) - 1
    return dup_groups, dup_loffs, np.array([ng, nd], dtype=np.int64)


@dataclass
class RankPlan:
    dst: np.ndarray              # [N]  canonical (negative = duplicate)
    cu_seqlens: np.ndarray       # [2*epn]
    experts_to_copy: np.ndarray  # [R, epn]
    remote_stats: np.ndarray     # [2]
    zero_fill_ranges: np.ndarray  # [2*epn, 2]


def plan_rank(gp: GlobalPlan, topk_flat: np.ndarray, rank: int) -> RankPlan:
    """What the reference planner returns on ``rank`` (as int32)."""
    raw = raw_dst_for_rank(gp, topk_flat, rank)
    dst = canonicalize_dst(raw, gp.K, gp.NvS)
    i32 = np.int32
    return RankPlan(dst.astype(i32), gp.cu_seqlens[rank].astype(i32),
                    gp.experts_to_copy.astype(i32), gp.remote_stats[rank].astype(i32),
                    gp.zero_fill[rank].astype(i32))


def plan(topk_all: np.ndarray, tpe: np.ndarray, rank: int, token_padding: int,
         NvS: int | None = None) -> RankPlan:
    """Convenience: topk_all is [R,S,K] (or [S,K] for this rank), tpe [R,E]."""
    topk_all = np.asarray(topk_all)
    tpe = np.asarray(tpe)
    R, E = tpe.shape
    if topk_all.ndim == 3:
        _, S, K = topk_all.shape
        mine = topk_all[rank]
    else:
        S, K = topk_all.shape
        mine = topk_all
    gp = plan_global(tpe, S, K, token_padding, NvS)
    return plan_rank(gp, mine.reshape(-1), rank)


def invariant_errors(gp: GlobalPlan, dst_all: np.ndarray, topk_all: np.ndarray) -> list[str]:
    """Structural checks in the spirit of reference
    tests/kernel_test_utils.py:324-414, plus the bijection property: over all
    ranks, decoded dst hits every real slot of every destination exactly once
    and inside the segment of its expert."""
    errs: list[str] = []
    R, E, S, K, NvS, tp = gp.R, gp.E, gp.S, gp.K, gp.NvS, gp.token_padding
    epn = E // R
    raw, drank, loff, _ = decode_dst(np.asarray(dst_all).reshape(R, S * K), NvS)
    if ((drank < 0) | (drank >= R)).any():
        errs.append("dst dest rank out of range")
        return errs
    for d in range(R):
        prev = 0
        for g, cur in enumerate(gp.cu_seqlens[d]):
            seg = cur - prev
            if seg < 0:
                errs.append(f"cu_seqlens[{d}] decreases at {g}")
            if seg and seg % tp:
                errs.append(f"cu_seqlens[{d}] segment {g} not padded")
            prev = cur
        if gp.cu_seqlens[d, -1] > NvS:
            errs.append(f"cu_seqlens[{d}] exceeds NvS")
        etc = gp.experts_to_copy[d]
        if not (((etc == -1) | ((etc >= 0) & (etc < E))).all()):
            errs.append("experts_to_copy invalid id")
    topk_all = np.asarray(topk_all).reshape(R, S * K)
    seen = np.zeros((R, NvS), dtype=np.int64)
    np.add.at(seen, (drank.reshape(-1), loff.reshape(-1)), 1)
    if (seen > 1).any():
        errs.append("two entries share one slot")
    if int(seen.sum()) != R * S * K:
        errs.append("slot count mismatch")
    # every entry inside its expert's segment on the destination
    start = gp.expert_off[drank, topk_all]
    cnt = gp.alloc[topk_all, drank]
    if ((loff < start) | (loff >= start + cnt)).any():
        errs.append("entry outside its expert segment")
    if not (seen.sum(axis=1) == S * K).all():
        errs.append("a rank does not receive exactly S*K tokens")
    return errs
