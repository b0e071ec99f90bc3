"""Writes tests/golden/planner_golden.npz: input/output vectors of the
reference's own planner oracle.

Run once, in the build container, where the reference checkout is mounted:

    python tests/golden/make_planner_golden.py [/root/reference]

It loads the reference's pure-torch CPU oracle
(reference tests/planning_reference.py:25-311) straight from its file and
calls it for every emulated rank of every case below.  The oracle calls
``torch.distributed.all_gather`` to see every rank's dst when it derives the
duplicate groups; with no process group that collective is replaced here by a
two-pass capture/replay (pass 1 records the dst each rank hands to the
collective, pass 2 serves the recorded tensors).  Nothing from the reference
is stored: the .npz holds inputs (topk, tpe, shape scalars) and the oracle's
outputs only.

Why these vectors exist: invariants and closed forms fix most of the planner,
but not which of several equally good greedy choices the reference makes
(first index on ties, assignment into z, donors that overshoot and become
receivers).  The cases below are built to hit exactly those choices.
"""

from __future__ import annotations

import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from moonep_amd import routing  # noqa: E402


def _load_reference(root: str):
    path = os.path.join(root, "tests", "planning_reference.py")
    spec = importlib.util.spec_from_file_location("_ref_planning_reference", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _align_up(x, a):
    return (x + a - 1) // a * a


def topk_from_counts(counts: np.ndarray, S: int, K: int, seed: int) -> torch.Tensor:
    """[R,E] per-rank expert counts (rows sum to S*K) -> shuffled topk[R,S,K]."""
    R, E = counts.shape
    g = torch.Generator().manual_seed(seed)
    out = []
    for r in range(R):
        assert counts[r].sum() == S * K, (counts[r].sum(), S * K)
        flat = torch.repeat_interleave(torch.arange(E), torch.as_tensor(counts[r]))
        flat = flat[torch.randperm(S * K, generator=g)]
        out.append(flat.reshape(S, K).to(torch.int32))
    return torch.stack(out)


def spread(total: int, weights) -> np.ndarray:
    """Integer split of ``total`` proportional to ``weights`` (largest first
    gets the remainder) -- used to build count matrices by hand."""
    w = np.asarray(weights, dtype=np.float64)
    base = np.floor(total * w / w.sum()).astype(np.int64)
    base[np.argmax(w)] += total - base.sum()
    return base


def cases():
    """Yield (name, topk[R,S,K] int32, token_padding)."""
    P = routing.popularity_biased
    RR = routing.round_robin
    PT = routing.pattern

    def stack(fn, R, *a, **kw):
        return torch.stack([fn(*a, rank=r, **kw) for r in range(R)])

    # --- shapes of the reference's planner case table (smaller S where the
    # oracle's Python loops would take minutes) -------------------------------
    yield "balanced_epn16_R8", stack(RR, 8, 256, 8, 128, 8, seed=42), 128
    yield "tiny_s1_k1_R1", stack(RR, 1, 1, 1, 1, 1, seed=42), 8
    yield "tiny_s1_k1_R4", stack(RR, 4, 1, 1, 4, 4, seed=42), 8
    yield "tiny_biased_prefetch_R2", stack(P, 2, 3, 5, 6, 2, sigma=1.0, seed=9002), 32
    yield "tiny_biased_prefetch_R8", stack(P, 8, 3, 5, 24, 8, sigma=1.0, seed=9002), 32
    yield "no_padding_R4", stack(P, 4, 33, 2, 8, 4, sigma=1.0, seed=10001), 1
    yield "non_power_mild_bias_R4", stack(P, 4, 17, 3, 12, 4, sigma=0.5, seed=10501), 16
    yield "small_balanced_R8", stack(RR, 8, 17, 3, 24, 8, seed=11001), 16
    yield "near_degenerate_bias_R8", stack(P, 8, 64, 2, 40, 8, sigma=5.0, seed=12001), 128
    yield "typical_bias_R8", stack(P, 8, 32, 4, 32, 8, sigma=1.0, seed=13001), 64
    yield "heavy_bias_R4", stack(P, 4, 96, 3, 28, 4, sigma=2.0, seed=14001), 128
    yield "wide_epn256_R8", stack(RR, 8, 256, 1, 2048, 8, seed=42), 1
    yield "wide_epn320_R4", stack(P, 4, 512, 1, 1280, 4, sigma=1.0, seed=7), 1
    yield "experts_gt_block_R2", stack(P, 2, 256, 1, 2050, 2, sigma=0.5, seed=3), 1
    yield "all_local_R4", stack(PT, 4, "all_local", 32, 4, 32, 4), 16
    yield "all_remote_R4", stack(PT, 4, "all_remote", 32, 4, 32, 4), 16
    yield "duplicate_topk_R4", stack(PT, 4, "duplicate_topk", 16, 4, 16, 4), 8
    yield "single_expert_exact_R4", stack(PT, 4, "single_expert", 8, 2, 16, 4), 8
    yield "single_expert_tail_R8", stack(PT, 8, "single_expert", 9, 2, 32, 8), 8
    # --- medium, production-like mix ----------------------------------------
    yield "medium_bias1_R8", stack(P, 8, 256, 8, 256, 8, sigma=1.0, seed=2024), 128
    yield "medium_bias2_R8", stack(P, 8, 128, 8, 128, 8, sigma=2.0, seed=2025), 128

    # --- hand-built count matrices: ties and overshoot -----------------------
    # R=4, epn=2, S*K = 40 per rank (S=20,K=2).  Group totals are set through
    # per-rank counts; every rank uses the same row so totals = 4*row.
    def same_rows(row, R):
        return np.tile(np.asarray(row, dtype=np.int64), (R, 1))

    # two equal donors, two equal (empty) receivers
    row = [11, 9, 10, 10, 0, 0, 0, 0]                    # groups 20,20,0,0 (sum 40)
    yield "tie_equal_surplus_R4", topk_from_counts(same_rows(row, 4), 20, 2, 1), 8
    # balances (+5,+20,-15,-10) scaled: CAP=40 -> totals 45,60,25,30
    counts = np.zeros((4, 8), dtype=np.int64)
    totals = [45, 60, 25, 30]
    # split every group's total over its 2 experts and over the 4 source ranks
    per_rank = np.zeros((4, 8), dtype=np.int64)
    cells = []
    for gidx, t in enumerate(totals):
        a = t // 2
        cells += [a, t - a]
    cells = np.asarray(cells)
    # distribute each expert's total across ranks so that every rank sums to 40
    remaining_rank = np.full(4, 40)
    for e in np.argsort(-cells):
        left = cells[e]
        for r in np.argsort(-remaining_rank):
            take = min(left, remaining_rank[r], (cells[e] + 3) // 4 + 1)
            per_rank[r, e] += take
            remaining_rank[r] -= take
            left -= take
        # dump what is left on whoever still has room
        for r in range(4):
            take = min(left, remaining_rank[r])
            per_rank[r, e] += take
            remaining_rank[r] -= take
            left -= take
        assert left == 0
    assert (per_rank.sum(1) == 40).all() and (per_rank.sum(0) == cells).all()
    yield "overshoot_donor_becomes_receiver_R4", topk_from_counts(per_rank, 20, 2, 2), 4
    # equal remaining among a home's experts + quota spanning several experts;
    # dest 1 receives both experts of home 0 (remote count == epn)
    row = [10, 10, 0, 0]                                  # R=2, epn=2, S*K=20
    yield "tie_equal_remaining_remote_eq_epn_R2", topk_from_counts(same_rows(row, 2), 10, 2, 3), 4
    # counts that are exact multiples of the padding (no zero-fill) and empty experts
    row = [8, 0, 8, 0, 8, 0, 8, 0]                        # R=4, epn=2, S*K=32
    yield "exact_multiple_no_pad_R4", topk_from_counts(same_rows(row, 4), 16, 2, 4), 8
    # three-way tie of donors and receivers, R=6, epn=1
    row = [10, 10, 10, 2, 2, 2]                           # S*K = 36
    yield "three_way_ties_R6", topk_from_counts(same_rows(row, 6), 12, 3, 5), 4
    # one giant donor feeding everyone (R=8, epn=3)
    row = [20, 20, 20] + [0] * 21                         # S*K=60
    yield "one_donor_R8", topk_from_counts(same_rows(row, 8), 20, 3, 6), 16

    # --- random tie-heavy matrices -------------------------------------------
    rng = np.random.default_rng(12345)
    for i, (R, epn, S, K, tp) in enumerate([
        (2, 1, 6, 2, 4), (3, 2, 8, 3, 4), (4, 3, 12, 2, 8), (5, 2, 10, 4, 1),
        (8, 2, 16, 4, 16), (4, 5, 25, 2, 8), (8, 4, 32, 2, 32), (3, 4, 9, 4, 2),
        (7, 3, 21, 3, 8), (8, 1, 8, 8, 4),
    ]):
        E = R * epn
        N = S * K
        # few distinct cell values -> many equal group totals / remainders
        w = rng.choice([0, 1, 1, 2, 4], size=E).astype(np.float64) + 1e-9
        rows = []
        for r in range(R):
            rows.append(spread(N, np.roll(w, r % 2)))
        yield f"random_ties_{i}_R{R}", topk_from_counts(np.stack(rows), S, K, 100 + i), tp


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = _load_reference(root)
    import torch.distributed as dist

    store = {}
    names = []
    for name, topk, tp in cases():
        R, S, K = topk.shape
        # the highest expert ids may be unused, so E comes from the table below
        E = CASE_E[name]
        epn = E // R
        tpe = routing.tokens_per_expert(topk, E)
        NvS = _align_up(S * K + (tp - 1) * 2 * epn, tp)
        ctx = {"R": R, "E": E, "S": S, "K": K, "NvS_capacity": S * K, "NvS": NvS,
               "token_padding": tp, "group": None}

        captured = {}
        state = {"pass": 1, "rank": 0}

        class _Captured(Exception):
            pass

        def fake_all_gather(gathered, t, group=None):
            if state["pass"] == 1:
                captured[state["rank"]] = t.clone()
                raise _Captured()   # pass 1 only wants the raw dst
            else:
                for r in range(R):
                    gathered[r].copy_(captured[r])

        real = dist.all_gather
        dist.all_gather = fake_all_gather
        try:
            results = []
            for p in (1, 2):
                state["pass"] = p
                results = []
                for r in range(R):
                    state["rank"] = r
                    c = dict(ctx, rank=r)
                    try:
                        results.append(ref.launch_planning_torch_reference(c, topk, tpe))
                    except _Captured:
                        pass
                if R == 1:
                    break
        finally:
            dist.all_gather = real

        dst = np.stack([x[0].numpy() for x in results]).astype(np.int32)
        cu = np.stack([x[1].numpy() for x in results]).astype(np.int32)
        etc = np.stack([x[2].numpy() for x in results]).astype(np.int32)
        stats = np.stack([x[3].numpy() for x in results]).astype(np.int32)
        zfr = np.stack([x[4].numpy() for x in results]).astype(np.int32)
        dcount = np.stack([x[5].dup_counts.numpy() for x in results]).astype(np.int32)
        gmax = max(1, int(dcount[:, 0].max()))
        lmax = max(1, int(dcount[:, 1].max()))
        dgroups = np.stack([x[5].dup_groups.numpy()[:gmax] for x in results]).astype(np.int32)
        dloffs = np.stack([x[5].dup_loffs.numpy()[:lmax] for x in results]).astype(np.int32)
        ctx0 = dict(ctx, rank=0)
        alloc = ref.launch_planning_torch_reference(ctx0, topk, tpe, return_alloc=True)
        store[f"{name}/shape"] = np.array([R, S, K, E, tp, NvS], dtype=np.int64)
        store[f"{name}/topk"] = topk.numpy().astype(np.int32)
        store[f"{name}/tpe"] = tpe.numpy().astype(np.int32)
        store[f"{name}/dst"] = dst
        store[f"{name}/cu_seqlens"] = cu
        store[f"{name}/experts_to_copy"] = etc
        store[f"{name}/remote_stats"] = stats
        store[f"{name}/zero_fill_ranges"] = zfr
        store[f"{name}/dup_counts"] = dcount
        store[f"{name}/dup_groups"] = dgroups
        store[f"{name}/dup_loffs"] = dloffs
        store[f"{name}/alloc_RE"] = alloc.numpy().astype(np.int32)
        names.append(name)
        print(f"{name}: R={R} S={S} K={K} E={E} tp={tp} NvS={NvS} "
              f"remote={stats[:, 0].tolist()} dups={dcount[:, 1].tolist()}", flush=True)
    store["names"] = np.array(names)
    out = os.path.join(HERE, "planner_golden.npz")
    np.savez_compressed(out, **store)
    print("wrote", out, os.path.getsize(out), "bytes")


# true expert counts for cases whose highest expert ids may be unused
CASE_E = {
    "balanced_epn16_R8": 128, "tiny_s1_k1_R1": 1, "tiny_s1_k1_R4": 4,
    "tiny_biased_prefetch_R2": 6, "tiny_biased_prefetch_R8": 24, "no_padding_R4": 8,
    "non_power_mild_bias_R4": 12, "small_balanced_R8": 24, "near_degenerate_bias_R8": 40,
    "typical_bias_R8": 32, "heavy_bias_R4": 28, "wide_epn256_R8": 2048,
    "wide_epn320_R4": 1280, "experts_gt_block_R2": 2050, "all_local_R4": 32,
    "all_remote_R4": 32, "duplicate_topk_R4": 16, "single_expert_exact_R4": 16,
    "single_expert_tail_R8": 32, "medium_bias1_R8": 256, "medium_bias2_R8": 128,
    "tie_equal_surplus_R4": 8, "overshoot_donor_becomes_receiver_R4": 8,
    "tie_equal_remaining_remote_eq_epn_R2": 4, "exact_multiple_no_pad_R4": 8,
    "three_way_ties_R6": 6, "one_donor_R8": 24,
    "random_ties_0_R2": 2, "random_ties_1_R3": 6, "random_ties_2_R4": 12,
    "random_ties_3_R5": 10, "random_ties_4_R8": 16, "random_ties_5_R4": 20,
    "random_ties_6_R8": 32, "random_ties_7_R3": 12, "random_ties_8_R7": 21,
    "random_ties_9_R8": 8,
}


if __name__ == "__main__":
    main()
