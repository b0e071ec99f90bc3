"""Pins the CPU planner oracles (no GPU).

1. Both restatements (numpy: oracle/planner_oracle.py, C: oracle/mep_oracle.c)
   against the vectors written by the reference's own oracle
   (tests/golden/planner_golden.npz, made by tests/golden/make_planner_golden.py).
2. Against each other on many random tiny inputs (ties are frequent there).
3. Against closed forms and invariants that follow from the mathematics.
"""

import numpy as np
import pytest
import torch

from moonep_amd import routing
from oracle import c_oracle as co
from oracle import planner_oracle as po
from tests.util import golden_case, golden_names, oracle_world_plan

FIELDS = ("dst", "cu_seqlens", "experts_to_copy", "zero_fill_ranges", "remote_stats")


@pytest.mark.parametrize("name", golden_names())
def test_numpy_oracle_matches_reference_vectors(golden, name):
    g = golden_case(golden, name)
    gp = po.plan_global(g["tpe"], g["S"], g["K"], g["tp"], g["NvS"])
    assert np.array_equal(gp.alloc.T, g["alloc_RE"])
    dst_all = []
    for r in range(g["R"]):
        rp = po.plan_rank(gp, g["topk"][r].reshape(-1), r)
        for f in FIELDS:
            assert np.array_equal(getattr(rp, f), g[f][r]), (name, r, f)
        dst_all.append(rp.dst)
    dst_all = np.stack(dst_all)
    for r in range(g["R"]):
        dg, dl, dc = po.dedup_structs(dst_all, r, g["S"], g["K"], g["NvS"])
        ng, nd = (int(v) for v in dc)
        assert [ng, nd] == g["dup_counts"][r].tolist()
        assert np.array_equal(dg[:ng], g["dup_groups"][r][:ng])
        assert np.array_equal(dl[:nd], g["dup_loffs"][r][:nd])
    assert not po.invariant_errors(gp, dst_all, g["topk"])


@pytest.mark.parametrize("name", golden_names())
def test_c_oracle_matches_reference_vectors(golden, name):
    g = golden_case(golden, name)
    for r in range(g["R"]):
        out = co.plan(g["tpe"], g["topk"][r], r, g["S"], g["K"], g["tp"], g["NvS"])
        for f, got in zip(FIELDS, out):
            assert np.array_equal(got, g[f][r]), (name, r, f)


def test_two_restatements_agree_on_random_tiny_inputs():
    rng = np.random.default_rng(2025)
    for trial in range(400):
        R = int(rng.integers(1, 6))
        epn = int(rng.integers(1, 6))
        S = int(rng.integers(1, 33))
        K = int(rng.integers(1, 5))
        tp = int(rng.choice([1, 2, 4, 8, 16]))
        E = R * epn
        # few distinct experts in use -> equal counts and equal balances are common
        used = rng.choice(E, size=int(rng.integers(1, E + 1)), replace=False)
        topk = rng.choice(used, size=(R, S, K)).astype(np.int32)
        tpe = routing.tokens_per_expert(torch.from_numpy(topk), E).numpy()
        NvS = po.nvs_for(S, K, E, R, tp)
        gp = po.plan_global(tpe, S, K, tp)
        dst_all = []
        for r in range(R):
            rp = po.plan_rank(gp, topk[r].reshape(-1), r)
            got = co.plan(tpe, topk[r], r, S, K, tp, NvS)
            for f, g in zip(FIELDS, got):
                assert np.array_equal(getattr(rp, f), g), (trial, r, f)
            dst_all.append(rp.dst)
        assert not po.invariant_errors(gp, np.stack(dst_all), topk), trial


def test_balanced_round_robin_closed_form():
    """Every home group receives exactly S*K tokens: nothing migrates, every
    token sits in its home rank, in (source rank, flat order) inside the
    padded segment of its expert."""
    S, K, E, R, tp = 64, 4, 32, 8, 16
    epn = E // R
    topk = torch.stack([routing.round_robin(S, K, E, R, r, seed=3) for r in range(R)]).numpy()
    tpe = routing.tokens_per_expert(torch.from_numpy(topk), E).numpy()
    gp, plans, dst_all = oracle_world_plan(topk, tpe, tp)
    assert (gp.z == 0).all()
    assert (gp.experts_to_copy == -1).all() and (gp.remote_stats == 0).all()
    cnt = tpe.sum(0)
    assert np.array_equal(gp.alloc[np.arange(E), np.arange(E) // epn], cnt)
    padded = (cnt + tp - 1) // tp * tp
    for d in range(R):
        ends = np.cumsum(padded[d * epn:(d + 1) * epn])
        assert np.array_equal(gp.cu_seqlens[d, :epn], ends)
        assert (gp.cu_seqlens[d, epn:] == ends[-1]).all()
    # slot of entry i of rank r = home*NvS + segment start + entries of the
    # same expert from earlier ranks + earlier entries of this rank
    NvS = gp.NvS
    starts = np.cumsum(padded.reshape(R, epn), axis=1) - padded.reshape(R, epn)
    before = np.cumsum(tpe, axis=0) - tpe
    for r in range(R):
        flat = topk[r].reshape(-1)
        seen = np.zeros(E, dtype=np.int64)
        raw, _, _, _ = po.decode_dst(plans[r].dst, NvS)
        for i, e in enumerate(flat):
            want = (e // epn) * NvS + starts[e // epn, e % epn] + before[r, e] + seen[e]
            assert raw[i] == want
            seen[e] += 1


def test_all_local_and_single_expert_closed_forms():
    S, K, R, epn, tp = 32, 4, 4, 8, 16
    E = R * epn
    topk = torch.stack([routing.pattern("all_local", S, K, E, R, r) for r in range(R)]).numpy()
    tpe = routing.tokens_per_expert(torch.from_numpy(topk), E).numpy()
    gp, plans, dst_all = oracle_world_plan(topk, tpe, tp)
    for r in range(R):
        _, drank, _, prim = po.decode_dst(plans[r].dst, gp.NvS)
        assert (drank == r).all()
        # all K copies of a token sit on one rank: only k = 0 is a primary
        assert prim.reshape(S, K)[:, 0].all() and not prim.reshape(S, K)[:, 1:].any()
    # single expert: R*S*K tokens of expert 0 are cut into R consecutive
    # chunks of S*K in (rank, flat) order; rank d hosts chunk d
    S, K, R, epn, tp = 9, 2, 4, 4, 8
    E = R * epn
    topk = torch.stack([routing.pattern("single_expert", S, K, E, R, r) for r in range(R)]).numpy()
    tpe = routing.tokens_per_expert(torch.from_numpy(topk), E).numpy()
    gp, plans, dst_all = oracle_world_plan(topk, tpe, tp)
    N = S * K
    assert (gp.alloc[0] == N).all() and gp.alloc[1:].sum() == 0
    for r in range(R):
        raw, drank, loff, _ = po.decode_dst(plans[r].dst, gp.NvS)
        assert (drank == r).all()
        # rank 0 hosts expert 0 as local group 0, the others as their first remote slot
        assert np.array_equal(loff, np.arange(N))
        want_etc = -np.ones(epn, dtype=np.int64)
        if r > 0:
            want_etc[0] = 0
        assert np.array_equal(gp.experts_to_copy[r], want_etc)
        pad = (N + tp - 1) // tp * tp - N
        g = 0 if r == 0 else epn
        assert gp.zero_fill[r, g].tolist() == ([N, pad] if pad else [0, 0])
    assert gp.remote_stats[0].tolist() == [0, R - 1]


def test_every_rank_receives_exactly_its_capacity():
    for seed, sigma in ((1, 0.5), (2, 2.0), (3, 5.0)):
        S, K, E, R, tp = 128, 8, 64, 8, 32
        topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed) for r in range(R)])
        tpe = routing.tokens_per_expert(topk, E).numpy()
        gp, plans, dst_all = oracle_world_plan(topk.numpy(), tpe, tp)
        assert (gp.alloc.sum(0) == S * K).all()
        assert np.array_equal(gp.alloc.sum(1), tpe.sum(0))
        assert not po.invariant_errors(gp, dst_all, topk.numpy())
        # a rank hosts experts of at most one foreign home group
        for d in range(R):
            etc = gp.experts_to_copy[d]
            homes = {int(e) // (E // R) for e in etc if e >= 0}
            assert len(homes) <= 1
