"""HIP planner vs the reference oracle's golden vectors and vs the CPU oracle
at the headline shapes.  Everything is bit-exact (integer work)."""

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, routing
from moonep_amd.dispatch import launch_build_dedup
from moonep_amd.planning import (allocate_planning_outputs, launch_planning,
                                 launch_planning_all_ranks)
from oracle import planner_oracle as po
from tests.util import golden_case, golden_names, oracle_world_plan

pytestmark = pytest.mark.gpu


def _check_rank(plan, cu, ref, r, name):
    for field, got in (("dst", plan.dst), ("cu_seqlens", cu),
                       ("experts_to_copy", plan.experts_to_copy),
                       ("remote_stats", plan.remote_stats),
                       ("zero_fill_ranges", plan.zero_fill_ranges)):
        want = ref[field][r] if field != "experts_to_copy" else ref[field][r]
        got = got.cpu().numpy()
        assert np.array_equal(got, want), f"{name} rank {r}: {field} differs"


@pytest.mark.parametrize("name", golden_names())
def test_planner_matches_reference_golden(cuda, golden, name):
    g = golden_case(golden, name)
    R, S, K, E, tp = g["R"], g["S"], g["K"], g["E"], g["tp"]
    topk = torch.from_numpy(g["topk"]).to(cuda)
    tpe = torch.from_numpy(g["tpe"]).to(cuda)
    print(f"case {name} R={R} S={S} K={K} E={E} tp={tp}", flush=True)
    dst_all = None
    for r in range(R):
        buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=r)
        ctx = buf._require_ctx()
        assert ctx["NvS"] == g["NvS"]
        plan, cu = allocate_planning_outputs(ctx)
        assert launch_planning(ctx, topk[r].reshape(-1).contiguous(), tpe, cu, plan) is None
        torch.cuda.synchronize()
        _check_rank(plan, cu, g, r, name)
        if r == 0:
            dst_all, cu_all, etc, zfr, stats = launch_planning_all_ranks(ctx, topk, tpe)
            torch.cuda.synchronize()
            assert np.array_equal(dst_all.cpu().numpy(), g["dst"])
            assert np.array_equal(cu_all.cpu().numpy(), g["cu_seqlens"])
            assert np.array_equal(etc.cpu().numpy(), g["experts_to_copy"][0])
            assert np.array_equal(zfr.cpu().numpy(), g["zero_fill_ranges"])
            assert np.array_equal(stats.cpu().numpy(), g["remote_stats"])
        # duplicate groups of this rank, deterministic (source rank, token) order
        launch_build_dedup(ctx, dst_all, plan)
        torch.cuda.synchronize()
        ng, nd = (int(v) for v in plan.dup_counts.cpu())
        assert [ng, nd] == g["dup_counts"][r].tolist()
        assert np.array_equal(plan.dup_groups.cpu().numpy()[:ng], g["dup_groups"][r][:ng])
        assert np.array_equal(plan.dup_loffs.cpu().numpy()[:nd], g["dup_loffs"][r][:nd])
        buf.destroy()


@pytest.mark.parametrize("S,H,K,E,R,mv", [
    (4096, 7168, 8, 256, 8, 1.0),
    (4096, 7168, 8, 256, 8, 0.0),
    (4096, 7168, 8, 256, 8, 4.0),
    (8192, 4096, 8, 128, 8, 2.0),
    (8192, 7168, 8, 384, 8, 1.0),   # the configuration of the reference's own figure (48 experts per rank)
])
def test_planner_matches_oracle_at_headline_shapes(cuda, S, H, K, E, R, mv):
    topk, _, tpe, real_mv, _ = routing.logit_routing(S, K, E, R, mv, seed=1234, want_weights=False)
    print(f"S={S} E={E} target maxvio={mv} realised={real_mv:.3f}", flush=True)
    gp, plans, dst_all_ref = oracle_world_plan(topk.numpy(), tpe.numpy(), 128)
    assert not po.invariant_errors(gp, dst_all_ref, topk.numpy())
    buf = Buffer(S, 16, K, E, R, token_padding=128, rank=0)  # H is irrelevant to the planner
    ctx = buf._require_ctx()
    dst_all, cu, etc, zfr, stats = launch_planning_all_ranks(ctx, topk.to(cuda), tpe.to(cuda))
    torch.cuda.synchronize()
    assert np.array_equal(dst_all.cpu().numpy(), dst_all_ref)
    assert np.array_equal(cu.cpu().numpy(), gp.cu_seqlens)
    assert np.array_equal(etc.cpu().numpy(), gp.experts_to_copy)
    assert np.array_equal(zfr.cpu().numpy(), gp.zero_fill)
    assert np.array_equal(stats.cpu().numpy(), gp.remote_stats)
    # single-rank entry point on a rank in the middle
    buf3 = Buffer(S, 16, K, E, R, token_padding=128, rank=3)
    plan, cu3 = allocate_planning_outputs(buf3._require_ctx())
    launch_planning(buf3._require_ctx(), topk[3].reshape(-1).to(cuda), tpe.to(cuda), cu3, plan)
    torch.cuda.synchronize()
    assert np.array_equal(plan.dst.cpu().numpy(), plans[3].dst)
    assert np.array_equal(cu3.cpu().numpy(), plans[3].cu_seqlens)
    assert np.array_equal(plan.remote_stats.cpu().numpy(), plans[3].remote_stats)
    buf.destroy()
    buf3.destroy()


@pytest.mark.parametrize("R,epn,S,K,tp,sigma", [
    (16, 4, 64, 4, 16, 1.0),      # one DPP row of balances
    (24, 3, 48, 6, 8, 2.0),       # full-wave reductions
    (70, 2, 35, 4, 4, 1.5),       # ranks beyond lane 63
    (128, 1, 64, 2, 8, 1.0),      # the encoding's rank limit
    (12, 70, 96, 5, 32, 1.0),     # more than 64 experts per rank
    (8, 8, 262144, 8, 128, 1.0),  # counts too large for packed (value, index) keys
    (8, 512, 512, 4, 16, 1.0),    # E = 4096: per-expert arrays beyond 64 KB of LDS
    (8, 726, 600, 4, 16, 1.0),    # E = 5808: exactly the 160 KB of LDS a workgroup can have (5816 is refused)
    # several workgroups per rank whose slices start off 16-byte boundaries (the count of
    # earlier or later entries then has a scalar head and tail), ranks whose rows start
    # unaligned (S*K odd), the compile-time R=8/K=8 kernel beside the generic one
    (4, 4, 1501, 3, 8, 1.0),      # 1023 entries per workgroup, odd S*K
    (8, 4, 1203, 7, 16, 1.5),     # 1022 entries per workgroup, R=8 without K=8
    (8, 8, 2100, 8, 32, 1.0),     # R=8 and K=8, 17 workgroups, the last one partial
    (4, 8, 3000, 8, 64, 2.0),     # the compile-time R=4/K=8 kernel
    (16, 4, 1100, 8, 16, 1.0),    # the compile-time R=16/K=8 kernel: more ranks than leave counting waves free
    (4, 8, 2500, 4, 64, 2.0),     # K=4, R=4: counting beside planning in the generic kernel
    (16, 4, 2050, 4, 16, 1.0),    # more ranks than leave counting waves free
    (3, 40, 1300, 5, 8, 1.0),     # experts per rank neither a power of two nor below 33
    (2, 1200, 700, 4, 8, 1.0),    # 256-thread workgroups with tables in scratch and two ranks: one wave counts beside the planning phases
    (2, 600, 900, 2, 4, 1.5),     # 256-thread workgroups with tables in LDS, two ranks
])
def test_planner_wide_groups_match_oracle(cuda, R, epn, S, K, tp, sigma):
    """Shapes outside the golden table (R > 8, large counts): the CPU oracle,
    itself pinned by the golden vectors, is the reference."""
    E = R * epn
    if S >= 100000:
        g = torch.Generator().manual_seed(5)
        pop = torch.exp(torch.normal(0.0, sigma, (E,), generator=g))
        topk = torch.multinomial(pop.expand(R * S, E), K, replacement=False, generator=g)
        topk = topk.to(torch.int32).reshape(R, S, K)
    else:
        topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed=31) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    print(f"R={R} epn={epn} S={S} K={K} tp={tp}", flush=True)
    gp, plans, dst_all_ref = oracle_world_plan(topk.numpy(), tpe.numpy(), tp)
    buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=0)
    dst_all, cu, etc, zfr, stats = launch_planning_all_ranks(buf._require_ctx(), topk.to(cuda),
                                                             tpe.to(cuda))
    torch.cuda.synchronize()
    assert np.array_equal(dst_all.cpu().numpy(), dst_all_ref)
    assert np.array_equal(cu.cpu().numpy(), gp.cu_seqlens)
    assert np.array_equal(etc.cpu().numpy(), gp.experts_to_copy)
    assert np.array_equal(zfr.cpu().numpy(), gp.zero_fill)
    assert np.array_equal(stats.cpu().numpy(), gp.remote_stats)
    buf.destroy()


def test_planner_random_small_shapes_match_oracle(cuda):
    """Seeded sweep of small shapes with awkward routing: equal balances (ties in
    every argmax/argmin), experts nobody routes to, one hot expert, repeated
    experts inside a token, padding 1 and padding larger than any group."""
    rng = np.random.default_rng(20240)
    checked = 0
    for it in range(120):
        R = int(rng.choice([1, 2, 3, 4, 5, 8]))
        epn = int(rng.integers(1, 6))
        K = int(rng.integers(1, 5))
        S = int(rng.integers(1, 49))
        tp = int(rng.choice([1, 2, 4, 16, 64]))
        E = R * epn
        kind = it % 4
        if kind == 0:      # uniform with replacement: duplicates inside a token
            topk = rng.integers(0, E, (R, S, K))
        elif kind == 1:    # every rank sends every token to the same few experts
            hot = rng.integers(0, E, (max(1, min(E, 2)),))
            topk = hot[rng.integers(0, hot.size, (R, S, K))]
        elif kind == 2:    # identical routing on every rank: equal balances everywhere
            one = rng.integers(0, E, (1, S, K))
            topk = np.repeat(one, R, axis=0)
        else:              # skewed popularity, distinct experts per token where possible
            p = np.exp(rng.normal(0.0, 2.0, E))
            p /= p.sum()
            topk = np.stack([[rng.choice(E, K, replace=K > E, p=p) for _ in range(S)]
                             for _ in range(R)])
        topk = topk.astype(np.int32)
        tpe = np.stack([np.bincount(topk[r].reshape(-1), minlength=E) for r in range(R)]).astype(np.int32)
        try:
            gp, plans, dst_all_ref = oracle_world_plan(topk, tpe, tp)
        except AssertionError:
            continue   # more remote experts than slots on some rank: the reference asserts too
        buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=0)
        dst_all, cu, etc, zfr, stats = launch_planning_all_ranks(
            buf._require_ctx(), torch.from_numpy(topk).to(cuda), torch.from_numpy(tpe).to(cuda))
        torch.cuda.synchronize()
        tag = f"iter {it}: R={R} epn={epn} S={S} K={K} tp={tp} kind={kind}"
        assert np.array_equal(dst_all.cpu().numpy(), dst_all_ref), tag
        assert np.array_equal(cu.cpu().numpy(), gp.cu_seqlens), tag
        assert np.array_equal(etc.cpu().numpy(), gp.experts_to_copy), tag
        assert np.array_equal(zfr.cpu().numpy(), gp.zero_fill), tag
        assert np.array_equal(stats.cpu().numpy(), gp.remote_stats), tag
        buf.destroy()
        checked += 1
    print(f"{checked} random shapes checked", flush=True)
    assert checked >= 80


def test_planner_random_multi_workgroup_shapes_match_oracle(cuda):
    """Seeded sweep of shapes with several workgroups per rank (2 to 24), through every kernel
    variant (compile-time R with top-8, the generic one), with the awkward routings of the
    small-shape sweep: duplicates inside a token, a few hot experts, identical routing on all
    ranks, skewed popularity."""
    rng = np.random.default_rng(77031)
    checked = 0
    for it in range(48):
        R = int(rng.choice([2, 4, 8, 16]))
        epn = int(rng.integers(1, 17))
        K = int(rng.choice([1, 2, 3, 5, 8, 8]))
        S = int(rng.integers(300, 3001))
        tp = int(rng.choice([1, 8, 16, 128]))
        E = R * epn
        kind = it % 4
        if kind == 0:
            topk = rng.integers(0, E, (R, S, K))
        elif kind == 1:
            hot = rng.integers(0, E, (max(1, min(E, 3)),))
            topk = hot[rng.integers(0, hot.size, (R, S, K))]
        elif kind == 2:
            topk = np.repeat(rng.integers(0, E, (1, S, K)), R, axis=0)
        else:
            p = np.exp(rng.normal(0.0, 1.5, E))
            p /= p.sum()
            if K <= E:   # distinct experts per token: Gumbel top-k
                g = rng.gumbel(size=(R, S, E)) + np.log(p)
                topk = np.argsort(-g, axis=2)[:, :, :K]
            else:
                topk = rng.choice(E, (R, S, K), p=p)
        topk = np.ascontiguousarray(topk).astype(np.int32)
        tpe = np.stack([np.bincount(topk[r].reshape(-1), minlength=E) for r in range(R)]).astype(np.int32)
        try:
            gp, plans, dst_all_ref = oracle_world_plan(topk, tpe, tp)
        except AssertionError:
            continue   # more remote experts than slots on some rank: the reference asserts too
        buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=0)
        dst_all, cu, etc, zfr, stats = launch_planning_all_ranks(
            buf._require_ctx(), torch.from_numpy(topk).to(cuda), torch.from_numpy(tpe).to(cuda))
        torch.cuda.synchronize()
        tag = f"iter {it}: R={R} epn={epn} S={S} K={K} tp={tp} kind={kind}"
        assert np.array_equal(dst_all.cpu().numpy(), dst_all_ref), tag
        assert np.array_equal(cu.cpu().numpy(), gp.cu_seqlens), tag
        assert np.array_equal(etc.cpu().numpy(), gp.experts_to_copy), tag
        assert np.array_equal(zfr.cpu().numpy(), gp.zero_fill), tag
        assert np.array_equal(stats.cpu().numpy(), gp.remote_stats), tag
        buf.destroy()
        checked += 1
    print(f"{checked} random multi-workgroup shapes checked", flush=True)
    assert checked >= 30


@pytest.mark.parametrize("S,K,E,R,tp,warm_elems", [
    (4096, 8, 256, 8, 128, 4096 * 7168),   # the headline shape with its token rows
    (40, 3, 8, 4, 8, 40 * 64),             # one warming workgroup, mostly clamped loads
    (17, 2, 6, 3, 4, 7),                   # fewer than 16 bytes: nothing to warm
    (64, 4, 4096, 8, 16, 64 * 256),        # the 256-thread planner variant with scratch tables
])
def test_planner_with_cache_warming_is_the_same_planner(cuda, S, K, E, R, tp, warm_elems):
    """mep_plan_warm = mep_plan plus workgroups that only read `warm`: same
    outputs as the oracle, and the warmed tensor is left as it was."""
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, 1.0, seed=3) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    gp, plans, _ = oracle_world_plan(topk.numpy(), tpe.numpy(), tp)
    g = torch.Generator().manual_seed(1)
    warm = torch.randn(warm_elems, generator=g).to(torch.bfloat16).to(cuda)
    before = warm.clone()
    rank = R - 1
    buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=rank)
    ctx = buf._require_ctx()
    plan, cu = allocate_planning_outputs(ctx)
    launch_planning(ctx, topk[rank].reshape(-1).contiguous().to(cuda), tpe.to(cuda), cu, plan, warm=warm)
    torch.cuda.synchronize()
    assert np.array_equal(plan.dst.cpu().numpy(), plans[rank].dst)
    assert np.array_equal(cu.cpu().numpy(), plans[rank].cu_seqlens)
    assert np.array_equal(plan.experts_to_copy.cpu().numpy(), gp.experts_to_copy)
    assert np.array_equal(plan.zero_fill_ranges.cpu().numpy(), plans[rank].zero_fill_ranges)
    assert np.array_equal(plan.remote_stats.cpu().numpy(), plans[rank].remote_stats)
    assert torch.equal(warm.view(torch.int16), before.view(torch.int16))
    buf.destroy()


def test_invalid_expert_ids_become_entries_that_nobody_copies(cuda):
    """An id outside [0, E) gets destination rank R (dst = R*NvS, never marked a
    duplicate): dispatch writes nothing for it, combine reads nothing, the other
    entries are planned as if it were not there."""
    from moonep_amd.combine import launch_combine
    from moonep_amd.dispatch import launch_dispatch
    from oracle import ops_oracle as oo
    S, H, K, E, R, tp, rank = 96, 256, 4, 12, 3, 8, 1
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, 1.0, seed=9) for r in range(R)])
    bad = topk[rank].clone()
    bad[3, 1] = E            # one past the last expert
    bad[3, 2] = -5           # negative
    bad[40, 0] = 1 << 20
    bad[95, 3] = E + 7
    valid = (bad >= 0) & (bad < E)
    tpe = routing.tokens_per_expert(topk, E)
    flat = bad.reshape(-1)
    tpe[rank] = torch.bincount(flat[valid.reshape(-1)].long(), minlength=E).to(torch.int32)
    gp = po.plan_global(tpe.numpy(), S, K, tp)
    NvS = gp.NvS
    raw = np.full(S * K, R * NvS, dtype=np.int64)
    vmask = valid.reshape(-1).numpy()
    raw[vmask] = po.raw_dst_for_rank(gp, flat.numpy()[vmask], rank)
    want = po.canonicalize_dst(raw, K, NvS)
    want[~vmask] = R * NvS                      # an invalid entry is never a duplicate
    buf = Buffer(S, H, K, E, R, token_padding=tp, rank=rank)
    ctx = buf._require_ctx()
    ctx["hidden_buf"].fill_(-3.0)
    plan, cu = allocate_planning_outputs(ctx)
    launch_planning(ctx, flat.contiguous().to(cuda), tpe.to(cuda), cu, plan)
    torch.cuda.synchronize()
    assert np.array_equal(plan.dst.cpu().numpy(), want.astype(np.int32))
    assert np.array_equal(cu.cpu().numpy(), gp.cu_seqlens[rank])
    # rows: only the valid entries are written, nothing outside the shards is touched
    g = torch.Generator().manual_seed(2)
    hid = torch.randint(-4, 5, (S, H), generator=g).to(torch.bfloat16)     # small integers: exact sums
    launch_dispatch(ctx, hid.to(cuda), None, plan, build_dedup_map=False, write_dups=True)
    out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
    launch_combine(ctx, out, plan.dst, mode="all")
    torch.cuda.synchronize()
    shards = ctx["hidden_buf"].view(R, NvS, H).cpu()
    written = torch.zeros(R * NvS, dtype=torch.bool)
    written[torch.from_numpy(raw[vmask])] = True
    for d in range(R):
        zf = gp.zero_fill[d] if d == rank else None
        if zf is not None:
            for start, n in zf:
                written[d * NvS + int(start): d * NvS + int(start) + int(n)] = True
    assert bool((shards.view(R * NvS, H)[~written] == -3.0).all())
    assert torch.equal(out.cpu().float(), hid.float() * valid.sum(1, keepdim=True).float())
    buf.destroy()


@pytest.mark.parametrize("S,K,E,R,tp,rank", [
    (1400, 8, 32, 8, 16, 5),    # 11 workgroups: ids to ignore in slices counted forwards and backwards
    (1301, 3, 12, 4, 8, 1),     # slices off 16-byte boundaries
])
def test_invalid_expert_ids_across_workgroups(cuda, S, K, E, R, tp, rank):
    """Ids outside [0, E) spread over a rank's entries, several workgroups per rank:
    a workgroup counts the entries before its slice or those after it, whichever
    are fewer, and neither count may include such an id."""
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, 1.0, seed=12) for r in range(R)])
    g = torch.Generator().manual_seed(77)
    bad = topk[rank].clone().reshape(-1)
    hit = torch.randperm(bad.numel(), generator=g)[: bad.numel() // 40]
    junk = torch.tensor([E, -1, E + 3, 1 << 24, -(1 << 30)], dtype=torch.int32)
    bad[hit] = junk[torch.randint(0, junk.numel(), (hit.numel(),), generator=g)]
    valid = (bad >= 0) & (bad < E)
    tpe = routing.tokens_per_expert(topk, E)
    tpe[rank] = torch.bincount(bad[valid].long(), minlength=E).to(torch.int32)
    gp = po.plan_global(tpe.numpy(), S, K, tp)
    NvS = gp.NvS
    raw = np.full(S * K, R * NvS, dtype=np.int64)
    vmask = valid.numpy()
    raw[vmask] = po.raw_dst_for_rank(gp, bad.numpy()[vmask], rank)
    want = po.canonicalize_dst(raw, K, NvS)
    want[~vmask] = R * NvS
    buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=rank)
    ctx = buf._require_ctx()
    plan, cu = allocate_planning_outputs(ctx)
    launch_planning(ctx, bad.contiguous().to(cuda), tpe.to(cuda), cu, plan)
    torch.cuda.synchronize()
    assert np.array_equal(plan.dst.cpu().numpy(), want.astype(np.int32))
    assert np.array_equal(cu.cpu().numpy(), gp.cu_seqlens[rank])
    buf.destroy()
