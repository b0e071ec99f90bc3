"""Dispatch / epilogue / prologue / combine kernels vs the CPU oracle.

Dispatch, the duplicate expansion and the weight round trip are pure copies:
bit-exact.  Combine is an fp32 sum in a fixed order with one (or, in the
reference's two-kernel pipeline, two) bf16 roundings: compared bit-exact with
the oracle that adds in the same order, and within 1 bf16 ulp of a
single-rounding fp32 K-sum (tolerance of reference tests/test_combine.py:202-211).
"""

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, EmulatedWorld, routing
from moonep_amd.combine import launch_combine, launch_combine_prologue
from moonep_amd.dispatch import launch_build_dedup, launch_dispatch, launch_dispatch_epilogue
from moonep_amd.planning import MoonEPCommPlan
from oracle import ops_oracle as oo
from oracle import planner_oracle as po
from tests.util import oracle_world_plan, traceable_hidden, traceable_weights

pytestmark = pytest.mark.gpu

POISON_ROW = 7.0
POISON_W = 0x55555555


def _plan_from_oracle(rp, gp, dev, dups=None):
    R, E, NvS, K = gp.R, gp.E, gp.NvS, gp.K
    i32 = dict(dtype=torch.int32, device=dev)
    if dups is None:
        dg, dl, dc = np.zeros((NvS, 3)), np.zeros(NvS), np.zeros(2)
    else:
        dg, dl, dc = dups
    return MoonEPCommPlan(
        dst=torch.from_numpy(rp.dst).to(dev),
        experts_to_copy=torch.from_numpy(rp.experts_to_copy).to(dev),
        zero_fill_ranges=torch.from_numpy(rp.zero_fill_ranges).to(dev),
        remote_stats=torch.from_numpy(rp.remote_stats).to(dev),
        dup_groups=torch.as_tensor(dg, **i32).contiguous(),
        dup_loffs=torch.as_tensor(dl, **i32).contiguous(),
        dup_counts=torch.as_tensor(dc, **i32).contiguous(),
        N=gp.S * K, R=R, E=E, NvS=NvS, K=K)


CASES = [
    # name, S, H, K, epn, R, tp, routing
    ("tiny_k1", 5, 8, 1, 1, 2, 4, ("biased", 1.0)),
    ("ragged_h", 17, 200, 3, 3, 4, 16, ("biased", 0.5)),
    ("dups_all_local", 32, 256, 4, 8, 4, 16, ("pattern", "all_local")),
    ("dups_one_expert", 16, 512, 4, 4, 4, 8, ("pattern", "duplicate_topk")),
    ("single_expert", 9, 128, 2, 4, 8, 8, ("pattern", "single_expert")),
    ("no_padding", 33, 64, 2, 2, 4, 1, ("biased", 1.0)),
    ("h7168_rows", 64, 7168, 8, 4, 8, 32, ("biased", 1.0)),
    ("h4096_rows", 48, 4096, 8, 2, 8, 16, ("biased", 2.0)),
    ("k32", 8, 1024, 32, 8, 4, 8, ("biased", 1.0)),
    # rows of 3, 10 and 16 whole 1-KiB wave tiles, and one just past a tile (the strided loop)
    ("h1536_rows", 40, 1536, 4, 2, 4, 8, ("biased", 1.0)),
    ("h5120_rows", 24, 5120, 6, 4, 4, 16, ("biased", 1.5)),
    ("h8192_rows", 24, 8192, 8, 2, 8, 16, ("biased", 1.0)),
    ("h8200_rows", 12, 8200, 2, 2, 4, 4, ("biased", 1.0)),
]


def _random_cases(n, seed=99):
    """Seeded small shapes: row lengths that are odd multiples of 8 elements, K
    up to 6, 1 to 8 ranks, paddings from 1 to 64."""
    import random
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        R = rnd.choice([1, 2, 3, 4, 8])
        epn = rnd.randint(1, 5)
        K = rnd.randint(1, min(6, R * epn))
        out.append((f"rand{i}", rnd.randint(1, 40), 8 * rnd.randint(1, 160), K, epn, R,
                    rnd.choice([1, 4, 16, 64]), ("biased", rnd.choice([0.0, 1.0, 3.0]))))
    return out


CASES += _random_cases(24)


def _topk(case):
    name, S, H, K, epn, R, tp, (kind, arg) = case
    E = epn * R
    if kind == "biased":
        return torch.stack([routing.popularity_biased(S, K, E, R, r, arg, seed=77) for r in range(R)])
    return torch.stack([routing.pattern(arg, S, K, E, R, r) for r in range(R)])


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_world_dispatch_combine_matches_oracle(cuda, case):
    name, S, H, K, epn, R, tp, _ = case
    E = epn * R
    topk = _topk(case)
    tpe = routing.tokens_per_expert(topk, E)
    gp, plans, dst_all = oracle_world_plan(topk.numpy(), tpe.numpy(), tp)
    NvS = gp.NvS
    print(f"case {name}: S={S} H={H} K={K} E={E} R={R} tp={tp} NvS={NvS}", flush=True)
    world = EmulatedWorld(S, H, K, E, R, tp)
    bufs = [Buffer(S, H, K, E, R, token_padding=tp, rank=r, world=world) for r in range(R)]
    mcp = world.layout["meta_chunk_padded"]
    hid = [traceable_hidden(S, H, r) for r in range(R)]
    wts = [traceable_weights(S, K, r) for r in range(R)]

    # ---------------- oracle world: primaries, then epilogue on every rank
    sh_ref = torch.full((R, NvS, H), POISON_ROW, dtype=torch.bfloat16)
    ws_ref = torch.full((R, NvS), POISON_W, dtype=torch.int32).view(torch.float32)
    sh_fused = sh_ref.clone()
    ws_fused = ws_ref.clone()
    for r in range(R):
        zf = torch.from_numpy(plans[r].zero_fill_ranges)
        oo.dispatch(hid[r], wts[r], torch.from_numpy(plans[r].dst), zf, sh_ref, ws_ref, r, K)
        oo.dispatch(hid[r], wts[r], torch.from_numpy(plans[r].dst), zf, sh_fused, ws_fused, r, K,
                    include_dups=True)
    prim_only = sh_ref.clone()
    dups = [po.dedup_structs(dst_all, r, S, K, NvS) for r in range(R)]
    for r in range(R):
        oo.dispatch_epilogue(sh_ref[r], *dups[r])
    # dispatch + epilogue == fused dispatch, on every real or padding row
    assert torch.equal(sh_ref.view(torch.int16), sh_fused.view(torch.int16))

    # ---------------- GPU: two-kernel path (primaries + epilogue)
    world.hidden_buf.fill_(POISON_ROW)
    world.meta_buf.fill_(POISON_W)
    gplans = [_plan_from_oracle(plans[r], gp, cuda) for r in range(R)]
    dst_all_dev = torch.from_numpy(dst_all).to(cuda)
    for r in range(R):
        launch_dispatch(bufs[r]._require_ctx(), hid[r].to(cuda), wts[r].to(cuda), gplans[r],
                        build_dedup_map=True, dst_all_ranks=dst_all_dev)
    torch.cuda.synchronize()
    got = world.hidden_buf.view(R, NvS, H).cpu()
    assert torch.equal(got.view(torch.int16), prim_only.view(torch.int16)), "primaries-only dispatch"
    got_w = world.meta_buf.view(R, mcp)[:, :NvS].cpu()
    assert torch.equal(got_w, ws_ref.view(torch.int32)), "weight slots"
    for r in range(R):
        # duplicate groups built on the GPU equal the oracle's, in order
        ng, nd = (int(v) for v in gplans[r].dup_counts.cpu())
        assert [ng, nd] == dups[r][2].tolist()
        assert np.array_equal(gplans[r].dup_groups.cpu().numpy()[:ng], dups[r][0][:ng])
        assert np.array_equal(gplans[r].dup_loffs.cpu().numpy()[:nd], dups[r][1][:nd])
        launch_dispatch_epilogue(bufs[r]._require_ctx(), gplans[r])
    torch.cuda.synchronize()
    got = world.hidden_buf.view(R, NvS, H).cpu()
    assert torch.equal(got.view(torch.int16), sh_ref.view(torch.int16)), "dispatch + epilogue"

    # ---------------- GPU: fused path (what Buffer.dispatch runs)
    world.hidden_buf.fill_(POISON_ROW)
    world.meta_buf.fill_(POISON_W)
    for r in range(R):
        launch_dispatch(bufs[r]._require_ctx(), hid[r].to(cuda), wts[r].to(cuda), gplans[r],
                        build_dedup_map=False, write_dups=True)
    torch.cuda.synchronize()
    got = world.hidden_buf.view(R, NvS, H).cpu()
    assert torch.equal(got.view(torch.int16), sh_ref.view(torch.int16)), "fused dispatch"
    # rows outside every segment keep the poison (dispatch writes nothing else)
    for r in range(R):
        end = int(gp.cu_seqlens[r, -1])
        assert (got[r, end:] == POISON_ROW).all()
        assert (got_w[r, end:] == POISON_W).all()
        # padding rows and their weight slots are zero
        for start, n in plans[r].zero_fill_ranges.tolist():
            if n:
                assert (got[r, start:start + n] == 0).all()
                assert (got_w[r, start:start + n] == 0).all()

    # ---------------- combine: "expert outputs" = deterministic transform of the rows
    g = torch.Generator().manual_seed(5)
    expert_out = (torch.randn(R, NvS, H, generator=g) * 3).to(torch.bfloat16)
    world.hidden_buf.copy_(expert_out.view(R * NvS, H))
    ws_dev = ws_ref.clone()
    for mode in ("all", "two_level"):
        for r in range(R):
            dst_r = torch.from_numpy(plans[r].dst)
            want, want_w = oo.combine(expert_out, ws_dev, dst_r, K, mode=mode)
            out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
            out_w = torch.empty(S, K, dtype=torch.float32, device=cuda)
            launch_combine(bufs[r]._require_ctx(), out, gplans[r].dst, out_w, mode=mode)
            torch.cuda.synchronize()
            assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16)), (mode, r)
            assert torch.equal(out_w.cpu().view(torch.int32), want_w.view(torch.int32))
            # the gathered weights are the ones this rank scattered
            assert torch.equal(out_w.cpu().view(torch.int32), wts[r].view(torch.int32))
    # weighted extension: bit-exact against the oracle that rounds product and sum separately
    # (ordinary route weights: the traceable ones above are bit patterns, not magnitudes)
    ws_w = torch.rand(R, NvS, generator=g) * 0.95 + 0.05
    world.meta_buf.view(R, mcp)[:, :NvS] = ws_w.view(torch.int32).to(cuda)
    for r in range(R):
        dst_r = torch.from_numpy(plans[r].dst)
        want, _ = oo.combine(expert_out, ws_w, dst_r, K, mode="weighted")
        out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
        launch_combine(bufs[r]._require_ctx(), out, gplans[r].dst, None, mode="weighted")
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16)), ("weighted", r)
    world.meta_buf.view(R, mcp)[:, :NvS] = ws_ref.view(torch.int32).to(cuda)
    # Tolerance of the reference's own test (tests/test_combine.py:202-211):
    # within 1 bf16 ulp (+0.5 slack) of the single-rounding fp32 K-sum, on
    # same-sign data (with cancellation the group rounding of the reference
    # pipeline is not small against the final result's ulp).
    pos = (expert_out.float().abs() + 0.25).to(torch.bfloat16)
    world.hidden_buf.copy_(pos.view(R * NvS, H))
    for r in range(R):
        dst_r = torch.from_numpy(plans[r].dst)
        ref_all, _ = oo.combine(pos, None, dst_r, K, mode="all")
        out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
        launch_combine(bufs[r]._require_ctx(), out, gplans[r].dst, None, mode="two_level")
        torch.cuda.synchronize()
        err = (out.cpu().float() - ref_all.float()).abs() / oo.bf16_ulp(ref_all)
        assert float(err.max()) <= 1.5, (r, float(err.max()))
    world.hidden_buf.copy_(expert_out.view(R * NvS, H))
    # reference pipeline: prologue on every rank, then primaries-only combine
    pro_ref = expert_out.clone()
    for r in range(R):
        oo.combine_prologue(pro_ref[r], *dups[r])
        launch_combine_prologue(bufs[r]._require_ctx(), gplans[r])
    torch.cuda.synchronize()
    got = world.hidden_buf.view(R, NvS, H).cpu()
    assert torch.equal(got.view(torch.int16), pro_ref.view(torch.int16)), "combine prologue"
    for r in range(R):
        dst_r = torch.from_numpy(plans[r].dst)
        want, _ = oo.combine(pro_ref, None, dst_r, K, mode="primaries")
        two, _ = oo.combine(expert_out, None, dst_r, K, mode="two_level")
        assert torch.equal(want.view(torch.int16), two.view(torch.int16)), "oracle: two_level == pipeline"
        out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
        launch_combine(bufs[r]._require_ctx(), out, gplans[r].dst, None, mode="primaries")
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16)), ("primaries", r)
    for b in bufs:
        b.destroy()


def test_combine_exact_cases(cuda):
    """Cases where the fp32 sum is exact, so every mode must agree bit for bit
    with plain arithmetic: K = 1 (a pure gather) and small-integer payloads."""
    S, H, K, epn, R, tp = 24, 384, 4, 2, 4, 8
    E = epn * R
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, 1.0, seed=3) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    gp, plans, dst_all = oracle_world_plan(topk.numpy(), tpe.numpy(), tp)
    world = EmulatedWorld(S, H, K, E, R, tp)
    buf = Buffer(S, H, K, E, R, token_padding=tp, rank=1, world=world)
    g = torch.Generator().manual_seed(9)
    ints = torch.randint(-8, 9, (R, gp.NvS, H), generator=g).to(torch.bfloat16)
    world.hidden_buf.copy_(ints.view(-1, H))
    dst = torch.from_numpy(plans[1].dst)
    drank, loff, _ = oo.decode(dst, gp.NvS)
    want = ints.view(-1, H)[drank * gp.NvS + loff].float().view(S, K, H).sum(1).to(torch.bfloat16)
    for mode in ("all", "two_level"):
        out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
        launch_combine(buf._require_ctx(), out, dst.to(cuda), None, mode=mode)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want), mode
    buf.destroy()


@pytest.mark.parametrize("S,H,K,E,mv", [(4096, 7168, 8, 256, 1.0), (8192, 4096, 8, 128, 2.0),
                                         (8192, 7168, 16, 256, 1.0)])  # last: 16 GB of shards, large strides
def test_headline_shape_round_trip(cuda, S, H, K, E, mv):
    """Full-size single-rank share through the public API: properties that do
    not need an oracle pass over 4.7 GB."""
    R, tp, rank = 8, 128, 2
    topk, w, tpe, real_mv, _ = routing.logit_routing(S, K, E, R, mv, seed=4321)
    print(f"S={S} H={H} E={E} maxvio={real_mv:.3f}", flush=True)
    buf = Buffer(S, H, K, E, R, token_padding=tp, rank=rank)
    ctx = buf._require_ctx()
    NvS = ctx["NvS"]
    g = torch.Generator().manual_seed(11)
    hidden = torch.randn(S, H, generator=g).to(torch.bfloat16).to(cuda)
    wk = w[rank].contiguous().to(cuda)
    ctx["hidden_buf"].zero_()
    hidden_nvsh, w_nvs, cu, plan = buf.dispatch(hidden, wk, topk[rank].contiguous().to(cuda),
                                                tpe.to(cuda), zero_copy=True,
                                                router_weights_zero_copy=True)
    torch.cuda.synchronize()
    # planner output equals the oracle
    gp = po.plan_global(tpe.numpy(), S, K, tp)
    rp = po.plan_rank(gp, topk[rank].reshape(-1).numpy(), rank)
    assert np.array_equal(plan.dst.cpu().numpy(), rp.dst)
    assert np.array_equal(cu.cpu().numpy(), rp.cu_seqlens)
    # every copy of every token landed: gather rows back by decoded dst
    drank, loff, _ = oo.decode(plan.dst.cpu(), NvS)
    rows = (drank * ctx["NvS_padded"] + loff).to(cuda)
    back = ctx["hidden_buf"][rows].view(S, K, H)
    assert torch.equal(back, hidden[:, None, :].expand(S, K, H)), "dispatched rows"
    # number of non-zero rows == S*K (zero-initialised shards, randn rows are never all-zero)
    nz = int((ctx["hidden_buf"] != 0).any(dim=1).sum())
    assert nz == S * K
    # combine of the untouched shards = K * hidden up to the rounding of the sum
    out, w_back, _ = buf.combine(plan=plan, hidden_nvsh=hidden_nvsh, route_weights_nvs=w_nvs,
                                 zero_copy=True, router_weights_zero_copy=True)
    torch.cuda.synchronize()
    assert torch.equal(w_back.view(torch.int32), wk.view(torch.int32)), "weight round trip"
    ref = (hidden.float() * K).to(torch.bfloat16)
    err = (out.float() - ref.float()).abs() / oo.bf16_ulp(ref.cpu()).to(cuda)
    # K identical addends: partial sums j*x round at most once more than K*x
    assert float(err.max()) <= 1.5
    # linearity: combine(all-ones rows) == K exactly
    ctx["hidden_buf"].fill_(1.0)
    out1, _, _ = buf.combine(plan=plan, hidden_nvsh=hidden_nvsh, zero_copy=True)
    torch.cuda.synchronize()
    assert bool((out1 == float(K)).all())
    buf.destroy()


def test_saved_plan_hidden_only_dispatch_reuses_dst_and_skips_weights(cuda):
    """Mirror of reference tests/test_dispatch.py:351-416: a plan saved from an
    earlier dispatch is reused for a hidden-only dispatch after another plan
    has used the buffers.  The rows must follow the saved dst, the padding rows
    must be zero, the weight slots must keep what the other dispatch left and
    the saved duplicate structures must not change."""
    from moonep_amd.planning import allocate_planning_outputs, launch_planning, \
        launch_planning_all_ranks

    S, K, epn, H, tp, R = 17, 3, 8, 64, 16, 4
    E = R * epn
    world = EmulatedWorld(S, H, K, E, R, tp)
    bufs = [Buffer(S, H, K, E, R, token_padding=tp, rank=r, world=world) for r in range(R)]
    NvS = world.NvS
    mcp = world.layout["meta_chunk_padded"]

    def plan_all(kind):
        topk = torch.stack([routing.pattern(kind, S, K, E, R, r) for r in range(R)])
        tpe = routing.tokens_per_expert(topk, E).to(cuda)
        dst_all = launch_planning_all_ranks(bufs[0]._require_ctx(), topk.to(cuda), tpe)[0]
        plans = []
        for r in range(R):
            plan, cu = allocate_planning_outputs(bufs[r]._require_ctx())
            launch_planning(bufs[r]._require_ctx(), topk[r].reshape(-1).to(cuda), tpe, cu, plan)
            plans.append(plan)
        return plans, dst_all

    hid_a = [traceable_hidden(S, H, r).to(cuda) for r in range(R)]
    wts_a = [traceable_weights(S, K, r).to(cuda) for r in range(R)]
    plans_a, dst_all_a = plan_all("all_remote")
    for r in range(R):
        launch_dispatch(bufs[r]._require_ctx(), hid_a[r], wts_a[r], plans_a[r], build_dedup_map=True,
                        dst_all_ranks=dst_all_a)
    for r in range(R):
        launch_dispatch_epilogue(bufs[r]._require_ctx(), plans_a[r])
    torch.cuda.synchronize()
    saved = [(p.dup_groups.clone(), p.dup_loffs.clone(), p.dup_counts.clone()) for p in plans_a]
    assert sum(int(c[2][1]) for c in saved) > 0, "the saved plans should hold duplicates"

    g = torch.Generator().manual_seed(3)
    plans_b, dst_all_b = plan_all("all_local")
    for r in range(R):
        hb = torch.randn(S, H, generator=g).to(torch.bfloat16).to(cuda)
        wb = torch.rand(S, K, generator=g).to(cuda)
        launch_dispatch(bufs[r]._require_ctx(), hb, wb, plans_b[r], build_dedup_map=True,
                        dst_all_ranks=dst_all_b)
    for r in range(R):
        launch_dispatch_epilogue(bufs[r]._require_ctx(), plans_b[r])
    torch.cuda.synchronize()
    weights_after_b = world.meta_buf.view(R, mcp)[:, :NvS].clone()

    for r in range(R):   # the reuse: no weights, no duplicate-map build
        launch_dispatch(bufs[r]._require_ctx(), hid_a[r], None, plans_a[r], build_dedup_map=False)
    for r in range(R):
        launch_dispatch_epilogue(bufs[r]._require_ctx(), plans_a[r])
    torch.cuda.synchronize()

    shards = world.hidden_buf.view(R, NvS, H).cpu()
    checked = 0
    for r in range(R):
        drank, loff, _ = oo.decode(plans_a[r].dst.cpu(), NvS)
        rows = shards[drank, loff]                      # [S*K, H], duplicates included
        want = hid_a[r].cpu().repeat_interleave(K, dim=0)
        assert torch.equal(rows.view(torch.int16), want.view(torch.int16)), f"rank {r} rows"
        checked += rows.shape[0]
        padded = 0
        for start, n in plans_a[r].zero_fill_ranges.cpu().tolist():
            if n:
                assert (shards[r, start:start + n] == 0).all()
                padded += n
        assert padded > 0
    assert checked == R * S * K
    assert torch.equal(world.meta_buf.view(R, mcp)[:, :NvS], weights_after_b), \
        "weight slots changed during a hidden-only dispatch"
    for p, (dg, dl, dc) in zip(plans_a, saved):
        assert torch.equal(p.dup_groups, dg) and torch.equal(p.dup_loffs, dl) and \
            torch.equal(p.dup_counts, dc), "saved duplicate structures changed during reuse"
    for b in bufs:
        b.destroy()
