"""The configurations the benchmark quotes, at their full sizes, checked through
properties that do not need an oracle pass over gigabytes:

* plan -> dispatch -> combine recorded in one HIP graph and replayed with new
  tokens, at every point of the maxvio sweep on both shapes: the plan equals
  the oracle's, every copy of every token is where its decoded dst says, nothing
  else was written, padding rows are zero, the weights come back bit for bit,
  all-ones rows combine to exactly K;
* prefetch_weight and reduce_grad at [32, 7168, 2048] per rank, R = 8, driven
  by the PLANNER's experts_to_copy: every requested slot holds the owner's
  expert, every other slot its sentinel; affine integer grads give the closed
  form of the sum; own occupied slots are zero afterwards;
* the weighted top-k sum at the headline shape with small-integer rows and
  power-of-two weights, where the fp32 arithmetic is exact.
"""

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, routing
from moonep_amd.combine import launch_combine
from moonep_amd.dispatch import launch_dispatch
from moonep_amd.grad_reduce import launch_grad_reduce
from moonep_amd.planning import allocate_planning_outputs, launch_planning, launch_planning_all_ranks
from moonep_amd.prefetch import launch_prefetch, launch_prefetch_pull
from oracle import ops_oracle as oo
from oracle import planner_oracle as po

pytestmark = pytest.mark.gpu

R, K, TP = 8, 8, 128
SWEEP = [(4096, 7168, 256, mv) for mv in (0.0, 0.5, 1.0, 2.0, 4.0)] + \
        [(8192, 4096, 128, mv) for mv in (0.0, 0.5, 1.0, 2.0, 4.0)] + \
        [(8192, 7168, 384, 1.0),      # the configuration of the reference's own figure
         (4096, 7168, 256, 20.0)]     # the largest imbalance of that figure (maxvio 0.2 .. 20)


@pytest.mark.parametrize("S,H,E,mv", SWEEP, ids=[f"S{s}_H{h}_E{e}_maxvio{m}" for s, h, e, m in SWEEP])
def test_chain_from_a_hip_graph_at_every_sweep_point(cuda, S, H, E, mv):
    rank = 5
    topk, w, tpe, real_mv, _ = routing.logit_routing(S, K, E, R, mv, seed=77)
    print(f"S={S} H={H} E={E} target maxvio={mv} realised={real_mv:.3f}", flush=True)
    buf = Buffer(S, H, K, E, R, token_padding=TP, rank=rank)
    ctx = buf._require_ctx()
    NvS, NvSp = int(ctx["NvS"]), int(ctx["NvS_padded"])
    d_topk = topk[rank].reshape(-1).contiguous().to(cuda)
    d_tpe = tpe.to(cuda)
    d_w = w[rank].contiguous().to(cuda)
    hidden = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)       # static graph inputs
    out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
    out_w = torch.empty(S, K, dtype=torch.float32, device=cuda)
    plan, cu = allocate_planning_outputs(ctx)

    def chain():
        launch_planning(ctx, d_topk, d_tpe, cu, plan, warm=hidden)
        launch_dispatch(ctx, hidden, d_w, plan, build_dedup_map=False, write_dups=True)
        launch_combine(ctx, out, plan.dst, out_w, mode="two_level")

    g = torch.Generator(device=cuda).manual_seed(5)
    hidden.copy_(torch.randn(S, H, device=cuda, generator=g))
    chain()                                   # eager once, then capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()

    gp = po.plan_global(tpe.numpy(), S, K, TP)
    rp = po.plan_rank(gp, topk[rank].reshape(-1).numpy(), rank)
    drank, loff, _ = oo.decode(torch.from_numpy(rp.dst), NvS)
    rows = (drank * NvSp + loff).to(cuda)
    pad = torch.zeros(R * NvSp, dtype=torch.bool)
    for start, n in rp.zero_fill_ranges:
        pad[rank * NvSp + int(start): rank * NvSp + int(start) + int(n)] = True
    pad = pad.to(cuda)
    for replay in range(2):
        # new tokens, poisoned plan outputs and shards: everything must come from this replay
        hidden.copy_(torch.randn(S, H, device=cuda, generator=g))
        plan.dst.fill_(-7)
        cu.fill_(-7)
        ctx["hidden_buf"].zero_()
        ctx["hidden_buf"].view(R * NvSp, H)[pad] = 9.0          # padding rows must be zeroed again
        ctx["meta_buf"].zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(plan.dst.cpu().numpy(), rp.dst), f"replay {replay}: dst"
        assert np.array_equal(cu.cpu().numpy(), rp.cu_seqlens)
        assert np.array_equal(plan.experts_to_copy.cpu().numpy(), gp.experts_to_copy)
        assert np.array_equal(plan.zero_fill_ranges.cpu().numpy(), rp.zero_fill_ranges)
        shards = ctx["hidden_buf"].view(R * NvSp, H)
        back = shards[rows].view(S, K, H)
        assert torch.equal(back, hidden[:, None, :].expand(S, K, H)), "dispatched rows"
        assert int((shards != 0).any(dim=1).sum()) == S * K, "rows written besides the S*K copies"
        assert not bool(shards[pad].any()), "padding rows"
        assert torch.equal(out_w.view(torch.int32), d_w.view(torch.int32)), "weight round trip"
        ref = (hidden.float() * K).to(torch.bfloat16)
        err = (out.float() - ref.float()).abs() / oo.bf16_ulp(ref.cpu()).to(cuda)
        assert float(err.max()) <= 1.5          # K equal addends: the reference's tolerance
    # linearity: all-ones tokens come back as exactly K
    hidden.fill_(1.0)
    graph.replay()
    torch.cuda.synchronize()
    assert bool((out == float(K)).all())
    del graph
    buf.destroy()


def test_prefetch_and_grad_reduce_at_the_real_shape_with_the_planners_table(cuda):
    S, E, H, Hp = 4096, 256, 7168, 2048
    epn = E // R
    topk, _, tpe, mv, _ = routing.logit_routing(S, K, E, R, 1.0, seed=2024, want_weights=False)
    buf = Buffer(S, 16, K, E, R, token_padding=TP, rank=0)          # H plays no part in planning
    _, _, etc_dev, _, _ = launch_planning_all_ranks(buf._require_ctx(), topk.to(cuda), tpe.to(cuda))
    torch.cuda.synchronize()
    etc = etc_dev.cpu().numpy()
    assert np.array_equal(etc, po.plan_global(tpe.numpy(), S, K, TP).experts_to_copy)
    owners = [(int(((etc // epn) == r).sum()), r) for r in range(R)]
    n_busiest, busiest = max(owners)
    assert n_busiest > 0, "this routing hosts remote experts"
    print(f"maxvio={mv:.3f} slots per owner={sorted(owners)} busiest={busiest}", flush=True)

    # ---- prefetch: local expert le of owner r is the constant (r*epn+le)/8 (bf16-exact)
    SENT = -1.0
    pool = torch.full((R, epn, H, Hp), SENT, dtype=torch.bfloat16, device=cuda)     # 7.5 GB
    for owner in sorted({busiest, (busiest + 3) % R}):
        ids = (torch.arange(epn, device=cuda) + owner * epn).to(torch.bfloat16) / 8
        local = ids[:, None, None].expand(epn, H, Hp).contiguous()
        launch_prefetch((local,) * 3, (pool,) * 3, etc_dev, rank=owner)
        torch.cuda.synchronize()
        flat = pool.view(R * epn, H * Hp)
        lo, hi = flat.min(dim=1).values.float().cpu(), flat.max(dim=1).values.float().cpu()
        for d in range(R):
            for b in range(epn):
                e = int(etc[d, b])
                want = e / 8 if (e >= 0 and e // epn == owner) else None
                got = (float(lo[d * epn + b]), float(hi[d * epn + b]))
                if want is not None:
                    assert got == (want, want), (owner, d, b, e, got)
                else:       # not this owner's: still the sentinel, or an earlier owner's expert
                    assert got[0] == got[1] and (got[0] == SENT or got[0] == e / 8), (owner, d, b, got)
        del local
    # ---- the pull view: the fullest rank's slots from all owners in one launch
    pool.fill_(SENT)
    ids = (torch.arange(R * epn, device=cuda).to(torch.bfloat16) / 8).view(R, epn)
    all_local = ids[:, :, None, None].expand(R, epn, H, Hp).contiguous()                 # 7.5 GB
    n_full, fullest = max((int((etc[r] >= 0).sum()), r) for r in range(R))
    launch_prefetch_pull((all_local,) * 3, (pool,) * 3, etc_dev, rank=fullest)
    torch.cuda.synchronize()
    flat = pool.view(R * epn, H * Hp)
    lo, hi = flat.min(dim=1).values.float().cpu(), flat.max(dim=1).values.float().cpu()
    for d in range(R):
        for b in range(epn):
            e = int(etc[d, b])
            want = e / 8 if (d == fullest and e >= 0) else SENT
            assert (float(lo[d * epn + b]), float(hi[d * epn + b])) == (want, want), (d, b, e)
    print(f"pull: rank {fullest} filled {n_full} slots", flush=True)
    del pool, all_local
    torch.cuda.empty_cache()

    # ---- grad reduce: slot (src, b) = src*64 + b, local grad of expert le = 1000 + le
    rank = busiest
    red = torch.empty(R, epn, H, Hp, dtype=torch.float32, device=cuda)               # 15 GB
    vals = (torch.arange(R, device=cuda)[:, None] * 64 + torch.arange(epn, device=cuda)[None, :]).float()
    red.copy_(vals[:, :, None, None].expand(R, epn, H, Hp))
    grad = (1000.0 + torch.arange(epn, device=cuda).float())[:, None, None].expand(epn, H, Hp).contiguous()
    launch_grad_reduce(grad, red, etc_dev, rank=rank)
    torch.cuda.synchronize()
    want = 1000.0 + torch.arange(epn).float()
    for src in range(R):
        for b in range(epn):
            e = int(etc[src, b])
            if e >= 0 and e // epn == rank:
                want[e % epn] += src * 64 + b
    g2 = grad.view(epn, -1)
    assert torch.equal(g2.min(dim=1).values.cpu(), want) and torch.equal(g2.max(dim=1).values.cpu(), want)
    r2 = red.view(R * epn, -1)
    lo, hi = r2.min(dim=1).values.cpu(), r2.max(dim=1).values.cpu()
    for src in range(R):
        for b in range(epn):
            cleared = src == rank and int(etc[src, b]) >= 0
            v = 0.0 if cleared else float(src * 64 + b)
            assert (float(lo[src * epn + b]), float(hi[src * epn + b])) == (v, v), (src, b)
    buf.destroy()


def test_weighted_combine_at_the_headline_shape_is_exact_on_exact_data(cuda):
    S, H, E, rank = 4096, 7168, 256, 3
    topk, _, tpe, _, _ = routing.logit_routing(S, K, E, R, 1.0, seed=99, want_weights=False)
    buf = Buffer(S, H, K, E, R, token_padding=TP, rank=rank)
    ctx = buf._require_ctx()
    NvS, NvSp = int(ctx["NvS"]), int(ctx["NvS_padded"])
    g = torch.Generator(device=cuda).manual_seed(3)
    # rows in [-4, 4], weights 2^-j, j in 0..3: every product and partial sum is a multiple of
    # 1/8 below 32 in magnitude, exact in fp32 and representable in bf16
    hidden = torch.randint(-4, 5, (S, H), device=cuda, generator=g).to(torch.bfloat16)
    wk = torch.pow(2.0, -torch.randint(0, 4, (S, K), device=cuda, generator=g).float())
    plan, cu = allocate_planning_outputs(ctx)
    launch_planning(ctx, topk[rank].reshape(-1).contiguous().to(cuda), tpe.to(cuda), cu, plan)
    ctx["hidden_buf"].zero_()
    launch_dispatch(ctx, hidden, wk, plan, build_dedup_map=False, write_dups=True)
    # the "experts" negate every second row of the shards, so that the rows of a token differ
    ctx["hidden_buf"].view(R * NvSp, H)[1::2].neg_()
    out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
    launch_combine(ctx, out, plan.dst, None, mode="weighted")
    torch.cuda.synchronize()
    drank, loff, _ = oo.decode(plan.dst.cpu(), NvS)
    rows = (drank * NvSp + loff).to(cuda)
    want = torch.zeros(S, H, dtype=torch.float32, device=cuda)
    gathered = ctx["hidden_buf"].view(R * NvSp, H)
    for k in range(K):                          # ascending k, as the kernel adds
        want += wk[:, k:k + 1] * gathered[rows.view(S, K)[:, k]].float()
    assert float(want.abs().max()) <= 32.0
    assert torch.equal(out.float(), want), "weighted top-k sum"
    assert bool((want.to(torch.bfloat16).float() == want).all())      # nothing was rounded
    buf.destroy()
