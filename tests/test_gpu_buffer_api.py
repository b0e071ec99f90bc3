"""The public Buffer API end to end on one GPU (ideas of reference
tests/test_e2e.py, test_dispatch.py and test_combine.py): sync vs async vs
plan reuse vs zero-copy give the same bits; a world of R Buffers sharing the
emulated shards reproduces the all-rank result of the oracle; bad inputs raise
the reference's assertions; the whole chain replays from a HIP graph."""

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, EmulatedWorld, MoonEPCommPlan, routing
from oracle import ops_oracle as oo
from oracle import planner_oracle as po
from tests.util import oracle_world_plan

pytestmark = pytest.mark.gpu

S, H, K, EPN, R, TP = 48, 256, 4, 3, 4, 16
E = EPN * R


def _routing(seed=21, sigma=1.0):
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed) for r in range(R)])
    return topk, routing.tokens_per_expert(topk, E)


def _tokens(seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(S, H, generator=g).to(torch.bfloat16), torch.rand(S, K, generator=g)


def test_world_of_buffers_matches_oracle(cuda):
    topk, tpe = _routing()
    gp, plans, dst_all = oracle_world_plan(topk.numpy(), tpe.numpy(), TP)
    NvS = gp.NvS
    world = EmulatedWorld(S, H, K, E, R, TP)
    world.hidden_buf.zero_()
    bufs = [Buffer(S, H, K, E, R, token_padding=TP, rank=r, world=world) for r in range(R)]
    hid, wts = zip(*[_tokens(100 + r) for r in range(R)])
    sh_ref = torch.zeros(R, NvS, H, dtype=torch.bfloat16)
    ws_ref = torch.zeros(R, NvS)
    outs = []
    for r in range(R):
        oo.dispatch(hid[r], wts[r], torch.from_numpy(plans[r].dst),
                    torch.from_numpy(plans[r].zero_fill_ranges), sh_ref, ws_ref, r, K, include_dups=True)
        # all ranks' routing given: the plan carries this rank's duplicate groups too
        outs.append(bufs[r].dispatch(hid[r].to(cuda), wts[r].to(cuda), topk.to(cuda), tpe.to(cuda),
                                     zero_copy=True, router_weights_zero_copy=True))
    torch.cuda.synchronize()
    for r in range(R):
        hidden_nvsh, w_nvs, cu, plan = outs[r]
        assert hidden_nvsh.data_ptr() == bufs[r].hidden_nvsh_buffer_view.data_ptr()
        assert w_nvs.data_ptr() == bufs[r].router_weight_buffer_view.data_ptr()
        assert torch.equal(hidden_nvsh.cpu().view(torch.int16), sh_ref[r].view(torch.int16))
        assert torch.equal(w_nvs.cpu().view(torch.int32), ws_ref[r].view(torch.int32))
        assert np.array_equal(plan.dst.cpu().numpy(), plans[r].dst)
        assert np.array_equal(cu.cpu().numpy(), plans[r].cu_seqlens)
        assert np.array_equal(plan.experts_to_copy.cpu().numpy(), gp.experts_to_copy)
        assert np.array_equal(plan.zero_fill_ranges.cpu().numpy(), plans[r].zero_fill_ranges)
        assert np.array_equal(plan.remote_stats.cpu().numpy(), plans[r].remote_stats)
        dg, dl, dc = po.dedup_structs(dst_all, r, S, K, NvS)
        ng, nd = (int(v) for v in plan.dup_counts.cpu())
        assert [ng, nd] == dc.tolist()
        assert np.array_equal(plan.dup_groups.cpu().numpy()[:ng], dg[:ng])
        assert np.array_equal(plan.dup_loffs.cpu().numpy()[:nd], dl[:nd])
    # "expert" = scale every row by a per-rank factor, in place on the shards
    for r in range(R):
        bufs[r].hidden_nvsh_buffer_view.mul_(1.0 + 0.25 * r)
        sh_ref[r] = (sh_ref[r].float() * (1.0 + 0.25 * r)).to(torch.bfloat16)
    torch.cuda.synchronize()
    for r in range(R):
        out, w_back, ev = bufs[r].combine(plan=outs[r][3], hidden_nvsh=outs[r][0],
                                          route_weights_nvs=outs[r][1], zero_copy=True,
                                          router_weights_zero_copy=True)
        assert ev is None
        want, want_w = oo.combine(sh_ref, ws_ref, torch.from_numpy(plans[r].dst), K, mode="two_level")
        assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
        assert torch.equal(w_back.cpu().view(torch.int32), wts[r].view(torch.int32))
        ref1, _ = oo.combine(sh_ref, None, torch.from_numpy(plans[r].dst), K, mode="all")
        err = (out.cpu().float() - ref1.float()).abs() / oo.bf16_ulp(ref1)
        assert float(err.max()) <= 1.5     # same-sign rows of one token: the reference's tolerance
    for b in bufs:
        b.destroy()


def test_sync_async_reuse_and_copy_modes_agree(cuda):
    topk, tpe = _routing(seed=22)
    rank = 2
    hid, w = _tokens(7)
    hid_d, w_d = hid.to(cuda), w.to(cuda)
    topk_d, tpe_d = topk[rank].contiguous().to(cuda), tpe.to(cuda)

    def fresh():
        b = Buffer(S, H, K, E, R, token_padding=TP, rank=rank)
        b._require_ctx()["hidden_buf"].zero_()
        b._require_ctx()["meta_buf"].zero_()
        return b

    b0 = fresh()
    h0, w0, cu0, p0 = b0.dispatch(hid_d, w_d, topk_d, tpe_d)
    assert h0.data_ptr() != b0.hidden_nvsh_buffer_view.data_ptr()
    assert cu0.shape == (2 * EPN,) and isinstance(p0, MoonEPCommPlan)
    o0, wb0, _ = b0.combine(plan=p0, hidden_nvsh=h0, route_weights_nvs=w0)
    torch.cuda.synchronize()

    # async on the comm stream
    b1 = fresh()
    h1, w1, cu1, p1, ev = b1.dispatch(hid_d, w_d, topk_d, tpe_d, async_finish=True)
    ev.synchronize()
    assert torch.equal(h1, h0) and torch.equal(w1, w0) and torch.equal(cu1, cu0)
    assert torch.equal(p1.dst, p0.dst)
    o1, wb1, ev = b1.combine(plan=p1, hidden_nvsh=h1, route_weights_nvs=w1, async_finish=True)
    ev.synchronize()
    assert torch.equal(o1, o0) and torch.equal(wb1, wb0)

    # plan reuse (the combine-backward path): no planning, no cu_seqlens, same rows
    snap = {f: getattr(p0, f).clone() for f in ("dst", "dup_groups", "dup_loffs", "dup_counts")}
    h2, w2, cu2, p2 = b0.dispatch(hid_d, None, plan=p0)
    torch.cuda.synchronize()
    assert cu2 is None and w2 is None and p2 is p0
    assert torch.equal(h2, h0)
    for f, v in snap.items():
        assert torch.equal(getattr(p0, f), v)
    # weights=None leaves the weight slots of the earlier dispatch alone
    assert torch.equal(b0.router_weight_buffer_view.clone(), w0)
    o2, wb2, _ = b0.combine(plan=p0, hidden_nvsh=h2)
    torch.cuda.synchronize()
    assert wb2 is None and torch.equal(o2, o0)

    # zero-copy views alias the shard; combine insists on exactly that view
    b3 = fresh()
    h3, w3, cu3, p3 = b3.dispatch(hid_d, w_d, topk_d, tpe_d, zero_copy=True,
                                  router_weights_zero_copy=True)
    torch.cuda.synchronize()
    assert torch.equal(h3, h0) and torch.equal(w3, w0)
    o3, wb3, _ = b3.combine(plan=p3, hidden_nvsh=h3, route_weights_nvs=w3, zero_copy=True,
                            router_weights_zero_copy=True)
    torch.cuda.synchronize()
    assert torch.equal(o3, o0) and torch.equal(wb3, wb0)
    with pytest.raises(AssertionError, match="must alias"):
        b3.combine(plan=p3, hidden_nvsh=h0.clone(), zero_copy=True)
    with pytest.raises(AssertionError, match="must alias"):
        b3.combine(plan=p3, hidden_nvsh=h3, route_weights_nvs=w0.clone(), zero_copy=True,
                   router_weights_zero_copy=True)
    for b in (b0, b1, b3):
        b.destroy()


def test_bad_inputs_raise_like_the_reference(cuda):
    topk, tpe = _routing(seed=23)
    b = Buffer(S, H, K, E, R, token_padding=TP, rank=0)
    hid, w = _tokens(8)
    hid_d, w_d, topk_d, tpe_d = hid.to(cuda), w.to(cuda), topk[0].contiguous().to(cuda), tpe.to(cuda)
    with pytest.raises(AssertionError):
        b.dispatch(hid_d, w_d)                                   # neither plan nor routing
    with pytest.raises(AssertionError):
        b.dispatch(hid_d, w_d, topk_d.long(), tpe_d)             # wrong dtype
    # one rank's counts only is the reference's call shape, but with nobody playing the other
    # ranks their rows of the gathered table would be stale: refused (rank threads do it,
    # tests/test_gpu_dropin_threads.py)
    with pytest.raises(NotImplementedError, match="host_threads=True"):
        b.dispatch(hid_d, w_d, topk_d, tpe_d[0].contiguous())
    with pytest.raises(AssertionError, match="hidden_sh"):
        b.dispatch(hid_d.float(), w_d, topk_d, tpe_d)
    with pytest.raises(AssertionError, match="hidden_sh"):
        b.dispatch(hid_d[:, :H // 2].contiguous(), w_d, topk_d, tpe_d)
    with pytest.raises(AssertionError, match="route_weights_sk"):
        b.dispatch(hid_d, w_d.double(), topk_d, tpe_d)
    h, wn, cu, plan = b.dispatch(hid_d, w_d, topk_d, tpe_d)
    with pytest.raises(AssertionError, match="plan is required"):
        b.combine(hidden_nvsh=h)
    with pytest.raises(AssertionError):
        b.combine(plan=plan, hidden_nvsh=h[:-1])
    with pytest.raises(AssertionError):
        b.combine(plan=plan, hidden_nvsh=h.float())
    with pytest.raises(TypeError):
        b.combine(plan=plan, hidden_nvsh=h, bogus=True)
    with pytest.raises(AssertionError, match="plan is required"):
        b.prefetch_weight()
    with pytest.raises(AssertionError, match="provided together"):
        b.prefetch_weight(plan=plan, local_gate_weight=torch.zeros(EPN, 128, 128, device=cuda))
    with pytest.raises(AssertionError, match="provided together"):
        b.reduce_grad(plan=plan)
    # a plan of another shape is rejected
    other = Buffer(S, H, K, E * 2, R, token_padding=TP, rank=0)
    _, _, _, plan2 = other.dispatch(hid_d, w_d, topk_d, torch.cat([tpe_d, tpe_d], 1).contiguous())
    with pytest.raises(AssertionError, match="zero_fill_ranges|plan"):
        b.dispatch(hid_d, plan=plan2)
    other.destroy()
    b.destroy()
    assert b.destroyed
    b.destroy()                                                  # idempotent
    with pytest.raises(AssertionError, match="has been destroyed"):
        b.dispatch(hid_d, plan=plan)
    with pytest.warns(ResourceWarning):
        leak = Buffer(S, H, K, E, R, token_padding=TP, rank=0, explicitly_destroy=True)
        leak.__del__()
    leak.destroy()


def test_prefetch_and_reduce_grad_through_the_api(cuda):
    topk, tpe = _routing(seed=24, sigma=2.0)
    gp, plans, dst_all = oracle_world_plan(topk.numpy(), tpe.numpy(), TP)
    assert (gp.experts_to_copy >= 0).any()
    Hw, Hp = 128, 256
    g = torch.Generator().manual_seed(3)
    locals_ = [[torch.randn(EPN, Hw, Hp, generator=g).to(torch.bfloat16) for _ in range(3)] for _ in range(R)]
    pools_ref = [torch.full((R, EPN, Hw, Hp), -123.0, dtype=torch.bfloat16) for _ in range(3)]
    pools = [p.to(cuda) for p in pools_ref]
    grads = [[torch.randn(EPN, Hw, Hp, generator=g) for _ in range(3)] for _ in range(R)]
    red0 = [torch.randn(R, EPN, Hw, Hp, generator=g) for _ in range(3)]
    etc = torch.from_numpy(gp.experts_to_copy.astype(np.int32))
    hid, w = _tokens(9)
    for r in range(R):
        b = Buffer(S, H, K, E, R, token_padding=TP, rank=r)
        _, _, _, plan = b.dispatch(hid.to(cuda), None, topk[r].contiguous().to(cuda), tpe.to(cuda))
        ev = b.prefetch_weight(plan=plan, async_finish=True,
                               local_gate_weight=locals_[r][0].to(cuda), local_up_weight=locals_[r][1].to(cuda),
                               local_down_weight=locals_[r][2].to(cuda), gate_prefetch_buffer=pools[0],
                               up_prefetch_buffer=pools[1], down_prefetch_buffer=pools[2])
        ev.synchronize()
        dg = [x.to(cuda) for x in grads[r]]
        dr = [x.to(cuda) for x in red0]
        assert b.reduce_grad(plan=plan, local_gate_grad=dg[0], local_up_grad=dg[1], local_down_grad=dg[2],
                             gate_reduce_buffer=dr[0], up_reduce_buffer=dr[1],
                             down_reduce_buffer=dr[2]) is None
        torch.cuda.synchronize()
        for t in range(3):
            oo.prefetch(locals_[r][t], pools_ref[t], etc, r)
            want_g, want_r = grads[r][t].clone(), red0[t].clone()
            oo.grad_reduce(want_g, want_r, etc, r)
            assert torch.equal(dg[t].cpu().view(torch.int32), want_g.view(torch.int32))
            assert torch.equal(dr[t].cpu().view(torch.int32), want_r.view(torch.int32))
        b.destroy()
    for t in range(3):
        assert torch.equal(pools[t].cpu().view(torch.int16), pools_ref[t].view(torch.int16))


def test_chain_replays_from_a_hip_graph(cuda):
    """plan -> dispatch -> combine captured once, replayed with fresh inputs in
    the same buffers and with eager work in between; every replay equals the
    eager result."""
    from moonep_amd.combine import launch_combine
    from moonep_amd.dispatch import launch_dispatch
    from moonep_amd.planning import allocate_planning_outputs, launch_planning

    rank = 1
    b = Buffer(S, H, K, E, R, token_padding=TP, rank=rank)
    ctx = b._require_ctx()
    ctx["hidden_buf"].zero_()
    topk_d = torch.empty(S * K, dtype=torch.int32, device=cuda)
    tpe_d = torch.empty(R, E, dtype=torch.int32, device=cuda)
    hid_d = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
    w_d = torch.empty(S, K, dtype=torch.float32, device=cuda)
    out = torch.empty(S, H, dtype=torch.bfloat16, device=cuda)
    out_w = torch.empty(S, K, dtype=torch.float32, device=cuda)
    plan, cu = allocate_planning_outputs(ctx)

    def chain():
        launch_planning(ctx, topk_d, tpe_d, cu, plan)
        launch_dispatch(ctx, hid_d, w_d, plan, build_dedup_map=False, write_dups=True)
        launch_combine(ctx, out, plan.dst, out_w, mode="two_level")

    def load(seed):
        topk, tpe = _routing(seed=seed, sigma=0.5 + seed % 3)
        hid, w = _tokens(seed)
        topk_d.copy_(topk[rank].reshape(-1)); tpe_d.copy_(tpe); hid_d.copy_(hid); w_d.copy_(w)

    load(40)
    chain()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()
    for seed in (41, 42, 43, 44):
        load(seed)
        ctx["hidden_buf"].zero_()
        chain()                                   # eager
        torch.cuda.synchronize()
        want = (out.clone(), out_w.clone(), plan.dst.clone(), cu.clone(), ctx["hidden_buf"].clone())
        out.zero_(); out_w.zero_(); plan.dst.zero_(); cu.zero_(); ctx["hidden_buf"].zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = (out, out_w, plan.dst, cu, ctx["hidden_buf"])
        for a, g in zip(want, got):
            assert torch.equal(a, g), seed
    b.destroy()


def test_single_rank_group(cuda):
    """R = 1: one rank is its own group; the [E]-shaped count vector of the
    reference signature is accepted as is."""
    S1, H1, K1, E1 = 20, 64, 2, 4
    topk = routing.popularity_biased(S1, K1, E1, 1, 0, 1.0, seed=2)
    tpe = routing.tokens_per_expert(topk, E1)
    g = torch.Generator().manual_seed(2)
    hid = torch.randn(S1, H1, generator=g).to(torch.bfloat16)
    b = Buffer(S1, H1, K1, E1, 1, token_padding=4)
    assert b._require_ctx()["rank"] == 0
    h, w, cu, plan = b.dispatch(hid.to(cuda), None, topk.to(cuda), tpe.to(cuda))
    out, _, _ = b.combine(plan=plan, hidden_nvsh=h)
    torch.cuda.synchronize()
    rp = po.plan(topk.numpy(), tpe.numpy().reshape(1, E1), 0, 4)
    assert np.array_equal(plan.dst.cpu().numpy(), rp.dst)
    assert (plan.experts_to_copy.cpu() == -1).all()
    NvS = b._require_ctx()["NvS"]
    sh = torch.zeros(1, NvS, H1, dtype=torch.bfloat16)
    oo.dispatch(hid, None, torch.from_numpy(rp.dst), torch.from_numpy(rp.zero_fill_ranges), sh, None, 0, K1,
                include_dups=True)
    want, _ = oo.combine(sh, None, torch.from_numpy(rp.dst), K1, mode="two_level")
    assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
    b.destroy()
