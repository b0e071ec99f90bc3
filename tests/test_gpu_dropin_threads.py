"""The reference's own per-rank call sequence (reference tests/test_e2e.py:199-340),
unchanged: every rank passes ITS ``topk_experts_sk[S, K]`` and ITS
``tokens_per_expert[E]``.  R host threads, one per rank, drive R Buffers on one
EmulatedWorld(host_threads=True); the world's rendezvous stand in for the
reference's cross-rank barriers.  Everything is checked against the oracle,
including the fresh plan's duplicate groups, and against the closed forms the
reference test uses for prefetch and reduce_grad.

Also here: what one host thread may and may not do with several Buffers on one
world (copy-out needs zero_copy; a plan made from one rank's routing has no
duplicate map)."""

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, EmulatedWorld, MoonEPCommPlan, routing
from moonep_amd.api import launch_combine_prologue, launch_dispatch_epilogue
from oracle import ops_oracle as oo
from oracle import planner_oracle as po
from tests.util import oracle_world_plan

pytestmark = pytest.mark.gpu

S, H, K, R, EPN, TP, HP = 256, 1024, 4, 4, 8, 128, 128
E = R * EPN


def _inputs(rank):
    g = torch.Generator().manual_seed(1234 + rank)
    hidden = torch.randn(S, H, generator=g).to(torch.bfloat16)
    weights = torch.rand(S, K, generator=g)
    topk = routing.popularity_biased(S, K, E, R, rank, 1.5, seed=5)
    return hidden, weights, topk, routing.tokens_per_expert(topk, E)


def _weight_base(rank, off):
    """bf16-exact values naming (rank, local expert, projection)."""
    le = torch.arange(EPN, dtype=torch.float32)[:, None, None]
    col = (torch.arange(HP) % 8).to(torch.float32)[None, None, :]
    return (rank * 64 + le * 4 + off + col / 8).expand(EPN, H, HP).to(torch.bfloat16).contiguous()


def test_reference_call_sequence_on_rank_threads(cuda):
    world = EmulatedWorld(S, H, K, E, R, TP, host_threads=True)
    world.hidden_buf.zero_()
    NvS = world.NvS
    # symmetric memory of the group: every rank sees the same pools
    pre_pools = [torch.full((R, EPN, H, HP), -1.0, dtype=torch.bfloat16, device=cuda) for _ in range(3)]
    red_pools = [torch.zeros(R, EPN, H, HP, dtype=torch.float32, device=cuda) for _ in range(3)]
    for t in range(3):      # slot (r, b) holds r*100 + b + t/4 everywhere: sums are exact in fp32
        v = (torch.arange(R)[:, None] * 100 + torch.arange(EPN)[None, :]).float() + t / 4
        red_pools[t].copy_(v[:, :, None, None].expand(R, EPN, H, HP))
    torch.cuda.synchronize()
    inputs = [_inputs(r) for r in range(R)]

    def per_rank(rank):
        hidden, weights, topk, tpe = (x.to(cuda) for x in inputs[rank])
        assert tuple(topk.shape) == (S, K) and tuple(tpe.shape) == (E,)
        buffer = Buffer(S, H, K, E, R, num_sms=32, token_padding=TP, rank=rank, world=world)
        out = {}
        # --- sync
        h_sync, w_sync, cu_sync, plan_sync = buffer.dispatch(hidden, weights, topk, tpe)
        assert isinstance(plan_sync, MoonEPCommPlan)
        h_sync_c, w_sync_c, cu_sync_c = h_sync.clone(), w_sync.clone(), cu_sync.clone()
        snap = plan_sync.clone()
        local_w = [_weight_base(rank, t).to(cuda) for t in range(3)]
        buffer.prefetch_weight(plan=snap, local_gate_weight=local_w[0], local_up_weight=local_w[1],
                               local_down_weight=local_w[2], gate_prefetch_buffer=pre_pools[0],
                               up_prefetch_buffer=pre_pools[1], down_prefetch_buffer=pre_pools[2])
        # --- async, fresh plan
        h_a, w_a, cu_a, plan_a, ev = buffer.dispatch(hidden, weights, topk, tpe, async_finish=True)
        ev.wait(torch.cuda.current_stream())
        assert torch.equal(h_sync_c, h_a) and torch.equal(w_sync_c, w_a) and torch.equal(cu_sync_c, cu_a)
        for name in ("dst", "experts_to_copy", "zero_fill_ranges", "remote_stats", "dup_counts"):
            assert torch.equal(getattr(snap, name), getattr(plan_a, name)), name
        # --- plan reuse: planning skipped, dedup fields untouched, no weights, no cu
        before = [t.clone() for t in (snap.dup_groups, snap.dup_loffs, snap.dup_counts)]
        h_r, w_r, cu_r, plan_r = buffer.dispatch(hidden, plan=snap)
        assert w_r is None and cu_r is None and plan_r is snap
        assert torch.equal(h_r, h_sync_c)
        for a, b in zip(before, (snap.dup_groups, snap.dup_loffs, snap.dup_counts)):
            assert torch.equal(a, b)
        # --- combine of the dispatched rows (identity "experts"), without and with weights
        h_c, w_c, _, _ = buffer.dispatch(hidden, weights, topk, tpe)
        out_plain, none_w, _ = buffer.combine(plan=snap, hidden_nvsh=h_c)
        assert none_w is None
        h_c, w_c, _, _ = buffer.dispatch(hidden, weights, topk, tpe)
        out_w, gathered, _ = buffer.combine(plan=snap, hidden_nvsh=h_c, route_weights_nvs=w_c)
        assert torch.equal(out_plain, out_w)
        assert torch.equal(gathered, weights)
        # --- zero copy round trip gives the same bits
        h_z, w_z, _, plan_z = buffer.dispatch(hidden, weights, topk, tpe, zero_copy=True,
                                              router_weights_zero_copy=True)
        assert h_z.data_ptr() == buffer._require_ctx()["hidden_buf_local"].data_ptr()
        assert torch.equal(h_z, h_c) and torch.equal(w_z, w_c)
        out_z, gathered_z, _ = buffer.combine(plan=plan_z, hidden_nvsh=h_z, route_weights_nvs=w_z,
                                              zero_copy=True, router_weights_zero_copy=True)
        assert torch.equal(out_z, out_w) and torch.equal(gathered_z, weights)
        # --- reduce_grad on the group's shared pools
        grads = [torch.full((EPN, H, HP), float(rank + 1), device=cuda) for _ in range(3)]
        buffer.reduce_grad(plan=snap, local_gate_grad=grads[0], local_up_grad=grads[1],
                           local_down_grad=grads[2], gate_reduce_buffer=red_pools[0],
                           up_reduce_buffer=red_pools[1], down_reduce_buffer=red_pools[2])
        torch.cuda.synchronize()
        out.update(h=h_sync_c.cpu(), w=w_sync_c.cpu(), cu=cu_sync_c.cpu(), plan=snap, combined=out_w.cpu(),
                   grads=[g_[:, 0, 0].cpu() for g_ in grads], grads_flat=all(
                       bool((g_ == g_[:, :1, :1]).all()) for g_ in grads))
        buffer.destroy()
        return out

    res = world.run_ranks(per_rank)
    torch.cuda.synchronize()

    # ---------------- oracle of the whole group
    topk_all = torch.stack([inputs[r][2] for r in range(R)])
    tpe_all = torch.stack([inputs[r][3] for r in range(R)])
    gp, plans, dst_all = oracle_world_plan(topk_all.numpy(), tpe_all.numpy(), TP)
    assert gp.NvS == NvS
    sh_ref = torch.zeros(R, NvS, H, dtype=torch.bfloat16)
    ws_ref = torch.zeros(R, NvS)
    for r in range(R):
        oo.dispatch(inputs[r][0], inputs[r][1], torch.from_numpy(plans[r].dst),
                    torch.from_numpy(plans[r].zero_fill_ranges), sh_ref, ws_ref, r, K, include_dups=True)
    etc = gp.experts_to_copy
    for r in range(R):
        plan = res[r]["plan"]
        assert np.array_equal(plan.dst.cpu().numpy(), plans[r].dst), f"rank {r} dst"
        assert np.array_equal(res[r]["cu"].numpy(), plans[r].cu_seqlens)
        assert np.array_equal(plan.experts_to_copy.cpu().numpy(), etc)
        assert np.array_equal(plan.zero_fill_ranges.cpu().numpy(), plans[r].zero_fill_ranges)
        assert np.array_equal(plan.remote_stats.cpu().numpy(), plans[r].remote_stats)
        # the copied-out shard holds EVERY rank's rows for this destination
        used = int(plans[r].cu_seqlens[-1])
        assert torch.equal(res[r]["h"][:used].view(torch.int16), sh_ref[r, :used].view(torch.int16))
        assert torch.equal(res[r]["w"][:used].view(torch.int32), ws_ref[r, :used].view(torch.int32))
        # fresh plan: duplicate groups of this destination from all ranks' dst
        dg, dl, dc = po.dedup_structs(dst_all, r, S, K, NvS)
        ng, nd = (int(v) for v in plan.dup_counts.cpu())
        assert [ng, nd] == dc.tolist() and ng > 0
        assert np.array_equal(plan.dup_groups.cpu().numpy()[:ng], dg[:ng])
        assert np.array_equal(plan.dup_loffs.cpu().numpy()[:nd], dl[:nd])
        want, _ = oo.combine(sh_ref, None, torch.from_numpy(plans[r].dst), K, mode="two_level")
        assert torch.equal(res[r]["combined"].view(torch.int16), want.view(torch.int16))
    # prefetch: pool[d, b] == owner's expert; untouched elsewhere
    for t in range(3):
        pool = pre_pools[t].cpu()
        for d in range(R):
            for b in range(EPN):
                e = int(etc[d, b])
                if e < 0:
                    assert bool((pool[d, b] == -1.0).all())
                else:
                    assert torch.equal(pool[d, b], _weight_base(e // EPN, t)[e % EPN])
    # reduce_grad: every owner summed EVERY slot holding its experts before anyone cleared
    for r in range(R):
        assert res[r]["grads_flat"]
        for t in range(3):
            want = torch.full((EPN,), float(r + 1))
            for src in range(R):
                for b in range(EPN):
                    e = int(etc[src, b])
                    if e // EPN == r and e >= 0:
                        want[e % EPN] += src * 100 + b + t / 4
            assert torch.equal(res[r]["grads"][t], want), (r, t)
    for t in range(3):
        pool = red_pools[t].cpu()
        for d in range(R):
            for b in range(EPN):
                if int(etc[d, b]) >= 0:
                    assert not bool(pool[d, b].any())
                else:
                    assert bool((pool[d, b] == d * 100 + b + t / 4).all())
    assert int((etc >= 0).sum()) > 0      # the routing really makes remote experts


def test_a_failing_rank_does_not_hang_the_others(cuda):
    world = EmulatedWorld(S, H, K, E, R, TP, host_threads=True)

    def per_rank(rank):
        if rank == 1:
            raise ValueError("rank 1 gives up")
        world.rendezvous(rank)

    with pytest.raises(ValueError, match="rank 1 gives up"):
        world.run_ranks(per_rank, timeout=30.0)


def test_one_thread_and_several_buffers(cuda):
    world = EmulatedWorld(S, H, K, E, R, TP)
    world.hidden_buf.zero_()
    bufs = [Buffer(S, H, K, E, R, token_padding=TP, rank=r, world=world) for r in range(R)]
    inputs = [_inputs(r) for r in range(R)]
    tpe_all = torch.stack([inputs[r][3] for r in range(R)]).to(cuda)
    hidden, weights, topk, _ = (x.to(cuda) for x in inputs[0])
    # a copy-out right after rank 0's dispatch would miss the other ranks' rows
    with pytest.raises(AssertionError, match="zero_copy=True"):
        bufs[0].dispatch(hidden, weights, topk, tpe_all)
    h, w, cu, plan = bufs[0].dispatch(hidden, weights, topk, tpe_all, zero_copy=True,
                                      router_weights_zero_copy=True)
    with pytest.raises(AssertionError, match="zero_copy=True"):
        bufs[0].combine(plan=plan, hidden_nvsh=h.clone())
    # planned from rank 0's routing alone: no duplicate map, and the kernels that need one say so
    with pytest.raises(AssertionError, match="no duplicate map"):
        launch_dispatch_epilogue(bufs[0]._require_ctx(), plan)
    with pytest.raises(AssertionError, match="no duplicate map"):
        launch_combine_prologue(bufs[0]._require_ctx(), plan)
    out, _, _ = bufs[0].combine(plan=plan, hidden_nvsh=h, zero_copy=True)   # the fused path needs none
    torch.cuda.synchronize()
    gp, plans, _ = oracle_world_plan(torch.stack([i[2] for i in inputs]).numpy(), tpe_all.cpu().numpy(), TP)
    assert np.array_equal(plan.dst.cpu().numpy(), plans[0].dst)
    for b in bufs:
        b.destroy()
    assert world.attached == 0
