"""Several ranks on ONE host thread and one shared EmulatedWorld: the calls that would
silently give wrong results there are refused, the ways that work give the oracle's
bits; and the compute-unit bound of the standalone duplicate kernels
(MOONEP_NUM_SMS_DEDUP, reference moonep/api.py:100-120) changes no result."""

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, EmulatedWorld, routing
from moonep_amd.combine import launch_combine_prologue
from moonep_amd.dispatch import dup_cu_bound, launch_dispatch_epilogue
from oracle import ops_oracle as oo
from tests.util import oracle_world_plan

pytestmark = pytest.mark.gpu

S, H, K, E, R, TP = 96, 256, 4, 16, 4, 8
EPN = E // R


def _world_of_buffers(cuda, sigma=2.0, seed=31, pattern=None):
    if pattern is None:
        topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed=seed) for r in range(R)])
    else:
        topk = torch.stack([routing.pattern(pattern, S, K, E, R, r) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    world = EmulatedWorld(S, H, K, E, R, TP)
    bufs = [Buffer(S, H, K, E, R, token_padding=TP, rank=r, world=world) for r in range(R)]
    return topk, tpe, world, bufs


def test_reduce_grad_of_several_ranks_on_one_thread(cuda):
    """reduce_grad in one piece zeroes this rank's slots, which hold OTHER ranks' experts,
    before their owners have summed them (the reference has a barrier there,
    moonep/grad_reduce.py:369-372): refused on a shared world; the two phases give
    what all-read-then-all-clear gives."""
    topk, tpe, world, bufs = _world_of_buffers(cuda)
    gp, plans, _ = oracle_world_plan(topk.numpy(), tpe.numpy(), TP)
    etc = torch.from_numpy(gp.experts_to_copy.astype(np.int32))
    assert (etc >= 0).any()
    g = torch.Generator().manual_seed(4)
    hid = torch.randn(S, H, generator=g).to(torch.bfloat16).to(cuda)
    dplans = []
    for r in range(R):
        _, _, _, plan = bufs[r].dispatch(hid, None, topk.to(cuda), tpe.to(cuda), zero_copy=True)
        dplans.append(plan)
    Hw, Hp = 128, 128
    grads = [[torch.randn(EPN, Hw, Hp, generator=g) for _ in range(3)] for _ in range(R)]
    red0 = [torch.randn(R, EPN, Hw, Hp, generator=g) for _ in range(3)]
    dgr = [[x.to(cuda) for x in grads[r]] for r in range(R)]
    dre = [x.to(cuda) for x in red0]           # ONE set of reduce buffers for all ranks

    def call(r, **kw):
        return bufs[r].reduce_grad(plan=dplans[r], local_gate_grad=dgr[r][0], local_up_grad=dgr[r][1],
                                   local_down_grad=dgr[r][2], gate_reduce_buffer=dre[0],
                                   up_reduce_buffer=dre[1], down_reduce_buffer=dre[2], **kw)

    with pytest.raises(AssertionError, match='phase="reduce"'):
        call(0)
    with pytest.raises(AssertionError, match="phase must be"):
        call(0, phase="sum")
    torch.cuda.synchronize()
    for t in range(3):   # the refused call launched nothing
        assert torch.equal(dre[t].cpu(), red0[t]) and torch.equal(dgr[0][t].cpu(), grads[0][t])
    for r in range(R):
        call(r, phase="reduce")
    for r in range(R):
        call(r, phase="clear")
    torch.cuda.synchronize()
    for t in range(3):
        cleared = red0[t].clone()
        for r in range(R):
            want_g, scratch = grads[r][t].clone(), red0[t].clone()   # every rank sums the untouched slots
            oo.grad_reduce(want_g, scratch, etc, r)
            assert torch.equal(dgr[r][t].cpu().view(torch.int32), want_g.view(torch.int32)), (t, r)
            oo.grad_reduce(torch.zeros(EPN, Hw, Hp), cleared, etc, r)   # ... and all clears happen
        assert torch.equal(dre[t].cpu().view(torch.int32), cleared.view(torch.int32)), t
    for b in bufs:
        b.destroy()


def test_per_rank_counts_from_one_thread_are_refused(cuda):
    """tokens_per_expert[E] of one rank is only a plan input beside the other ranks' rows;
    nobody fills those when one thread drives the Buffer."""
    topk, tpe, world, bufs = _world_of_buffers(cuda)
    hid = torch.zeros(S, H, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(NotImplementedError, match=r"tokens_per_expert\[R=4, E=16\]"):
        bufs[1].dispatch(hid, None, topk[1].contiguous().to(cuda), tpe[1].contiguous().to(cuda),
                         zero_copy=True)
    lone = Buffer(S, H, K, E, R, token_padding=TP, rank=2)     # a world of its own: the same
    with pytest.raises(NotImplementedError, match="host_threads=True"):
        lone.dispatch(hid, None, topk[2].contiguous().to(cuda), tpe[2].contiguous().to(cuda))
    # the gathered table works from one thread
    _, _, cu, plan = lone.dispatch(hid, None, topk[2].contiguous().to(cuda), tpe.to(cuda))
    gp, plans, _ = oracle_world_plan(topk.numpy(), tpe.numpy(), TP)
    assert np.array_equal(plan.dst.cpu().numpy(), plans[2].dst)
    lone.destroy()
    for b in bufs:
        b.destroy()


@pytest.mark.parametrize("pattern", ["duplicate_topk", "all_local"])
def test_duplicate_kernels_give_the_same_bits_under_a_cu_bound(cuda, pattern):
    topk, tpe, world, bufs = _world_of_buffers(cuda, pattern=pattern)
    g = torch.Generator().manual_seed(8)
    NvS = world.NvS
    rows = (torch.randn(R * NvS, H, generator=g) * 2).to(torch.bfloat16).to(cuda)
    hid = torch.randn(S, H, generator=g).to(torch.bfloat16).to(cuda)
    plans = []
    for r in range(R):
        _, _, _, plan = bufs[r].dispatch(hid, None, topk.to(cuda), tpe.to(cuda), zero_copy=True)
        plans.append(plan)
    torch.cuda.synchronize()
    assert sum(int(p.dup_counts[0]) for p in plans) > 0, "the routing must produce duplicate groups"
    max_cus = int(bufs[0]._require_ctx()["max_sms"])
    results = {}
    for bound in (max_cus, 1, 32):
        outs = []
        for kernel in (launch_dispatch_epilogue, launch_combine_prologue):
            world.hidden_buf.copy_(rows)
            for r in range(R):
                ctx = bufs[r]._require_ctx()
                ctx["num_sms_dedup"] = bound
                assert dup_cu_bound(ctx) == (0 if bound == max_cus else bound)
                kernel(ctx, plans[r])
            torch.cuda.synchronize()
            outs.append(world.hidden_buf.clone())
        results[bound] = outs
    for bound in (1, 32):
        for a, b in zip(results[max_cus], results[bound]):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), bound
    assert not torch.equal(results[max_cus][0].view(torch.int16), rows.view(torch.int16)), "epilogue copied rows"
    for b in bufs:
        b.destroy()


def test_env_bound_reaches_the_context(cuda, monkeypatch):
    monkeypatch.setenv("MOONEP_NUM_SMS_DEDUP", "24")
    buf = Buffer(S, H, K, E, R, token_padding=TP, rank=0)
    assert dup_cu_bound(buf._require_ctx()) == 24
    buf.destroy()
    monkeypatch.delenv("MOONEP_NUM_SMS_DEDUP")
    buf = Buffer(S, H, K, E, R, token_padding=TP, rank=0)
    assert dup_cu_bound(buf._require_ctx()) == 0          # all CUs: no bound
    buf.destroy()
