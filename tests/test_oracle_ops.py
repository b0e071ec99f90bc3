"""Pins the CPU oracles of the data-movement ops (no GPU): the torch
restatement (oracle/ops_oracle.py) against the independent scalar C
restatement (oracle/mep_oracle.c) and against closed forms."""

import numpy as np
import pytest
import torch

from moonep_amd import routing
from oracle import c_oracle as co
from oracle import ops_oracle as oo
from oracle import planner_oracle as po
from tests.util import oracle_world_plan, traceable_hidden, traceable_weights


def _u16(t):
    return t.view(torch.int16).numpy().view(np.uint16)


def _world(S, H, K, epn, R, tp, sigma=1.0, seed=11):
    E = epn * R
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    gp, plans, dst_all = oracle_world_plan(topk.numpy(), tpe.numpy(), tp)
    return gp, plans, dst_all


@pytest.mark.parametrize("S,H,K,epn,R,tp", [(17, 24, 3, 3, 4, 16), (32, 64, 8, 2, 8, 8), (9, 8, 1, 4, 2, 4)])
def test_dispatch_and_combine_torch_vs_c(S, H, K, epn, R, tp):
    gp, plans, dst_all = _world(S, H, K, epn, R, tp)
    NvS = gp.NvS
    for dups in (False, True):
        sh_t = torch.full((R, NvS, H), 7.0, dtype=torch.bfloat16)
        ws_t = torch.full((R, NvS), 3.0)
        sh_c = _u16(sh_t.clone()).copy()
        ws_c = ws_t.numpy().copy()
        for r in range(R):
            hid, w = traceable_hidden(S, H, r), traceable_weights(S, K, r)
            zf = torch.from_numpy(plans[r].zero_fill_ranges)
            oo.dispatch(hid, w, torch.from_numpy(plans[r].dst), zf, sh_t, ws_t, r, K, include_dups=dups)
            co.dispatch(_u16(hid).copy(), w.numpy().copy(), plans[r].dst, plans[r].zero_fill_ranges,
                        sh_c, ws_c, r, K, NvS, dups)
        assert np.array_equal(_u16(sh_t), sh_c)
        assert np.array_equal(ws_t.numpy().view(np.int32), ws_c.view(np.int32))
    # traceable payload: every entry's row names its source token and rank
    for r in range(R):
        _, drank, loff, _ = po.decode_dst(plans[r].dst, NvS)
        rows = _u16(sh_t)[drank, loff]
        assert np.array_equal(rows[:, 0], np.repeat(np.arange(S), K) & 0x7F7F)
        if H > 1:
            assert (rows[:, 1] == r).all()
    g = torch.Generator().manual_seed(1)
    vals = (torch.randn(R, NvS, H, generator=g) * 2).to(torch.bfloat16)
    for r in range(R):
        dst = plans[r].dst
        for mode_i, mode in enumerate(("primaries", "all", "two_level")):
            out_t, w_t = oo.combine(vals, ws_t, torch.from_numpy(dst), K, mode=mode)
            out_c, w_c = co.combine(_u16(vals).copy(), ws_t.numpy().copy(), dst, S, K, NvS, mode_i)
            assert np.array_equal(_u16(out_t), out_c), (r, mode)
            assert np.array_equal(w_t.numpy().view(np.int32), w_c.view(np.int32))


def test_two_level_equals_prologue_then_primaries():
    S, H, K, epn, R, tp = 24, 40, 6, 2, 4, 8
    gp, plans, dst_all = _world(S, H, K, epn, R, tp, sigma=2.0)
    NvS = gp.NvS
    g = torch.Generator().manual_seed(2)
    vals = (torch.randn(R, NvS, H, generator=g) * 5).to(torch.bfloat16)
    pre = vals.clone()
    ndup = 0
    for r in range(R):
        dg, dl, dc = po.dedup_structs(dst_all, r, S, K, NvS)
        ndup += int(dc[1])
        oo.combine_prologue(pre[r], dg, dl, dc)
    assert ndup > 0
    for r in range(R):
        dst = torch.from_numpy(plans[r].dst)
        a, _ = oo.combine(pre, None, dst, K, mode="primaries")
        b, _ = oo.combine(vals, None, dst, K, mode="two_level")
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_combine_closed_forms():
    S, H, K, epn, R, tp = 16, 32, 4, 2, 4, 8
    gp, plans, dst_all = _world(S, H, K, epn, R, tp)
    NvS = gp.NvS
    dst = torch.from_numpy(plans[2].dst)
    ones = torch.ones(R, NvS, H, dtype=torch.bfloat16)
    for mode in ("all", "two_level"):
        out, _ = oo.combine(ones, None, dst, K, mode=mode)
        assert (out == K).all()
    # small integers: every partial sum is exact, all modes equal the plain sum
    g = torch.Generator().manual_seed(3)
    ints = torch.randint(-8, 9, (R, NvS, H), generator=g).to(torch.bfloat16)
    drank, loff, _ = oo.decode(dst, NvS)
    want = ints.view(-1, H)[drank * NvS + loff].float().view(S, K, H).sum(1).to(torch.bfloat16)
    for mode in ("all", "two_level"):
        out, _ = oo.combine(ints, None, dst, K, mode=mode)
        assert torch.equal(out, want)
    # weighted mode: power-of-two weights and small integers keep every product and
    # partial sum exact, so the result is the plain weighted sum; weight 1 reduces to "all"
    w2 = (2.0 ** torch.randint(-3, 3, (R, NvS), generator=g).float())
    wk = w2.view(-1)[drank * NvS + loff].view(S, K, 1)
    want_w = (ints.view(-1, H)[drank * NvS + loff].float().view(S, K, H) * wk).sum(1)
    out, _ = oo.combine(ints, w2, dst, K, mode="weighted")
    assert torch.equal(out, want_w.to(torch.bfloat16))
    rnd = torch.randn(R, NvS, H, generator=g).to(torch.bfloat16)
    a, _ = oo.combine(rnd, torch.ones(R, NvS), dst, K, mode="weighted")
    b, _ = oo.combine(rnd, None, dst, K, mode="all")
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # dispatch then combine returns K * token (up to the rounding of the sum)
    hid = (torch.randn(S, H, generator=g)).to(torch.bfloat16)
    sh = torch.zeros(R, NvS, H, dtype=torch.bfloat16)
    oo.dispatch(hid, None, dst, torch.from_numpy(plans[2].zero_fill_ranges), sh, None, 2, K,
                include_dups=True)
    out, _ = oo.combine(sh, None, dst, K, mode="all")
    ref = (hid.float() * K).to(torch.bfloat16)
    assert float(((out.float() - ref.float()).abs() / oo.bf16_ulp(ref)).max()) <= 1.5


def test_bf16_rounding_of_c_oracle_is_round_to_nearest_even():
    S, H, K, NvS = 1, 8, 2, 4
    # two rows whose fp32 sum falls exactly between two bf16 values
    a = torch.tensor([1.0, 1.0, 256.0, -1.0, 3.0, 0.5, 1e30, 0.0])
    b = torch.tensor([2.0 ** -8, 3 * 2.0 ** -8, 1.0, -(2.0 ** -8), 2.0 ** -7, 2.0 ** -9, 1e30, -0.0])
    sh = torch.zeros(1, NvS, H, dtype=torch.bfloat16)
    sh[0, 0], sh[0, 1] = a.to(torch.bfloat16), b.to(torch.bfloat16)
    dst = np.array([0, -1 - 1], dtype=np.int32)  # second entry is a duplicate on the same rank
    want = (sh[0, 0].float() + sh[0, 1].float()).to(torch.bfloat16)
    out_c, _ = co.combine(_u16(sh).copy(), None, dst, S, K, NvS, 1)
    assert np.array_equal(out_c[0], _u16(want))
    out_t, _ = oo.combine(sh, None, torch.from_numpy(dst), K, mode="all")
    assert torch.equal(out_t[0].view(torch.int16), want.view(torch.int16))


def test_prefetch_and_grad_reduce_torch_vs_c():
    R, epn, n = 4, 6, 40
    g = torch.Generator().manual_seed(4)
    live = torch.rand((R, epn), generator=g) < 0.7
    etc = torch.where(live, torch.randint(0, R * epn, (R, epn), generator=g, dtype=torch.int32),
                      torch.full((R, epn), -1, dtype=torch.int32))
    for rank in range(R):
        local = torch.randint(0, 255, (epn, n), generator=g, dtype=torch.int32).to(torch.uint8)
        pool_t = torch.full((R, epn, n), 0xAB, dtype=torch.uint8)
        pool_c = pool_t.numpy().copy()
        oo.prefetch(local, pool_t, etc, rank)
        co.prefetch(local.numpy().copy(), pool_c, etc.numpy(), rank)
        assert np.array_equal(pool_t.numpy(), pool_c)
        for d in range(R):
            for b in range(epn):
                e = int(etc[d, b])
                if rank * epn <= e < (rank + 1) * epn:
                    assert torch.equal(pool_t[d, b], local[e - rank * epn])
                else:
                    assert (pool_t[d, b] == 0xAB).all()
        grad_t = torch.randn(epn, n, generator=g)
        red_t = torch.randn(R, epn, n, generator=g)
        grad_c, red_c = grad_t.numpy().copy(), red_t.numpy().copy()
        oo.grad_reduce(grad_t, red_t, etc, rank)
        co.grad_reduce(grad_c, red_c, etc.numpy(), rank)
        assert np.array_equal(grad_t.numpy().view(np.int32), grad_c.view(np.int32))
        assert np.array_equal(red_t.numpy().view(np.int32), red_c.view(np.int32))


def test_grad_reduce_order_is_observable():
    """fp32 addition does not associate: a different slot order changes bits,
    so the bit-exact GPU test really pins the (src, slot)-ascending order."""
    R, epn, n = 4, 2, 4096
    etc = torch.tensor([[1, -1], [1, -1], [1, -1], [1, -1]], dtype=torch.int32)  # expert 1 of rank 0
    g = torch.Generator().manual_seed(6)
    red = torch.randn(R, epn, n, generator=g) * torch.tensor([1e4, 1.0, 1e-4, 1e2]).view(R, 1, 1)
    grad = torch.randn(epn, n, generator=g)
    fwd = grad.clone()
    oo.grad_reduce(fwd, red.clone(), etc, 0)
    rev = grad[1].clone()
    for src in reversed(range(R)):
        rev += red[src, 0]
    assert not torch.equal(fwd[1], rev)
    assert torch.equal(fwd[0], grad[0])
