"""prefetch_weight (owner push) and reduce_grad kernels vs the CPU oracle.
Pure copies and an fp32 sum in a fixed order: everything bit-exact.

Plans and data follow the ideas of reference tests/test_prefetch.py and
tests/test_grad_reduce.py: hand-made experts_to_copy tables with holes,
duplicates, self-sends, high fan-in and empty plans; sentinels in unused slots
and in the padding between ranks must survive; affine data (exact under any
add order) and random data (pins the (src rank, slot)-ascending order).
"""

import pytest
import torch

from moonep_amd.grad_reduce import launch_grad_reduce
from moonep_amd.prefetch import (launch_prefetch, launch_prefetch_pull, prefetch_retile_nbytes,
                                 retile_for_prefetch)
from oracle import ops_oracle as oo

pytestmark = pytest.mark.gpu

SENTINEL = -123.0


# ---------------------------------------------------------------- plans
def plan_ring(R, epn, seed=0):
    p = torch.full((R, epn), -1, dtype=torch.int32)
    for src in range(R):
        p[src, 0] = ((src + 1) % R) * epn + (src % epn)
        if epn > 1:
            p[src, 1] = ((src + 2) % R) * epn + ((src + 1) % epn)
        if epn > 2:
            p[src, 2] = ((src + R - 1) % R) * epn + ((src + 2) % epn)
        if epn > 3:
            p[src, 3] = ((src + 1) % R) * epn + (epn - 1 - (src % epn))
    return p


def plan_fan_in(R, epn, seed=0):
    """one expert per owner receives 2 slots from every rank (self-sends and
    same-source duplicates included)"""
    assert 2 * R <= epn
    p = torch.full((R, epn), -1, dtype=torch.int32)
    for owner in range(R):
        e = owner * epn + (owner % epn)
        for src in range(R):
            p[src, 2 * owner] = e
            p[src, 2 * owner + 1] = e
    return p


def plan_empty(R, epn, seed=0):
    return torch.full((R, epn), -1, dtype=torch.int32)


def plan_asymmetric(R, epn, seed=0):
    p = torch.full((R, epn), -1, dtype=torch.int32)
    for src in range(R):
        if src == 1:
            continue
        owner = src + 1 if src + 1 < R else 1
        p[src, 0] = owner * epn + (src % epn)
        if epn > 1:
            p[src, 1] = owner * epn + ((src + 1) % epn)
    return p


def plan_random(R, epn, seed=0):
    g = torch.Generator().manual_seed(seed)
    live = torch.rand((R, epn), generator=g) < 0.6
    ids = torch.randint(0, R * epn, (R, epn), generator=g, dtype=torch.int32)
    return torch.where(live, ids, torch.full_like(ids, -1))


PLANS = {"ring": plan_ring, "fan_in": plan_fan_in, "empty": plan_empty,
         "asymmetric": plan_asymmetric, "random": plan_random}


def strided_pool(R, per_rank_shape, dtype, pad_elems, fill, dev, lead_elems=0):
    """[R, *per_rank_shape] view with `pad_elems` elements of padding between
    ranks and `lead_elems` before the first, everything (padding included)
    pre-filled with `fill`."""
    numel = 1
    for s in per_rank_shape:
        numel *= s
    stride = numel + pad_elems
    backing = torch.full((lead_elems + R * stride,), fill, dtype=dtype, device=dev)
    backing = backing[lead_elems:]
    strides = [stride]
    acc = numel
    for s in per_rank_shape:
        acc //= s
        strides.append(acc)
    return backing, backing.as_strided((R, *per_rank_shape), strides)


# ---------------------------------------------------------------- prefetch
PREFETCH_CASES = [
    # name, R, epn, H, Hp, dtype, plan, seed, pad_elems
    ("single_tile", 4, 2, 128, 128, torch.bfloat16, "ring", 0, 0),
    ("rect_tiles", 4, 4, 256, 384, torch.bfloat16, "ring", 0, 64),
    ("random_holes_dups", 8, 32, 256, 128, torch.bfloat16, "random", 1, 8),
    ("random2", 8, 32, 128, 256, torch.bfloat16, "random", 2, 0),
    ("fan_in", 4, 8, 128, 128, torch.bfloat16, "fan_in", 0, 128),
    ("empty", 8, 3, 128, 128, torch.bfloat16, "empty", 0, 8),
    ("epn1", 2, 1, 128, 128, torch.bfloat16, "ring", 0, 0),
    ("uint8_packed", 4, 8, 256, 128, torch.uint8, "random", 3, 16),
    ("int8", 4, 3, 128, 384, torch.int8, "asymmetric", 0, 16),
    ("offset_128B_pool", 4, 3, 384, 640, torch.bfloat16, "ring", 0, 64),
]


def _fill(shape, dtype, g):
    if dtype.is_floating_point:
        return torch.randn(shape, generator=g).to(dtype)
    info = torch.iinfo(dtype)
    return torch.randint(info.min, info.max + 1, shape, generator=g, dtype=torch.int32).to(dtype)


@pytest.mark.parametrize("case", PREFETCH_CASES, ids=[c[0] for c in PREFETCH_CASES])
def test_prefetch_matches_oracle(cuda, case):
    name, R, epn, H, Hp, dtype, plan_name, seed, pad = case
    print(f"prefetch case {name}", flush=True)
    etc = PLANS[plan_name](R, epn, seed)
    sent = SENTINEL if dtype.is_floating_point else (0xAB if dtype == torch.uint8 else 123)
    g = torch.Generator().manual_seed(100 + seed)
    # every rank's local experts for the three projections (different shapes per projection)
    shapes = [(H, Hp), (H, Hp), (Hp, H)]
    locals_ = [[_fill((epn, *shp), dtype, g) for shp in shapes] for _ in range(R)]
    ref_pools, dev_pools, dev_backing = [], [], []
    for t, shp in enumerate(shapes):
        lead = 64 * (t + 1) if name.startswith("offset") else 0   # 128-byte steps into the allocation
        _, rp = strided_pool(R, (epn, *shp), dtype, pad * (t + 1), sent, "cpu", lead)
        bk, dp = strided_pool(R, (epn, *shp), dtype, pad * (t + 1), sent, cuda, lead)
        ref_pools.append(rp)
        dev_pools.append(dp)
        dev_backing.append(bk)
    etc_dev = etc.to(cuda)
    for rank in range(R):
        for t in range(3):
            oo.prefetch(locals_[rank][t], ref_pools[t], etc, rank)
        launch_prefetch(tuple(x.to(cuda) for x in locals_[rank]), tuple(dev_pools), etc_dev,
                        rank=rank)
    torch.cuda.synchronize()
    for t in range(3):
        assert torch.equal(dev_pools[t].cpu(), ref_pools[t]), f"tensor {t}"
        # padding between ranks untouched
        stride = dev_pools[t].stride(0)
        numel = dev_pools[t][0].numel()
        bk = dev_backing[t].cpu().view(R, stride)
        if stride > numel:
            assert (bk[:, numel:] == sent).all(), "inter-rank padding was written"
    # unused slots keep the sentinel
    for d in range(R):
        for b in range(epn):
            if int(etc[d, b]) < 0:
                assert (dev_pools[0][d, b].cpu() == sent).all()


def test_prefetch_with_scales_and_large_offsets(cuda):
    """uint8 weights + re-tiled scale tensors in one launch; a pool whose
    slot offsets exceed 2**31 bytes."""
    R, epn, H, Hp = 4, 3, 256, 256
    etc = torch.full((R, epn), -1, dtype=torch.int32)
    for d in range(R):
        etc[d, 0] = ((d + 1) % R) * epn + 2
        etc[d, 1] = ((d + 2) % R) * epn + 0
    g = torch.Generator().manual_seed(5)
    scale_shape = (64, 64)  # fp32: 16 KiB per expert = one re-tile unit
    locals_w = [[_fill((epn, H, Hp), torch.uint8, g) for _ in range(3)] for _ in range(R)]
    locals_s = [[torch.randn((epn, *scale_shape), generator=g) for _ in range(3)] for _ in range(R)]
    assert retile_for_prefetch(locals_s[0][0]).shape == (epn, 128, 128)
    assert prefetch_retile_nbytes(100) == 16384
    ref_w = [torch.full((R, epn, H, Hp), 0xAB, dtype=torch.uint8) for _ in range(3)]
    ref_s = [torch.full((R, epn, *scale_shape), SENTINEL) for _ in range(3)]
    dev_w = [x.to(cuda) for x in ref_w]
    dev_s = [x.to(cuda) for x in ref_s]
    for rank in range(R):
        for t in range(3):
            oo.prefetch(locals_w[rank][t], ref_w[t], etc, rank)
            oo.prefetch(locals_s[rank][t], ref_s[t], etc, rank)
        launch_prefetch(tuple(x.to(cuda) for x in locals_w[rank]), tuple(dev_w), etc.to(cuda),
                        rank=rank,
                        scales=tuple((locals_s[rank][t].to(cuda), dev_s[t]) for t in range(3)))
    torch.cuda.synchronize()
    for t in range(3):
        assert torch.equal(dev_w[t].cpu(), ref_w[t])
        assert torch.equal(dev_s[t].cpu().view(torch.int32), ref_s[t].view(torch.int32))

    # > 2**31-byte offsets: 3 ranks x 2 slots of 512 MiB; only the last slot is used
    R, epn, H, Hp = 3, 2, 16384, 16384
    etc = torch.full((R, epn), -1, dtype=torch.int32)
    etc[2, 1] = 0 * epn + 1            # rank 0's expert 1 -> pool[2, 1] (byte offset 2.5 GiB)
    local = torch.empty(epn, H, Hp, dtype=torch.bfloat16, device=cuda)
    local[1] = torch.arange(Hp, device=cuda, dtype=torch.float32).to(torch.bfloat16)[None, :]
    local[1, -1, -1] = 42.0
    pool = torch.zeros(R, epn, H, Hp, dtype=torch.bfloat16, device=cuda)
    launch_prefetch((local, local, local), (pool, pool, pool), etc.to(cuda), rank=0)
    torch.cuda.synchronize()
    assert torch.equal(pool[2, 1], local[1])
    assert not bool(pool[2, 0].any()) and not bool(pool[:2].any())


PULL_CASES = ["rect_tiles", "random_holes_dups", "fan_in", "empty", "uint8_packed", "offset_128B_pool"]


@pytest.mark.parametrize("case", [c for c in PREFETCH_CASES if c[0] in PULL_CASES],
                         ids=[c[0] for c in PREFETCH_CASES if c[0] in PULL_CASES])
def test_prefetch_pull_fills_one_ranks_slots_like_all_owner_pushes(cuda, case):
    """The pull view (one launch per destination rank, reading every owner's experts) leaves in
    pool[rank] what the R owner pushes leave there, and touches nothing else: slots of other
    ranks, free slots and the padding between ranks keep their sentinel (the per-rank check of
    reference tests/test_prefetch.py:448-464)."""
    name, R, epn, H, Hp, dtype, plan_name, seed, pad = case
    print(f"prefetch pull case {name}", flush=True)
    etc = PLANS[plan_name](R, epn, seed)
    sent = SENTINEL if dtype.is_floating_point else (0xAB if dtype == torch.uint8 else 123)
    g = torch.Generator().manual_seed(300 + seed)
    shapes = [(H, Hp), (H, Hp), (Hp, H)]
    owners_ref, owners_dev, ref_pools = [], [], []
    for t, shp in enumerate(shapes):
        # every owner's local experts side by side, with padding between the owners too
        _, ow = strided_pool(R, (epn, *shp), dtype, 16 * (t + 1), 0, "cpu")
        ow.copy_(_fill((R, epn, *shp), dtype, g))
        _, od = strided_pool(R, (epn, *shp), dtype, 16 * (t + 1), 0, cuda)
        od.copy_(ow)
        owners_ref.append(ow)
        owners_dev.append(od)
        _, rp = strided_pool(R, (epn, *shp), dtype, pad * (t + 1), sent, "cpu")
        for owner in range(R):
            oo.prefetch(ow[owner], rp, etc, owner)
        ref_pools.append(rp)
    etc_dev = etc.to(cuda)
    for rank in range(R):
        dev_pools, dev_backing = [], []
        for t, shp in enumerate(shapes):
            lead = 64 * (t + 1) if name.startswith("offset") else 0
            bk, dp = strided_pool(R, (epn, *shp), dtype, pad * (t + 1), sent, cuda, lead)
            dev_pools.append(dp)
            dev_backing.append(bk)
        launch_prefetch_pull(tuple(owners_dev), tuple(dev_pools), etc_dev, rank=rank)
        torch.cuda.synchronize()
        for t in range(3):
            got = dev_pools[t].cpu()
            assert torch.equal(got[rank], ref_pools[t][rank]), f"rank {rank} tensor {t}"
            others = [d for d in range(R) if d != rank]
            assert (got[others] == sent).all(), "a pull wrote into another rank's slots"
            stride, numel = dev_pools[t].stride(0), dev_pools[t][0].numel()
            if stride > numel:
                assert (dev_backing[t].cpu().view(R, stride)[:, numel:] == sent).all()


def test_prefetch_pull_with_scales(cuda):
    R, epn, H, Hp = 4, 3, 256, 256
    etc = torch.full((R, epn), -1, dtype=torch.int32)
    for d in range(R):
        etc[d, 0] = ((d + 1) % R) * epn + 2
        etc[d, 2] = ((d + 3) % R) * epn + 1
    g = torch.Generator().manual_seed(6)
    scale_shape = (64, 64)
    own_w = [_fill((R, epn, H, Hp), torch.uint8, g) for _ in range(3)]
    own_s = [torch.randn((R, epn, *scale_shape), generator=g) for _ in range(3)]
    ref_w = [torch.full((R, epn, H, Hp), 0xAB, dtype=torch.uint8) for _ in range(3)]
    ref_s = [torch.full((R, epn, *scale_shape), SENTINEL) for _ in range(3)]
    dev_w = [x.to(cuda) for x in ref_w]
    dev_s = [x.to(cuda) for x in ref_s]
    dow, dos = [x.to(cuda) for x in own_w], [x.to(cuda) for x in own_s]
    for rank in range(R):
        for t in range(3):
            oo.prefetch(own_w[t][rank], ref_w[t], etc, rank)
            oo.prefetch(own_s[t][rank], ref_s[t], etc, rank)
        launch_prefetch_pull(tuple(dow), tuple(dev_w), etc.to(cuda), rank=rank,
                             scales=tuple((dos[t], dev_s[t]) for t in range(3)))
    torch.cuda.synchronize()
    for t in range(3):
        assert torch.equal(dev_w[t].cpu(), ref_w[t])
        assert torch.equal(dev_s[t].cpu().view(torch.int32), ref_s[t].view(torch.int32))


# ---------------------------------------------------------------- grad reduce
REDUCE_CASES = [
    # name, R, epn, H, Hp, plan, seed, data, pad
    ("ring_affine", 4, 4, 128, 128, "ring", 0, "affine", 0),
    ("ring_randn", 8, 4, 128, 256, "ring", 0, "randn", 32),
    ("fan_in_randn", 4, 8, 128, 128, "fan_in", 0, "randn", 4),
    ("fan_in_affine", 2, 4, 256, 128, "fan_in", 0, "affine", 0),
    ("empty", 4, 3, 128, 128, "empty", 0, "randn", 8),
    ("asymmetric", 4, 2, 128, 128, "asymmetric", 0, "randn", 0),
    ("random1", 8, 8, 128, 128, "random", 1, "randn", 16),
    ("random2", 8, 16, 128, 128, "random", 2, "randn", 0),
    ("epn1", 2, 1, 128, 128, "ring", 0, "randn", 0),
    # 192 KiB per matrix: one 128 KiB block in the spread tile layout, then four tiles of adjacent pieces
    ("spread_plus_tail", 4, 4, 384, 128, "random", 3, "randn", 16),
]


def _grad_data(kind, R, epn, H, Hp, g):
    if kind == "affine":
        # small integers: every fp32 add is exact, any order gives the same bits
        grads = [torch.randint(-64, 64, (epn, H, Hp), generator=g).float() for _ in range(R)]
        slots = torch.randint(-64, 64, (R, epn, H, Hp), generator=g).float()
    else:
        grads = [torch.randn(epn, H, Hp, generator=g) for _ in range(R)]
        slots = torch.randn(R, epn, H, Hp, generator=g) * 1e-3 + torch.randn(R, epn, 1, 1, generator=g)
    return grads, slots


@pytest.mark.parametrize("case", REDUCE_CASES, ids=[c[0] for c in REDUCE_CASES])
def test_grad_reduce_matches_oracle(cuda, case):
    name, R, epn, H, Hp, plan_name, seed, kind, pad = case
    print(f"grad_reduce case {name}", flush=True)
    etc = PLANS[plan_name](R, epn, seed)
    g = torch.Generator().manual_seed(200 + seed)
    grads, slots = _grad_data(kind, R, epn, H, Hp, g)
    bk, pool = strided_pool(R, (epn, H, Hp), torch.float32, pad, SENTINEL, cuda)
    pool.copy_(slots)
    ref_pool = slots.clone()
    etc_dev = etc.to(cuda)
    # The reference runs the ranks concurrently: every rank reads before any
    # rank clears.  Emulate with reads from a snapshot for the oracle and, on
    # the GPU, by restoring the pool before each rank's launch.
    final_pool = slots.clone()
    for rank in range(R):
        want_grad = grads[rank].clone()
        scratch = slots.clone()
        oo.grad_reduce(want_grad, scratch, etc, rank)
        pool.copy_(slots)
        got = grads[rank].to(cuda)
        launch_grad_reduce(got, pool, etc_dev, rank=rank)
        torch.cuda.synchronize()
        assert torch.equal(got.cpu().view(torch.int32), want_grad.view(torch.int32)), f"rank {rank} grad"
        assert torch.equal(pool.cpu().view(torch.int32), scratch.view(torch.int32)), f"rank {rank} clears"
        final_pool[rank] = scratch[rank]
        stride = pool.stride(0)
        numel = pool[0].numel()
        if stride > numel:
            assert (bk.cpu().view(R, stride)[:, numel:] == SENTINEL).all()
    # repeated launches on the cleared pool are stable: second call adds zeros or leftovers
    pool.copy_(final_pool)
    again = grads[0].to(cuda)
    launch_grad_reduce(again, pool, etc_dev, rank=0)
    want = grads[0].clone()
    oo.grad_reduce(want, final_pool.clone(), etc, 0)
    torch.cuda.synchronize()
    assert torch.equal(again.cpu().view(torch.int32), want.view(torch.int32))


def test_grad_reduce_with_a_table_beyond_64_kb_of_lds(cuda):
    """R = 128 ranks x 32 slots: the slot table and the per-entry offsets need more dynamic LDS
    than the default limit; a few ranks against the oracle, bit for bit."""
    R, epn, H, Hp = 128, 32, 128, 128
    etc = PLANS["random"](R, epn, 11)
    g = torch.Generator().manual_seed(77)
    slots = torch.randn(R, epn, H, Hp, generator=g) * 1e-3 + torch.randn(R, epn, 1, 1, generator=g)
    pool = slots.to(cuda)
    etc_dev = etc.to(cuda)
    for rank in (0, 63, 127):
        grad = torch.randn(epn, H, Hp, generator=g)
        want, scratch = grad.clone(), slots.clone()
        oo.grad_reduce(want, scratch, etc, rank)
        pool.copy_(slots)
        got = grad.to(cuda)
        launch_grad_reduce(got, pool, etc_dev, rank=rank)
        torch.cuda.synchronize()
        assert torch.equal(got.cpu().view(torch.int32), want.view(torch.int32)), f"rank {rank} grad"
        assert torch.equal(pool.cpu().view(torch.int32), scratch.view(torch.int32)), f"rank {rank} clears"


def test_grad_reduce_large_offsets(cuda):
    """slot offsets beyond 2**31 elements"""
    R, epn, H, Hp = 3, 2, 16384, 32768       # 2 GiB per slot, 12 GiB pool
    etc = torch.full((R, epn), -1, dtype=torch.int32)
    etc[2, 1] = 0 * epn + 1
    etc[0, 0] = 1 * epn + 0                  # rank 0 hosts someone else's expert -> cleared
    pool = torch.empty(R, epn, H, Hp, dtype=torch.float32, device=cuda)
    pool[2, 1].fill_(0.5)
    pool[0, 0].fill_(3.0)
    pool[0, 1].fill_(7.0)
    local = torch.ones(epn, H, Hp, dtype=torch.float32, device=cuda)
    launch_grad_reduce(local, pool, etc.to(cuda), rank=0)
    torch.cuda.synchronize()
    assert bool((local[1] == 1.5).all()) and bool((local[0] == 1.0).all())
    assert not bool(pool[0, 0].any())          # own occupied slot cleared
    assert bool((pool[0, 1] == 7.0).all())     # own free slot untouched
    assert bool((pool[2, 1] == 0.5).all())     # a peer's slot is never written
