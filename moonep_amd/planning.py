"""Planner host side: the plan container and the launcher of the HIP planner.

Mirrors the host half of reference moonep/planning.py: ``MoonEPCommPlan``
(:31-86), ``allocate_planning_outputs`` (:1168-1215), the bounds checks
(:1218-1255) and ``launch_planning`` (:1258-1280).  The device half is
csrc/planner.hip, reached through ``mep_plan`` / ``mep_plan_ranks``.

One GPU stands in for the R expert-parallel ranks, so the planner takes every
rank's ``tokens_per_expert`` as an ``[R, E]`` table (the reference gathers the
rows from its peers inside the kernel, planning.py:577-583).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib
from .constants import KIDX_BITS


@dataclass(frozen=True, slots=True)
class MoonEPCommPlan:
    """Routing plan of one rank; same fields and checks as the reference's."""

    dst: torch.Tensor               # [N] int32; negative = duplicate, -(raw)-1
    experts_to_copy: torch.Tensor   # [R, epn] remote experts hosted per rank, -1 = free
    zero_fill_ranges: torch.Tensor  # [2*epn, 2] (first padding row, rows)
    remote_stats: torch.Tensor      # [2]
    N: int
    R: int
    E: int
    NvS: int
    K: int
    # destination-side duplicate groups; only the first dup_counts[0] groups
    # and dup_counts[1] offsets are meaningful
    dup_groups: torch.Tensor        # [NvS, 3] (primary row, first offset index, count)
    dup_loffs: torch.Tensor         # [NvS]
    dup_counts: torch.Tensor        # [2]

    def __post_init__(self) -> None:
        N, R, E, NvS = int(self.N), int(self.R), int(self.E), int(self.NvS)
        epn = E // R

        def chk(t, shape):
            assert t.dtype == torch.int32 and t.is_contiguous()
            assert tuple(t.shape) == shape

        assert self.dst.dtype == torch.int32 and self.dst.is_contiguous()
        assert self.dst.numel() == N
        chk(self.experts_to_copy, (R, epn))
        chk(self.remote_stats, (2,))
        chk(self.zero_fill_ranges, (2 * epn, 2))
        chk(self.dup_groups, (NvS, 3))
        chk(self.dup_loffs, (NvS,))
        chk(self.dup_counts, (2,))

    def clone(self) -> "MoonEPCommPlan":
        return type(self)(
            dst=self.dst.clone(), experts_to_copy=self.experts_to_copy.clone(),
            zero_fill_ranges=self.zero_fill_ranges.clone(),
            remote_stats=self.remote_stats.clone(), dup_groups=self.dup_groups.clone(),
            dup_loffs=self.dup_loffs.clone(), dup_counts=self.dup_counts.clone(),
            N=self.N, R=self.R, E=self.E, NvS=self.NvS, K=self.K,
        )


def allocate_planning_outputs(ctx: dict):
    """A fresh ``(MoonEPCommPlan, cu_seqlens)`` pair on ctx's device.

    ``dup_counts`` starts at zero so that a plan whose duplicate groups were
    never built reads as "no groups" in the epilogue/prologue kernels.
    """
    E, R, NvS, K = ctx["E"], ctx["R"], ctx["NvS"], ctx["K"]
    epn = E // R
    N = ctx["S"] * K
    dev = ctx["meta_buf"].device
    i32 = dict(dtype=torch.int32, device=dev)
    plan = MoonEPCommPlan(
        dst=torch.empty(N, **i32),
        experts_to_copy=torch.empty(R, epn, **i32),
        zero_fill_ranges=torch.empty(2 * epn, 2, **i32),
        remote_stats=torch.empty(2, **i32),
        dup_groups=torch.empty(NvS, 3, **i32),
        dup_loffs=torch.empty(NvS, **i32),
        dup_counts=torch.zeros(2, **i32),
        N=N, R=R, E=E, NvS=NvS, K=K,
    )
    return plan, torch.empty(2 * epn, **i32)


def _check_planning_outputs(ctx: dict, cu_seqlens, plan) -> None:
    assert isinstance(plan, MoonEPCommPlan)
    epn = ctx["E"] // ctx["R"]
    assert plan.N == ctx["S"] * ctx["K"]
    assert plan.R == ctx["R"]
    assert plan.E == ctx["E"]
    assert plan.NvS == ctx["NvS"]
    assert plan.K == ctx["K"]
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.is_contiguous()
    assert tuple(cu_seqlens.shape) == (2 * epn,)


def _check_dedup_encoding_bounds(ctx: dict) -> None:
    """Bounds of the packed encodings (reference moonep/planning.py:1231-1255)."""
    R, S, K, NvS = int(ctx["R"]), int(ctx["S"]), int(ctx["K"]), int(ctx["NvS"])
    nvs_bits = 32 - 1 - KIDX_BITS
    N = S * K
    int32_max = 2**31 - 1
    assert N <= NvS, f"slot encoding requires S*K <= NvS, got S*K={N}, NvS={NvS}"
    assert R * NvS <= int32_max, (
        f"dst encoding requires R*NvS <= int32_max: R={R}, NvS={NvS}, R*NvS={R * NvS}"
    )
    assert R <= 128, f"duplicate canonicalization requires R <= 128, got {R}"
    assert K <= (1 << KIDX_BITS) - 1, f"K must be <= {(1 << KIDX_BITS) - 1}, got {K}"
    assert NvS <= (1 << nvs_bits) - 1, f"NvS must be <= {(1 << nvs_bits) - 1}, got {NvS}"
    assert K <= 32, f"per-token lane ownership requires K <= 32, got {K}"


def _tpe_table(ctx: dict, tokens_per_expert: torch.Tensor) -> torch.Tensor:
    """The ``[R, E]`` count table the planner reads.  A per-rank ``[E]`` row is
    deposited into the world's gathered table (the reference's planner writes
    its row into its peers' meta chunks, planning.py:577-583) and the table of
    this rank's meta chunk is returned after a rendezvous of the rank threads, so that
    every row is in; without rank threads there is nobody to fill the other rows and the
    call is refused."""
    R, E = int(ctx["R"]), int(ctx["E"])
    assert tokens_per_expert.dtype == torch.int32 and tokens_per_expert.is_contiguous()
    if tokens_per_expert.dim() == 2:
        assert tuple(tokens_per_expert.shape) == (R, E), (
            f"tokens_per_expert must be [R={R}, E={E}], got {tuple(tokens_per_expert.shape)}"
        )
        return tokens_per_expert
    assert tokens_per_expert.numel() == E
    if R == 1:
        return tokens_per_expert.reshape(1, E)
    world, rank = ctx["world"], int(ctx["rank"])
    if not world.host_threads:
        raise NotImplementedError(
            "launch_planning(tokens_per_expert[E]) of one rank needs the other ranks' counts: pass "
            f"the gathered tokens_per_expert[R={R}, E={E}], or run every rank on its own host "
            "thread of an EmulatedWorld(host_threads=True)")
    world.deposit_tokens_per_expert(rank, tokens_per_expert)
    world.rendezvous(rank)
    return world.tpe_table(rank)


def plan_scratch(ctx: dict, nranks: int = 1) -> torch.Tensor | None:
    """Device scratch the planner needs for this shape (None when its tables
    fit in LDS).  ``allocate_launch_scratch`` fills the cache for one rank and
    for all R ranks when the context is made, so no launcher allocates."""
    key = ("plan_scratch", nranks)
    if key not in ctx:
        n = _lib.lib().mep_plan_scratch_bytes(ctx["S"], ctx["K"], ctx["E"], ctx["R"], nranks)
        ctx[key] = (torch.empty(n, dtype=torch.uint8, device=ctx["meta_buf"].device)
                    if n else None)
    return ctx[key]


def allocate_launch_scratch(ctx: dict) -> None:
    """Every scratch buffer the launchers of this context use, allocated once:
    the planner's tables (one rank / all ranks) and the duplicate-group
    builder's counters."""
    lib = _lib.lib()
    plan_scratch(ctx, 1)
    plan_scratch(ctx, int(ctx["R"]))
    n = lib.mep_dedup_scratch_bytes(int(ctx["S"]), int(ctx["R"]))
    ctx["dedup_scratch"] = torch.empty(n, dtype=torch.uint8, device=ctx["meta_buf"].device)


def launch_planning(ctx: dict, topk_experts_flat, tokens_per_expert, cu_seqlens, plan, *,
                    warm: torch.Tensor | None = None) -> None:
    """Run the planner of ctx['rank']; writes ``plan.dst``,
    ``plan.experts_to_copy``, ``plan.zero_fill_ranges``, ``plan.remote_stats``
    and ``cu_seqlens`` in place, asynchronously on the current stream.

    ``warm`` (not in the reference): a contiguous tensor -- the tokens the
    following dispatch will copy -- that the CUs the planner leaves idle read
    once while it runs, so that dispatch finds them in the last-level cache."""
    _check_planning_outputs(ctx, cu_seqlens, plan)
    _check_dedup_encoding_bounds(ctx)
    tpe = _tpe_table(ctx, tokens_per_expert)
    assert topk_experts_flat.dtype == torch.int32 and topk_experts_flat.is_contiguous()
    assert topk_experts_flat.numel() == plan.N
    assert topk_experts_flat.is_cuda and tpe.device == topk_experts_flat.device
    scratch = plan_scratch(ctx)
    if warm is not None:
        assert warm.is_cuda and warm.is_contiguous() and warm.device == topk_experts_flat.device
    rc = _lib.lib().mep_plan_warm(
        tpe.data_ptr(), topk_experts_flat.data_ptr(), int(ctx["rank"]),
        int(ctx["S"]), int(ctx["K"]), int(ctx["E"]), int(ctx["R"]),
        int(ctx["token_padding"]), int(ctx["NvS"]),
        plan.dst.data_ptr(), cu_seqlens.data_ptr(), plan.experts_to_copy.data_ptr(),
        plan.zero_fill_ranges.data_ptr(), plan.remote_stats.data_ptr(),
        _lib.ptr(scratch), 0 if scratch is None else scratch.numel(),
        _lib.ptr(warm), 0 if warm is None else warm.numel() * warm.element_size(),
        _lib.current_stream(),
    )
    _lib.check(rc, "mep_plan")


def launch_planning_all_ranks(ctx: dict, topk_experts_RSK, tokens_per_expert_RE):
    """Plan every rank in one launch (one GPU standing in for R ranks).

    Returns (dst[R,N], cu_seqlens[R,2*epn], experts_to_copy[R,epn],
    zero_fill_ranges[R,2*epn,2], remote_stats[R,2]) as fresh int32 tensors.
    """
    _check_dedup_encoding_bounds(ctx)
    R, E, S, K = int(ctx["R"]), int(ctx["E"]), int(ctx["S"]), int(ctx["K"])
    epn = E // R
    tpe = _tpe_table(ctx, tokens_per_expert_RE)
    topk = topk_experts_RSK
    assert topk.dtype == torch.int32 and topk.is_contiguous() and topk.is_cuda
    assert topk.numel() == R * S * K
    i32 = dict(dtype=torch.int32, device=topk.device)
    dst = torch.empty(R, S * K, **i32)
    cu = torch.empty(R, 2 * epn, **i32)
    etc = torch.empty(R, epn, **i32)
    zfr = torch.empty(R, 2 * epn, 2, **i32)
    stats = torch.empty(R, 2, **i32)
    scratch = plan_scratch(ctx, R)
    rc = _lib.lib().mep_plan_ranks(
        tpe.data_ptr(), topk.data_ptr(), 0, R, S, K, E, R, int(ctx["token_padding"]),
        int(ctx["NvS"]), dst.data_ptr(), cu.data_ptr(), etc.data_ptr(), zfr.data_ptr(),
        stats.data_ptr(), _lib.ptr(scratch), 0 if scratch is None else scratch.numel(),
        _lib.current_stream(),
    )
    _lib.check(rc, "mep_plan_ranks")
    return dst, cu, etc, zfr, stats
