"""Dispatch host side: fused permute, duplicate-group builder and the
destination-side duplicate expansion.

Mirrors the launchers of reference moonep/dispatch.py:838-983
(``launch_dispatch``) and moonep/dispatch_epilogue.py:366-415
(``launch_dispatch_epilogue``); kernels are in csrc/dispatch.hip.
"""

from __future__ import annotations

import torch

from . import _lib
from .planning import MoonEPCommPlan


def _check_dispatch_plan(ctx: dict, hidden_sh: torch.Tensor, plan: MoonEPCommPlan) -> None:
    S, K, R, E, NvS = (int(ctx[k]) for k in ("S", "K", "R", "E", "NvS"))
    N, epn, dev = S * K, E // R, hidden_sh.device
    assert plan.N == N, f"plan.N must be S*K={N}, got {plan.N}"
    assert plan.R == R, f"plan.R must match ctx R={R}, got {plan.R}"
    assert plan.K == K, f"plan.K must match ctx K={K}, got {plan.K}"
    assert plan.NvS == NvS, f"plan.NvS must match ctx NvS={NvS}, got {plan.NvS}"

    def chk(t, name, shape):
        assert t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32"
        assert tuple(t.shape) == shape, f"{name} must be shape {shape}, got {tuple(t.shape)}"
        assert t.device == dev, f"{name} must be on {dev}, got {t.device}"

    chk(plan.dst, "dst", (N,))
    chk(plan.zero_fill_ranges, "zero_fill_ranges", (2 * epn, 2))
    chk(plan.dup_groups, "dup_groups", (NvS, 3))
    chk(plan.dup_loffs, "dup_loffs", (NvS,))
    chk(plan.dup_counts, "dup_counts", (2,))


def check_dispatch_inputs(ctx: dict, hidden_sh, route_weights_sk) -> None:
    """The token and weight tensors of a dispatch, checked as reference
    moonep/dispatch.py:880-905 checks them (no device access)."""
    H, S, K = (int(ctx[k]) for k in ("H", "S", "K"))
    assert hidden_sh.dtype == torch.bfloat16 and hidden_sh.is_contiguous(), \
        "hidden_sh must be contiguous bf16"
    assert hidden_sh.is_cuda, "hidden_sh must be a CUDA tensor"
    assert tuple(hidden_sh.shape) == (S, H), \
        f"hidden_sh must be shape [S={S}, H={H}], got {tuple(hidden_sh.shape)}"
    assert ctx["hidden_buf"].device == hidden_sh.device
    if route_weights_sk is not None:
        assert route_weights_sk.dtype == torch.float32 and route_weights_sk.is_contiguous(), \
            "route_weights_sk must be contiguous fp32"
        assert tuple(route_weights_sk.shape) == (S, K), \
            f"route_weights_sk must be shape [S={S}, K={K}], got {tuple(route_weights_sk.shape)}"
        assert route_weights_sk.device == hidden_sh.device
    assert H % 8 == 0, "H must be multiple of 8 for 16-B row vectors"


def _require_dedup_map(ctx: dict, plan: MoonEPCommPlan, what: str) -> None:
    world = ctx.get("world")
    assert world is None or world.has_dedup(plan), (
        f"{what}: this plan has no duplicate map (it was planned from one rank's topk only, so "
        "the other ranks' dst were unknown); plan with topk[R, S, K], or drive the ranks from "
        "host threads of an EmulatedWorld(host_threads=True)")


def launch_dispatch(ctx: dict, hidden_sh, route_weights_sk, plan, *, build_dedup_map: bool = True,
                    pdl_trigger: bool = False, write_dups: bool = False,
                    dst_all_ranks: torch.Tensor | None = None) -> None:
    """Scatter ``hidden_sh[S,H]`` (and ``route_weights_sk[S,K]``) of ctx['rank']
    into every destination's shard and zero-fill the local padding rows.

    ``write_dups`` also copies the rows of duplicate (negative) entries, which
    makes a following ``launch_dispatch_epilogue`` on the destinations
    unnecessary.  ``build_dedup_map`` (fresh plans only, as in the reference)
    fills ``plan.dup_*`` from ``dst_all_ranks[R, N]``; without that table the
    duplicate groups stay empty.  ``pdl_trigger`` is accepted for signature
    compatibility; HIP kernels on one stream already run back to back.
    """
    assert isinstance(plan, MoonEPCommPlan)
    H, R, S, K, E = (int(ctx[k]) for k in ("H", "R", "S", "K", "E"))
    check_dispatch_inputs(ctx, hidden_sh, route_weights_sk)
    _check_dispatch_plan(ctx, hidden_sh, plan)
    meta = ctx["meta_buf"]
    wslots = None
    if route_weights_sk is not None:
        wslots = meta.data_ptr() + 4 * int(ctx["WEIGHTS_OFF"])
    flags = _lib.DISPATCH_WRITE_DUPS if write_dups else 0
    rc = _lib.lib().mep_dispatch(
        hidden_sh.data_ptr(), _lib.ptr(route_weights_sk), plan.dst.data_ptr(),
        plan.zero_fill_ranges.data_ptr(), ctx["hidden_buf"].data_ptr(), int(ctx["NvS_padded"]),
        wslots, int(ctx["meta_chunk_padded"]), int(ctx["rank"]), S, H, K, R, E // R,
        int(ctx["NvS"]), int(ctx["token_padding"]), flags, _lib.current_stream(),
    )
    _lib.check(rc, "mep_dispatch")
    if build_dedup_map and dst_all_ranks is not None:
        launch_build_dedup(ctx, dst_all_ranks, plan)


def launch_build_dedup(ctx: dict, dst_all_ranks: torch.Tensor, plan: MoonEPCommPlan) -> None:
    """Fill ``plan.dup_groups / dup_loffs / dup_counts`` of ctx['rank'] from
    every source rank's ``dst`` ([R, N], canonical or raw)."""
    R, S, K, NvS = (int(ctx[k]) for k in ("R", "S", "K", "NvS"))
    assert dst_all_ranks.dtype == torch.int32 and dst_all_ranks.is_contiguous()
    assert tuple(dst_all_ranks.shape) == (R, S * K)
    if "dedup_scratch" not in ctx:
        n = _lib.lib().mep_dedup_scratch_bytes(S, R)
        ctx["dedup_scratch"] = torch.empty(n, dtype=torch.uint8, device=dst_all_ranks.device)
    scratch = ctx["dedup_scratch"]
    rc = _lib.lib().mep_build_dedup(
        dst_all_ranks.data_ptr(), int(ctx["rank"]), S, K, R, NvS, plan.dup_groups.data_ptr(),
        plan.dup_loffs.data_ptr(), plan.dup_counts.data_ptr(), scratch.data_ptr(),
        scratch.numel(), _lib.current_stream(),
    )
    _lib.check(rc, "mep_build_dedup")


def dup_cu_bound(ctx: dict) -> int:
    """Compute units the standalone duplicate kernels may use: the context's
    ``num_sms_dedup`` (``MOONEP_NUM_SMS_DEDUP``, reference moonep/api.py:100-120) when it
    is below the device's CU count, else 0 = no bound (the kernels then pick the grid that
    fills the GPU)."""
    n, all_cus = int(ctx.get("num_sms_dedup", 0) or 0), int(ctx.get("max_sms", 0) or 0)
    return n if 0 < n < all_cus else 0


def launch_dispatch_epilogue(ctx: dict, plan: MoonEPCommPlan, *, pdl_launch: bool = False) -> None:
    """Copy every primary row of the local shard to its duplicate rows."""
    assert isinstance(plan, MoonEPCommPlan)
    _require_dedup_map(ctx, plan, "launch_dispatch_epilogue")
    shard = ctx["hidden_buf_local"]
    assert shard.dtype == torch.bfloat16 and shard.is_contiguous()
    rc = _lib.lib().mep_dispatch_epilogue(
        shard.data_ptr(), plan.dup_groups.data_ptr(), plan.dup_loffs.data_ptr(),
        plan.dup_counts.data_ptr(), int(ctx["NvS"]), int(ctx["H"]), dup_cu_bound(ctx),
        _lib.current_stream(),
    )
    _lib.check(rc, "mep_dispatch_epilogue")
