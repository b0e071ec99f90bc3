"""Combine host side: duplicate pre-reduction and the top-k unpermute.

Mirrors the launchers of reference moonep/combine_prologue.py:544-599
(``launch_combine_prologue``) and moonep/combine.py:565-654
(``launch_combine``); kernels are in csrc/dispatch.hip and csrc/combine.hip.
"""

from __future__ import annotations

import torch

from . import _lib
from .planning import MoonEPCommPlan

_MODES = {
    "primaries": _lib.COMBINE_PRIMARIES,
    "all": _lib.COMBINE_ALL,
    "two_level": _lib.COMBINE_TWO_LEVEL,
    "weighted": _lib.COMBINE_WEIGHTED,
}


def launch_combine_prologue(ctx: dict, plan: MoonEPCommPlan, *, pdl_trigger: bool = False) -> None:
    """In place on the local shard: primary row <- bf16(fp32 sum of the
    primary and its duplicate rows)."""
    assert isinstance(plan, MoonEPCommPlan)
    from .dispatch import _require_dedup_map, dup_cu_bound
    _require_dedup_map(ctx, plan, "launch_combine_prologue")
    H, NvS = int(ctx["H"]), int(ctx["NvS"])
    shard = ctx["hidden_buf_local"]
    assert shard.dtype == torch.bfloat16 and shard.is_contiguous()
    assert tuple(shard.shape) == (NvS, H), \
        f"hidden_buf_local must be shape ({NvS}, {H}), got {tuple(shard.shape)}"
    assert plan.K <= 32
    rc = _lib.lib().mep_combine_prologue(
        shard.data_ptr(), plan.dup_groups.data_ptr(), plan.dup_loffs.data_ptr(),
        plan.dup_counts.data_ptr(), NvS, H, dup_cu_bound(ctx), _lib.current_stream(),
    )
    _lib.check(rc, "mep_combine_prologue")


def launch_combine(ctx: dict, output_sh, dst, output_sk=None, *, pdl_launch: bool = False,
                   mode: str = "primaries") -> None:
    """K-sum of each token's rows into ``output_sh[S,H]`` (fp32 accumulation,
    one bf16 rounding) and gather of its K route weights into ``output_sk``.

    mode "primaries": rows of non-negative ``dst`` entries only -- the
        reference kernel, to be preceded by ``launch_combine_prologue`` on
        every destination rank;
    mode "all": all K rows, one rounding;
    mode "two_level": all K rows, grouped and rounded exactly as prologue +
        "primaries" would, without modifying the shards;
    mode "weighted": not a reference mode -- all K rows, each multiplied by the
        route weight in its slot (product and sum rounded separately in fp32).
    """
    assert output_sh.dtype == torch.bfloat16 and output_sh.is_contiguous(), \
        "output_sh must be contiguous bf16"
    assert dst.dtype == torch.int32 and dst.is_contiguous(), "dst must be contiguous int32"
    H, R, S, K, NvS = (int(ctx[k]) for k in ("H", "R", "S", "K", "NvS"))
    assert tuple(output_sh.shape) == (S, H)
    assert dst.numel() == S * K
    wslots = None
    if output_sk is not None:
        assert output_sk.dtype == torch.float32 and output_sk.is_contiguous(), \
            "output_sk must be contiguous fp32"
        assert output_sk.numel() == S * K
    if output_sk is not None or mode == "weighted":
        wslots = ctx["meta_buf"].data_ptr() + 4 * int(ctx["WEIGHTS_OFF"])
    assert H % 8 == 0, "H must be a multiple of 8 (16-B row vectors)"
    rc = _lib.lib().mep_combine(
        ctx["hidden_buf"].data_ptr(), int(ctx["NvS_padded"]), wslots,
        int(ctx["meta_chunk_padded"]), dst.data_ptr(), output_sh.data_ptr(),
        _lib.ptr(output_sk), S, H, K, R, NvS, _MODES[mode], _lib.current_stream(),
    )
    _lib.check(rc, "mep_combine")
