"""Shared helpers of the test-suite (no GPU needed to import)."""

from __future__ import annotations

import numpy as np
import torch

from oracle import planner_oracle as po


def golden_case(golden, name):
    R, S, K, E, tp, NvS = (int(v) for v in golden[f"{name}/shape"])
    g = {k: golden[f"{name}/{k}"] for k in
         ("topk", "tpe", "dst", "cu_seqlens", "experts_to_copy", "remote_stats",
          "zero_fill_ranges", "dup_counts", "dup_groups", "dup_loffs", "alloc_RE")}
    g.update(R=R, S=S, K=K, E=E, tp=tp, NvS=NvS)
    return g


def golden_names(path=None):
    import os
    p = path or os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                             "planner_golden.npz")
    return [str(n) for n in np.load(p)["names"]]


def oracle_world_plan(topk_RSK: np.ndarray, tpe_RE: np.ndarray, tp: int):
    """Oracle plans of all ranks: (GlobalPlan, [RankPlan]*R, dst_all[R,N])."""
    R, S, K = topk_RSK.shape
    gp = po.plan_global(tpe_RE, S, K, tp)
    plans = [po.plan_rank(gp, topk_RSK[r].reshape(-1), r) for r in range(R)]
    return gp, plans, np.stack([p.dst for p in plans])


def traceable_hidden(S: int, H: int, rank: int) -> torch.Tensor:
    """bf16 rows whose bit patterns name their origin: col0 = token index,
    col1 = source rank, the rest a per-(token, column) pattern (idea of
    reference tests/test_dispatch.py:130-146)."""
    s = torch.arange(S, dtype=torch.int32)[:, None]
    c = torch.arange(H, dtype=torch.int32)[None, :]
    bits = ((s * 31 + c * 7 + rank * 131) & 0x7F7F)        # finite bf16 patterns
    bits[:, 0] = (torch.arange(S) & 0x7F7F).to(torch.int32)
    if H > 1:
        bits[:, 1] = rank
    return bits.to(torch.int16).view(torch.bfloat16)


def traceable_weights(S: int, K: int, rank: int) -> torch.Tensor:
    """fp32 whose bit pattern is a ramp: exact round trips are visible."""
    ramp = torch.arange(S * K, dtype=torch.int32) + rank * S * K + 1
    return ramp.view(torch.float32).reshape(S, K)


def grouped_ffn(rows, slots, cu_seqlens, gate, up, down):
    """Plain-PyTorch consumer of one rank's dispatched rows (library GEMMs per group, group
    bounds read on the host): what the HIP expert FFN is checked against.

    rows [NvS,H] bf16, slots [NvS] fp32 route weights, cu_seqlens [2*epn]
    (padded end offset of every group), gate/up/down [2*epn,H,H'] compute
    views.  Group g applies ``w * (silu(x @ gate[g]) * (x @ up[g])) @ down[g].T``
    to its rows; rows outside every group are zero (reference README.md:43-58).
    """
    out = torch.zeros_like(rows)
    start = 0
    for g, end in enumerate(cu_seqlens.tolist()):
        if end > start:
            x = rows[start:end]
            h = torch.nn.functional.silu(x @ gate[g]) * (x @ up[g])
            y = (h @ down[g].t()).float() * slots[start:end, None]
            out[start:end] = y.to(rows.dtype)
        start = end
    return out
