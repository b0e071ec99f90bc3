"""Autograd glue and the expert-side consumer contract around ``Buffer``.

How a training framework wires MoonEP into an MoE layer (reference
README.md:43-156): dispatch forward pairs with combine as its backward, combine
forward pairs with a plan-reusing dispatch as its backward, ``prefetch_weight``
pairs with ``reduce_grad``, and the expert FFN consumes the dispatched rows as
``2*epn`` groups (``epn`` local experts, then ``epn`` prefetch slots) delimited
by ``cu_seqlens``.

One GPU stands in for all R ranks here, so the functions below act on the
whole emulated group at once (``[R, ...]`` tensors, one ``Buffer`` per rank on a
shared ``EmulatedWorld``): every rank dispatches before any rank's experts
run, every rank's experts finish before any rank combines -- the ordering the
reference gets from its cross-rank barriers.

``group_expert_ffn_hip`` is the expert stage of the layer on the matrix cores,
forward and backward: the compute views of every rank (its local experts, then
its prefetch slots filled by one ``launch_prefetch_pull``), the grouped SwiGLU FFN
of every rank, and in backward the grouped input / weight gradient GEMMs followed
by ``reduce_grad`` in fp32 -- no PyTorch GEMM on either pass.
"""

from __future__ import annotations

import torch

from . import ffn
from .api import Buffer, EmulatedWorld
from .grad_reduce import launch_grad_reduce
from .prefetch import launch_prefetch_pull


class EmulatedGroup:
    """R Buffers (one per rank) on one shared set of shards."""

    def __init__(self, S, H, K, E, R, token_padding=128):
        self.S, self.H, self.K, self.E, self.R = S, H, K, E, R
        self.epn = E // R
        self.world = EmulatedWorld(S, H, K, E, R, token_padding)
        self.buffers = [Buffer(S, H, K, E, R, token_padding=token_padding, rank=r,
                               world=self.world) for r in range(R)]
        self.NvS = self.world.NvS
        lay = self.world.layout
        self._mcp = lay["meta_chunk_padded"]

    def shards(self) -> torch.Tensor:
        return self.world.hidden_buf.view(self.R, self.NvS, self.H)

    def weight_slots(self) -> torch.Tensor:
        return self.world.meta_buf.view(self.R, self._mcp)[:, :self.NvS].view(torch.float32)

    def destroy(self):
        for b in self.buffers:
            b.destroy()


class _GroupDispatch(torch.autograd.Function):
    """tokens [R,S,H] (+ weights [R,S,K]) -> rows [R,NvS,H] (+ slots [R,NvS])."""

    @staticmethod
    def forward(ctx, group, x_all, w_all, topk_all, tpe):
        R = group.R
        group.world.hidden_buf.zero_()
        group.world.meta_buf.zero_()
        plans, cus = [], []
        for r in range(R):
            _, _, cu, plan = group.buffers[r].dispatch(
                x_all[r].contiguous(), None if w_all is None else w_all[r].contiguous(),
                topk_all, tpe, zero_copy=True, router_weights_zero_copy=True)
            plans.append(plan)
            cus.append(cu)
        ctx.group, ctx.plans, ctx.has_w = group, plans, w_all is not None
        group.last_plans, group.last_cu_seqlens = plans, torch.stack(cus)
        hidden = group.shards().clone()
        slots = group.weight_slots().clone() if w_all is not None else None
        ctx.mark_non_differentiable(group.last_cu_seqlens)
        return hidden, slots, group.last_cu_seqlens

    @staticmethod
    def backward(ctx, g_hidden, g_slots, _g_cu):
        group = ctx.group
        group.shards().copy_(g_hidden.to(torch.bfloat16))
        if ctx.has_w:
            group.weight_slots().copy_(g_slots if g_slots is not None else 0.0)
        gx, gw = [], []
        for r in range(group.R):
            b = group.buffers[r]
            out, w_back, _ = b.combine(
                plan=ctx.plans[r], hidden_nvsh=b.hidden_nvsh_buffer_view,
                route_weights_nvs=b.router_weight_buffer_view if ctx.has_w else None,
                zero_copy=True, router_weights_zero_copy=True)
            gx.append(out)
            gw.append(w_back)
        return (None, torch.stack(gx), torch.stack(gw) if ctx.has_w else None, None, None)


class _GroupCombine(torch.autograd.Function):
    """expert outputs [R,NvS,H] -> token-major [R,S,H] (unweighted K-sum)."""

    @staticmethod
    def forward(ctx, group, plans, y_all):
        group.shards().copy_(y_all.to(torch.bfloat16))
        outs = []
        for r in range(group.R):
            b = group.buffers[r]
            out, _, _ = b.combine(plan=plans[r], hidden_nvsh=b.hidden_nvsh_buffer_view, zero_copy=True)
            outs.append(out)
        ctx.group, ctx.plans = group, plans
        return torch.stack(outs)

    @staticmethod
    def backward(ctx, g_out):
        group = ctx.group
        group.world.hidden_buf.zero_()
        for r in range(group.R):
            group.buffers[r].dispatch(g_out[r].to(torch.bfloat16).contiguous(), plan=ctx.plans[r],
                                      zero_copy=True)
        return None, None, group.shards().clone()


class _GroupPrefetch(torch.autograd.Function):
    """fp32 master weights [R,epn,H,H'] -> bf16 compute views [R,2*epn,H,H']:
    each rank's local experts followed by its prefetch slots.  Backward is
    ``reduce_grad``: the slots' grads are summed into their owners' grads in
    fp32."""

    @staticmethod
    def forward(ctx, group, experts_to_copy, master):
        R, epn = group.R, group.epn
        local = master.to(torch.bfloat16).contiguous()
        pool = torch.zeros_like(local)
        for r in range(R):     # a rank's slots filled from all owners in one launch
            launch_prefetch_pull((local,) * 3, (pool,) * 3, experts_to_copy, rank=r)
        ctx.group, ctx.etc = group, experts_to_copy
        return torch.cat([local, pool], dim=1)

    @staticmethod
    def backward(ctx, g_views):
        group = ctx.group
        R, epn = group.R, group.epn
        grad = g_views[:, :epn].float().contiguous()
        slots = g_views[:, epn:].float().contiguous()
        for r in range(R):
            # every rank reads before any rank clears (a barrier in the reference): only
            # the summing half runs here, the slot grads are temporaries nobody reads again
            launch_grad_reduce(grad[r], slots, ctx.etc, rank=r, phase="reduce")
        return None, None, grad


class _GroupExpertFFN(torch.autograd.Function):
    """Rows of every rank through its experts on the matrix cores.

    fp32 master weights in the orientation the kernels read: gate / up
    [R, epn, H', H], down [R, epn, H, H'].  Forward: bf16 compute views (local
    experts, then the prefetch slots filled by ``launch_prefetch_pull``), then per rank
    the fused gate/up GEMM and the down GEMM with the route weight applied.
    Backward: the grouped gradient GEMMs per rank, then ``launch_grad_reduce``
    sums every slot's fp32 weight gradient into its owner's."""

    @staticmethod
    def forward(ctx, group, experts_to_copy, cu_all, rows_all, slots_all, gate_m, up_m, down_m):
        R, tp = group.R, group.world.token_padding
        local = [m.detach().to(torch.bfloat16).contiguous() for m in (gate_m, up_m, down_m)]
        pools = [torch.zeros_like(t) for t in local]
        for r in range(R):     # a rank's slots filled from all owners in one launch
            launch_prefetch_pull(tuple(local), tuple(pools), experts_to_copy, rank=r)
        views = [torch.cat([l, p], dim=1) for l, p in zip(local, pools)]      # [R, 2*epn, ...]
        outs, saved = [], []
        for r in range(R):
            y, keep = ffn.grouped_ffn_hip_forward(rows_all[r], None if slots_all is None else slots_all[r],
                                                  cu_all[r], views[0][r], views[1][r], views[2][r],
                                                  token_padding=tp)
            outs.append(y)
            saved.append(keep)
        ctx.group, ctx.etc, ctx.cu_all, ctx.views, ctx.saved = group, experts_to_copy, cu_all, views, saved
        ctx.rows_all, ctx.slots_all = rows_all, slots_all
        return torch.stack(outs)

    @staticmethod
    def backward(ctx, g_out):
        group = ctx.group
        R, epn, tp = group.R, group.epn, group.world.token_padding
        g_out = g_out.to(torch.bfloat16).contiguous()
        drows, dslots, dw = [], [], ([], [], [])
        for r in range(R):
            res = ffn.grouped_ffn_hip_backward(
                g_out[r], ctx.rows_all[r], None if ctx.slots_all is None else ctx.slots_all[r],
                ctx.cu_all[r], ctx.views[0][r], ctx.views[1][r], ctx.views[2][r], ctx.saved[r],
                token_padding=tp, skip_unused_slots=True)   # grad reduce reads occupied slots only
            drows.append(res[0])
            dslots.append(res[1])
            for acc, g in zip(dw, res[2:]):
                acc.append(g)                                                   # [2*epn, ...] fp32
        grads = []
        for per_rank in dw:
            full = torch.stack(per_rank)                                        # [R, 2*epn, ...]
            own = full[:, :epn].contiguous()
            slots = full[:, epn:].contiguous()
            for r in range(R):     # every rank reads before any rank would clear: summing half only
                launch_grad_reduce(own[r], slots, ctx.etc, rank=r, phase="reduce")
            grads.append(own)
        return (None, None, None, torch.stack(drows),
                None if ctx.slots_all is None else torch.stack(dslots), *grads)


def group_expert_ffn_hip(group, experts_to_copy, cu_all, rows_all, slots_all, gate_m, up_m, down_m):
    """rows [R,NvS,H] bf16, slots [R,NvS] fp32 | None, cu_all [R,2*epn]; fp32 masters gate / up
    [R,epn,H',H], down [R,epn,H,H'] -> expert outputs [R,NvS,H] bf16.  Differentiable in rows,
    slots and the three masters; needs token_padding % 128 == 0 and H, H' multiples of 256."""
    return _GroupExpertFFN.apply(group, experts_to_copy, cu_all, rows_all, slots_all, gate_m, up_m, down_m)


def group_dispatch(group, x_all, w_all, topk_all, tpe):
    """-> (rows [R,NvS,H], weight slots [R,NvS] | None, cu_seqlens [R,2*epn], plans)"""
    hidden, slots, cu = _GroupDispatch.apply(group, x_all, w_all, topk_all, tpe)
    return hidden, slots, cu, group.last_plans


def group_combine(group, plans, y_all):
    return _GroupCombine.apply(group, plans, y_all)


def group_compute_views(group, experts_to_copy, master_weights):
    return _GroupPrefetch.apply(group, experts_to_copy, master_weights)
