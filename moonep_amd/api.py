"""moonep_amd top-level API: the ``Buffer`` of reference moonep/api.py on one
MI355X.

Same constructor, methods, argument meaning, return tuples and assertion
behaviour as reference moonep/api.py:430-1208, so a caller written against
``moonep.Buffer`` runs unchanged::

    buffer = Buffer(S, H, K, E, num_ep_ranks, token_padding=128, rank=r)
    hidden_nvsh, w_nvs, cu_seqlens, plan = buffer.dispatch(hidden_sh, w_sk, topk_sk, tpe_RE)
    buffer.prefetch_weight(plan=plan, local_gate_weight=..., gate_prefetch_buffer=..., ...)
    out_sh, w_sk_back, _ = buffer.combine(plan=plan, hidden_nvsh=ffn_out, route_weights_nvs=w_nvs)
    buffer.reduce_grad(plan=plan, local_gate_grad=..., gate_reduce_buffer=..., ...)
    buffer.destroy()

What differs, because one GPU stands in for the R expert-parallel ranks:

* the ranks' communication shards are one ``[R * NvS, H]`` tensor in local
  HBM (plus an ``[R * meta_chunk]`` int32 tensor for the route-weight slots)
  instead of peer-mapped symmetric memory; several Buffers of one emulated
  group can share them through ``world=EmulatedWorld(...)``;
* ``rank=`` says which rank this Buffer plays (default: the
  ``torch.distributed`` rank if a group is initialised, else 0);
* ``tokens_per_expert`` is every rank's count table ``[R, E]`` (the reference
  gathers the rows from peers inside its planner);
* the duplicate expansion / pre-reduction that the reference runs as separate
  destination-side kernels is folded into dispatch and combine: dispatch
  writes all K copies, combine groups and rounds exactly as the reference's
  prologue + combine pair does, so outputs are bit-identical; the standalone
  kernels stay available as ``launch_dispatch_epilogue`` /
  ``launch_combine_prologue``;
* ``inter_rank_sync``, ``enable_pdl``, ``num_sms`` and ``comm_stream_priority``
  are validated like the reference and otherwise have no effect (no peers; HIP
  kernels on one stream run back to back; the kernels size their own grids;
  all streams stay at the default priority).
"""

from __future__ import annotations

import logging
import os
import warnings

import torch

from .combine import launch_combine, launch_combine_prologue  # noqa: F401
from .dispatch import launch_build_dedup, launch_dispatch, launch_dispatch_epilogue  # noqa: F401
from .grad_reduce import launch_grad_reduce
from .planning import (MoonEPCommPlan, allocate_planning_outputs, launch_planning,
                       launch_planning_all_ranks)
from .prefetch import _ELEM_TYPES, launch_prefetch

logger = logging.getLogger(__name__)


def _align_up(x: int, alignment: int) -> int:
    return ((x + alignment - 1) // alignment) * alignment


def _validate_rank_strided_pool(pool: torch.Tensor) -> int:
    """A pool is contiguous inside each rank, ranks may be padded apart
    (reference moonep/api.py:85-97)."""
    assert pool.is_cuda and pool.ndim >= 2 and pool.shape[0] > 0
    assert pool[0].is_contiguous(), "pools must be contiguous within each rank"
    rank_numel = pool[0].numel()
    rank_stride = int(pool.stride(0))
    assert rank_numel > 0 and rank_stride >= rank_numel, "rank payloads must not overlap"
    stride_bytes = rank_stride * pool.element_size()
    assert stride_bytes % 16 == 0 and 0 < stride_bytes < (1 << 40)
    assert pool.data_ptr() % 16 == 0, "pools must be 16-byte aligned"
    end = pool.storage_offset() + (pool.shape[0] - 1) * rank_stride + rank_numel
    assert end * pool.element_size() <= pool.untyped_storage().nbytes()
    return rank_stride


def _num_sms_dedup_from_env(max_sms: int) -> int:
    raw = os.environ.get("MOONEP_NUM_SMS_DEDUP")
    if raw is None or raw == "":
        return max_sms
    try:
        value = int(raw)
    except ValueError as exc:
        raise ValueError(
            f"MOONEP_NUM_SMS_DEDUP must be an integer in [1, {max_sms}], got {raw!r}"
        ) from exc
    if not (1 <= value <= max_sms):
        raise ValueError(f"MOONEP_NUM_SMS_DEDUP must be in [1, {max_sms}], got {value}")
    return value


def meta_layout(S: int, K: int, E: int, R: int, NvS: int) -> dict:
    """int32 offsets inside one rank's meta chunk; same arithmetic as
    reference moonep/api.py:298-324 (only the route-weight slots at
    WEIGHTS_OFF are used here, the rest keeps the reference's numbering)."""
    epn = E // R
    N = S * K
    TPE_OFF = _align_up(NvS, 4)
    PLAN_OFF = _align_up(TPE_OFF + R * E, 4)
    planning_out_elems = 3 * E * R + R * (2 * epn) + 2 * R * (2 * epn) + epn * R + 2 * R
    N4 = _align_up(N, 4)
    TOPK0_OFF = _align_up(PLAN_OFF + planning_out_elems, 4)
    ORDER_OFF = TOPK0_OFF + N4
    ORDER0_OFF = ORDER_OFF + N4
    BARRIER_OFF = ORDER0_OFF + N4
    SRC_INFO_OFF = BARRIER_OFF + 3
    logical = SRC_INFO_OFF + NvS
    return dict(WEIGHTS_OFF=0, TPE_OFF=TPE_OFF, PLAN_OFF=PLAN_OFF, TOPK0_OFF=TOPK0_OFF,
                ORDER_OFF=ORDER_OFF, ORDER0_OFF=ORDER0_OFF, BARRIER_OFF=BARRIER_OFF,
                SRC_INFO_OFF=SRC_INFO_OFF, meta_chunk_logical=logical,
                meta_chunk_padded=_align_up(logical, 4))


class EmulatedWorld:
    """The communication memory of one emulated EP group on one GPU: every
    rank's ``[NvS, H]`` bf16 shard and meta chunk, side by side.  Buffers
    created with ``world=`` share it, so R Buffers on one GPU see each other's
    dispatched rows just as R GPUs see each other's symmetric memory."""

    def __init__(self, S: int, H: int, K: int, E: int, R: int, token_padding: int = 128,
                 device=None):
        assert E % R == 0, f"E ({E}) must be divisible by R ({R})"
        epn = E // R
        self.S, self.H, self.K, self.E, self.R, self.token_padding = S, H, K, E, R, token_padding
        self.NvS = _align_up(S * K + (token_padding - 1) * 2 * epn, token_padding)
        self.NvS_padded = self.NvS
        self.layout = meta_layout(S, K, E, R, self.NvS)
        dev = torch.device("cuda", torch.cuda.current_device()) if device is None else device
        self.hidden_buf = torch.empty(R * self.NvS_padded, H, dtype=torch.bfloat16, device=dev)
        self.meta_buf = torch.zeros(R * self.layout["meta_chunk_padded"], dtype=torch.int32,
                                    device=dev)

    def matches(self, S, H, K, E, R, token_padding) -> bool:
        return (self.S, self.H, self.K, self.E, self.R, self.token_padding) == \
            (S, H, K, E, R, token_padding)


def _create_context(S: int, H: int, K: int, E: int, num_ep_ranks: int, num_sms=None,
                    token_padding: int = 128, group=None, rank=None, world=None) -> dict:
    """Validate the configuration and allocate (or attach to) the buffers.

    ``num_sms`` is validated before anything touches the device, as in
    reference moonep/api.py:231-248.
    """
    if num_sms is not None:
        if not isinstance(num_sms, int) or isinstance(num_sms, bool):
            raise TypeError(f"num_sms must be a positive int, got {type(num_sms).__name__}")
        if num_sms <= 0:
            raise ValueError(f"num_sms must be a positive int, got {num_sms}")

    device = torch.cuda.current_device()
    max_sms = torch.cuda.get_device_properties(device).multi_processor_count
    if num_sms is None:
        num_sms = min(32, max_sms)
    if num_sms > max_sms:
        raise ValueError(f"num_sms ({num_sms}) must not exceed the device SM count ({max_sms})")

    R = num_ep_ranks
    if rank is None:
        import torch.distributed as dist
        rank = dist.get_rank(group=group) if dist.is_available() and dist.is_initialized() else 0
    assert isinstance(rank, int) and 0 <= rank < R, f"rank must be in [0, {R}), got {rank}"
    N = S * K
    num_sms_dedup = _num_sms_dedup_from_env(max_sms)

    epn = E // R
    assert E % R == 0, f"E ({E}) must be divisible by R ({R})"
    assert isinstance(token_padding, int) and token_padding > 0, \
        f"token_padding must be a positive int, got {token_padding}"
    NvS_capacity = S * K
    token_padding_extra = (token_padding - 1) * 2 * epn
    NvS = _align_up(NvS_capacity + token_padding_extra, token_padding)
    int32_max = 2**31 - 1
    assert 0 < N < int32_max, (
        f"planning requires 0 < S*K < int32_max: S={S}, K={K}, S*K={N}, int32_max={int32_max}"
    )
    if world is None:
        world = EmulatedWorld(S, H, K, E, R, token_padding)
    else:
        assert world.matches(S, H, K, E, R, token_padding), "world was built for another shape"
    NvS_padded = world.NvS_padded
    lay = world.layout
    mcp = lay["meta_chunk_padded"]
    max_hidden_index = (R - 1) * NvS_padded + NvS - 1
    assert max_hidden_index <= int32_max, (
        f"dst rank-stride indexing would overflow int32: max_index={max_hidden_index}"
    )
    hidden_buf, meta_buf = world.hidden_buf, world.meta_buf
    ctx = {
        "rank": rank, "group": group, "R": R, "E": E, "S": S, "K": K, "H": H, "N": N,
        "NvS": NvS, "NvS_capacity": NvS_capacity, "NvS_padded": NvS_padded,
        "num_sms": num_sms, "num_sms_dedup": num_sms_dedup, "token_padding": token_padding,
        "device": device, "token_padding_extra": token_padding_extra,
        "world": world, "hidden_buf": hidden_buf, "meta_buf": meta_buf,
        "meta_chunk_padded": mcp,
        **{k: lay[k] for k in ("WEIGHTS_OFF", "TPE_OFF", "PLAN_OFF", "TOPK0_OFF", "ORDER_OFF",
                               "ORDER0_OFF", "BARRIER_OFF", "SRC_INFO_OFF")},
        "hidden_buf_local": hidden_buf[rank * NvS_padded: rank * NvS_padded + NvS],
        "weights_buf_local": meta_buf[rank * mcp + lay["WEIGHTS_OFF"]:
                                      rank * mcp + lay["WEIGHTS_OFF"] + NvS],
    }
    if rank == 0:
        logger.info(
            "moonep_amd buffers: R=%d S=%d H=%d E=%d K=%d NvS=%d hidden=%.2f MiB/rank "
            "meta=%.2f KiB/rank", R, S, H, E, K, NvS, NvS_padded * H * 2 / 2**20, mcp * 4 / 2**10)
    return ctx


class Buffer:
    """Owner of the communication buffers and the comm stream; see the module
    docstring for the differences to the reference."""

    def __init__(self, S: int, H: int, K: int, E: int, num_ep_ranks: int, num_sms=None,
                 token_padding: int = 128, group=None, comm_stream_priority: int = -1,
                 enable_pdl: bool = True, explicitly_destroy: bool = False, *,
                 rank: int | None = None, world: EmulatedWorld | None = None):
        assert isinstance(comm_stream_priority, int), (
            f"comm_stream_priority must be an int, got {type(comm_stream_priority).__name__}"
        )
        assert isinstance(enable_pdl, bool), (
            f"enable_pdl must be a bool, got {type(enable_pdl).__name__}"
        )
        self.explicitly_destroy = explicitly_destroy
        self.comm_stream_priority = comm_stream_priority
        self.enable_pdl = enable_pdl
        self._comm_stream = None
        self._destroyed = False
        self._ctx = _create_context(S, H, K, E, num_ep_ranks, num_sms=num_sms,
                                    token_padding=token_padding, group=group, rank=rank,
                                    world=world)
        # default priority on purpose: mixed stream priorities are not used on this hardware
        self._comm_stream = torch.cuda.Stream(device=int(self._ctx["device"]))

    # -- lifecycle -----------------------------------------------------------
    @property
    def destroyed(self) -> bool:
        return self._destroyed

    @property
    def hidden_nvsh_buffer_view(self) -> torch.Tensor:
        """This rank's ``[NvS, H]`` bf16 shard (aliases persistent comm state)."""
        return self._require_ctx()["hidden_buf_local"]

    @property
    def router_weight_buffer_view(self) -> torch.Tensor:
        """fp32 view of this rank's ``[NvS]`` route-weight slots."""
        return self._require_ctx()["weights_buf_local"].view(torch.float32)

    def _require_ctx(self) -> dict:
        assert not self._destroyed, "MoonEP Buffer has been destroyed"
        assert self._ctx is not None, "MoonEP Buffer is not initialized"
        return self._ctx

    def destroy(self) -> None:
        """Synchronize and drop every buffer this object holds.  Idempotent."""
        if self._destroyed:
            return
        ctx = self._ctx
        if ctx is None:
            self._destroyed = True
            return
        if self._comm_stream is not None:
            self._comm_stream.synchronize()
        torch.cuda.synchronize()
        ctx.clear()
        self._ctx = None
        self._comm_stream = None
        self._destroyed = True

    def __del__(self):
        if getattr(self, "_destroyed", True):
            return
        if getattr(self, "explicitly_destroy", False):
            warnings.warn("MoonEP Buffer was not destroyed explicitly; resources may leak.",
                          ResourceWarning)
            return
        try:
            self.destroy()
        except Exception as exc:  # pragma: no cover - interpreter shutdown
            warnings.warn(f"MoonEP Buffer destructor failed to destroy resources: {exc!r}",
                          ResourceWarning)

    # -- helpers -------------------------------------------------------------
    @staticmethod
    def _record_streams(tensors, stream) -> None:
        for t in tensors:
            if t is not None:
                t.record_stream(stream)

    @staticmethod
    def _plan_runtime_tensors(plan: MoonEPCommPlan):
        return (plan.dst, plan.experts_to_copy, plan.zero_fill_ranges, plan.remote_stats,
                plan.dup_groups, plan.dup_loffs, plan.dup_counts)

    def _on_comm_stream(self, tensors, fn):
        """Run ``fn`` on the comm stream after the current stream's work and
        return the completion event (reference moonep/api.py:818-851)."""
        main_stream = torch.cuda.current_stream()
        comm = self._comm_stream
        assert comm is not None, "MoonEP Buffer communication stream is not initialized"
        self._record_streams(tensors, comm)
        comm.wait_event(main_stream.record_event())
        with torch.cuda.stream(comm):
            fn()
            return comm.record_event()

    def _run_dispatch(self, ctx, hidden_sh, route_weights_sk, planning_args, plan, hidden_nvsh,
                      route_weights_nvs, zero_copy, route_weights_zero_copy) -> None:
        dst_all = None
        if planning_args is not None:
            topk, tpe, cu_seqlens = planning_args
            if topk.dim() == 3:
                # every rank's routing is known: plan all ranks in one launch
                # so that this rank's duplicate groups can be built as well
                dst_all, cu, etc, zfr, stats = launch_planning_all_ranks(ctx, topk, tpe)
                r = int(ctx["rank"])
                plan.dst.copy_(dst_all[r])
                cu_seqlens.copy_(cu[r])
                plan.experts_to_copy.copy_(etc)
                plan.zero_fill_ranges.copy_(zfr[r])
                plan.remote_stats.copy_(stats[r])
            else:
                launch_planning(ctx, topk.reshape(-1), tpe, cu_seqlens, plan, warm=hidden_sh)
        launch_dispatch(ctx, hidden_sh, route_weights_sk, plan,
                        build_dedup_map=planning_args is not None, write_dups=True,
                        dst_all_ranks=dst_all, pdl_trigger=self.enable_pdl)
        if not zero_copy:
            hidden_nvsh.copy_(ctx["hidden_buf_local"])
        if route_weights_nvs is not None and not route_weights_zero_copy:
            route_weights_nvs.copy_(ctx["weights_buf_local"].view(torch.float32))

    def _run_combine(self, ctx, hidden_sh, plan, hidden_nvsh, route_weights_nvs, route_weights_sk,
                     zero_copy, router_weights_zero_copy) -> None:
        if not zero_copy:
            ctx["hidden_buf_local"].copy_(hidden_nvsh)
        if route_weights_nvs is not None and not router_weights_zero_copy:
            ctx["weights_buf_local"].copy_(route_weights_nvs.view(torch.int32))
        launch_combine(ctx, hidden_sh, plan.dst, output_sk=route_weights_sk, mode="two_level",
                       pdl_launch=self.enable_pdl)

    # -- public operators ------------------------------------------------------
    def dispatch(self, hidden_sh: torch.Tensor, route_weights_sk=None, topk_experts_sk=None,
                 tokens_per_expert=None, plan: MoonEPCommPlan | None = None,
                 async_finish: bool = False, *, inter_rank_sync: bool = True,
                 zero_copy: bool = False, router_weights_zero_copy: bool = False):
        """Plan (unless ``plan`` is given) and scatter this rank's tokens to
        their expert-grouped slots on every rank.

        Args and return tuple as reference moonep/api.py:713-851.
        ``tokens_per_expert`` is ``[R, E]``; ``topk_experts_sk`` is ``[S, K]``
        for this rank, or ``[R, S, K]`` for all ranks -- then the plan also
        carries this rank's duplicate groups.
        Returns ``(hidden_nvsh, route_weights_nvs, cu_seqlens, plan[, event])``.
        """
        ctx = self._require_ctx()
        if plan is None:
            assert topk_experts_sk is not None and tokens_per_expert is not None
            assert topk_experts_sk.dtype == torch.int32
            N, R = int(ctx["N"]), int(ctx["R"])
            if topk_experts_sk.dim() == 3:
                assert topk_experts_sk.numel() == R * N and topk_experts_sk.is_contiguous()
            else:
                assert topk_experts_sk.numel() == N
                topk_experts_sk = topk_experts_sk.contiguous()
            assert tokens_per_expert.dtype == torch.int32
            assert tokens_per_expert.numel() in (int(ctx["E"]), R * int(ctx["E"]))
            assert tokens_per_expert.is_contiguous()
            plan, cu_seqlens = allocate_planning_outputs(ctx)
            planning_args = (topk_experts_sk, tokens_per_expert, cu_seqlens)
        else:
            cu_seqlens = None
            planning_args = None
            assert isinstance(plan, MoonEPCommPlan)

        hidden_nvsh = (ctx["hidden_buf_local"] if zero_copy
                       else torch.empty_like(ctx["hidden_buf_local"]))
        if route_weights_sk is None:
            route_weights_nvs = None
        elif router_weights_zero_copy:
            route_weights_nvs = ctx["weights_buf_local"].view(torch.float32)
        else:
            route_weights_nvs = torch.empty(ctx["NvS"], dtype=torch.float32,
                                            device=ctx["meta_buf"].device)

        def run():
            self._run_dispatch(ctx, hidden_sh, route_weights_sk, planning_args, plan, hidden_nvsh,
                               route_weights_nvs, zero_copy, router_weights_zero_copy)

        if not async_finish:
            run()
            return hidden_nvsh, route_weights_nvs, cu_seqlens, plan
        tensors = [hidden_sh, route_weights_sk, hidden_nvsh, route_weights_nvs,
                   *self._plan_runtime_tensors(plan)]
        if planning_args is not None:
            tensors.extend(planning_args)
        done = self._on_comm_stream(tensors, run)
        return hidden_nvsh, route_weights_nvs, cu_seqlens, plan, done

    def prefetch_weight(self, plan: MoonEPCommPlan | None = None, async_finish: bool = False, *,
                        local_gate_weight=None, local_up_weight=None, local_down_weight=None,
                        gate_prefetch_buffer=None, up_prefetch_buffer=None,
                        down_prefetch_buffer=None, local_gate_scale=None, local_up_scale=None,
                        local_down_scale=None, gate_scale_prefetch_buffer=None,
                        up_scale_prefetch_buffer=None, down_scale_prefetch_buffer=None):
        """Push this rank's expert weights selected by ``plan`` into every
        rank's prefetch slots (reference moonep/api.py:853-984)."""
        ctx = self._require_ctx()
        assert isinstance(plan, MoonEPCommPlan), "Buffer.prefetch_weight: plan is required"
        R = int(ctx["R"])
        epn = int(ctx["E"]) // R
        local_weights = (local_gate_weight, local_up_weight, local_down_weight)
        pools = (gate_prefetch_buffer, up_prefetch_buffer, down_prefetch_buffer)
        assert all(t is not None for t in (*local_weights, *pools)), \
            "prefetch_weight tensors must be provided together"
        for local, pool in zip(local_weights, pools, strict=True):
            assert local.dtype in _ELEM_TYPES, \
                f"prefetch_weight: unsupported weight dtype {local.dtype}"
            assert local.is_contiguous()
            assert local.ndim == 3 and int(local.shape[0]) == epn
            assert pool.dtype == local.dtype and _validate_rank_strided_pool(pool)
            assert pool.ndim == 4 and tuple(pool.shape[:2]) == (R, epn)
            assert tuple(pool.shape[2:]) == tuple(local.shape[1:])
            assert pool.device == local.device
        local_scales = (local_gate_scale, local_up_scale, local_down_scale)
        scale_pools = (gate_scale_prefetch_buffer, up_scale_prefetch_buffer,
                       down_scale_prefetch_buffer)
        scales = None
        if any(t is not None for t in (*local_scales, *scale_pools)):
            assert all(t is not None for t in (*local_scales, *scale_pools)), \
                "prefetch_weight scales must be provided together"
            for local, pool in zip(local_scales, scale_pools, strict=True):
                assert local.is_contiguous()
                assert local.ndim >= 2 and int(local.shape[0]) == epn
                assert pool.dtype == local.dtype and _validate_rank_strided_pool(pool)
                assert pool.ndim == local.ndim + 1
                assert tuple(pool.shape[:2]) == (R, epn)
                assert tuple(pool.shape[2:]) == tuple(local.shape[1:])
                assert pool.device == local.device
            scales = tuple(zip(local_scales, scale_pools, strict=True))

        def run():
            launch_prefetch(local_weights, pools, plan.experts_to_copy, scales=scales,
                            rank=int(ctx["rank"]), num_sms=int(ctx["num_sms"]))

        if not async_finish:
            run()
            return None
        extra = (*local_scales, *scale_pools) if scales else ()
        return self._on_comm_stream((plan.experts_to_copy, *local_weights, *pools, *extra), run)

    def combine(self, plan: MoonEPCommPlan | None = None, hidden_nvsh=None, route_weights_nvs=None,
                async_finish: bool = False, inter_rank_sync: bool = True, *,
                zero_copy: bool = False, router_weights_zero_copy: bool = False):
        """Gather each token's K rows back and sum them (unweighted, fp32) to
        token-major ``[S, H]``; gather the route weights back to ``[S, K]``
        (reference moonep/api.py:986-1119).
        Returns ``(hidden_sh, route_weights_sk | None, event | None)``."""
        ctx = self._require_ctx()
        assert isinstance(plan, MoonEPCommPlan), "Buffer.combine: plan is required"
        assert hidden_nvsh is not None
        assert hidden_nvsh.dtype == torch.bfloat16
        assert hidden_nvsh.is_contiguous()
        assert tuple(hidden_nvsh.shape) == (int(ctx["NvS"]), int(ctx["H"]))
        if route_weights_nvs is not None:
            assert route_weights_nvs.dtype == torch.float32
            assert route_weights_nvs.is_contiguous()
            assert tuple(route_weights_nvs.shape) == (int(ctx["NvS"]),)
        if zero_copy:
            assert hidden_nvsh.data_ptr() == ctx["hidden_buf_local"].data_ptr(), (
                "combine(zero_copy=True): hidden_nvsh must alias the shard view returned by "
                "dispatch(zero_copy=True)"
            )
        if router_weights_zero_copy and route_weights_nvs is not None:
            assert route_weights_nvs.data_ptr() == ctx["weights_buf_local"].data_ptr(), (
                "combine(router_weights_zero_copy=True): route_weights_nvs must alias the "
                "weights view returned by dispatch(router_weights_zero_copy=True)"
            )
        hidden_sh = torch.empty(int(ctx["S"]), int(ctx["H"]), dtype=hidden_nvsh.dtype,
                                device=hidden_nvsh.device)
        route_weights_sk = (
            torch.empty(int(ctx["S"]), int(ctx["K"]), dtype=torch.float32,
                        device=hidden_nvsh.device)
            if route_weights_nvs is not None else None
        )

        def run():
            self._run_combine(ctx, hidden_sh, plan, hidden_nvsh, route_weights_nvs,
                              route_weights_sk, zero_copy, router_weights_zero_copy)

        if not async_finish:
            run()
            return hidden_sh, route_weights_sk, None
        done = self._on_comm_stream(
            (hidden_sh, *self._plan_runtime_tensors(plan), hidden_nvsh, route_weights_nvs,
             route_weights_sk), run)
        return hidden_sh, route_weights_sk, done

    def reduce_grad(self, plan: MoonEPCommPlan | None = None, async_finish: bool = False, *,
                    local_gate_grad=None, local_up_grad=None, local_down_grad=None,
                    gate_reduce_buffer=None, up_reduce_buffer=None, down_reduce_buffer=None):
        """Sum the weight grads that other ranks accumulated for this rank's
        experts back into its local grads, then zero this rank's own occupied
        slots (reference moonep/api.py:1121-1208)."""
        ctx = self._require_ctx()
        R = int(ctx["R"])
        epn = int(ctx["E"]) // R
        local_grads = (local_gate_grad, local_up_grad, local_down_grad)
        pools = (gate_reduce_buffer, up_reduce_buffer, down_reduce_buffer)
        assert all(t is not None for t in (*local_grads, *pools)), \
            "reduce_grad tensors must be provided together"
        assert isinstance(plan, MoonEPCommPlan), "Buffer.reduce_grad: plan is required"
        for local, pool in zip(local_grads, pools, strict=True):
            assert local.dtype == torch.float32 and local.is_contiguous()
            assert local.ndim == 3 and int(local.shape[0]) == epn
            assert pool.dtype == torch.float32 and _validate_rank_strided_pool(pool)
            assert pool.ndim == 4 and tuple(pool.shape[:2]) == (R, epn)
            assert tuple(pool.shape[2:]) == tuple(local.shape[1:])
            assert pool.device == local.device

        def run():
            for local, pool in zip(local_grads, pools, strict=True):
                launch_grad_reduce(local, pool, plan.experts_to_copy, rank=int(ctx["rank"]),
                                   num_sms=int(ctx["num_sms"]))

        if not async_finish:
            run()
            return None
        return self._on_comm_stream((plan.experts_to_copy, *local_grads, *pools), run)
