"""moonep_amd top-level API: the ``Buffer`` of reference moonep/api.py on one
MI355X.

Same constructor, methods, argument meaning, return tuples and assertion
behaviour as reference moonep/api.py:430-1208::

    buffer = Buffer(S, H, K, E, num_ep_ranks, token_padding=128, rank=r, world=world)
    hidden_nvsh, w_nvs, cu_seqlens, plan = buffer.dispatch(hidden_sh, w_sk, topk_sk, tpe)
    buffer.prefetch_weight(plan=plan, local_gate_weight=..., gate_prefetch_buffer=..., ...)
    out_sh, w_sk_back, _ = buffer.combine(plan=plan, hidden_nvsh=ffn_out, route_weights_nvs=w_nvs)
    buffer.reduce_grad(plan=plan, local_gate_grad=..., gate_reduce_buffer=..., ...)
    buffer.destroy()

One GPU stands in for the R expert-parallel ranks.  What that changes:

* the ranks' communication shards are one ``[R * NvS, H]`` tensor in local
  HBM (plus an ``[R * meta_chunk]`` int32 tensor for the route-weight slots and
  the gathered count table) instead of peer-mapped symmetric memory: an
  ``EmulatedWorld``.  ``rank=`` says which rank a Buffer plays (default: the
  ``torch.distributed`` rank if a group is initialised, else 0);
* a caller written against ``moonep.Buffer`` -- per-rank ``topk_experts_sk[S, K]``
  and ``tokens_per_expert[E]`` -- runs unchanged when every rank is driven by its
  own host thread on a world made with ``host_threads=True``
  (``EmulatedWorld.run_ranks`` starts them): the points where the reference
  synchronises its ranks (count all-gather, after the row writes, before combine
  reads, between the read and the clear of ``reduce_grad``) become thread
  rendezvous that also order the ranks' streams, so the count table, the
  fresh plan's duplicate groups and every shard are complete when they are read;
* one host thread can still drive a rank (or all of them in turn) by passing
  what the gather would have produced: ``tokens_per_expert[R, E]``, and
  ``topk_experts_sk[R, S, K]`` when the plan's duplicate groups are wanted.
  With per-rank ``[S, K]`` routing and no host threads the other ranks' ``dst``
  are unknown: the plan is then marked as having no duplicate map and the
  kernels that need one (``launch_dispatch_epilogue``, ``launch_combine_prologue``)
  refuse it.  Several Buffers sharing a world from one thread must use
  ``zero_copy=True``: a copy-out taken right after one rank's dispatch would
  miss the rows the other ranks have not written yet;
* the duplicate expansion / pre-reduction that the reference runs as separate
  destination-side kernels is folded into dispatch and combine: dispatch
  writes all K copies, combine groups and rounds exactly as the reference's
  prologue + combine pair does, so outputs are bit-identical; the standalone
  kernels stay available as ``launch_dispatch_epilogue`` /
  ``launch_combine_prologue``;
* ``num_sms`` given explicitly bounds every kernel of this Buffer to that many
  compute units: the comm stream is created with a CU mask and all operators
  (synchronous ones too, the caller's stream then waits for them) launch on
  it -- the reference's "communication on 32 SMs beside the expert GEMMs".
  Left at ``None`` the kernels use the whole GPU on the caller's stream;
* ``inter_rank_sync`` selects whether a threaded world's rendezvous are taken;
  ``enable_pdl`` and ``comm_stream_priority`` are validated like the reference
  and otherwise have no effect (HIP kernels on one stream run back to back; all
  streams stay at the default priority).
"""

from __future__ import annotations

import logging
import os
import threading
import warnings
import weakref

import torch

from .combine import launch_combine, launch_combine_prologue  # noqa: F401
from .dispatch import (check_dispatch_inputs, launch_build_dedup, launch_dispatch,  # noqa: F401
                       launch_dispatch_epilogue)
from .grad_reduce import launch_grad_reduce
from .planning import (MoonEPCommPlan, allocate_launch_scratch, allocate_planning_outputs,
                       launch_planning, launch_planning_all_ranks)
from .prefetch import _ELEM_TYPES, launch_prefetch

logger = logging.getLogger(__name__)


def _lib_init_device() -> None:
    from . import _lib
    _lib.init_device()


def _align_up(x: int, alignment: int) -> int:
    return ((x + alignment - 1) // alignment) * alignment


def _rank_stride_of(pool: torch.Tensor, what: str = "pool") -> int:
    """Elements between two ranks' blocks of an all-rank pool ``[R, ...]``.

    The kernels address rank r's block as ``base + r * stride``; the block itself must be
    dense.  Blocks may be spaced apart (a caller that carves pools out of a larger arena)
    as long as they do not overlap, every block starts on a 16-byte boundary and the last
    one ends inside the storage -- what reference moonep/api.py:85-97 asks of a pool."""
    assert pool.is_cuda and pool.ndim >= 2 and pool.shape[0] > 0, f"{what}: not an [R, ...] device tensor"
    block = pool[0]
    assert block.is_contiguous(), f"{what}: pools must be contiguous within each rank"
    stride, size, width = int(pool.stride(0)), block.numel(), pool.element_size()
    assert 0 < size <= stride, f"{what}: rank payloads must not overlap"
    assert (stride * width) % 16 == 0 and pool.data_ptr() % 16 == 0, \
        f"{what}: pools must be 16-byte aligned rank by rank"
    assert stride * width < (1 << 40), f"{what}: rank stride too large"
    end = pool.storage_offset() + stride * (int(pool.shape[0]) - 1) + size
    assert end * width <= pool.untyped_storage().nbytes(), f"{what}: last rank's block leaves the storage"
    return stride


def _check_local_pool_pairs(what: str, locals_, pools, epn: int, R: int, *, dtypes=None,
                            fixed_ndim: int | None = 3) -> None:
    """The (this rank's tensor, all-rank pool) pairs of one operator call.

    Each local tensor is dense ``[epn, ...]`` (exactly ``fixed_ndim`` dimensions when given)
    of a dtype in ``dtypes``; its pool has the same dtype and device, the shape
    ``[R, epn, ...]`` with the local tensor's trailing dimensions, and a valid rank stride."""
    for which, (local, pool) in enumerate(zip(locals_, pools, strict=True)):
        tag = f"{what}[{which}]"
        if dtypes is not None:
            assert local.dtype in dtypes, f"{what}: unsupported weight dtype {local.dtype}"
        assert local.is_contiguous(), f"{tag}: local tensor must be contiguous"
        if fixed_ndim is not None:
            assert local.ndim == fixed_ndim, f"{tag}: local tensor must have {fixed_ndim} dimensions"
        assert local.ndim >= 2 and int(local.shape[0]) == epn, f"{tag}: local tensor must be [epn={epn}, ...]"
        assert pool.dtype == local.dtype and pool.device == local.device, \
            f"{tag}: pool and local tensor differ in dtype or device"
        assert tuple(pool.shape) == (R, epn, *local.shape[1:]), \
            f"{tag}: pool must be [R={R}, epn={epn}, {', '.join(str(int(x)) for x in local.shape[1:])}]"
        _rank_stride_of(pool, tag)


def _num_sms_dedup_from_env(max_sms: int) -> int:
    """CU count for the standalone duplicate kernels: ``MOONEP_NUM_SMS_DEDUP`` when
    set (an integer in [1, max_sms]), else all of them."""
    text = os.environ.get("MOONEP_NUM_SMS_DEDUP", "")
    if text == "":
        return max_sms
    if not text.lstrip("+-").isdigit():
        raise ValueError(f"MOONEP_NUM_SMS_DEDUP must be an integer in [1, {max_sms}], got {text!r}")
    value = int(text)
    if value < 1 or value > max_sms:
        raise ValueError(f"MOONEP_NUM_SMS_DEDUP must be in [1, {max_sms}], got {value}")
    return value


def _check_num_sms(num_sms, max_sms: int) -> int:
    """``num_sms`` as the reference validates it (moonep/api.py:231-248): type and
    sign before anything touches the device, default min(32, CUs)."""
    if num_sms is None:
        return min(32, max_sms)
    if isinstance(num_sms, bool) or not isinstance(num_sms, int):
        raise TypeError(f"num_sms must be a positive int, got {type(num_sms).__name__}")
    if num_sms < 1:
        raise ValueError(f"num_sms must be a positive int, got {num_sms}")
    if num_sms > max_sms:
        raise ValueError(f"num_sms ({num_sms}) must not exceed the device SM count ({max_sms})")
    return num_sms


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
    dispatched rows just as R GPUs see each other's symmetric memory.

    ``host_threads=True`` prepares the world for R host threads, one per rank,
    each running the reference's per-rank call sequence: ``rendezvous`` is then
    the emulation of the reference's cross-rank barriers (it blocks the calling
    thread until all R ranks have arrived and makes every rank's stream wait
    for the work the other ranks enqueued before arriving).  Without it
    ``rendezvous`` does nothing.
    """

    def __init__(self, S: int, H: int, K: int, E: int, R: int, token_padding: int = 128,
                 device=None, host_threads: bool = False):
        assert E % R == 0, f"E ({E}) must be divisible by R ({R})"
        epn = E // R
        self.S, self.H, self.K, self.E, self.R, self.token_padding = S, H, K, E, R, token_padding
        self.NvS = _align_up(S * K + (token_padding - 1) * 2 * epn, token_padding)
        self.NvS_padded = self.NvS
        self.layout = meta_layout(S, K, E, R, self.NvS)
        dev = torch.device("cuda", torch.cuda.current_device()) if device is None else device
        self.device = dev
        self.hidden_buf = torch.empty(R * self.NvS_padded, H, dtype=torch.bfloat16, device=dev)
        self.meta_buf = torch.zeros(R * self.layout["meta_chunk_padded"], dtype=torch.int32,
                                    device=dev)
        # every rank's dst, deposited by its fresh planning: what the duplicate-group
        # builder of every destination reads (the reference publishes the same
        # provenance as src_info in the peers' meta chunks, planning.py:1036-1041)
        self.dst_all = torch.zeros(R, S * K, dtype=torch.int32, device=dev)
        self.attached = 0                      # Buffers created on this world
        self.host_threads = bool(host_threads) and R > 1
        self._barrier = threading.Barrier(R) if self.host_threads else None
        self._arrived = [None] * R             # per rank: event recorded on arrival
        # dup_counts tensors of plans without a duplicate map, by id (a tensor's == is
        # elementwise, so a WeakSet cannot hold them)
        self._no_dedup = weakref.WeakValueDictionary()

    def matches(self, S, H, K, E, R, token_padding) -> bool:
        return (self.S, self.H, self.K, self.E, self.R, self.token_padding) == \
            (S, H, K, E, R, token_padding)

    # -- gathered tokens_per_expert ------------------------------------------
    def tpe_table(self, rank: int) -> torch.Tensor:
        """The ``[R, E]`` count table inside ``rank``'s meta chunk (at TPE_OFF)."""
        mcp, off = self.layout["meta_chunk_padded"], self.layout["TPE_OFF"]
        return self.meta_buf[rank * mcp + off: rank * mcp + off + self.R * self.E].view(self.R, self.E)

    def deposit_tokens_per_expert(self, rank: int, row: torch.Tensor) -> None:
        """Write ``rank``'s ``[E]`` counts into every rank's table, as the
        reference's planner does into its peers' meta chunks (planning.py:577-583)."""
        mcp, off = self.layout["meta_chunk_padded"], self.layout["TPE_OFF"] + rank * self.E
        self.meta_buf.view(self.R, mcp)[:, off: off + self.E].copy_(row.reshape(1, self.E))

    # -- cross-rank barrier ------------------------------------------------------
    def rendezvous(self, rank: int) -> None:
        """All R host threads meet here (no-op without ``host_threads``): work that
        any rank enqueued before arriving is ordered before work that any rank
        enqueues after leaving, whatever streams the ranks use."""
        if not self.host_threads:
            return
        stream = torch.cuda.current_stream()
        self._arrived[rank] = stream.record_event()
        self._barrier.wait()
        for ev in self._arrived:
            stream.wait_event(ev)
        self._barrier.wait()       # nobody re-records before everybody has waited

    def run_ranks(self, fn, *, timeout: float = 120.0):
        """Run ``fn(rank)`` on R host threads (one per rank) and return the list of
        results; the first exception of any rank is re-raised.  A rank that fails
        breaks the barrier so that the others do not wait for it."""
        assert self.host_threads, "run_ranks needs EmulatedWorld(..., host_threads=True)"
        results, errors = [None] * self.R, []
        device = self.device

        def body(r):
            try:
                torch.cuda.set_device(device)
                results[r] = fn(r)
            except BaseException as exc:  # noqa: BLE001 - reported to the caller below
                errors.append((r, exc))
                self._barrier.abort()

        threads = [threading.Thread(target=body, args=(r,), name=f"moonep-rank{r}") for r in range(self.R)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout)
        alive = [t.name for t in threads if t.is_alive()]
        if errors:
            first = [e for e in errors if not isinstance(e[1], threading.BrokenBarrierError)] or errors
            self._barrier.reset()
            raise first[0][1]
        assert not alive, f"rank threads did not finish within {timeout} s: {alive}"
        return results

    # -- plans without a duplicate map ----------------------------------------------
    def mark_no_dedup(self, plan: MoonEPCommPlan) -> None:
        self._no_dedup[id(plan.dup_counts)] = plan.dup_counts

    def has_dedup(self, plan: MoonEPCommPlan) -> bool:
        return self._no_dedup.get(id(plan.dup_counts)) is not plan.dup_counts


def _create_context(S: int, H: int, K: int, E: int, num_ep_ranks: int, num_sms=None,
                    token_padding: int = 128, group=None, rank=None, world=None) -> dict:
    """Validate the configuration, allocate (or attach to) the communication
    buffers and every scratch buffer a launcher of this context uses.

    ``num_sms`` is validated before anything touches the device, as in
    reference moonep/api.py:231-248; shape arithmetic as :260-347.
    """
    if num_sms is not None and (isinstance(num_sms, bool) or not isinstance(num_sms, int)):
        raise TypeError(f"num_sms must be a positive int, got {type(num_sms).__name__}")
    if num_sms is not None and num_sms < 1:
        raise ValueError(f"num_sms must be a positive int, got {num_sms}")
    device = torch.cuda.current_device()
    max_sms = torch.cuda.get_device_properties(device).multi_processor_count
    num_sms = _check_num_sms(num_sms, max_sms)

    R = num_ep_ranks
    if rank is None:
        import torch.distributed as dist
        rank = dist.get_rank(group=group) if dist.is_available() and dist.is_initialized() else 0
    assert isinstance(rank, int) and 0 <= rank < R, f"rank must be in [0, {R}), got {rank}"
    num_sms_dedup = _num_sms_dedup_from_env(max_sms)

    assert E % R == 0, f"E ({E}) must be divisible by R ({R})"
    assert isinstance(token_padding, int) and token_padding > 0, \
        f"token_padding must be a positive int, got {token_padding}"
    epn, N = E // R, S * K
    token_padding_extra = (token_padding - 1) * 2 * epn
    NvS = _align_up(N + token_padding_extra, token_padding)
    int32_max = 2**31 - 1
    assert 0 < N < int32_max, (
        f"planning requires 0 < S*K < int32_max: S={S}, K={K}, S*K={N}, int32_max={int32_max}"
    )
    # one value past the last slot, R * NvS, marks an entry that nobody copies (an
    # invalid expert id): it has to be an int32 too
    assert R * NvS <= int32_max, f"dst encoding requires R*NvS <= int32_max, got {R * NvS}"
    _lib_init_device()
    if world is None:
        world = EmulatedWorld(S, H, K, E, R, token_padding)
    else:
        assert world.matches(S, H, K, E, R, token_padding), "world was built for another shape"
    world.attached += 1
    NvS_padded, lay = world.NvS_padded, world.layout
    mcp = lay["meta_chunk_padded"]
    max_hidden_index = (R - 1) * NvS_padded + NvS - 1
    assert max_hidden_index <= int32_max, (
        f"dst rank-stride indexing would overflow int32: max_index={max_hidden_index}"
    )
    first_row, first_slot = rank * NvS_padded, rank * mcp + lay["WEIGHTS_OFF"]
    ctx = dict(
        rank=rank, group=group, R=R, E=E, S=S, K=K, H=H, N=N, NvS=NvS, NvS_capacity=N,
        NvS_padded=NvS_padded, num_sms=num_sms, num_sms_dedup=num_sms_dedup, max_sms=max_sms,
        token_padding=token_padding, token_padding_extra=token_padding_extra, device=device,
        world=world, hidden_buf=world.hidden_buf, meta_buf=world.meta_buf, meta_chunk_padded=mcp,
        hidden_buf_local=world.hidden_buf[first_row: first_row + NvS],
        weights_buf_local=world.meta_buf[first_slot: first_slot + NvS],
    )
    for key in ("WEIGHTS_OFF", "TPE_OFF", "PLAN_OFF", "TOPK0_OFF", "ORDER_OFF", "ORDER0_OFF",
                "BARRIER_OFF", "SRC_INFO_OFF"):
        ctx[key] = lay[key]
    allocate_launch_scratch(ctx)
    if rank == 0:
        logger.info(
            "moonep_amd buffers: R=%d S=%d H=%d E=%d K=%d NvS=%d hidden=%.2f MiB/rank "
            "meta=%.2f KiB/rank", R, S, H, E, K, NvS, NvS_padded * H * 2 / 2**20, mcp * 4 / 2**10)
    return ctx


_LIMITED_STREAMS: dict = {}
_LIMITED_LOCK = threading.Lock()


def _limited_stream(device: int, num_cus: int):
    """(raw handle, torch stream) of THE stream of ``device`` that is bound to
    ``num_cus`` compute units.  One per (device, num_cus), shared by the Buffers
    that ask for it.  The library owns these streams (torch only wraps the handle)
    and destroys them when the interpreter exits (``_release_limited_streams``): a
    process that ended with such a queue still open crashed inside a profiler's exit
    handlers.  For that to be safe no tensor is ever ``record_stream``-ed on them --
    torch's allocator would touch the stream again when such a tensor is freed,
    possibly after the stream is gone -- see ``Buffer._on_comm_stream``."""
    import atexit
    import ctypes

    from . import _lib
    key = (int(device), int(num_cus))
    with _LIMITED_LOCK:
        if key not in _LIMITED_STREAMS:
            handle = ctypes.c_void_p()
            with torch.cuda.device(device):
                _lib.check(_lib.lib().mep_stream_create_limited(num_cus, ctypes.byref(handle)),
                           "mep_stream_create_limited")
            if not _LIMITED_STREAMS:
                atexit.register(_release_limited_streams)
            _LIMITED_STREAMS[key] = (handle.value, torch.cuda.ExternalStream(handle.value, device=device))
        return _LIMITED_STREAMS[key]


def _release_limited_streams() -> None:
    """Wait for the device(s) and destroy every CU-masked stream this process made.
    Runs at interpreter exit; may also be called once no Buffer with ``num_sms`` is in use."""
    from . import _lib
    with _LIMITED_LOCK:
        streams = dict(_LIMITED_STREAMS)
        _LIMITED_STREAMS.clear()
    for (device, _), (handle, _) in streams.items():
        try:
            with torch.cuda.device(device):
                torch.cuda.synchronize()
                _lib.lib().mep_stream_destroy(handle)
        except Exception:  # noqa: BLE001 - the process is ending; nothing to report to
            pass


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
        self._limited_stream = None      # raw handle of a CU-masked comm stream, if any
        self._inflight = []              # (event, tensors) of asynchronous work on such a stream
        self._destroyed = False
        self._ctx = _create_context(S, H, K, E, num_ep_ranks, num_sms=num_sms,
                                    token_padding=token_padding, group=group, rank=rank,
                                    world=world)
        # default priority on purpose: mixed stream priorities are not used on this hardware
        if num_sms is None:
            self._comm_stream = torch.cuda.Stream(device=int(self._ctx["device"]))
        else:
            # an explicit num_sms: every kernel of this Buffer runs on that many CUs
            self._limited_stream, self._comm_stream = _limited_stream(
                int(self._ctx["device"]), int(self._ctx["num_sms"]))

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
        """Wait for this Buffer's work and let go of every buffer it holds (the
        world's memory is freed with its last user).  Calling it again is harmless."""
        if not self._destroyed and self._ctx is not None:
            if self._comm_stream is not None:
                self._comm_stream.synchronize()
            torch.cuda.synchronize()
            world = self._ctx.get("world")
            if world is not None:
                world.attached -= 1
            self._ctx.clear()
        self._ctx = None
        self._comm_stream = None
        self._limited_stream = None      # the stream itself is shared (see _limited_stream)
        self._inflight = []              # everything was waited for above
        self._destroyed = True

    def __del__(self):
        # a half-constructed object has no _destroyed attribute: nothing to release
        if getattr(self, "_destroyed", True):
            return
        if getattr(self, "explicitly_destroy", False):
            warnings.warn("MoonEP Buffer was not destroyed explicitly; resources may leak.",
                          ResourceWarning)
        else:
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

    def _finish(self, tensors, fn, async_finish: bool):
        """Run an operator body: directly on the caller's stream, or -- when the
        result is wanted asynchronously or the Buffer is bound to ``num_sms`` CUs --
        on the comm stream.  Returns the completion event for ``async_finish``,
        else None (the caller's stream then already waits for the work)."""
        if not async_finish and self._limited_stream is None:
            fn()
            return None
        done = self._on_comm_stream(tensors, fn)
        if async_finish:
            return done
        torch.cuda.current_stream().wait_event(done)
        return None

    def _on_comm_stream(self, tensors, fn):
        """Run ``fn`` on the comm stream after the current stream's work and
        return the completion event (reference moonep/api.py:818-851)."""
        main_stream = torch.cuda.current_stream()
        comm = self._comm_stream
        assert comm is not None, "MoonEP Buffer communication stream is not initialized"
        if self._limited_stream is None:
            self._record_streams(tensors, comm)
        comm.wait_event(main_stream.record_event())
        with torch.cuda.stream(comm):
            fn()
            done = comm.record_event()
        if self._limited_stream is not None:
            # A CU-masked stream is the library's and gets destroyed at exit, so the
            # allocator must never hold it: instead of record_stream the tensors are kept
            # alive here until the work on them has finished.  (A synchronous caller's
            # stream waits for `done` at once, which already orders any reuse.)
            if not torch.cuda.is_current_stream_capturing():   # events cannot be queried under capture
                self._inflight = [(ev, ts) for ev, ts in self._inflight if not ev.query()]
            self._inflight.append((done, [t for t in tensors if t is not None]))
        return done

    def _run_dispatch(self, ctx, hidden_sh, route_weights_sk, planning_args, plan, hidden_nvsh,
                      route_weights_nvs, zero_copy, route_weights_zero_copy, sync) -> None:
        world, rank = ctx["world"], int(ctx["rank"])
        dst_all = None
        if planning_args is not None:
            topk, tpe, cu_seqlens = planning_args
            if topk.dim() == 3:
                # every rank's routing is known: plan all ranks in one launch
                # so that this rank's duplicate groups can be built as well
                dst_all, cu, etc, zfr, stats = launch_planning_all_ranks(ctx, topk, tpe)
                plan.dst.copy_(dst_all[rank])
                cu_seqlens.copy_(cu[rank])
                plan.experts_to_copy.copy_(etc)
                plan.zero_fill_ranges.copy_(zfr[rank])
                plan.remote_stats.copy_(stats[rank])
            else:
                if tpe.dim() == 1 and int(ctx["R"]) > 1:
                    # the reference's count all-gather: my row into every rank's
                    # table; the planner reads the table once all rows are in
                    world.deposit_tokens_per_expert(rank, tpe)
                    world.rendezvous(rank)
                    tpe = world.tpe_table(rank)
                launch_planning(ctx, topk.reshape(-1), tpe, cu_seqlens, plan, warm=hidden_sh)
                if world.host_threads:
                    # the other ranks' threads build their duplicate groups from it
                    world.dst_all[rank].copy_(plan.dst)
        launch_dispatch(ctx, hidden_sh, route_weights_sk, plan, build_dedup_map=False,
                        write_dups=True, pdl_trigger=self.enable_pdl)
        if sync:
            world.rendezvous(rank)   # every rank's rows and dst have landed
        if planning_args is not None:
            # duplicate groups are built by the dispatch that follows fresh planning only
            if dst_all is None and world.host_threads and sync:
                dst_all = world.dst_all
            if dst_all is not None:
                launch_build_dedup(ctx, dst_all, plan)
            elif int(ctx["R"]) > 1:
                world.mark_no_dedup(plan)    # the other ranks' dst are not known here
        if not zero_copy:
            hidden_nvsh.copy_(ctx["hidden_buf_local"])
        if route_weights_nvs is not None and not route_weights_zero_copy:
            route_weights_nvs.copy_(ctx["weights_buf_local"].view(torch.float32))

    def _run_combine(self, ctx, hidden_sh, plan, hidden_nvsh, route_weights_nvs, route_weights_sk,
                     zero_copy, router_weights_zero_copy, sync) -> None:
        if not zero_copy:
            ctx["hidden_buf_local"].copy_(hidden_nvsh)
        if route_weights_nvs is not None and not router_weights_zero_copy:
            ctx["weights_buf_local"].copy_(route_weights_nvs.view(torch.int32))
        if sync:
            ctx["world"].rendezvous(int(ctx["rank"]))   # every rank's expert output is in its shard
        launch_combine(ctx, hidden_sh, plan.dst, output_sk=route_weights_sk, mode="two_level",
                       pdl_launch=self.enable_pdl)
        if sync:
            ctx["world"].rendezvous(int(ctx["rank"]))   # nobody overwrites a shard that is still read

    def _check_copy_mode(self, ctx, zero_copy: bool, what: str) -> None:
        """Several Buffers on one world driven from one host thread: a copy taken
        right after this rank's kernel misses what the other ranks write later."""
        world = ctx["world"]
        if not zero_copy and world.attached > 1 and not world.host_threads and int(ctx["R"]) > 1:
            raise AssertionError(
                f"{what}(zero_copy=False) on an EmulatedWorld shared by {world.attached} Buffers "
                "driven from one host thread would copy the shard before the other ranks have "
                "written (or read) their rows: use zero_copy=True, or a world with "
                "host_threads=True and one thread per rank")

    @staticmethod
    def _check_count_gather(ctx, tokens_per_expert, sync: bool) -> None:
        """A per-rank ``tokens_per_expert[E]`` is only a plan input once the other
        ranks' rows have been gathered beside it.  That happens at a rendezvous of R
        rank threads; from a single host thread the other rows of the table would be
        zero or left over from an earlier step and the ranks' plans would disagree
        (rows of different ranks landing on the same slots)."""
        R, E = int(ctx["R"]), int(ctx["E"])
        if R == 1 or tokens_per_expert.numel() != E:
            return
        world = ctx["world"]
        if not (world.host_threads and sync):
            raise NotImplementedError(
                "dispatch(tokens_per_expert[E]) of one rank needs the other ranks' counts: pass the "
                f"gathered tokens_per_expert[R={R}, E={E}], or run every rank on its own host thread "
                "of an EmulatedWorld(host_threads=True) with inter_rank_sync=True")

    # -- public operators ------------------------------------------------------
    def dispatch(self, hidden_sh: torch.Tensor, route_weights_sk=None, topk_experts_sk=None,
                 tokens_per_expert=None, plan: MoonEPCommPlan | None = None,
                 async_finish: bool = False, *, inter_rank_sync: bool = True,
                 zero_copy: bool = False, router_weights_zero_copy: bool = False):
        """Plan (unless ``plan`` is given) and scatter this rank's tokens to
        their expert-grouped slots on every rank.

        Args and return tuple as reference moonep/api.py:713-851:
        ``topk_experts_sk[S, K]`` and ``tokens_per_expert[E]`` of this rank.  The
        other ranks' counts reach the planner through the world (every rank
        deposits its row; complete when the ranks run on host threads of a
        ``host_threads`` world, see the module docstring).  One host thread may
        pass the gathered ``tokens_per_expert[R, E]`` instead, and
        ``topk_experts_sk[R, S, K]`` to get this rank's duplicate groups too.
        Returns ``(hidden_nvsh, route_weights_nvs, cu_seqlens, plan[, event])``.
        """
        ctx = self._require_ctx()
        # the inputs are checked before any kernel (the planner's cache warming
        # included) reads them
        check_dispatch_inputs(ctx, hidden_sh, route_weights_sk)
        self._check_copy_mode(ctx, zero_copy, "dispatch")
        if plan is None:
            assert topk_experts_sk is not None and tokens_per_expert is not None
            assert topk_experts_sk.dtype == torch.int32
            assert topk_experts_sk.device == hidden_sh.device
            N, R = int(ctx["N"]), int(ctx["R"])
            if topk_experts_sk.dim() == 3:
                assert topk_experts_sk.numel() == R * N and topk_experts_sk.is_contiguous()
            else:
                assert topk_experts_sk.numel() == N
                topk_experts_sk = topk_experts_sk.contiguous()
            assert tokens_per_expert.dtype == torch.int32
            assert tokens_per_expert.numel() in (int(ctx["E"]), R * int(ctx["E"]))
            assert tokens_per_expert.is_contiguous()
            assert tokens_per_expert.device == hidden_sh.device
            self._check_count_gather(ctx, tokens_per_expert, bool(inter_rank_sync))
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
                               route_weights_nvs, zero_copy, router_weights_zero_copy,
                               bool(inter_rank_sync))

        tensors = [hidden_sh, route_weights_sk, hidden_nvsh, route_weights_nvs,
                   *self._plan_runtime_tensors(plan)]
        if planning_args is not None:
            tensors.extend(planning_args)
        done = self._finish(tensors, run, async_finish)
        if not async_finish:
            return hidden_nvsh, route_weights_nvs, cu_seqlens, plan
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
        _check_local_pool_pairs("prefetch_weight", local_weights, pools, epn, R, dtypes=_ELEM_TYPES)
        local_scales = (local_gate_scale, local_up_scale, local_down_scale)
        scale_pools = (gate_scale_prefetch_buffer, up_scale_prefetch_buffer,
                       down_scale_prefetch_buffer)
        given = sum(t is not None for t in (*local_scales, *scale_pools))
        assert given in (0, 6), "prefetch_weight scales must be provided together"
        scales = None
        if given:
            _check_local_pool_pairs("prefetch_weight scales", local_scales, scale_pools, epn, R,
                                    fixed_ndim=None)
            scales = tuple(zip(local_scales, scale_pools, strict=True))

        def run():
            launch_prefetch(local_weights, pools, plan.experts_to_copy, scales=scales,
                            rank=int(ctx["rank"]), num_sms=int(ctx["num_sms"]))
            ctx["world"].rendezvous(int(ctx["rank"]))   # every owner has pushed into every pool

        extra = (*local_scales, *scale_pools) if scales else ()
        return self._finish((plan.experts_to_copy, *local_weights, *pools, *extra), run, async_finish)

    def combine(self, plan: MoonEPCommPlan | None = None, hidden_nvsh=None, route_weights_nvs=None,
                async_finish: bool = False, inter_rank_sync: bool = True, *,
                zero_copy: bool = False, router_weights_zero_copy: bool = False):
        """Gather each token's K rows back and sum them (unweighted, fp32) to
        token-major ``[S, H]``; gather the route weights back to ``[S, K]``
        (reference moonep/api.py:986-1119).
        Returns ``(hidden_sh, route_weights_sk | None, event | None)``."""
        ctx = self._require_ctx()
        assert isinstance(plan, MoonEPCommPlan), "Buffer.combine: plan is required"
        self._check_copy_mode(ctx, zero_copy, "combine")
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
                              route_weights_sk, zero_copy, router_weights_zero_copy,
                              bool(inter_rank_sync))

        done = self._finish(
            (hidden_sh, *self._plan_runtime_tensors(plan), hidden_nvsh, route_weights_nvs,
             route_weights_sk), run, async_finish)
        return hidden_sh, route_weights_sk, done

    def reduce_grad(self, plan: MoonEPCommPlan | None = None, async_finish: bool = False, *,
                    local_gate_grad=None, local_up_grad=None, local_down_grad=None,
                    gate_reduce_buffer=None, up_reduce_buffer=None, down_reduce_buffer=None,
                    phase: str = "both"):
        """Sum the weight grads that other ranks accumulated for this rank's
        experts back into its local grads, then zero this rank's own occupied
        slots (reference moonep/api.py:1121-1208).

        ``phase`` (not in the reference) splits the call where the reference has its
        cross-rank barrier (moonep/grad_reduce.py:369-372): "reduce" only sums, "clear"
        only zeroes.  One host thread that plays several ranks on shared pools must run
        "reduce" for every rank before "clear" for any -- a rank's clear wipes slots that
        hold *other* ranks' experts -- so "both" is refused there; ranks on the host
        threads of a ``host_threads`` world meet at a rendezvous between the halves."""
        ctx = self._require_ctx()
        R = int(ctx["R"])
        epn = int(ctx["E"]) // R
        local_grads = (local_gate_grad, local_up_grad, local_down_grad)
        pools = (gate_reduce_buffer, up_reduce_buffer, down_reduce_buffer)
        assert all(t is not None for t in (*local_grads, *pools)), \
            "reduce_grad tensors must be provided together"
        assert isinstance(plan, MoonEPCommPlan), "Buffer.reduce_grad: plan is required"
        assert phase in ("both", "reduce", "clear"), f"phase must be both, reduce or clear, got {phase!r}"
        _check_local_pool_pairs("reduce_grad", local_grads, pools, epn, R, dtypes=(torch.float32,))
        world, rank = ctx["world"], int(ctx["rank"])
        if phase == "both" and R > 1 and world.attached > 1 and not world.host_threads:
            raise AssertionError(
                f"reduce_grad on an EmulatedWorld shared by {world.attached} Buffers driven from one "
                "host thread: this rank's clear would zero slots that other ranks have not summed "
                "yet.  Call reduce_grad(..., phase=\"reduce\") for every rank, then "
                "reduce_grad(..., phase=\"clear\") for every rank, or use a world with "
                "host_threads=True and one thread per rank")

        def launch(which):
            for local, pool in zip(local_grads, pools, strict=True):
                launch_grad_reduce(local, pool, plan.experts_to_copy, rank=rank,
                                   num_sms=int(ctx["num_sms"]), phase=which)

        def run():
            if phase != "both" or not world.host_threads:
                launch(phase)
                return
            # ranks on host threads: every rank reads before any rank clears
            world.rendezvous(rank)
            launch("reduce")
            world.rendezvous(rank)
            launch("clear")

        return self._finish((plan.experts_to_copy, *local_grads, *pools), run, async_finish)
