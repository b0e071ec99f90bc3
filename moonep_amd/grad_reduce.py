"""fp32 slot reduction host side; mirrors ``launch_grad_reduce`` of reference
moonep/grad_reduce.py:437-543.  The kernels are in csrc/prefetch.hip."""

from __future__ import annotations

import torch

from . import _lib

M_BLOCK = 128
N_BLOCK = 128


def launch_grad_reduce(local_expert_grads, reduce_buffers, experts_to_copy, rank, num_sms=None,
                       meta_buf=None, meta_stride=None, barrier_off=None,
                       grid_sync_bar=None, *, phase: str = "both") -> None:
    """``local_expert_grads[le] += sum of reduce_buffers[src, b]`` over the
    slots holding expert ``rank*epn+le`` in (src, b)-ascending order, then zero
    ``reduce_buffers[rank, b]`` for every occupied slot b of this rank.

    ``phase`` (not in the reference): "both" (one launch), "reduce" (sum only)
    or "clear" (zero the own occupied slots only).  The reference puts a
    cross-rank barrier between the two halves; whoever drives several ranks on
    one GPU calls "reduce" for every rank, then "clear" for every rank.
    ``num_sms`` and the barrier arguments of the reference are accepted and
    unused.
    """
    flags = {"both": 0, "reduce": _lib.REDUCE_NO_CLEAR, "clear": _lib.REDUCE_CLEAR_ONLY}[phase]
    if reduce_buffers.numel() == 0 or experts_to_copy.numel() == 0:
        return
    assert local_expert_grads.dtype == torch.float32 and local_expert_grads.is_contiguous(), \
        "local_expert_grads must be contiguous fp32 [epn, H, H']"
    assert reduce_buffers.dtype == torch.float32, "reduce_buffers must be fp32 [R, epn, H, H']"
    assert experts_to_copy.dtype == torch.int32 and experts_to_copy.is_contiguous(), \
        "experts_to_copy must be contiguous int32 [R, epn]"
    assert local_expert_grads.ndim == 3, \
        f"local_expert_grads must have rank 3, got shape={tuple(local_expert_grads.shape)}"
    assert reduce_buffers.ndim == 4, \
        f"reduce_buffers must have rank 4, got shape={tuple(reduce_buffers.shape)}"
    assert experts_to_copy.ndim == 2, \
        f"experts_to_copy must have rank 2, got shape={tuple(experts_to_copy.shape)}"
    epn, H, Hp = (int(x) for x in local_expert_grads.shape)
    R, _, bH, bHp = (int(x) for x in reduce_buffers.shape)
    assert tuple(reduce_buffers.shape[:2]) == (R, epn), \
        f"reduce_buffers must have leading shape [R, epn]=[{R}, {epn}]"
    assert tuple(experts_to_copy.shape) == (R, epn), f"experts_to_copy must be [R, epn]=[{R}, {epn}]"
    assert bH == H and bHp == Hp, (
        f"reduce_buffers shape {tuple(reduce_buffers.shape)} incompatible with "
        f"local_expert_grads {tuple(local_expert_grads.shape)}"
    )
    assert 0 <= int(rank) < R, f"rank must be in [0, {R}), got {rank}"
    assert H % M_BLOCK == 0 and Hp % N_BLOCK == 0, \
        f"H and H' must be multiples of ({M_BLOCK}, {N_BLOCK}), got ({H}, {Hp})"
    assert reduce_buffers[0].is_contiguous(), "reduce_buffers must be contiguous within each rank"
    dev = local_expert_grads.device
    assert dev.type == "cuda", "local_expert_grads must be a CUDA tensor"
    assert reduce_buffers.device == dev and experts_to_copy.device == dev
    rc = _lib.lib().mep_grad_reduce(
        local_expert_grads.data_ptr(), reduce_buffers.data_ptr(), int(reduce_buffers.stride(0)),
        experts_to_copy.data_ptr(), int(rank), epn, R, H * Hp, flags, _lib.current_stream(),
    )
    _lib.check(rc, "mep_grad_reduce")
