"""Expert-weight prefetch host side.

Mirrors reference moonep/prefetch.py:524-543 (``prefetch_retile_nbytes``,
``retile_for_prefetch``) and :632-738 (``launch_prefetch``); the kernel is in
csrc/prefetch.hip.
"""

from __future__ import annotations

import ctypes as C

import torch

from . import _lib

_ELEM_TYPES = {torch.bfloat16: 2, torch.int8: 1, torch.uint8: 1}
M_BLOCK = 128
N_BLOCK = 128


def prefetch_retile_nbytes(per_expert_nbytes: int) -> int:
    """Per-expert byte count rounded up to what ``retile_for_prefetch`` takes."""
    tile = M_BLOCK * N_BLOCK
    return (per_expert_nbytes + tile - 1) // tile * tile


def retile_for_prefetch(t: torch.Tensor) -> torch.Tensor:
    """View a contiguous ``[N, ...]`` tensor as ``[N, 128, X]`` uint8."""
    assert t.is_contiguous(), "retile_for_prefetch requires a contiguous tensor"
    n = int(t.shape[0])
    per_expert = t.nbytes // n if n else 0
    tile = M_BLOCK * N_BLOCK
    assert per_expert % tile == 0, (
        f"retile_for_prefetch: per-expert extent {per_expert} bytes is not a multiple of "
        f"{tile}; allocate {prefetch_retile_nbytes(per_expert)} bytes per expert instead"
    )
    return t.view(torch.uint8).reshape(n, M_BLOCK, -1)


def _validate_pair(local, pool, EPN, R, dtype, device_index) -> None:
    assert local.dtype == dtype and local.is_contiguous(), \
        f"local tensors must be contiguous with dtype {dtype}"
    assert local.ndim == 3 and int(local.shape[0]) == EPN, f"local tensors must be [EPN={EPN}, H, H']"
    assert pool.dtype == dtype, f"prefetch pools must have dtype {dtype}"
    assert pool.ndim == 4 and tuple(pool.shape[:2]) == (R, EPN), \
        f"prefetch pools must have leading shape [R, EPN]=[{R}, {EPN}]"
    assert tuple(pool.shape[2:]) == tuple(local.shape[1:]), \
        "local tensor and prefetch pool trailing shapes must match"
    assert local.device.index == device_index and pool.device.index == device_index, \
        "all prefetch tensors must be on the same CUDA device"
    H, Hp = (int(x) for x in local.shape[1:])
    assert H % M_BLOCK == 0 and Hp % N_BLOCK == 0, (
        f"prefetch tensor trailing dimensions must be multiples of ({M_BLOCK}, {N_BLOCK}), "
        f"got ({H}, {Hp})"
    )
    assert pool[0].is_contiguous(), "pools must be contiguous within each rank"


def launch_prefetch(local_weights, prefetch_buffers, experts_to_copy, rank, num_sms=None,
                    meta_buf=None, meta_stride=None, barrier_off=None, grid_sync_bar=None,
                    scales=None) -> None:
    """One launch pushing rank's owned experts (3 weight tensors, optionally 3
    scale tensors) into every requesting ``pool[dst_rank, slot]``.

    ``num_sms`` and the barrier arguments of the reference are accepted and
    unused: the kernel sizes its own grid and one GPU needs no peer barrier.
    """
    assert len(local_weights) == 3 and len(prefetch_buffers) == 3, \
        "prefetch requires three local weights and three prefetch buffers"
    dtype = local_weights[0].dtype
    assert dtype in _ELEM_TYPES, (
        f"prefetch: unsupported dtype {dtype}; supported: {sorted(str(d) for d in _ELEM_TYPES)}"
    )
    assert local_weights[0].ndim == 3 and prefetch_buffers[0].ndim == 4
    EPN = int(local_weights[0].shape[0])
    R = int(prefetch_buffers[0].shape[0])
    device_index = prefetch_buffers[0].device.index
    assert device_index is not None, "prefetch buffers must be CUDA tensors"
    for lw, pb in zip(local_weights, prefetch_buffers, strict=True):
        _validate_pair(lw, pb, EPN, R, dtype, device_index)
    assert experts_to_copy.dtype == torch.int32 and experts_to_copy.is_contiguous(), \
        "experts_to_copy must be contiguous int32 [R, EPN]"
    assert tuple(experts_to_copy.shape) == (R, EPN), f"experts_to_copy must be [R, EPN]=[{R}, {EPN}]"
    assert experts_to_copy.device.index == device_index
    assert 0 <= int(rank) < R, f"rank must be in [0, {R}), got {rank}"

    locals_, pools = list(local_weights), list(prefetch_buffers)
    if scales is not None:
        assert len(scales) == 3, "prefetch scales must contain three local/pool pairs"
        assert dtype == torch.uint8, "weight and re-tiled scale tensors must share uint8 copy dtype"
        for ls, sp in scales:
            assert ls.is_contiguous() and int(ls.shape[0]) == EPN
            assert tuple(sp.shape[:2]) == (R, EPN) and sp.dtype == ls.dtype
            assert tuple(sp.shape[2:]) == tuple(ls.shape[1:])
            assert ls.device.index == device_index and sp.device.index == device_index
            assert sp[0].is_contiguous()
            retile_for_prefetch(ls)  # same size rule as the reference
            locals_.append(ls)
            pools.append(sp)
    n = len(locals_)
    arr_p = (C.c_void_p * n)
    arr_i = (C.c_int64 * n)
    bytes_per = [t.nbytes // EPN for t in locals_]
    strides = [int(p.stride(0)) * p.element_size() for p in pools]
    rc = _lib.lib().mep_prefetch(
        n, arr_p(*[t.data_ptr() for t in locals_]), arr_p(*[p.data_ptr() for p in pools]),
        arr_i(*strides), arr_i(*bytes_per), experts_to_copy.data_ptr(), int(rank), EPN, R,
        _lib.current_stream(),
    )
    _lib.check(rc, "mep_prefetch")


def launch_prefetch_pull(owner_weights, prefetch_buffers, experts_to_copy, rank, scales=None) -> None:
    """Pull view of ``launch_prefetch`` (not in the reference, whose ranks push): fill the
    occupied prefetch slots of ONE rank from every owner's experts in one launch,
    ``pool[rank, b] = owner_weights[e // epn, e % epn]`` for ``e = experts_to_copy[rank, b] >= 0``.

    ``owner_weights``: three ``[R, epn, H, H']`` tensors holding every rank's local experts
    (what one GPU emulating the R ranks has at hand; rank-strided like a pool);
    ``prefetch_buffers`` and ``scales`` (three ``(owner_scales[R, epn, ...], pool)`` pairs) as
    for ``launch_prefetch``.  Leaves in ``pool[rank]`` exactly what the R owners' pushes
    leave there (the per-rank check of reference tests/test_prefetch.py:448-464)."""
    assert len(owner_weights) == 3 and len(prefetch_buffers) == 3, \
        "prefetch requires three owner weight tensors and three prefetch buffers"
    dtype = owner_weights[0].dtype
    assert dtype in _ELEM_TYPES, (
        f"prefetch: unsupported dtype {dtype}; supported: {sorted(str(d) for d in _ELEM_TYPES)}"
    )
    assert owner_weights[0].ndim == 4 and prefetch_buffers[0].ndim == 4
    R, EPN = (int(x) for x in prefetch_buffers[0].shape[:2])
    device_index = prefetch_buffers[0].device.index
    assert device_index is not None, "prefetch buffers must be CUDA tensors"
    for ow, pb in zip(owner_weights, prefetch_buffers, strict=True):
        assert ow.ndim == 4 and tuple(ow.shape[:2]) == (R, EPN) and ow[0].is_contiguous(), \
            f"owner weights must be [R, EPN]=[{R}, {EPN}] leading, contiguous within each rank"
        _validate_pair(ow[0], pb, EPN, R, dtype, device_index)
        assert (int(ow.stride(0)) * ow.element_size()) % 16 == 0 and ow.data_ptr() % 16 == 0, \
            "owner weights must be 16-byte aligned rank by rank"
    assert experts_to_copy.dtype == torch.int32 and experts_to_copy.is_contiguous(), \
        "experts_to_copy must be contiguous int32 [R, EPN]"
    assert tuple(experts_to_copy.shape) == (R, EPN), f"experts_to_copy must be [R, EPN]=[{R}, {EPN}]"
    assert experts_to_copy.device.index == device_index
    assert 0 <= int(rank) < R, f"rank must be in [0, {R}), got {rank}"
    owners, pools = list(owner_weights), list(prefetch_buffers)
    if scales is not None:
        assert len(scales) == 3, "prefetch scales must contain three owner/pool pairs"
        assert dtype == torch.uint8, "weight and re-tiled scale tensors must share uint8 copy dtype"
        for os_, sp in scales:
            assert tuple(os_.shape[:2]) == (R, EPN) and os_[0].is_contiguous()
            assert tuple(sp.shape) == tuple(os_.shape) and sp.dtype == os_.dtype
            assert os_.device.index == device_index and sp.device.index == device_index
            assert sp[0].is_contiguous()
            retile_for_prefetch(os_[0])  # same size rule as the reference
            owners.append(os_)
            pools.append(sp)
    n = len(owners)
    arr_p = (C.c_void_p * n)
    arr_i = (C.c_int64 * n)
    bytes_per = [t[0].nbytes // EPN for t in owners]
    rc = _lib.lib().mep_prefetch_pull(
        n, arr_p(*[t.data_ptr() for t in owners]),
        arr_i(*[int(t.stride(0)) * t.element_size() for t in owners]),
        arr_p(*[p.data_ptr() for p in pools]),
        arr_i(*[int(p.stride(0)) * p.element_size() for p in pools]),
        arr_i(*bytes_per), experts_to_copy.data_ptr(), int(rank), EPN, R, _lib.current_stream(),
    )
    _lib.check(rc, "mep_prefetch_pull")
