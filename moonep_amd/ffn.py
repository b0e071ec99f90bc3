"""Expert-side consumer of a rank's dispatched rows on the matrix cores.

The reference leaves the expert FFN to the training framework and fixes only
its contract (reference README.md:43-58): the rows of a rank form ``2*epn``
groups -- the rank's local experts, then its prefetch slots -- whose padded end
offsets are ``cu_seqlens``; group ``g`` uses the ``g``-th matrix of the compute
views.  ``launch_grouped_gemm_nt`` runs one such grouped GEMM straight from the
device-resident ``cu_seqlens`` (no host read, so the whole layer stays
capturable in a HIP graph); ``grouped_ffn_hip`` chains the fused gate/up
(SwiGLU) GEMM and the down GEMM with the route weight applied per row.

Weights are K-contiguous: gate and up views are ``[2*epn, H', H]``, the down
view is ``[2*epn, H, H']`` -- the layout ``x @ W.T`` reads directly.
"""

from __future__ import annotations

import torch

from . import _lib


def launch_grouped_gemm_nt(rows, weights, cu_seqlens, out=None, *, up_weights=None, row_scale=None,
                           token_padding: int = 128):
    """``out[m] = rows[m] @ weights[g(m)].T`` (fp32 accumulation, bf16 out).

    rows [M,K] bf16; weights [G,N,K] bf16; cu_seqlens [G] int32 on the device,
    every entry a multiple of 128.  With ``up_weights`` [G,N,K] the result is
    ``silu(rows @ weights[g].T) * (rows @ up_weights[g].T)``; otherwise
    ``row_scale`` [M] fp32 (optional) multiplies each row.  Rows at or beyond
    ``cu_seqlens[-1]`` are not written (``out`` is zero-filled when allocated
    here).  ``token_padding`` is the padding the plan behind ``cu_seqlens`` was
    made with: the kernel gives every 128-row tile to ONE group, so group ends
    must be multiples of 128 (checked here on the host, no device read).
    """
    assert isinstance(token_padding, int) and token_padding > 0 and token_padding % 128 == 0, (
        f"grouped GEMM needs group ends on 128-row tiles: token_padding must be a multiple of "
        f"128, got {token_padding}")
    assert rows.is_cuda and rows.dtype == torch.bfloat16 and rows.is_contiguous() and rows.dim() == 2
    assert weights.dtype == torch.bfloat16 and weights.is_contiguous() and weights.dim() == 3
    M, K = rows.shape
    G, N, K2 = weights.shape
    assert K2 == K, f"weights must be [G, N, K={K}], got {tuple(weights.shape)}"
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.is_contiguous() and cu_seqlens.numel() == G
    assert cu_seqlens.device == rows.device == weights.device
    if up_weights is not None:
        assert up_weights.shape == weights.shape and up_weights.dtype == torch.bfloat16 \
            and up_weights.is_contiguous() and row_scale is None
    if row_scale is not None:
        assert row_scale.dtype == torch.float32 and row_scale.is_contiguous() and row_scale.numel() == M
    if out is None:
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=rows.device)
    assert out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N)
    rc = _lib.lib().mep_grouped_gemm_nt(
        rows.data_ptr(), weights.data_ptr(), _lib.ptr(up_weights), cu_seqlens.data_ptr(), G,
        out.data_ptr(), _lib.ptr(row_scale), M, N, K, 1 if up_weights is not None else 0,
        _lib.current_stream())
    _lib.check(rc, "mep_grouped_gemm_nt")
    return out


def grouped_ffn_hip(rows, slots, cu_seqlens, gate_t, up_t, down, *, token_padding: int = 128):
    """SwiGLU FFN of one rank's rows.  rows [NvS,H] bf16, slots [NvS] fp32 route
    weights (or None), cu_seqlens [2*epn]; gate_t/up_t [2*epn,H',H], down
    [2*epn,H,H'].  Rows outside every group come out as zeros.  ``token_padding``:
    that of the Buffer whose plan produced ``cu_seqlens`` (a multiple of 128)."""
    hmid = launch_grouped_gemm_nt(rows, gate_t, cu_seqlens, up_weights=up_t,
                                  token_padding=token_padding)
    return launch_grouped_gemm_nt(hmid, down, cu_seqlens, row_scale=slots,
                                  token_padding=token_padding)
