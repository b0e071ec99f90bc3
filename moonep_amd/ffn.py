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

The backward pass runs on the same kernels with the operands as the passes hold
them: the input gradients read the forward weights in ``[K, N]`` form
(``launch_grouped_gemm_nn``, ``launch_grouped_gemm_dual_nn``), the weight
gradients the activations as ``[rows, features]``
(``launch_grouped_gemm_wgrad_tn``; shapes it does not take go through
``transpose_bf16`` and ``launch_grouped_gemm_wgrad``).  The weight gradients
come out in fp32 ``[2*epn, ...]`` -- local experts first, then the slots --
which is what ``launch_grad_reduce`` sums.
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


def _check_groups(rows, cu_seqlens, token_padding):
    assert isinstance(token_padding, int) and token_padding > 0 and token_padding % 128 == 0, (
        f"grouped GEMM needs group ends on 128-row tiles: token_padding must be a multiple of "
        f"128, got {token_padding}")
    assert rows.is_cuda and rows.dtype == torch.bfloat16 and rows.is_contiguous() and rows.dim() == 2
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.is_contiguous() and cu_seqlens.dim() == 1
    assert cu_seqlens.device == rows.device


def _check_weights(w, G, N=None, K=None):
    assert w.dtype == torch.bfloat16 and w.is_contiguous() and w.dim() == 3 and w.shape[0] == G, (
        f"weights must be contiguous bf16 [G={G}, N, K], got {tuple(w.shape)} {w.dtype}")
    if N is not None:
        assert tuple(w.shape[1:]) == (N, K), f"weights must be [G, {N}, {K}], got {tuple(w.shape)}"


def launch_grouped_swiglu(rows, gate_t, up_t, cu_seqlens, *, save_preactivations=True,
                          token_padding: int = 128):
    """-> (act, gate_pre, up_pre), each [M, H'] bf16: ``act = silu(g) * u`` with
    ``g = rows @ gate_t[grp].T``, ``u = rows @ up_t[grp].T``; the pre-activations
    are what ``launch_swiglu_bwd`` needs (None, None without them)."""
    _check_groups(rows, cu_seqlens, token_padding)
    M, K = rows.shape
    G = cu_seqlens.numel()
    _check_weights(gate_t, G)
    N = gate_t.shape[1]
    _check_weights(gate_t, G, N, K)
    _check_weights(up_t, G, N, K)
    act = torch.zeros(M, N, dtype=torch.bfloat16, device=rows.device)
    gp = torch.zeros_like(act) if save_preactivations else None
    up = torch.zeros_like(act) if save_preactivations else None
    rc = _lib.lib().mep_grouped_swiglu_nt(
        rows.data_ptr(), gate_t.data_ptr(), up_t.data_ptr(), cu_seqlens.data_ptr(), G,
        act.data_ptr(), _lib.ptr(gp), _lib.ptr(up), M, N, K, _lib.current_stream())
    _lib.check(rc, "mep_grouped_swiglu_nt")
    return act, gp, up


def launch_grouped_gemm_dual_nt(a1, w1, a2, w2, cu_seqlens, out=None, *, token_padding: int = 128):
    """``a1 @ w1[grp].T + a2 @ w2[grp].T`` -> [M, N] bf16 (one K loop over both pairs).
    Rows at or beyond ``cu_seqlens[-1]`` are not written (zero when ``out`` is allocated here)."""
    _check_groups(a1, cu_seqlens, token_padding)
    assert a2.shape == a1.shape and a2.dtype == torch.bfloat16 and a2.is_contiguous()
    M, K = a1.shape
    G = cu_seqlens.numel()
    _check_weights(w1, G)
    N = w1.shape[1]
    _check_weights(w1, G, N, K)
    _check_weights(w2, G, N, K)
    if out is None:
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=a1.device)
    assert out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N)
    rc = _lib.lib().mep_grouped_gemm_dual_nt(
        a1.data_ptr(), w1.data_ptr(), a2.data_ptr(), w2.data_ptr(), cu_seqlens.data_ptr(), G,
        out.data_ptr(), M, N, K, _lib.current_stream())
    _lib.check(rc, "mep_grouped_gemm_dual_nt")
    return out


def launch_grouped_gemm_nn(rows, weights_kn, cu_seqlens, out=None, *, row_scale=None, token_padding: int = 128):
    """``out[m] = rows[m] @ weights_kn[g(m)]`` -> [M, N] bf16; weights_kn [G, K, N] bf16
    (the tensor a forward ``launch_grouped_gemm_nt`` took as [G, N', K'] = [G, K, N]: its
    input gradient needs no transposed copy).  Rows at or beyond ``cu_seqlens[-1]`` are
    not written (zero when ``out`` is allocated here)."""
    _check_groups(rows, cu_seqlens, token_padding)
    M, K = rows.shape
    G = cu_seqlens.numel()
    _check_weights(weights_kn, G)
    N = weights_kn.shape[2]
    _check_weights(weights_kn, G, K, N)
    if row_scale is not None:
        assert row_scale.dtype == torch.float32 and row_scale.is_contiguous() and row_scale.numel() == M
    if out is None:
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=rows.device)
    assert out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N)
    rc = _lib.lib().mep_grouped_gemm_nn(rows.data_ptr(), weights_kn.data_ptr(), cu_seqlens.data_ptr(), G,
                                        out.data_ptr(), _lib.ptr(row_scale), M, N, K, _lib.current_stream())
    _lib.check(rc, "mep_grouped_gemm_nn")
    return out


def launch_grouped_gemm_dual_nn(a1, w1_kn, a2, w2_kn, cu_seqlens, out=None, *, token_padding: int = 128):
    """``a1 @ w1_kn[grp] + a2 @ w2_kn[grp]`` -> [M, N] bf16, weights [G, K, N] (one K loop
    over both pairs).  Rows at or beyond ``cu_seqlens[-1]`` are not written."""
    _check_groups(a1, cu_seqlens, token_padding)
    assert a2.shape == a1.shape and a2.dtype == torch.bfloat16 and a2.is_contiguous()
    M, K = a1.shape
    G = cu_seqlens.numel()
    _check_weights(w1_kn, G)
    N = w1_kn.shape[2]
    _check_weights(w1_kn, G, K, N)
    _check_weights(w2_kn, G, K, N)
    if out is None:
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=a1.device)
    assert out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N)
    rc = _lib.lib().mep_grouped_gemm_dual_nn(
        a1.data_ptr(), w1_kn.data_ptr(), a2.data_ptr(), w2_kn.data_ptr(), cu_seqlens.data_ptr(), G,
        out.data_ptr(), M, N, K, _lib.current_stream())
    _lib.check(rc, "mep_grouped_gemm_dual_nn")
    return out


def launch_grouped_gemm_wgrad(at, bt, cu_seqlens, out=None, *, skip_empty_from=None, token_padding: int = 128):
    """Weight gradients from transposed activations: ``out[g] = at[:, rows of g] @
    bt[:, rows of g].T`` -> fp32 [G, Ma, Nb]; at [Ma, M], bt [Nb, M] bf16 with
    the rank's M rows along the contiguous dimension.  A group without rows gets zeros,
    unless its index is >= ``skip_empty_from`` (then it is left unwritten: the slots that
    hold no expert, which ``launch_grad_reduce`` never reads)."""
    _check_groups(at, cu_seqlens, token_padding)
    assert bt.dtype == torch.bfloat16 and bt.is_contiguous() and bt.dim() == 2 and bt.shape[1] == at.shape[1]
    Ma, ld = at.shape
    Nb = bt.shape[0]
    G = cu_seqlens.numel()
    if out is None:
        out = torch.empty(G, Ma, Nb, dtype=torch.float32, device=at.device)
    assert out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (G, Ma, Nb)
    rc = _lib.lib().mep_grouped_gemm_wgrad(at.data_ptr(), bt.data_ptr(), cu_seqlens.data_ptr(), G,
                                           out.data_ptr(), Ma, Nb, ld, G if skip_empty_from is None else skip_empty_from,
                                           _lib.current_stream())
    _lib.check(rc, "mep_grouped_gemm_wgrad")
    return out


def wgrad_tn_supported(Ma: int, Nb: int, G: int) -> bool:
    """Shapes `launch_grouped_gemm_wgrad_tn` takes (an expert's: multiples of 256, G even)."""
    return Ma % 256 == 0 and Nb % 256 == 0 and G % 2 == 0


def launch_grouped_gemm_wgrad_tn(x1, x2, cu_seqlens, out=None, *, skip_empty_from=None, token_padding: int = 128):
    """Weight gradients from the activations as they are: ``out[g] = x1[rows of g].T @
    x2[rows of g]`` -> fp32 [G, Ma, Nb]; x1 [M, Ma], x2 [M, Nb] bf16, no transposed copies.
    ``skip_empty_from`` as in ``launch_grouped_gemm_wgrad``."""
    _check_groups(x1, cu_seqlens, token_padding)
    assert x2.dtype == torch.bfloat16 and x2.is_contiguous() and x2.dim() == 2 and x2.shape[0] == x1.shape[0]
    M, Ma = x1.shape
    Nb = x2.shape[1]
    G = cu_seqlens.numel()
    assert wgrad_tn_supported(Ma, Nb, G), f"needs Ma, Nb multiples of 256 and an even G, got {Ma}, {Nb}, {G}"
    if out is None:
        out = torch.empty(G, Ma, Nb, dtype=torch.float32, device=x1.device)
    assert out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (G, Ma, Nb)
    rc = _lib.lib().mep_grouped_gemm_wgrad_tn(x1.data_ptr(), x2.data_ptr(), cu_seqlens.data_ptr(), G,
                                              out.data_ptr(), Ma, Nb, M, G if skip_empty_from is None else skip_empty_from,
                                              _lib.current_stream())
    _lib.check(rc, "mep_grouped_gemm_wgrad_tn")
    return out


def transpose_bf16(t, out=None):
    """[..., rows, cols] -> [..., cols, rows], contiguous (rows, cols multiples of 64)."""
    assert t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous() and t.dim() >= 2
    rows, cols = t.shape[-2:]
    batch = t.numel() // (rows * cols)
    if out is None:
        out = torch.empty(*t.shape[:-2], cols, rows, dtype=t.dtype, device=t.device)
    assert out.dtype == t.dtype and out.is_contiguous() and tuple(out.shape) == (*t.shape[:-2], cols, rows)
    rc = _lib.lib().mep_transpose_bf16(t.data_ptr(), out.data_ptr(), batch, rows, cols, _lib.current_stream())
    _lib.check(rc, "mep_transpose_bf16")
    return out


def launch_swiglu_bwd(dh, gate_pre, up_pre, row_scale, cu_seqlens, outs=None):
    """-> (dgate, dup, hs, dscale): gradients of the two pre-activations, the scaled
    activation ``hs = s * silu(g) * u`` and the gradient of the row scale (None
    without ``row_scale``), from ``dh = dy @ W_down`` of the unscaled activation."""
    assert dh.is_cuda and all(t.dtype == torch.bfloat16 and t.is_contiguous() and t.shape == dh.shape
                              for t in (dh, gate_pre, up_pre))
    M, N = dh.shape
    if row_scale is not None:
        assert row_scale.dtype == torch.float32 and row_scale.is_contiguous() and row_scale.numel() == M
    if outs is None:
        dg, du, hs = (torch.empty_like(dh) for _ in range(3))
        ds = torch.empty(M, dtype=torch.float32, device=dh.device) if row_scale is not None else None
    else:       # buffers of an earlier call
        dg, du, hs, ds = outs
        assert all(t.shape == dh.shape and t.dtype == dh.dtype and t.is_contiguous() for t in (dg, du, hs))
        assert (ds is None) == (row_scale is None)
    rc = _lib.lib().mep_swiglu_bwd(dh.data_ptr(), gate_pre.data_ptr(), up_pre.data_ptr(), _lib.ptr(row_scale),
                                   cu_seqlens.data_ptr(), cu_seqlens.numel(), dg.data_ptr(), du.data_ptr(),
                                   hs.data_ptr(), _lib.ptr(ds), M, N, _lib.current_stream())
    _lib.check(rc, "mep_swiglu_bwd")
    return dg, du, hs, ds


def grouped_ffn_hip_forward(rows, slots, cu_seqlens, gate_t, up_t, down, *, token_padding: int = 128):
    """Forward for training: -> (y, saved) where ``saved`` is what
    ``grouped_ffn_hip_backward`` needs (the two pre-activations)."""
    act, gp, up = launch_grouped_swiglu(rows, gate_t, up_t, cu_seqlens, token_padding=token_padding)
    y = launch_grouped_gemm_nt(act, down, cu_seqlens, row_scale=slots, token_padding=token_padding)
    return y, (gp, up)


def grouped_ffn_hip_backward(dy, rows, slots, cu_seqlens, gate_t, up_t, down, saved, *,
                             token_padding: int = 128, skip_unused_slots: bool = False):
    """Backward of ``grouped_ffn_hip``: -> (drows [M,H] bf16, dslots [M] fp32 | None,
    dgate_t, dup_t [G,H',H] fp32, ddown [G,H,H'] fp32).  Every GEMM runs on the
    matrix cores through the grouped kernels: the input gradients read the weights
    as they are ([K, N] form), the weight gradients the activations as they are
    (transposed copies only for shapes the untransposed form does not take).
    ``skip_unused_slots``: the weight gradients of slot groups (the upper half of the
    groups) that have no rows are left unwritten instead of zeroed -- they belong to slots that
    hold no expert, which ``launch_grad_reduce`` never reads."""
    gp, up = saved
    dy = dy.contiguous()
    # gradient of the unscaled activation: dy @ down[g], down[g] is [H, H'] = [K, N]
    dh = launch_grouped_gemm_nn(dy, down, cu_seqlens, token_padding=token_padding)
    dg, du, hs, dslots = launch_swiglu_bwd(dh, gp, up, slots, cu_seqlens)
    # input gradient: dg @ gate_t[g] + du @ up_t[g], both [H', H] = [K, N]
    drows = launch_grouped_gemm_dual_nn(dg, gate_t, du, up_t, cu_seqlens, token_padding=token_padding)
    G = cu_seqlens.numel()
    kw = dict(token_padding=token_padding, skip_empty_from=G // 2 if skip_unused_slots else None)
    if wgrad_tn_supported(dg.shape[1], rows.shape[1], G):
        # an expert's shapes: the weight gradients read the activations as they are
        dgate_t = launch_grouped_gemm_wgrad_tn(dg, rows, cu_seqlens, **kw)
        dup_t = launch_grouped_gemm_wgrad_tn(du, rows, cu_seqlens, **kw)
        ddown = launch_grouped_gemm_wgrad_tn(dy, hs, cu_seqlens, **kw)
        return drows, dslots, dgate_t, dup_t, ddown
    rows_t, dy_t = transpose_bf16(rows), transpose_bf16(dy)
    dgate_t = launch_grouped_gemm_wgrad(transpose_bf16(dg), rows_t, cu_seqlens, **kw)
    dup_t = launch_grouped_gemm_wgrad(transpose_bf16(du), rows_t, cu_seqlens, **kw)
    ddown = launch_grouped_gemm_wgrad(dy_t, transpose_bf16(hs), cu_seqlens, **kw)
    return drows, dslots, dgate_t, dup_t, ddown
