"""Backward pass of the expert FFN on the matrix cores: every piece against a
plain PyTorch fp32 reference of the same op, then the whole backward against
torch autograd of the fp32 FFN.

Tolerances: GEMM results are rounded once to bf16 (2^-8 relative) on top of
fp32 accumulation in a different order: |got - ref| <= 2^-7 |ref| + 2^-7 *
(largest |ref| of the row).  The full backward chains three rounded stages
(dh, dgate/dup, the final GEMM) and feeds bf16-rounded pre-activations to
silu': compared at 3 % of the largest magnitude of the row / matrix."""

import pytest
import torch

from moonep_amd import ffn

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=[128, 256])
def row_tile(request):
    """Every test runs on both row tilings of the grouped kernel (the library picks by shape;
    the small shapes here would only ever see one of them)."""
    from moonep_amd import _lib

    _lib.check(_lib.lib().mep_set_gemm_row_tile(request.param), "mep_set_gemm_row_tile")
    yield request.param
    _lib.check(_lib.lib().mep_set_gemm_row_tile(0), "mep_set_gemm_row_tile")


def _groups(G, M, seed, tail):
    g = torch.Generator().manual_seed(seed)
    tiles = (M - tail) // 128
    cuts = torch.sort(torch.randint(0, tiles + 1, (G - 1,), generator=g)).values
    return (torch.cat([cuts, torch.tensor([tiles])]) * 128).to(torch.int32)


def _close(got, ref, what, rel=2.0 ** -7):
    err = (got.float() - ref).abs()
    tol = rel * ref.abs() + rel * ref.abs().amax(dim=-1, keepdim=True).clamp(min=1e-6)
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off, worst {float((err / tol).max()):.2f}x tolerance"


@pytest.mark.parametrize("shape", [(1, 64, 64), (3, 128, 320), (2, 448, 64), (1, 1024, 2048)])
def test_transpose_is_exact(cuda, shape):
    g = torch.Generator().manual_seed(sum(shape))
    t = torch.randn(*shape, generator=g).to(torch.bfloat16).to(cuda)
    got = ffn.transpose_bf16(t)
    torch.cuda.synchronize()
    assert got.is_contiguous() and torch.equal(got, t.transpose(-1, -2).contiguous())


@pytest.mark.parametrize("M,K,N,G,tail", [(128, 64, 128, 1, 0), (1024, 448, 384, 6, 256), (1152, 1024, 256, 3, 0)])
def test_swiglu_forward_keeps_the_preactivations(cuda, M, K, N, G, tail):
    g = torch.Generator().manual_seed(M + K + N)
    rows = torch.randn(M, K, generator=g).to(torch.bfloat16)
    wg = (torch.randn(G, N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    wu = (torch.randn(G, N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    ends = _groups(G, M, seed=G + M, tail=tail)
    act, gp, up = ffn.launch_grouped_swiglu(rows.to(cuda), wg.to(cuda), wu.to(cuda), ends.to(cuda))
    plain = ffn.launch_grouped_gemm_nt(rows.to(cuda), wg.to(cuda), ends.to(cuda), up_weights=wu.to(cuda))
    torch.cuda.synchronize()
    assert torch.equal(act, plain), "saving the pre-activations must not change the activation"
    start = 0
    for gi, end in enumerate(ends.tolist()):
        if end > start:
            x = rows[start:end].float()
            rg, ru = x @ wg[gi].float().t(), x @ wu[gi].float().t()
            _close(gp[start:end].cpu(), rg, f"gate pre-activation, group {gi}")
            _close(up[start:end].cpu(), ru, f"up pre-activation, group {gi}")
        start = max(start, end)
    last = int(ends[-1])
    assert not gp[last:].any() and not up[last:].any()


@pytest.mark.parametrize("M,K,N,G,tail", [(128, 64, 256, 1, 0), (1024, 192, 768, 6, 256), (1152, 1024, 512, 3, 0)])
def test_dual_gemm_sums_both_products(cuda, M, K, N, G, tail):
    g = torch.Generator().manual_seed(M + K + N + 1)
    a1, a2 = (torch.randn(M, K, generator=g).to(torch.bfloat16) for _ in range(2))
    w1, w2 = ((torch.randn(G, N, K, generator=g) / K ** 0.5).to(torch.bfloat16) for _ in range(2))
    ends = _groups(G, M, seed=G * 3 + M, tail=tail)
    got = ffn.launch_grouped_gemm_dual_nt(a1.to(cuda), w1.to(cuda), a2.to(cuda), w2.to(cuda), ends.to(cuda))
    torch.cuda.synchronize()
    ref = torch.zeros(M, N)
    start = 0
    for gi, end in enumerate(ends.tolist()):
        if end > start:
            ref[start:end] = a1[start:end].float() @ w1[gi].float().t() + a2[start:end].float() @ w2[gi].float().t()
        start = max(start, end)
    _close(got.cpu(), ref, "dual")
    assert not got[int(ends[-1]):].any()


@pytest.mark.parametrize("M,K,N,G,tail", [(128, 64, 256, 1, 0), (640, 192, 512, 5, 128), (2304, 512, 768, 64, 256),
                                          (6400, 128, 256, 96, 128)])
def test_products_with_weights_in_k_by_n_form(cuda, M, K, N, G, tail):
    """rows @ w[g] with w [G, K, N] (the input gradient's orientation: no transposed copy):
    against the fp32 product, alone with a row scale and as the sum of two pairs.  The
    weights carry a different value in every (k, n): a lane that took its K values from the
    wrong rows or columns of the transposing LDS read would not pass."""
    g = torch.Generator().manual_seed(M + K + N + 7)
    a1, a2 = (torch.randn(M, K, generator=g).to(torch.bfloat16) for _ in range(2))
    w1, w2 = ((torch.randn(G, K, N, generator=g) / K ** 0.5).to(torch.bfloat16) for _ in range(2))
    scale = torch.rand(M, generator=g) + 0.5
    ends = _groups(G, M, seed=G * 7 + M, tail=tail)
    one = ffn.launch_grouped_gemm_nn(a1.to(cuda), w1.to(cuda), ends.to(cuda), row_scale=scale.to(cuda))
    two = ffn.launch_grouped_gemm_dual_nn(a1.to(cuda), w1.to(cuda), a2.to(cuda), w2.to(cuda), ends.to(cuda))
    torch.cuda.synchronize()
    ref1, ref2 = torch.zeros(M, N), torch.zeros(M, N)
    start = 0
    for gi, end in enumerate(ends.tolist()):
        if end > start:
            p1 = a1[start:end].float() @ w1[gi].float()
            ref1[start:end] = scale[start:end, None] * p1
            ref2[start:end] = p1 + a2[start:end].float() @ w2[gi].float()
        start = max(start, end)
    _close(one.cpu(), ref1, "nn")
    _close(two.cpu(), ref2, "dual nn")
    assert not one[int(ends[-1]):].any() and not two[int(ends[-1]):].any()
    # the same product through the [N, K] kernel on a transposed copy: same accumulation order
    # per output element, so the two agree to the bit
    nt = ffn.launch_grouped_gemm_nt(a1.to(cuda), ffn.transpose_bf16(w1.to(cuda)), ends.to(cuda),
                                    row_scale=scale.to(cuda))
    assert torch.equal(nt, one)


# 128 x 256 tiles (an output dimension that is no multiple of 256, or an odd group count) and
# 256 x 256 tiles (both are, G even): either output dimension the longer one, 7 tiles over 8 XCDs
@pytest.mark.parametrize("M,Ma,Nb,G,tail", [(128, 128, 256, 1, 0), (1024, 256, 512, 6, 256), (2304, 384, 256, 64, 128),
                                            (1152, 512, 1792, 4, 128), (1920, 1792, 256, 8, 0), (768, 256, 256, 3, 0)])
def test_weight_gradients_per_group(cuda, M, Ma, Nb, G, tail):
    g = torch.Generator().manual_seed(M + Ma + Nb)
    at = torch.randn(Ma, M, generator=g).to(torch.bfloat16)
    bt = torch.randn(Nb, M, generator=g).to(torch.bfloat16)
    ends = _groups(G, M, seed=G * 5 + M, tail=tail)
    got = ffn.launch_grouped_gemm_wgrad(at.to(cuda), bt.to(cuda), ends.to(cuda))
    if ffn.wgrad_tn_supported(Ma, Nb, G):
        # the same products from the untransposed activations: same K order per output element,
        # so the same bits
        tn = ffn.launch_grouped_gemm_wgrad_tn(at.t().contiguous().to(cuda), bt.t().contiguous().to(cuda),
                                              ends.to(cuda))
        assert torch.equal(tn, got)
    # groups without rows from index G // 2 on are left as they are when the caller says so
    # (slots that hold no expert); the others do not change
    half = G // 2
    kept = torch.full_like(got, 7.0)
    ffn.launch_grouped_gemm_wgrad(at.to(cuda), bt.to(cuda), ends.to(cuda), kept, skip_empty_from=half)
    lens = torch.diff(ends, prepend=torch.zeros(1, dtype=torch.int32)).clamp(min=0)
    for gi in range(G):
        if gi >= half and int(lens[gi]) == 0:
            assert bool((kept[gi] == 7.0).all()), f"group {gi} was written"
        else:
            assert torch.equal(kept[gi], got[gi]), f"group {gi}"
    if ffn.wgrad_tn_supported(Ma, Nb, G):
        kept.fill_(7.0)
        ffn.launch_grouped_gemm_wgrad_tn(at.t().contiguous().to(cuda), bt.t().contiguous().to(cuda), ends.to(cuda),
                                         kept, skip_empty_from=half)
        for gi in range(G):
            if gi >= half and int(lens[gi]) == 0:
                assert bool((kept[gi] == 7.0).all()), f"group {gi} was written"
            else:
                assert torch.equal(kept[gi], got[gi]), f"group {gi}"
    torch.cuda.synchronize()
    got = got.cpu()
    start, empty = 0, 0
    for gi, end in enumerate(ends.tolist()):
        if end > start:
            ref = at[:, start:end].float() @ bt[:, start:end].float().t()
            err = (got[gi] - ref).abs()
            assert float(err.max()) <= 2.0 ** -12 * float(ref.abs().max()) * (end - start) ** 0.5, f"group {gi}"
        else:
            empty += 1
            assert not got[gi].any(), f"group {gi} has no rows: its gradient is zero"
        start = max(start, end)
    print(f"{empty} empty groups of {G}", flush=True)


def test_swiglu_backward_matches_autograd(cuda):
    M, N, G = 640, 256, 4
    g = torch.Generator().manual_seed(9)
    ends = torch.tensor([128, 128, 384, 512], dtype=torch.int32)
    gp = torch.randn(M, N, generator=g).to(torch.bfloat16)
    up = torch.randn(M, N, generator=g).to(torch.bfloat16)
    dh = torch.randn(M, N, generator=g).to(torch.bfloat16)
    s = torch.rand(M, generator=g) + 0.25
    dg, du, hs, ds = ffn.launch_swiglu_bwd(dh.to(cuda), gp.to(cuda), up.to(cuda), s.to(cuda), ends.to(cuda))
    torch.cuda.synchronize()
    a, b, c = gp.float().requires_grad_(), up.float().requires_grad_(), s.clone().requires_grad_()
    h = c[:, None] * torch.nn.functional.silu(a) * b
    (h * dh.float()).sum().backward()
    last = int(ends[-1])
    _close(dg.cpu()[:last], a.grad[:last], "dgate", rel=2.0 ** -6)   # fast exponential in silu'
    _close(du.cpu()[:last], b.grad[:last], "dup", rel=2.0 ** -6)
    _close(hs.cpu()[:last], h.detach()[:last], "scaled activation", rel=2.0 ** -6)
    assert float((ds.cpu()[:last] - c.grad[:last]).abs().max()) <= 1e-3 * float(c.grad.abs().max())
    for t in (dg, du, hs):
        assert not t[last:].any(), "rows outside every group come out as zeros"
    # without a row scale: s = 1, no dscale
    dg1, du1, hs1, ds1 = ffn.launch_swiglu_bwd(dh.to(cuda), gp.to(cuda), up.to(cuda), None, ends.to(cuda))
    torch.cuda.synchronize()
    assert ds1 is None
    a.grad = b.grad = None
    (torch.nn.functional.silu(a) * b * dh.float()).sum().backward()
    _close(dg1.cpu()[:last], a.grad[:last], "dgate, no scale", rel=2.0 ** -6)


@pytest.mark.parametrize("NvS,H,Hp,G,tail", [(1536, 512, 256, 8, 128), (768, 256, 512, 3, 0)])
def test_ffn_backward_matches_fp32_autograd(cuda, NvS, H, Hp, G, tail):
    g = torch.Generator().manual_seed(NvS + H)
    rows = torch.randn(NvS, H, generator=g).to(torch.bfloat16)
    slots = torch.rand(NvS, generator=g) + 0.25
    gate_t = (torch.randn(G, Hp, H, generator=g) / H ** 0.5).to(torch.bfloat16)
    up_t = (torch.randn(G, Hp, H, generator=g) / H ** 0.5).to(torch.bfloat16)
    down = (torch.randn(G, H, Hp, generator=g) / Hp ** 0.5).to(torch.bfloat16)
    dy = torch.randn(NvS, H, generator=g).to(torch.bfloat16)
    ends = _groups(G, NvS, seed=NvS, tail=tail)
    last = int(ends[-1])
    d = [t.to(cuda) for t in (rows, slots, ends, gate_t, up_t, down)]
    y, saved = ffn.grouped_ffn_hip_forward(*d)
    assert torch.equal(y, ffn.grouped_ffn_hip(*d)), "the training forward equals the inference forward"
    drows, dslots, dgate, dup, ddown = ffn.grouped_ffn_hip_backward(dy.to(cuda), *d, saved)
    torch.cuda.synchronize()

    # fp32 reference on the bf16-rounded inputs, autograd for every gradient
    x, s = rows.float().to(cuda).requires_grad_(), slots.to(cuda).requires_grad_()
    wg, wu, wd = (t.float().to(cuda).requires_grad_() for t in (gate_t, up_t, down))
    out = torch.zeros(NvS, H, device=cuda)
    start = 0
    for gi, end in enumerate(ends.tolist()):
        if end > start:
            xs = x[start:end]
            hmid = torch.nn.functional.silu(xs @ wg[gi].t()) * (xs @ wu[gi].t())
            out[start:end] = s[start:end, None] * (hmid @ wd[gi].t())
        start = max(start, end)
    (out * dy.float().to(cuda)).sum().backward()

    def rel(got, ref, dim):
        scale = ref.abs().amax(dim=dim, keepdim=True).clamp(min=1e-6)
        return float(((got.float() - ref).abs() / scale).max())

    assert rel(y[:last], out.detach()[:last], 1) < 0.02, "forward"
    assert rel(drows[:last], x.grad[:last], 1) < 0.03, "input gradient"
    assert not drows[last:].any()
    assert float((dslots[:last] - s.grad[:last]).abs().max()) < 0.03 * float(s.grad.abs().max()), "slot gradient"
    for name, got, ref in (("gate", dgate, wg.grad), ("up", dup, wu.grad), ("down", ddown, wd.grad)):
        assert got.dtype == torch.float32 and got.shape == ref.shape
        assert rel(got, ref, (1, 2)) < 0.03 or float(ref.abs().max()) == 0.0, f"{name} weight gradient"
        start = 0
        for gi, end in enumerate(ends.tolist()):
            if end <= start:
                assert not got[gi].any(), f"{name}: group {gi} has no rows"
            start = max(start, end)
