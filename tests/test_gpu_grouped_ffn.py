"""Grouped bf16 GEMM on the matrix cores (the expert-side consumer of the
dispatched rows) against a plain PyTorch fp32 reference of the same op.

Tolerance: products and sums are fp32 in both; the kernel rounds once to bf16
(relative step 2^-8), and the fused SwiGLU evaluates silu in fp32 with a fast
exponential.  |got - ref| <= 2^-7 * |ref| + 2^-7 * (row scale of the result)
covers one bf16 rounding plus accumulation-order differences."""

import pytest
import torch

from moonep_amd.ffn import grouped_ffn_hip, launch_grouped_gemm_nt

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
    """Padded group ends (multiples of 128), some groups empty, `tail` unused rows."""
    g = torch.Generator().manual_seed(seed)
    tiles = (M - tail) // 128
    cuts = torch.sort(torch.randint(0, tiles + 1, (G - 1,), generator=g)).values
    ends = torch.cat([cuts, torch.tensor([tiles])]) * 128
    return ends.to(torch.int32)


def _ref_gemm(rows, w, ends, up=None, scale=None):
    out = torch.zeros(rows.shape[0], w.shape[1], dtype=torch.float32)
    start = 0
    for g, end in enumerate(ends.tolist()):
        if end > start:
            x = rows[start:end].float()
            y = x @ w[g].float().t()
            if up is not None:
                y = torch.nn.functional.silu(y) * (x @ up[g].float().t())
            if scale is not None:
                y = y * scale[start:end, None]
            out[start:end] = y
        start = max(start, end)
    return out


def _close(got, ref, what):
    err = (got.float() - ref).abs()
    tol = 2.0 ** -7 * ref.abs() + 2.0 ** -7 * ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-6)
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off, worst {float((err / tol).max()):.2f}x tolerance"


@pytest.mark.parametrize("M,K,N,G,tail", [
    (128, 64, 256, 1, 0),          # one tile, one K step
    (512, 256, 256, 4, 0),
    (1024, 448, 768, 6, 256),      # K = 7 steps, unused rows at the end, empty groups likely
    (2304, 1024, 512, 64, 128),    # more groups than row tiles
    (1152, 2048, 1280, 3, 0),      # tile counts that are no multiples of eight
    (6400, 128, 256, 96, 256),     # more than 64 groups (E = 384 on 8 ranks): the group search takes two rounds
])
def test_grouped_gemm_matches_fp32_reference(cuda, M, K, N, G, tail):
    g = torch.Generator().manual_seed(M + K + N)
    rows = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(G, N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    up = (torch.randn(G, N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    scale = torch.rand(M, generator=g) + 0.1
    ends = _groups(G, M, seed=G * 7 + M, tail=tail)
    print(f"M={M} K={K} N={N} G={G} ends={ends.tolist()[:8]}...", flush=True)
    d = dict(device=cuda)
    # plain and scaled
    got = launch_grouped_gemm_nt(rows.to(**d), w.to(**d), ends.to(**d))
    torch.cuda.synchronize()
    _close(got.cpu(), _ref_gemm(rows, w, ends), "plain")
    got = launch_grouped_gemm_nt(rows.to(**d), w.to(**d), ends.to(**d), row_scale=scale.to(**d))
    torch.cuda.synchronize()
    _close(got.cpu(), _ref_gemm(rows, w, ends, scale=scale), "scaled")
    # fused SwiGLU; rows past the last group stay untouched
    out = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=cuda)
    launch_grouped_gemm_nt(rows.to(**d), w.to(**d), ends.to(**d), out, up_weights=up.to(**d))
    torch.cuda.synchronize()
    last = int(ends[-1])
    _close(out.cpu()[:last], _ref_gemm(rows, w, ends, up=up)[:last], "swiglu")
    assert (out.cpu()[last:] == 3.0).all()


def test_no_rows_at_all(cuda):
    """Every group empty (a rank that received nothing): the products write nothing, the
    weight gradients are zero."""
    from moonep_amd import ffn
    M, K, N, G = 512, 128, 256, 4
    rows = torch.randn(M, K).to(torch.bfloat16).to(cuda)
    w = torch.randn(G, N, K).to(torch.bfloat16).to(cuda)
    ends = torch.zeros(G, dtype=torch.int32, device=cuda)
    out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=cuda)
    launch_grouped_gemm_nt(rows, w, ends, out)
    ffn.launch_grouped_gemm_nn(rows, w.transpose(1, 2).contiguous(), ends, out)
    assert bool((out == 7.0).all())
    wide = torch.cat([rows, rows], 1)   # [M, 256]
    dw = ffn.launch_grouped_gemm_wgrad_tn(wide, wide, ends)
    assert not dw.any()


def test_grouped_ffn_matches_the_torch_consumer(cuda):
    """Same contract as the plain-PyTorch consumer (library GEMMs per group)."""
    from tests.util import grouped_ffn

    NvS, H, Hp, G = 1536, 512, 256, 8
    g = torch.Generator().manual_seed(11)
    rows = torch.randn(NvS, H, generator=g).to(torch.bfloat16).to(cuda)
    slots = torch.rand(NvS, generator=g).to(cuda)
    gate = (torch.randn(G, H, Hp, generator=g) / H ** 0.5).to(torch.bfloat16).to(cuda)
    up = (torch.randn(G, H, Hp, generator=g) / H ** 0.5).to(torch.bfloat16).to(cuda)
    down = (torch.randn(G, H, Hp, generator=g) / Hp ** 0.5).to(torch.bfloat16).to(cuda)
    ends = _groups(G, NvS, seed=5, tail=128).to(cuda)
    want = grouped_ffn(rows, slots, ends, gate, up, down)
    got = grouped_ffn_hip(rows, slots, ends, gate.transpose(1, 2).contiguous(),
                          up.transpose(1, 2).contiguous(), down)
    torch.cuda.synchronize()
    # the torch consumer rounds to bf16 after every GEMM and after silu: looser
    err = (got.float() - want.float()).abs()
    scale = want.float().abs().amax(dim=1, keepdim=True).clamp(min=1e-6)
    assert float((err / scale).max()) < 0.03
    assert (got[int(ends[-1]):] == 0).all()


def test_grouped_gemm_at_the_real_shape(cuda):
    """One rank's shard at the headline shape (NvS = 40960 rows, H = 7168,
    H' = 2048, 64 groups of uneven size): the fused SwiGLU GEMM is bit-identical
    from launch to launch, and three groups (first, middle, last) match the fp32
    reference."""
    M, H, Hp, G = 40960, 7168, 2048, 64
    sizes = 384 + 128 * (torch.arange(G) % 4)            # 384 .. 768 rows per group
    ends = sizes.cumsum(0).to(torch.int32).to(cuda)
    assert int(ends[-1]) <= M
    g = torch.Generator(device=cuda).manual_seed(3)
    rows = torch.randn(M, H, device=cuda, generator=g).to(torch.bfloat16)
    gate = (torch.randn(G, Hp, H, device=cuda, generator=g) * 0.02).to(torch.bfloat16)
    up = (torch.randn(G, Hp, H, device=cuda, generator=g) * 0.02).to(torch.bfloat16)
    first = launch_grouped_gemm_nt(rows, gate, ends, up_weights=up)
    torch.cuda.synchronize()
    for _ in range(3):
        again = launch_grouped_gemm_nt(rows, gate, ends, up_weights=up)
        torch.cuda.synchronize()
        assert torch.equal(first.view(torch.int16), again.view(torch.int16))
    start = 0
    for gi, end in enumerate(ends.tolist()):
        if gi in (0, G // 2, G - 1):
            x = rows[start:end].float()
            want = torch.nn.functional.silu(x @ gate[gi].float().t()) * (x @ up[gi].float().t())
            _close(first[start:end].cpu(), want.cpu(), f"group {gi}")
        start = end
    assert (first[int(ends[-1]):] == 0).all()
