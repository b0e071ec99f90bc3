"""End-to-end MoE layer on the emulated group: dispatch -> grouped FFN over
(local experts + prefetch slots) -> combine, forward and backward through
autograd, against a dense PyTorch MoE that never permutes anything.

The communication ops are exact copies / ordered sums; what differs from the
dense fp32 reference is bf16 rounding of rows and GEMM inputs, so values are
compared at bf16-level tolerance (stated at the asserts)."""

import pytest
import torch

from moonep_amd import moe, routing
from tests.util import grouped_ffn

pytestmark = pytest.mark.gpu


def _dense_reference(x, w, topk, master, epn):
    """y[r,s] = sum_k w[r,s,k] * FFN_{topk[r,s,k]}(x[r,s]); bf16-rounded inputs, fp32 math."""
    gate, up, down = (m.to(torch.bfloat16).float() for m in master)
    R, S, K = topk.shape
    xb = x.to(torch.bfloat16).float()
    y = torch.zeros_like(xb)
    for k in range(K):
        e = topk[:, :, k].long()
        g, u, d = gate[e // epn, e % epn], up[e // epn, e % epn], down[e // epn, e % epn]  # [R,S,H,Hp]
        h = torch.nn.functional.silu(torch.einsum("rsh,rshp->rsp", xb, g)) * torch.einsum("rsh,rshp->rsp", xb, u)
        y = y + w[:, :, k, None] * torch.einsum("rsp,rshp->rsh", h, d)
    return y


@pytest.mark.parametrize("sigma", [0.0, 2.0])
def test_moe_layer_forward_backward_matches_dense(cuda, sigma):
    R, epn, S, K, H, Hp, tp = 4, 2, 24, 3, 128, 128, 8
    E = R * epn
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed=5) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(R, S, H, generator=g).to(cuda).requires_grad_()
    w = torch.softmax(torch.randn(R, S, K, generator=g), -1).to(cuda).requires_grad_()
    master = [(torch.randn(R, epn, H, Hp, generator=g) * 0.08).to(cuda).requires_grad_() for _ in range(3)]
    gout = torch.randn(R, S, H, generator=g).to(cuda)
    topk_d, tpe_d = topk.to(cuda), tpe.to(cuda)

    group = moe.EmulatedGroup(S, H, K, E, R, token_padding=tp)
    rows, slots, cu, plans = moe.group_dispatch(group, x.to(torch.bfloat16), w, topk_d, tpe_d)
    etc = plans[0].experts_to_copy
    if sigma > 0:
        assert bool((etc >= 0).any()), "the skewed routing must exercise prefetch slots"
    views = [moe.group_compute_views(group, etc, m) for m in master]
    y = torch.stack([grouped_ffn(rows[r], slots[r], cu[r], views[0][r], views[1][r], views[2][r])
                     for r in range(R)])
    out = moe.group_combine(group, plans, y)
    (out.float() * gout).sum().backward()
    got = dict(out=out.float().detach(), x=x.grad.clone(), w=w.grad.clone(),
               **{f"m{i}": m.grad.clone() for i, m in enumerate(master)})

    for t in (x, w, *master):
        t.grad = None
    ref = _dense_reference(x, w, topk_d, master, epn)
    (ref * gout).sum().backward()
    want = dict(out=ref.detach(), x=x.grad, w=w.grad, **{f"m{i}": m.grad for i, m in enumerate(master)})

    for name in want:
        a, b = got[name], want[name]
        scale = float(b.abs().max())
        err = float((a - b).abs().max())
        # bf16 has 8 significand bits: rows, GEMM inputs and the K-sum are each rounded
        # once or twice on the way, so 3 % of the tensor's largest magnitude bounds it
        assert err <= 0.03 * scale + 1e-6, (name, err, scale)
        # and the direction agrees closely
        cos = float(torch.nn.functional.cosine_similarity(a.flatten(), b.flatten(), dim=0))
        assert cos > 0.999, (name, cos)
    # experts never hosted remotely get grads only from their home rank; every
    # master weight that received tokens has a non-zero grad
    used = tpe.sum(0).reshape(R, epn) > 0
    assert bool(((got["m0"].abs().amax(dim=(2, 3)) > 0).cpu() == used).all())
    group.destroy()


def test_moe_layer_forward_on_hip_kernels_only(cuda):
    """The same layer, forward only, with every step a HIP kernel of this
    library: dispatch -> prefetch -> grouped MFMA FFN (cu_seqlens stay on the
    device) -> combine.  One rank's chain is also captured in a HIP graph and
    replayed.  Compared with the dense reference at the same bf16 tolerance."""
    from moonep_amd.ffn import grouped_ffn_hip
    from moonep_amd.prefetch import launch_prefetch

    R, epn, S, K, H, Hp, tp = 4, 2, 40, 3, 256, 128, 128
    E = R * epn
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, 2.0, seed=9) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(R, S, H, generator=g).to(cuda)
    w = torch.softmax(torch.randn(R, S, K, generator=g), -1).to(cuda)
    master = [(torch.randn(R, epn, H, Hp, generator=g) * 0.08).to(cuda) for _ in range(3)]
    topk_d, tpe_d = topk.to(cuda), tpe.to(cuda)

    group = moe.EmulatedGroup(S, H, K, E, R, token_padding=tp)
    with torch.no_grad():
        rows, slots, cu, plans = moe.group_dispatch(group, x.to(torch.bfloat16), w, topk_d, tpe_d)
        etc = plans[0].experts_to_copy
        assert bool((etc >= 0).any()), "the skewed routing must exercise prefetch slots"
        # compute views, K-contiguous: gate/up [R, 2*epn, H', H], down [R, 2*epn, H, H']
        local = [master[0].transpose(2, 3).contiguous().to(torch.bfloat16),
                 master[1].transpose(2, 3).contiguous().to(torch.bfloat16),
                 master[2].to(torch.bfloat16).contiguous()]
        pools = [torch.zeros_like(t) for t in local]
        for r in range(R):
            launch_prefetch(tuple(t[r] for t in local), tuple(pools), etc, rank=r)
        views = [torch.cat([l, p], dim=1) for l, p in zip(local, pools)]
        y = torch.stack([grouped_ffn_hip(rows[r].contiguous(), slots[r].contiguous(), cu[r].contiguous(),
                                         views[0][r], views[1][r], views[2][r]) for r in range(R)])
        out = moe.group_combine(group, plans, y)
        ref = _dense_reference(x, w, topk_d, master, epn)
        torch.cuda.synchronize()
    err = float((out.float() - ref).abs().max())
    scale = float(ref.abs().max())
    assert err <= 0.03 * scale + 1e-6, (err, scale)
    cos = float(torch.nn.functional.cosine_similarity(out.float().flatten(), ref.flatten(), dim=0))
    assert cos > 0.999, cos

    # rank 0's FFN under a HIP graph: cu_seqlens are read by the kernel, not by the host
    r0 = (rows[0].contiguous(), slots[0].contiguous(), cu[0].contiguous())
    eager = grouped_ffn_hip(*r0, views[0][0], views[1][0], views[2][0])
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = grouped_ffn_hip(*r0, views[0][0], views[1][0], views[2][0])
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured.view(torch.int16), eager.view(torch.int16))
    group.destroy()


_ATEN_GEMMS = {"aten::mm", "aten::bmm", "aten::addmm", "aten::baddbmm", "aten::matmul", "aten::linear",
               "aten::einsum", "aten::_scaled_mm", "aten::addbmm", "aten::mv", "aten::addmv"}


@pytest.mark.parametrize("sigma", [0.0, 2.0])
def test_moe_layer_forward_and_backward_without_a_torch_gemm(cuda, sigma):
    """dispatch -> prefetch + grouped FFN on the matrix cores -> combine, forward
    AND backward through autograd, every GEMM (forward, input gradients, weight
    gradients) a launch of this library's grouped kernel: the op trace of the
    whole step holds no aten matrix product.  Values and all gradients against
    the dense fp32 reference at the bf16 tolerance of the test above."""
    R, epn, S, K, H, Hp, tp = 4, 2, 40, 3, 256, 256, 128
    E = R * epn
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed=13) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(R, S, H, generator=g).to(cuda).requires_grad_()
    w = torch.softmax(torch.randn(R, S, K, generator=g), -1).to(cuda).requires_grad_()
    master = [(torch.randn(R, epn, H, Hp, generator=g) * 0.08).to(cuda).requires_grad_() for _ in range(3)]
    gout = torch.randn(R, S, H, generator=g).to(cuda)
    topk_d, tpe_d = topk.to(cuda), tpe.to(cuda)
    # the orientation the kernels read: gate / up [R, epn, H', H], down [R, epn, H, H']
    gate_m = master[0].detach().transpose(2, 3).contiguous().requires_grad_()
    up_m = master[1].detach().transpose(2, 3).contiguous().requires_grad_()
    down_m = master[2].detach().clone().requires_grad_()

    # the op trace sees the autograd thread too: a library product and its two backward products
    a, b = (torch.randn(8, 8, device=cuda, requires_grad=True) for _ in range(2))
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU]) as probe:
        (a @ b).sum().backward()
        torch.cuda.synchronize()
    assert sum(e.count for e in probe.key_averages() if e.key == "aten::mm") == 3

    group = moe.EmulatedGroup(S, H, K, E, R, token_padding=tp)
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU]) as prof:
        rows, slots, cu, plans = moe.group_dispatch(group, x.to(torch.bfloat16), w, topk_d, tpe_d)
        etc = plans[0].experts_to_copy
        y = moe.group_expert_ffn_hip(group, etc, cu, rows, slots, gate_m, up_m, down_m)
        out = moe.group_combine(group, plans, y)
        (out.float() * gout).sum().backward()
        torch.cuda.synchronize()
    ops = {e.key for e in prof.key_averages()}
    assert "aten::mul" in ops, "the trace must have recorded this step's ops"
    assert not (ops & _ATEN_GEMMS), f"library matrix products in the step: {sorted(ops & _ATEN_GEMMS)}"
    if sigma > 0:
        assert bool((etc >= 0).any()), "the skewed routing must exercise prefetch slots"
    got = dict(out=out.float().detach(), x=x.grad.clone(), w=w.grad.clone(),
               m0=gate_m.grad.transpose(2, 3), m1=up_m.grad.transpose(2, 3), m2=down_m.grad)
    for t in (x, w):
        t.grad = None
    ref = _dense_reference(x, w, topk_d, master, epn)
    (ref * gout).sum().backward()
    want = dict(out=ref.detach(), x=x.grad, w=w.grad, **{f"m{i}": m.grad for i, m in enumerate(master)})
    for name in want:
        a, b = got[name].float(), want[name]
        scale, err = float(b.abs().max()), float((a - b).abs().max())
        assert err <= 0.03 * scale + 1e-6, (name, err, scale)
        cos = float(torch.nn.functional.cosine_similarity(a.flatten(), b.flatten(), dim=0))
        assert cos > 0.999, (name, cos)
    assert gate_m.grad.dtype == torch.float32
    group.destroy()
