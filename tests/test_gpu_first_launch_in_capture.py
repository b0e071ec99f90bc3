"""The very first launch of a kernel that needs more than 64 KB of dynamic LDS may come
from inside a HIP-graph capture: the opt-ins are made when the library is loaded
(mep_init), not by the launch.  A fresh process captures, as its first use of each, a
grouped GEMM, a slot reduction with a 128 x 32 table and the planner for E = 4096, replays
the graph and compares with eager launches made afterwards."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
import torch
sys.path.insert(0, %(root)r)
from moonep_amd import Buffer, ffn, routing
from moonep_amd.grad_reduce import launch_grad_reduce
from moonep_amd.planning import allocate_planning_outputs, launch_planning

dev = torch.device("cuda", 0)
torch.cuda.set_device(dev)
g = torch.Generator().manual_seed(3)
# grouped GEMM: 4 groups of 128 rows
M, Kd, N, G = 512, 256, 256, 4
rows = torch.randn(M, Kd, generator=g).to(torch.bfloat16).to(dev)
wts = (torch.randn(G, N, Kd, generator=g) / 16).to(torch.bfloat16).to(dev)
ends = torch.tensor([128, 256, 384, 512], dtype=torch.int32, device=dev)
out = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
# slot reduction with a table beyond 64 KB of LDS
R, epn, H, Hp = 128, 32, 128, 128
live = torch.rand((R, epn), generator=g) < 0.6
etc = torch.where(live, torch.randint(0, R * epn, (R, epn), generator=g, dtype=torch.int32),
                  torch.full((R, epn), -1, dtype=torch.int32)).to(dev)
slots = (torch.randn(R, epn, H, Hp, generator=g) * 1e-3).to(dev)
pool, grad0 = slots.clone(), torch.randn(epn, H, Hp, generator=g).to(dev)
grad = grad0.clone()
# planner with E = 4096
S, K, E, Rp, tp = 512, 4, 4096, 8, 16
topk = torch.stack([routing.popularity_biased(S, K, E, Rp, r, 1.0, seed=31) for r in range(Rp)])
tpe = routing.tokens_per_expert(topk, E).to(dev)
buf = Buffer(S, 16, K, E, Rp, token_padding=tp, rank=3)
ctx = buf._require_ctx()
plan, cu = allocate_planning_outputs(ctx)
d_topk = topk[3].reshape(-1).contiguous().to(dev)
torch.cuda.synchronize()

side = torch.cuda.Stream()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph, stream=side):
    ffn.launch_grouped_gemm_nt(rows, wts, ends, out)
    launch_grad_reduce(grad, pool, etc, rank=63)
    launch_planning(ctx, d_topk, tpe, cu, plan)
graph.replay()
torch.cuda.synchronize()
got = (out.clone(), grad.clone(), pool.clone(), plan.dst.clone(), cu.clone())

out.zero_(); grad.copy_(grad0); pool.copy_(slots); plan.dst.zero_(); cu.zero_()
ffn.launch_grouped_gemm_nt(rows, wts, ends, out)
launch_grad_reduce(grad, pool, etc, rank=63)
launch_planning(ctx, d_topk, tpe, cu, plan)
torch.cuda.synchronize()
want = (out, grad, pool, plan.dst, cu)
for i, (a, b) in enumerate(zip(got, want)):
    assert torch.equal(a, b), f"captured first launch differs from the eager one: output {i}"
assert bool(out.any()) and bool((plan.dst != 0).any())
print("CAPTURED_FIRST_LAUNCHES_OK", flush=True)
"""


def test_first_launches_of_large_lds_kernels_inside_a_graph_capture():
    r = subprocess.run([sys.executable, "-c", CHILD % {"root": ROOT}], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0 and "CAPTURED_FIRST_LAUNCHES_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
