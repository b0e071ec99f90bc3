"""Headline benchmark: one rank's share of plan -> dispatch -> combine on one
MI355X at S=4096, H=7168, K=8, E=256, R=8, token_padding=128, bf16, routing at
maxvio ~= 1 (synthetic, seeded).

    python bench.py [--gpus 1] [--steps 20] [--warmup 5] [--sections chain,extras,sweep,weights,ffn]

A step is one pass planner -> dispatch -> combine over one of six rotating
token sets; the K timed steps are recorded into one HIP graph and replayed
once (K single-step replays are timed beside it).  Prints ONE JSON line.
`value` is the chain's throughput: algorithmic bytes of dispatch + combine
(each S*H*2 + S*K*H*2) divided by the time of a whole step (planner included),
in GB/s, inputs resident in HBM.  Per-kernel durations are measured with HIP
events on the launching stream.  `roofline` describes the dominant kernel from
its COLD, standalone duration (every launch reads a token set that is not in
any cache); its duration inside the timed steps, where the planner launch has
already pulled the tokens into the last-level cache, is reported beside it.

Sections (all by default; `--sections chain` is the headline alone):
  chain    config 1 as above and the CPU baseline (the scalar C restatement
           oracle/mep_oracle.c on the host, same inputs); always measured;
  extras   the chain bounded to 32 .. 256 compute units (`chain_on_limited_cus`: 32 is
           the reference's default `num_sms`), the chain with six rotating sets of
           destination shards, the reference's separate kernels for duplicate rows
           (all-rank plan, duplicate-group builder, epilogue, prologue), and the chain
           called eagerly through Buffer.dispatch / Buffer.combine (`buffer_api_eager`);
  sweep    the chain at maxvio 0 .. 4 on both shapes with the headline's steps and
           warm-ups, three timings per point, the fastest kept (`maxvio_sweep`), and
           the chain at the configuration of the reference's own figure;
  weights  prefetch_weight (owner push, and the pull of one rank's slots) and
           reduce_grad at [32, 7168, 2048] per rank on the planner's own slot table
           and on a table with 8 slots per rank.  Three different tensors for the three
           projections and renumbered variants of each table in turn, so no launch
           re-reads what the one before left in the last-level cache;
  ffn      the expert-side grouped FFN.
Every section carries its own `roofline` record; the short summary keys
(`maxvio_sweep_spread_pct`, `maxvio_sweep_chain_us`, the fractions of HBM peak)
come last in the line.  A 512 MiB device copy runs first: the known-size kernel
that hardware counters of a profiled run are scaled by.
"""

from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

HBM_PEAK_GBPS = 8000.0
ROOT = os.path.dirname(os.path.abspath(__file__))
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def kernel_source_digest() -> str:
    """Identifies the kernel sources a traffic measurement belongs to."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "moonep_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(key: str, grid=None):
    """(HBM-side bytes per launch, note) for the record `key` of profiles/traffic.json: L2
    fetches + writes counted by rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over this program and
    scaled by the factors its 512 MiB copy gives.  The figure is only used when the file was
    made from the kernel sources (and, where given, the launch grid) that run now; otherwise
    (None, why)."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError) as exc:
        return None, f"no traffic record: {exc}"
    if rec.get("source_digest") != kernel_source_digest():
        return None, "profiles/traffic.json was measured on other kernel sources: re-run the PMC profile"
    k = rec.get("kernels", {}).get(key)
    if k is None:
        return None, f"profiles/traffic.json has no entry for {key}"
    if grid is not None and int(k.get("grid", -1)) != int(grid):
        return None, f"profiles/traffic.json: {key} was measured with grid {k.get('grid')}, not {grid}"
    return float(k["fetch_bytes"]) + float(k["write_bytes"]), None


SECTIONS = ("chain", "extras", "sweep", "weights", "ffn")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--sections", default=",".join(SECTIONS),
                    help="comma-separated subset of chain,extras,sweep,weights,ffn (default: all); the headline "
                         "chain is always measured")
    ap.add_argument("--chain-only", action="store_true", help="same as --sections chain")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--maxvio", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=2024)
    args = ap.parse_args()
    args.sections = {"chain"} if args.chain_only else set(x for x in args.sections.split(",") if x)
    unknown = args.sections - set(SECTIONS)
    if unknown:
        ap.error(f"unknown section(s): {sorted(unknown)}")
    return args


def hbm_roofline(kernel, algorithmic_bytes, us, traffic=None, **extra):
    """A roofline record of an HBM-bound kernel: algorithmic bytes per launch over its
    average launch duration against the 8 TB/s of MI355X."""
    achieved = algorithmic_bytes / us / 1e3 if us > 0 and algorithmic_bytes else 0.0
    return {"bound": "hbm", "kernel": kernel, "algorithmic_bytes": algorithmic_bytes,
            "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, **extra}


def time_launches(fn, iters, warmup=2):
    """Average duration in microseconds of one `fn()` (a kernel launch on the current
    stream): `iters` launches are captured into one HIP graph, so that host-side
    launch cost (larger than a 10 us kernel when it comes from Python) stays out of
    the figure; HIP events bracket the replay on the launching stream."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(iters):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    graph.replay()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) * 1e3 / iters


class Chain:
    """plan -> dispatch -> combine of one rank on its real shapes."""

    def __init__(self, S, H, K, E, R, tp, rank, maxvio, seed, nsets=6):
        import torch

        from moonep_amd import Buffer, routing
        from moonep_amd.combine import launch_combine
        from moonep_amd.dispatch import launch_dispatch
        from moonep_amd.planning import allocate_planning_outputs, launch_planning

        self.S, self.H, self.K, self.E, self.R = S, H, K, E, R
        dev = torch.device("cuda", 0)
        topk, w, tpe, self.maxvio, self.sigma = routing.logit_routing(S, K, E, R, maxvio, seed)
        self.topk_all, self.tpe_cpu, self.w_cpu = topk, tpe, w
        self.buf = Buffer(S, H, K, E, R, token_padding=tp, rank=rank)
        self.ctx = ctx = self.buf._require_ctx()
        self.rank = rank
        self.topk = topk[rank].reshape(-1).contiguous().to(dev)
        self.tpe = tpe.to(dev)
        self.wk = w[rank].contiguous().to(dev)
        g = torch.Generator().manual_seed(seed + 99)
        # six input/output sets (352 MB each way): more than the 256 MB of last-level
        # cache, so a launch never finds its token rows cached from the previous one
        self.hidden = [torch.randn(S, H, generator=g).to(torch.bfloat16).to(dev) for _ in range(nsets)]
        self.out = [torch.empty(S, H, dtype=torch.bfloat16, device=dev) for _ in range(nsets)]
        self.out_w = torch.empty(S, K, dtype=torch.float32, device=dev)
        self.plan, self.cu = allocate_planning_outputs(ctx)
        ctx["hidden_buf"].zero_()

        def plan_fn(i=None):
            # as Buffer.dispatch does on a fresh plan: the idle CUs read the token set
            # that the following dispatch copies
            launch_planning(ctx, self.topk, self.tpe, self.cu, self.plan,
                            warm=None if i is None else self.hidden[i])

        def dispatch_fn(i=0):
            launch_dispatch(ctx, self.hidden[i], self.wk, self.plan, build_dedup_map=False,
                            write_dups=True)

        def combine_fn(i=0):
            launch_combine(ctx, self.out[i], self.plan.dst, self.out_w, mode="two_level")

        def combine_weighted_fn(i=0):
            # extension: sum_k w*row (the reference combine is unweighted); timed beside it
            launch_combine(ctx, self.out[i], self.plan.dst, None, mode="weighted")

        self.plan_fn, self.dispatch_fn, self.combine_fn = plan_fn, dispatch_fn, combine_fn
        self.combine_weighted_fn = combine_weighted_fn
        # eager once (also validates), then capture one graph per buffer set
        plan_fn(); dispatch_fn(); combine_fn()
        torch.cuda.synchronize()
        self.graphs = []
        for i in range(nsets):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                plan_fn(i); dispatch_fn(i); combine_fn(i)
            self.graphs.append(gr)
        torch.cuda.synchronize()

    def bytes_one_way(self):
        return self.S * self.H * 2 + self.S * self.K * self.H * 2

    def step(self, i):
        self.graphs[i % len(self.graphs)].replay()

    def destroy(self):
        self.graphs = []
        self.buf.destroy()


def measure_chain(ch, steps, warmup, kernels=True):
    """W warm-up steps, then exactly K timed steps.  The K steps (plan, dispatch,
    combine on the rotating buffer sets) are recorded into one HIP graph, as the
    reference's harness does (benchmarks/bench_comm.py:118-156: events around one
    replay of a graph of `iters` launches), so the per-replay start-up of a graph
    is paid once and not once per step.  The time of K single-step replays is
    reported beside it."""
    import torch

    for i in range(warmup):
        ch.step(i)
    torch.cuda.synchronize()
    big = torch.cuda.CUDAGraph()
    with torch.cuda.graph(big):
        for i in range(steps):
            j = i % len(ch.hidden)
            ch.plan_fn(j); ch.dispatch_fn(j); ch.combine_fn(j)
    big.replay()   # first replay of a new graph uploads it: untimed
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    a.record()
    big.replay()
    b.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = a.elapsed_time(b) / steps
    a.record()
    for i in range(steps):
        ch.step(i)
    b.record()
    torch.cuda.synchronize()
    single_ms = a.elapsed_time(b) / steps
    # the three kernels as they run inside a step: events between the launches of
    # an eager loop (the host issues a step in ~60 us, the GPU needs ~200, so the
    # queue never runs dry and the events bracket GPU time)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    for i in range(steps):
        j = i % len(ch.hidden)
        evs[i][0].record(); ch.plan_fn(j)
        evs[i][1].record(); ch.dispatch_fn(j)
        evs[i][2].record(); ch.combine_fn(j)
        evs[i][3].record()
    torch.cuda.synchronize()
    skip = min(2, steps - 1)
    in_chain = [sum(e[q].elapsed_time(e[q + 1]) for e in evs[skip:]) * 1e3 / (steps - skip) for q in range(3)]
    per = {}
    per["single_replay_ms"] = single_ms
    per["plan_us_in_chain"], per["dispatch_us_in_chain"], per["combine_us_in_chain"] = in_chain
    if not kernels:      # the sweep only needs the chain and its kernels as they run in it
        return wall_ms, ev_ms, per
    n = max(steps, 10)
    per["plan_us"] = time_launches(ch.plan_fn, n)
    k = [0]

    def pw():   # the planner as the chain launches it: idle CUs read the next token set
        k[0] += 1
        ch.plan_fn(k[0] % len(ch.hidden))

    per["plan_with_cache_warming_us"] = time_launches(pw, n)

    def d():
        k[0] += 1
        ch.dispatch_fn(k[0] % len(ch.hidden))

    def c():
        k[0] += 1
        ch.combine_fn(k[0] % len(ch.out))

    per["dispatch_us"] = time_launches(d, n)
    per["combine_us"] = time_launches(c, n)
    # the same token buffer every launch: rows stay in the last-level cache, as they
    # do when dispatch follows the kernel that produced them
    per["dispatch_us_warm_input"] = time_launches(lambda: ch.dispatch_fn(0), n)

    def cw():
        k[0] += 1
        ch.combine_weighted_fn(k[0] % len(ch.out))

    per["combine_weighted_us"] = time_launches(cw, n)
    by = ch.bytes_one_way()
    per["dispatch_GBps"] = by / per["dispatch_us"] / 1e3
    per["combine_GBps"] = by / per["combine_us"] / 1e3
    per["single_replay_ms"] = single_ms
    per["plan_us_in_chain"], per["dispatch_us_in_chain"], per["combine_us_in_chain"] = in_chain
    return wall_ms, ev_ms, per


def chain_on_limited_cus(ch, steps):
    """What the chain costs when it may only use N compute units (a CU-masked stream, what
    Buffer(num_sms=N) launches on): the figure a caller needs who runs the expert GEMMs beside
    it on the other CUs.  Eager launches, HIP events on that stream (the GPU needs more time per
    step than the host needs to issue one, so the queue never runs dry)."""
    import torch

    from moonep_amd.api import _limited_stream

    out = {}
    by = ch.bytes_one_way()
    for n in (32, 64, 128, 256):
        _, st = _limited_stream(0, n)
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            for i in range(2):
                ch.plan_fn(i); ch.dispatch_fn(i); ch.combine_fn(i)
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
            t = [0.0, 0.0, 0.0]
            for i in range(steps):
                j = i % len(ch.hidden)
                evs[0].record(); ch.plan_fn(j)
                evs[1].record(); ch.dispatch_fn(j)
                evs[2].record(); ch.combine_fn(j)
                evs[3].record()
                evs[3].synchronize()
                for q in range(3):
                    t[q] += evs[q].elapsed_time(evs[q + 1]) * 1e3 / steps
        torch.cuda.current_stream().wait_stream(st)
        out[f"{n}_cus"] = {"plan_us": t[0], "dispatch_us": t[1], "combine_us": t[2],
                           "chain_us": sum(t), "GBps": 2 * by / sum(t) / 1e3}
    return out


def chain_on_rotating_shards(ch, steps, nsets=6):
    """The chain with the destination shards rotated too: dispatch of step i writes shard set i,
    combine reads set i+3, written three steps (1.5 GB of rows) earlier, as in a layer whose
    expert GEMMs run between the two.  Beside it the chain as timed above (one shard set) in
    the same form.  Equal figures say that the headline does not live on rows that combine
    finds in the 256 MB last-level cache right after dispatch wrote them."""
    import torch

    from moonep_amd.combine import launch_combine
    from moonep_amd.dispatch import launch_dispatch

    ctxs = [ch.ctx]
    for _ in range(1, nsets):
        c = dict(ch.ctx)
        c["hidden_buf"] = torch.zeros_like(ch.ctx["hidden_buf"])
        c["meta_buf"] = ch.ctx["meta_buf"].clone()
        ctxs.append(c)
    ch.plan_fn()
    for i in range(nsets):
        launch_dispatch(ctxs[i], ch.hidden[i % len(ch.hidden)], ch.wk, ch.plan, build_dedup_map=False,
                        write_dups=True)
    torch.cuda.synchronize()
    k = [0]

    def chain(shift, rotate):
        def fn():
            k[0] += 1
            i = k[0] % nsets
            j = i % len(ch.hidden)
            ch.plan_fn(j)
            launch_dispatch(ctxs[i if rotate else 0], ch.hidden[j], ch.wk, ch.plan,
                            build_dedup_map=False, write_dups=True)
            launch_combine(ctxs[(i + shift) % nsets if rotate else 0], ch.out[j], ch.plan.dst,
                           ch.out_w, mode="two_level")
        return fn

    out = {"one_shard_set_us": time_launches(chain(0, False), steps),
           "rotating_shard_sets_us": time_launches(chain(nsets // 2, True), steps),
           "shard_sets": nsets, "GB_per_shard_set": ch.ctx["hidden_buf"].numel() * 2 / 1e9}
    del ctxs
    torch.cuda.empty_cache()
    return out


def buffer_api_eager(ch, steps):
    """Buffer.dispatch + Buffer.combine called eagerly, as a training loop without graphs calls
    them (fresh plan every step, zero-copy views): what the host needs to issue a step (Python,
    argument checks, ctypes) and what a step takes on the GPU with the queue kept full."""
    import torch

    buf = ch.buf
    wk, tk = ch.wk, ch.topk

    def step(i):
        rows, rw, _, plan = buf.dispatch(ch.hidden[i % len(ch.hidden)], wk, tk, ch.tpe, zero_copy=True)
        return buf.combine(plan, rows, rw, zero_copy=True)

    for i in range(5):
        step(i)
    torch.cuda.synchronize()
    n = max(50, 5 * steps)
    t0 = time.perf_counter()
    for i in range(n):
        step(i)
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    return {"steps": n, "host_issue_us_per_step": (t1 - t0) * 1e6 / n, "us_per_step": (t2 - t0) * 1e6 / n}


def split_duplicate_flow(ch, iters):
    """The reference's separate kernels for duplicate rows, on the headline configuration:
    every rank planned in one launch (the all-rank `dst` the duplicate map is built from), the
    duplicate-group builder (reference moonep/dispatch.py:502-681), dispatch of the primaries
    alone + the epilogue that expands them on the destination (dispatch_epilogue.py:44-304), the
    prologue that folds duplicates into their primaries + the primaries-only combine
    (combine_prologue.py:41-484), beside the fused forms the chain uses.  The epilogue and the
    prologue work on this rank's shard as all R ranks' rows would fill it; the groups come from
    the real all-rank plan, the rows' contents do not matter to the timing.  Launches repeat on
    the same rows, part of which the 256 MB last-level cache still holds."""
    import torch

    from moonep_amd.combine import launch_combine, launch_combine_prologue
    from moonep_amd.dispatch import launch_build_dedup, launch_dispatch, launch_dispatch_epilogue
    from moonep_amd.planning import launch_planning_all_ranks

    ctx, dev = ch.ctx, ch.topk.device
    topk_all = ch.topk_all.to(torch.int32).contiguous().to(dev)
    ch.plan_fn()
    dst_all = launch_planning_all_ranks(ctx, topk_all, ch.tpe)[0]
    torch.cuda.synchronize()
    assert torch.equal(dst_all[ch.rank], ch.plan.dst)
    out = {"plan_all_ranks_us": time_launches(lambda: launch_planning_all_ranks(ctx, topk_all, ch.tpe), iters),
           "build_dedup_us": time_launches(lambda: launch_build_dedup(ctx, dst_all, ch.plan), iters)}
    torch.cuda.synchronize()
    groups, dups = (int(x) for x in ch.plan.dup_counts.cpu())
    row = ch.H * 2
    own_dups = int((ch.plan.dst < 0).sum())
    out.update({"duplicate_groups_on_this_rank": groups, "duplicate_rows_on_this_rank": dups,
                "duplicate_entries_of_this_rank": own_dups})
    us = time_launches(lambda: launch_dispatch(ctx, ch.hidden[0], ch.wk, ch.plan, build_dedup_map=False,
                                               write_dups=False), iters)
    out["dispatch_primaries_us"] = us
    us = time_launches(lambda: launch_dispatch_epilogue(ctx, ch.plan), iters)
    out["dispatch_epilogue_us"] = us
    out["dispatch_epilogue_roofline"] = hbm_roofline("dup_rows_kernel<false> (dispatch epilogue)", (groups + dups) * row, us,
                                                     measured_traffic("dispatch_epilogue")[0])
    us = time_launches(lambda: launch_combine_prologue(ctx, ch.plan), iters)
    out["combine_prologue_us"] = us
    out["combine_prologue_roofline"] = hbm_roofline("dup_rows_kernel<true> (combine prologue)", (2 * groups + dups) * row, us,
                                                    measured_traffic("combine_prologue")[0])
    out["combine_primaries_us"] = time_launches(
        lambda: launch_combine(ctx, ch.out[0], ch.plan.dst, ch.out_w, mode="primaries"), iters)
    ctx["hidden_buf"].zero_()
    torch.cuda.synchronize()
    return out


def cpu_baseline(ch, budget_s=10.0):
    """Scalar C port of plan + dispatch + combine on the same inputs, host cores."""
    import numpy as np
    import torch

    from oracle import c_oracle as co

    S, H, K, E, R = ch.S, ch.H, ch.K, ch.E, ch.R
    ctx = ch.ctx
    NvS, tp = int(ctx["NvS"]), int(ctx["token_padding"])
    topk = ch.topk_all[ch.rank].numpy()
    tpe = ch.tpe_cpu.numpy()
    hidden = ch.hidden[0].cpu().view(torch.int16).numpy().view(np.uint16)
    w = ch.w_cpu[ch.rank].contiguous().numpy()
    shards = np.empty((R, NvS, H), np.uint16)   # pages are touched only where rows land
    wslots = np.empty((R, NvS), np.float32)
    times = []
    t_all = time.perf_counter()
    while True:
        t0 = time.perf_counter()
        dst, cu, etc, zf, st = co.plan(tpe, topk, ch.rank, S, K, tp, NvS)
        t1 = time.perf_counter()
        co.dispatch(hidden, w, dst, zf, shards, wslots, ch.rank, K, NvS, True)
        t2 = time.perf_counter()
        out, out_w = co.combine(shards, wslots, dst, S, K, NvS, 2)
        t3 = time.perf_counter()
        times.append((t1 - t0, t2 - t1, t3 - t2))
        if len(times) >= 2 and time.perf_counter() - t_all > budget_s or len(times) >= 64:
            break
    # first pass pays the page faults of the fresh shards: report the best later pass
    p, d, c = min(times[1:], key=lambda t: sum(t))
    total = p + d + c
    ch.plan_fn(); ch.dispatch_fn(0); ch.combine_fn(0)   # the GPU's answer for the same token set
    torch.cuda.synchronize()
    got = ch.out[0].cpu().view(torch.int16).numpy().view(np.uint16)
    # the same two data movements as torch-CPU index ops on every host core the
    # process may use (the comparison the reference's own harness would make)
    tdst = torch.from_numpy(dst.astype(np.int64))
    rows = torch.where(tdst < 0, -tdst - 1, tdst)
    th = ch.hidden[0].cpu()
    tsh = torch.from_numpy(shards.view(np.int16)).view(torch.bfloat16).view(R * NvS, H)
    tok = torch.arange(S).repeat_interleave(K)
    tt = []
    for _ in range(3):
        t0 = time.perf_counter()
        tsh.index_copy_(0, rows, th[tok])
        t1 = time.perf_counter()
        tout = tsh.index_select(0, rows).float().view(S, K, H).sum(1).to(torch.bfloat16)
        t2 = time.perf_counter()
        tt.append((t1 - t0, t2 - t1))
    td, tc = min(tt, key=lambda t: sum(t))
    nthreads = torch.get_num_threads()
    torch.set_num_threads(1)
    t0 = time.perf_counter()
    tsh.index_copy_(0, rows, th[tok])
    t1 = time.perf_counter()
    tsh.index_select(0, rows).float().view(S, K, H).sum(1).to(torch.bfloat16)
    t2 = time.perf_counter()
    torch.set_num_threads(nthreads)
    return {
        "torch_cpu_threads": nthreads,
        "torch_cpu_dispatch_GBps": ch.bytes_one_way() / td / 1e9,
        "torch_cpu_combine_GBps": ch.bytes_one_way() / tc / 1e9,
        "torch_cpu_1thread_dispatch_GBps": ch.bytes_one_way() / (t1 - t0) / 1e9,
        "torch_cpu_1thread_combine_GBps": ch.bytes_one_way() / (t2 - t1) / 1e9,
        "value": 2 * ch.bytes_one_way() / total / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"full workload (S={S} tokens of one rank), best of {len(times) - 1} passes after 1 warm-up "
                  f"({time.perf_counter() - t_all:.0f} s of CPU work)",
        "plan_us": p * 1e6, "dispatch_GBps": ch.bytes_one_way() / d / 1e9,
        "combine_GBps": ch.bytes_one_way() / c / 1e9, "host_cpus": os.cpu_count(),
        "matches_gpu_output": bool(np.array_equal(out, got)),
    }


def gpu_plan_all_ranks(S, K, E, R, tp, topk, tpe):
    """All ranks' plans from the HIP planner: (cu_seqlens [R,2*epn] on the device,
    experts_to_copy [R,epn] as numpy, NvS)."""
    import torch

    from moonep_amd import Buffer
    from moonep_amd.planning import launch_planning_all_ranks

    buf = Buffer(S, 16, K, E, R, token_padding=tp, rank=0)   # H plays no part in planning
    ctx = buf._require_ctx()
    dev = torch.device("cuda", 0)
    _, cu, etc, _, _ = launch_planning_all_ranks(ctx, topk.to(dev), tpe.to(dev))
    torch.cuda.synchronize()
    out = cu.clone(), etc.cpu().numpy().astype("int64"), int(ctx["NvS"])
    buf.destroy()
    return out


def bench_weights(seed, steps, cpu=True):
    """prefetch_weight (3 projections, one launch: the owner's push, and the pull of one
    rank's slots from all owners) and reduce_grad (one projection) at H=7168, H'=2048,
    epn=32, R=8 for two slot tables: the planner's own at maxvio~1 (busiest owner /
    fullest rank) and a denser ring (every rank hosts 8 remote experts)."""
    import numpy as np
    import torch

    from moonep_amd import routing
    from moonep_amd.grad_reduce import launch_grad_reduce
    from moonep_amd.prefetch import launch_prefetch, launch_prefetch_pull

    S, K, E, R, H, Hp = 4096, 8, 256, 8, 7168, 2048
    epn = E // R
    dev = torch.device("cuda", 0)
    topk, _, tpe, mv, _ = routing.logit_routing(S, K, E, R, 1.0, seed, want_weights=False)
    planned = gpu_plan_all_ranks(S, K, E, R, 128, topk, tpe)[1]
    ring = -np.ones((R, epn), dtype=np.int64)
    for d in range(R):
        for b in range(8):
            ring[d, b] = ((d + 1 + b) % R) * epn + (d * 8 + b) % epn
    per = H * Hp
    # three projections = three different local tensors and three different pools (25 GB), and
    # every table in three renumbered variants (other local experts, other slots, same counts)
    # that the timed launches take in turn: no launch finds its experts or its slots in the
    # 256 MB last-level cache from the projection or the launch before it
    local = [(torch.randn(epn, H, Hp, device=dev) * 0.02).to(torch.bfloat16) for _ in range(3)]
    pool = [torch.empty(R, epn, H, Hp, dtype=torch.bfloat16, device=dev) for _ in range(3)]
    # every rank's local experts side by side, for the pull (contents do not matter to a copy)
    owners = [torch.empty(R, epn, H, Hp, dtype=torch.bfloat16, device=dev) for _ in range(3)]
    res = {"plan_maxvio": mv}
    tables = {"planner": planned, "ring8": ring}
    NROT = 3

    def renumbered(etc_np, v):
        """Local expert le -> (le + 11 v) % epn, slot b -> (b + 5 v) % epn."""
        e = etc_np.copy()
        m = e >= 0
        e[m] = (e[m] // epn) * epn + (e[m] % epn + 11 * v) % epn
        return np.roll(e, 5 * v, axis=1)

    stats = {}
    for name, etc_np in tables.items():
        owned = [(int(((etc_np // epn) == r).sum()), r) for r in range(R)]
        n_slots, rank = max(owned)
        active = len({int(e) for e in etc_np.reshape(-1) if e >= 0 and e // epn == rank})
        own_slots = int((etc_np[rank] >= 0).sum())
        variants = [torch.from_numpy(renumbered(etc_np, v).astype("int32")).to(dev) for v in range(NROT)]
        stats[name] = (variants, rank, n_slots, active, own_slots)
        k = [0]

        def pf():
            k[0] += 1
            launch_prefetch(tuple(local), tuple(pool), variants[k[0] % NROT], rank=rank)

        us = time_launches(pf, steps)
        by = 3 * (active + n_slots) * per * 2   # each owned expert read once, every slot written
        res[name] = {"rank": rank, "slots": n_slots, "active_experts": active,
                     "own_occupied_slots": own_slots, "prefetch_us_3proj": us,
                     "prefetch_bytes": by, "prefetch_GBps": by / us / 1e3 if by else 0.0,
                     "prefetch_roofline": hbm_roofline("prefetch_kernel", by, us,
                                                       measured_traffic(f"prefetch_kernel@{name}")[0])}
        # the pull view: the fullest rank's slots from all owners in one launch
        pull_slots, pull_rank = max((int((etc_np[r] >= 0).sum()), r) for r in range(R))

        def pl():
            k[0] += 1
            launch_prefetch_pull(tuple(owners), tuple(pool), variants[k[0] % NROT], rank=pull_rank)

        us = time_launches(pl, steps)
        by = 3 * 2 * pull_slots * per * 2       # every occupied slot: one expert read, one written
        res[name].update({"pull_rank": pull_rank, "pull_slots": pull_slots, "prefetch_pull_us_3proj": us,
                          "prefetch_pull_bytes": by, "prefetch_pull_GBps": by / us / 1e3 if by else 0.0,
                          "prefetch_pull_roofline": hbm_roofline(
                              "prefetch_pull_kernel", by, us, measured_traffic(f"prefetch_pull_kernel@{name}")[0])})
    del local, pool, owners
    torch.cuda.empty_cache()
    grad = torch.zeros(epn, H, Hp, dtype=torch.float32, device=dev)
    red = torch.randn(R, epn, H, Hp, dtype=torch.float32, device=dev) * 1e-3
    for name, (variants, rank, n_slots, active, own_slots) in stats.items():
        k = [0]

        def gr():
            k[0] += 1
            launch_grad_reduce(grad, red, variants[k[0] % NROT], rank=rank)

        us = time_launches(gr, steps)
        by = (n_slots + 2 * active + own_slots) * per * 4   # slots read, grads read+written, clears
        res[name].update({"grad_reduce_us": us, "grad_reduce_bytes": by,
                          "grad_reduce_GBps": by / us / 1e3 if by else 0.0,
                          "grad_reduce_roofline": hbm_roofline(
                              "grad_reduce_kernel", by, us, measured_traffic(f"grad_reduce_kernel@{name}")[0])})
    del grad, red
    torch.cuda.empty_cache()
    if not cpu:
        return res
    # host-core figures on a bounded sample of one projection: 16 slot copies
    # (index_copy_) and 8 slot sums (add_ then zero_), all torch threads; a 1 GiB
    # fill between warm-up and timing pushes the sample out of the host caches
    n, m = 16, 8
    lc = (torch.randn(n, H, Hp) * 0.02).to(torch.bfloat16)
    pc = torch.empty(2 * n, H, Hp, dtype=torch.bfloat16)
    idx = torch.arange(n) * 2 + 1
    gc, rc = torch.zeros(m, H, Hp), torch.randn(m, H, Hp) * 1e-3
    pc.index_copy_(0, idx, lc)
    flush = torch.empty(1 << 28, dtype=torch.float32)
    flush.fill_(1.0)
    t0 = time.perf_counter()
    pc.index_copy_(0, idx, lc)
    t1 = time.perf_counter()
    flush.fill_(2.0)
    t2 = time.perf_counter()
    for i in range(m):
        gc[i].add_(rc[i])
        rc[i].zero_()
    t3 = time.perf_counter()
    res["cpu_baseline"] = {
        "torch_cpu_threads": torch.get_num_threads(),
        "sample": f"{n} slot copies / {m} slot sums of one projection",
        "prefetch_GBps": 2 * n * per * 2 / (t1 - t0) / 1e9,
        "grad_reduce_GBps": 4 * m * per * 4 / (t3 - t2) / 1e9}
    return res


def bench_ffn(seed, steps):
    """Expert-side consumer at the real shape: one rank's dispatched rows
    (planner's own cu_seqlens at maxvio ~ 1, NvS = 40960 rows, H = 7168) through
    the grouped SwiGLU gate/up GEMM (H' = 2048) and the grouped down GEMM, 64
    groups.  FLOPs count the rows inside groups (padding rows included)."""
    import torch

    from moonep_amd import routing
    from moonep_amd import ffn
    from moonep_amd.ffn import launch_grouped_gemm_nt

    S, K, E, R, H, Hp = 4096, 8, 256, 8, 7168, 2048
    G = 2 * (E // R)
    dev = torch.device("cuda", 0)
    topk, _, tpe, mv, _ = routing.logit_routing(S, K, E, R, 1.0, seed, want_weights=False)
    cu_all, _, NvS = gpu_plan_all_ranks(S, K, E, R, 128, topk, tpe)
    cu = cu_all[0].contiguous()
    used = int(cu[-1])
    g = torch.Generator(device=dev).manual_seed(seed)
    rows = torch.randn(NvS, H, device=dev, generator=g).to(torch.bfloat16)
    gate = (torch.randn(G, Hp, H, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    up = (torch.randn(G, Hp, H, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    down = (torch.randn(G, H, Hp, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    slots = torch.rand(NvS, device=dev, generator=g)
    hmid = torch.zeros(NvS, Hp, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(NvS, H, dtype=torch.bfloat16, device=dev)
    t1 = time_launches(lambda: launch_grouped_gemm_nt(rows, gate, cu, hmid, up_weights=up), steps)
    t2 = time_launches(lambda: launch_grouped_gemm_nt(hmid, down, cu, out, row_scale=slots), steps)
    f1, f2 = 4.0 * used * H * Hp, 2.0 * used * H * Hp
    # the library's dense GEMM of the same volume, for scale (one weight matrix, no groups)
    c = torch.empty(used, Hp, dtype=torch.bfloat16, device=dev)
    t3 = time_launches(lambda: torch.matmul(rows[:used], gate[0].t(), out=c), steps)
    peak = 2500.0
    # backward of the same FFN: every GEMM on the grouped kernels, operands as the passes hold them
    del c
    dy = torch.randn(NvS, H, device=dev, generator=g).to(torch.bfloat16)
    _, saved = ffn.grouped_ffn_hip_forward(rows, slots, cu, gate, up, down)
    bw = {}
    # the input gradients read the forward pass's weight tensors as they are ([K, N] form)
    dh = ffn.launch_grouped_gemm_nn(dy, down, cu)
    bw["dh_gemm_us"] = time_launches(lambda: ffn.launch_grouped_gemm_nn(dy, down, cu, dh), steps)
    sb = ffn.launch_swiglu_bwd(dh, saved[0], saved[1], slots, cu)
    dg, du = sb[0], sb[1]
    bw["swiglu_bwd_us"] = time_launches(lambda: ffn.launch_swiglu_bwd(dh, saved[0], saved[1], slots, cu, sb), steps)
    drows = ffn.launch_grouped_gemm_dual_nn(dg, gate, du, up, cu)
    bw["dual_dgrad_gemm_us"] = time_launches(
        lambda: ffn.launch_grouped_gemm_dual_nn(dg, gate, du, up, cu, drows), steps)
    del drows
    # the weight gradients read the activations as they are (an expert's shapes: no transposes)
    # ... and leave the gradients of slots that hold no expert unwritten, as the layer does
    # (reduce_grad never reads them); with those 58.7 MB per unused slot zeroed beside it
    dwg = ffn.launch_grouped_gemm_wgrad_tn(dg, rows, cu)
    bw["wgrad_gemm_us_each_zeroing_unused_slots"] = time_launches(
        lambda: ffn.launch_grouped_gemm_wgrad_tn(dg, rows, cu, dwg), steps)
    bw["wgrad_gemm_us_each"] = time_launches(
        lambda: ffn.launch_grouped_gemm_wgrad_tn(dg, rows, cu, dwg, skip_empty_from=G // 2), steps)
    del dg, du, sb, dh, dwg
    gemm_us = bw["dh_gemm_us"] + bw["dual_dgrad_gemm_us"] + 3 * bw["wgrad_gemm_us_each"]
    bw["gemm_TFLOPs"] = 12.0 * used * H * Hp / gemm_us / 1e6
    bw["total_us"] = gemm_us + bw["swiglu_bwd_us"]
    bw["TFLOPs"] = 12.0 * used * H * Hp / bw["total_us"] / 1e6
    return {
        "rows_in_groups": used, "NvS": NvS, "groups": G, "maxvio": mv, "backward": bw,
        "swiglu_gate_up_us": t1, "swiglu_gate_up_TFLOPs": f1 / t1 / 1e6,
        "down_us": t2, "down_TFLOPs": f2 / t2 / 1e6,
        "roofline": {"bound": "mfma", "kernel": "grouped_gemm256_kernel (SwiGLU gate/up + down)",
                     "achieved": (f1 + f2) / (t1 + t2) / 1e6, "peak": peak, "unit": "TFLOP/s",
                     "frac": (f1 + f2) / (t1 + t2) / 1e6 / peak,
                     "traffic": measured_traffic("grouped_gemm_forward")[0]},
        "library_dense_gemm_TFLOPs": 2.0 * used * H * Hp / t3 / 1e6,
    }


def dispatch_grid(S, K, E, R, tp):
    """Workgroups of one mep_dispatch launch (csrc/dispatch.hip: four (token, k) copies per
    workgroup, then the zero-fill workgroups of 2*epn groups)."""
    zpg = max(1, min(32, (tp - 1 + 3) // 4))
    return (S * K + 3) // 4 + (2 * (E // R) * zpg if tp > 1 else 0)


def sweep_point(ch, steps, warmup, repeats=3):
    """One point of the maxvio sweep, timed like the headline: `warmup` steps, then the
    `steps` steps of one HIP graph between two events, `repeats` times; returns (the
    per-step microseconds of every repeat, the kernels' durations inside an eager chain)."""
    import torch

    for i in range(warmup):
        ch.step(i)
    torch.cuda.synchronize()
    big = torch.cuda.CUDAGraph()
    with torch.cuda.graph(big):
        for i in range(steps):
            j = i % len(ch.hidden)
            ch.plan_fn(j); ch.dispatch_fn(j); ch.combine_fn(j)
    big.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    for _ in range(repeats):
        a.record()
        big.replay()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b) * 1e3 / steps)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    for i in range(steps):
        j = i % len(ch.hidden)
        evs[i][0].record(); ch.plan_fn(j)
        evs[i][1].record(); ch.dispatch_fn(j)
        evs[i][2].record(); ch.combine_fn(j)
        evs[i][3].record()
    torch.cuda.synchronize()
    skip = min(2, steps - 1)
    in_chain = [sum(e[q].elapsed_time(e[q + 1]) for e in evs[skip:]) * 1e3 / (steps - skip) for q in range(3)]
    return times, in_chain


def calibration_copy(repeats=3):
    """A 512 MiB device-to-device copy: the kernel of known size (reads 512 MiB, writes
    512 MiB) that FETCH_SIZE / WRITE_SIZE of a counter run of this program are scaled by."""
    import torch

    src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda").view(torch.float32)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(repeats):
        dst.copy_(src)
    b.record()
    b.synchronize()
    us = a.elapsed_time(b) * 1e3 / repeats
    del src, dst
    torch.cuda.empty_cache()
    return {"bytes_each_way": 512 << 20, "us": us, "GBps": 2 * (512 << 20) / us / 1e3}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one rank's share on ONE GPU; --gpus > 1 is not part of this "
              "build (no collectives, no sharding).", file=sys.stderr)
        sys.exit(2)
    import torch

    torch.cuda.set_device(0)
    copy_rec = calibration_copy()
    S, H, K, E, R, tp, rank = 4096, 7168, 8, 256, 8, 128, 0
    ch = Chain(S, H, K, E, R, tp, rank, args.maxvio, args.seed)
    wall_ms, ev_ms, per = measure_chain(ch, args.steps, args.warmup)
    by = ch.bytes_one_way()
    value = 2 * by / (wall_ms * 1e-3) / 1e9
    # roofline: the dominant kernel, from its cold standalone duration (the duration inside
    # the timed steps, with the tokens already pulled into cache by the planner launch, beside it)
    dom = "dispatch" if per["dispatch_us"] >= per["combine_us"] else "combine"
    grid = dispatch_grid(S, K, E, R, tp) if dom == "dispatch" else S * 7 // 4
    traffic, traffic_note = measured_traffic(f"{dom}_kernel", grid)
    roof = hbm_roofline(f"{dom}_kernel", by, per[f"{dom}_us"], traffic,
                        duration_us=per[f"{dom}_us"], duration_us_in_timed_steps=per[f"{dom}_us_in_chain"],
                        frac_in_timed_steps=by / per[f"{dom}_us_in_chain"] / 1e3 / HBM_PEAK_GBPS)
    if traffic_note:
        roof["traffic_note"] = traffic_note
    line = {
        "metric": "dispatch+combine GB/s of one rank's plan->dispatch->combine chain (plan us reported beside)",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "config 1: single-rank dispatch+combine, S=4096 H=7168 K=8 E=256 R=8 "
                               "token_padding=128, the timed plan->dispatch->combine steps recorded in one HIP graph; "
                               "kernels on the whole GPU (the reference's default bounds them to 32 SMs: see "
                               "chain_on_limited_cus)",
                   "maxvio": round(ch.maxvio, 3), "seed": args.seed, "rank": rank},
        "roofline": roof,
        "combine_roofline": hbm_roofline("combine_kernel", by, per["combine_us"],
                                         measured_traffic("combine_kernel", S * 7 // 4)[0]),
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBPS,
        "graph_ms_per_step_events": ev_ms,
        "ms_per_step_one_graph_replay_per_step": per["single_replay_ms"],
        "plan_us": per["plan_us"], "plan_with_cache_warming_us": per["plan_with_cache_warming_us"],
        "dispatch_us": per["dispatch_us"], "combine_us": per["combine_us"],
        "plan_us_in_chain": per["plan_us_in_chain"], "dispatch_us_in_chain": per["dispatch_us_in_chain"],
        "combine_us_in_chain": per["combine_us_in_chain"],
        "combine_weighted_us": per["combine_weighted_us"],
        "dispatch_GBps": per["dispatch_GBps"], "combine_GBps": per["combine_GBps"],
        "dispatch_us_warm_input": per["dispatch_us_warm_input"],
        "calibration_copy": copy_rec,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(ch)
    sub_steps = max(5, args.steps // 2)
    if "extras" in args.sections:
        line["chain_on_limited_cus"] = chain_on_limited_cus(ch, sub_steps)
        line["chain_on_rotating_shards"] = chain_on_rotating_shards(ch, args.steps)
        line["split_duplicate_flow"] = split_duplicate_flow(ch, sub_steps)
        line["buffer_api_eager"] = buffer_api_eager(ch, args.steps)
    ch.destroy()
    torch.cuda.empty_cache()
    tail = {}          # short summary keys, appended last
    if "sweep" in args.sections:
        sweep, spread, chain_us = {}, {}, {}
        # maxvio 0 .. 4 on both shapes; on the headline shape also 10 and 20, the upper end of the
        # reference's own figure (README.md:15-25: maxvio 0.2, 1, 10, 20), reported beside the five
        for shape in ((4096, 7168, 256), (8192, 4096, 128)):
            tag = f"S{shape[0]}_H{shape[1]}_E{shape[2]}"
            best, beyond = [], []
            for mv in (0.0, 0.5, 1.0, 2.0, 4.0) + ((10.0, 20.0) if shape[0] == 4096 else ()):
                c2 = Chain(shape[0], shape[1], K, shape[2], R, tp, rank, mv, args.seed)
                times, p2 = sweep_point(c2, args.steps, args.warmup)
                us = min(times)
                b2 = c2.bytes_one_way()
                sweep[f"{tag}_maxvio{mv}"] = {
                    "maxvio": round(c2.maxvio, 3), "chain_us": us, "chain_us_repeats": times,
                    "GBps": 2 * b2 / us / 1e3, "pct_hbm_peak": 2 * b2 / us / 1e3 / HBM_PEAK_GBPS * 100.0,
                    "plan_us_in_chain": p2[0], "dispatch_us_in_chain": p2[1], "combine_us_in_chain": p2[2]}
                (best if mv <= 4.0 else beyond).append(round(us, 1))
                c2.destroy()
                torch.cuda.empty_cache()
            chain_us[tag] = best
            spread[tag] = round(100.0 * (max(best) - min(best)) / min(best), 2)
            if beyond:
                chain_us[tag + "_maxvio10_20"] = beyond
                every = best + beyond
                spread[tag + "_with_maxvio10_20"] = round(100.0 * (max(every) - min(every)) / min(every), 2)
        sweep["timing"] = (f"{args.steps} steps in one HIP graph after {args.warmup} warm-up steps, 3 replays per "
                           "point, the fastest kept; maxvio 0, 0.5, 1, 2, 4 in that order (10 and 20 beside them on the headline shape)")
        line["maxvio_sweep"] = sweep
        tail["maxvio_sweep_chain_us"] = chain_us
        tail["maxvio_sweep_spread_pct"] = spread
        # the configuration of the reference's own figure (figure/comm_vs_deepep.png: ep = 8,
        # E = 384, H = 7168, K = 8, S = 8192; H20, read off the chart: planning ~40-50 us,
        # dispatch + epilogue ~1835-1855 us, combine ~1932-1975 us, both bound by NVLink)
        c3 = Chain(8192, 7168, K, 384, R, tp, rank, 1.0, args.seed, nsets=3)
        t3, p3 = sweep_point(c3, sub_steps, 2)
        w3 = min(t3)
        b3 = c3.bytes_one_way()
        line["reference_figure_config"] = {
            "workload": "S=8192 H=7168 K=8 E=384 R=8 token_padding=128, one rank's share on one GPU (HBM-bound; "
                        "the reference's figure is NVLink-bound on H20: not the same quantity)",
            "maxvio": round(c3.maxvio, 3), "chain_us": w3, "GBps": 2 * b3 / w3 / 1e3,
            "pct_hbm_peak": 2 * b3 / w3 / 1e3 / HBM_PEAK_GBPS * 100.0,
            "plan_us_in_chain": p3[0], "dispatch_us_in_chain": p3[1], "combine_us_in_chain": p3[2],
            "reference_read_off_its_figure_us": {"planning": "40-50", "dispatch_and_epilogue": "1835-1855",
                                                 "combine": "1932-1975", "hardware": "H20, 8 GPUs, NVLink"}}
        c3.destroy()
        torch.cuda.empty_cache()
    if "weights" in args.sections:
        line["weights"] = bench_weights(args.seed, sub_steps, cpu=not args.no_cpu)
        torch.cuda.empty_cache()
        tail["weights_frac_of_hbm_peak"] = {
            f"{op}@{name}": round(line["weights"][name][f"{op}_roofline"]["frac"], 3)
            for name in ("planner", "ring8") for op in ("prefetch", "prefetch_pull", "grad_reduce")}
    if "ffn" in args.sections:
        line["ffn"] = bench_ffn(args.seed, sub_steps)
        tail["ffn_frac_of_mfma_peak"] = round(line["ffn"]["roofline"]["frac"], 3)
    # the summary comes last, so that the end of the line shows it
    tail.update({
        "chain_us": round(wall_ms * 1e3, 1), "plan_us_summary": round(per["plan_us"], 1),
        "dispatch_us_cold": round(per["dispatch_us"], 1), "dispatch_us_in_chain_summary": round(per["dispatch_us_in_chain"], 1),
        "combine_us_summary": round(per["combine_us"], 1),
        "dispatch_pct_hbm_peak": round(100.0 * per["dispatch_GBps"] / HBM_PEAK_GBPS, 1),
        "combine_pct_hbm_peak": round(100.0 * per["combine_GBps"] / HBM_PEAK_GBPS, 1),
        "chain_pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 1),
        "roofline_frac": round(roof["frac"], 3)})
    line.update(tail)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
