"""CPU restatement of MoonEP's data-movement ops -- TEST INFRASTRUCTURE ONLY.

Checker for the HIP kernels.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it; moonep_amd never does.

Plain torch-CPU indexing and elementwise fp32 adds in explicit loops, so the
summation order is visible in the source.  Each function names the reference
code whose semantics it restates.  The R ranks' communication shards, weight
slots, prefetch pools and reduce buffers are ordinary ``[R, ...]`` tensors.

Pinned by: every op is a textbook index copy / ordered sum, checked in
tests/test_oracle_ops.py against closed forms (traceable payloads, integer
payloads that make fp32 sums exact, K=1) and against the independent C
restatement in oracle/mep_oracle.c.
"""

from __future__ import annotations

import torch


def decode(dst: torch.Tensor, NvS: int):
    """reference moonep/dispatch.py:406-415"""
    d = dst.long()
    raw = torch.where(d < 0, -d - 1, d)
    return raw // NvS, raw % NvS, d >= 0


def dispatch(hidden_sh, weights_sk, dst, zero_fill, shards, wslots, rank, K,
             include_dups=False):
    """Scatter this rank's tokens into all destination shards.

    reference moonep/dispatch.py:394-433 (row + weight puts) and :467-497
    (zero-fill of the local shard's padding rows and weight slots).
    ``include_dups`` also writes the rows of negative-encoded entries, i.e.
    the result of dispatch followed by every destination's epilogue
    (reference moonep/dispatch_epilogue.py:167-304) for this rank's tokens.
    shards: [R, NvS, H] bf16; wslots: [R, NvS] fp32 or None.
    """
    R, NvS, H = shards.shape
    S = hidden_sh.shape[0]
    drank, loff, primary = decode(dst, NvS)
    tok = torch.arange(S).repeat_interleave(K)
    sel = torch.ones_like(primary) if include_dups else primary
    shards.view(R * NvS, H)[(drank * NvS + loff)[sel]] = hidden_sh[tok[sel]]
    if weights_sk is not None:
        wslots.view(-1)[drank * NvS + loff] = weights_sk.reshape(-1)
    for start, n in zero_fill.tolist():
        if n > 0:
            shards[rank, start:start + n] = 0
            if weights_sk is not None:
                wslots[rank, start:start + n] = 0


def dispatch_epilogue(shard, dup_groups, dup_loffs, dup_counts):
    """reference moonep/dispatch_epilogue.py:167-304: primary row -> each
    duplicate row of its group, inside one rank's shard."""
    for g in range(int(dup_counts[0])):
        p, start, n = (int(v) for v in dup_groups[g])
        for j in range(n):
            shard[int(dup_loffs[start + j])] = shard[p]


def combine_prologue(shard, dup_groups, dup_loffs, dup_counts):
    """reference moonep/combine_prologue.py:380-478: fp32 sum, starting from
    0.0, of the primary row then its duplicates in dup_loffs order, rounded
    once to bf16 and stored over the primary row."""
    for g in range(int(dup_counts[0])):
        p, start, n = (int(v) for v in dup_groups[g])
        acc = torch.zeros(shard.shape[1], dtype=torch.float32)
        acc += shard[p].float()
        for j in range(n):
            acc += shard[int(dup_loffs[start + j])].float()
        shard[p] = acc.to(torch.bfloat16)


def combine(shards, wslots, dst, K, mode="primaries"):
    """Gather + K-sum back to token-major.

    mode "primaries": reference moonep/combine.py:379-435 -- fp32 sum from
        0.0 over the non-negative entries in ascending k, one bf16 rounding.
    mode "all": the same sum over all K entries (what the chain computes when
        no duplicate rows were pre-reduced; single rounding).
    mode "two_level": per destination-rank group an fp32 sum (primary first,
        then its duplicates in ascending k) rounded to bf16, then the fp32 sum
        of the group results in order of their primaries -- the bits the
        reference's prologue + combine pair produces, without touching the
        shards.
    mode "weighted" (an extension, not in the reference): all K entries, each
        row scaled by the fp32 route weight in its slot.
    Weight gather (reference moonep/combine.py:485-511): every entry reads its
    own slot.  Returns (out[S,H] bf16, weights[S,K] fp32 | None).
    """
    R, NvS, H = shards.shape
    N = dst.numel()
    S = N // K
    drank, loff, primary = decode(dst, NvS)
    rows = (drank * NvS + loff).view(S, K)
    prim = primary.view(S, K)
    dr = drank.view(S, K)
    flat = shards.view(R * NvS, H)
    out = torch.empty(S, H, dtype=torch.bfloat16)
    if mode in ("primaries", "all"):
        acc = torch.zeros(S, H, dtype=torch.float32)
        for k in range(K):
            v = flat[rows[:, k]].float()
            if mode == "primaries":
                v = torch.where(prim[:, k:k + 1], v, torch.zeros_like(v))
                # adding +0.0 never changes a running fp32 sum that started at +0.0
            acc += v
        out = acc.to(torch.bfloat16)
    elif mode == "two_level":
        acc = torch.zeros(S, H, dtype=torch.float32)
        for k in range(K):
            is_p = prim[:, k]
            grp = torch.zeros(S, H, dtype=torch.float32)
            grp += flat[rows[:, k]].float()
            for j in range(k + 1, K):
                member = (~prim[:, j]) & (dr[:, j] == dr[:, k])
                v = flat[rows[:, j]].float()
                grp += torch.where(member[:, None], v, torch.zeros_like(v))
            grp = grp.to(torch.bfloat16).float()
            acc += torch.where(is_p[:, None], grp, torch.zeros_like(grp))
        out = acc.to(torch.bfloat16)
    elif mode == "weighted":
        # not a reference mode: sum_k w[s,k] * row_k, product and sum each rounded to fp32
        wk = wslots.view(-1)[drank * NvS + loff].view(S, K)
        acc = torch.zeros(S, H, dtype=torch.float32)
        for k in range(K):
            acc += wk[:, k:k + 1] * flat[rows[:, k]].float()
        out = acc.to(torch.bfloat16)
    else:
        raise ValueError(mode)
    w = None
    if wslots is not None:
        w = wslots.view(-1)[drank * NvS + loff].view(S, K).clone()
    return out, w


def _owned_slots(experts_to_copy, rank, epn):
    """(dest rank, slot, local expert) of every slot holding one of ``rank``'s
    experts, in (dest, slot)-ascending order (reference
    moonep/prefetch.py:322-368, moonep/grad_reduce.py:221-276)."""
    out = []
    R = experts_to_copy.shape[0]
    for d in range(R):
        for b in range(epn):
            e = int(experts_to_copy[d, b])
            if rank * epn <= e < (rank + 1) * epn:
                out.append((d, b, e - rank * epn))
    return out


def prefetch(local, pool, experts_to_copy, rank):
    """Owner push: reference moonep/prefetch.py:398-465.
    local [epn, ...], pool [R, epn, ...] (any dtype)."""
    epn = local.shape[0]
    for d, b, le in _owned_slots(experts_to_copy, rank, epn):
        pool[d, b] = local[le]


def grad_reduce(local_grad, reduce_buf, experts_to_copy, rank):
    """reference moonep/grad_reduce.py:326-389: per owned expert, seed with the
    local grad and add its slots in (src rank, slot)-ascending order in fp32;
    then zero this rank's own slots that hold any expert."""
    epn = local_grad.shape[0]
    for d, b, le in _owned_slots(experts_to_copy, rank, epn):
        local_grad[le] += reduce_buf[d, b]
    for b in range(epn):
        if int(experts_to_copy[rank, b]) >= 0:
            reduce_buf[rank, b] = 0


def bf16_ulp(x: torch.Tensor) -> torch.Tensor:
    """Size of one bf16 step at |x| (8 significand bits), floor at the
    smallest normal exponent; same metric as reference
    tests/kernel_test_utils.py:304-307."""
    ax = x.abs().float().clamp(min=2.0 ** -126)
    return (2.0 ** (torch.floor(torch.log2(ax)) - 7)).clamp(min=2.0 ** -133)
