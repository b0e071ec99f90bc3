"""mep_build_dedup_static -- the entry point that allocates nothing -- against
mep_build_dedup on the same inputs, through the C ABI.  Integer work:
bit-exact.  Two calls in a row, the second with a smaller input, so that what
the first call left in the library's fixed scratch cannot leak into the second."""

import numpy as np
import pytest
import torch

from moonep_amd import _lib, routing
from oracle import planner_oracle as po
from tests.util import oracle_world_plan

pytestmark = pytest.mark.gpu


def _both(cuda, R, S, K, E, tp, sigma, seed):
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, sigma, seed=seed) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E)
    gp, _, dst_all = oracle_world_plan(topk.numpy(), tpe.numpy(), tp)
    NvS = gp.NvS
    lib = _lib.lib()
    d_dst = torch.from_numpy(dst_all).to(cuda)
    nbytes = lib.mep_dedup_scratch_bytes(S, R)
    work = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
    st = _lib.current_stream()
    for rank in range(R):
        print(f"dedup static vs scratch: R={R} S={S} K={K} E={E} rank={rank}", flush=True)
        outs = []
        for static in (False, True):
            # poison, so that an entry the builder fails to write shows
            dg = torch.full((NvS, 3), -7, dtype=torch.int32, device=cuda)
            dl = torch.full((NvS,), -7, dtype=torch.int32, device=cuda)
            dc = torch.full((2,), -7, dtype=torch.int32, device=cuda)
            if static:
                rc = lib.mep_build_dedup_static(d_dst.data_ptr(), rank, S, K, R, NvS, dg.data_ptr(),
                                                dl.data_ptr(), dc.data_ptr(), st)
            else:
                rc = lib.mep_build_dedup(d_dst.data_ptr(), rank, S, K, R, NvS, dg.data_ptr(),
                                         dl.data_ptr(), dc.data_ptr(), work.data_ptr(), nbytes, st)
            assert rc == 0, lib.mep_strerror(rc)
            torch.cuda.synchronize()
            outs.append((dg.cpu().numpy(), dl.cpu().numpy(), dc.cpu().numpy()))
        (g0, l0, c0), (g1, l1, c1) = outs
        assert np.array_equal(c0, c1)
        assert np.array_equal(g0, g1) and np.array_equal(l0, l1)      # poison included
        # and both equal the oracle's deterministic order
        og, ol, oc = po.dedup_structs(dst_all, rank, S, K, NvS)
        ng, nd = int(c1[0]), int(c1[1])
        assert [ng, nd] == list(oc)
        assert np.array_equal(g1[:ng], og[:ng]) and np.array_equal(l1[:nd], ol[:nd])
    return ng


def test_static_scratch_dedup_matches_scratch_argument_variant(cuda):
    # duplicate-heavy routing (few experts per rank), then a smaller input
    _both(cuda, R=4, S=512, K=8, E=16, tp=16, sigma=1.0, seed=3)
    _both(cuda, R=2, S=96, K=4, E=8, tp=8, sigma=0.5, seed=4)
