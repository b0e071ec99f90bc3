"""Buffer(num_sms=N): every kernel of the Buffer runs on N compute units (a
CU-masked comm stream), results are the same bits as on the whole GPU."""

import ctypes

import numpy as np
import pytest
import torch

from moonep_amd import Buffer, _lib, routing

pytestmark = pytest.mark.gpu

S, H, K, E, R, TP = 512, 1024, 4, 16, 4, 16


def _distinct_cus(stream_handle, cuda, nblocks=8192):
    out = torch.zeros(nblocks, dtype=torch.int32, device=cuda)
    rc = _lib.lib().mep_stream_cu_census(out.data_ptr(), nblocks, stream_handle)
    assert rc == 0, _lib.lib().mep_strerror(rc)
    torch.cuda.synchronize()
    ids = np.unique(out.cpu().numpy())
    return len(ids), len(np.unique(ids >> 16))


@pytest.mark.parametrize("num_sms", [32, 64])
def test_num_sms_bounds_the_compute_units_and_keeps_the_bits(cuda, num_sms):
    topk = torch.stack([routing.popularity_biased(S, K, E, R, r, 1.0, seed=5) for r in range(R)])
    tpe = routing.tokens_per_expert(topk, E).to(cuda)
    g = torch.Generator().manual_seed(1)
    hidden = torch.randn(S, H, generator=g).to(torch.bfloat16).to(cuda)
    w = torch.rand(S, K, generator=g).to(cuda)
    rank = 1
    results = []
    for n in (None, num_sms):
        buf = Buffer(S, H, K, E, R, num_sms=n, token_padding=TP, rank=rank)
        buf._require_ctx()["hidden_buf"].zero_()
        torch.cuda.synchronize()
        if n is not None:
            cus, xccs = _distinct_cus(buf._comm_stream.cuda_stream, cuda)
            print(f"num_sms={n}: probe kernel ran on {cus} CUs of {xccs} XCDs", flush=True)
            assert cus == n and xccs == 8
        h, wn, cu, plan = buf.dispatch(hidden, w, topk[rank].contiguous().to(cuda), tpe)
        out, w_back, ev = buf.combine(plan=plan, hidden_nvsh=h, route_weights_nvs=wn)
        assert ev is None
        h2, wn2, cu2, plan2, ev2 = buf.dispatch(hidden, w, topk[rank].contiguous().to(cuda), tpe,
                                                async_finish=True)
        ev2.wait(torch.cuda.current_stream())
        assert torch.equal(h2, h) and torch.equal(plan2.dst, plan.dst)
        torch.cuda.synchronize()
        results.append((h.cpu(), wn.cpu(), cu.cpu(), plan.dst.cpu(), out.cpu(), w_back.cpu()))
        buf.destroy()
    for a, b in zip(*results):
        assert torch.equal(a, b)
    whole, _ = _distinct_cus(None, cuda)
    assert whole > num_sms          # the null stream is not bounded


def test_limited_stream_argument_checks():
    lib = _lib.lib()
    h = ctypes.c_void_p()
    assert lib.mep_stream_create_limited(4, None) == -1
    assert lib.mep_stream_destroy(None) == -1
    assert lib.mep_stream_cu_census(None, 4, None) == -1
