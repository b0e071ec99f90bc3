"""Host-side behaviour of the public API that needs no GPU: argument
validation order and messages (the reference pins these in
tests/test_api_validation.py and the bad-input tests of test_dispatch.py /
test_combine.py), shape arithmetic, the plan container."""

import pytest
import torch

import moonep_amd
from moonep_amd import Buffer, MoonEPCommPlan, api, routing
from moonep_amd.planning import _check_dedup_encoding_bounds


def test_num_sms_is_validated_before_any_device_access(monkeypatch):
    def boom(*a, **k):
        raise AssertionError("device was touched before num_sms validation")

    monkeypatch.setattr(torch.cuda, "current_device", boom)
    with pytest.raises(TypeError, match="num_sms must be a positive int, got str"):
        Buffer(4, 16, 2, 8, 2, num_sms="8")
    with pytest.raises(TypeError, match="got bool"):
        Buffer(4, 16, 2, 8, 2, num_sms=True)
    with pytest.raises(ValueError, match="num_sms must be a positive int, got 0"):
        Buffer(4, 16, 2, 8, 2, num_sms=0)
    with pytest.raises(ValueError, match="got -3"):
        Buffer(4, 16, 2, 8, 2, num_sms=-3)


def test_num_sms_above_device_count(monkeypatch):
    class Props:
        multi_processor_count = 256

    monkeypatch.setattr(torch.cuda, "current_device", lambda: 0)
    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda d: Props())
    with pytest.raises(ValueError, match=r"num_sms \(257\) must not exceed the device SM count \(256\)"):
        Buffer(4, 16, 2, 8, 2, num_sms=257)


def test_constructor_type_checks():
    with pytest.raises(AssertionError, match="comm_stream_priority must be an int"):
        Buffer(4, 16, 2, 8, 2, comm_stream_priority="high")
    with pytest.raises(AssertionError, match="enable_pdl must be a bool"):
        Buffer(4, 16, 2, 8, 2, enable_pdl=1)
    with pytest.raises(TypeError):
        Buffer(4, 16, 2, 8, 2, bogus=1)


def test_env_override_of_dedup_sms(monkeypatch):
    monkeypatch.setenv("MOONEP_NUM_SMS_DEDUP", "abc")
    with pytest.raises(ValueError, match="MOONEP_NUM_SMS_DEDUP must be an integer"):
        api._num_sms_dedup_from_env(64)
    monkeypatch.setenv("MOONEP_NUM_SMS_DEDUP", "65")
    with pytest.raises(ValueError, match=r"must be in \[1, 64\]"):
        api._num_sms_dedup_from_env(64)
    monkeypatch.setenv("MOONEP_NUM_SMS_DEDUP", "8")
    assert api._num_sms_dedup_from_env(64) == 8
    monkeypatch.delenv("MOONEP_NUM_SMS_DEDUP")
    assert api._num_sms_dedup_from_env(64) == 64


def test_meta_layout_matches_reference_arithmetic():
    # reference moonep/api.py:298-324 and tests/kernel_test_utils.py:339-367
    S, K, E, R, tp = 4096, 8, 256, 8, 128
    epn = E // R
    NvS = (S * K + (tp - 1) * 2 * epn + tp - 1) // tp * tp
    assert NvS == 40960
    lay = api.meta_layout(S, K, E, R, NvS)
    N = S * K
    plan_out = 3 * E * R + R * 2 * epn + 2 * R * 2 * epn + R * epn + 2 * R
    assert lay["TPE_OFF"] == NvS and lay["PLAN_OFF"] == NvS + R * E
    assert lay["TOPK0_OFF"] == (lay["PLAN_OFF"] + plan_out + 3) // 4 * 4
    assert lay["ORDER_OFF"] == lay["TOPK0_OFF"] + N
    assert lay["ORDER0_OFF"] == lay["ORDER_OFF"] + N
    assert lay["BARRIER_OFF"] == lay["ORDER0_OFF"] + N
    assert lay["SRC_INFO_OFF"] == lay["BARRIER_OFF"] + 3
    assert lay["meta_chunk_padded"] >= lay["SRC_INFO_OFF"] + NvS
    # second headline shape
    assert (8192 * 8 + 127 * 2 * 16 + 127) // 128 * 128 == 69632


def _plan(N=8, R=2, E=4, NvS=16, K=2, **over):
    epn = E // R
    i32 = torch.int32
    f = dict(dst=torch.zeros(N, dtype=i32), experts_to_copy=torch.zeros(R, epn, dtype=i32),
             zero_fill_ranges=torch.zeros(2 * epn, 2, dtype=i32), remote_stats=torch.zeros(2, dtype=i32),
             dup_groups=torch.zeros(NvS, 3, dtype=i32), dup_loffs=torch.zeros(NvS, dtype=i32),
             dup_counts=torch.zeros(2, dtype=i32), N=N, R=R, E=E, NvS=NvS, K=K)
    f.update(over)
    return MoonEPCommPlan(**f)


def test_plan_container_checks_and_clone():
    p = _plan()
    q = p.clone()
    assert q is not p and torch.equal(q.dst, p.dst) and q.dst.data_ptr() != p.dst.data_ptr()
    assert (q.N, q.R, q.E, q.NvS, q.K) == (p.N, p.R, p.E, p.NvS, p.K)
    with pytest.raises(AssertionError):
        _plan(dst=torch.zeros(8, dtype=torch.int64))
    with pytest.raises(AssertionError):
        _plan(dst=torch.zeros(7, dtype=torch.int32))
    with pytest.raises(AssertionError):
        _plan(dup_groups=torch.zeros(16, 2, dtype=torch.int32))
    with pytest.raises(AssertionError):
        _plan(zero_fill_ranges=torch.zeros(4, 2, dtype=torch.int32).t())
    with pytest.raises(Exception):
        p.N = 3  # frozen


def test_encoding_bounds():
    ok = dict(R=8, S=4096, K=8, NvS=40960)
    _check_dedup_encoding_bounds(ok)
    with pytest.raises(AssertionError, match="K <= 32"):
        _check_dedup_encoding_bounds(dict(ok, K=33, NvS=4096 * 33 + 128))
    with pytest.raises(AssertionError, match="R <= 128"):
        _check_dedup_encoding_bounds(dict(ok, R=129))
    with pytest.raises(AssertionError, match="S\\*K <= NvS"):
        _check_dedup_encoding_bounds(dict(ok, NvS=100))
    with pytest.raises(AssertionError, match="NvS must be <="):
        _check_dedup_encoding_bounds(dict(ok, S=3_000_000, NvS=24_000_128))


def test_package_surface():
    assert moonep_amd.__all__ == ["Buffer", "MoonEPCommPlan", "EmulatedWorld"]
    for name in ("dispatch", "combine", "prefetch_weight", "reduce_grad", "destroy", "destroyed",
                 "hidden_nvsh_buffer_view", "router_weight_buffer_view", "_require_ctx"):
        assert hasattr(Buffer, name)


def test_routing_generators():
    S, K, E, R = 64, 4, 32, 8
    rr = torch.stack([routing.round_robin(S, K, E, R, r, seed=1) for r in range(R)])
    tpe = routing.tokens_per_expert(rr, E)
    assert tpe.shape == (R, E) and int(tpe.sum()) == R * S * K
    assert (tpe.sum(0).reshape(R, E // R).sum(1) == S * K).all()
    assert routing.maxvio(tpe) == pytest.approx(0.0, abs=1e-9) or routing.maxvio(tpe) < 0.2
    topk, w, tpe, mv, sigma = routing.logit_routing(256, 8, 64, 8, 1.0, seed=3)
    assert topk.shape == (8, 256, 8) and topk.dtype == torch.int32
    assert abs(mv - 1.0) < 0.1 and sigma > 0
    assert torch.allclose(w.sum(-1), torch.ones(8, 256))
    # top-k without replacement
    assert (topk.sort(-1).values.diff(dim=-1) != 0).all()
    topk2, *_ = routing.logit_routing(256, 8, 64, 8, 1.0, seed=3)
    assert torch.equal(topk, topk2)
    assert routing.pattern("duplicate_topk", 4, 3, 8, 4, 1).unique().tolist() == [4]


def test_grouped_gemm_rejects_paddings_that_split_a_tile():
    """The grouped GEMM gives every 128-row tile to one group: a plan made with a
    smaller token_padding is refused on the host, before any tensor is looked at."""
    from moonep_amd.ffn import grouped_ffn_hip, launch_grouped_gemm_nt
    x = torch.zeros(128, 64, dtype=torch.bfloat16)
    for tp in (16, 64, 192, 0):
        with pytest.raises(AssertionError, match="multiple of 128"):
            launch_grouped_gemm_nt(x, x, x, token_padding=tp)
        with pytest.raises(AssertionError, match="multiple of 128"):
            grouped_ffn_hip(x, None, x, x, x, x, token_padding=tp)


def test_the_reference_import_name_resolves_to_this_package():
    """``from moonep import Buffer, MoonEPCommPlan`` (reference moonep/__init__.py:1-9) and the
    reference's module paths of the launchers work unchanged."""
    import moonep
    from moonep import Buffer as B2, MoonEPCommPlan as P2
    from moonep.combine_prologue import launch_combine_prologue
    from moonep.dispatch_epilogue import launch_dispatch_epilogue
    from moonep.planning import launch_planning
    import moonep.api

    assert B2 is Buffer and P2 is MoonEPCommPlan
    assert moonep.api is api and moonep.__all__ == ["Buffer", "MoonEPCommPlan"]
    assert launch_dispatch_epilogue.__module__ == "moonep_amd.dispatch"
    assert launch_combine_prologue.__module__ == "moonep_amd.combine"
    assert launch_planning.__module__ == "moonep_amd.planning"


def test_per_rank_counts_need_rank_threads():
    """A one-rank tokens_per_expert[E] reaches the planner only through the gathered table,
    which nobody fills without rank threads: refused before any device access."""
    from moonep_amd.planning import _tpe_table

    class World:
        host_threads = False

    ctx = dict(R=4, E=8, rank=1, world=World())
    with pytest.raises(NotImplementedError, match=r"tokens_per_expert\[R=4, E=8\]"):
        _tpe_table(ctx, torch.zeros(8, dtype=torch.int32))
    table = torch.zeros(4, 8, dtype=torch.int32)
    assert _tpe_table(ctx, table) is table


def test_reduce_grad_phase_argument_and_pool_checks_are_host_side():
    """Shape / dtype / stride checks of the (local, pool) pairs in own words; the messages the
    reference's tests match by substring are kept."""
    local = torch.zeros(2, 4, 4)
    pool = torch.zeros(3, 2, 4, 4)
    with pytest.raises(AssertionError, match="unsupported weight dtype"):
        api._check_local_pool_pairs("prefetch_weight", [local], [pool], 2, 3, dtypes=(torch.bfloat16,))
    with pytest.raises(AssertionError, match=r"must be \[epn=5"):
        api._check_local_pool_pairs("reduce_grad", [local], [pool], 5, 3, dtypes=(torch.float32,))
    with pytest.raises(AssertionError, match=r"pool must be \[R=4, epn=2"):
        api._check_local_pool_pairs("reduce_grad", [local], [pool], 2, 4, dtypes=(torch.float32,))
    with pytest.raises(AssertionError, match="3 dimensions"):
        api._check_local_pool_pairs("reduce_grad", [local[0]], [pool[:, 0]], 4, 3, dtypes=(torch.float32,))
