"""The C-ABI library loads without a GPU and exports every symbol that
include/moonep_hip.h declares; host-side argument validation returns error
codes without touching a device."""

import ctypes
import os
import re

from moonep_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "moonep_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mep_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert _declared() == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name


def test_version_and_error_strings():
    lib = _lib.lib()
    assert lib.mep_version() >= 100
    assert lib.mep_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert len(lib.mep_strerror(code)) > 3


def test_argument_validation_needs_no_device():
    lib = _lib.lib()
    # null pointers / bad sizes are rejected before any launch
    assert lib.mep_plan(None, None, 0, 4, 2, 8, 2, 8, 64, None, None, None, None, None, None, 0, None) == -1
    assert lib.mep_dispatch(None, None, None, None, None, 0, None, 0, 0, 4, 64, 2, 2, 4, 64, 8, 0, None) == -1
    assert lib.mep_combine(None, 0, None, 0, None, None, None, 4, 64, 2, 2, 64, 0, None) == -1
    assert lib.mep_grad_reduce(None, None, 0, None, 0, 4, 2, 16, 0, None) == -1
    assert lib.mep_plan_scratch_bytes(4096, 8, 256, 8, 1) == 0          # tables fit in LDS
    assert lib.mep_plan_scratch_bytes(256, 1, 2050, 2, 2) > 0           # they do not
    assert lib.mep_dedup_scratch_bytes(4096, 8) >= 4096 * 8 * 4


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    try:
        _lib.lib()
    except RuntimeError as e:
        assert "no CPU or eager fallback" in str(e)
    else:
        raise AssertionError("expected RuntimeError")


def test_error_codes_for_unsupported_shapes_alignment_and_scratch():
    """Specific MEP_ERR_* codes; every check sits before the launch, so fake
    (never dereferenced) device addresses are enough and no GPU is needed."""
    lib = _lib.lib()
    A = 0x10000          # 16-byte aligned stand-in for a device pointer
    ok_plan = dict(S=4, K=2, E=8, R=2, tp=8, NvS=64)

    def plan(**kw):
        a = dict(ok_plan, scratch=None, sbytes=0)
        a.update(kw)
        return lib.mep_plan(A, A, 0, a["S"], a["K"], a["E"], a["R"], a["tp"], a["NvS"], A, A, A, A, A,
                            a["scratch"], a["sbytes"], None)

    assert plan(K=33) == -2                      # more than 32 routes per token
    assert plan(R=3) == -1                       # E not divisible by R
    assert plan(NvS=4) == -2                     # NvS below S*K
    assert plan(R=2, NvS=1 << 30) == -2          # R*NvS does not fit the int32 encoding
    assert plan(E=2050, S=256, K=1, NvS=1024) == -3        # planner tables need caller scratch
    assert plan(E=2050, S=256, K=1, NvS=1024, scratch=A + 4, sbytes=1 << 30) == -4   # misaligned scratch
    assert plan(E=1 << 16, R=2, S=256, K=1, NvS=1024, scratch=A, sbytes=1 << 40) == -2  # beyond the LDS limit
    assert plan(E=5816, R=8, S=256, K=1, NvS=1024, scratch=A, sbytes=1 << 40) == -2     # one step beyond it (E = 5808 fills the 160 KB)
    assert lib.mep_plan_warm(A, A, 0, 4, 2, 8, 2, 8, 64, A, A, A, A, A, None, 0, A + 4, 64, None) == -4  # misaligned warm range
    # dispatch / combine: misaligned rows, weights without slots, bad mode, ragged H
    assert lib.mep_dispatch(A + 2, None, A, A, A, 64, None, 0, 0, 4, 64, 2, 2, 4, 64, 8, 0, None) == -4
    assert lib.mep_dispatch(A, A, A, A, A, 64, None, 0, 0, 4, 64, 2, 2, 4, 64, 8, 0, None) == -1
    assert lib.mep_dispatch(A, None, A, A, A, 64, None, 0, 5, 4, 64, 2, 2, 4, 64, 8, 0, None) == -1  # rank >= R
    assert lib.mep_combine(A, 64, None, 0, A, A, None, 4, 64, 2, 2, 64, 7, None) == -1     # unknown mode
    assert lib.mep_combine(A, 64, None, 0, A, A, None, 4, 64, 2, 2, 64, 3, None) == -1     # weighted without slots
    assert lib.mep_combine(A, 64, None, 0, A, A, None, 4, 60, 2, 2, 64, 0, None) == -2     # H % 8 != 0
    assert lib.mep_combine(A, 64, None, 0, A, A, None, 4, 64, 33, 2, 64, 0, None) == -2    # K > 32
    assert lib.mep_combine(A, 32, None, 0, A, A, None, 4, 64, 2, 2, 64, 0, None) == -1     # stride < NvS
    assert lib.mep_grad_reduce(A, A, 16 * 4, A, 0, 4, 2, 18, 0, None) == -2                   # elems % 4 != 0
    assert lib.mep_grad_reduce(A, A, 8, A, 0, 4, 2, 16, 0, None) == -1                      # stride too small
    assert lib.mep_grad_reduce(A + 4, A, 64, A, 0, 4, 2, 16, 0, None) == -4
    assert lib.mep_grad_reduce(A, A, 64, A, 0, 4, 2, 16, 3, None) == -1                        # both phase flags at once
    # grouped GEMM: tile multiples, swiglu needs the up weights and no row scale
    assert lib.mep_grouped_gemm_nt(A, A, None, A, 4, A, None, 100, 256, 64, 0, None) == -2
    assert lib.mep_grouped_gemm_nt(A, A, None, A, 4, A, None, 128, 128, 64, 0, None) == -2
    assert lib.mep_grouped_gemm_nt(A, A, None, A, 4, A, None, 128, 256, 32, 0, None) == -2
    assert lib.mep_grouped_gemm_nt(A, A, None, A, 4, A, None, 128, 128, 64, 1, None) == -1
    assert lib.mep_grouped_gemm_nt(A, A, A, A, 4, A, A, 128, 128, 64, 1, None) == -1
    assert lib.mep_grouped_gemm_nt(A + 8, A, None, A, 4, A, None, 128, 256, 64, 0, None) == -4
    # the backward pieces
    assert lib.mep_grouped_swiglu_nt(A, A, None, A, 4, A, A, A, 128, 128, 64, None) == -1   # no up weights
    assert lib.mep_grouped_swiglu_nt(A, A, A, A, 4, A, A, A, 128, 192, 64, None) == -2      # N % 128 != 0
    assert lib.mep_grouped_gemm_dual_nt(A, A, None, A, A, 4, A, 128, 256, 64, None) == -1   # second pair missing
    assert lib.mep_grouped_gemm_dual_nt(A, A, A, A, A, 4, A, 128, 128, 64, None) == -2      # N % 256 != 0
    assert lib.mep_grouped_gemm_dual_nt(A, A, A + 2, A, A, 4, A, 128, 256, 64, None) == -4
    assert lib.mep_grouped_gemm_nn(A, None, A, 4, A, None, 128, 256, 64, None) == -1        # weights missing
    assert lib.mep_grouped_gemm_nn(A, A, A, 4, A, None, 128, 256, 96, None) == -2           # K % 64 != 0
    assert lib.mep_grouped_gemm_nn(A, A + 2, A, 4, A, None, 128, 256, 64, None) == -4
    assert lib.mep_grouped_gemm_dual_nn(A, A, None, A, A, 4, A, 128, 256, 64, None) == -1   # second pair missing
    assert lib.mep_grouped_gemm_dual_nn(A, A, A, A, A, 4, A, 128, 128, 64, None) == -2      # N % 256 != 0
    assert lib.mep_grouped_gemm_wgrad(A, A, A, 4, A, 100, 256, 1024, 4, None) == -2            # Ma % 128 != 0
    assert lib.mep_grouped_gemm_wgrad(A, A, A, 4, A, 128, 256, 1000, 4, None) == -2            # ld % 128 != 0
    assert lib.mep_grouped_gemm_wgrad(A, None, A, 4, A, 128, 256, 1024, 4, None) == -1
    assert lib.mep_grouped_gemm_wgrad_tn(A, A, A, 4, A, 128, 256, 1024, 4, None) == -2         # Ma % 256 != 0
    assert lib.mep_grouped_gemm_wgrad_tn(A, A, A, 3, A, 256, 256, 1024, 3, None) == -2         # G odd
    assert lib.mep_grouped_gemm_wgrad_tn(A, A, None, 4, A, 256, 256, 1024, 4, None) == -1
    assert lib.mep_transpose_bf16(A, A, 1, 64, 64, None) == -1                              # in place
    assert lib.mep_transpose_bf16(A, A + 8192, 1, 64, 96, None) == -2                       # cols % 64 != 0
    assert lib.mep_swiglu_bwd(A, A, A, None, A, 4, A, A, A, None, 128, 100, None) == -2     # N % 8 != 0
    assert lib.mep_swiglu_bwd(A, A, None, None, A, 4, A, A, A, None, 128, 128, None) == -1


def test_argument_checks_of_the_entry_points_added_with_abi_200():
    import ctypes as C

    lib = _lib.lib()
    A = 0x10000
    assert lib.mep_version() == _lib.ABI_VERSION == 200
    # pull prefetch: host arrays of pointers / strides / sizes
    arr_p, arr_i = (C.c_void_p * 3), (C.c_int64 * 3)
    ok = dict(owners=arr_p(A, A, A), ostride=arr_i(4096, 4096, 4096), pool=arr_p(A, A, A),
              pstride=arr_i(4096, 4096, 4096), per=arr_i(1024, 1024, 1024))

    def pull(n=3, rank=0, epn=4, R=2, etc=A, **kw):
        a = dict(ok, **kw)
        return lib.mep_prefetch_pull(n, a["owners"], a["ostride"], a["pool"], a["pstride"], a["per"], etc,
                                     rank, epn, R, None)

    assert pull(etc=None) == -1
    assert pull(n=7) == -1                                   # more than six tensors
    assert pull(rank=2) == -1                                # rank outside [0, R)
    assert pull(per=arr_i(1024, 1000, 1024)) == -2           # bytes per expert not a multiple of 16
    assert pull(ostride=arr_i(4096, 2048, 4096)) == -1       # owners' experts would overlap
    assert pull(pool=arr_p(A, A + 8, A)) == -4               # misaligned pool
    assert pull(owners=arr_p(A, None, A)) == -1
    # duplicate kernels: the CU bound is an ordinary int; the usual checks come first
    assert lib.mep_dispatch_epilogue(None, A, A, A, 64, 64, 32, None) == -1
    assert lib.mep_combine_prologue(A, A, A, A, 64, 60, 0, None) == -2        # H % 8 != 0
    assert lib.mep_combine_prologue(A + 2, A, A, A, 64, 64, 1, None) == -4
    # the GEMM tiling hook takes 0, 128 or 256
    assert lib.mep_set_gemm_row_tile(7) == -1 and lib.mep_set_gemm_row_tile(256) == 0
    assert lib.mep_set_gemm_row_tile(0) == 0
    # the dst encoding bound is checked by every consumer of dst, not only by the planner
    assert lib.mep_dispatch(A, None, A, A, A, 1 << 30, None, 0, 0, 4, 64, 2, 2, 4, 1 << 30, 8, 0, None) == -2
    assert lib.mep_combine(A, 1 << 30, None, 0, A, A, None, 4, 64, 2, 2, 1 << 30, 0, None) == -2


def test_static_scratch_entry_point_rejects_inputs_beyond_its_fixed_size():
    """mep_build_dedup_static allocates nothing: its scratch is a fixed 1 MiB device
    array; a larger input is refused with its own error code before any device call."""
    lib = _lib.lib()
    A = 0x10000
    assert lib.mep_dedup_scratch_bytes(4096, 8) <= (1 << 20)     # the headline shape fits
    assert lib.mep_dedup_scratch_bytes(37500, 8) > (1 << 20)     # 300 000 tokens do not
    assert lib.mep_build_dedup_static(A, 0, 37500, 8, 8, 37500 * 8 + 8192, A, A, A, None) == -5
    assert lib.mep_build_dedup_static(None, 0, 64, 8, 8, 1024, A, A, A, None) == -1
    assert b"fixed scratch" in lib.mep_strerror(-5)
