"""The C ABI driven from plain C++ (tests/host/cabi_roundtrip.cpp): hipMalloc'd
buffers, no Python and no torch in the calling process.  The program checks
every entry point against the scalar C checker and exits non-zero on any
difference.  It is built beforehand (`make -C tests/host`, also done by
__graft_entry__.build())."""

import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "host", "cabi_roundtrip")


def test_cabi_roundtrip_from_plain_cpp(cuda):
    assert os.path.exists(EXE), f"{EXE} is missing: run `make -C tests/host`"
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(res.stdout, flush=True)
    print(res.stderr, flush=True)
    assert res.returncode == 0, res.stdout[-2000:]
    assert "ALL OK" in res.stdout
