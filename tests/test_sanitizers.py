"""Sanitizer builds of the host code (GPU AddressSanitizer is not available on the test machines; host code is what
these cover).  `make -C oracle asan-oracle` compiles the CPU oracle with its driver under AddressSanitizer + UBSan and
runs it; `make -C oracle asan-abi` compiles the HOST side of every engine source under the same sanitizers and runs the
C client of the ABI (blob parsing, shape inference, error paths, no GPU call) against that build.  The second takes
about a minute of compilation on 8 cores, so it runs only when D3D_ASAN_ENGINE=1 is set."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _make(target, timeout):
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-j8", target], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=timeout)
    assert res.returncode == 0, res.stdout[-4000:]
    return res.stdout


def test_oracle_under_asan_and_ubsan():
    out = _make("asan-oracle", 300)
    assert "asan_check: ok" in out


@pytest.mark.skipif(os.environ.get("D3D_ASAN_ENGINE") != "1", reason="set D3D_ASAN_ENGINE=1: compiles every engine "
                    "source with host sanitizers (about a minute)")
def test_engine_host_code_under_asan_and_ubsan():
    out = _make("asan-abi", 1500)
    assert "abi_check ok" in out
