"""The host library (cache bookkeeping and scheduler, C++) under the address and
undefined-behaviour sanitizers: its sources are built together with ``csrc/host/selftest.cpp``
into one program (the sanitizer runtimes linked in statically, so nothing has to be preloaded)
that drives the C entry points through random request lifetimes, windowed groups, truncation
and scheduler runs with cancelled and failed requests."""

import subprocess

import pytest


def test_host_library_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    from flyweight_amd.kernels import build
    try:
        program = build.build_host_selftest(str(tmp_path))
    except RuntimeError as error:
        if "asan" in str(error).lower() or "ubsan" in str(error).lower() or "sanitize" in str(error).lower():
            pytest.skip(f"this compiler has no static sanitizer runtimes: {str(error).splitlines()[-1]}")
        raise
    result = subprocess.run([program], capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr[-4000:]
    assert "selftest: ok" in result.stdout
    assert "runtime error" not in result.stderr and "Sanitizer" not in result.stderr, result.stderr[-4000:]
