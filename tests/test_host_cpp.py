"""The C++ host mirror (rustingbrain_amd/host/rusting_brain_moe.hpp) through its
driver program: configuration, accounting and error paths on the CPU, and the
tutorial scenario plus the reference's unit-test expectations on the GPU."""
import os
import subprocess

import pytest

from conftest import ROOT

BIN = os.path.join(ROOT, "rustingbrain_amd", "host", "moe_tutorial")


def run(*args):
    if not os.path.exists(BIN):
        from rustingbrain_amd import build
        build.build_host()
    return subprocess.run([BIN, *args], capture_output=True, text=True, timeout=120)


def test_cpp_host_configuration_and_error_paths():
    res = run("--cpu-checks")
    assert res.returncode == 0, res.stdout + res.stderr
    assert "all checks passed" in res.stdout
    # the parameter table of reference tutorials/15_mixture_of_experts.md:276-283
    for line in ("1   32.5M    32.5M    1.00x", "8   55.2M    35.7M    1.54x", "32  133.1M    35.8M    3.72x"):
        assert line in res.stdout


@pytest.mark.gpu
def test_cpp_host_drives_the_layer_like_the_tutorial():
    res = run()
    assert res.returncode == 0, res.stdout + res.stderr
    assert "all checks passed" in res.stdout
    assert "identical tokens, collapsed routing:" in res.stdout and "dead experts 6/8" in res.stdout
