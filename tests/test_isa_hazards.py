"""The streaming kernel waits for its inline-assembly loads by hand; this compiles it to
assembly with the library's own flags and checks, over every path of every instantiation,
that no instruction touches a register whose load can still be outstanding."""
import os
import shutil
import subprocess
import tempfile

import pytest

import isa_check
from rustingbrain_amd import build as rb_build

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "..", "rustingbrain_amd", "csrc", "grouped_stream.hip")


def test_checker_flags_a_use_before_the_wait():
    asm = "\n".join(["_Zk:", "\tglobal_load_dwordx4 v[4:7], v1, s[0:1]", "\tglobal_load_dwordx4 v[8:11], v1, s[2:3]",
                     "\ts_waitcnt vmcnt(1)", "\tv_add_u32_e32 v0, v4, v5", "\tv_mov_b32_e32 v2, v9",
                     "\ts_waitcnt vmcnt(0)", "\tv_mov_b32_e32 v3, v9", "\ts_endpgm", ".Lfunc_end0:"])
    res = isa_check.check_asm(asm)["_Zk"]
    assert len(res) == 1 and "v_mov_b32_e32 v2, v9" in res[0]


def test_checker_follows_loops():
    asm = "\n".join(["_Zk:", ".LBB0_1:", "\tv_mov_b32_e32 v2, v9", "\tglobal_load_dwordx4 v[8:11], v1, s[2:3]",
                     "\ts_cbranch_scc1 .LBB0_1", "\ts_waitcnt vmcnt(0)", "\ts_endpgm", ".Lfunc_end0:"])
    res = isa_check.check_asm(asm)["_Zk"]
    assert any("v_mov_b32_e32 v2, v9" in h for h in res)


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_streaming_kernel_has_no_use_of_outstanding_loads():
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "grouped_stream.s")
        cmd = [rb_build.HIPCC] + [f for f in rb_build.FLAGS if f != "-fPIC"] + ["-S", "--cuda-device-only", "-o", out, SRC]
        subprocess.run(cmd, check=True, capture_output=True)
        res = isa_check.check_asm(open(out).read(), "grouped_stream_kernel")
    assert len(res) >= 4, "expected every instantiation of the kernel in the assembly"
    bad = {k: v[:5] for k, v in res.items() if v}
    assert not bad, bad


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_static_scratch_array_is_a_symbol_the_runtime_can_look_up():
    # rbmoe_forward_static's scratch is a static device array whose address the host asks the runtime for by name
    # (hipGetSymbolAddress).  The runtime searches the code object's global symbols, and a missing one ends the
    # process rather than returning an error - so the array must come out of the device compilation as a global
    # object of the declared size, not as a local one.
    src = os.path.join(HERE, "..", "rustingbrain_amd", "csrc", "rbmoe_api.hip")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "rbmoe_api.s")
        cmd = [rb_build.HIPCC] + [f for f in rb_build.FLAGS if f != "-fPIC"] + ["-S", "--cuda-device-only", "-o", out, src]
        subprocess.run(cmd, check=True, capture_output=True)
        lines = [ln.strip() for ln in open(out) if "rbmoe_static_scratch" in ln]
    name = next(ln.split()[1].split(",")[0] for ln in lines if ln.startswith(".type"))
    assert f".globl {name}" in [" ".join(ln.split()) for ln in lines], lines
    assert not any(ln.startswith(".local") for ln in lines), lines
    assert any(ln.startswith(".size") and ln.endswith(str(8 << 20)) for ln in lines), lines
