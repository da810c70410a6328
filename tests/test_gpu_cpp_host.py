"""GPU: the compiled C++ host side above the C ABI (include/dt_hip.hpp driven by csrc/dt_cpp_check.cpp)."""
import pytest

pytestmark = pytest.mark.gpu


def test_compiled_host_program_over_the_c_abi(dthip):
    """The C++ operator mirror (include/dt_hip.hpp) driven by a compiled program, with no Python or torch between it
    and the library: Dense over a plain and a q8p weight against the identity (bit-exact), RMSNorm on a constant row,
    two-segment attention with constant V, and the error paths.  The program is built next to the library."""
    import os
    import subprocess

    exe = os.path.join(os.path.dirname(dthip.LIB_PATH), "dt_cpp_check")
    assert os.path.exists(exe), f"{exe} is missing: build it with `make -C {dthip.CSRC}`"
    print("compiled host program", flush=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "dt_cpp_check ok" in res.stdout
