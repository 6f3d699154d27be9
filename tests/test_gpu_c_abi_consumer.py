"""The C ABI used from a plain C program (``tests/c_abi/consumer.c``, built by ``__graft_entry__.build()``): device
buffers from the HIP runtime, ``include/siirl_hip.h`` and the shared library -- no Python, no torch in the process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "consumer")


def test_plain_c_program_drives_the_library():
    if not os.path.exists(BIN):  # normally prebuilt; a sub-second gcc run of one C file otherwise
        import __graft_entry__ as entry

        try:
            entry.build_c_consumer()
        except Exception as e:  # no compiler on this machine: nothing to run
            pytest.skip(f"tests/c_abi/consumer is not built and cannot be built here: {e}")
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("OK"), r.stdout
