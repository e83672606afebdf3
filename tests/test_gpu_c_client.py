"""The C ABI without Python in between: a plain HIP/C++ program
(oslo_amd/csrc/c_abi_client.cpp, built by the library's Makefile) allocates with
hipMalloc, calls oslo_ln_fwd / oslo_ln_bwd / oslo_softmax_causal_fwd on its own
stream and checks the results against double-precision loops of its own."""
import os
import subprocess

import pytest

from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

CLIENT = os.path.join(os.path.dirname(_C.LIBRARY_PATH), "c_abi_client")


def test_c_client_runs_the_library_without_torch():
    assert os.path.exists(CLIENT), "build it with `make -C oslo_amd/csrc` (build() does)"
    proc = subprocess.run([CLIENT], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout[-2000:]
    assert "c_abi_client: ok" in proc.stdout
    assert "gfx950" in proc.stdout
