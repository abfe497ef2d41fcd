"""Runs the C++ tests of the host-side layer (tests/cpp) on the GPU.

The binaries are built beforehand by __graft_entry__.build() (make -C tests/cpp);
each returns 0 when every check passed.  Each runs in a process of its own beside
this one; the file is named to be collected after the in-process GPU tests."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BUILD = os.path.join(HERE, "cpp", "build")


@pytest.mark.parametrize("name", ["test_halo_exchange_virtual", "test_shuffle_virtual",
                                  "test_batchnorm_softmax", "test_h2_frontend", "test_algorithms"])
def test_cpp(name):
    exe = os.path.join(BUILD, name)
    assert os.path.exists(exe), f"{exe} is missing: run `make -C tests/cpp`"
    print("running", exe, flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(r.stdout[-2000:], r.stderr[-2000:])
    assert r.returncode == 0, f"exit status {r.returncode}\n" + r.stdout[-2000:] + r.stderr[-2000:]
