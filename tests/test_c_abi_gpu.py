"""Runs tests/c_abi/gpu_check: a program without Python or PyTorch that drives the C ABI from C++ (hipMalloc, its own
stream, a plain host array of chunk descriptors) and compares every result bit for bit with the CPU restatement of the
reference operator, host-decided and device-decided steps alike.  The binary is built on the CPU beforehand
(make -C tests/c_abi, also done by __graft_entry__.build())."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "c_abi", "gpu_check")


@pytest.mark.gpu
def test_c_program_drives_the_abi_on_the_gpu():
    if not os.path.exists(EXE):
        subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "c_abi")])
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "c abi gpu check ok" in r.stdout, (r.returncode, r.stdout[-2000:], r.stderr[-2000:])
