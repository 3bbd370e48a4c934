"""The library driven by a host written in C (tests/cpp/abi_host.c): four hipMalloc'ed rank buffers, the ring
collectives in both forms, the single-launch all-reduce, AdamW on a float64 shard (against the same operations in C
doubles) and the refusals, through include/tandem_hip.h alone.
The program is built beforehand (__graft_entry__.build(), or `make -C tests/cpp`); only if it is missing
is it built here. Run with -m gpu."""

import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "_build", "abi_host")


def test_a_c_program_drives_the_library():
    if not os.path.exists(EXE):
        subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp")], check=True)
    res = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0, res.stdout[-2000:]
    assert "abi_host: ok" in res.stdout
