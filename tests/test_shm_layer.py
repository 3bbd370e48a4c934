"""The process-rank engine's shared-memory layer (tandem_amd/csrc/engine_shm.h: the
region a rank publishes, the message rings in it, the waiting helpers) on the CPU: a
small C++ program, tests/cpp/shm_test.cpp, built here with g++ against the same header
the engine is built from, once plainly, once with the host's address and
undefined-behaviour sanitizers and once with its data-race sanitizer (the cases that
stay in one process). What the reference tests of its SharedMemory and
Channel classes (tests/test_engine.py:27-178 there), as far as this engine has a
counterpart. No GPU call is made; libamdhip64 is only linked for an error-string
function the common header names."""

import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(HERE, "cpp", "shm_test.cpp")
CASES = [("region_roundtrip",), ("region_two_processes",), ("region_errors",), ("ring_one_process",),
         ("ring_two_processes", "1", "3000"), ("ring_two_processes", "2", "20000"), ("ring_two_processes", "16", "20000"),
         ("ring_two_threads", "1", "3000"), ("ring_two_threads", "2", "20000"), ("ring_two_threads", "16", "20000"),
         ("waiting",)]
FORKS = {"region_two_processes", "ring_two_processes"}  # the data-race sanitizer follows threads, not a forked child
VARIANTS = {"plain": ["-O2"],
            "race": ["-O1", "-g", "-fsanitize=thread", "-fno-omit-frame-pointer"],
            "sanitized": ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
                          "-static-libasan"]}


@pytest.fixture(scope="module")
def programs(tmp_path_factory):
    if shutil.which("g++") is None or not os.path.isdir("/opt/rocm/include"):
        pytest.skip("needs g++ and the ROCm headers")
    out = {}
    for name, flags in VARIANTS.items():
        exe = str(tmp_path_factory.mktemp("shm") / f"shm_test_{name}")
        res = subprocess.run(["g++", "-std=c++17", *flags, "-Wall", "-Wextra", "-Werror", "-pthread", "-D__HIP_PLATFORM_AMD__",
                              "-I/opt/rocm/include", "-o", exe, SOURCE, "-L/opt/rocm/lib", "-Wl,-rpath,/opt/rocm/lib",
                              "-lamdhip64", "-lrt"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out[name] = (exe if res.returncode == 0 else None, res.stdout[-2000:])
    assert out["plain"][0], "the test program does not build:\n" + out["plain"][1]
    return out


@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("case", CASES, ids=["-".join(c) for c in CASES])
def test_shared_memory_layer(programs, case, variant):
    exe, log = programs[variant]
    if exe is None:
        pytest.skip("this toolchain does not build the sanitized variant: " + log[-300:])
    if variant == "race" and case[0] in FORKS:
        pytest.skip("a forked child is outside the data-race sanitizer's view")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1",
               TSAN_OPTIONS="halt_on_error=1:exitcode=66")
    res = subprocess.run([exe, *case], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120, env=env)
    assert res.returncode == 0, f"{' '.join(case)} ({variant}) exit {res.returncode}:\n{res.stdout[-3000:]}"
