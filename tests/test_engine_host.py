"""The process-rank engine's host side without a GPU: tests/cpp/engine_host_test.cpp builds the engine from the
library's own sources (tandem_amd/csrc/engine.hip, engine_abi.hip, abi.hip) against a stand-in for the HIP runtime and
for the four kernel launchers (tests/cpp/fake_hip.cpp, fake_kernels.cpp: a stream is a thread with a queue, so work on
two streams overlaps unless the engine orders it, and the data-race sanitizer sees every pair of accesses it left
unordered), forks one process per rank and drives every collective through the C ABI: tensors produced by a slow
producer and consumed right behind the waits on a stream of the caller's, many in flight, both waits, the staged and the slot-ring protocol, staging windows of
4 KiB, arenas, more collectives in flight than done words, refusals, close, and what the ranks that remain are told
when one leaves or brings a tensor of another length. Built plainly, with the host's data-race
sanitizer and with its address and undefined-behaviour sanitizers (which cannot share a process with the real runtime).
The stand-ins serve this program only: the package's library is never built from them, and what the kernels compute
is the GPU tests' business."""

import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = [os.path.join(ROOT, "tandem_amd", "csrc", f) for f in ("engine.hip", "engine_abi.hip", "abi.hip")]
DOUBLES = [os.path.join(HERE, "cpp", f) for f in ("fake_hip.cpp", "fake_kernels.cpp", "engine_host_test.cpp")]
CASES = [("2", "staged"), ("3", "staged"), ("4", "staged"), ("5", "staged"), ("8", "staged"), ("2", "ring"), ("3", "ring"), ("4", "ring"),
         ("3", "staged", "4096"),
         # the engine's other ways of ordering streams: gathers on a side stream, the caller's stream waited for on the
         # GPU instead of by polling, every wait parking the stream instead of blocking the host
         ("3", "staged", "0", "-", "TANDEM_HIP_GATHER=stream,TANDEM_HIP_READY=gpu,TANDEM_HIP_WAIT=stream"),
         ("2", "ring", "0", "-", "TANDEM_HIP_READY=gpu,TANDEM_HIP_WAIT=stream"),
         # a single hardware queue: parked waits are taken on the host instead
         ("3", "staged", "0", "-", "GPU_MAX_HW_QUEUES=1,TANDEM_HIP_WAIT=stream,TANDEM_HIP_GATHER=stream"),
         ("3", "staged", "0", "-", "TANDEM_HIP_GATHER=stream-events"), ("2", "staged", "0", "-", "TANDEM_HIP_GATHER=stream,FAKE_HIP_JITTER_US=200"),
         ("3", "staged", "0", "-", "TANDEM_HIP_GATHER=stream-words,FAKE_HIP_JITTER_US=200"),
         # streams that lag behind the host by varying amounts (every piece of work on a stream starts up to 200 us late),
         # with staging windows of 4 KiB so that the two halves are reused many times
         ("3", "staged", "4096", "-", "FAKE_HIP_JITTER_US=200"), ("3", "ring", "0", "-", "FAKE_HIP_JITTER_US=200"),
         ("2", "staged", "4096", "-", "FAKE_HIP_JITTER_US=200,TANDEM_HIP_GATHER=stream,TANDEM_HIP_READY=gpu,TANDEM_HIP_WAIT=stream"),
         # slot hand-over ordered by interprocess events (TANDEM_HIP_SYNC=event), which the machines this was built on
         # refuse and the stand-in can offer: the only place that path runs
         ("3", "ring", "0", "-", "TANDEM_HIP_SYNC=event,FAKE_HIP_IPC_EVENTS=1"),
         ("4", "ring", "0", "-", "TANDEM_HIP_SYNC=event,FAKE_HIP_IPC_EVENTS=1,FAKE_HIP_JITTER_US=200"),
         # the group falls apart: a rank that leaves without a word, ranks that bring tensors of different lengths
         ("3", "staged", "0", "dies"), ("3", "ring", "0", "dies"), ("3", "staged", "0", "out_of_step"), ("2", "ring", "0", "out_of_step"),
         # a parked stream whose collective does not end in time lets itself go, and the engine says so
         ("2", "staged", "0", "park_gives_up", "TANDEM_HIP_PARK_LIMIT_S=0.05"), ("3", "ring", "0", "park_gives_up", "TANDEM_HIP_PARK_LIMIT_S=0.05"),
         # an engine that cannot start (no interprocess events for TANDEM_HIP_SYNC=event; bad arguments) leaves nothing behind
         ("2", "staged", "0", "no_ipc_events")]
VARIANTS = {"plain": ["-O2"],
            "race": ["-O1", "-g", "-fsanitize=thread", "-fno-omit-frame-pointer"],
            "sanitized": ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
                          "-static-libasan"]}


@pytest.fixture(scope="module")
def programs(tmp_path_factory):
    if shutil.which("g++") is None or not os.path.isdir("/opt/rocm/include"):
        pytest.skip("needs g++ and the ROCm headers")
    out, builds = {}, {}
    for name, flags in VARIANTS.items():  # the three builds side by side
        exe = str(tmp_path_factory.mktemp("engine") / f"engine_host_{name}")
        builds[name] = (exe, subprocess.Popen(["g++", "-std=c++17", *flags, "-Wall", "-Wextra", "-Werror", "-pthread", "-D__HIP_PLATFORM_AMD__",
                                               "-I/opt/rocm/include", "-o", exe, "-x", "c++", *SOURCES, *DOUBLES, "-lrt"],
                                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    for name, (exe, proc) in builds.items():
        log = proc.communicate()[0]
        out[name] = (exe if proc.returncode == 0 else None, log[-3000:])
    assert out["plain"][0], "the test program does not build:\n" + out["plain"][1]
    return out


@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("case", CASES, ids=["-".join(c) for c in CASES])
def test_engine_host_side(programs, case, variant):
    exe, log = programs[variant]
    if exe is None:
        pytest.skip("this toolchain does not build the sanitized variant: " + log[-300:])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1",
               TSAN_OPTIONS="halt_on_error=1:exitcode=66")
    res = subprocess.run([exe, *case], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=env)
    assert res.returncode == 0, f"{' '.join(case)} ({variant}) exit {res.returncode}:\n{res.stdout[-4000:]}"
