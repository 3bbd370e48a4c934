"""bench.py's command-line contract, as far as it can be checked without a GPU."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "one GPU" in res.stderr


def test_without_a_gpu_it_says_so_instead_of_falling_back():
    import torch

    if torch.cuda.is_available():
        return
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--quick"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "no CPU path" in res.stderr and "{" not in res.stdout


def test_help_names_the_contract_flags():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True)
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in res.stdout


def test_traffic_record_names_this_build_or_is_withheld():
    """roofline.traffic comes from profiles/k1_traffic.json, which says which launch geometry it
    was measured on: bench.k1_traffic returns the figure for that geometry and workload and
    None for any other (a tile-size change must not leave a stale number in the bench line)."""
    import json

    sys.path.insert(0, ROOT)
    import bench
    from tandem_amd import _lib

    rec = json.load(open(bench.K1_TRAFFIC_FILE))
    got = bench.k1_traffic(256, _lib)
    assert got == rec["hbm_bytes_per_launch"] and abs(got / rec["algorithmic_bytes_per_launch"] - 1) < 0.01
    assert bench.k1_traffic(64, _lib) is None

    class OtherBuild:  # a library whose K1 tiles are 8 KiB
        check = staticmethod(_lib.check)

        @staticmethod
        def lib():
            real = _lib.lib()

            class L:
                @staticmethod
                def tdm_build_geometry(a, b, c):
                    status = real.tdm_build_geometry(a, b, c)
                    a._obj.value *= 2
                    return status

            return L

    assert bench.k1_traffic(256, OtherBuild) is None
