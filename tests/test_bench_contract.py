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


def _line(**sections):
    line = {"config": {"workload": "w", "algorithmic_bytes_per_step": 1, "algbw_GBps": 1.0, "frac_of_hbm_peak": 0.5},
            "roofline": {"peak": 8000.0, "frac": 0.9}}
    line.update(sections)
    return line


def _full_sections():
    rows = [{"MiB": m, "k1_frac_of_hbm": 0.5, "default_form": "one_launch", "one_launch_ms": 1.0, "one_launch_frac_of_hbm": 0.5,
             "ring_ms": 1.0, "ring_GBps": 4000.0, "fold_ms": 1.0} for m in (0.0625, 1.0, 4.0, 16.0, 64.0, 256.0)]
    mix = {k: {"GBps": 6000.0, "frac_of_hbm_peak": 0.75} for k in
           ("k1_reduce", "ring_copy", "bucket_fold_w2", "adamw", "adamw_gather_w4", "zero2_step_one_launch_w4")}
    z = {"one_launch_ms": 0.7, "ms": 0.9, "one_launch_GBps": 6000.0, "adamw_4_shards_ms": 0.37, "adamw_frac_of_hbm_peak": 0.8,
         "adamw_GBps": 6400.0, "adamw_gather_GBps": 6000.0}
    return dict(sweep=rows, stream_mix=mix, zero2_step=z, bucket_path={"ms": 0.2, "frac_of_hbm_peak": 0.8, "GBps": 6400.0},
                unit_gather={"us_per_unit": 18.0, "frac_of_hbm_peak": 0.57, "GBps": 4560.0})


def test_the_first_keys_of_config_hold_the_whole_metric():
    """A record that keeps only the first CONFIG_KEYS_KEPT keys of `config` must still answer the
    metric: the ZeRO-2 step in ms comes before the ring pass's sizes, and nothing is cut."""
    sys.path.insert(0, ROOT)
    import bench

    line = _line(**_full_sections())
    bench.summarize(line)
    keys = list(line["config"])
    assert len(keys) <= bench.CONFIG_KEYS_KEPT
    for k in ("zero2_step_one_launch_ms", "zero2_step_ms", "zero2_step_one_launch_frac", "adamw_frac", "bucket_path_frac",
              "unit_gather_frac", "pass_ms_4MiB", "pass_frac_256MiB", "pass_steps_frac_64MiB", "pass_steps_frac_256MiB"):
        assert k in keys
    assert keys.index("zero2_step_ms") < keys.index("pass_ms_4MiB")
    assert "k1_frac_64MiB" in line["roofline"] and "zero2_step_mix_ceiling_frac" in line["roofline"]


def test_a_figure_above_the_roofline_is_named():
    sys.path.insert(0, ROOT)
    import bench

    line = _line(**_full_sections())
    bench.summarize(line)
    assert bench.accounting_offenders(line) == []
    line["zero2_step"]["all_gather_GBps"] = 9260.7  # the ring's bytes over the one-launch form's time
    line["unit_gather"]["frac_of_hbm_peak"] = 1.01
    line["zero2_step"]["one_launch_frac_of_mix_ceiling"] = 1.02  # allowed: the probe is a yardstick, not a bound
    got = dict(bench.accounting_offenders(line))
    assert got == {"zero2_step.all_gather_GBps": 9260.7, "unit_gather.frac_of_hbm_peak": 1.01}
