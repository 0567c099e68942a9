"""bench.py's constants against the committed profiles (no GPU): every HBM traffic figure that a roofline object may
carry names the profile it was read from and the kernel it was read for; that file must exist, hold the figure and name
that kernel as the dominant one. A profile regenerated for another kernel, or a figure typed over, fails here instead
of going out with a bench line."""
import os
import re

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_traffic_figure_is_the_one_of_its_profile():
    assert bench.MEASURED_TRAFFIC, "no traffic figures"
    for workload, (bytes_per_launch, profile, kernel) in bench.MEASURED_TRAFFIC.items():
        path = os.path.join(ROOT, profile)
        assert os.path.isfile(path), (workload, profile)
        text = open(path).read()
        dominant = re.search(r"Dominant kernel: `([^`]*)`", text)
        assert dominant and kernel in dominant.group(1), (workload, kernel, dominant and dominant.group(1)[:120])
        total = re.search(r"= ([0-9.]+) GB per launch", text)
        assert total, (workload, "no traffic line in " + profile)
        assert abs(float(total.group(1)) * 1e9 - bytes_per_launch) <= 0.006 * bytes_per_launch + 5e5, (workload, total.group(1), bytes_per_launch)


def test_roofline_objects_carry_the_source_or_null():
    assert bench.traffic_of("no such workload") == {"traffic": None}
    entry = bench.traffic_of("cfg3")
    assert entry["traffic"] == bench.MEASURED_TRAFFIC["cfg3"][0] and "profiles/hgemm_8192_colNT.md" in entry["traffic_source"]


def test_the_bench_line_keeps_every_baseline_configuration_in_config():
    """The driver keeps `config`, not the extra top-level keys: the compact per-configuration map is built there, from
    every workload whose name starts with cfg plus the headline, each entry numbers only."""
    names = [name for name in bench.EXTRA_WORKLOADS if name.startswith("cfg")]
    for wanted in ("cfg1_sgemm_1024_colNN", "cfg2_dgemm_8192_rowTN", "cfg3_hgemm_8192_colNT", "cfg4_sgemm_strided_batched_8192x32",
                   "cfg5_sgemm_1000_colNN", "cfg5_sgemm_4099x17x4096_colNN", "cfg5_sgemm_17x4099x4096_colNN",
                   "cfg5_sgemm_8191x8191x127_colNN"):
        assert wanted in names, wanted
    entry = bench.compact({"ms": 0.75, "gflops": 1466000.0, "gbs": 716.0, "roofline": {"bound": "mfma", "frac": 0.58}})
    assert entry == {"ms": 0.75, "tflops": 1466.0, "gbs": 716.0, "bound": "mfma", "frac": 0.58}
    source = open(os.path.join(ROOT, "bench.py")).read()
    assert 'result["config"]["baseline"] = baseline' in source and 'HEADLINE_NAME: compact(headline_entry)' in source
    assert bench.HEADLINE_NAME == "cfg2_sgemm_8192_rowTN"
