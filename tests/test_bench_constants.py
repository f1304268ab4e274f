"""bench.py carries HBM traffic figures that no timed run can measure (a counter run cannot share a process with the timed
passes): each must be the figure of the rocprofv3 summary it names, so that a kernel change that is re-profiled cannot leave a
stale constant behind unnoticed."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_every_profiled_traffic_constant_is_the_figure_of_its_profile():
    import bench
    assert set(bench.PROFILED_TRAFFIC) == {"config0", "config1", "config1_32k", "config2", "config3", "config4"}
    for workload, (traffic, source) in bench.PROFILED_TRAFFIC.items():
        path = os.path.join(ROOT, source)
        assert os.path.isfile(path), f"{workload}: {source} is not there"
        text = open(path).read()
        # the summaries print the figure the bench line carries in bold: **626.9 MB**
        stated = [float(number) for number in re.findall(r"\*\*([0-9]+(?:\.[0-9]+)?) MB\*\*", text)]
        assert stated, f"{source} states no traffic figure in bold"
        assert any(abs(traffic / 1e6 - figure) < 0.051 for figure in stated), f"{workload}: bench.py says {traffic / 1e6:.1f} MB, {source} says {stated}"
