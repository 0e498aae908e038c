"""The HBM-traffic figure bench.py prints is a profiled constant: it has to be the one its profile records."""
import os
import re

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_constant_is_the_profiled_figure():
    text = open(os.path.join(ROOT, bench.PROFILED_TRAFFIC_SOURCE)).read()
    m = re.search(r"Traffic per launch = ([\d ]+) B", text)
    assert m, "the profile no longer states the traffic per launch"
    assert int(m.group(1).replace(" ", "")) == bench.PROFILED_TRAFFIC_BYTES
    # the figure is the two scaled counters added up, and the profile shows both
    fetch = re.search(r"\| FETCH_SIZE \| [\d .]+ \| ([\d ]+) \|", text)
    write = re.search(r"\| WRITE_SIZE \| [\d .]+ \| ([\d ]+) \|", text)
    assert int(fetch.group(1).replace(" ", "")) + int(write.group(1).replace(" ", "")) == bench.PROFILED_TRAFFIC_BYTES
    # and it cannot be below what the algorithm has to move
    assert bench.PROFILED_TRAFFIC_BYTES >= bench.gemv_bytes(bench.Q4K, 14336, 4096)
