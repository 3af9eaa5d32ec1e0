"""bench.py's measured-traffic tables are keyed by what the timed launches move: a change of the
benchmark's shapes must not leave `roofline.traffic` / `roofline_mmq.traffic` silently null."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench
from infr_amd import DType


def test_sweep_traffic_is_recorded_for_the_in_f_4096_group_of_the_default_sweep():
    nbytes = sum(bench.weight_bytes(DType.Q4K, out_f, in_f) for _, out_f, in_f in bench.LAYER if in_f == 4096)
    key = nbytes * bench.N_LAYERS
    assert key in bench.MEASURED_TRAFFIC, (key, sorted(bench.MEASURED_TRAFFIC))
    # every weight byte is fetched about once: the recorded figure is within 2 % of the key
    assert 1.0 <= bench.MEASURED_TRAFFIC[key] / key < 1.02


def test_prefill_traffic_is_recorded_for_the_op_the_metric_is_quoted_on():
    ops = int(2.0 * 512 * 12288 * 4096)
    assert ops in bench.MEASURED_TRAFFIC_MMQ, sorted(bench.MEASURED_TRAFFIC_MMQ)
    algorithmic = 512 * 4096 * 4 + bench.weight_bytes(DType.Q4K, 12288, 4096) + 512 * 12288 * 4
    assert 1.0 <= bench.MEASURED_TRAFFIC_MMQ[ops] / algorithmic < 2.0
