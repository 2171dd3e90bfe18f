"""bench.py takes its HBM-traffic figures from the tracked counter summaries: every entry must resolve."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


@pytest.mark.parametrize("key", sorted(bench.PROFILE_TRAFFIC))
def test_traffic_entry_resolves(key):
    nbytes, source = bench.profile_traffic(key)
    assert os.path.isfile(os.path.join(ROOT, source))
    # every entry moves at least its smallest tensor and at most a few GB
    assert 1e8 < nbytes < 4e9


def test_missing_kernel_is_an_error(monkeypatch):
    monkeypatch.setitem(bench.PROFILE_TRAFFIC, "gemm_fwd", (bench._STEP, [("ag::no_such_kernel", "avg")]))
    with pytest.raises(RuntimeError, match="no_such_kernel"):
        bench.profile_traffic("gemm_fwd")


def test_traffic_is_close_to_the_algorithmic_bytes():
    # bordered planes: 60 x 57 floats per channel plane; a measured figure far above the algorithmic one means re-reads
    x_bordered, gy_bordered = 256 * 64 * 60 * 57 * 4, 256 * 128 * 60 * 57 * 4
    y = 256 * 128 * 56 * 56 * 4
    assert bench.profile_traffic("gemm_input_grad")[0] < 1.10 * (gy_bordered + 256 * 64 * 56 * 56 * 4)
    assert bench.profile_traffic("gemm_fwd")[0] < 1.25 * (x_bordered + y)
    pool = 4 * (256 * 128 * 56 * 56 + 2 * 256 * 128 * 27 * 27)
    assert bench.profile_traffic("maxpool_fwd")[0] < 1.06 * pool
    assert bench.profile_traffic("maxpool_bwd")[0] < 1.06 * pool
