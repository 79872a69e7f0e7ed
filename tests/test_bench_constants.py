"""The figures bench.py carries as constants agree with what they stand for."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_the_profiled_traffic_of_the_gate_up_launch_is_near_its_algorithmic_bytes():
    """roofline.traffic is read off a counter profile made offline; a kernel change that moved the launch's traffic would
    leave the constant behind: it must stay within a few per cent of the bytes the launch has to read (eight slots' gate and
    up rows of the Qwen3-shaped layer, Q4_K: 144 bytes a 256-value super-block)."""
    import bench
    algorithmic = bench.TOP_K * 2 * bench.FF * (bench.HIDDEN // 256) * 144
    assert algorithmic == 14155776
    assert 0.98 <= bench.GATE_UP_X_TRAFFIC_BYTES / algorithmic <= 1.05
