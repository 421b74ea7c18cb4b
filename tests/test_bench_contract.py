"""CPU checks of bench.py's own bookkeeping."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_traffic_figure_belongs_to_the_kernel_sources_in_the_tree():
    """roofline.traffic is read under a profiler, not in the bench run; bench.py keeps a digest of the kernel sources it was
    read on and reports no figure on other sources.  A change to those sources therefore needs the counters read again
    (commands in profiles/k_strip_config3.txt) before this passes."""
    sys.path.insert(0, ROOT)
    import bench
    value, note = bench.traffic_c3()
    assert value is not None, note
    assert 38535168 < value < 2 * 43786050
