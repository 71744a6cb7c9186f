"""The kernel names bench.py reports are the ones the committed kernel trace of the benchmark shows.

The library does not say which kernel a call was dispatched to; bench.py names, per workload, the kernel it expects
(bench.KERNELS) and looks its HBM traffic up in the committed counter summary.  These checks fail when a dispatch rule or
a kernel's template arguments change without the profiles being regenerated from the new build."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_every_named_kernel_is_in_the_committed_trace():
    traced = bench.traced_kernels()
    assert traced, "profiles/bench_all_layers_kernel_trace.txt is missing or has no kernel lines"
    for workload, kernel in bench.KERNELS.items():
        assert kernel in traced, "%s: %s is not in the committed kernel trace" % (workload, kernel)


def test_every_named_kernel_has_one_traffic_figure():
    table = bench.profiled_traffic()
    assert table, "profiles/bench_all_layers_hbm_traffic.txt is missing or has no rows"
    for workload, kernel in bench.KERNELS.items():
        got = bench.traffic_for(table, kernel)
        assert got is not None and got > 0, "%s: no single traffic row for %s" % (workload, kernel)
