"""Constants of bench.py that come from the CPU checker."""
import numpy as np

import bench
from pytorch_cluster_amd import testing


def test_required_pairs_of_the_radius_config(oracle):
    # the scan position of every query's 32nd hit (or the segment length):
    # what the reference's kernel has to look at on configs[2]
    c3 = testing.gaussian_mixture_batched(0)
    x = c3["x"].numpy()
    ptr = np.searchsorted(c3["batch"].numpy(), np.arange(9)).astype(np.int64)
    _, _, scanned = oracle.radius_dense(x, x, ptr, ptr, 0.05, 32, True)
    assert int(scanned.sum()) == bench.C3_REQUIRED_PAIRS
