"""pca_knn_fixed_scratch: the kNN entry point that takes no workspace and
allocates nothing (its scratch is a fixed buffer inside the library's device
code) returns what pca_knn returns -- bit for bit, edges and distances -- on
calls in a row that share that buffer, the second one smaller than the first.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(x, y, ptr_x, ptr_y, k, cosine=False, drop_self=False):
    from gpu_common import dev
    from pytorch_cluster_amd import capi
    args = (dev(x), dev(y), dev(ptr_x, torch.long), dev(ptr_y, torch.long), k,
            cosine)
    want_e, want_d = capi.knn_edges(*args, want_dist=True,
                                    drop_self=drop_self)
    got_e, got_d = capi.knn_edges(*args, want_dist=True, drop_self=drop_self,
                                  fixed_scratch=True)
    torch.cuda.synchronize()
    return (want_e.cpu().numpy(), want_d.cpu().numpy(),
            got_e.cpu().numpy(), got_d.cpu().numpy())


def test_fixed_scratch_matches_pca_knn_on_consecutive_calls(oracle):
    from gpu_common import oracle_knn_edges
    rng = np.random.default_rng(5)
    # 1. three clouds of 3-D points (sliced scan: shared bounds, partial
    # lists and the merge all live in the scratch)
    x1 = rng.random((6000, 3), dtype=np.float32)
    ptr1 = np.array([0, 2500, 2500, 6000], dtype=np.int64)
    # 2. right after it a smaller search of another shape (feature space)
    x2 = rng.standard_normal((700, 24)).astype(np.float32)
    y2 = rng.standard_normal((90, 24)).astype(np.float32)
    # 3. and a tiny one
    x3 = rng.random((40, 2), dtype=np.float32)
    cases = [(x1, x1, ptr1, ptr1, 17, False, True),
             (x2, y2, None, None, 9, False, False),
             (x2, y2, None, None, 9, True, False),
             (x3, x3[:7], None, None, 50, False, False)]
    for x, y, px, py, k, cosine, drop_self in cases:
        want_e, want_d, got_e, got_d = _both(x, y, px, py, k, cosine,
                                             drop_self)
        assert got_e.shape == want_e.shape
        assert (got_e == want_e).all()
        assert (got_d == want_d).all()  # bit-exact, fp32
        if not drop_self:
            oe, od = oracle_knn_edges(oracle, x, y, px, py, k, cosine)
            assert (got_e == oe).all() and (got_d == od).all()


def test_fixed_scratch_call_allocates_nothing():
    # the entry point's defining property: with the outputs allocated by the
    # caller, a direct call through the C ABI leaves the device's free memory
    # as it was (the driver's own figure, not the caching allocator's) -- on
    # the first calls of three kernel families and on repeated ones
    from gpu_common import dev
    from pytorch_cluster_amd._native import capi as lib
    rng = np.random.default_rng(6)
    cases = [(rng.random((5000, 3), dtype=np.float32), 12, 0),
             (rng.standard_normal((900, 40)).astype(np.float32), 7, 1),
             (rng.random((300, 2)).astype(np.float64), 5, 0)]
    # everything the calls touch exists before the first reading
    prepared = []
    for x, k, cosine in cases:
        xd = dev(x)
        m = x.shape[0]
        edges = torch.empty(2 * m * k, dtype=torch.long, device="cuda:0")
        count = torch.empty(1, dtype=torch.long, device="cuda:0")
        # (distances come with fp32 points only)
        dist = (torch.empty(m * k, dtype=torch.float32, device="cuda:0")
                if xd.dtype == torch.float32 else None)
        prepared.append((xd, k, cosine, edges, count, dist))
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()

    def call(xd, k, cosine, edges, count, dist):
        dtype = 1 if xd.dtype == torch.float64 else 0
        rc = lib.pca_knn_fixed_scratch(
            xd.data_ptr(), xd.data_ptr(), None, None, xd.shape[0],
            xd.shape[0], xd.shape[1], 1, k, cosine, dtype, 0,
            edges.data_ptr(), count.data_ptr(),
            dist.data_ptr() if dist is not None else None, stream)
        assert rc == 0, lib.pca_last_error()

    # (one round first: the runtime loads a library's kernels into device
    # memory at the first launch in a process, whoever launches)
    for item in prepared:
        call(*item)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for rounds in range(3):
        for item in prepared:
            call(*item)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_after == free_before, (free_before, free_after)
    for xd, k, cosine, edges, count, dist in prepared:
        assert int(count.item()) == xd.shape[0] * k


def test_fixed_scratch_refuses_what_does_not_fit():
    from pytorch_cluster_amd import capi
    from pytorch_cluster_amd._native import PCA_FIXED_SCRATCH_BYTES
    from pytorch_cluster_amd._native import capi as lib
    n = m = 1 << 20
    assert lib.pca_knn_workspace_bytes(n, m, 3, 1, 32, 0) \
        > PCA_FIXED_SCRATCH_BYTES
    x = torch.zeros(n, 3, device="cuda:0")
    with pytest.raises(capi.PcaError) as err:
        capi.knn_launch(x, x, None, None, 32, fixed_scratch=True)
    assert err.value.status == -3  # PCA_ERR_WORKSPACE
    assert "fixed buffer" in str(err.value)
    # invalid arguments are reported as by pca_knn
    with pytest.raises(capi.PcaError) as err:
        capi.knn_launch(x[:10], x[:10], None, None, 101, fixed_scratch=True)
    assert err.value.status == -2
    # and the entry point still works afterwards
    e, _ = capi.knn_edges(x[:10], x[:10], None, None, 3, fixed_scratch=True)
    assert e.shape == (2, 30)
