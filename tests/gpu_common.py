"""Helpers for the GPU parity tests (imported only by tests marked gpu)."""
import numpy as np
import torch

from pytorch_cluster_amd import capi

DEV = "cuda:0"


def dev(a, dtype=None):
    if a is None:
        return None
    t = torch.as_tensor(np.asarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV).contiguous()


def gpu_knn(x, y, ptr_x, ptr_y, k, cosine=False, want_dist=True):
    """pca_knn through the C ABI -> numpy ([2,E] edges, [E] distances)."""
    e, d = capi.knn_edges(dev(x), dev(y), dev(ptr_x, torch.long),
                          dev(ptr_y, torch.long), k, cosine, want_dist)
    torch.cuda.synchronize()
    return e.cpu().numpy(), (None if d is None else d.cpu().numpy())


def gpu_radius(x, y, ptr_x, ptr_y, r, max_nn, ignore_same=False):
    e = capi.radius_edges(dev(x), dev(y), dev(ptr_x, torch.long),
                          dev(ptr_y, torch.long), r, max_nn, ignore_same)
    torch.cuda.synchronize()
    return e.cpu().numpy()


def oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine=False):
    """Oracle edges and per-edge distances in the operator's layout."""
    _, col, dist = oracle.knn_dense(x, y, ptr_x, ptr_y, k, cosine, fma_mode=1)
    mask = col.reshape(-1) != -1
    rows = np.repeat(np.arange(len(y)), k)[mask]
    return (np.stack([rows, col.reshape(-1)[mask]]),
            dist.reshape(-1)[mask])


def ragged_ptrs(rng, total, segments, allow_empty=True):
    """Random non-decreasing CSR pointers over `total` rows."""
    if segments == 1:
        return np.array([0, total], dtype=np.int64)
    cuts = np.sort(rng.integers(0, total + 1, segments - 1))
    if allow_empty and segments > 2:
        cuts[1] = cuts[0]  # force one empty segment
    return np.concatenate([[0], cuts, [total]]).astype(np.int64)


def use_strategy(name):
    """Context manager: the package's search strategy for the block."""
    import contextlib
    import pytorch_cluster_amd as pca

    @contextlib.contextmanager
    def scope():
        before = pca.get_search_strategy()
        pca.set_search_strategy(name)
        try:
            yield
        finally:
            pca.set_search_strategy(before)
    return scope()
