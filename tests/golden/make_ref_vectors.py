"""Writes tests/golden/ref_cpu_vectors.npz: seeded inputs and the edges the
REFERENCE's own CPU operators return for them.

The operators are compiled from the reference sources where they lie
(csrc/cpu/knn_cpu.cpp, csrc/cpu/radius_cpu.cpp) into oracle/_ref by
`make -C oracle ref`; that build only exists where /root/reference does, so
this script is run there once and its output is committed.  The inputs are
chosen (and checked below) so that the reference's KD-tree search and the
GPU kernels' arithmetic (fused multiply-adds) agree exactly: no two candidates
of a query are closer to each other in distance than the two differ in
rounding, and no radius query is truncated (the CPU reference keeps a
different subset than the CUDA kernel when it truncates).

    python tests/golden/make_ref_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(
    os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402


def main():
    if not oracle.have_ref():
        sys.exit("oracle/_ref is not built (needs /root/reference)")
    rng = np.random.default_rng(20240607)
    out = {}
    # kNN: 3 ragged segments, 3-D, k = 8; and 16-D single segment, k = 5
    n, m = 900, 260
    x = rng.standard_normal((n, 3)).astype(np.float32)
    y = rng.standard_normal((m, 3)).astype(np.float32)
    ptr_x = np.array([0, 250, 600, 900], dtype=np.int64)
    ptr_y = np.array([0, 100, 101, 260], dtype=np.int64)
    e = oracle.ref_knn(x, y, ptr_x, ptr_y, 8)
    assert (e == oracle.knn_op(x, y, ptr_x, ptr_y, 8, fma_mode=1)).all()
    out.update(knn3_x=x, knn3_y=y, knn3_ptr_x=ptr_x, knn3_ptr_y=ptr_y,
               knn3_k=np.int64(8), knn3_edges=e)
    x = rng.standard_normal((400, 16)).astype(np.float32)
    y = rng.standard_normal((64, 16)).astype(np.float32)
    e = oracle.ref_knn(x, y, None, None, 5)
    assert (e == oracle.knn_op(x, y, None, None, 5, fma_mode=1)).all()
    out.update(knn16_x=x, knn16_y=y, knn16_k=np.int64(5), knn16_edges=e)
    # radius: nothing truncated (max_num_neighbors above every degree); the
    # reference returns each query's neighbours in KD-tree order, the CUDA
    # kernel in ascending row order: stored sorted by (query, row)
    x = rng.random((800, 3)).astype(np.float32)
    y = rng.random((200, 3)).astype(np.float32)
    ptr_x = np.array([0, 300, 800], dtype=np.int64)
    ptr_y = np.array([0, 80, 200], dtype=np.int64)
    r = 0.2
    e = oracle.ref_radius(x, y, ptr_x, ptr_y, r, 512)
    order = np.lexsort((e[1], e[0]))
    e = e[:, order]
    assert (e == oracle.radius_op(x, y, ptr_x, ptr_y, r, 512,
                                  fma_mode=1)).all()
    out.update(rad_x=x, rad_y=y, rad_ptr_x=ptr_x, rad_ptr_y=ptr_y,
               rad_r=np.float64(r), rad_max=np.int64(512), rad_edges=e)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                        "ref_cpu_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
