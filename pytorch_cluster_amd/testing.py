"""Seeded synthetic workloads for tests and the benchmark.

Every generator draws on the CPU from ``torch.Generator().manual_seed(seed)``
so that a CPU checker and the GPU see identical bits, and returns CPU tensors.
"""
import math
from typing import Dict

import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def uniform_cloud(seed: int = 0, n: int = 1024, d: int = 3) -> Dict:
    """One cloud, uniform in the unit cube (the CPU-sized plumbing case:
    ``knn_graph(x, k=16, loop=False)``)."""
    return {"x": torch.rand(n, d, generator=_gen(seed))}


def uniform_batched(seed: int = 0, clouds: int = 16, points: int = 4096,
                    d: int = 3) -> Dict:
    """``clouds`` clouds of ``points`` points each, uniform in the unit cube,
    batch vector sorted ascending (``knn_graph(x, k=20, batch)``)."""
    x = torch.rand(clouds * points, d, generator=_gen(seed))
    batch = torch.arange(clouds).repeat_interleave(points)
    return {"x": x, "batch": batch, "batch_size": clouds}


def gaussian_mixture_batched(seed: int = 0, clouds: int = 8,
                             points: int = 16384, components: int = 32,
                             sigma: float = 0.02) -> Dict:
    """Each cloud is a mixture of isotropic 3-D Gaussians with centres uniform
    in the unit cube; points stay in generation order, components interleaved
    (``radius_graph(x, r=0.05, batch, max_num_neighbors=32)``)."""
    g = _gen(seed)
    parts = []
    for _ in range(clouds):
        centres = torch.rand(components, 3, generator=g)
        comp = torch.randint(0, components, (points,), generator=g)
        parts.append(centres[comp] + sigma * torch.randn(points, 3,
                                                         generator=g))
    x = torch.cat(parts, 0)
    batch = torch.arange(clouds).repeat_interleave(points)
    return {"x": x, "batch": batch, "batch_size": clouds}


def feature_space(seed: int = 0, n: int = 200000, m: int = 50000,
                  d: int = 128) -> Dict:
    """Standard-normal feature rows (``knn(x, y, k=32)``, Euclidean and
    cosine)."""
    g = _gen(seed)
    x = torch.randn(n, d, generator=g)
    y = torch.randn(m, d, generator=g)
    return {"x": x, "y": y}


def lidar_scans(seed: int = 0, scans: int = 8, min_points: int = 60000,
                max_points: int = 200000, beams: int = 64,
                query_stride: int = 4) -> Dict:
    """Ragged LiDAR-like scans: ranges with density proportional to 1/rho^2
    on [1, 80] m, 64 elevation beams between -25 and +3 degrees, uniform
    azimuth, 2 cm vertical noise; the queries are every ``query_stride``-th
    point of each scan (``knn(x, y, k=16, batch_x, batch_y)``)."""
    g = _gen(seed)
    sizes = torch.randint(min_points, max_points + 1, (scans,), generator=g)
    theta = torch.linspace(math.radians(-25.0), math.radians(3.0), beams)
    xs, ys, bx, by = [], [], [], []
    for b, nb in enumerate(sizes.tolist()):
        beam = torch.randint(0, beams, (nb,), generator=g)
        u = torch.rand(nb, generator=g)
        rho = 1.0 / (1.0 - u * (1.0 - 1.0 / 80.0))
        phi = 2.0 * math.pi * torch.rand(nb, generator=g)
        z = rho * torch.tan(theta[beam]) + 0.02 * torch.randn(nb, generator=g)
        pts = torch.stack([rho * torch.cos(phi), rho * torch.sin(phi), z], 1)
        pts = pts.to(torch.float32).contiguous()
        q = pts[::query_stride].contiguous()
        xs.append(pts)
        ys.append(q)
        bx.append(torch.full((pts.size(0),), b, dtype=torch.long))
        by.append(torch.full((q.size(0),), b, dtype=torch.long))
    return {"x": torch.cat(xs), "y": torch.cat(ys), "batch_x": torch.cat(bx),
            "batch_y": torch.cat(by), "batch_size": scans,
            "sizes": sizes.tolist()}


def pointers(batch: torch.Tensor, batch_size: int) -> torch.Tensor:
    """CSR pointers ``[batch_size + 1]`` of a sorted batch vector."""
    return torch.bucketize(torch.arange(batch_size + 1), batch)
