"""
Seeded synthetic inputs for the five k-means workloads this package is measured on.

Everything is generated on the CPU with ``torch.Generator().manual_seed(seed)`` in fixed 1 Mi-row
chunks, so a CPU checker and the GPU path see identical bytes regardless of thread count; callers
move the result to the device themselves.  ``scale`` shrinks N (for tests and bounded CPU timing)
without changing the distribution.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

_CHUNK = 1 << 20


@dataclass
class Workload:
    name: str
    x: torch.Tensor  # (N, D) float32
    init: Optional[torch.Tensor]  # (K, D) float32, None for the cdist-only workload
    y: Optional[torch.Tensor]  # (M, D) float32, only for the cdist-only workload
    k: int
    max_iter: int
    seed: int


def _randn_rows(n: int, d: int, gen: torch.Generator) -> torch.Tensor:
    out = torch.empty((n, d), dtype=torch.float32)
    for s in range(0, n, _CHUNK):
        e = min(n, s + _CHUNK)
        out[s:e] = torch.randn((e - s, d), generator=gen, dtype=torch.float32)
    return out


def _blobs(
    sizes: torch.Tensor, centres: torch.Tensor, sigma: torch.Tensor, gen: torch.Generator
) -> torch.Tensor:
    """Rows of cluster j ~ N(centres[j], diag(sigma[j]**2)); sigma is (K,1) or (K,D). Unshuffled."""
    n = int(sizes.sum())
    d = centres.shape[1]
    lab = torch.repeat_interleave(torch.arange(sizes.numel()), sizes)
    x = _randn_rows(n, d, gen)
    for s in range(0, n, _CHUNK):
        l = lab[s : s + _CHUNK]
        x[s : s + _CHUNK].mul_(sigma[l]).add_(centres[l])
    return x


def _shuffle(x: torch.Tensor, gen: torch.Generator) -> torch.Tensor:
    perm = torch.randperm(x.shape[0], generator=gen)
    return x[perm].contiguous()


def config1(scale: float = 1.0) -> Workload:
    """N=100 000, D=8, K=16: 16 equal blobs, centres U[-10,10]^8, sigma 1; init = first 16 rows; 20 it."""
    seed, k, d = 1001, 16, 8
    gen = torch.Generator().manual_seed(seed)
    per = max(int(6250 * scale), 2)
    centres = torch.rand((k, d), generator=gen) * 20.0 - 10.0
    x = _blobs(torch.full((k,), per, dtype=torch.int64), centres, torch.ones((k, 1)), gen)
    x = _shuffle(x, gen)
    return Workload("c1_n100k_d8_k16", x, x[:k].clone(), None, k, 20, seed)


def config2(scale: float = 1.0) -> Workload:
    """cdist+argmin only: X 1 048 576 x 64, Y 1024 x 64, both i.i.d. N(0,1)."""
    seed = 1002
    gen = torch.Generator().manual_seed(seed)
    n = max(int(1048576 * scale), 64)
    x = _randn_rows(n, 64, gen)
    y = _randn_rows(1024, 64, gen)
    return Workload("c2_cdist_argmin_n1m_d64_m1024", x, None, y, 1024, 1, seed)


def config3(scale: float = 1.0) -> Workload:
    """Headline: N=10 000 000, D=32, K=256; centres U[-5,5]^32, sizes ~ Dirichlet(1)*N, sigma .5; 10 it."""
    seed, k, d = 1003, 256, 32
    gen = torch.Generator().manual_seed(seed)
    n = max(int(10_000_000 * scale), 4 * k)
    centres = torch.rand((k, d), generator=gen) * 10.0 - 5.0
    # Dirichlet(1) = normalised Exp(1) draws
    w = -torch.log(torch.rand((k,), generator=gen, dtype=torch.float64).clamp_min(1e-300))
    w = w / w.sum()
    sizes = torch.floor(w * n).to(torch.int64)
    sizes[torch.argmax(sizes)] += n - int(sizes.sum())
    x = _blobs(sizes, centres, torch.full((k, 1), 0.5), gen)
    x = _shuffle(x, gen)
    pick = torch.randperm(n, generator=gen)[:k]
    return Workload("c3_n10m_d32_k256", x, x[pick].clone(), None, k, 10, seed)


def config4(scale: float = 1.0) -> Workload:
    """MFMA-bound: N=2 000 000, D=512, K=1024; centres N(0,4I), per-cluster sigma U[.5,1.5]; 5 it."""
    seed, k, d = 1004, 1024, 512
    gen = torch.Generator().manual_seed(seed)
    n = max(int(2_000_000 * scale), 2 * k)
    centres = torch.randn((k, d), generator=gen) * 2.0
    sigma = torch.rand((k, 1), generator=gen) + 0.5
    base, rem = divmod(n, k)
    sizes = torch.full((k,), base, dtype=torch.int64)
    sizes[:rem] += 1
    x = _blobs(sizes, centres, sigma, gen)
    x = _shuffle(x, gen)
    pick = torch.randperm(n, generator=gen)[:k]
    return Workload("c4_n2m_d512_k1024", x, x[pick].clone(), None, k, 5, seed)


def config5(scale: float = 1.0) -> Workload:
    """HBM-bound: N=200 000 000, D=3, K=8; anisotropic blobs + 5 % uniform background; 10 it."""
    seed, k, d = 1005, 8, 3
    gen = torch.Generator().manual_seed(seed)
    n = max(int(200_000_000 * scale), 64)
    centres = torch.rand((k, d), generator=gen) * 200.0 - 100.0
    sigma = torch.rand((k, d), generator=gen) * 9.0 + 1.0
    n_noise = n // 20
    n_blob = n - n_noise
    base, rem = divmod(n_blob, k)
    sizes = torch.full((k,), base, dtype=torch.int64)
    sizes[:rem] += 1
    x = torch.empty((n, d), dtype=torch.float32)
    x[:n_blob] = _blobs(sizes, centres, sigma, gen)
    lo = x[:n_blob].min(dim=0).values
    hi = x[:n_blob].max(dim=0).values
    for s in range(n_blob, n, _CHUNK):
        e = min(n, s + _CHUNK)
        x[s:e] = torch.rand((e - s, d), generator=gen) * (hi - lo) + lo
    x = _shuffle(x, gen)
    pick = torch.randperm(n, generator=gen)[:k]
    return Workload("c5_n200m_d3_k8", x, x[pick].clone(), None, k, 10, seed)


def shape(n: int, d: int, k: int, seed: int = 1100) -> Workload:
    """Any (N, D, K): K equal blobs, centres U[-10,10]^D, sigma 1, shuffled; init = first K rows.  For timing
    shapes between the five workloads (``bench.py --shape N D K``)."""
    gen = torch.Generator().manual_seed(seed)
    centres = torch.rand((k, d), generator=gen) * 20.0 - 10.0
    sizes = torch.full((k,), n // k, dtype=torch.int64)
    sizes[: n - int(sizes.sum())] += 1
    x = _shuffle(_blobs(sizes, centres, torch.ones((k, 1)), gen), gen)
    return Workload(f"shape_n{n}_d{d}_k{k}", x, x[:k].clone(), None, k, 20, seed)


CONFIGS = {"c1": config1, "c2": config2, "c3": config3, "c4": config4, "c5": config5}


def spherical_dataset(num_samples_cluster: int, radius: float = 1.0, offset: float = 4.0,
                      dtype: torch.dtype = torch.float32, seed: int = 1) -> torch.Tensor:
    """
    Four balls of ``num_samples_cluster`` points each, centred on the space diagonal of R^3 at
    (+-offset) and (+-2 offset) in every coordinate: the shape of the data set the reference's
    clustering tests use (heat/utils/data/spherical.py:7-55).  The same points (polar coordinates
    with uniform radius and angles) are shifted to all four centres.
    """
    gen = torch.Generator().manual_seed(int(seed))
    r = torch.rand(num_samples_cluster, generator=gen) * radius
    theta = torch.rand(num_samples_cluster, generator=gen) * 3.1415
    phi = torch.rand(num_samples_cluster, generator=gen) * 2 * 3.1415
    pts = torch.stack((r * theta.sin() * phi.cos(), r * theta.sin() * phi.sin(), r * theta.cos()), dim=1)
    data = torch.cat([pts + s * offset for s in (1.0, 2.0, -1.0, -2.0)], dim=0)
    return data.to(dtype)
