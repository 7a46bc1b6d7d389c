"""
Random draws used by the centroid initialisers.

The reference draws from two unrelated streams: Heat's counter-based generator for
``ht.random.randint`` / ``ht.random.rand`` (heat/cluster/_kcluster.py:126-131,150,318) and torch's
global generator, left unseeded, for the k-means++ reclustering
(heat/cluster/batchparallelclustering.py:35-46 called with ``random_state=None`` from
_kcluster.py:216-225).  Neither stream can be reproduced outside the reference, so the draws here
come from one torch generator on the data's device, seeded with ``random_state``.  All draws go
through this small interface so a test can hand the same numbers to two implementations.
"""

from __future__ import annotations

from typing import Optional

import torch


class DeviceSampler:
    # the k-means++ seeding of a small row set may take all its draws at once, as uniform numbers
    fused_seeding = True

    def __init__(self, device: torch.device, seed: Optional[int] = None):
        self.device = torch.device(device)
        self._gen = torch.Generator(device=self.device)
        if seed is None:
            self._gen.seed()
        else:
            self._gen.manual_seed(int(seed))

    def randint(self, high: int) -> int:
        """One integer in [0, high)."""
        return int(torch.randint(0, int(high), (1,), generator=self._gen, device=self.device).item())

    def randint_rows(self, high: int, count: int) -> torch.Tensor:
        """``count`` integers in [0, high) as an int64 vector on the device, without a host round trip."""
        return torch.randint(0, int(high), (int(count),), generator=self._gen, device=self.device)

    def uniform(self, n: int) -> torch.Tensor:
        """n float32 numbers in [0, 1) on the device."""
        return torch.rand((int(n),), generator=self._gen, device=self.device, dtype=torch.float32)

    def multinomial(self, weights: torch.Tensor) -> int:
        """One index drawn with probability proportional to ``weights`` (non-negative, not all zero)."""
        return int(torch.multinomial(weights, 1, generator=self._gen).item())

    def multinomial_on_device(self, weights: torch.Tensor) -> torch.Tensor:
        """The same draw as :meth:`multinomial`, left on the device as a 0-d int64 tensor."""
        return torch.multinomial(weights, 1, generator=self._gen).reshape(())


def draw_rows(sampler, high: int, count: int, device) -> torch.Tensor:
    """``count`` row indices in [0, high) on ``device``: one vector draw where the sampler offers it
    (no host round trip), its scalar draws otherwise (test samplers that replay recorded numbers)."""
    vec = getattr(sampler, "randint_rows", None)
    if vec is not None:
        return vec(high, count).to(device=device, dtype=torch.int64)
    return torch.tensor([sampler.randint(high) for _ in range(count)], dtype=torch.int64, device=device)
