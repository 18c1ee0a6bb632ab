"""Per-coordinate scales of a sub-layer's output."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.parts.base import Fetch, Part
from tokamak_amd.weights.spec import TensorSpec


class LayerScale(Part):
    """delta = scale * (weight_a * a + weight_b * b), float32: the weighted sum of one or two
    branches of a sub-layer times a learned vector, formed in 32-bit on the way into the
    residual stream (the norm that follows adds ``delta``).  A branch is [N, H] in the compute
    dtype or float32, or the float32 partial sums of a split product."""

    capturable = True
    replayable = True

    def __init__(self, *, dim: int, dtype, device, tensor: str = "weight") -> None:
        super().__init__(dtype=dtype, device=device)
        self.dim = int(dim)
        self.tensor = str(tensor)
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + self.tensor: TensorSpec((self.dim,), role="vector")}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + self.tensor)

    def forward(self, a, weight_a: float = 1.0, b=None, weight_b: float = 0.0) -> torch.Tensor:
        return scaled_sum(a, weight_a, b, weight_b, self.weight, self.dim, self.dtype)


def scaled_sum(a, weight_a, b, weight_b, scale, dim, dtype) -> torch.Tensor:
    n = a.shape[-2]
    out = torch.empty((n, dim), dtype=torch.float32, device=a.device)
    ops.scaled_sum(a, weight_a, b, weight_b, scale, out, dtype)
    return out


register_part("scale", "layer_scale", LayerScale)
