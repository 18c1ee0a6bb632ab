"""Token embedding and the output head."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import Embedding, Fetch, Head
from tokamak_amd.weights.spec import TensorSpec


class TokenEmbedding(Embedding):
    """Row gather into the float32 residual stream (reference: src/tokamak/model/transformer.py:140),
    times ``scale`` if the design has one.  ``add_to`` adds the same rows into a stream once more,
    for a model that feeds its input in again further up (``LayerCall.adds_embedding``)."""

    capturable = True

    def __init__(self, *, vocab_size: int, dim: int, dtype, device, tensor: str = "weight", scale: float = 1.0) -> None:
        super().__init__(dtype=dtype, device=device)
        self.vocab_size, self.dim = int(vocab_size), int(dim)
        self.scale = float(scale)
        self.tensor = str(tensor)       # the matrix's name behind the part's prefix
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + self.tensor: TensorSpec((self.vocab_size, self.dim))}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + self.tensor)

    def tied_matrix(self) -> torch.Tensor:
        return self.weight

    def forward(self, batch) -> torch.Tensor:
        resid = torch.empty((batch.num_tokens, self.dim), dtype=torch.float32, device=self.device)
        ops.embed_gather(self.weight, batch.token_ids, resid, self.scale)
        return resid

    def add_to(self, batch, resid: torch.Tensor) -> None:
        ops.embed_gather(self.weight, batch.token_ids, resid, self.scale, accumulate=True)


class LinearHead(Head):
    """logits = h @ W^T in float32; a tied head uses the embedding matrix itself
    (reference: src/tokamak/model/transformer.py:154-156,173-176).  With ``scale`` the logits
    are multiplied by it, and with ``softcap`` c they then become c * tanh(logits / c)."""

    capturable = True

    def __init__(self, *, vocab_size: int, dim: int, tied: bool, dtype, device, tensor: str = "weight",
                 scale: float = 1.0, softcap: float | None = None) -> None:
        super().__init__(dtype=dtype, device=device)
        self.vocab_size, self.dim, self.tied = int(vocab_size), int(dim), bool(tied)
        self.scale = float(scale)
        self.softcap = None if softcap is None else float(softcap)
        if self.softcap is not None and self.softcap <= 0:
            raise ValueError(f"softcap must be positive, got {softcap}")
        self.tensor = str(tensor)
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        # a tied checkpoint may still carry its own copy: it is skipped
        # (reference: src/tokamak/model/loader.py:79-80)
        return {prefix + self.tensor: TensorSpec((self.vocab_size, self.dim), ignored=self.tied)}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        if not self.tied:
            self.weight = fetch(prefix + self.tensor)

    def tie(self, embedding: Embedding) -> None:
        weight = embedding.tied_matrix()
        if tuple(weight.shape) != (self.vocab_size, self.dim):
            raise ValueError(f"a tied head of {(self.vocab_size, self.dim)} cannot share an embedding "
                             f"matrix of {tuple(weight.shape)}")
        self.weight = weight

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        logits = linear(h, self.weight, out_dtype=torch.float32)
        if self.scale != 1.0 or self.softcap is not None:
            ops.scale_softcap(logits, self.scale, self.softcap)
        return logits


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
