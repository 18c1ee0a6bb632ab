"""Gated linear attention: a recurrence with a decayed matrix state per head."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import Fetch, Mixer, PositionData, StateArray
from tokamak_amd.weights.spec import TensorSpec


class GatedLinearAttention(Mixer):
    """Linear attention with a data-dependent decay per key channel and an output gate.

    q = W_q h * ``head_dim``^(-1/2), k = W_k h (``num_heads`` heads of ``head_dim``), v = W_v h
    (heads of ``value_dim``); the decay of key channel c is a_c = sigmoid(z_c)^(1 / ``tau``) with
    z = W_a2 (W_a1 h) + b (the low rank of W_a1 is read off the checkpoint unless ``decay_rank``
    gives it).  Per head, with the state S [head_dim, value_dim] (zeros before a sequence's
    first token):

        S  <- diag(a_t) S + k_t v_t^T
        o_t = S^T q_t                      (the newest token is in S when it is read)

    o is divided by its root mean square per head, multiplied by ``norm`` ([value_dim], the same
    for every head) and by silu(W_g h), and projected by W_o.  S is the request's state
    (float32), carried from step to step; the decay with its logarithm and exponential, the
    recurrence, its operands' scaling and the norm are float32.
    Tensors: q, k, v, g, o, norm, a1, a2, a2.b.
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, tau: float,
                 norm_eps: float, decay_rank: int | None = None, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        if not (1 <= self.head_dim <= ops.WKV_MAX_DIM and 1 <= self.value_dim <= ops.WKV_MAX_DIM):
            raise ValueError(f"head_dim and value_dim must be 1 to {ops.WKV_MAX_DIM} for the scan kernel")
        if not tau > 0:
            raise ValueError(f"tau must be positive, got {tau}")
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.q = self.k = self.v = self.g = self.o = self.a1 = self.a2 = None
        self.bias = self.gain = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, kw, vw, rank = self.hidden_size, self.num_heads * self.head_dim, self.num_heads * self.value_dim, self.decay_rank
        return {
            prefix + "q": TensorSpec((kw, h)), prefix + "k": TensorSpec((kw, h)),
            prefix + "v": TensorSpec((vw, h)), prefix + "g": TensorSpec((vw, h)),
            prefix + "o": TensorSpec((h, vw)),
            prefix + "norm": TensorSpec((self.value_dim,), role="vector"),
            prefix + "a1": TensorSpec((rank, h)), prefix + "a2": TensorSpec((kw, rank)),
            prefix + "a2.b": TensorSpec((kw,), held="float32"),
        }

    def bind(self, prefix: str, fetch: Fetch) -> None:
        for n in ("q", "k", "v", "g", "o", "a1", "a2"):
            setattr(self, n, fetch(prefix + n))
        if self.a2.shape[1] != self.a1.shape[0]:
            raise ValueError(f"the two matrices of the decay disagree on its rank: {tuple(self.a1.shape)} and {tuple(self.a2.shape)}")
        self.bias = fetch(prefix + "a2.b")
        self.gain = fetch(prefix + "norm")

    def state_request(self) -> dict[str, StateArray]:
        return {"S": StateArray((self.num_heads, self.head_dim, self.value_dim), torch.float32)}

    def forward(self, h, batch, store, writes_cache: bool = True, position: PositionData | None = None):
        n = h.shape[0]
        # (split products leave float32 partial sums, which the scan adds as it loads)
        q, k, v, gate = (linear(h, w, allow_partials=True) for w in (self.q, self.k, self.v, self.g))
        low = linear(h, self.a1)
        # (few rows: float32 or split partial sums from the streaming product; a long portion: the
        # library's product in the compute dtype, as for the other projections)
        few = n <= ops.STREAM_MAX_ROWS
        decay_in = linear(low, self.a2, out_dtype=torch.float32 if few else None, allow_partials=True)
        out = torch.empty((n, self.num_heads * self.value_dim), dtype=self.dtype, device=h.device)
        ops.gla_scan(q, k, v, gate, decay_in, self.bias, self.gain, store.state["S"], out, batch,
                     heads=self.num_heads, dim=self.head_dim, vdim=self.value_dim,
                     q_scale=self.head_dim ** -0.5, tau=self.tau, eps=self.norm_eps)
        return linear(out, self.o, allow_partials=True)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
