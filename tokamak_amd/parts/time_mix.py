"""Recurrent token mixing with a matrix-valued state per head."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import Fetch, Mixer, PositionData, StateArray
from tokamak_amd.weights.spec import TensorSpec

MIXES = ("r", "k", "v", "g", "w")


class DecayedStateTimeMix(Mixer):
    """Linear-attention recurrence with a per-channel, data-dependent decay.

    With x' the row before x in its sequence (zeros before the first), each of the five inputs
    is x + (x' - x) * mu_s.  r, k, v are projections of theirs into ``num_heads`` heads of
    ``head_dim`` channels, gate = silu(W_g .), and the decay of key channel c is
    w_c = exp(-exp((W_w2 tanh(W_w1 .))_c + w0_c)) (W_w1's rank is read off the checkpoint unless
    ``decay_rank`` gives it).  Per head, with the state S [head_dim, head_dim] (all zeros before a sequence's first token):

        o_t = (S + diag(u) k_t v_t^T)^T r_t          (u weights the newest key-value product, which S does not hold yet)
        S  <- diag(w_t) S + k_t v_t^T

    o is divided by its root mean square per head, multiplied by ``norm`` and by the gate, and
    projected by W_o.  S and the newest input row are the request's state (float32), carried
    from step to step; decays, exponentials, the recurrence and the norm are float32.
    Tensors: mu.r mu.k mu.v mu.g mu.w, r, k, v, g, w1, w2, w0, u, norm, o.
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float,
                 decay_rank: int | None = None, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        if not 1 <= self.head_dim <= ops.WKV_MAX_DIM:
            raise ValueError(f"head_dim must be 1 to {ops.WKV_MAX_DIM} for the scan kernel, got {head_dim}")
        self.norm_eps = float(norm_eps)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.width = self.num_heads * self.head_dim
        self.mu: torch.Tensor | None = None
        self.r = self.k = self.v = self.g = self.w1 = self.w2 = self.o = None
        self.w0 = self.u = self.gain = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, w, rank = self.hidden_size, self.width, self.decay_rank
        out = {prefix + "mu." + s: TensorSpec((h,), role="vector") for s in MIXES}
        out.update({prefix + n: TensorSpec((w, h)) for n in ("r", "k", "v", "g")})
        out.update({
            prefix + "w1": TensorSpec((rank, h)), prefix + "w2": TensorSpec((w, rank)),
            prefix + "w0": TensorSpec((w,), held="float32"),
            prefix + "u": TensorSpec((self.num_heads, self.head_dim), held="float32"),
            prefix + "norm": TensorSpec((w,), role="vector"),
            prefix + "o": TensorSpec((h, w)),
        })
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.mu = torch.stack([fetch(prefix + "mu." + s) for s in MIXES]).contiguous()
        for n in ("r", "k", "v", "g", "w1", "w2", "o", "w0"):
            setattr(self, n, fetch(prefix + n))
        if self.w2.shape[1] != self.w1.shape[0]:
            raise ValueError(f"the two matrices of the decay disagree on its rank: {tuple(self.w1.shape)} and {tuple(self.w2.shape)}")
        self.u = fetch(prefix + "u").reshape(-1).contiguous()
        self.gain = fetch(prefix + "norm")

    def state_request(self) -> dict[str, StateArray]:
        return {"last": StateArray((self.hidden_size,), torch.float32),
                "S": StateArray((self.num_heads, self.head_dim, self.head_dim), torch.float32)}

    def forward(self, h, batch, store, writes_cache: bool = True, position: PositionData | None = None):
        n = h.shape[0]
        mixes = torch.empty((len(MIXES), n, self.hidden_size), dtype=self.dtype, device=h.device)
        ops.token_shift(h, self.mu, store.state["last"], mixes, batch)
        # (split products leave float32 partial sums, which the scan adds as it loads)
        r, k, v, gate = (linear(mixes[i], getattr(self, s), allow_partials=True) for i, s in enumerate(MIXES[:4]))
        low = torch.empty((n, self.w1.shape[0]), dtype=self.dtype, device=h.device)
        ops.tanh(linear(mixes[4], self.w1, allow_partials=True), low)
        decay_in = linear(low, self.w2, out_dtype=torch.float32, allow_partials=True)
        out = torch.empty((n, self.width), dtype=self.dtype, device=h.device)
        ops.wkv_scan(r, k, v, gate, decay_in, self.w0, self.u, self.gain, store.state["S"], out, batch,
                     heads=self.num_heads, dim=self.head_dim, eps=self.norm_eps)
        return linear(out, self.o, allow_partials=True)


register_part("mixer", "decayed_state_time_mix", DecayedStateTimeMix)
