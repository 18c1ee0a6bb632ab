"""Attention over a sliding window with pooled blocks behind it."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.attention import CONTEXT_LENGTH
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import CacheRequest, Fetch, Mixer, PagedArray, PositionData
from tokamak_amd.weights.spec import TensorSpec


class PooledWindowAttention(Mixer):
    """Grouped-query attention without rotation whose queries see two kinds of entries under
    one softmax: the last ``window`` positions (their own included) one by one, and every block
    of ``pool`` positions whose last position is behind that window by ONE key and value, the means of
    the block's cached keys and values.  Positions that have left the window while their block
    is not yet complete behind it are not seen.

    q = W_q h + b_q and k = W_k h + b_k are each divided by the root mean square of the whole
    projection (all heads at once; statistics in float32) and multiplied by a weight per
    coordinate; v = W_v h + b_v.  score = q . k * ``softmax_scale``.  After the softmax the
    heads' weights are mixed, w'_a = sum_g talk[a, g] w_g, and query head a applies w'_a to the
    values of kv head a // (num_heads / num_kv_heads).  Keys have ``head_dim`` channels, values
    ``value_dim``.  Tensors: q, k, v (matrices) with q.b, k.b, v.b, q.norm, k.norm, talk, o.

    The cache holds four paged arrays: keys and values of every position in the compute dtype,
    and the blocks' mean keys and values in float32 (``pool`` times narrower), written by the
    token that completes a block from the rows the cache holds.  A query then reads ``window``
    rows and one mean per block behind them, not the whole context.
    """

    capturable = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 window: int, pool: int, softmax_scale: float, norm_eps: float, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be divisible by num_kv_heads ({num_kv_heads})")
        if window < 1 or pool < 1:
            raise ValueError(f"window and pool must be >= 1, got {window} and {pool}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.window, self.pool = int(window), int(pool)
        self.softmax_scale, self.norm_eps = float(softmax_scale), float(norm_eps)
        self.q_width = self.num_heads * self.head_dim
        self.k_width = self.num_kv_heads * self.head_dim
        self.v_width = self.num_kv_heads * self.value_dim
        ops.pooled_window_plan(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, 1)   # sizes the kernel takes
        self.qkv: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None
        self.talk: torch.Tensor | None = None
        self.o: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, qw, kw, vw = self.hidden_size, self.q_width, self.k_width, self.v_width
        return {
            prefix + "q": TensorSpec((qw, h)), prefix + "k": TensorSpec((kw, h)), prefix + "v": TensorSpec((vw, h)),
            prefix + "q.b": TensorSpec((qw,), held="float32"), prefix + "k.b": TensorSpec((kw,), held="float32"),
            prefix + "v.b": TensorSpec((vw,), held="float32"),
            prefix + "q.norm": TensorSpec((qw,), role="vector"), prefix + "k.norm": TensorSpec((kw,), role="vector"),
            prefix + "talk": TensorSpec((self.num_heads, self.num_heads), held="float32"),
            prefix + "o": TensorSpec((h, self.num_heads * self.value_dim)),
        }

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.qkv = torch.cat([fetch(prefix + n) for n in "qkv"], dim=0).contiguous()
        self.bias = torch.cat([fetch(prefix + n + ".b") for n in "qkv"], dim=0).contiguous()
        self.q_norm = fetch(prefix + "q.norm")
        self.k_norm = fetch(prefix + "k.norm")
        self.talk = fetch(prefix + "talk")
        self.o = fetch(prefix + "o")

    def cache_request(self) -> CacheRequest:
        return CacheRequest.of(window=None, k=self.k_width, v=self.v_width,
                               k_pool=PagedArray(ops.pooled_elems(self.k_width, self.pool), torch.float32),
                               v_pool=PagedArray(ops.pooled_elems(self.v_width, self.pool), torch.float32))

    def step_planner(self):
        return CONTEXT_LENGTH

    def pair_flops(self) -> float:
        return 2.0 * self.num_heads * (self.head_dim + self.value_dim)

    def forward(self, h, batch, store, writes_cache: bool = True, position: PositionData | None = None):
        if position is not None and (position.cos is not None or position.score_slopes is not None):
            raise ops.KernelError("this attention part takes no position data: positions do not enter its scores")
        n = h.shape[0]
        tables = batch.block_tables[store.group]
        qkv = linear(h, self.qkv if writes_cache else self.qkv[: self.q_width], allow_partials=True)
        q = torch.empty((n, self.q_width), dtype=self.dtype, device=h.device)
        ops.bias_norm_store(qkv, self.bias, self.q_norm, self.k_norm, batch.positions, batch.req_of_token, tables, q,
                            store.arrays["k"], store.arrays["v"], q_width=self.q_width, k_width=self.k_width,
                            v_width=self.v_width, page_size=store.page_size, eps=self.norm_eps, store=writes_cache)
        if writes_cache:
            ops.pool_blocks(store.arrays["k"], store.arrays["v"], store.arrays["k_pool"], store.arrays["v_pool"],
                            batch.positions, batch.req_of_token, tables, n, k_width=self.k_width,
                            v_width=self.v_width, pool=self.pool, page_size=store.page_size)
        attended = torch.empty((n, self.num_heads * self.value_dim), dtype=self.dtype, device=h.device)
        ops.pooled_window_attention(q, store.arrays["k"], store.arrays["v"], store.arrays["k_pool"],
                                    store.arrays["v_pool"], tables, batch, self.talk, attended,
                                    num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, dim=self.head_dim,
                                    vdim=self.value_dim, window=self.window, pool=self.pool,
                                    page_size=store.page_size, scale=self.softmax_scale)
        return linear(attended, self.o, allow_partials=True)


register_part("mixer", "pooled_window_attention", PooledWindowAttention)
