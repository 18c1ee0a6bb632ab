"""Rorosun: typed config from its ``config.json`` keys, and its model plan.

A decoder-only model whose layers are pre-norm blocks with a single-number RMS norm, two
mixers side by side on the same normed input (attention over a sliding window with pooled
blocks behind it and mixed heads; a recurrent time mix with a decayed matrix state per
head), a weighted sum of the two, per-coordinate layer scales, and an optional gated
feed-forward.  ``config.json`` lists the layers one by one, each with sizes of its own:

    {"architecture": "Rorosun", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "parallel",
                 "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size", "pool"}},
                           "right": {"heads", "dim"}, "left_scale": a, "right_scale": b},
                 "mlp": {"kind": "dense", "ff": F} | null}, ...]}

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.left.*``, ``l<i>.mix.right.*``,
``l<i>.mlp.{gate,up,down}``, ``l<i>.ls1``, ``l<i>.ls2``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any

from tokamak_amd.config.model_config import LayerCall, LayerSpec, ModelPlan, PartSpec, SubPart
from tokamak_amd.config.registry import Architecture, register_architecture

NAME = "Rorosun"
# the design has no position table and no length of its own: the cache is the only limit
MAX_POSITIONS = 1 << 20


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    pool: int


@dataclass(frozen=True)
class TimeMixConfig:
    heads: int
    dim: int
    # the decay's low rank is not a configuration key: a checkpoint's tensors give it; only the
    # random-weights mode needs a number here
    decay_rank: int | None = None


@dataclass(frozen=True)
class RorosunLayer:
    left: WindowAttentionConfig
    right: TimeMixConfig
    left_scale: float
    right_scale: float
    ff: int | None              # None: the layer has no feed-forward


@dataclass(frozen=True)
class RorosunConfig:
    architecture: str
    vocab_size: int
    width: int
    norm_eps: float
    layers: tuple[RorosunLayer, ...]
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: int = MAX_POSITIONS

    def __post_init__(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be >= 1")
        for i, layer in enumerate(self.layers):
            a = layer.left
            if a.heads < 1 or a.kv_heads < 1 or a.heads % a.kv_heads:
                raise ValueError(f"layer {i}: heads ({a.heads}) must be a multiple of kv_heads ({a.kv_heads})")
            if min(a.dim, a.vdim, a.window, a.pool, layer.right.heads, layer.right.dim) < 1:
                raise ValueError(f"layer {i}: every size must be >= 1")
            if layer.ff is not None and layer.ff < 1:
                raise ValueError(f"layer {i}: ff must be >= 1")

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def _need(raw: dict[str, Any], key: str, where: str) -> Any:
    if not isinstance(raw, dict) or key not in raw or raw[key] is None:
        raise ValueError(f"config.json lacks required key {key!r} in {where}")
    return raw[key]


def _layer(raw: dict[str, Any], i: int) -> RorosunLayer:
    where = f"layers[{i}]"
    kind = _need(raw, "type", where)
    if kind != "parallel":
        raise ValueError(f"{where}: unknown layer type {kind!r}; this design has 'parallel'")
    mixer = _need(raw, "mixer", where)
    left, right = _need(mixer, "left", where + ".mixer"), _need(mixer, "right", where + ".mixer")
    mask = _need(left, "mask", where + ".mixer.left")
    mlp = raw.get("mlp")
    if mlp is not None and _need(mlp, "kind", where + ".mlp") != "dense":
        raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r}; this design has 'dense'")
    lw = where + ".mixer.left"
    return RorosunLayer(
        left=WindowAttentionConfig(
            heads=int(_need(left, "heads", lw)), kv_heads=int(_need(left, "kv_heads", lw)),
            dim=int(_need(left, "dim", lw)), vdim=int(_need(left, "vdim", lw)), scale=float(_need(left, "scale", lw)),
            window=int(_need(mask, "size", lw + ".mask")), pool=int(_need(mask, "pool", lw + ".mask"))),
        right=TimeMixConfig(heads=int(_need(right, "heads", where + ".mixer.right")),
                            dim=int(_need(right, "dim", where + ".mixer.right"))),
        left_scale=float(_need(mixer, "left_scale", where + ".mixer")),
        right_scale=float(_need(mixer, "right_scale", where + ".mixer")),
        ff=None if mlp is None else int(_need(mlp, "ff", where + ".mlp")),
    )


def parse(raw: dict[str, Any], eos_token_ids: tuple[int, ...] = ()) -> RorosunConfig:
    name = raw.get("architecture")
    if name != NAME:
        raise ValueError(f"Unsupported architecture {name!r}; supported: {NAME}")
    layers = _need(raw, "layers", "config.json")
    return RorosunConfig(
        architecture=NAME,
        vocab_size=int(_need(raw, "vocab", "config.json")),
        width=int(_need(raw, "width", "config.json")),
        norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
        layers=tuple(_layer(layer, i) for i, layer in enumerate(layers)),
        eos_token_ids=tuple(int(t) for t in eos_token_ids),
    )


def to_config_json(cfg: RorosunConfig) -> dict[str, Any]:
    """The ``config.json`` dict that parses back to ``cfg`` (the decay's rank is not a key: the
    tensors carry it)."""
    return {
        "architecture": cfg.architecture,
        "vocab": cfg.vocab_size,
        "width": cfg.width,
        "norm": {"eps": cfg.norm_eps},
        "layers": [{
            "type": "parallel",
            "mixer": {
                "left": {"heads": L.left.heads, "kv_heads": L.left.kv_heads, "dim": L.left.dim, "vdim": L.left.vdim,
                         "scale": L.left.scale, "mask": {"size": L.left.window, "pool": L.left.pool}},
                "right": {"heads": L.right.heads, "dim": L.right.dim},
                "left_scale": L.left_scale, "right_scale": L.right_scale,
            },
            "mlp": None if L.ff is None else {"kind": "dense", "ff": L.ff},
        } for L in cfg.layers],
    }


def plan(cfg: RorosunConfig) -> ModelPlan:
    width = cfg.width
    norm = PartSpec.of("scalar_rmsnorm", dim=width, eps=cfg.norm_eps, tensor="")
    scale = PartSpec.of("layer_scale", dim=width, tensor="")
    layers = []
    for L in cfg.layers:
        parts = dict(
            mixer_norm=SubPart("norm", norm, "norm1"),
            left=SubPart("mixer", PartSpec.of(
                "pooled_window_attention", hidden_size=width, num_heads=L.left.heads, num_kv_heads=L.left.kv_heads,
                head_dim=L.left.dim, value_dim=L.left.vdim, window=L.left.window, pool=L.left.pool,
                softmax_scale=L.left.scale, norm_eps=cfg.norm_eps), "mix.left."),
            right=SubPart("mixer", PartSpec.of(
                "decayed_state_time_mix", hidden_size=width, num_heads=L.right.heads, head_dim=L.right.dim,
                norm_eps=cfg.norm_eps, decay_rank=L.right.decay_rank), "mix.right."),
            mixer_scale=SubPart("scale", scale, "ls1"),
        )
        if L.ff is not None:
            parts.update(
                feed_forward_norm=SubPart("norm", norm, "norm2"),
                feed_forward=SubPart("feed_forward", PartSpec.of(
                    "swiglu", hidden_size=width, intermediate_size=L.ff, names=("gate", "up", "down")), "mlp."),
                feed_forward_scale=SubPart("scale", scale, "ls2"),
            )
        layers.append(LayerSpec.of(
            PartSpec.of("parallel_mixers", left_weight=L.left_scale, right_weight=L.right_scale), **parts))
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=width,
        max_position_embeddings=cfg.max_position_embeddings,
        tie_word_embeddings=False,
        embedding=PartSpec.of("token_embedding", vocab_size=cfg.vocab_size, dim=width, tensor=""),
        layers=tuple(layers),
        # a cache slot for each mixer of a layer: the attention's pages, the time mix's state
        order=tuple(LayerCall(i, (2 * i, 2 * i + 1)) for i in range(len(layers))),
        final_norm=norm,
        head=PartSpec.of("linear_head", vocab_size=cfg.vocab_size, dim=width, tied=False, tensor=""),
        embedding_prefix="embed",
        layer_prefix="l{}.",
        final_norm_prefix="final.norm",
        head_prefix="head",
        eos_token_ids=cfg.eos_token_ids,
    )


def _shape(vocab, width, layers, heads, kv, dim, window, pool, r_heads, r_dim, ff, rank) -> RorosunConfig:
    layer = RorosunLayer(
        left=WindowAttentionConfig(heads, kv, dim, dim, float(dim) ** -0.5, window, pool),
        right=TimeMixConfig(r_heads, r_dim, rank), left_scale=0.5, right_scale=0.5, ff=ff)
    return RorosunConfig(NAME, vocab, width, 1e-6, (layer,) * layers)


# Shapes for the random-weights mode (sizes only; no trained weights exist here): two tiny
# ones, and layers of the widths of 0.6B- and 8B-class models for measurements.
PRESETS = {
    "rorosun-tiny": _shape(256, 64, 2, 4, 2, 16, 12, 4, 2, 16, 96, 8),
    "rorosun-0.6b": _shape(151936, 1024, 28, 16, 8, 128, 1024, 16, 16, 64, 3072, 64),
    "rorosun-8b": _shape(151936, 4096, 36, 32, 8, 128, 1024, 16, 64, 64, 12288, 64),
}


def shorten(cfg: RorosunConfig, num_layers: int) -> RorosunConfig:
    return replace(cfg, layers=cfg.layers[:num_layers])


register_architecture(Architecture(name=NAME, parse=parse, plan=plan, to_json=to_config_json, presets=PRESETS,
                                   shorten=shorten))
