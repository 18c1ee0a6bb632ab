"""Gubanex: typed config from its ``config.json`` keys, and its model plan.

A decoder-only model of pre-norm layers (RMS norms whose weights are stored around zero) whose
mixer is, layer by layer, either gated linear attention (a recurrence with a decayed matrix
state per head) or softmax attention with partial rotary positions, a weightless unit norm of
queries and keys after the rotation and a chunked mask; the feed-forward is a mixture of small
gated experts with a sigmoid router whose weights scale the experts' input, or absent.  The
embedding is scaled; a stretch of the layers may run several times in a row with the same
weights, each pass with a cache of its own and the embedding's output added to the stream
before every pass but the first; the logits are scaled and soft-capped.

    {"architecture": "Gubanex", "vocab": V, "width": W, "norm": {"eps": e},
     "embedding": {"scale": s}, "logit_scale": a, "logit_softcap": c,
     "loop": {"start": i, "stop": j, "times": n},
     "layers": [{"type": "gla", "mixer": {"heads", "dim", "vdim", "tau"}, "mlp": M},
                {"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"},
                           "rot": {"base", "dims", "scaling": {"factor", "low", "high", "original"}}},
                 "mlp": M}, ...]}
    M = {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff"}} | null

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.router``,
``l<i>.mlp.e<j>.{gate,up,down}``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any

from tokamak_amd.config.model_config import LayerCall, LayerSpec, ModelPlan, PartSpec, SubPart
from tokamak_amd.config.registry import Architecture, register_architecture

NAME = "Gubanex"
# the design has no position table and no length of its own: the cache is the only limit
MAX_POSITIONS = 1 << 20


@dataclass(frozen=True)
class FrequencyScaling:
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: FrequencyScaling | None = None


@dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    # the decay's low rank is not a configuration key: a checkpoint's tensors give it; only the
    # random-weights mode needs a number here
    decay_rank: int | None = None


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int | None = None            # None: every earlier position is seen
    rot: RotaryConfig | None = None     # None: no rotation


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class GubanexLayer:
    mixer: GlaConfig | AttentionConfig
    mlp: ExpertsConfig | None           # None: the layer has no feed-forward

    @property
    def type(self) -> str:
        return "gla" if isinstance(self.mixer, GlaConfig) else "attention"


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class GubanexConfig:
    architecture: str
    vocab_size: int
    width: int
    norm_eps: float
    layers: tuple[GubanexLayer, ...]
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float | None = None
    loop: LoopConfig | None = None
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: int = MAX_POSITIONS

    def __post_init__(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be >= 1")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if min(m.heads, m.dim, m.vdim) < 1:
                raise ValueError(f"layer {i}: every size must be >= 1")
            if isinstance(m, AttentionConfig):
                if m.kv_heads < 1 or m.heads % m.kv_heads:
                    raise ValueError(f"layer {i}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
                if m.chunk is not None and m.chunk < 1:
                    raise ValueError(f"layer {i}: mask.size must be >= 1")
                if m.rot is not None and (m.rot.dims % 2 or not 0 <= m.rot.dims <= m.dim):
                    raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
            elif not m.tau > 0:
                raise ValueError(f"layer {i}: tau must be positive")
            if layer.mlp is not None and (layer.mlp.ff < 1 or not 1 <= layer.mlp.top <= layer.mlp.experts):
                raise ValueError(f"layer {i}: ff >= 1 and 1 <= top <= experts are required")
        if self.loop is not None:
            lp = self.loop
            if not (0 <= lp.start < lp.stop <= len(self.layers)) or lp.times < 1:
                raise ValueError(f"loop {lp} does not fit {len(self.layers)} layers")

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def _need(raw: Any, key: str, where: str) -> Any:
    if not isinstance(raw, dict) or key not in raw or raw[key] is None:
        raise ValueError(f"config.json lacks required key {key!r} in {where}")
    return raw[key]


def _mlp(raw: Any, where: str) -> ExpertsConfig | None:
    if raw is None:
        return None
    kind = _need(raw, "kind", where)
    if kind != "moe":
        raise ValueError(f"{where}: unknown feed-forward kind {kind!r}; this design has 'moe'")
    router = _need(raw, "router", where)
    return ExpertsConfig(experts=int(_need(router, "experts", where + ".router")),
                         top=int(_need(router, "top", where + ".router")),
                         ff=int(_need(_need(raw, "expert", where), "ff", where + ".expert")))


def _rot(raw: Any, where: str) -> RotaryConfig | None:
    if raw is None:
        return None
    scaling = raw.get("scaling")
    if scaling is not None:
        scaling = FrequencyScaling(*(float(_need(scaling, k, where + ".scaling")) for k in ("factor", "low", "high", "original")))
    return RotaryConfig(base=float(_need(raw, "base", where)), dims=int(_need(raw, "dims", where)), scaling=scaling)


def _layer(raw: Any, i: int) -> GubanexLayer:
    where = f"layers[{i}]"
    kind = _need(raw, "type", where)
    m = _need(raw, "mixer", where)
    mw = where + ".mixer"
    if kind == "gla":
        mixer: GlaConfig | AttentionConfig = GlaConfig(
            heads=int(_need(m, "heads", mw)), dim=int(_need(m, "dim", mw)), vdim=int(_need(m, "vdim", mw)),
            tau=float(_need(m, "tau", mw)))
    elif kind == "attention":
        heads = int(_need(m, "heads", mw))
        mask = m.get("mask")
        mixer = AttentionConfig(
            heads=heads, kv_heads=int(m["kv_heads"]) if m.get("kv_heads") is not None else heads,
            dim=int(_need(m, "dim", mw)), vdim=int(_need(m, "vdim", mw)), scale=float(_need(m, "scale", mw)),
            chunk=None if mask is None else int(_need(mask, "size", mw + ".mask")),
            rot=_rot(m.get("rot"), mw + ".rot"))
    else:
        raise ValueError(f"{where}: unknown layer type {kind!r}; this design has 'gla' and 'attention'")
    return GubanexLayer(mixer=mixer, mlp=_mlp(raw.get("mlp"), where + ".mlp"))


def parse(raw: dict[str, Any], eos_token_ids: tuple[int, ...] = ()) -> GubanexConfig:
    name = raw.get("architecture")
    if name != NAME:
        raise ValueError(f"Unsupported architecture {name!r}; supported: {NAME}")
    layers = _need(raw, "layers", "config.json")
    loop = raw.get("loop")
    if loop is not None:
        loop = LoopConfig(*(int(_need(loop, k, "loop")) for k in ("start", "stop", "times")))
    softcap = raw.get("logit_softcap")
    return GubanexConfig(
        architecture=NAME,
        vocab_size=int(_need(raw, "vocab", "config.json")),
        width=int(_need(raw, "width", "config.json")),
        norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
        layers=tuple(_layer(layer, i) for i, layer in enumerate(layers)),
        embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
        logit_scale=float(raw.get("logit_scale", 1.0)),
        logit_softcap=None if softcap is None else float(softcap),
        loop=loop,
        eos_token_ids=tuple(int(t) for t in eos_token_ids),
    )


def _mixer_json(m: GlaConfig | AttentionConfig) -> dict[str, Any]:
    if isinstance(m, GlaConfig):
        return {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau}
    out: dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
    if m.chunk is not None:
        out["mask"] = {"size": m.chunk}
    if m.rot is not None:
        out["rot"] = {"base": m.rot.base, "dims": m.rot.dims}
        if m.rot.scaling is not None:
            s = m.rot.scaling
            out["rot"]["scaling"] = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
    return out


def to_config_json(cfg: GubanexConfig) -> dict[str, Any]:
    """The ``config.json`` dict that parses back to ``cfg`` (the decay's rank is not a key: the
    tensors carry it)."""
    out: dict[str, Any] = {
        "architecture": cfg.architecture,
        "vocab": cfg.vocab_size,
        "width": cfg.width,
        "norm": {"eps": cfg.norm_eps},
        "embedding": {"scale": cfg.embedding_scale},
        "logit_scale": cfg.logit_scale,
        "layers": [{
            "type": L.type,
            "mixer": _mixer_json(L.mixer),
            "mlp": None if L.mlp is None else {"kind": "moe", "router": {"experts": L.mlp.experts, "top": L.mlp.top},
                                               "expert": {"ff": L.mlp.ff}},
        } for L in cfg.layers],
    }
    if cfg.logit_softcap is not None:
        out["logit_softcap"] = cfg.logit_softcap
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop.start, "stop": cfg.loop.stop, "times": cfg.loop.times}
    return out


def run_order(cfg: GubanexConfig) -> tuple[LayerCall, ...]:
    """The layers before the loop once, the loop's layers ``times`` times in a row, the rest once.
    Every call has a cache slot of its own (each pass keeps its own keys, values and states); the
    first call of every pass but the first adds the embedding's output to the stream."""
    n = len(cfg.layers)
    lp = cfg.loop or LoopConfig(0, n, 1)
    layers = list(range(lp.start))
    first_of_pass = set()
    for p in range(lp.times):
        if p > 0:
            first_of_pass.add(len(layers))
        layers += range(lp.start, lp.stop)
    layers += range(lp.stop, n)
    return tuple(LayerCall(layer, slot, adds_embedding=slot in first_of_pass) for slot, layer in enumerate(layers))


def plan(cfg: GubanexConfig) -> ModelPlan:
    width = cfg.width
    norm = PartSpec.of("rmsnorm", dim=width, eps=cfg.norm_eps, tensor="", offset=1.0)
    layers = []
    for L in cfg.layers:
        m = L.mixer
        parts = dict(mixer_norm=SubPart("norm", norm, "norm1"))
        if isinstance(m, GlaConfig):
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "gated_linear_attention", hidden_size=width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                tau=m.tau, norm_eps=cfg.norm_eps, decay_rank=m.decay_rank), "mix.")
        else:
            parts["mixer"] = SubPart("mixer", PartSpec.of(
                "rotated_unit_attention", hidden_size=width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                value_dim=m.vdim, softmax_scale=m.scale, norm_eps=cfg.norm_eps, chunk=m.chunk), "mix.")
            if m.rot is not None and m.rot.dims > 0:
                s = m.rot.scaling
                parts["position"] = SubPart("position", PartSpec.of(
                    "rotary_half", rotary_dim=m.rot.dims, theta=m.rot.base,
                    scaling=None if s is None else (s.factor, s.low, s.high, s.original)), shared=True)
        if L.mlp is not None:
            parts.update(
                feed_forward_norm=SubPart("norm", norm, "norm2"),
                feed_forward=SubPart("feed_forward", PartSpec.of(
                    "routed_experts", hidden_size=width, intermediate_size=L.mlp.ff, num_experts=L.mlp.experts,
                    top=L.mlp.top, weight_on="input"), "mlp."),
            )
        layers.append(LayerSpec.of(PartSpec.of("pre_norm"), **parts))
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=width,
        max_position_embeddings=cfg.max_position_embeddings,
        tie_word_embeddings=False,
        embedding=PartSpec.of("token_embedding", vocab_size=cfg.vocab_size, dim=width, tensor="", scale=cfg.embedding_scale),
        layers=tuple(layers),
        order=run_order(cfg),
        final_norm=norm,
        head=PartSpec.of("linear_head", vocab_size=cfg.vocab_size, dim=width, tied=False, tensor="",
                         scale=cfg.logit_scale, softcap=cfg.logit_softcap),
        embedding_prefix="embed",
        layer_prefix="l{}.",
        final_norm_prefix="final.norm",
        head_prefix="head",
        eos_token_ids=cfg.eos_token_ids,
    )


def _shape(vocab, width, pairs, *, gla_heads, gla_dim, heads, kv, dim, chunk, experts, top, ff, rank,
           loop: LoopConfig | None = None) -> GubanexConfig:
    """``pairs`` times a gated-linear-attention layer followed by an attention layer."""
    mlp = ExpertsConfig(experts, top, ff)
    gla = GubanexLayer(GlaConfig(gla_heads, gla_dim, gla_dim, 8.0, rank), mlp)
    att = GubanexLayer(AttentionConfig(heads, kv, dim, dim, float(dim) ** -0.5, chunk,
                                       RotaryConfig(5e5, dim // 2, FrequencyScaling(4.0, 1.0, 4.0, 8192.0))), mlp)
    return GubanexConfig(NAME, vocab, width, 1e-6, (gla, att) * pairs, embedding_scale=float(width) ** 0.5,
                         logit_scale=1.0, logit_softcap=30.0, loop=loop)


# Shapes for the random-weights mode (sizes only; no trained weights exist here): a tiny one,
# and layers of the widths of 0.6B- and 8B-class models for measurements (the experts' sizes
# chosen so that a token's experts together are as wide as the dense feed-forward of that class).
PRESETS = {
    "gubanex-tiny": _shape(256, 64, 2, gla_heads=2, gla_dim=16, heads=4, kv=2, dim=16, chunk=24, experts=4, top=2,
                           ff=32, rank=8, loop=LoopConfig(1, 3, 2)),
    "gubanex-0.6b": _shape(151936, 1024, 14, gla_heads=8, gla_dim=128, heads=16, kv=8, dim=128, chunk=1024,
                           experts=16, top=2, ff=1536, rank=64),
    "gubanex-8b": _shape(151936, 4096, 18, gla_heads=32, gla_dim=128, heads=32, kv=8, dim=128, chunk=1024,
                         experts=16, top=2, ff=6144, rank=64),
}


def shorten(cfg: GubanexConfig, num_layers: int) -> GubanexConfig:
    layers = cfg.layers[:num_layers]
    loop = cfg.loop
    if loop is not None and loop.stop > len(layers):
        loop = None
    return replace(cfg, layers=layers, loop=loop)


register_architecture(Architecture(name=NAME, parse=parse, plan=plan, to_json=to_config_json, presets=PRESETS,
                                   shorten=shorten))
