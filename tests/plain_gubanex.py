"""Plain, slow implementation of the Gubanex design, one function per mechanism.

Written from the design's equations with torch on the CPU, a token at a time where the design
is sequential; it shares no code with the engine.  ``cfg`` is the ``config.json`` dict itself
and ``w`` a dict of tensors by checkpoint name.  Everything runs in the dtype of the tensors
it is given (the tests use float64 or float32).
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight lies around zero."""
    return rms(x, eps) * (1.0 + weight)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotary_frequencies(rot: dict, dtype=torch.float64) -> torch.Tensor:
    """f_i = base^(-2i/dims), rescaled by wavelength if ``rot`` has a ``scaling`` entry."""
    dims = int(rot["dims"])
    out = []
    scaling = rot.get("scaling")
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=dtype)


def rotate(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x [T, heads, dim]; the first 2 * len(freqs) dimensions of every head are rotated, dimension i
    paired with i + len(freqs)."""
    half = freqs.numel()
    if half == 0:
        return x
    angle = positions.to(freqs.dtype)[:, None] * freqs[None, :]
    cos, sin = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    u, v, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


def chunk_visible(i: int, j: int, size: int) -> bool:
    return j <= i and i // size == j // size


def chunked_attention(h: torch.Tensor, w: dict, prefix: str, m: dict, eps: float, first_position: int = 0,
                      past: tuple | None = None):
    """h [T, width]: the mixer's input for positions first_position ... ; ``past`` = (keys, values) of the
    positions before, as this function returned them.  Returns (output [T, width], (keys, values))."""
    heads, kv, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    t = h.shape[0]
    positions = torch.arange(first_position, first_position + t)
    q = (h @ w[prefix + "q"].T).view(t, heads, dim)
    k = (h @ w[prefix + "k"].T).view(t, kv, dim)
    v = (h @ w[prefix + "v"].T).view(t, kv, vdim)
    freqs = rotary_frequencies(m["rot"]) if m.get("rot") else torch.zeros(0, dtype=torch.float64)
    q, k = rms(rotate(q, positions, freqs), eps), rms(rotate(k, positions, freqs), eps)
    if past is not None:
        k, v = torch.cat([past[0], k]), torch.cat([past[1], v])
    size = int(m["mask"]["size"]) if m.get("mask") else None
    group = heads // kv
    out = torch.zeros(t, heads, vdim, dtype=h.dtype)
    for a in range(t):
        i = first_position + a
        seen = [j for j in range(i + 1) if size is None or chunk_visible(i, j, size)]
        for head in range(heads):
            scores = (k[seen, head // group] @ q[a, head]) * float(m["scale"])
            out[a, head] = torch.softmax(scores, dim=0) @ v[seen, head // group]
    return out.reshape(t, heads * vdim) @ w[prefix + "o"].T, (k, v)


def gated_linear_attention(h: torch.Tensor, w: dict, prefix: str, m: dict, eps: float, state: torch.Tensor | None = None):
    """h [T, width].  ``state`` [heads, dim, vdim] (None: zeros).  Returns (output [T, width], state)."""
    heads, dim, vdim, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    t = h.shape[0]
    q = (h @ w[prefix + "q"].T).view(t, heads, dim) * dim ** -0.5
    k = (h @ w[prefix + "k"].T).view(t, heads, dim)
    v = (h @ w[prefix + "v"].T).view(t, heads, vdim)
    z = (h @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).view(t, heads, dim)
    gate = silu(h @ w[prefix + "g"].T).view(t, heads, vdim)
    s = torch.zeros(heads, dim, vdim, dtype=h.dtype) if state is None else state.clone()
    out = torch.zeros(t, heads, vdim, dtype=h.dtype)
    for a in range(t):
        s = alpha[a][:, :, None] * s + k[a][:, :, None] * v[a][:, None, :]
        out[a] = torch.einsum("hkv,hk->hv", s, q[a])
    out = rms(out, eps) * w[prefix + "norm"] * gate
    return out.reshape(t, heads * vdim) @ w[prefix + "o"].T, s


def routed_experts(h: torch.Tensor, w: dict, prefix: str, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """Sigmoid router; the chosen experts' scores weigh the experts' INPUT and are not renormalised.
    ``margins`` receives, per token, how far the last chosen expert's logit lies above the first one
    left out, relative to their size (infinite if every expert is chosen)."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ w[prefix + "router"].T
    scores = torch.sigmoid(z)
    out = torch.zeros_like(h)
    for a in range(h.shape[0]):
        order = sorted(range(experts), key=lambda e: (-float(scores[a, e]), e))
        chosen = order[:top]
        if margins is not None:
            last, nxt = (float(z[a, order[top - 1]]), float(z[a, order[top]])) if top < experts else (math.inf, 0.0)
            margins.append((last - nxt) / (abs(last) + abs(nxt) + 1.0) if top < experts else math.inf)
        for e in chosen:
            x = scores[a, e] * h[a]
            name = f"{prefix}e{e}."
            out[a] += (silu(x @ w[name + "gate"].T) * (x @ w[name + "up"].T)) @ w[name + "down"].T
    return out


def layer_calls(cfg: dict) -> list[tuple[int, bool]]:
    """(layer, whether the embedding output is added to the stream before it), in run order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    calls = [(i, False) for i in range(start)]
    for p in range(times):
        calls += [(i, p > 0 and i == start) for i in range(start, stop)]
    return calls + [(i, False) for i in range(stop, n)]


class PlainGubanex:
    """The whole model over one sequence; ``forward`` may be called with portions, one after the
    other (keys, values and recurrent states are kept per layer call)."""

    def __init__(self, cfg: dict, weights: dict, dtype=torch.float64) -> None:
        self.cfg = cfg
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
        self.dtype = dtype
        self.calls = layer_calls(cfg)
        self.kept: list = [None] * len(self.calls)
        self.length = 0
        self.margins: list[float] = []      # per position, the narrowest choice of experts in any layer call

    def forward(self, tokens: list[int], trace: list | None = None) -> torch.Tensor:
        """Logits [T, vocab] for the next ``tokens`` of the sequence.  ``trace`` receives the stream
        after every layer call."""
        cfg, w = self.cfg, self.w
        eps = float(cfg["norm"]["eps"])
        embedded = w["embed"][torch.tensor(tokens)] * float(cfg.get("embedding", {}).get("scale", 1.0))
        x = embedded.clone()
        narrowest = [math.inf] * len(tokens)
        for at, (i, add) in enumerate(self.calls):
            layer, base = cfg["layers"][i], f"l{i}."
            if add:
                x = x + embedded
            h = offset_norm(x, w[base + "norm1"], eps)
            if layer["type"] == "gla":
                y, self.kept[at] = gated_linear_attention(h, w, base + "mix.", layer["mixer"], eps, self.kept[at])
            elif layer["type"] == "attention":
                y, self.kept[at] = chunked_attention(h, w, base + "mix.", layer["mixer"], eps, self.length, self.kept[at])
            else:
                raise ValueError(layer["type"])
            x = x + y
            if layer.get("mlp") is not None:
                margins: list[float] = []
                x = x + routed_experts(offset_norm(x, w[base + "norm2"], eps), w, base + "mlp.", layer["mlp"], margins)
                narrowest = [min(a, b) for a, b in zip(narrowest, margins)]
            if trace is not None:
                trace.append(x.clone())
        self.length += len(tokens)
        self.margins += narrowest
        logits = (offset_norm(x, w["final.norm"], eps) @ w["head"].T) * float(cfg.get("logit_scale", 1.0))
        if cfg.get("logit_softcap") is None:
            return logits
        cap = float(cfg["logit_softcap"])
        return cap * torch.tanh(logits / cap)
