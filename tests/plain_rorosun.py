"""A plain, slow implementation of the Rorosun design, one function per mechanism.

Whole sequences only, no cache, no batching, float64 by default: the oracle the engine's
parts, kernels and schedules are compared with.  It shares no code with the engine.

Notation: ``x`` [T, width] is the residual stream of one sequence, positions 0 .. T-1.
Weights are a dict name -> tensor with the checkpoint's names.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open


# -- mechanisms -----------------------------------------------------------------
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return rms(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def visible_tokens(i: int, size: int) -> range:
    """Positions position ``i`` sees one by one: 0 <= i - j < size."""
    return range(max(0, i - size + 1), i + 1)


def visible_blocks(i: int, size: int, pool: int) -> range:
    """Blocks of ``pool`` positions whose last position is behind the window of position ``i``:
    block b (positions b*pool .. b*pool + pool - 1) with b*pool + pool - 1 <= i - size."""
    if i - size < pool - 1:
        return range(0)
    return range((i - size - (pool - 1)) // pool + 1)


def pooled_window_weights(scores: torch.Tensor, block_scores: torch.Tensor, size: int, pool: int):
    """Softmax weights of one head.  ``scores`` [T, T]: query i against key j;
    ``block_scores`` [T, B]: query i against the mean key of block b.  Returns
    (token weights [T, T], block weights [T, B]); what is not visible has weight 0.  One
    softmax runs over the scores of the visible tokens and the visible blocks together."""
    t, nb = scores.shape[0], block_scores.shape[1]
    wt = torch.zeros_like(scores)
    wb = torch.zeros_like(block_scores)
    for i in range(t):
        js = list(visible_tokens(i, size))
        bs = list(visible_blocks(i, size, pool))
        both = torch.cat([scores[i, js], block_scores[i, bs]]) if bs else scores[i, js]
        p = torch.softmax(both, dim=0)
        wt[i, js] = p[:len(js)]
        if bs:
            wb[i, bs] = p[len(js):]
    assert nb >= 0
    return wt, wb


def block_means(a: torch.Tensor, pool: int) -> torch.Tensor:
    """[T, ...] -> [T // pool, ...]: means over complete blocks of ``pool`` positions."""
    nb = a.shape[0] // pool
    return a[:nb * pool].reshape(nb, pool, *a.shape[1:]).mean(1)


def mix_heads(weights: torch.Tensor, talk: torch.Tensor) -> torch.Tensor:
    """weights [H, T, S] -> sum_g talk[h, g] weights[g]."""
    return torch.einsum("hg,gts->hts", talk, weights)


def pooled_window_attention(h, w, p, cfg, eps, cache_dtype=None):
    """The left mixer: biased q/k/v, RMS norm of the whole q and k projections, no rotation,
    a sliding window plus pooled blocks behind it, softmax, head mixing, output projection.
    ``cache_dtype``: round keys and values to it before they are used and pooled (what a
    cache of that dtype holds)."""
    nh, nkv, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    size, pool, scale = cfg["mask"]["size"], cfg["mask"]["pool"], cfg["scale"]
    t = h.shape[0]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    q = rms(q, eps) * w[p + "q.norm"]
    k = rms(k, eps) * w[p + "k.norm"]
    if cache_dtype is not None:
        k = k.to(cache_dtype).to(h.dtype)
        v = v.to(cache_dtype).to(h.dtype)
    q = q.reshape(t, nh, d)
    k = k.reshape(t, nkv, d)
    v = v.reshape(t, nkv, dv)
    kb, vb = block_means(k, pool), block_means(v, pool)
    group = nh // nkv
    wts, wbs = [], []
    for a in range(nh):
        c = a // group
        s = (q[:, a] @ k[:, c].T) * scale
        sb = (q[:, a] @ kb[:, c].T) * scale
        wt, wb = pooled_window_weights(s, sb, size, pool)
        wts.append(wt)
        wbs.append(wb)
    wts = mix_heads(torch.stack(wts), w[p + "talk"])
    wbs = mix_heads(torch.stack(wbs), w[p + "talk"])
    out = []
    for a in range(nh):
        c = a // group
        out.append(wts[a] @ v[:, c] + wbs[a] @ vb[:, c])
    return torch.cat(out, dim=-1) @ w[p + "o"].T


def shifted(h: torch.Tensor) -> torch.Tensor:
    """The previous token's row; zeros for the first token."""
    return torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)


def decay(mix_w, w, p):
    """exp(-exp(w2 tanh(w1 x) + w0)), per head and key channel."""
    return torch.exp(-torch.exp(torch.tanh(mix_w @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"]))


def wkv_scan(r, k, v, dec, u):
    """Per head: o_t = (S + diag(u) k_t v_t^T)^T r_t; then S <- diag(w_t) S + k_t v_t^T.
    r, k, dec [T, heads, dim]; v [T, heads, dim]; u [heads, dim].  S = 0 before the first token."""
    t, nh, d = r.shape
    s = torch.zeros(nh, d, d, dtype=r.dtype)
    out = torch.zeros(t, nh, d, dtype=r.dtype)
    for i in range(t):
        kv = k[i].unsqueeze(-1) * v[i].unsqueeze(-2)                    # [heads, dim_k, dim_v]
        out[i] = torch.einsum("hk,hkv->hv", r[i], s + u.unsqueeze(-1) * kv)
        s = dec[i].unsqueeze(-1) * s + kv
    return out


def time_mix(h, w, p, cfg, eps):
    """The right mixer: token shift, receptance / key / value / gate / decay, the scan,
    unit norm per head, gain, gate, output projection."""
    nh, d = cfg["heads"], cfg["dim"]
    t = h.shape[0]
    prev = shifted(h)

    def mixed(name):
        return h + (prev - h) * w[p + "mu." + name]

    r = (mixed("r") @ w[p + "r"].T).reshape(t, nh, d)
    k = (mixed("k") @ w[p + "k"].T).reshape(t, nh, d)
    v = (mixed("v") @ w[p + "v"].T).reshape(t, nh, d)
    gate = silu(mixed("g") @ w[p + "g"].T)
    dec = decay(mixed("w"), w, p).reshape(t, nh, d)
    o = wkv_scan(r, k, v, dec, w[p + "u"])
    o = rms(o, eps).reshape(t, nh * d) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


def dense_feed_forward(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def parallel_layer(x, w, p, layer, eps, cache_dtype=None):
    mixer = layer["mixer"]
    h = scalar_norm(x, w[p + "norm1"], eps)
    left = pooled_window_attention(h, w, p + "mix.left.", mixer["left"], eps, cache_dtype)
    right = time_mix(h, w, p + "mix.right.", mixer["right"], eps)
    x = x + (mixer["left_scale"] * left + mixer["right_scale"] * right) * w[p + "ls1"]
    if layer.get("mlp") is not None:
        if layer["mlp"]["kind"] != "dense":
            raise ValueError(layer["mlp"]["kind"])
        h = scalar_norm(x, w[p + "norm2"], eps)
        x = x + dense_feed_forward(h, w, p + "mlp.") * w[p + "ls2"]
    return x


# -- the model ------------------------------------------------------------------
def residual_streams(tokens, cfg, w, cache_dtype=None):
    """The stream after every layer, [layers, T, width]."""
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    eps = cfg["norm"]["eps"]
    out = []
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        x = parallel_layer(x, w, f"l{i}.", layer, eps, cache_dtype)
        out.append(x)
    return torch.stack(out)


def logits(tokens, cfg, w, cache_dtype=None):
    """[T, vocab] in the weights' dtype."""
    x = residual_streams(tokens, cfg, w, cache_dtype)[-1]
    return scalar_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T


def read_folder(folder, dtype=torch.float64):
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    w = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            w[name] = t.to(dtype) if t.is_floating_point() else t
    return cfg, w
