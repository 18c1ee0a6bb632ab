"""Test-side helpers for the Gubanex design: small ``config.json`` dicts written by hand,
random weights under the design's tensor names (listed here independently of the engine),
model folders, and the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file

import plain_gubanex as plain


def experts(n=4, top=2, ff=32):
    return {"kind": "moe", "router": {"experts": n, "top": top}, "expert": {"ff": ff}}


def gla(heads=2, dim=16, vdim=16, tau=8.0, mlp="default"):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau},
            "mlp": experts() if mlp == "default" else mlp}


def attention(heads=4, kv_heads=2, dim=16, vdim=16, chunk=12, rot=8, scale=None, base=10000.0, scaling=None,
              mlp="default"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
             "scale": float(dim) ** -0.5 if scale is None else scale}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    if rot:
        mixer["rot"] = {"base": base, "dims": rot}
        if scaling is not None:
            mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": mixer, "mlp": experts() if mlp == "default" else mlp}


def model_json(layers, vocab=200, width=64, eps=1e-5, loop=None, embedding_scale=4.0, logit_scale=1.5, softcap=20.0):
    cfg = {"architecture": "Gubanex", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": embedding_scale}, "logit_scale": logit_scale, "logit_softcap": softcap,
           "layers": list(layers)}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def random_weights(cfg, seed, rank=8):
    """name -> float32 tensor holding bfloat16-representable values."""
    g = torch.Generator().manual_seed(seed)
    w = {}

    def put(name, t):
        w[name] = t.to(torch.bfloat16).float()

    def mat(name, out, inp, gain=1.0):
        put(name, torch.randn(out, inp, generator=g) * gain * inp ** -0.5)

    W = cfg["width"]
    put("embed", torch.randn(cfg["vocab"], W, generator=g) / float(cfg["embedding"]["scale"]))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        put(p + "norm1", 0.2 * torch.randn(W, generator=g))
        if L["type"] == "gla":
            kw, vw = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            # (queries lean towards their own keys: the readout of the first positions, a sum of one or
            # two terms that the head's norm rescales, then has a sign that rounding cannot turn)
            mat(p + "mix.k", kw, W)
            put(p + "mix.q", 2.0 * w[p + "mix.k"] + torch.randn(kw, W, generator=g) * W ** -0.5)
            mat(p + "mix.v", vw, W)
            mat(p + "mix.g", vw, W)
            mat(p + "mix.o", W, vw)
            put(p + "mix.norm", 1.0 + 0.2 * torch.randn(m["vdim"], generator=g))
            mat(p + "mix.a1", rank, W)
            mat(p + "mix.a2", kw, rank, 2.0)
            put(p + "mix.a2.b", 2.0 + 2.0 * torch.randn(kw, generator=g))
        else:
            mat(p + "mix.q", m["heads"] * m["dim"], W)
            mat(p + "mix.k", m["kv_heads"] * m["dim"], W)
            mat(p + "mix.v", m["kv_heads"] * m["vdim"], W)
            mat(p + "mix.o", W, m["heads"] * m["vdim"])
        if L["mlp"] is not None:
            put(p + "norm2", 0.2 * torch.randn(W, generator=g))
            ff = L["mlp"]["expert"]["ff"]
            mat(p + "mlp.router", L["mlp"]["router"]["experts"], W, 2.0)
            for e in range(L["mlp"]["router"]["experts"]):
                mat(p + f"mlp.e{e}.gate", ff, W, 2.0)
                mat(p + f"mlp.e{e}.up", ff, W, 2.0)
                mat(p + f"mlp.e{e}.down", W, ff)
    put("final.norm", 0.2 * torch.randn(W, generator=g))
    mat("head", cfg["vocab"], W)
    return w


def write_folder(folder, cfg, weights) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=1))
    save_file({n: t.to(torch.bfloat16).contiguous() for n, t in weights.items()}, str(folder / "model.safetensors"))
    return folder


def oracle_logits(cfg, weights, tokens):
    return plain.PlainGubanex(cfg, weights, torch.float64).forward(list(tokens)).float().numpy()


def oracle_with_margins(cfg, weights, tokens):
    """(logits, per position the narrowest choice of experts in any layer call)."""
    model = plain.PlainGubanex(cfg, weights, torch.float64)
    return model.forward(list(tokens)).float().numpy(), list(model.margins)


def every_expert(cfg):
    """The same model with every expert chosen for every token: no choice that rounding could turn."""
    out = json.loads(json.dumps(cfg))
    for layer in out["layers"]:
        if layer["mlp"] is not None:
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return out


def tokens(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()
