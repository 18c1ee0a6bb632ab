"""Test-side helpers for the Rorosun design: small ``config.json`` dicts written by hand,
random weights under the design's tensor names (listed here independently of the engine),
model folders, and the engine's step function driven by a list of steps."""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import save_file

import plain_rorosun as plain


def layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, pool=4, scale=None, r_heads=2, r_dim=16, ff=96,
          left_scale=0.7, right_scale=0.4):
    return {
        "type": "parallel",
        "mixer": {
            "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                     "scale": float(dim) ** -0.5 if scale is None else scale, "mask": {"size": window, "pool": pool}},
            "right": {"heads": r_heads, "dim": r_dim},
            "left_scale": left_scale, "right_scale": right_scale,
        },
        "mlp": None if ff is None else {"kind": "dense", "ff": ff},
    }


def model_json(layers, vocab=200, width=64, eps=1e-5):
    return {"architecture": "Rorosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}


def random_weights(cfg, seed, rank=8):
    """name -> float32 tensor holding bfloat16-representable values."""
    g = torch.Generator().manual_seed(seed)
    w = {}

    def put(name, t):
        w[name] = t.to(torch.bfloat16).float()

    def mat(name, out, inp, gain=1.0):
        put(name, torch.randn(out, inp, generator=g) * gain * inp ** -0.5)

    def vec(name, n, mean=0.0, std=1.0):
        put(name, mean + std * torch.randn(n, generator=g))

    W = cfg["width"]
    put("embed", torch.randn(cfg["vocab"], W, generator=g))
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        a, b = L["mixer"]["left"], L["mixer"]["right"]
        put(p + "norm1", 1.0 + 0.2 * torch.randn((), generator=g))
        qw, kw, vw = a["heads"] * a["dim"], a["kv_heads"] * a["dim"], a["kv_heads"] * a["vdim"]
        mat(p + "mix.left.q", qw, W, 2.0)
        mat(p + "mix.left.k", kw, W, 2.0)
        mat(p + "mix.left.v", vw, W)
        vec(p + "mix.left.q.b", qw, std=0.3)
        vec(p + "mix.left.k.b", kw, std=0.3)
        vec(p + "mix.left.v.b", vw, std=0.3)
        vec(p + "mix.left.q.norm", qw, 1.0, 0.2)
        vec(p + "mix.left.k.norm", kw, 1.0, 0.2)
        put(p + "mix.left.talk", torch.eye(a["heads"]) + 0.3 * torch.randn(a["heads"], a["heads"], generator=g))
        mat(p + "mix.left.o", W, a["heads"] * a["vdim"])
        hd = b["heads"] * b["dim"]
        for s in "rkvgw":
            put(p + "mix.right.mu." + s, torch.rand(W, generator=g))
        for s in "rkvg":
            mat(p + "mix.right." + s, hd, W)
        mat(p + "mix.right.w1", rank, W)
        mat(p + "mix.right.w2", hd, rank)
        put(p + "mix.right.w0", -4.0 * torch.rand(hd, generator=g))      # decays between 0.37 and 0.98
        put(p + "mix.right.u", 0.5 * torch.randn(b["heads"], b["dim"], generator=g))
        vec(p + "mix.right.norm", hd, 1.0, 0.2)
        mat(p + "mix.right.o", W, hd)
        vec(p + "ls1", W, 1.0, 0.3)
        if L["mlp"] is not None:
            put(p + "norm2", 1.0 + 0.2 * torch.randn((), generator=g))
            mat(p + "mlp.gate", L["mlp"]["ff"], W)
            mat(p + "mlp.up", L["mlp"]["ff"], W)
            mat(p + "mlp.down", W, L["mlp"]["ff"])
            vec(p + "ls2", W, 1.0, 0.3)
    put("final.norm", 1.0 + 0.2 * torch.randn((), generator=g))
    mat("head", cfg["vocab"], W)
    return w


def write_folder(folder, cfg, weights) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=1))
    save_file({n: t.to(torch.bfloat16).contiguous() for n, t in weights.items()}, str(folder / "model.safetensors"))
    return folder


def oracle_logits(cfg, weights, tokens, cache_dtype=None):
    w = {n: t.double() for n, t in weights.items()}
    return plain.logits(tokens, cfg, w, cache_dtype).float().numpy()


def tokens(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_steps(runner, steps):
    """Feed a list of steps ({"step", "entries": [{"id", "tokens", "want"}], "end"}) through
    ``ModelRunner.step``; {step: float32 [wanted, vocab]}."""
    from tokamak_amd.engine.runner import StepEntry

    got = {}
    for rec in steps:
        entries = [StepEntry(e["id"], list(e["tokens"]), list(e.get("want", []))) for e in rec["entries"]]
        logits = runner.step(entries)
        if logits.shape[0]:
            got[rec["step"]] = logits.float().cpu().numpy()
        for rid in rec.get("end", []):
            runner.end(rid)
    return got


def worst_error(steps, got, expected):
    """Largest |difference| relative to the largest |logit| of the row, over every wanted row;
    with the place it was found."""
    cursor = {rid: 0 for rid in expected}
    worst, where = 0.0, None
    for rec in steps:
        row = 0
        for e in rec["entries"]:
            start = cursor[e["id"]]
            for w in e.get("want", []):
                want = expected[e["id"]][start + w]
                err = float(np.abs(got[rec["step"]][row] - want).max() / max(1e-6, np.abs(want).max()))
                if not err <= worst:
                    worst, where = err, (rec["step"], e["id"], start + w, len(e["tokens"]))
                row += 1
            cursor[e["id"]] = start + len(e["tokens"])
    return worst, where


LIMIT = {"float32": 2e-4, "bfloat16": 6e-2}
