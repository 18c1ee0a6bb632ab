"""The Gubanex design in the engine against the plain implementation (plain_gubanex.py):
each mechanism alone, then whole models of several small shapes through the step function:
whole prompts, tails one by one, portions down to two tokens, mixed batches with pages and
state slots used again, chunk edges with sharp attention, a far key among hundreds, long
decoding through recorded steps, greedy generation through ``LLM.generate``, and the trace
runner.

float32 runs compare every row.  In bfloat16 a choice between two experts whose scores lie within
rounding of each other may fall the other way than in the plain implementation, and what follows
in that sequence then differs by more than rounding; so a bfloat16 run compares a request's rows
up to the first position where the plain implementation's choice was that narrow, and every row
of the same models with all experts chosen for every token (``every_expert``).  The choice itself
is compared in bfloat16 where both sides see the same input (``test_routed_experts_alone``)."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_gubanex as plain
from gubanex_util import (attention, every_expert, experts, gla, model_json, oracle_logits, oracle_with_margins,
                          random_weights, tokens, write_folder)
from kernel_util import make_batch
from replay_util import mixed, portions, tail_one_by_one, whole
from rorosun_util import run_steps

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = Path(__file__).resolve().parent.parent
REL = {torch.float32: 3e-5, torch.bfloat16: 2.5e-2}
# (bfloat16: models 40 to 72 wide average little rounding away; float32 is the sharp comparison)
LIMIT = {"float32": 2e-4, "bfloat16": 1e-1}
NARROW = 0.1       # a choice of experts that bfloat16 rounding may turn (relative distance of the logits)


def close(got, want, dtype):
    """Largest difference against the largest value of the expected tensor."""
    err = float((got - want).abs().max() / want.abs().max())
    assert err <= REL[dtype], err


def row_errors(steps, got, expected):
    """[(error relative to the row's largest logit, where)] of every wanted row."""
    cursor = {rid: 0 for rid in expected}
    out = []
    for rec in steps:
        row = 0
        for e in rec["entries"]:
            start = cursor[e["id"]]
            for w in e.get("want", []):
                want = expected[e["id"]][start + w]
                err = float(np.abs(got[rec["step"]][row] - want).max() / max(1e-6, np.abs(want).max()))
                out.append((err if err == err else float("inf"), (rec["step"], e["id"], start + w, len(e["tokens"]))))
                row += 1
            cursor[e["id"]] = start + len(e["tokens"])
    return out


def check_rows(steps, got, expected, dtype, what="", margins=None):
    """Every wanted row; in bfloat16 with ``margins`` (request -> per position) only the rows before
    a request's first narrow choice of experts."""
    errors = row_errors(steps, got, expected)
    if dtype == "bfloat16" and margins is not None:
        sure = {rid: next((i for i, m in enumerate(ms) if m < NARROW), len(ms)) for rid, ms in margins.items()}
        errors = [(e, where) for e, where in errors if where[2] < sure[where[1]]]
    over = [(e, where) for e, where in errors if not e <= LIMIT[dtype]]
    assert not over, (what, dtype, len(over), len(errors), sorted(over)[-1])
    return len(errors)


def fetcher(tensors, dtype):
    def fetch(name):
        t = tensors[name]
        held = dtype if t.dim() == 2 and not name.endswith("router") else torch.float32
        return t.to(DEV, held).contiguous()
    return fetch


def double(w):
    return {k: v.double() for k, v in w.items()}


def summed(out):
    return (out.sum(0) if out.dim() == 3 else out).float().cpu()


# -- mechanisms alone -------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_offset_norm_scaled_embedding_and_capped_head(dtype):
    from tokamak_amd.config import get_part

    g = torch.Generator().manual_seed(0)
    stored = (0.3 * torch.randn(72, generator=g)).to(torch.bfloat16).float()
    norm = get_part("norm", "rmsnorm")(dim=72, eps=1e-4, tensor="", offset=1.0, dtype=dtype, device=DEV)
    norm.bind("n", lambda name: stored.to(DEV))
    resid, delta = torch.randn(5, 72, generator=g) * 3, torch.randn(5, 72, generator=g)
    r = resid.to(DEV)
    h = norm.forward(r, delta.to(DEV))
    want = plain.offset_norm((resid + delta).double(), stored.double(), 1e-4).float()
    close(h.cpu().float(), want, dtype)

    table = torch.randn(30, 72, generator=g).to(torch.bfloat16).float()
    emb = get_part("embedding", "token_embedding")(vocab_size=30, dim=72, tensor="", scale=7.5, dtype=dtype, device=DEV)
    emb.bind("embed", lambda name: table.to(DEV, dtype))
    batch = make_batch([(4, 0, [0])])
    ids = torch.tensor([3, 29, 0, 3], dtype=torch.int32)
    batch.token_ids.copy_(ids)
    x = emb.forward(batch)
    torch.testing.assert_close(x.cpu(), table[ids.long()] * 7.5, rtol=0, atol=0)
    emb.add_to(batch, x)                       # the input fed in once more
    torch.testing.assert_close(x.cpu(), table[ids.long()] * 15.0, rtol=0, atol=0)

    weight = (torch.randn(50, 72, generator=g) * 0.5).to(torch.bfloat16).float()
    head = get_part("head", "linear_head")(vocab_size=50, dim=72, tied=False, tensor="", scale=3.0, softcap=4.0,
                                           dtype=dtype, device=DEV)
    head.bind("head", lambda name: weight.to(DEV, dtype))
    hidden = torch.randn(6, 72, generator=g).to(dtype)
    got = head.forward(hidden.to(DEV)).cpu()
    want = 4.0 * torch.tanh(hidden.double() @ weight.double().T * 3.0 / 4.0)
    assert float(want.abs().max()) > 3.9        # the cap bites
    torch.testing.assert_close(got, want.float(), rtol=1e-4, atol=1e-4)
    plain_head = get_part("head", "linear_head")(vocab_size=50, dim=72, tied=False, tensor="", dtype=dtype, device=DEV)
    plain_head.bind("head", lambda name: weight.to(DEV, dtype))
    torch.testing.assert_close(plain_head.forward(hidden.to(DEV)).cpu(), (hidden.double() @ weight.double().T).float(),
                               rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("heads,dim,vdim,rank", [(2, 16, 16, 8), (3, 8, 24, 5), (1, 64, 32, 16), (2, 130, 20, 7), (2, 12, 200, 8)])
def test_gated_linear_attention_alone_in_portions_and_slots(dtype, heads, dim, vdim, rank):
    """Two sequences in unlike portions (one of a single token, one that starts later), state slots
    that are not in request order; against the plain recurrence over the whole sequences."""
    from tokamak_amd.config import get_part
    from tokamak_amd.engine.storage import SlotStore

    width, eps, tau = 48, 1e-5, 5.0
    cfg = model_json([gla(heads=heads, dim=dim, vdim=vdim, tau=tau)], width=width, eps=eps)
    w = random_weights(cfg, seed=dim + vdim, rank=rank)
    part = get_part("mixer", "gated_linear_attention")(hidden_size=width, num_heads=heads, head_dim=dim, value_dim=vdim,
                                                       tau=tau, norm_eps=eps, dtype=dtype, device=DEV)
    assert set(part.expected_tensors("l0.mix.")) == {n for n in w if n.startswith("l0.mix.")}
    part.bind("l0.mix.", fetcher(w, dtype))
    g = torch.Generator().manual_seed(1)
    seqs = [torch.randn(n, width, generator=g).to(dtype) for n in (23, 9)]
    want = [plain.gated_linear_attention(s.double(), double(w), "l0.mix.", cfg["layers"][0]["mixer"], eps)[0].float() for s in seqs]
    state = {n: torch.zeros((4, *a.shape), dtype=a.dtype, device=DEV) for n, a in part.state_request().items()}
    state["S"][1].fill_(7.0)             # another request's slot: must stay as it is
    store = SlotStore(0, 16, {}, state)
    slots = [2, 0]
    cuts = [[(0, 10), (10, 11), (11, 19), (19, 23)], [None, (0, 2), (2, 3), (3, 9)]]
    got = [[], []]
    for step in range(4):
        spans, rows = [], []
        for r in (0, 1):
            if cuts[r][step] is not None:
                lo, hi = cuts[r][step]
                spans.append((hi - lo, lo, [0]))
                rows.append((r, lo, hi))
        batch = make_batch(spans)
        batch.state_slots.copy_(torch.tensor([slots[r] for r, _, _ in rows], dtype=torch.int32))
        out = summed(part.forward(torch.cat([seqs[r][lo:hi] for r, lo, hi in rows]).to(DEV), batch, store))
        at = 0
        for r, lo, hi in rows:
            got[r].append(out[at:at + hi - lo])
            at += hi - lo
    for r in (0, 1):
        close(torch.cat(got[r]), want[r], dtype)
    assert float(state["S"][1].min()) == 7.0 and float(state["S"][3].abs().max()) == 0.0
    final = plain.gated_linear_attention(seqs[0].double(), double(w), "l0.mix.", cfg["layers"][0]["mixer"], eps)[1].float()
    close(state["S"][2].cpu(), final, dtype)
    # a long portion (a head's value columns are then shared by several blocks where there are 16 and
    # more), two tokens and single tokens after it, in the slot that another request has left
    from tokamak_amd.kernels import ops
    long = torch.randn(140, width, generator=g).to(dtype)
    assert (ops.gla_column_splits(1, heads, vdim, 120) > 1) == (vdim >= 16)
    want = plain.gated_linear_attention(long.double(), double(w), "l0.mix.", cfg["layers"][0]["mixer"], eps)[0].float()
    state["S"][2].zero_()
    got, at = [], 0
    for count in (120, 2, 1, 16, 1):
        batch = make_batch([(count, at, [0])])
        batch.state_slots.copy_(torch.tensor([2], dtype=torch.int32))
        got.append(summed(part.forward(long[at:at + count].to(DEV), batch, store)))
        at += count
    close(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("a", [dict(heads=4, kv_heads=2, dim=16, vdim=16, chunk=12, rot=8),
                               dict(heads=3, kv_heads=1, dim=24, vdim=48, chunk=5, rot=24, scaling=(4.0, 1.0, 2.0, 16.0)),
                               dict(heads=2, kv_heads=2, dim=40, vdim=16, chunk=33, rot=0),
                               dict(heads=8, kv_heads=2, dim=128, vdim=128, chunk=16, rot=64, base=1e5),
                               dict(heads=2, kv_heads=1, dim=64, vdim=64, chunk=None, rot=32),
                               dict(heads=2, kv_heads=1, dim=16, vdim=16, chunk=1, rot=2),
                               dict(heads=4, kv_heads=1, dim=64, vdim=64, chunk=50, rot=64),
                               dict(heads=3, kv_heads=1, dim=20, vdim=36, chunk=9, rot=10),
                               dict(heads=2, kv_heads=2, dim=6, vdim=2, chunk=14, rot=6)],
                         ids=["g2", "g3", "g1", "wide", "full", "one", "mid", "pad", "tiny"])
def test_chunked_attention_alone(dtype, a):
    """A portion from position zero, one that ends inside a page and inside a chunk, two tokens, then
    single tokens; the request's pages scattered; the position that starts a chunk given a key that
    every later query prefers, so a chunk cut one position early or late shows."""
    from tokamak_amd.config import get_part
    from tokamak_amd.engine.storage import SlotStore

    width, eps = 64, 1e-5
    page = 16 if a["dim"] >= 64 else 8       # (heads of 64 and 128 with pages of 16: the matrix-core kernel for portions in bfloat16)
    cfg = model_json([attention(**a)], width=width, eps=eps)
    m = cfg["layers"][0]["mixer"]
    w = random_weights(cfg, seed=a["dim"])
    part = get_part("mixer", "rotated_unit_attention")(
        hidden_size=width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
        softmax_scale=m["scale"], norm_eps=eps, chunk=a["chunk"], dtype=dtype, device=DEV)
    assert set(part.expected_tensors("l0.mix.")) == {n for n in w if n.startswith("l0.mix.")}
    part.bind("l0.mix.", fetcher(w, dtype))
    position = None
    if a["rot"]:
        rot = m["rot"]
        scaling = rot.get("scaling")
        position = get_part("position", "rotary_half")(
            rotary_dim=rot["dims"], theta=rot["base"], dtype=dtype, device=DEV,
            scaling=None if scaling is None else tuple(scaling[k] for k in ("factor", "low", "high", "original")))
    T = 150
    g = torch.Generator().manual_seed(2)
    h = torch.randn(T, width, generator=g).to(dtype)
    want = plain.chunked_attention(h.double(), double(w), "l0.mix.", m, eps)[0].float()
    if a["chunk"] not in (None, 1):
        # the mask matters: a chunk one position longer changes the output by far more than the tolerance
        other = dict(m, mask={"size": a["chunk"] + 1})
        near = plain.chunked_attention(h.double(), double(w), "l0.mix.", other, eps)[0].float()
        assert float((near - want).abs().max() / want.abs().max()) > 0.02
    pages = 40
    # (what no token has written must not be read: NaN there; but sizes that do not fill the pages' pieces are
    # padded with the zeros that the engine's pages start with)
    padded = (part.key_size, part.value_size) != (m["dim"], m["vdim"])
    assert padded == (a["dim"] % 8 != 0 or a["vdim"] % 16 != 0)
    store = SlotStore(0, page, {name: torch.full((pages, array.elems_per_token * page), 0.0 if padded else float("nan"),
                                                 dtype=dtype, device=DEV)
                                for name, array in part.cache_request().arrays})
    table = [(7 * i + 3) % pages for i in range(-(-T // page))]
    got, at = [], 0
    for n in [37, 30, 2] + [1] * (T - 69):
        batch = make_batch([(n, at, table)])
        data = None if position is None else position.prepare(batch)
        got.append(summed(part.forward(h[at:at + n].to(DEV), batch, store, True, data)))
        at += n
    close(torch.cat(got), want, dtype)


def clear_of(h, w, top, n):
    """The rows whose choice of experts is no close call."""
    scores = torch.sigmoid(h.double() @ w["l0.mlp.router"].double().T).sort(dim=1, descending=True).values
    return torch.ones(h.shape[0], dtype=torch.bool) if top == n else (scores[:, top - 1] - scores[:, top]) > 1e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("width,ff,n,top", [(64, 32, 4, 2), (48, 24, 12, 1), (72, 40, 5, 5), (36, 20, 7, 3), (256, 136, 3, 2),
                                            (128, 192, 2, 1)])
def test_routed_experts_alone(dtype, width, ff, n, top):
    """Numbers of experts that are no power of two, one expert a token, every expert a token, sizes
    that do not fill 16-byte pieces; the rows whose choice of experts is no close call are compared."""
    from tokamak_amd.config import get_part

    cfg = model_json([gla(mlp=experts(n, top, ff))], width=width)
    w = random_weights(cfg, seed=width + n)
    part = get_part("feed_forward", "routed_experts")(hidden_size=width, intermediate_size=ff, num_experts=n, top=top,
                                                      weight_on="input", dtype=dtype, device=DEV)
    assert set(part.expected_tensors("l0.mlp.")) == {k for k in w if k.startswith("l0.mlp.")}
    part.bind("l0.mlp.", fetcher(w, dtype))
    g = torch.Generator().manual_seed(3)
    rows = 70 if n > 2 else 500         # (two experts and 500 tokens, K in chunks of 64: full tiles, their activations through LDS)
    h = torch.randn(rows, width, generator=g).to(dtype)
    want = plain.routed_experts(h.double(), double(w), "l0.mlp.", cfg["layers"][0]["mlp"]).float()
    got = part.forward(h.to(DEV), make_batch([(rows, 0, [0])]))
    assert got.dtype == torch.float32 and got.shape == (top, rows, width)      # a layer per chosen expert, added by the reader
    got = got.sum(0).cpu()
    few = part.forward(h[:9].to(DEV), make_batch([(9, 0, [0])])).sum(0).cpu()   # the form for few tokens
    close(few[clear_of(h[:9], w, top, n)], want[:9][clear_of(h[:9], w, top, n)], dtype)
    clear = clear_of(h, w, top, n)
    assert int(clear.sum()) >= 0.85 * rows
    close(got[clear], want[clear], dtype)
    # the weight acts on the expert's input: it is not the same as weighting the output
    one = plain.routed_experts(h[:1].double(), double(w), "l0.mlp.", cfg["layers"][0]["mlp"])
    assert float(one.abs().max()) > 0


# -- whole models -------------------------------------------------------------------
# Shapes that differ in everything: groups of 2, 1 and 3 query heads a kv head; key and value sizes
# that differ, also ones that fill no 16-byte piece; chunks that do not divide a page, a chunk of one, no chunks; rotation of a part, of
# the whole and of nothing; one expert a token, several, all; layers without a feed-forward; a loop
# over the middle, over everything, none; two layers of one kind in a row.
SHAPES = {
    "base": dict(cfg=model_json([gla(), attention(), gla(heads=4, dim=8, vdim=16), attention(chunk=9, rot=16)],
                                loop=(1, 3, 2)), rank=8, page=16),
    "odd": dict(cfg=model_json([attention(heads=3, kv_heads=3, dim=20, vdim=40, chunk=7, rot=12, scaling=(4.0, 1.0, 2.0, 16.0),
                                          mlp=experts(5, 1, 24)),
                                attention(heads=6, kv_heads=2, dim=8, vdim=16, chunk=20, rot=8, mlp=None),
                                gla(heads=3, dim=20, vdim=12, tau=3.0, mlp=experts(3, 3, 40))],
                               vocab=131, width=72, eps=1e-6, loop=(0, 3, 3), embedding_scale=1.0, logit_scale=1.0, softcap=9.0),
                rank=5, page=8),
    "ones": dict(cfg=model_json([gla(heads=1, dim=64, vdim=8, tau=1.0, mlp=None),
                                 attention(heads=5, kv_heads=1, dim=8, vdim=16, chunk=1, rot=2, mlp=experts(7, 2, 16)),
                                 attention(heads=2, kv_heads=1, dim=64, vdim=32, chunk=None, rot=0, mlp=experts(2, 1, 48))],
                                vocab=97, width=40, eps=1e-4, loop=None, softcap=None), rank=6, page=16),
}
SHAPES["ones"]["cfg"].pop("logit_softcap")


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("gubanex")
    out = {}
    for name, spec in SHAPES.items():
        w = random_weights(spec["cfg"], seed=len(name), rank=spec["rank"])
        out[name] = (write_folder(root / name, spec["cfg"], w), spec["cfg"], w, spec["page"])
        all_cfg = every_expert(spec["cfg"])
        out[name + "-all"] = (write_folder(root / (name + "-all"), all_cfg, w), all_cfg, w, spec["page"])
    return out


def runner_for(models, name, dtype, pool_tokens=1024, max_requests=4, **kw):
    from tokamak_amd.engine.runner import ModelRunner

    folder, cfg, w, page = models[name]
    return ModelRunner.from_folder(folder, dtype=dtype, page_size=page, kv_pool_tokens=pool_tokens,
                                   max_requests=max_requests, **kw), cfg, w


LENGTHS = [1, 2, 23, 61, 150]


def requests_for(cfg, seed=0):
    return {f"r{i}": tokens(cfg["vocab"], n, 100 * seed + i) for i, n in enumerate(LENGTHS)}


def expected_for(cfg, w, requests):
    return {rid: oracle_logits(cfg, w, toks) for rid, toks in requests.items()}


def expected_and_margins(cfg, w, requests):
    both = {rid: oracle_with_margins(cfg, w, toks) for rid, toks in requests.items()}
    return {rid: b[0] for rid, b in both.items()}, {rid: b[1] for rid, b in both.items()}


@pytest.fixture(scope="module")
def oracle(models):
    """Plain logits of every shape's requests, computed once."""
    out = {}
    for name, (folder, cfg, w, page) in models.items():
        for seed in (0, 1):
            requests = requests_for(cfg, seed)
            if seed == 1:
                requests.update({f"s{i}": tokens(cfg["vocab"], n, 900 + i) for i, n in enumerate([40, 64, 17])})
            out[name, seed] = (requests, *expected_and_margins(cfg, w, requests))
    return out


ALL_SHAPES = [n + tail for n in SHAPES for tail in ("", "-all")]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ALL_SHAPES)
def test_every_cutting(models, oracle, name, dtype):
    """Whole prompts; most of a prompt and its tail token by token (prefill against decoding
    through the cache and the state); portions of 16 down to 2 tokens."""
    runner, cfg, w = runner_for(models, name, dtype)
    requests, expected, margins = oracle[name, 0]
    checked = 0
    for steps in [whole(requests)] + [f(rid, toks) for rid, toks in requests.items() for f in (tail_one_by_one, portions)]:
        checked += check_rows(steps, run_steps(runner, steps), expected, dtype, name, margins)
    assert checked >= (3 * sum(LENGTHS) if name.endswith("-all") or dtype == "float32" else 3)
    runner.manager.check()
    assert runner.manager.num_free_pages() == runner.manager.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ALL_SHAPES)
def test_mixed_batches_with_pages_and_slots_used_again(models, oracle, name, dtype):
    """Up to four live requests, portions beside single tokens, requests left out of steps;
    eight requests over four state slots and a pool that only holds what is live."""
    requests, expected, margins = oracle[name, 1]
    steps, peak = mixed(requests, seed=5)
    assert max(len(s["entries"]) for s in steps) >= 3
    runner, _, _ = runner_for(models, name, dtype, pool_tokens=peak, max_requests=4)
    check_rows(steps, run_steps(runner, steps), expected, dtype, name, margins)
    runner.manager.check()
    # a request in a batch computes what it computes alone, beyond rounding
    alone = whole({"r4": requests["r4"]})
    check_rows(alone, run_steps(runner, alone), expected, dtype, name, margins)


def test_chunk_edges_and_a_far_key_show(tmp_path):
    """Attention so sharp (scores times eight) that a key one position inside or outside a chunk moves
    the logits by far more than the tolerance, in a prompt, in portions and in decoding; chunks
    longer than several pages, so that a chunk's first key lies hundreds of positions back."""
    from tokamak_amd.engine.runner import ModelRunner

    cfg = model_json([attention(chunk=11, scale=2.0, mlp=None), attention(heads=2, kv_heads=1, chunk=200, rot=16, scale=2.0),
                      gla()], width=64)
    w = random_weights(cfg, seed=3)
    folder = write_folder(tmp_path / "sharp", cfg, w)
    toks = tokens(cfg["vocab"], 450, 7)
    expected = {"x": oracle_logits(cfg, w, toks)}
    for layer, size in ((0, 12), (0, 10), (1, 201), (1, 199)):
        other = json.loads(json.dumps(cfg))
        other["layers"][layer]["mixer"]["mask"]["size"] = size
        assert np.abs(oracle_logits(other, w, toks) - expected["x"]).max() > 0.1
    runner = ModelRunner.from_folder(folder, dtype="float32", page_size=16, kv_pool_tokens=512, max_requests=2)
    for steps in (whole({"x": toks}), tail_one_by_one("x", toks, tail=64), portions("x", toks)):
        check_rows(steps, run_steps(runner, steps), expected, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(models, dtype):
    """One prompt token, then 260 tokens one by one (the recorded step of each shape replayed
    many times, two requests side by side at different lengths); and the same without recorded
    steps and without recorded layers gives the same bits."""
    shape = "base" if dtype == "float32" else "base-all"
    runner, cfg, w = runner_for(models, shape, dtype)
    assert runner.use_graphs
    a, b = tokens(cfg["vocab"], 261, 11), tokens(cfg["vocab"], 200, 12)
    expected = expected_for(cfg, w, {"a": a, "b": b})
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:1], "want": [0]}], "end": []}]
    for i in range(1, 261):
        entries = [{"id": "a", "tokens": [a[i]], "want": [0]}]
        if i >= 61:
            entries.append({"id": "b", "tokens": [b[i - 61]], "want": [0]})
        steps.append({"step": i, "entries": entries, "end": []})
    got = run_steps(runner, steps)
    check_rows(steps, got, expected, dtype)
    plain_runner, _, _ = runner_for(models, shape, dtype, use_graphs=False)
    plain_runner.model.replay_layers = False
    again = run_steps(plain_runner, steps)
    for step in got:
        assert np.array_equal(got[step], again[step]), step


def test_greedy_generation_through_the_entry_point(models):
    """``LLM.generate``: scheduler, portions of prompts, batched decoding, greedy sampling; a
    pool so tight that requests are evicted and computed again (their state slots too)."""
    from tokamak_amd import LLM, SamplingParams

    folder, cfg, w, page = models["base"]
    prompts = [tokens(cfg["vocab"], n, 40 + n) for n in (3, 30, 17, 9, 1)]
    new = 14

    def greedy(prompt):
        ids = list(prompt)
        for _ in range(new):
            ids.append(int(np.argmax(oracle_logits(cfg, w, ids)[-1])))
        return ids[len(prompt):]

    want = [greedy(p) for p in prompts]
    params = SamplingParams(temperature=0.0, max_new_tokens=new)
    for kwargs in (dict(kv_pool_tokens=512), dict(kv_pool_tokens=64, prefill_chunk=8, max_batch_size=3)):
        llm = LLM(folder, dtype="float32", max_seq_len=64, block_size=page, **kwargs)
        out = llm.generate(prompt_token_ids=prompts, sampling_params=params)
        assert [o.output_token_ids for o in out] == want, kwargs


def test_trace_runner_and_command_line(models, tmp_path):
    from test_gpu_rorosun import run_trace_any

    folder, cfg, w, page = models["odd"]
    requests = {f"r{i}": tokens(cfg["vocab"], n, 300 + i) for i, n in enumerate([5, 33, 70, 12, 41])}
    steps, peak = mixed(requests, seed=2)
    expected = expected_for(cfg, w, requests)
    got = run_trace_any(folder, "float32", steps, peak, tmp_path / "out", page, cfg["vocab"])
    check_rows(steps, got, expected, "float32")
    done = subprocess.run([sys.executable, "-m", "tokamak_amd.cli", "--model", str(folder), "--prompt-ids", "5,6,7",
                           "--max-new-tokens", "4", "--dtype", "float32", "--temperature", "0", "--max-seq-len", "64",
                           "--page-size", str(page), "--quiet"], cwd=ROOT, capture_output=True,
                          text=True, timeout=240)
    assert done.returncode == 0, done.stderr[-2000:]
    ids = [5, 6, 7]
    for _ in range(4):
        ids.append(int(np.argmax(oracle_logits(cfg, w, ids)[-1])))
    assert ",".join(map(str, ids[3:])) in done.stdout.replace(" ", ""), done.stdout
    done = subprocess.run([sys.executable, "-m", "tokamak_amd.cli", "--random-weights", "gubanex-tiny", "--prompt-ids",
                           "1,2,3", "--max-new-tokens", "3", "--quiet"], cwd=ROOT, capture_output=True, text=True, timeout=240)
    assert done.returncode == 0, done.stderr[-2000:]
