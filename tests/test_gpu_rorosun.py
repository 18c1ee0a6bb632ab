"""The Rorosun design in the engine against the plain implementation (plain_rorosun.py):
each mechanism alone, then whole models of several small shapes through the step function:
whole prompts, tails one by one, portions down to two tokens, mixed batches with pages and
state slots used again, window and pool edges with sharp attention, long decoding through
recorded steps, greedy generation through ``LLM.generate``, and the trace runner."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_rorosun as plain
from kernel_util import make_batch
from replay_util import mixed, portions, tail_one_by_one, whole
from rorosun_util import (LIMIT, layer, model_json, oracle_logits, random_weights, run_steps, tokens, worst_error,
                          write_folder)

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = Path(__file__).resolve().parent.parent
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {torch.float32: dict(rtol=2e-4, atol=2e-5), torch.bfloat16: dict(rtol=4e-2, atol=4e-2)}

REL = {torch.float32: 3e-5, torch.bfloat16: 2.5e-2}


def close(got, want, dtype):
    """Largest difference against the largest value of the expected tensor."""
    err = float((got - want).abs().max() / want.abs().max())
    assert err <= REL[dtype], err


# Shapes that differ in everything: groups of 2, 1 and 5 query heads a kv head; key and value
# sizes that differ; pools that do not divide a page, a pool of one, a pool longer than the
# window, a window of one; one layer without a feed-forward; layers of unlike sizes in one
# model; widths and ranks that are no multiple of 8.
SHAPES = {
    "base": dict(cfg=model_json([layer(), layer(window=9, pool=5, r_heads=4, r_dim=8)]), rank=8, page=16),
    "odd": dict(cfg=model_json([layer(heads=3, kv_heads=3, dim=24, vdim=40, window=7, pool=3, r_heads=3, r_dim=20, ff=None),
                                layer(heads=6, kv_heads=2, dim=8, vdim=16, window=20, pool=2, r_heads=1, r_dim=48, ff=56)],
                               vocab=131, width=72, eps=1e-6), rank=5, page=8),
    "ones": dict(cfg=model_json([layer(heads=5, kv_heads=1, dim=8, vdim=8, window=1, pool=1, r_heads=1, r_dim=64, ff=40),
                                 layer(heads=2, kv_heads=1, dim=64, vdim=32, window=5, pool=16, r_heads=2, r_dim=33, ff=None)],
                                vocab=97, width=36, eps=1e-4), rank=6, page=16),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("rorosun")
    out = {}
    for name, spec in SHAPES.items():
        w = random_weights(spec["cfg"], seed=len(name), rank=spec["rank"])
        out[name] = (write_folder(root / name, spec["cfg"], w), spec["cfg"], w, spec["page"])
    return out


def runner_for(models, name, dtype, pool_tokens=1024, max_requests=4, **kw):
    from tokamak_amd.engine.runner import ModelRunner

    folder, cfg, w, page = models[name]
    return ModelRunner.from_folder(folder, dtype=dtype, page_size=page, kv_pool_tokens=pool_tokens,
                                   max_requests=max_requests, **kw), cfg, w


# -- mechanisms alone -------------------------------------------------------------
def fetcher(tensors, dtype):
    def fetch(name):
        t = tensors[name]
        return t.to(DEV, dtype if t.dim() == 2 and not name.endswith(("talk", ".u")) else torch.float32).contiguous()
    return fetch


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_scalar_norm_and_layer_scale(dtype):
    from tokamak_amd.config import get_part

    norm = get_part("norm", "scalar_rmsnorm")(dim=72, eps=1e-4, tensor="", dtype=dtype, device=DEV)
    assert {n: s.shape for n, s in norm.expected_tensors("l0.norm1").items()} == {"l0.norm1": ()}
    norm.bind("l0.norm1", lambda name: torch.tensor(1.25, device=DEV))
    g = torch.Generator().manual_seed(0)
    resid, delta = torch.randn(5, 72, generator=g) * 3, torch.randn(5, 72, generator=g)
    r = resid.to(DEV)
    h = norm.forward(r, delta.to(DEV))            # a float32 sub-layer output, as the layer scale leaves it
    torch.testing.assert_close(h.cpu().float(), plain.scalar_norm(resid + delta, 1.25, 1e-4), **TOL[dtype])
    torch.testing.assert_close(r.cpu(), resid + delta, rtol=0, atol=0)

    scale = get_part("scale", "layer_scale")(dim=72, tensor="", dtype=dtype, device=DEV)
    assert list(scale.expected_tensors("l0.ls1")) == ["l0.ls1"]
    ls = torch.rand(72, generator=g) + 0.5
    scale.bind("l0.ls1", lambda name: ls.to(DEV))
    a = torch.randn(5, 72, generator=g).to(dtype)
    b = torch.randn(3, 5, 72, generator=g)        # float32 partial sums of a split product
    got = scale.forward(a.to(DEV), 0.6, b.to(DEV), -0.5)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), ls * (0.6 * a.float() - 0.5 * b.sum(0)), rtol=1e-5, atol=1e-5)
    got = scale.forward(b.to(DEV))
    torch.testing.assert_close(got.cpu(), ls * b.sum(0), rtol=1e-5, atol=1e-5)


def time_mix_part(dtype, width, heads, dim, rank, eps, seed):
    from tokamak_amd.config import get_part

    cfg = model_json([layer(r_heads=heads, r_dim=dim)], width=width, eps=eps)
    w = random_weights(cfg, seed, rank=rank)
    part = get_part("mixer", "decayed_state_time_mix")(hidden_size=width, num_heads=heads, head_dim=dim, norm_eps=eps,
                                                       dtype=dtype, device=DEV)
    names = {n for n in w if n.startswith("l0.mix.right.")}
    assert set(part.expected_tensors("l0.mix.right.")) == names
    assert part.expected_tensors("l0.mix.right.")["l0.mix.right.w1"].shape == (None, width)   # the rank is the tensor's
    part.bind("l0.mix.right.", fetcher(w, dtype))
    return part, w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("heads,dim", [(2, 16), (3, 20), (1, 64), (2, 130)])
def test_time_mix_alone_in_portions_and_slots(dtype, heads, dim):
    """Two sequences in unlike portions (one of a single token, one that starts later), state
    slots that are not in request order; against the plain scan over the whole sequences."""
    from tokamak_amd.engine.storage import SlotStore

    width, eps = 48, 1e-5
    part, w = time_mix_part(dtype, width, heads, dim, 7, eps, seed=dim)
    g = torch.Generator().manual_seed(1)
    seqs = [torch.randn(n, width, generator=g).to(dtype) for n in (23, 9)]
    want = [plain.time_mix(s.double(), {k: v.double() for k, v in w.items()}, "l0.mix.right.",
                           {"heads": heads, "dim": dim}, eps).float() for s in seqs]
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
        h = torch.cat([seqs[r][lo:hi] for r, lo, hi in rows]).to(DEV)
        out = part.forward(h, batch, store)
        out = (out.sum(0) if out.dim() == 3 else out).float().cpu()
        at = 0
        for r, lo, hi in rows:
            got[r].append(out[at:at + hi - lo])
            at += hi - lo
    for r in (0, 1):
        close(torch.cat(got[r]), want[r], dtype)
    assert float(state["S"][1].min()) == 7.0 and float(state["S"][3].abs().max()) == 0.0
    torch.testing.assert_close(state["last"][2].cpu(), seqs[0][-1].float(), rtol=0, atol=0)


def attention_part(dtype, width, a, eps, seed):
    from tokamak_amd.config import get_part

    cfg = model_json([layer(**a)], width=width, eps=eps)
    left = cfg["layers"][0]["mixer"]["left"]
    w = random_weights(cfg, seed)
    part = get_part("mixer", "pooled_window_attention")(
        hidden_size=width, num_heads=left["heads"], num_kv_heads=left["kv_heads"], head_dim=left["dim"],
        value_dim=left["vdim"], window=left["mask"]["size"], pool=left["mask"]["pool"], softmax_scale=left["scale"],
        norm_eps=eps, dtype=dtype, device=DEV)
    assert set(part.expected_tensors("l0.mix.left.")) == {n for n in w if n.startswith("l0.mix.left.")}
    part.bind("l0.mix.left.", fetcher(w, dtype))
    return part, w, left


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("a", [dict(heads=4, kv_heads=2, dim=16, vdim=16, window=12, pool=4),
                               dict(heads=3, kv_heads=1, dim=24, vdim=8, window=5, pool=3),
                               dict(heads=2, kv_heads=2, dim=40, vdim=56, window=33, pool=7),
                               dict(heads=8, kv_heads=2, dim=128, vdim=128, window=16, pool=8)],
                         ids=["g2", "g3", "g1", "wide"])
def test_pooled_window_attention_alone(dtype, a):
    """A portion from position zero, a portion that ends inside a page, then single tokens; the
    request's pages scattered; one position's value made to stand out so that the steps in
    which it leaves the window, is hidden, and comes back inside a pooled block show in the output."""
    from tokamak_amd.engine.storage import SlotStore

    width, eps, page = 64, 1e-5, 8
    part, w, left = attention_part(dtype, width, a, eps, seed=a["dim"])
    T = 150
    g = torch.Generator().manual_seed(2)
    h = torch.randn(T, width, generator=g)
    h[4] *= 20.0                                      # position 4: a value far larger than the others
    h = h.to(dtype)
    want = plain.pooled_window_attention(h.double(), {k: v.double() for k, v in w.items()}, "l0.mix.left.", left, eps,
                                         cache_dtype=dtype).float()
    # the standing-out position matters: its leaving the window changes the output by far more than the tolerance
    near = plain.pooled_window_attention(h.double(), {k: v.double() for k, v in w.items()}, "l0.mix.left.",
                                         dict(left, mask={"size": a["window"] + 1, "pool": a["pool"]}), eps).float()
    assert float((near - want).abs().max() / want.abs().max()) > 0.02       # a thousand times the float32 tolerance
    pages = 40
    store = SlotStore(0, page, {
        "k": torch.full((pages, left["kv_heads"] * left["dim"] * page), float("nan"), dtype=dtype, device=DEV),
        "v": torch.full((pages, left["kv_heads"] * left["vdim"] * page), float("nan"), dtype=dtype, device=DEV),
        **{name: torch.full((pages, array.elems_per_token * page), float("nan"), dtype=array.dtype, device=DEV)
           for name, array in part.cache_request().arrays if name.endswith("_pool")}})
    table = [(7 * i + 3) % pages for i in range(-(-T // page))]
    assert len(set(table)) == len(table)
    got, at = [], 0
    for n in [37, 30, 2] + [1] * (T - 69):
        batch = make_batch([(n, at, table)])
        out = part.forward(h[at:at + n].to(DEV), batch, store)
        got.append((out.sum(0) if out.dim() == 3 else out).float().cpu())
        at += n
    close(torch.cat(got), want, dtype)


# -- whole models -------------------------------------------------------------------
LENGTHS = [1, 2, 23, 61, 150]


def requests_for(cfg, seed=0):
    return {f"r{i}": tokens(cfg["vocab"], n, 100 * seed + i) for i, n in enumerate(LENGTHS)}


def expected_for(cfg, w, requests, dtype="float32"):
    cache = torch.bfloat16 if dtype == "bfloat16" else None
    return {rid: oracle_logits(cfg, w, toks, cache) for rid, toks in requests.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_every_cutting(models, name, dtype):
    """Whole prompts; most of a prompt and its tail token by token (prefill against decoding
    through the cache and the state); portions of 16 down to 2 tokens."""
    runner, cfg, w = runner_for(models, name, dtype)
    requests = requests_for(cfg)
    expected = expected_for(cfg, w, requests, dtype)
    for steps in [whole(requests)] + [f(rid, toks) for rid, toks in requests.items() for f in (tail_one_by_one, portions)]:
        worst, where = worst_error(steps, run_steps(runner, steps), expected)
        assert worst <= LIMIT[dtype], (name, dtype, worst, where)
    runner.manager.check()
    assert runner.manager.num_free_pages() == runner.manager.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_mixed_batches_with_pages_and_slots_used_again(models, name, dtype):
    """Up to four live requests, portions beside single tokens, requests left out of steps;
    eight requests over four state slots and a pool that only holds what is live."""
    folder, cfg, w, page = models[name]
    requests = requests_for(cfg, seed=1)
    requests.update({f"s{i}": tokens(cfg["vocab"], n, 900 + i) for i, n in enumerate([40, 64, 17])})
    steps, peak = mixed(requests, seed=5)
    assert max(len(s["entries"]) for s in steps) >= 3
    runner, _, _ = runner_for(models, name, dtype, pool_tokens=peak, max_requests=4)
    expected = expected_for(cfg, w, requests, dtype)
    worst, where = worst_error(steps, run_steps(runner, steps), expected)
    assert worst <= LIMIT[dtype], (name, dtype, worst, where)
    runner.manager.check()
    # a request in a batch computes what it computes alone, beyond rounding
    alone = whole({"r4": requests["r4"]})
    worst, where = worst_error(alone, run_steps(runner, alone), expected)
    assert worst <= LIMIT[dtype], (name, dtype, worst, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_kernel_form_of_the_attention(models, dtype, monkeypatch):
    """The form for sizes the four-kernel form does not take (more than 16 query heads a kv
    head, more than 256 value channels), forced here on a small shape: every cutting, and a
    wide group for real."""
    from tokamak_amd.kernels import ops

    monkeypatch.setattr(ops, "POOLED_ONE_KERNEL_ONLY", True)
    runner, cfg, w = runner_for(models, "odd", dtype, use_graphs=False)
    requests = requests_for(cfg, seed=3)
    expected = expected_for(cfg, w, requests, dtype)
    for steps in (whole(requests), tail_one_by_one("r4", requests["r4"]), portions("r4", requests["r4"])):
        worst, where = worst_error(steps, run_steps(runner, steps), expected)
        assert worst <= LIMIT[dtype], (dtype, worst, where)
    monkeypatch.setattr(ops, "POOLED_ONE_KERNEL_ONLY", False)
    assert ops.pooled_split_plan(34, 2, 8, 8, 6, 3, 10, 10, 100) is None       # 17 heads a kv head


def test_a_group_of_seventeen_heads(tmp_path):
    from tokamak_amd.engine.runner import ModelRunner

    cfg = model_json([layer(heads=17, kv_heads=1, dim=8, vdim=8, window=6, pool=3)], vocab=50, width=40)
    w = random_weights(cfg, seed=9)
    folder = write_folder(tmp_path / "g17", cfg, w)
    toks = tokens(50, 70, 4)
    runner = ModelRunner.from_folder(folder, dtype="float32", page_size=16, kv_pool_tokens=128, max_requests=2)
    expected = {"x": oracle_logits(cfg, w, toks)}
    for steps in (whole({"x": toks}), tail_one_by_one("x", toks, tail=20)):
        worst, where = worst_error(steps, run_steps(runner, steps), expected)
        assert worst <= LIMIT["float32"], (worst, where)


def test_window_and_pool_edges_show(tmp_path):
    """Attention so sharp (scores times eight) that a key which is one position inside or
    outside the window, or a block that is pooled one step early or late, moves the logits by
    far more than the tolerance: in a prompt, in portions, and in decoding."""
    from tokamak_amd.engine.runner import ModelRunner

    cfg = model_json([layer(window=8, pool=4, scale=2.0, left_scale=1.5, right_scale=0.1),
                      layer(window=6, pool=3, scale=2.0, left_scale=1.5, right_scale=0.1)])
    w = random_weights(cfg, seed=3)
    folder = write_folder(tmp_path / "sharp", cfg, w)
    toks = tokens(cfg["vocab"], 300, 7)      # 70 and more pooled blocks: more entries than one chunk of the kernel
    expected = {"x": oracle_logits(cfg, w, toks)}
    for off_by in (dict(size=9, pool=4), dict(size=8, pool=5)):
        other = json.loads(json.dumps(cfg))
        other["layers"][0]["mixer"]["left"]["mask"] = off_by
        assert np.abs(oracle_logits(other, w, toks) - expected["x"]).max() > 0.1
    runner = ModelRunner.from_folder(folder, dtype="float32", page_size=16, kv_pool_tokens=320, max_requests=2)
    for steps in (whole({"x": toks}), tail_one_by_one("x", toks, tail=64), portions("x", toks)):
        worst, where = worst_error(steps, run_steps(runner, steps), expected)
        assert worst <= LIMIT["float32"], (worst, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(models, dtype):
    """One prompt token, then 260 tokens one by one (the recorded step of each shape replayed
    many times, two requests side by side at different lengths); and the same without recorded
    steps and without recorded layers gives the same bits."""
    runner, cfg, w = runner_for(models, "base", dtype)
    assert runner.use_graphs
    a, b = tokens(cfg["vocab"], 261, 11), tokens(cfg["vocab"], 200, 12)
    expected = expected_for(cfg, w, {"a": a, "b": b}, dtype)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:1], "want": [0]}], "end": []}]
    for i in range(1, 261):
        entries = [{"id": "a", "tokens": [a[i]], "want": [0]}]
        if i >= 61:
            entries.append({"id": "b", "tokens": [b[i - 61]], "want": [0]})
        steps.append({"step": i, "entries": entries, "end": []})
    got = run_steps(runner, steps)
    worst, where = worst_error(steps, got, expected)
    assert worst <= LIMIT[dtype], (dtype, worst, where)
    plain_runner, _, _ = runner_for(models, "base", dtype, use_graphs=False)
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
    folder, cfg, w, page = models["odd"]
    requests = {f"r{i}": tokens(cfg["vocab"], n, 300 + i) for i, n in enumerate([5, 33, 70, 12, 41])}
    steps, peak = mixed(requests, seed=2)
    expected = expected_for(cfg, w, requests)
    got = run_trace_any(folder, "float32", steps, peak, tmp_path / "out", page, cfg["vocab"])
    worst, where = worst_error(steps, got, expected)
    assert worst <= LIMIT["float32"], (worst, where)
    done = subprocess.run([sys.executable, "-m", "tokamak_amd.cli", "--model", str(folder), "--prompt-ids", "5,6,7",
                           "--max-new-tokens", "4", "--dtype", "float32", "--temperature", "0", "--max-seq-len", "64",
                           "--page-size", str(page), "--quiet"], cwd=ROOT, capture_output=True,
                          text=True, timeout=240)
    assert done.returncode == 0, done.stderr[-2000:]
    ids = [5, 6, 7]
    for _ in range(4):
        ids.append(int(np.argmax(oracle_logits(cfg, w, ids)[-1])))
    assert ",".join(map(str, ids[3:])) in done.stdout.replace(" ", ""), done.stdout


def run_trace_any(folder, dtype, steps, max_tokens, out_dir, page_size, vocab):
    """``replay_util.run_trace`` for a folder whose config.json names its vocabulary otherwise."""
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens), "--page-size", str(page_size)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for rec in steps:
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            assert line.strip() == f"done {rec['step']}", (line, proc.poll())
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    out = {}
    for rec in steps:
        wanted = sum(len(e.get("want", [])) for e in rec["entries"])
        if wanted:
            out[rec["step"]] = np.fromfile(Path(out_dir) / f"{rec['step']}.f32", dtype="<f4").reshape(wanted, vocab)
    return out
