"""Rorosun without a GPU: its configuration and plan, its tensor names against a list written
independently, free dimensions of tensor specs, and properties of the plain implementation
that the GPU tests lean on."""

import json

import pytest
import torch

import plain_rorosun as plain
from rorosun_util import layer, model_json, random_weights, write_folder


def test_config_round_trip_and_errors():
    from tokamak_amd.config import get_architecture
    from tokamak_amd.models.rorosun import parse, to_config_json

    raw = model_json([layer(), layer(heads=6, kv_heads=3, dim=8, vdim=24, window=5, pool=3, ff=None)], vocab=77, width=48)
    cfg = parse(raw)
    assert (cfg.vocab_size, cfg.width, cfg.num_layers, cfg.norm_eps) == (77, 48, 2, 1e-5)
    assert cfg.layers[1].ff is None and cfg.layers[0].ff == 96
    assert (cfg.layers[1].left.window, cfg.layers[1].left.pool, cfg.layers[1].left.vdim) == (5, 3, 24)
    assert json.loads(json.dumps(to_config_json(cfg))) == raw
    assert get_architecture("Rorosun").parse(raw, (3,)).eos_token_ids == (3,)
    for breaker, message in [(lambda r: r["layers"][0].update(type="serial"), "layer type"),
                             (lambda r: r["layers"][0]["mlp"].update(kind="routed"), "feed-forward kind"),
                             (lambda r: r["layers"][0]["mixer"]["left"].pop("vdim"), "vdim"),
                             (lambda r: r.pop("norm"), "norm"),
                             (lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3), "multiple")]:
        bad = json.loads(json.dumps(raw))
        breaker(bad)
        with pytest.raises(ValueError, match=message):
            parse(bad)


def test_folder_is_found_by_its_architecture_key_and_names_match(tmp_path):
    from tokamak_amd.config import load_model_description
    from tokamak_amd.engine.model import LayeredModel
    from tokamak_amd.weights import SafetensorsSource, WeightError, validate

    raw = model_json([layer(), layer(ff=None, r_heads=3, r_dim=24)])
    w = random_weights(raw, 0, rank=6)
    folder = write_folder(tmp_path / "m", raw, w)
    arch, cfg, plan = load_model_description(folder)
    assert arch.name == "Rorosun" and plan.num_cache_slots == 4
    model = LayeredModel(plan, dtype=torch.float32, device="meta")
    expected = model.expected_tensors()
    assert set(expected) == set(w)
    for name, spec in expected.items():
        assert spec.fits(w[name].shape), name
    assert expected["l0.mix.right.w1"].shape == (None, 64) and expected["l1.mix.right.w2"].shape == (72, None)
    validate(expected, SafetensorsSource(folder).names())
    groups, slots = model.cache_layout()
    assert [g.window for g in groups] == [None] and sorted(slots) == [0, 2]      # the attention's pages
    assert sorted(model.state_requests()) == [1, 3]                               # the time mix's state
    assert model.capturable and all(b.replayable for b in model.blocks)
    del w["l1.ls1"]
    w["l1.ls2"] = torch.zeros(64)
    write_folder(tmp_path / "bad", raw, w)
    with pytest.raises(WeightError) as err:
        validate(expected, SafetensorsSource(tmp_path / "bad").names())
    assert err.value.missing == ["l1.ls1"] and err.value.unexpected == ["l1.ls2"]


def test_random_weights_mode_and_presets():
    from tokamak_amd.config import find_preset, preset_names
    from tokamak_amd.weights.random_init import expected_tensors_of

    assert {"rorosun-tiny", "rorosun-0.6b", "rorosun-8b"} <= set(preset_names())
    arch, cfg = find_preset("rorosun-tiny")
    expected = expected_tensors_of(arch.plan(cfg))
    assert expected["l0.mix.right.w1"].shape == (8, 64)       # a preset gives the rank, a checkpoint's tensors do otherwise
    assert expected["l0.norm1"].shape == () and expected["embed"].shape == (256, 64)


def test_free_dimensions_of_a_tensor_spec():
    from tokamak_amd.weights import TensorSpec

    spec = TensorSpec((None, 8))
    assert spec.fits((3, 8)) and spec.fits((1, 8)) and not spec.fits((3, 9)) and not spec.fits((8,))
    assert TensorSpec(()).fits(()) and not TensorSpec(()).fits((1,))


def test_attention_kernel_plan_fits_the_lds():
    from tokamak_amd.kernels import ops

    for heads, kv, dim, vdim in [(4, 2, 16, 16), (32, 8, 128, 128), (64, 8, 128, 128), (5, 1, 8, 8), (16, 16, 256, 64)]:
        for span in (1, 2048):
            rows, chunk, threads = ops.pooled_window_plan(heads, kv, dim, vdim, span)
            floats = rows * heads * dim + chunk * (kv * (dim + vdim) + 2) + 2 * rows * heads * chunk + 2 * rows * heads + heads * heads
            assert 4 * floats <= ops.POOLED_LDS_BYTES and chunk >= 1 and rows * heads * vdim <= ops.POOLED_ACC * threads
            assert rows == 1 if span == 1 else rows >= 1
    with pytest.raises(ops.KernelError):
        ops.pooled_window_plan(256, 1, 64, 128, 1)


# -- the plain implementation -------------------------------------------------------
def test_visibility_sets():
    for size, pool in [(1, 1), (5, 3), (8, 4), (3, 7), (24, 6)]:
        for i in range(0, 70):
            seen = set(plain.visible_tokens(i, size))
            assert seen == {j for j in range(i + 1) if i - j < size}
            blocks = set(plain.visible_blocks(i, size, pool))
            assert blocks == {b for b in range(i // pool + 1) if b * pool + pool - 1 <= i - size}
            pooled = {b * pool + t for b in blocks for t in range(pool)}
            assert not (pooled & seen)                                   # nothing is seen twice
            hidden = set(range(i + 1)) - seen - pooled
            assert len(hidden) < pool                                    # only an incomplete block behind the window


def test_pool_of_one_and_window_of_one_is_full_causal_attention():
    """Every earlier position is then a block of its own: the same weights as a plain causal softmax."""
    g = torch.Generator().manual_seed(0)
    s = torch.randn(9, 9, generator=g, dtype=torch.float64)
    wt, wb = plain.pooled_window_weights(s, s, 1, 1)
    full = torch.softmax(s.masked_fill(torch.ones(9, 9).triu(1).bool(), float("-inf")), dim=-1)
    torch.testing.assert_close(wt + wb, full)
    assert float((wt * wb).abs().max()) == 0.0


def test_scan_against_its_closed_form():
    g = torch.Generator().manual_seed(1)
    T, H, D = 7, 2, 5
    r, k, v = (torch.randn(T, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    dec = torch.rand(T, H, D, generator=g, dtype=torch.float64)
    u = torch.randn(H, D, generator=g, dtype=torch.float64)
    got = plain.wkv_scan(r, k, v, dec, u)
    for t in range(T):
        want = torch.einsum("hk,hk,hk,hv->hv", r[t], u, k[t], v[t])
        for s in range(t):
            between = torch.ones(H, D, dtype=torch.float64)
            for x in range(s + 1, t):
                between = between * dec[x]
            want = want + torch.einsum("hk,hk,hk,hv->hv", r[t], between, k[s], v[s])
        torch.testing.assert_close(got[t], want)


def test_a_layer_without_feed_forward_and_the_shift():
    raw = model_json([layer(ff=None)], vocab=30, width=16)
    w = {n: t.double() for n, t in random_weights(raw, 2).items()}
    assert "l0.norm2" not in w and "l0.ls2" not in w
    toks = [3, 9, 9, 1, 0, 22]
    whole_logits = plain.logits(toks, raw, w)
    assert whole_logits.shape == (6, 30)
    torch.testing.assert_close(plain.logits(toks[:4], raw, w), whole_logits[:4])      # causal
    h = torch.arange(6.0).reshape(3, 2)
    assert plain.shifted(h).tolist() == [[0, 0], [0, 1], [2, 3]]
