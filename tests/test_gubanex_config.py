"""The Gubanex design's configuration, plan and run order (no GPU)."""

import json

import pytest
import torch

import plain_gubanex as plain
from gubanex_util import attention, experts, gla, model_json, random_weights, write_folder


def test_parse_plan_and_tensor_names(tmp_path):
    from tokamak_amd.config.registry import load_model_description
    from tokamak_amd.engine.model import LayeredModel

    cfg = model_json([gla(heads=3, dim=8, vdim=24), attention(heads=6, kv_heads=3, dim=24, vdim=16, chunk=10, rot=12,
                                                               scaling=(4.0, 1.0, 2.0, 64.0)),
                      gla(mlp=None), attention(chunk=None, rot=0, mlp=experts(5, 5, 24))], vocab=90, width=40,
                     loop=(1, 3, 3))
    w = random_weights(cfg, 0, rank=5)
    folder = write_folder(tmp_path / "m", cfg, w)
    arch, typed, plan = load_model_description(folder)
    assert arch.name == "Gubanex" and typed.loop.times == 3 and typed.layers[2].mlp is None
    assert typed.layers[3].mixer.chunk is None and typed.layers[3].mixer.rot is None
    assert arch.parse(arch.to_json(typed)) == typed
    # layers 1 and 2 three times in a row; every call a cache slot of its own; the embedding comes
    # in again at the first layer of the second and third pass
    assert [c.layer for c in plan.order] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [c.cache for c in plan.order] == list(range(8))
    assert [c.adds_embedding for c in plan.order] == [False, False, False, True, False, True, False, False]
    assert [(i, add) for i, add in plain.layer_calls(cfg)] == [(c.layer, c.adds_embedding) for c in plan.order]
    model = LayeredModel(plan, dtype=torch.float32, device="cpu")
    expected = model.expected_tensors()
    assert set(expected) == set(w)
    assert all(expected[n].fits(t.shape) for n, t in w.items())
    assert expected["l0.mix.a1"].shape == (None, 40)       # the decay's rank is the tensor's
    groups, slots = model.cache_layout()
    assert [g.slots for g in groups] == [(1, 3, 5, 7)] and sorted(model.state_requests()) == [0, 2, 4, 6]
    assert model.state_requests()[0]["S"].shape == (3, 8, 24)
    assert model.capturable


def test_config_errors():
    from tokamak_amd.models.gubanex import parse

    good = model_json([gla(), attention()])
    parse(good)
    for path, value, text in [(("layers", 0, "type"), "conv", "unknown layer type"),
                              (("layers", 1, "mlp", "kind"), "dense", "unknown feed-forward kind"),
                              (("layers", 1, "mixer", "kv_heads"), 3, "multiple of kv_heads"),
                              (("layers", 1, "mixer", "rot", "dims"), 7, "rot.dims"),
                              (("layers", 0, "mixer", "tau"), 0.0, "tau"),
                              (("layers", 0, "mlp", "router", "top"), 9, "top")]:
        bad = json.loads(json.dumps(good))
        at = bad
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ValueError, match=text):
            parse(bad)
    with pytest.raises(ValueError, match="loop"):
        parse(model_json([gla(), attention()], loop=(1, 3, 2)))
    missing = json.loads(json.dumps(good))
    del missing["layers"][0]["mixer"]["vdim"]
    with pytest.raises(ValueError, match="vdim"):
        parse(missing)


def test_scaled_frequencies_against_the_plain_ones():
    from tokamak_amd.parts.rotary import scaled_frequencies

    for rot in ({"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 64.0}},
                {"base": 500.0, "dims": 6, "scaling": {"factor": 2.5, "low": 0.5, "high": 8.0, "original": 80.0}}):
        s = rot["scaling"]
        got = scaled_frequencies(rot["dims"], rot["base"], s["factor"], s["low"], s["high"], s["original"])
        want = plain.rotary_frequencies(rot)
        assert torch.allclose(torch.tensor(got, dtype=torch.float64), want, rtol=1e-12, atol=0)
        plainf = plain.rotary_frequencies({"base": rot["base"], "dims": rot["dims"]})
        kept = [abs(a / b - 1) < 1e-12 for a, b in zip(got, plainf.tolist())]
        assert any(kept) and not all(kept)        # all three regimes of wavelengths occur


def test_presets_build():
    from tokamak_amd.config.registry import find_preset

    for name in ("gubanex-tiny", "gubanex-0.6b", "gubanex-8b"):
        arch, cfg = find_preset(name)
        plan = arch.plan(arch.shorten(cfg, 2))
        assert len(plan.layers) == 2 and arch.parse(arch.to_json(arch.shorten(cfg, 2))).layers[0].mixer.heads == cfg.layers[0].mixer.heads
