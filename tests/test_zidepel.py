"""Zidepel without a GPU: its configuration and registry entry, the parts and cache entries it is made of, the
tensors it asks a checkpoint for, and the plain implementation's own consistency (prompt against token by token)."""
import copy
import json
import os

import numpy as np
import pytest
import torch

from plain import zidepel_plain as Z

RAW = {
    "architecture": "Zidepel", "vocab": 97, "width": 40, "max_positions": 90, "norm": {"eps": 1e-5}, "streams": 2,
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "attention", "mlp": {"kind": "dense", "ff": 56},
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "scale": 0.25, "softcap": 7.5, "q_temp": {"coef": 0.4, "every": 3}}},
        {"type": "gla", "mlp": None, "mixer": {"heads": 2, "dim": 8, "vdim": 12, "tau": 5.0, "rank": 4}},
        {"type": "attention", "mlp": {"kind": "dense", "ff": 24},
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.3, "softcap": None, "q_temp": None}},
        {"type": "gla", "mlp": {"kind": "dense", "ff": 32}, "mixer": {"heads": 1, "dim": 16, "vdim": 8, "tau": 2.0}},
    ],
}


def typed(raw=RAW):
    from rust_inference_amd.config import config_from_dict
    return config_from_dict(raw)


def test_the_registry_finds_the_design_by_its_architecture_key():
    from rust_inference_amd.config import ZidepelConfig, known_architectures
    arch, cfg = typed()
    assert arch.name == "Zidepel" and isinstance(cfg, ZidepelConfig) and "Zidepel" in known_architectures()
    assert cfg.order() == [0, 1, 2, 1, 2, 1, 2, 3]
    assert cfg.layers[0].mixer.temper_every == 3 and cfg.layers[2].mixer.softcap is None and cfg.layers[1].ff is None
    again = typed(json.loads(json.dumps(cfg.to_dict())))[1]
    assert again == cfg


def test_no_loop_and_no_streams():
    raw = {k: v for k, v in RAW.items() if k not in ("loop", "streams")}
    arch, cfg = typed(raw)
    assert cfg.order() == [0, 1, 2, 3] and cfg.streams is None
    spec = arch.build_spec(cfg)
    assert spec.stream.kind == "residual" and all(layer.arrangement == "prenorm" for layer in spec.layers)
    assert "mixer_connection" not in spec.layers[0].parts


@pytest.mark.parametrize("change, message", [
    (lambda r: r["layers"][0].update(type="conv"), "mixer type"),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), "not divisible"),
    (lambda r: r["layers"][0]["mlp"].update(kind="moe"), "feed-forward kind"),
    (lambda r: r["loop"].update(stop=9), "loop"),
    (lambda r: r["layers"][1]["mixer"].update(tau=0.0), "tau"),
    (lambda r: r.pop("norm"), "lacks norm"),
    (lambda r: r["layers"][0]["mixer"].update(softcap=-1.0), "softcap"),
])
def test_configurations_that_are_refused(change, message):
    from rust_inference_amd.errors import InferenceError
    raw = copy.deepcopy(RAW)
    change(raw)
    with pytest.raises(InferenceError, match=message):
        typed(raw)


def test_parts_schedule_and_cache_entries():
    from rust_inference_amd.cache import KVNeed, StateNeed
    from rust_inference_amd.parts import DecoderModel
    arch, cfg = typed()
    spec = arch.build_spec(cfg)
    model = DecoderModel(spec)
    assert [(r.layer, r.cache) for r in spec.schedule] == [(0, 0), (1, 1), (2, 2), (1, 3), (2, 4), (1, 5), (2, 6), (3, 7)]
    needs = model.cache_needs()
    assert needs[0] == KVNeed(2, 8, None, 12) and needs[2] == KVNeed(2, 16, None, None)
    assert needs[1] == needs[3] == needs[5] == StateNeed((2, 8, 12), torch.float32) and needs[7] == StateNeed((1, 16, 8), torch.float32)
    assert spec.stream.kind == "hyper" and spec.stream.params == {"streams": 2}
    names = model.tensors()
    for name, shape in {"embed": (97, 40), "pos": (90, 40), "embed.norm.b": (40,), "l0.mix.q": (32, 40), "l0.mix.v": (24, 40),
                        "l0.mix.o": (40, 48), "l0.mix.q.norm": (8,), "l0.hc2.mix": (2, 2), "l1.mix.a1": (4, 40),
                        "l1.mix.a2": (16, 4), "l1.mix.a2.b": (16,), "l1.mix.norm": (12,), "l1.mix.g": (24, 40),
                        "l3.mix.a1": (None, 40), "l3.mlp.down": (40, 32), "final.norm.b": (40,), "head": (97, 40)}.items():
        assert names[name].shape == shape, name
    assert "l1.norm2" not in names and "l1.hc2.in" not in names and "l1.mlp.up" not in names


def test_a_checkpoint_gives_the_width_of_the_decay_product(tmp_path):
    """The narrow middle of a gla mixer's decay product is named by no configuration key: any width loads, as long
    as the two tensors agree; a wrong size anywhere else is still refused."""
    from rust_inference_amd.errors import WeightsError
    from rust_inference_amd.parts.model import expected_tensors
    from rust_inference_amd.weights import write_random_model
    from rust_inference_amd.weights.loader import load_checked
    from safetensors.torch import load_file, save_file
    raw = copy.deepcopy(RAW)
    raw["layers"][3]["mixer"]["rank"] = 6
    folder = write_random_model(str(tmp_path / "m"), raw, 0)
    raw["layers"][3]["mixer"].pop("rank")
    raw["layers"][1]["mixer"].pop("rank")
    arch, cfg = typed(raw)
    want = expected_tensors(arch.build_spec(cfg))
    got = load_checked(folder, want)
    assert got["l3.mix.a1"].shape == (6, 40) and got["l1.mix.a2"].shape == (16, 4)
    w = load_file(os.path.join(folder, "model.safetensors"))
    w["l3.mix.a2.b"] = torch.zeros(17)
    save_file(w, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError, match="l3.mix.a2.b"):
        load_checked(folder, want)


def test_random_weights_need_the_width_named():
    from rust_inference_amd.errors import InferenceError
    from rust_inference_amd.weights import write_random_model
    with pytest.raises(InferenceError, match="rank"):
        write_random_model("/nonexistent/never-made", RAW, 0)


def small_model(seed=0):
    rng = np.random.default_rng(seed)
    cfg = copy.deepcopy(RAW)
    cfg["layers"][3]["mixer"]["rank"] = 3
    from rust_inference_amd.parts.model import expected_tensors
    arch, c = typed(cfg)
    w = {}
    for name, spec in expected_tensors(arch.build_spec(c)).items():
        x = rng.normal(size=spec.shape) * (0.3 if len(spec.shape) == 2 else 0.1)
        if name.endswith(("norm", ".in", ".out")):
            x = 1 + x
        if name.endswith(".mix"):
            x = np.eye(spec.shape[0]) + x * 0.3
        w[name] = x
    return cfg, w


def test_the_plain_form_token_by_token_is_its_prompt_form():
    cfg, w = small_model()
    toks = [int(t) for t in np.random.default_rng(1).integers(0, cfg["vocab"], 30)]
    whole = Z.logits(cfg, w, toks)
    d = Z.Decoder(cfg, w)
    pieces = np.concatenate([d.feed(toks[:7]), d.feed(toks[7:9])] + [d.feed([t]) for t in toks[9:]])
    assert np.abs(pieces - whole).max() < 1e-9 * np.abs(whole).max()


def test_the_plain_form_has_every_mechanism_switched_on():
    """Each constant and tensor of the design changes the logits: none is read and dropped."""
    cfg, w = small_model()
    toks = [int(t) for t in np.random.default_rng(2).integers(0, cfg["vocab"], 20)]
    base = Z.logits(cfg, w, toks)

    def moved(c=None, ww=None):
        return np.abs(Z.logits(c or cfg, ww or w, toks) - base).max() > 1e-6

    for path, value in ((("layers", 0, "mixer", "softcap"), 1.0), (("layers", 0, "mixer", "scale"), 0.5),
                        (("layers", 0, "mixer", "q_temp"), {"coef": 0.9, "every": 2}), (("layers", 1, "mixer", "tau"), 1.0),
                        (("loop", "times"), 2), (("norm", "eps"), 0.1)):
        c = copy.deepcopy(cfg)
        at = c
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        assert moved(c=c), path
    rng = np.random.default_rng(3)
    for name in w:
        if name == "l0.hc1.in":          # all streams are still equal there, and the norm takes a common factor out
            continue
        ww = dict(w)
        ww[name] = w[name] + 0.05 * rng.normal(size=w[name].shape)        # (not a constant: a norm's mean would take it out)
        assert moved(ww=ww), name
    # the mix matrix is indexed [from, to]: its transpose is another model
    ww = dict(w)
    ww["l0.hc1.mix"] = w["l0.hc1.mix"].T
    assert moved(ww=ww)
