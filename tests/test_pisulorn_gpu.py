"""The Pisulorn design through the engine, against the plain implementation (tests/plain/pisulorn_plain.py), in
float32 and in bfloat16, for configurations made here with random weights: whole prompts; the last tokens one by
one; prompts in portions down to two tokens; batches of unequal requests one after another, so that slots, pages,
states and convolution tails are used again; long decoding over page borders, window edges and temperature steps;
keys just inside and just outside a window, made to stand out; a state that must survive every cut; greedy
generation through the library's own entry point with and without graphs; the trace program and the command line."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import trace_plans as plans
from helpers import assert_logits_close, read_model_f64, rel_to_max
from plain import pisulorn_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def attention(heads, kv_heads, dim, vdim, scale, window, q_temp, mlp):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        mixer["mask"] = {"size": window}
    if q_temp:
        mixer["q_temp"] = q_temp
    return {"type": "attention", "mlp": mlp, "mixer": mixer}


def delta(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "delta", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


# Three streams, value heads larger than key heads, a window shorter than a page, a looped stretch that holds a
# recurrent layer, a layer without feed-forward, an attention layer with neither window nor temperature.
P_A = {"architecture": "Pisulorn", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "streams": 3, "residual_mult": 0.5,
       "loop": {"start": 1, "stop": 3, "times": 2},
       "layers": [attention(6, 2, 24, 40, 0.2, 19, {"coef": 0.5, "every": 5}, dense(136)),
                  delta(4, 2, 24, 16, 4, None),
                  attention(4, 4, 16, 16, 0.3, None, None, moe(6, 2, 40, 0.9))]}
# One plain residual (no streams) with a multiplier, no loop, one kv head, a temperature step at every position, a
# window longer than two pages, convolutions of two taps, every expert chosen.
P_B = {"architecture": "Pisulorn", "vocab": 300, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.4,
       "layers": [delta(2, 2, 40, 24, 2, moe(3, 3, 48, 2.0)),
                  attention(2, 1, 32, 32, 0.18, 70, {"coef": 0.2, "every": 1}, None)]}
# One stream with its coefficients, no multiplier, heads of 64 (the size the matrix cores take), a layer run three
# times, a window of exactly one page, one expert chosen of many, convolutions of one tap (no tail at all).
P_C = {"architecture": "Pisulorn", "vocab": 157, "width": 128, "norm": {"eps": 1e-5}, "streams": 1,
       "loop": {"start": 0, "stop": 1, "times": 3},
       "layers": [attention(8, 4, 64, 64, 0.11, 32, {"coef": 0.25, "every": 48}, moe(9, 1, 56, 1.2)),
                  delta(2, 1, 64, 48, 1, dense(96)),
                  delta(3, 3, 20, 72, 5, dense(40))]}
CONFIGS = {"A": P_A, "B": P_B, "C": P_C}


def sharpen(folder):
    """Random weights as the library draws them, with the tensors that small values would switch off made larger:
    the convolutions' taps, the router and its correction, the decay's constants.  (The projections of the decay and of
    beta stay as drawn: made larger they empty the state at one token and keep it whole at the next, and the norm of
    a read-out that is almost nothing then turns bfloat16's rounding into errors of ten per cent at those positions.)"""
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    g = torch.Generator().manual_seed(len(w))
    for name in w:
        if name.endswith(".conv"):
            w[name] = (torch.randn(w[name].shape, generator=g) * 0.8).to(w[name].dtype)
        elif name.endswith(".router"):
            w[name] = (w[name].float() * 2).to(w[name].dtype)
        elif name.endswith((".correction", ".A_log", ".dt_bias")):
            w[name] = (torch.randn(w[name].shape, generator=g) * 0.5).to(w[name].dtype)
    save_file(w, path)
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from rust_inference_amd.weights import write_random_model
    base = tmp_path_factory.mktemp("pisulorn")
    return {name: sharpen(write_random_model(str(base / name), cfg, seed, torch.bfloat16, matrix_std=0.12, gain_std=0.1))
            for seed, (name, cfg) in enumerate(CONFIGS.items())}


_models, _plain, _read = {}, {}, {}


def loaded(folders, name, dtype_name):
    from rust_inference_amd.parts import load_model
    if (name, dtype_name) not in _models:
        _models[(name, dtype_name)] = load_model(folders[name], DTYPES[dtype_name])
    return _models[(name, dtype_name)]


_settled = {}


def plain_logits(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain:
        if folder not in _read:
            _read[folder] = read_model_f64(folder)
        P.ROUTE_MARGINS = []
        _plain[key] = P.logits(*_read[folder], list(tokens))
        # the positions before a router's first close call (two experts' choice scores closer than float32 tells
        # apart reliably): from there on another implementation may rightly send a token elsewhere
        _settled[key] = np.min(P.ROUTE_MARGINS, axis=0) if P.ROUTE_MARGINS else np.ones(len(tokens))
        P.ROUTE_MARGINS = None
    return _plain[key]


def settled(folder, tokens, dtype_name):
    """The number of positions before a router's first close call: two experts' choice scores closer than the number
    format tells apart reliably (a bfloat16 input moves a score by a per cent).  From there on another
    implementation may rightly send a token elsewhere, and what follows the token sees it."""
    plain_logits(folder, tokens)
    close = _settled[(folder, tuple(tokens))] < (1e-5 if dtype_name == "float32" else 2e-2)
    return int(np.argmax(close)) if close.any() else len(tokens)


def requests_for(name, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"{name}{i}": [int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], n)] for i, n in enumerate(lengths)}


def replay(model, steps):
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    engine = engine_for_trace(model, plans.max_live_tokens(steps))
    player = Replayer(engine)
    outs = {}
    for s in steps:
        logits = player.feed(s)
        if logits is not None:
            outs[s["step"]] = logits.cpu().numpy()
    engine.cache.check_consistent()
    assert engine.cache.slots.free_count == engine.cache.num_slots
    assert all(f == g.pool.num_pages for f, g in zip(engine.cache.free_pages(), engine.cache.groups))
    return plans.collect(steps, lambda i: outs[i], model.spec.vocab_size)


def close_enough(got, want, dtype_name, what, bound=3e-2):
    """float32: every position within the library's bound.  bfloat16: a router's close call sends a token to another
    expert than the plain form's, and the per-head norm of a read-out that is close to nothing enlarges its rounding,
    which no bound on rounding covers; so a few positions (two, or 8%) may miss the bound, and float32 is the sharp
    test of everything a position could show."""
    if len(got) == 0:                                        # nothing is settled: a close call at the first token
        return
    if dtype_name == "float32":
        if bound < 1e-4:                                     # a caller's own, sharper float32 bound
            err = rel_to_max(got, want)
            assert err <= bound, f"{what}: differs by {err:.2e} of the largest logit (float32)"
            return
        return assert_logits_close(got, want, dtype_name, what)
    errs = np.abs(np.asarray(got, dtype=np.float64) - want).max(-1) / np.abs(want).max()
    over = int((errs > bound).sum())
    assert over <= max(2, 0.08 * len(errs)), f"{what}: {over} of {len(errs)} positions differ by more than {bound:.0e} (bfloat16), the worst by {errs.max():.2e}"


def against_plain(folder, got, requests, dtype_name, what, bound=3e-2):
    for rid, toks in requests.items():
        n = settled(folder, toks, dtype_name)
        assert n >= len(toks) // 2 or dtype_name != "float32", f"request {rid}: a router's close call at position {n} already: choose other tokens"
        close_enough(got[rid][:n], plain_logits(folder, toks)[:n], dtype_name, f"{what}, request {rid}", bound)


def in_portions(requests, sizes):
    """Each request alone, its prompt in portions of the given sizes in turn (the last portion takes what is left)."""
    steps = []
    for rid, toks in requests.items():
        at, i = 0, 0
        while at < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - at)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                          "end": [rid] if at + n == len(toks) else []})
            at, i = at + n, i + 1
    return steps


LENGTHS = {"A": [70, 3, 131], "B": [45, 1, 200], "C": [97, 33, 64]}


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompts(folders, name, dtype_name):
    reqs = requests_for(name, LENGTHS[name], 1)
    got = replay(loaded(folders, name, dtype_name), plans.whole(reqs))
    against_plain(folders[name], got, reqs, dtype_name, "whole")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_last_tokens_one_by_one_and_portions(folders, name, dtype_name):
    reqs = requests_for(name, [n + 40 for n in LENGTHS[name]], 2)
    model = loaded(folders, name, dtype_name)
    whole = replay(model, plans.whole(reqs))
    bound = 2e-5 if dtype_name == "float32" else 2e-2
    for what, steps in (("last 32 one by one", plans.tail_one_by_one(reqs, 32)),
                        ("portions of 2, 31 and 32", in_portions(reqs, [2, 31, 32])),
                        ("portions of 64, 1 and 7", in_portions(reqs, [64, 1, 7]))):
        got = replay(model, steps)
        against_plain(folders[name], got, reqs, dtype_name, what)
        for rid, toks in reqs.items():
            n = settled(folders[name], toks, dtype_name)
            close_enough(got[rid][:n], whole[rid][:n].astype(np.float64), dtype_name, f"{rid}, {what}: against the whole prompt", bound)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_unequal_batches_one_after_another(folders, name, dtype_name):
    rng = np.random.default_rng(7)
    batches, reqs = [], {}
    for b in range(3):                                       # three batches on one cache: slots, pages and states come back
        batch = {}
        for i in rng.permutation(len(LENGTHS[name])):
            p = LENGTHS[name][i]
            toks = [int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], p + int(rng.integers(0, 14)))]
            batch[f"{name}{b}_{i}"] = (toks, p)
            reqs[f"{name}{b}_{i}"] = toks
        batches.append(batch)
    model = loaded(folders, name, dtype_name)
    got = replay(model, plans.unequal_batches(batches))
    against_plain(folders[name], got, reqs, dtype_name, "unequal batches")
    alone = replay(model, plans.whole(reqs))
    bound = 2e-5 if dtype_name == "float32" else 2e-2
    for rid, toks in reqs.items():
        n = settled(folders[name], toks, dtype_name)
        close_enough(got[rid][:n], alone[rid][:n].astype(np.float64), dtype_name, f"{rid}: in a batch against itself alone", bound)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_float32_gives_the_same_bits_alone_and_in_a_batch(folders, name):
    """float32 has one form of every kernel: three unequal requests prefilled together and decoded together, and each
    alone with the same cut, give the same logits bit for bit."""
    rng = np.random.default_rng(11)
    batch = {f"{name}{i}": ([int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], p + 9)], p) for i, p in enumerate(LENGTHS[name])}
    model = loaded(folders, name, "float32")
    together = replay(model, plans.unequal_batches([batch]))
    for rid, (toks, p) in batch.items():
        alone = replay(model, plans.unequal_batches([{rid: (toks, p)}]))
        assert np.array_equal(together[rid].view(np.int32), alone[rid].view(np.int32)), f"{rid} differs from itself alone"


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding_from_the_first_tokens(folders, name, dtype_name):
    """Three tokens of prompt, then 150 one by one: over page borders, past both windows and many steps of the
    temperature, with the convolutions' tails still partly zeros at the first steps."""
    reqs = requests_for(name, [153], 3)
    got = replay(loaded(folders, name, dtype_name), plans.tail_one_by_one(reqs, 150))
    against_plain(folders[name], got, reqs, dtype_name, "long decoding")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_the_three_ways_through_the_experts_agree(folders, name, dtype_name):
    """A prompt of 330 tokens (its tokens sorted by expert), the same in portions of 100 (all experts for all tokens)
    and its last tokens one by one (only the chosen experts' rows are read), with a second request beside it."""
    reqs = requests_for(name, [330, 290], 9)
    model = loaded(folders, name, dtype_name)
    for what, steps in (("whole", plans.whole(reqs)), ("portions of 100", in_portions(reqs, [100])),
                        ("a batch, then one by one", plans.unequal_batches([{rid: (toks, len(toks) - 6) for rid, toks in reqs.items()}]))):
        against_plain(folders[name], replay(model, steps), reqs, dtype_name, what)


# ---------------------------------------------------------------- a window's edge, made to show
W_EDGE = {"architecture": "Pisulorn", "vocab": 64, "width": 32, "norm": {"eps": 1e-5},
          "layers": [attention(2, 1, 16, 16, 1.0, 37, None, None)]}


def edge_model(tmp_path_factory, window):
    """One attention layer whose queries and keys are (almost) the same vector for every token, scaled up, and whose
    values are the token's own embedding row: every visible key has the same product with the query, so each key's
    weight is set by the distance bias alone and a key one position outside the window is missing from a sum in
    which it would weigh as much as its neighbour."""
    from rust_inference_amd.weights import write_random_model
    cfg = copy.deepcopy(W_EDGE)
    cfg["layers"][0]["mixer"]["mask"] = {"size": window}
    folder = write_random_model(str(tmp_path_factory.mktemp(f"edge{window}")), cfg, window, torch.bfloat16, matrix_std=0.3)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    w["l0.mix.q"] = (w["l0.mix.q"].float() * 0.05).to(torch.bfloat16)          # scores nearly level: the far keys keep their weight
    save_file(w, path)
    return cfg, folder


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [37, 32, 33, 64, 1, 2])
def test_keys_just_inside_and_just_outside_the_window(tmp_path_factory, window, dtype_name):
    from rust_inference_amd.parts import load_model
    cfg, folder = edge_model(tmp_path_factory, window)
    rng = np.random.default_rng(window)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 3 * 32 + 9)]
    want = plain_logits(folder, toks)
    # the plain form itself must tell the edge: one token more or less in the window changes these logits clearly
    wider = copy.deepcopy(cfg)
    wider["layers"][0]["mixer"]["mask"]["size"] = window + 1
    moved = rel_to_max(P.logits(wider, read_model_f64(folder)[1], toks)[window + 2:], want[window + 2:])
    assert moved > (5e-2 if dtype_name == "bfloat16" else 1e-3), f"a window one token wider moves the logits by {moved:.1e} only"
    model = load_model(folder, DTYPES[dtype_name])
    reqs = {"e": toks}
    for what, steps in (("whole", plans.whole(reqs)), ("one by one", plans.tail_one_by_one(reqs, len(toks) - 1)),
                        ("portions", in_portions(reqs, [window + 1, 2, 31]))):
        got = replay(model, steps)
        assert_logits_close(got["e"], want, dtype_name, f"window {window}, {what}")


@pytest.mark.parametrize("cuts", [[300], [1] * 40 + [260], [33, 2, 265], [299, 1]])
def test_a_state_that_hardly_decays_survives_every_cut(folders, tmp_path_factory, cuts):
    """With the decay's constants far on the negative side (g close to 1) the delta rule's state keeps the first
    tokens for hundreds of steps: a state or a tail that is lost, reset or carried to the wrong slot at any cut
    changes the last logits."""
    from safetensors.torch import load_file, save_file
    from rust_inference_amd.parts import load_model
    folder = str(tmp_path_factory.mktemp("slow_decay"))
    w = load_file(os.path.join(folders["B"], "model.safetensors"))
    w["l0.mix.A_log"] = torch.full_like(w["l0.mix.A_log"], -6.0)
    w["l0.mix.b"] = w["l0.mix.b"] * 0
    w["l0.mix.o"] = w["l0.mix.o"] * 3
    save_file(w, os.path.join(folder, "model.safetensors"))
    # without the attention layer's window nothing but the state could carry the first token to the end; with it
    # (70 tokens) the same holds for a prompt of 300
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(P_B, f)
    toks = requests_for("B", [300], 4)["B0"]
    want = plain_logits(folder, toks)
    other = plain_logits(folder, [toks[0] ^ 1] + toks[1:])
    assert rel_to_max(other[-1], want[-1]) > 1e-3, "the first token does not reach the last logits: the test shows nothing"
    model = load_model(folder, torch.float32)
    steps, at = [], 0
    for n in cuts:
        # another request comes and goes between the portions, on the slot next to this one
        steps.append({"step": len(steps), "entries": [{"id": "x", "tokens": toks[at:at + n], "want": list(range(n))}], "end": []})
        steps.append({"step": len(steps), "entries": [{"id": f"o{at}", "tokens": toks[:5], "want": []}], "end": [f"o{at}"]})
        at += n
    steps[-1]["end"].append("x")
    got = replay(model, steps)
    assert_logits_close(got["x"], want, "float32", f"cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype_name, use_graphs", [("float32", False), ("float32", True), ("bfloat16", True)])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name, dtype_name, use_graphs):
    from rust_inference_amd import Model
    prompts = list(requests_for(name, [33, 2, 40, 7], 5).values())
    steps = 12
    cfg, w = read_model_f64(folders[name])
    model = Model.load(folders[name], dtype=dtype_name, max_batch=3, max_seq_len=128, use_graphs=use_graphs, graph_after=0)
    got = model.generate(prompts, max_new_tokens=steps).tokens          # four prompts on three slots: a second batch
    for g, p in zip(got, prompts):
        toks, rows = P.greedy(cfg, w, p, steps)
        for i, (a, b) in enumerate(zip(g, toks)):
            if a != b:
                top = np.sort(rows[i])
                fed = list(p) + toks[:i]
                assert (top[-1] - top[-2] < (1e-4 if dtype_name == "float32" else 0.08)
                        or settled(folders[name], fed, dtype_name) < len(fed)), f"token {i} is {a}, plain says {b}"
                break                                                   # from here on the two follow different texts
    model.cache.check_consistent()


def test_the_trace_program(folders, tmp_path):
    reqs = requests_for("A", [40, 9], 6)
    steps = plans.unequal_batches([{rid: (toks, len(toks) - 4) for rid, toks in reqs.items()}])
    out = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["A"], "--dtype", "float32",
                           "--out", out, "--max-tokens", str(plans.max_live_tokens(steps))],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    got = plans.collect(steps, lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4"), P_A["vocab"])
    against_plain(folders["A"], got, reqs, "float32", "trace program")


def drawn_config(seed):
    """A configuration drawn at random: sizes, head counts, order and number of layers, the looped stretch, the
    constants, with and without streams, multiplier, window, temperature and feed-forward of either kind."""
    rng = np.random.default_rng(2000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers = []
    for _ in range(int(rng.integers(2, 6))):
        mlp = pick([None, dense(40), dense(136), moe(pick([2, 4, 7]), 1, pick([24, 56]), float(rng.uniform(0.5, 3.0))),
                    moe(5, pick([2, 3, 5]), 32, 1.0)])
        if rng.random() < 0.55:
            kv = pick([1, 2, 3, 4])
            dim = pick([8, 16, 24, 32, 48, 64, 128])
            layers.append(attention(kv * pick([1, 2, 4]), kv, dim, pick([dim, dim, 8, 40, 64]), float(rng.uniform(0.05, 0.4)),
                                    pick([None, 1, 7, 31, 32, 33, 50, 100]),
                                    pick([None, {"coef": float(rng.uniform(0.05, 1.0)), "every": pick([1, 3, 32, 64])}]), mlp))
        else:
            kv = pick([1, 2, 3])
            layers.append(delta(kv * pick([1, 2]), kv, pick([8, 24, 32, 64, 128]), pick([4, 16, 24, 64, 128]), pick([1, 2, 4, 6]), mlp))
    cfg = {"architecture": "Pisulorn", "vocab": int(rng.integers(50, 400)), "width": pick([48, 80, 136, 192]),
           "norm": {"eps": pick([1e-5, 1e-6, 1e-3])}, "layers": layers}
    if rng.random() < 0.75:
        cfg["streams"] = pick([1, 2, 3, 4, 6])
    if rng.random() < 0.75:
        cfg["residual_mult"] = float(rng.uniform(0.2, 1.5))
    if rng.random() < 0.7:
        a = int(rng.integers(0, len(layers)))
        cfg["loop"] = {"start": a, "stop": int(rng.integers(a, len(layers) + 1)), "times": pick([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    cfg = drawn_config(seed)
    folder = sharpen(write_random_model(str(tmp_path / "m"), cfg, seed, torch.bfloat16, matrix_std=0.12, gain_std=0.1))
    rng = np.random.default_rng(seed)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab"], n)] for i, n in enumerate((150, 37, 1, 66))}
    batch = {rid: (toks, max(1, len(toks) - 9)) for rid, toks in reqs.items()}
    for dtype_name in ("float32", "bfloat16"):
        model = load_model(folder, DTYPES[dtype_name])
        for what, steps in (("whole", plans.whole(reqs)), ("last 32 one by one", plans.tail_one_by_one(reqs, 32)),
                            ("a batch", plans.unequal_batches([batch])), ("portions", in_portions(reqs, [33, 2, 64]))):
            got = replay(model, steps)
            if dtype_name == "float32":
                against_plain(folder, got, reqs, dtype_name, f"configuration {seed}, {what}")
                continue
            # bfloat16: a close call of a router sends a token to another expert, which float32 does not do; so the
            # sharp test is float32, and here the bound is wide and a few positions may miss it
            against_plain(folder, got, reqs, dtype_name, f"configuration {seed}, {what}", 8e-2)


def test_the_command_line_generates_what_the_plain_implementation_does(folders):
    """bin/runner on a Pisulorn folder, prompts as token ids: greedy in float32, sections timed, and a seeded
    temperature run that gives the same tokens twice."""
    cfg, w = read_model_f64(folders["A"])
    prompts = list(requests_for("A", [9, 14], 8).values())
    want = [P.greedy(cfg, w, p, 6)[0] for p in prompts]
    base = [sys.executable, os.path.join(ROOT, "bin", "runner"), folders["A"], "--dtype", "float32", "-n", "6"]
    two = subprocess.run(base + ["--prompt-ids", ",".join(map(str, prompts[0])), "--prompt-ids", ",".join(map(str, prompts[1])),
                                 "--profile"], capture_output=True, text=True, timeout=300)
    assert two.returncode == 0, two.stderr[-2000:]
    assert [[int(t) for t in ln.split()] for ln in two.stdout.strip().splitlines()] == want
    assert "section " in two.stderr and "attention" in two.stderr
    drawn = [subprocess.run(base + ["-p", " ".join(map(str, prompts[0])), "--temperature", "0.9", "--top-k", "20", "--seed", "5"],
                            capture_output=True, text=True, timeout=300) for _ in range(2)]
    assert drawn[0].returncode == 0, drawn[0].stderr[-2000:]
    assert drawn[0].stdout == drawn[1].stdout and len(drawn[0].stdout.split()) == 6
