"""The Zakelorn design through the engine, against the plain implementation (tests/plain/zakelorn_plain.py), in
float32 and in bfloat16, for configurations made here with random weights: whole prompts; the last tokens one by
one; prompts in portions down to two tokens; batches of unequal requests one after another, so that slots, pages
and states are used again; long decoding over page borders, past the window and the kept first tokens; keys just
inside and just outside the window and the kept tokens, made to stand out; a state that must survive every cut;
greedy generation through the library's own entry point with and without graphs; the trace program and the
command line."""
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
from plain import zakelorn_plain as P
from test_zakelorn import layer, left, moe, right

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dense(ff):
    return {"kind": "dense", "ff": ff}


# Heads that the matrix cores do not take and value heads of another size; a window shorter than a page with kept
# tokens; three query heads a key head; more heads on the right than key heads on the left; identity experts, groups
# of which half stay, a shared expert; a layer without feed-forward.
Z_A = {"architecture": "Zakelorn", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 9.8},
       "layers": [layer(left(6, 2, 24, 40, 0.2, 19, 5, 10, 300.0), right(3, 24, 16, [0.6, 0.9, 0.99]), 0.6, 0.9, dense(136)),
                  layer(left(3, 3, 16, 16, 0.3, 45, 0, 16, 10000.0), right(5, 8, 24, [0.5, 0.7, 0.9, 0.97, 1.0]), 1.3, 0.4,
                        moe(6, 2, 2, 40, 4, 2, 40)),
                  layer(left(4, 1, 8, 8, 0.5, 7, 9, 2, 50.0), right(1, 40, 8, [0.93]), 1.0, 1.0, None)]}
# Heads of 64 (the size the matrix cores take) with kept tokens beyond one page behind a window of more than two; a
# layer whose attention sees everything and turns nothing; every expert chosen, no groups, no identity experts, no
# shared expert; a decay of exactly 1; no constant on the embedding.
Z_B = {"architecture": "Zakelorn", "vocab": 300, "width": 64, "norm": {"eps": 1e-6},
       "layers": [layer(left(4, 2, 64, 64, 0.11, 70, 33, 64, 1000000.0), right(2, 40, 24, [1.0, 0.9]), 0.8, 1.1, moe(3, 0, 3, 48, 1, 1, None)),
                  layer(left(2, 1, 64, 64, 0.09, None, 0, 0), right(4, 16, 16, [0.3, 0.8, 0.95, 0.999]), 1.0, 0.7, dense(40))]}
# Heads of 32 and 128, a window and kept tokens of exactly one page each, a window of one token with the first tokens
# kept, one expert chosen of nine outputs of which four are identity experts, one group of three kept.
Z_C = {"architecture": "Zakelorn", "vocab": 157, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.5},
       "layers": [layer(left(8, 8, 32, 32, 0.15, 32, 32, 8, 777.0), right(2, 64, 48, [0.8, 0.95]), 1.0, 0.5, moe(5, 4, 1, 56, 3, 1, 24)),
                  layer(left(2, 1, 128, 128, 0.06, 1, 3, 128, 20000.0), right(3, 20, 72, [0.5, 0.9, 0.99]), 0.5, 1.5, dense(96)),
                  layer(left(4, 2, 32, 32, 0.2, 100, 1, 32, 100.0), right(4, 32, 32, [0.7, 0.8, 0.9, 0.95]), 0.9, 0.9, moe(4, 0, 2, 32, 2, 1, 64))]}
CONFIGS = {"A": Z_A, "B": Z_B, "C": Z_C}


def sharpen(folder):
    """Random weights as the library draws them, with the tensors that small or level values would switch off made to
    count: the router and its correction, the sinks, the layer scales, the norms' biases."""
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    g = torch.Generator().manual_seed(len(w))
    for name in w:
        if name.endswith(".router"):
            w[name] = (w[name].float() * 1.5).to(w[name].dtype)
        elif name.endswith(".correction"):
            w[name] = (torch.randn(w[name].shape, generator=g) * 0.08).to(w[name].dtype)
        elif name.endswith(".sink"):
            w[name] = (torch.randn(w[name].shape, generator=g) * 1.5).to(w[name].dtype)
        elif name.endswith((".ls1", ".ls2")):
            w[name] = (0.7 + 0.3 * torch.randn(w[name].shape, generator=g)).to(w[name].dtype)
        elif name.endswith(".b") and w[name].dim() == 1:
            w[name] = (torch.randn(w[name].shape, generator=g) * 0.2).to(w[name].dtype)
    save_file(w, path)
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from rust_inference_amd.weights import write_random_model
    base = tmp_path_factory.mktemp("zakelorn")
    return {name: sharpen(write_random_model(str(base / name), cfg, seed, torch.bfloat16, matrix_std=0.12, gain_std=0.1))
            for seed, (name, cfg) in enumerate(CONFIGS.items())}


_models, _plain, _read, _settled = {}, {}, {}, {}


def loaded(folders, name, dtype_name):
    from rust_inference_amd.parts import load_model
    if (name, dtype_name) not in _models:
        _models[(name, dtype_name)] = load_model(folders[name], DTYPES[dtype_name])
    return _models[(name, dtype_name)]


def plain_logits(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain:
        if folder not in _read:
            _read[folder] = read_model_f64(folder)
        gaps = []
        _plain[key] = P.forward(*_read[folder], list(tokens), gaps_out=gaps)
        _settled[key] = np.min(gaps, axis=0) if gaps else np.full(len(tokens), np.inf)
    return _plain[key]


def settled(folder, tokens, dtype_name):
    """The number of positions before a router's first close call: two outputs' choice scores closer than the number
    format tells apart reliably (a bfloat16 input moves a score by a per cent).  From there on another
    implementation may rightly send a token elsewhere, and what follows the token sees it."""
    plain_logits(folder, tokens)
    close = _settled[(folder, tuple(tokens))] < (1e-5 if dtype_name == "float32" else 1e-2)
    return int(np.argmax(close)) if close.any() else len(tokens)


def requests_for(cfg, prefix, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"{prefix}{i}": [int(t) for t in rng.integers(0, cfg["vocab"], n)] for i, n in enumerate(lengths)}


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
    expert than the plain form's, which no bound on rounding covers; so a few positions (two, or 8%) may miss the
    bound, and float32 is the sharp test of everything a position could show."""
    if len(got) == 0:
        return
    if dtype_name == "float32":
        if bound < 1e-4:
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
    reqs = requests_for(CONFIGS[name], name, LENGTHS[name], 1)
    got = replay(loaded(folders, name, dtype_name), plans.whole(reqs))
    against_plain(folders[name], got, reqs, dtype_name, "whole")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_last_tokens_one_by_one_and_portions(folders, name, dtype_name):
    reqs = requests_for(CONFIGS[name], name, [n + 40 for n in LENGTHS[name]], 2)
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
    rng = np.random.default_rng(8)
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


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_long_decoding_from_the_first_tokens(folders, name, dtype_name):
    """Three tokens of prompt, then 200 one by one: over page borders, while the kept first tokens fill up, past them
    and past every window, with pages behind the window given back and the kept ones held."""
    reqs = requests_for(CONFIGS[name], name, [203], 3)
    got = replay(loaded(folders, name, dtype_name), plans.tail_one_by_one(reqs, 200))
    against_plain(folders[name], got, reqs, dtype_name, "long decoding")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_the_ways_through_the_experts_agree(folders, name, dtype_name):
    """A prompt of 330 tokens (its tokens sorted by expert, identity experts among them), the same in portions of 100
    (all experts for all tokens) and its last tokens one by one (only the chosen experts' rows are read), with a
    second request beside it."""
    reqs = requests_for(CONFIGS[name], name, [330, 290], 9)
    model = loaded(folders, name, dtype_name)
    for what, steps in (("whole", plans.whole(reqs)), ("portions of 100", in_portions(reqs, [100])),
                        ("a batch, then one by one", plans.unequal_batches([{rid: (toks, len(toks) - 6) for rid, toks in reqs.items()}]))):
        against_plain(folders[name], replay(model, steps), reqs, dtype_name, what)


# ---------------------------------------------------------------- the edges of window and kept tokens, made to show
def edge_model(tmp_path_factory, dim, window, keep):
    """One layer whose attention has a scale close to nothing, so that every visible key weighs the same whatever it
    holds, a sink that weighs as much as a key, and whose linear attention hardly counts: a key one position outside
    the window, or one kept token more, is missing from a sum in which it would weigh as much as its neighbour."""
    from rust_inference_amd.weights import write_random_model
    cfg = {"architecture": "Zakelorn", "vocab": 64, "width": 32, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
           "layers": [layer(left(2, 1, dim, dim, 0.002, window, keep, 4, 100.0), right(1, 8, 8, [0.5]), 1.0, 0.02, None)]}
    folder = write_random_model(str(tmp_path_factory.mktemp(f"edge{dim}_{window}_{keep}")), cfg, window, torch.bfloat16, matrix_std=0.3)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    w["l0.mix.left.sink"] = torch.zeros_like(w["l0.mix.left.sink"])
    w["l0.mix.left.g"] = w["l0.mix.left.g"] * 0.1             # a gate near one half for every token
    save_file(w, path)
    return cfg, folder


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim", [16, 64])
@pytest.mark.parametrize("window, keep", [(37, 3), (32, 32), (33, 31), (64, 33), (1, 2), (2, 0), (20, 64), (31, 1)])
def test_keys_just_inside_and_just_outside_the_window_and_the_kept_tokens(tmp_path_factory, dim, window, keep, dtype_name):
    from rust_inference_amd.parts import load_model
    cfg, folder = edge_model(tmp_path_factory, dim, window, keep)
    rng = np.random.default_rng(window)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 4 * 32 + 9)]
    want = plain_logits(folder, toks)
    # the plain form itself must tell the edges: one token more in the window, or one more kept, changes the logits
    least = 2e-2 if dtype_name == "bfloat16" else 1e-3
    w = read_model_f64(folder)[1]
    for what, change in (("window", lambda m: m.update(size=window + 1)), ("kept tokens", lambda m: m.update(keep_first=keep + 1))):
        other = copy.deepcopy(cfg)
        change(other["layers"][0]["mixer"]["left"]["mask"])
        first = window + keep + 3
        moved = rel_to_max(P.forward(other, w, toks)[first:], want[first:])
        assert moved > least, f"one more of the {what} moves the logits by {moved:.1e} only"
    model = load_model(folder, DTYPES[dtype_name])
    reqs = {"e": toks}
    for what, steps in (("whole", plans.whole(reqs)), ("one by one", plans.tail_one_by_one(reqs, len(toks) - 1)),
                        ("portions", in_portions(reqs, [window + 1, 2, 31])), ("the last 40 one by one", plans.tail_one_by_one(reqs, 40))):
        got = replay(model, steps)
        assert_logits_close(got["e"], want, dtype_name, f"window {window}, {keep} kept, {what}")
        # (one layer: bfloat16 stays well under what one key more or less would do)
        assert rel_to_max(got["e"], want) < 1.5e-2, f"window {window}, {keep} kept, {what}"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompts_in_chunks_of_the_linear_attention(folders, monkeypatch, name):
    """bfloat16 with every step of two tokens and more sent through the chunked form of the state's walk (which small
    models and short prompts would not take by themselves): whole prompts, portions that end inside chunks, down to two
    tokens, and unequal batches, each going on from the state the step before left."""
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.parts import load_model
    monkeypatch.setattr(ops, "DECAY_CHUNKS_FORCED", True)
    calls, chunked_form = [], ops.decay_scan_chunked
    monkeypatch.setattr(ops, "decay_scan_chunked", lambda *a, **k: (calls.append(1), chunked_form(*a, **k))[1])
    cfg = CONFIGS[name]
    model = load_model(folders[name], DTYPES["bfloat16"])
    reqs = requests_for(cfg, "c", [300, 66, 129, 2], 77)
    batch = {rid: (toks, max(1, len(toks) - 5)) for rid, toks in reqs.items()}
    for what, steps in (("whole", plans.whole(reqs)), ("portions", in_portions(reqs, [70, 2, 150])),
                        ("a batch", plans.unequal_batches([batch]))):
        against_plain(folders[name], replay(model, steps), reqs, "bfloat16", f"{name} in chunks, {what}")
    monkeypatch.setattr(ops, "DECAY_CHUNKS_FORCED", False)
    walked = replay(model, plans.whole(reqs))
    monkeypatch.setattr(ops, "DECAY_CHUNKS_FORCED", True)
    chunked = replay(model, plans.whole(reqs))
    assert len(calls) >= 6 * len(cfg["layers"]), "the layers' linear attention did not go in chunks"
    for rid in reqs:                                  # the two forms differ by rounding alone
        n = settled(folders[name], reqs[rid], "bfloat16")
        if n:
            err = np.abs(chunked[rid][:n].astype(np.float64) - walked[rid][:n]).max() / np.abs(walked[rid][:n]).max()
            assert err < 2e-2, f"{name}, request {rid}: chunks and walk differ by {err:.2e} of the largest logit"


@pytest.mark.parametrize("cuts", [[300], [1] * 40 + [260], [33, 2, 265], [299, 1]])
def test_a_state_that_does_not_decay_survives_every_cut(folders, tmp_path_factory, cuts):
    """With a decay of 1 and 0.9999 the linear attention's state keeps the first token for hundreds of steps, and the
    attention beside it sees 20 tokens back and keeps none: a state that is lost, reset or carried to the wrong slot
    at any cut changes the last logits."""
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    cfg = {"architecture": "Zakelorn", "vocab": 90, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
           "layers": [layer(left(2, 1, 16, 16, 0.2, 20, 0, 8, 1000.0), right(2, 12, 20, [1.0, 0.9999]), 0.3, 1.0, dense(64))]}
    folder = write_random_model(str(tmp_path_factory.mktemp("no_decay")), cfg, 5, torch.bfloat16, matrix_std=0.12, gain_std=0.1)
    toks = requests_for(cfg, "s", [300], 4)["s0"]
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
    prompts = list(requests_for(CONFIGS[name], name, [33, 2, 40, 7], 5).values())
    steps = 12
    cfg, w = read_model_f64(folders[name])
    model = Model.load(folders[name], dtype=dtype_name, max_batch=3, max_seq_len=128, use_graphs=use_graphs, graph_after=0)
    got = model.generate(prompts, max_new_tokens=steps).tokens          # four prompts on three slots: a second batch
    for g, p in zip(got, prompts):
        toks = list(p)
        for i, a in enumerate(g):
            row = P.forward(cfg, w, toks)[-1]
            b = int(np.argmax(row))
            if a != b:
                top = np.sort(row)
                assert (top[-1] - top[-2] < (1e-4 if dtype_name == "float32" else 0.08) * np.abs(row).max()
                        or settled(folders[name], toks, dtype_name) < len(toks)), f"token {i} is {a}, plain says {b}"
                break                                                   # from here on the two follow different texts
            toks.append(a)
    model.cache.check_consistent()


def test_the_trace_program(folders, tmp_path):
    reqs = requests_for(Z_A, "t", [40, 9], 6)
    steps = plans.unequal_batches([{rid: (toks, len(toks) - 4) for rid, toks in reqs.items()}])
    out = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["A"], "--dtype", "float32",
                           "--out", out, "--max-tokens", str(plans.max_live_tokens(steps))],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    got = plans.collect(steps, lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4"), Z_A["vocab"])
    against_plain(folders["A"], got, reqs, "float32", "trace program")


def drawn_config(seed):
    """A configuration drawn at random: sizes, head counts, number of layers, windows, kept tokens, rotated
    dimensions, decays, constants, with feed-forwards of either kind and none, with and without groups, identity
    experts and a shared expert."""
    rng = np.random.default_rng(3000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        outs_groups = pick([(2, 0, 1), (4, 0, 2), (7, 0, 1), (5, 1, 3), (4, 4, 2), (6, 3, 3), (3, 1, 4)])
        experts, identity, groups = outs_groups
        keep = int(rng.integers(1, groups + 1))
        top = int(rng.integers(1, keep * ((experts + identity) // groups) + 1))
        mlp = pick([None, dense(40), dense(136), moe(experts, identity, top, pick([24, 56]), groups, keep, pick([None, 16, 72]))])
        kv = pick([1, 2, 3, 4])
        dim = pick([8, 16, 24, 32, 48, 64, 128])
        window = pick([None, 1, 7, 31, 32, 33, 50, 100])
        l = left(kv * pick([1, 2, 4]), kv, dim, pick([dim, dim, 8, 40, 64]), float(rng.uniform(0.05, 0.4)), window,
                 pick([0, 1, 5, 31, 32, 33, 70]), pick([0, 2, dim // 2, dim]), float(pick([100.0, 10000.0, 500000.0])))
        if rng.random() < 0.2:
            l.pop("rot")
        hr = pick([1, 2, 3, 5])
        r = right(hr, pick([8, 24, 32, 64, 128]), pick([4, 16, 24, 64, 128]), [float(pick([1.0, rng.uniform(0.2, 0.999)])) for _ in range(hr)])
        layers.append(layer(l, r, float(rng.uniform(0.3, 1.5)), float(rng.uniform(0.3, 1.5)), mlp))
    cfg = {"architecture": "Zakelorn", "vocab": int(rng.integers(50, 400)), "width": pick([48, 80, 136, 192]),
           "norm": {"eps": pick([1e-5, 1e-6, 1e-3])}, "layers": layers}
    if rng.random() < 0.75:
        cfg["embedding"] = {"scale": float(rng.uniform(0.5, 12.0))}
    return cfg


@pytest.mark.parametrize("seed", range(10))
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
            # bfloat16: a close call of a router sends a token to another expert, which float32 does not do; so the
            # sharp test is float32, and there the bound is wide and a few positions may miss it
            against_plain(folder, got, reqs, dtype_name, f"configuration {seed}, {what}", 3e-2 if dtype_name == "float32" else 8e-2)


def test_the_command_line_generates_what_the_plain_implementation_does(folders):
    """bin/runner on a Zakelorn folder, prompts as token ids: greedy in float32, sections timed, and a seeded
    temperature run that gives the same tokens twice."""
    cfg, w = read_model_f64(folders["A"])
    prompts = list(requests_for(Z_A, "c", [9, 14], 8).values())
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(6):
            toks.append(int(np.argmax(P.forward(cfg, w, toks)[-1])))
        want.append(toks[len(p):])
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
