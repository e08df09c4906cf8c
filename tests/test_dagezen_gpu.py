"""The Dagezen design through the engine, against the plain implementation (tests/plain/dagezen_plain.py), in
float32 and in bfloat16, for configurations made here with random weights: whole prompts; the last tokens one by
one; prompts in portions down to two tokens; batches of unequal requests one after another, so that slots, pages
and states are used again; long decoding over page borders and past every window; keys just inside and just outside
the window, made to stand out; a far key among hundreds; states that must survive every cut; greedy generation through
the library's own entry point with and without graphs; the trace program and the command line."""
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
from plain import dagezen_plain as P
from test_dagezen import dense, latent, layer, model, moe, par, ssm

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}

# Every mixer, in another order than usual and twice; heads that are no power of two; three query heads a key head; a
# window shorter than a page; a convolution of four taps and one of one; groups of one head and of all heads; normed
# parts that are half a head and several heads; all experts chosen and one of five; a layer without feed-forward.
D_A = model([layer(ssm(6, 8, 12, 3, 4, 12), moe(5, 1, 24)), layer(par(6, 2, 24, 0.2, 19, 3, 24, 0.6, 0.9), dense(136, 1.5)),
             layer(latent(5, 24, 8, 40, 48, 0.17, 300.0), None), layer(ssm(2, 40, 24, 1, 1, 1), dense(72, 0.7)),
             layer(par(3, 3, 16, 0.3, 45, 5, 8, 1.3, 0.4), moe(3, 3, 40))], vocab=211, width=96, alpha=2.2, cap=11.0)
# Sizes the matrix cores like (heads of 64 and 128, widths of 128), a window of more than two pages, one key head for
# eight query heads, a latent wider than a key row of 256, no cap on the logits, alpha of 1.
D_B = model([layer(latent(4, 64, 32, 64, 256, 0.08, 1000000.0), dense(256, 3.0)), layer(par(8, 1, 64, 0.11, 70, 2, 64, 0.8, 1.1, rank=16), moe(8, 2, 64)),
             layer(ssm(8, 64, 64, 2, 2, 4), None)], vocab=300, width=128, eps=1e-6, alpha=1.0, cap=None)
# A window of exactly one page and one of a single token; rotated parts of two elements; a state of one row; one
# expert; a convolution of five taps over a state-space mixer first in line.
D_C = model([layer(ssm(3, 16, 1, 3, 5, 3), dense(40, 2.0)), layer(par(4, 4, 32, 0.15, 32, 1, 40, 1.0, 0.5), moe(1, 1, 56)),
             layer(latent(2, 30, 2, 8, 20, 0.2, 100.0), moe(6, 4, 16)), layer(par(2, 1, 8, 0.5, 1, 4, 16, 0.5, 1.5), dense(96, 1.0))],
            vocab=157, width=64, eps=1e-5, alpha=3.0, cap=30.0)
# Sizes that 16-byte loads do not divide: a width of 100, heads of 12 and 20, a latent of 36 with six rotated elements,
# feed-forwards of 52 and 28, a window over more than a page beside one over everything a test sends.
D_D = model([layer(latent(5, 12, 6, 20, 36, 0.2), dense(52, 1.5)), layer(par(6, 3, 20, 0.2, 41, 3, 12, 0.8, 1.1, rank=5), moe(5, 2, 28)),
             layer(ssm(6, 12, 20, 3, 4, 3), dense(100, 3.0)), layer(par(5, 5, 12, 0.3, 500, 5, 20, 1.0, 1.0, rank=3), None)],
            vocab=333, width=100, eps=1e-5, alpha=2.6, cap=20.0)
CONFIGS = {"A": D_A, "B": D_B, "C": D_C, "D": D_D}


def sharpen(folder):
    """Random weights as the library draws them, with the tensors that small or level values would switch off made to
    count: the routers and their biases, the sinks, the distance bias, the bonus, the decay's bias, every bias."""
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    g = torch.Generator().manual_seed(len(w))
    draw = lambda like, std, mean=0.0: (mean + std * torch.randn(like.shape, generator=g)).to(like.dtype)
    for name in w:
        if name.endswith(".router"):
            w[name] = (w[name].float() * 1.5).to(w[name].dtype)
        elif name.endswith(".sink"):
            w[name] = draw(w[name], 1.5)
        elif name.endswith(".r1"):
            w[name] = draw(w[name], 0.3, 0.8)
        elif name.endswith(".r2"):
            w[name] = (0.2 + 2.0 * torch.rand(w[name].shape, generator=g)).to(w[name].dtype)
        elif name.endswith(".w0"):
            w[name] = draw(w[name], 1.0, -1.5)
        elif name.endswith((".A_log", ".dt_bias")):
            w[name] = draw(w[name], 0.7, -0.5)
        elif name.endswith(".mu.r") or ".mu." in name:
            w[name] = torch.rand(w[name].shape, generator=g).to(w[name].dtype)
        elif name.endswith(".b") and w[name].dim() == 1:
            w[name] = draw(w[name], 0.2)
    save_file(w, path)
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from rust_inference_amd.weights import write_random_model
    base = tmp_path_factory.mktemp("dagezen")
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
        _plain[key] = P.forward(*_read[folder], list(tokens), gaps=gaps)
        _settled[key] = np.min(gaps, axis=0) if gaps else np.full(len(tokens), np.inf)
    return _plain[key]


def settled(folder, tokens, dtype_name):
    """The number of positions before a router's first close call: two logits closer than the number format tells apart
    reliably.  From there on another implementation may rightly send a token elsewhere, and every state carries it on."""
    plain_logits(folder, tokens)
    close = _settled[(folder, tuple(tokens))] < (1e-5 if dtype_name == "float32" else 5e-2)
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


LENGTHS = {"A": [70, 3, 131], "B": [45, 1, 200], "C": [97, 33, 64], "D": [150, 2, 61]}


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
    # (bfloat16 at the sizes of B, keys of 288 elements among them: a twelfth of the positions sit between 3 and 4%)
    against_plain(folders[name], got, reqs, dtype_name, "unequal batches", 3e-2 if dtype_name == "float32" else 4e-2)
    alone = replay(model, plans.whole(reqs))
    bound = 2e-5 if dtype_name == "float32" else 2e-2
    for rid, toks in reqs.items():
        n = settled(folders[name], toks, dtype_name)
        close_enough(got[rid][:n], alone[rid][:n].astype(np.float64), dtype_name, f"{rid}: in a batch against itself alone", bound)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_long_decoding_from_the_first_tokens(folders, name, dtype_name):
    """Three tokens of prompt, then 200 one by one: over page borders and past every window, with the pages behind a
    window given back."""
    reqs = requests_for(CONFIGS[name], name, [203], 3)
    got = replay(loaded(folders, name, dtype_name), plans.tail_one_by_one(reqs, 200))
    against_plain(folders[name], got, reqs, dtype_name, "long decoding")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_the_ways_through_the_experts_agree(folders, dtype_name):
    """A prompt of 330 tokens (its tokens sorted by expert), the same in portions of 100 (all experts for all tokens) and
    its last tokens one by one, with a second request beside it."""
    reqs = requests_for(D_B, "B", [330, 290], 9)
    model = loaded(folders, "B", dtype_name)
    for what, steps in (("whole", plans.whole(reqs)), ("portions of 100", in_portions(reqs, [100])),
                        ("a batch, then one by one", plans.unequal_batches([{rid: (toks, len(toks) - 6) for rid, toks in reqs.items()}]))):
        against_plain(folders["B"], replay(model, steps), reqs, dtype_name, what)


# ---------------------------------------------------------------- the window's edge and a far key, made to show
def edge_model(tmp_path_factory, dim, window):
    """One layer whose windowed attention has a scale close to nothing and no distance bias, so that every visible key
    weighs the same whatever it holds, and whose time mixing hardly counts: a key one position outside the window is
    missing from a sum in which it would weigh as much as its neighbour."""
    from rust_inference_amd.weights import write_random_model
    cfg = model([layer(par(2, 1, dim, 0.002, window, 1, 8, 1.0, 0.02), None)], vocab=64, width=32, alpha=0.5, cap=None)
    folder = write_random_model(str(tmp_path_factory.mktemp(f"edge{dim}_{window}")), cfg, window, torch.bfloat16, matrix_std=0.3)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    w["l0.mix.left.r1"] = torch.zeros_like(w["l0.mix.left.r1"])
    w["l0.mix.left.g"] = w["l0.mix.left.g"] * 0.1             # a gate near one half for every token
    save_file(w, path)
    return cfg, folder


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim", [16, 64])
@pytest.mark.parametrize("window", [37, 32, 33, 64, 65, 1, 2, 31, 100])
def test_keys_just_inside_and_just_outside_the_window(tmp_path_factory, dim, window, dtype_name):
    from rust_inference_amd.parts import load_model
    cfg, folder = edge_model(tmp_path_factory, dim, window)
    rng = np.random.default_rng(window)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 4 * 32 + 9)]
    want = plain_logits(folder, toks)
    # the plain form itself must tell the edge: one token more in the window changes the logits
    least = 2e-2 if dtype_name == "bfloat16" else 1e-3
    w = read_model_f64(folder)[1]
    other = copy.deepcopy(cfg)
    other["layers"][0]["mixer"]["left"]["mask"]["size"] = window + 1
    first = window + 3
    moved = rel_to_max(P.forward(other, w, toks)[first:], want[first:])
    assert moved > least, f"one more token in the window moves the logits by {moved:.1e} only"
    model_ = load_model(folder, DTYPES[dtype_name])
    reqs = {"e": toks}
    for what, steps in (("whole", plans.whole(reqs)), ("one by one", plans.tail_one_by_one(reqs, len(toks) - 1)),
                        ("portions", in_portions(reqs, [window + 1, 2, 31])), ("the last 40 one by one", plans.tail_one_by_one(reqs, 40))):
        got = replay(model_, steps)
        assert_logits_close(got["e"], want, dtype_name, f"window {window}, {what}")
        assert rel_to_max(got["e"], want) < least * 0.75, f"window {window}, {what}"


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_and_the_sink(tmp_path_factory, dtype_name):
    """Attention over a latent with a score scale of 2, so that one key can take the softmax: the last logits must see a
    token 700 positions back, at a page's border, and lose weight to a sink of 8."""
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    cfg = model([layer(latent(2, 16, 8, 16, 24, 2.0, 10000.0), None)], vocab=80, width=32, alpha=0.3, cap=None)
    folder = write_random_model(str(tmp_path_factory.mktemp("far")), cfg, 3, torch.bfloat16, matrix_std=0.3)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    w["l0.mix.sink"] = torch.full_like(w["l0.mix.sink"], 8.0)
    save_file(w, path)
    rng = np.random.default_rng(5)
    toks = [int(t) for t in rng.integers(0, 40, 760)]
    toks[64] = 77                                              # a token seen nowhere else, at a page's first place
    want = plain_logits(folder, toks)
    cfg_, w_ = read_model_f64(folder)
    other = list(toks)
    other[64] = 78
    assert rel_to_max(P.forward(cfg_, w_, other)[-30:], want[-30:]) > 1e-2, "the far token does not reach the last logits"
    no_sink = dict(w_)
    no_sink["l0.mix.sink"] = np.full(2, -30.0)
    assert rel_to_max(P.forward(cfg_, no_sink, toks)[-30:], want[-30:]) > 1e-2, "the sink does not show"
    model_ = load_model(folder, DTYPES[dtype_name])
    reqs = {"f": toks}
    for what, steps in (("whole", plans.whole(reqs)), ("the last 40 one by one", plans.tail_one_by_one(reqs, 40)),
                        ("portions", in_portions(reqs, [300, 2, 255]))):
        assert_logits_close(replay(model_, steps)["f"], want, dtype_name, f"far key, {what}")


@pytest.mark.parametrize("cuts", [[300], [1] * 40 + [260], [33, 2, 265], [299, 1]])
def test_states_that_hardly_decay_survive_every_cut(tmp_path_factory, cuts):
    """A time mixing whose decay is exp(-exp(-9)) and a state-space mixer whose step sizes are small keep the first
    token for hundreds of steps, beside an attention that sees 20 tokens back: a state, a kept row or a convolution's
    tail that is lost, reset or carried to the wrong slot at any cut changes the last logits."""
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    cfg = model([layer(par(2, 1, 16, 0.2, 20, 2, 12, 0.3, 1.0), dense(64)), layer(ssm(2, 12, 8, 1, 4, 1), None)], vocab=90, width=48,
                alpha=0.2, cap=None)
    folder = write_random_model(str(tmp_path_factory.mktemp("no_decay")), cfg, 5, torch.bfloat16, matrix_std=0.12, gain_std=0.1)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    w["l0.mix.right.w0"] = torch.full_like(w["l0.mix.right.w0"], -9.0)
    w["l0.mix.right.w2"] = w["l0.mix.right.w2"] * 0.1
    w["l1.mix.A_log"] = torch.full_like(w["l1.mix.A_log"], -6.0)
    save_file(w, path)
    toks = requests_for(cfg, "s", [300], 4)["s0"]
    want = plain_logits(folder, toks)
    other = plain_logits(folder, [toks[0] ^ 1] + toks[1:])
    assert rel_to_max(other[-1], want[-1]) > 1e-3, "the first token does not reach the last logits: the test shows nothing"
    model_ = load_model(folder, torch.float32)
    steps, at = [], 0
    for n in cuts:
        # another request comes and goes between the portions, on the slot next to this one
        steps.append({"step": len(steps), "entries": [{"id": "x", "tokens": toks[at:at + n], "want": list(range(n))}], "end": []})
        steps.append({"step": len(steps), "entries": [{"id": f"o{at}", "tokens": toks[:5], "want": []}], "end": [f"o{at}"]})
        at += n
    steps[-1]["end"].append("x")
    got = replay(model_, steps)
    assert_logits_close(got["x"], want, "float32", f"cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype_name, use_graphs", [("float32", False), ("float32", True), ("bfloat16", True)])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name, dtype_name, use_graphs):
    from rust_inference_amd import Model
    prompts = list(requests_for(CONFIGS[name], name, [33, 2, 40, 7], 5).values())
    steps = 12
    cfg, w = read_model_f64(folders[name])
    model_ = Model.load(folders[name], dtype=dtype_name, max_batch=3, max_seq_len=128, use_graphs=use_graphs, graph_after=0)
    got = model_.generate(prompts, max_new_tokens=steps).tokens          # four prompts on three slots: a second batch
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
    model_.cache.check_consistent()


def test_the_trace_program(folders, tmp_path):
    reqs = requests_for(D_A, "t", [40, 9], 6)
    steps = plans.unequal_batches([{rid: (toks, len(toks) - 4) for rid, toks in reqs.items()}])
    out = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["A"], "--dtype", "float32",
                           "--out", out, "--max-tokens", str(plans.max_live_tokens(steps))],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    got = plans.collect(steps, lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4"), D_A["vocab"])
    against_plain(folders["A"], got, reqs, "float32", "trace program")


def drawn_config(seed):
    """A configuration drawn at random: sizes, head counts, number and order of layers, windows, constants, with
    feed-forwards of either kind and none."""
    rng = np.random.default_rng(7000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers = []
    for _ in range(int(rng.integers(1, 6))):
        experts = pick([1, 2, 4, 7])
        mlp = pick([None, dense(40, 0.8), dense(136, 2.5), moe(experts, int(rng.integers(1, experts + 1)), pick([8, 24, 56]))])
        kind = pick(["latent", "par", "ssm"])
        if kind == "latent":
            mixer = latent(pick([1, 2, 3, 6]), pick([8, 16, 24, 40, 64]), pick([2, 4, 8, 16, 32]), pick([8, 16, 40, 64]),
                           pick([8, 24, 64, 96]), float(rng.uniform(0.05, 0.4)), float(pick([100.0, 10000.0, 500000.0])))
        elif kind == "par":
            kv = pick([1, 2, 3, 4])
            mixer = par(kv * pick([1, 2, 4]), kv, pick([8, 16, 24, 32, 48, 64]), float(rng.uniform(0.05, 0.4)),
                        pick([None, 1, 7, 31, 32, 33, 50, 100, 150]), pick([1, 2, 3, 5]), pick([8, 24, 32, 48, 64, 100]),
                        float(rng.uniform(0.3, 1.5)), float(rng.uniform(0.3, 1.5)), rank=pick([1, 8, 16]))
        else:
            groups = pick([1, 2, 3])
            heads = groups * pick([1, 2, 3])
            vdim = pick([8, 16, 32, 64])
            parts = pick([g for g in (1, 2, heads, 2 * heads) if (heads * vdim) % g == 0])
            mixer = ssm(heads, vdim, pick([1, 8, 16, 32, 64, 100]), groups, pick([1, 2, 3, 4, 7]), parts)
        layers.append(layer(mixer, mlp))
    return model(layers, vocab=int(rng.integers(50, 400)), width=pick([48, 80, 136, 192]), eps=pick([1e-5, 1e-6, 1e-3]),
                 alpha=float(rng.uniform(0.5, 3.0)), cap=pick([None, 8.0, 30.0]))


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
        model_ = load_model(folder, DTYPES[dtype_name])
        for what, steps in (("whole", plans.whole(reqs)), ("last 32 one by one", plans.tail_one_by_one(reqs, 32)),
                            ("a batch", plans.unequal_batches([batch])), ("portions", in_portions(reqs, [33, 2, 64]))):
            got = replay(model_, steps)
            against_plain(folder, got, reqs, dtype_name, f"configuration {seed}, {what}", 3e-2 if dtype_name == "float32" else 8e-2)


def test_the_command_line_generates_what_the_plain_implementation_does(folders):
    """bin/runner on a Dagezen folder, prompts as token ids: greedy in float32, sections timed, and a seeded temperature
    run that gives the same tokens twice."""
    cfg, w = read_model_f64(folders["A"])
    prompts = list(requests_for(D_A, "c", [9, 14], 8).values())
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
