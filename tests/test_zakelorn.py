"""Zakelorn without a GPU: its configuration and registry entry, the parts and cache entries it is made of, the
tensors it asks a checkpoint for, and the plain implementation's own consistency (prompt against token by token;
every constant and tensor moves the logits; the mask, the sink, the groups and the identity experts by hand)."""
import copy
import json

import numpy as np
import pytest
import torch

from plain import zakelorn_plain as P


def left(heads, kv, dim, vdim, scale, size, keep, rot_dims, base=10000.0):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"dims": rot_dims, "base": base}}
    if size is not None:
        m["mask"] = {"size": size, "keep_first": keep}
    return m


def right(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def layer(l, r, ls, rs, mlp):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def moe(experts, identity, top, ff, groups, keep, shared):
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top, "identity": identity, "groups": {"count": groups, "keep": keep}}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


RAW = {
    "architecture": "Zakelorn", "vocab": 89, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.5},
    "layers": [
        layer(left(4, 2, 8, 12, 0.4, 5, 2, 4), right(3, 8, 4, [0.5, 0.9, 0.99]), 0.7, 1.2, {"kind": "dense", "ff": 40}),
        layer(left(2, 2, 16, 16, 0.2, 9, 0, 16, 500.0), right(2, 4, 12, [0.8, 1.0]), 1.0, 0.5, moe(5, 1, 3, 24, 3, 2, 16)),
        layer(left(3, 1, 8, 8, 0.3, None, 0, 2), right(1, 16, 8, [0.95]), 0.4, 0.9, None),
        layer(left(2, 1, 8, 4, 0.3, 3, 4, 8), right(2, 8, 8, [0.7, 0.3]), 1.1, 1.0, moe(4, 0, 2, 16, 1, 1, None)),
    ],
}


def typed(raw=RAW):
    from rust_inference_amd.config import config_from_dict
    return config_from_dict(raw)


def test_the_registry_finds_the_design_by_its_architecture_key():
    from rust_inference_amd.config import ZakelornConfig, known_architectures
    arch, cfg = typed()
    assert arch.name == "Zakelorn" and isinstance(cfg, ZakelornConfig) and "Zakelorn" in known_architectures()
    a = cfg.layers[0].mixer
    assert (a.left.window, a.left.keep_first, a.left.rot_dims, a.left.vdim) == (5, 2, 4, 12)
    assert a.right.decay == pytest.approx((0.5, 0.9, 0.99)) and a.left_scale == pytest.approx(0.7)
    assert cfg.layers[2].mixer.left.window is None and cfg.layers[2].mlp is None
    m = cfg.layers[1].mlp
    assert (m.experts, m.identity, m.top, m.groups, m.keep, m.shared_ff) == (5, 1, 3, 3, 2, 16)
    assert cfg.layers[3].mlp.shared_ff is None and cfg.embedding_scale == pytest.approx(3.5)
    again = typed(json.loads(json.dumps(cfg.to_dict())))[1]
    assert again == cfg


@pytest.mark.parametrize("change, message", [
    (lambda r: r["layers"][0].update(type="attention"), "mixer type"),
    (lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3), "not divisible"),
    (lambda r: r["layers"][0]["mlp"].update(kind="glu"), "feed-forward kind"),
    (lambda r: r["layers"][0]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda r: r["layers"][0]["mixer"]["right"].update(decay=[0.5, 0.5, 1.5]), "between 0 and 1"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=3), "even"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=10), "at most the head size"),
    (lambda r: r.pop("norm"), "lacks norm"),
    (lambda r: r["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=5), "best of"),
    (lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda r: r["layers"][0]["mixer"].pop("right"), "'right'"),
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
    # every layer keeps two things per sequence: the attention's keys and values, the linear attention's state
    assert [(r.layer, r.cache) for r in spec.schedule] == [(0, (0, 1)), (1, (2, 3)), (2, (4, 5)), (3, (6, 7))]
    needs = model.cache_needs()
    assert needs[0] == KVNeed(2, 8, 5, 12, 2) and needs[1] == StateNeed((3, 8, 4), torch.float32)
    assert needs[2] == KVNeed(2, 16, 9, None, None) and needs[4] == KVNeed(1, 8, None, None, None)
    assert needs[6] == KVNeed(1, 8, 3, 4, 4) and needs[7] == StateNeed((2, 8, 8), torch.float32)
    mixer = model.layers[0].mixer
    a, r = mixer.members
    assert mixer.scales == pytest.approx((0.7, 1.2)) and (a.window, a.keep_first, a.sinks, a.gate) == (5, 2, True, "sigmoid")
    assert a.unit_norm and a.scale == pytest.approx(0.4) and r.decay == pytest.approx((0.5, 0.9, 0.99))
    assert model.layers[2].feed_forward is None
    ff = model.layers[1].feed_forward
    assert (ff.experts, ff.identity, ff.outs, ff.groups, ff.keep, ff.shared, ff.normalize, ff.scores) == (5, 1, 6, 3, 2, 16, False, "softmax")
    names = model.tensors()
    for name, shape in {"embed": (89, 48), "l0.mix.left.q": (32, 48), "l0.mix.left.k": (16, 48), "l0.mix.left.v": (24, 48),
                        "l0.mix.left.g": (48, 48), "l0.mix.left.o": (48, 48), "l0.mix.left.sink": (4,),
                        "l0.mix.right.q": (24, 48), "l0.mix.right.v": (12, 48), "l0.mix.right.g": (12, 48),
                        "l0.mix.right.o": (48, 12), "l0.mix.right.norm": (12,), "l0.norm1": (48,), "l0.norm1.b": (48,),
                        "l0.norm2.b": (48,), "l0.ls1": (48,), "l0.ls2": (48,), "l0.mlp.up": (40, 48), "l0.mlp.down": (48, 40),
                        "l1.mlp.router": (6, 48), "l1.mlp.correction": (6,), "l1.mlp.e4.gate": (24, 48),
                        "l1.mlp.e0.down": (48, 24), "l1.mlp.shared.up": (16, 48), "l1.mlp.shared.sg": (1, 48),
                        "l3.mlp.router": (4, 48), "final.norm": (48,), "final.norm.b": (48,)}.items():
        assert names[name].shape == shape, name
    for absent in ("l2.norm2", "l2.ls2", "l2.mlp.up", "l1.mlp.e5.gate", "l3.mlp.shared.gate", "l0.mix.left.q_norm.weight"):
        assert absent not in names, absent
    assert names["head"].optional                     # the output matrix is the embedding table unless a checkpoint brings one


def small_model(seed=0, raw=RAW):
    rng = np.random.default_rng(seed)
    cfg = copy.deepcopy(raw)
    from rust_inference_amd.parts.model import expected_tensors
    arch, c = typed(cfg)
    w = {}
    for name, spec in expected_tensors(arch.build_spec(c)).items():
        if spec.optional:                 # an output matrix of its own, which the design does not have
            continue
        x = rng.normal(size=spec.shape) * (0.3 if len(spec.shape) == 2 else 0.2)
        if name.endswith(("norm", "norm1", "norm2", "ls1", "ls2")):
            x = 1 + x
        if name.endswith("router"):
            x = x * 0.5
        if name.endswith("correction"):
            x = x * 0.1
        if name == "embed":
            x = x / 3
        w[name] = x
    return cfg, w


def test_the_plain_form_token_by_token_is_its_prompt_form():
    cfg, w = small_model()
    toks = [int(t) for t in np.random.default_rng(1).integers(0, cfg["vocab"], 30)]
    whole = P.forward(cfg, w, toks)
    assert np.abs(P.token_by_token(cfg, w, toks) - whole).max() < 1e-9 * np.abs(whole).max()
    kept = [{} for _ in cfg["layers"]]
    pieces = np.concatenate([P.forward(cfg, w, toks[:7], kept, 0), P.forward(cfg, w, toks[7:9], kept, 7),
                             P.forward(cfg, w, toks[9:], kept, 9)])
    assert np.abs(pieces - whole).max() < 1e-9 * np.abs(whole).max()


def test_the_plain_form_has_every_mechanism_switched_on():
    """Each constant and tensor of the design changes the logits: none is read and dropped."""
    cfg, w = small_model()
    toks = [int(t) for t in np.random.default_rng(2).integers(0, cfg["vocab"], 40)]
    base = P.forward(cfg, w, toks)

    def moved(c=None, ww=None):
        return np.abs(P.forward(c or cfg, ww or w, toks) - base).max() > 1e-7

    L = lambda i, *path: ("layers", i, "mixer", *path)
    for path, value in ((L(0, "left", "mask", "size"), 4), (L(0, "left", "mask", "keep_first"), 3), (L(0, "left", "scale"), 0.5),
                        (L(0, "left", "rot", "dims"), 6), (L(1, "left", "rot", "base"), 100.0), (L(0, "left_scale"), 0.1),
                        (L(0, "right_scale"), 0.1), (L(2, "right", "decay"), [0.5]), (L(0, "right", "decay"), [0.5, 0.9, 0.9]),
                        (("layers", 1, "mlp", "router", "top"), 2), (("layers", 1, "mlp", "router", "groups", "keep"), 1),
                        (("layers", 1, "mlp", "router", "groups", "count"), 2), (("norm", "eps"), 0.1),
                        (("embedding", "scale"), 1.0)):
        c = copy.deepcopy(cfg)
        at = c
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        assert moved(c=c), path
    rng = np.random.default_rng(3)
    for name in w:
        ww = dict(w)
        ww[name] = w[name] + 0.05 * rng.normal(size=w[name].shape)        # (not a constant: a norm would take it out)
        if name.endswith("correction"):
            ww[name] = w[name] + np.linspace(3.0, -3.0, w[name].shape[0])  # enough to change who is chosen
        assert moved(ww=ww), name


def test_the_mask_by_hand():
    """A query sees itself and size - 1 tokens before it, and every token before keep_first."""
    see = [j for j in range(12) if P.sees(9, j, 3, 2)]
    assert see == [0, 1, 7, 8, 9]
    assert [j for j in range(6) if P.sees(3, j, 1, 0)] == [3]
    assert [j for j in range(6) if P.sees(2, j, 2, 5)] == [0, 1, 2]          # kept tokens after the query stay unseen


def test_the_sink_takes_weight_and_gives_nothing():
    q = np.zeros((1, 1, 2))
    k = np.zeros((3, 1, 2))
    v = np.array([[[3.0]], [[6.0]], [[9.0]]])
    pos = np.arange(3.0)
    # three level scores of 0 and a sink of ln 3: the denominator is 6, the result half the values' mean
    o = P.sink_attention(q, k, v, pos[2:], pos, 7.0, 10, 0, np.array([np.log(3.0)]))
    assert o[0, 0, 0] == pytest.approx(3.0)
    # a sink far below the scores changes nothing
    o = P.sink_attention(q, k, v, pos[2:], pos, 7.0, 10, 0, np.array([-50.0]))
    assert o[0, 0, 0] == pytest.approx(6.0)
    # the sink is not scaled: scores of 2 * scale against a sink of 2 * scale weigh the same
    q[:] = [1.0, 1.0]
    k[:] = [1.0, 1.0]
    o = P.sink_attention(q, k, v, pos[2:], pos, 0.5, 1, 0, np.array([1.0]))
    assert o[0, 0, 0] == pytest.approx(4.5)


def test_the_rotation_turns_neighbours_of_the_first_dimensions_only():
    x = np.arange(1.0, 7.0).reshape(1, 1, 6)
    y = P.rotate_pairs(x, np.array([2.0]), 4, 100.0)
    a0, a1 = 2.0, 2.0 * 100.0 ** (-0.5)
    assert y[0, 0, 0] == pytest.approx(1 * np.cos(a0) - 2 * np.sin(a0)) and y[0, 0, 1] == pytest.approx(2 * np.cos(a0) + 1 * np.sin(a0))
    assert y[0, 0, 2] == pytest.approx(3 * np.cos(a1) - 4 * np.sin(a1)) and y[0, 0, 4:].tolist() == [5.0, 6.0]


def test_the_router_by_hand():
    """Six outputs in three groups of which two stay; the correction chooses and does not weigh; a negative choice
    score inside a kept group still beats every output of a dropped group; the last output is an identity expert."""
    router = {"experts": 5, "identity": 1, "top": 2, "groups": {"count": 3, "keep": 2}}
    w = {"r.router": np.eye(6), "r.correction": np.array([0.0, 0.0, -2.0, -2.0, 0.0, 0.3])}
    h = np.log(np.array([[0.30, 0.05, 0.25, 0.05, 0.15, 0.20]]))             # softmax gives these scores back
    chosen, weights, gaps = P.route(h, w, "r.", router)
    # choice scores 0.30 0.05 | -1.75 -1.95 | 0.15 0.50: the groups 2 and 0 stay, their best outputs are 5 and 0
    assert chosen == [[5, 0]] and weights[0] == pytest.approx([0.20, 0.30]) and gaps[0] == pytest.approx(0.15)
    # with only the middle group to choose from, both of its (negative) outputs are taken
    w["r.correction"] = np.array([-5.0, -5.0, -2.0, -2.0, -5.0, -5.0])
    router["groups"]["keep"] = 1
    chosen, weights, _ = P.route(h, w, "r.", router)
    assert chosen == [[2, 3]] and weights[0] == pytest.approx([0.25, 0.05])
    # the identity expert hands the token's own row on, times its weight
    cfg_mlp = {"kind": "moe", "expert": {"ff": 2}, "router": {"experts": 1, "identity": 1, "top": 1}}
    ww = {"m.router": np.array([[0.0, 0.0], [50.0, 0.0]]), "m.correction": np.zeros(2), "m.e0.gate": np.ones((2, 2)),
          "m.e0.up": np.ones((2, 2)), "m.e0.down": np.ones((2, 2))}
    out = P.experts_ff(np.array([[1.0, 2.0]]), ww, "m.", cfg_mlp)
    assert out[0] == pytest.approx([1.0, 2.0])


def test_the_state_decays_by_its_head():
    q = np.ones((3, 2, 1))
    k = np.ones((3, 2, 1))
    v = np.array([[[1.0], [1.0]], [[0.0], [0.0]], [[0.0], [0.0]]])
    state = np.zeros((2, 1, 1))
    o = P.decayed_state_walk(q, k, v, [0.5, 1.0], state)
    assert o[:, 0, 0].tolist() == [1.0, 0.5, 0.25] and o[:, 1, 0].tolist() == [1.0, 1.0, 1.0]
    assert state[:, 0, 0].tolist() == [0.25, 1.0]
