"""The kernels of the Dagezen design alone, each against the plain function of its mechanism
(tests/plain/dagezen_plain.py), at sizes that are no power of two and differ from one another.

Like tests/test_kernels_gpu.py these run without a GPU when the environment says RI_TEST_KERNELS=emulated
(tests/test_kernels_emulated.py starts that run): the CPU build of the same sources between guard pages."""
import math
import os

import numpy as np
import pytest
import torch

from plain import dagezen_plain as P

EMULATED = os.environ.get("RI_TEST_KERNELS") == "emulated"
pytestmark = [] if EMULATED else pytest.mark.gpu
DEV = "cpu" if EMULATED else "cuda:0"
PAGE = 32


@pytest.fixture(scope="module")
def ops():
    if EMULATED:
        import emulated
        return emulated.ops()
    from rust_inference_amd.kernels import ops
    return ops


@pytest.fixture(autouse=True)
def _guarded_buffers_go_back():
    yield
    if EMULATED:
        import gc
        import emulated
        gc.collect()
        emulated.free_all()


def guarded(x):
    if EMULATED:
        import emulated
        return emulated.tensor(x.contiguous(), "a test's operand")
    return x


def t(a, dtype=torch.float32):
    return guarded(torch.tensor(np.asarray(a), dtype=dtype, device=DEV))


def f64(x):
    return x.detach().to("cpu", torch.float64).numpy()


def close(got, want, rel, what=""):
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(f64(got) - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= rel, f"{what}: error {err:.3e} of the largest value exceeds {rel:.0e}"


F32 = 5e-6


class Steps:
    """Sequences of unequal lengths cut into steps, with pages handed out in shuffled order: what a kernel gets of a
    step's layout (``tok_seq``, ``tok_pos``, ``cu_seqlens``, ``slots``, the page table)."""

    def __init__(self, lengths, slots, rng, pages=64):
        self.lengths, self.slots, self.done = list(lengths), list(slots), [0] * len(lengths)
        order = rng.permutation(pages)
        width = max(-(-n // PAGE) for n in lengths)
        self.table = np.full((len(lengths), width), -1, dtype=np.int32)
        at = 0
        for s, n in enumerate(lengths):
            for p in range(-(-n // PAGE)):
                self.table[s, p] = order[at]
                at += 1
        self.pages = pages

    def step(self, counts):
        """The next ``counts[s]`` tokens of every sequence (0: the sequence sits this step out)."""
        seqs = [s for s, c in enumerate(counts) if c > 0]
        tok_seq, tok_pos, cu, rows = [], [], [0], []
        for i, s in enumerate(seqs):
            for j in range(counts[s]):
                tok_seq.append(i)
                tok_pos.append(self.done[s] + j)
                rows.append((s, self.done[s] + j))
            cu.append(len(tok_seq))
            self.done[s] += counts[s]
        return dict(seqs=seqs, rows=rows, tok_seq=t(tok_seq, torch.int32), tok_pos=t(tok_pos, torch.int32),
                    cu=t(cu, torch.int32), slots=t([self.slots[s] for s in seqs], torch.int32),
                    table=t(self.table[seqs], torch.int32))


CUTS = [[(7, 3), (1, 1), (1, 0), (30, 36), (2, 1), (1, 1), (1, 1)]]      # (tokens of sequence 0, of sequence 1) step by step


# ---------------------------------------------------------------- the norm behind the sum, activations, the cap
@pytest.mark.parametrize("act", [None, torch.bfloat16])
@pytest.mark.parametrize("parts, dim", [(1, 70), (3, 256)])
def test_scaled_sum_norm(ops, act, parts, dim):
    rng = np.random.default_rng(1)
    rows, alpha, eps = 5, 2.5, 1e-5
    r, y = rng.standard_normal((rows, dim)), rng.standard_normal((parts, rows, dim))
    yb, g, b = rng.standard_normal(dim), 1 + 0.1 * rng.standard_normal(dim), 0.1 * rng.standard_normal(dim)
    res = t(r)
    got = ops.scaled_sum_norm(res, t(y if parts > 1 else y[0]), t(yb), alpha, t(g), t(b), eps, ops.NORM_LAYER, act)
    want = P.layer_norm(alpha * r + y.sum(0) + yb, g, b, eps)
    close(res, want, F32, "the residual")
    if act is not None:
        close(got, want, 8e-3, "its copy")
    res = t(r)
    ops.scaled_sum_norm(res, t(y[0]), None, alpha, t(g), None, eps, ops.NORM_RMS, None)
    close(res, P.rms_unit(alpha * r + y[0], eps) * g, F32, "rms")


def test_clamped_gate_with_biases_and_the_experts_plain_activation_and_the_cap(ops):
    rng = np.random.default_rng(2)
    rows, ff, limit = 6, 37, 1.5
    gu, bg, bu = 2 * rng.standard_normal((rows, 2 * ff)), rng.standard_normal(ff), rng.standard_normal(ff)
    g = np.minimum(gu[:, :ff] + bg, limit)
    u = np.clip(gu[:, ff:] + bu, -limit, limit)
    close(ops.glu_clamped_bias(t(gu), t(bg), t(bu), limit), g * P.sigmoid(1.702 * g) * (u + 1), F32, "clamped gate")
    wide = 2 * rng.standard_normal((3, 2 * 48))                       # bfloat16 rows of a multiple of 8: eight elements a thread
    gb, ub = rng.standard_normal(48), rng.standard_normal(48)
    rounded = f64(t(wide, torch.bfloat16))
    g8, u8 = np.minimum(rounded[:, :48] + gb, limit), np.clip(rounded[:, 48:] + ub, -limit, limit)
    close(ops.glu_clamped_bias(t(wide, torch.bfloat16), t(gb), t(ub), limit), g8 * P.sigmoid(1.702 * g8) * (u8 + 1), 8e-3,
          "clamped gate, bfloat16")
    experts = 5
    up, dense = rng.standard_normal((rows, experts * ff)), rng.random((rows, experts)) * (rng.random((rows, experts)) < 0.5)
    want = (P.gelu_erf(up).reshape(rows, experts, ff) * dense[:, :, None]).reshape(rows, -1)
    close(ops.experts_activate_plain(t(up), t(dense), ff, "gelu_erf"), want, F32, "experts without a gate")
    close(ops.gelu_erf(t(up)), P.gelu_erf(up), F32, "exact gelu")
    x = 40 * rng.standard_normal((3, 50))
    close(ops.softcap_rows(t(x), 15.0), 15.0 * np.tanh(x / 15.0), F32, "cap")


# ---------------------------------------------------------------- attention over a cached latent
@pytest.mark.parametrize("heads, dim, rot, vdim, rank", [(3, 20, 6, 12, 28), (2, 8, 16, 24, 72)])
def test_latent_attention_through_every_cut(ops, heads, dim, rot, vdim, rank):
    rng = np.random.default_rng(3)
    width, eps, scale = 40, 1e-5, 0.3
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"dims": rot, "base": 100.0}}
    w = {"q": rng.standard_normal((heads * (dim + rot), width)) / 6, "dkv": rng.standard_normal((rank + rot, width)) / 6,
         "dkv.norm": 1 + 0.1 * rng.standard_normal(rank), "uk": rng.standard_normal((heads * dim, rank)) / 5,
         "uv": rng.standard_normal((heads * vdim, rank)) / 5, "sink": rng.standard_normal(heads),
         "g": rng.standard_normal((heads, width)) / 6, "o": np.eye(heads * vdim)}
    inv_freq = t(100.0 ** (-2.0 * np.arange(rot // 2) / rot))
    w_uk = t(w["uk"].reshape(heads, dim, rank))
    w_uv = t(np.ascontiguousarray(w["uv"].reshape(heads, vdim, rank).transpose(0, 2, 1)))
    lengths = [43, 43]
    h = [rng.standard_normal((n, width)) for n in lengths]
    steps = Steps(lengths, [0, 1], rng)
    k_pages = guarded(torch.zeros((steps.pages, 1, PAGE, rank + rot), device=DEV))
    v_pages = guarded(torch.zeros((steps.pages, 1, rank, PAGE), device=DEV))
    states = [{}, {}]
    for counts in CUTS[0]:
        st = steps.step(counts)
        x = np.stack([h[s][p] for s, p in st["rows"]])
        proj = t(np.concatenate([x @ w["q"].T, x @ w["dkv"].T, x @ w["g"].T], 1))
        qw = heads * (dim + rot)
        ops.latent_prepare(proj, 0, qw, t(w["dkv.norm"]), eps, inv_freq, st["tok_pos"], st["tok_seq"], st["table"], k_pages,
                           v_pages, heads, dim, rot, rank)
        q = ops.head_products(proj, 0, dim + rot, w_uk, heads, dim, rank, extra=rot)
        o = ops.attention(q, k_pages, v_pages, st["tok_pos"], st["tok_seq"], st["table"], heads, 1, rank + rot, None, scale,
                          sinks=t(w["sink"]))
        got = ops.head_products(o, 0, rank, w_uv, heads, rank, vdim, gates=proj, g_off=qw + rank + rot)
        want, at = [], 0
        for s in st["seqs"]:
            n = sum(1 for r in st["rows"] if r[0] == s)
            want.append(P.latent_mixer(x[at:at + n], w, "", m, eps, states[s]))
            at += n
        close(got, np.concatenate(want), 2e-5, f"latent attention, step {counts}")


# ---------------------------------------------------------------- the windowed attention whose heads talk
@pytest.mark.parametrize("heads, kv_heads, dim, window, shares", [(4, 2, 12, 9, 1), (3, 3, 20, 33, 2), (6, 1, 8, 70, 1), (20, 2, 16, None, 3)])
def test_talking_attention_through_every_cut(ops, heads, kv_heads, dim, window, shares):
    rng = np.random.default_rng(4)
    width, eps, scale = 36, 1e-5, 0.4
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "mask": {"size": window or 10 ** 6}}
    w = {"q": rng.standard_normal((heads * dim, width)) / 3, "k": rng.standard_normal((kv_heads * dim, width)) / 3,
         "q.norm": 1 + 0.1 * rng.standard_normal(heads * dim), "k.norm": 1 + 0.1 * rng.standard_normal(kv_heads * dim),
         "r1": rng.random(heads), "r2": rng.random(heads) * 3, "talk": np.eye(heads) + 0.3 * rng.standard_normal((heads, heads)),
         "g": rng.standard_normal((heads * dim, width)) / 6, "o": np.eye(heads * dim)}
    lengths = [43, 43]
    h = [rng.standard_normal((n, width)) for n in lengths]
    steps = Steps(lengths, [1, 0], rng)
    k_pages = guarded(torch.zeros((steps.pages, kv_heads, PAGE, dim), device=DEV))
    v_pages = guarded(torch.zeros((steps.pages, kv_heads, dim, PAGE), device=DEV))
    states = [{}, {}]
    for counts in CUTS[0]:
        st = steps.step(counts)
        x = np.stack([h[s][p] for s, p in st["rows"]])
        proj = t(np.concatenate([x @ w["q"].T, x @ w["k"].T, x @ w["g"].T], 1))
        qw, kw = heads * dim, kv_heads * dim
        ops.whole_norm_kv_write(proj, 0, qw, t(w["q.norm"]), t(w["k.norm"]), eps, st["tok_pos"], st["tok_seq"], st["table"],
                                k_pages, v_pages, heads, kv_heads, dim)
        o = ops.talking_attention(proj, 0, k_pages, v_pages, st["tok_pos"], st["tok_seq"], st["table"], heads, kv_heads, dim,
                                  window, scale, t(w["r1"]), t(w["r2"]), t(w["talk"]), shares)
        got = guarded(torch.zeros((len(x), qw + 3), device=DEV))
        ops.gate_rows(got, 3, o, proj, qw + kw, 0.5, ops.GATE_SIGMOID)
        want, at = [], 0
        for s in st["seqs"]:
            n = sum(1 for r in st["rows"] if r[0] == s)
            want.append(P.talking_mixer(x[at:at + n], w, "", m, eps, states[s]))
            at += n
        close(got[:, 3:], 0.5 * np.concatenate(want), 2e-5, f"talking attention, step {counts}")


def test_a_key_at_the_windows_edge_counts_and_the_next_one_does_not(ops):
    """One loud key: at distance window - 1 it takes the softmax, at distance window it is not seen."""
    heads, dim, window, n = 2, 8, 37, 80
    k_pages = guarded(torch.zeros((4, 1, PAGE, dim), device=DEV))
    v_pages = guarded(torch.zeros((4, 1, dim, PAGE), device=DEV))
    for edge, seen in ((window - 1, True), (window, False)):
        loud = n - 1 - edge
        k_pages.zero_(), v_pages.zero_()
        k_pages[loud // PAGE, 0, loud % PAGE, :] = 30.0
        v_pages[loud // PAGE, 0, 0, loud % PAGE] = 1.0
        q = t(np.ones((1, heads * dim)))
        o = ops.talking_attention(q, 0, k_pages, v_pages, t([n - 1], torch.int32), t([0], torch.int32),
                                  t([[0, 1, 2, 3]], torch.int32), heads, 1, dim, window, 1.0, None, None, None, 1 if seen else 2)
        assert (f64(o)[0, 0] > 0.99) == seen


# ---------------------------------------------------------------- time mixing
@pytest.mark.parametrize("columns", [True, False])
@pytest.mark.parametrize("heads, dim", [(3, 12), (2, 40), (1, 70), (1, 130)])
def test_time_mixing_through_every_cut(ops, heads, dim, columns):
    rng = np.random.default_rng(5)
    width, eps, rank = 30, 1e-5, 5
    hw = heads * dim
    m = {"heads": heads, "dim": dim}
    w = {x: rng.standard_normal((hw, width)) / 3 for x in "rkvg"}
    w.update({"mu." + s: rng.random(width) for s in "rkvgw"})
    w.update({"w1": rng.standard_normal((rank, width)) / 3, "w2": rng.standard_normal((hw, rank)), "w0": rng.standard_normal(hw) - 1,
              "u": rng.standard_normal((heads, dim)), "norm": 1 + 0.1 * rng.standard_normal(hw), "o": np.eye(hw)})
    lengths = [43, 43]
    h = [rng.standard_normal((n, width)) for n in lengths]
    steps = Steps(lengths, [2, 0], rng)
    state = guarded(torch.zeros((3, heads, dim, dim), device=DEV))
    kept = guarded(torch.zeros((3, width), device=DEV))
    mu = t(np.stack([w["mu." + s] for s in "rkvgw"]))
    states = [{}, {}]
    for counts in CUTS[0]:
        st = steps.step(counts)
        x = np.stack([h[s][p] for s, p in st["rows"]])
        x32 = t(x)
        mixes = ops.shift_mix(x32, kept, mu, st["tok_seq"], st["cu"], st["slots"], torch.float32)
        ops.shift_keep(kept, x32, st["cu"], st["slots"])
        mx = f64(mixes)
        r, k, v, g = (t(mx[i] @ w[s].T) for i, s in enumerate("rkvg"))
        z = t(np.tanh(mx[4] @ w["w1"].T) @ w["w2"].T)
        out = guarded(torch.zeros((len(x), hw + 2), device=DEV))
        ops.timemix_scan(out, 2, 0.7, r, k, v, g, z, t(w["w0"]), t(w["u"].reshape(-1)), t(w["norm"]), eps, state, st["cu"],
                         st["slots"], heads, dim, columns)
        want, at = [], 0
        for s in st["seqs"]:
            n = sum(1 for r_ in st["rows"] if r_[0] == s)
            want.append(P.time_mixer(x[at:at + n], w, "", m, eps, states[s]))
            at += n
        close(out[:, 2:], 0.7 * np.concatenate(want), 3e-5, f"time mixing, step {counts}")
    close(ops.tanh_rows(t(x), torch.float32), np.tanh(x), F32, "tanh")


# ---------------------------------------------------------------- the state-space mixer
@pytest.mark.parametrize("columns", [True, False])
@pytest.mark.parametrize("heads, vdim, n, groups, taps, parts", [(4, 12, 10, 2, 3, 2), (2, 20, 40, 1, 1, 5), (3, 8, 70, 3, 5, 1),
                                                                 (1, 70, 130, 1, 2, 1)])
def test_state_space_mixer_through_every_cut(ops, heads, vdim, n, groups, taps, parts, columns):
    rng = np.random.default_rng(6)
    width, eps = 30, 1e-5
    inner = heads * vdim
    channels = inner + 2 * groups * n
    m = {"heads": heads, "vdim": vdim, "state": n, "groups": groups, "conv": taps, "norm_groups": parts}
    w = {"in": rng.standard_normal((inner + channels + heads, width)) / 3, "conv": rng.standard_normal((channels, taps)) / 2,
         "conv.b": rng.standard_normal(channels) / 3, "dt_bias": rng.standard_normal(heads), "A_log": rng.standard_normal(heads),
         "D": rng.standard_normal(heads), "norm": 1 + 0.1 * rng.standard_normal(inner), "o": np.eye(inner)}
    lengths = [43, 43]
    h = [rng.standard_normal((k, width)) for k in lengths]
    steps = Steps(lengths, [1, 2], rng)
    state = guarded(torch.zeros((3, heads, n, vdim), device=DEV))
    tails = guarded(torch.zeros((3, max(taps - 1, 1), channels), device=DEV))
    states = [{}, {}]
    for counts in CUTS[0]:
        st = steps.step(counts)
        x = np.stack([h[s][p] for s, p in st["rows"]])
        proj = t(x @ w["in"].T)
        xbc = ops.causal_conv_silu(proj, inner, channels, t(w["conv"]), t(w["conv.b"]), tails, st["tok_seq"], st["cu"], st["slots"])
        y = ops.ssd_scan(xbc, inner, inner + groups * n, proj, 0, inner + channels, t(w["dt_bias"]), t(w["A_log"]), t(w["D"]),
                         state, st["cu"], st["slots"], heads, groups, n, vdim, columns)
        got = ops.group_rms_norm(y, t(w["norm"]), eps, parts, torch.float32)
        want, at = [], 0
        for s in st["seqs"]:
            k = sum(1 for r in st["rows"] if r[0] == s)
            want.append(P.mamba2_mixer(x[at:at + k], w, "", m, eps, states[s]))
            at += k
        close(got, np.concatenate(want), 3e-5, f"state-space mixer, step {counts}")


# ---------------------------------------------------------------- the products per head through the library
@pytest.mark.parametrize("heads, k, n, extra, gated", [(3, 24, 40, 6, False), (5, 40, 12, 0, True), (2, 16, 16, 10, True)])
def test_batched_head_products_are_the_products_per_head(ops, heads, k, n, extra, gated):
    """bfloat16 rows with the heads somewhere inside a wider row, columns in front and behind: the batched product with the
    copied elements and a gate a head against the sums written out in float64, and beside the kernel that does it alone."""
    rng = np.random.default_rng(heads)
    tokens, x_off, x_head = 37, 5, k + extra + 3
    stride = x_off + heads * x_head + heads + 4
    x = t(rng.standard_normal((tokens, stride)), torch.bfloat16)
    w = t(rng.standard_normal((heads, k, n)) / 4, torch.bfloat16)
    g_off = x_off + heads * x_head + 2
    got = ops.head_products_batched(x, x_off, x_head, w, heads, k, n, extra=extra, gates=x if gated else None, g_off=g_off)
    alone = ops.head_products(x, x_off, x_head, w, heads, k, n, extra=extra, gates=x if gated else None, g_off=g_off)
    xs, ws = f64(x), f64(w)
    want = np.zeros((tokens, heads, n + extra))
    for h in range(heads):
        rows = xs[:, x_off + h * x_head: x_off + (h + 1) * x_head]
        want[:, h, :n] = rows[:, :k] @ ws[h]
        want[:, h, n:] = rows[:, k:k + extra]
        if gated:
            want[:, h] *= (1 / (1 + np.exp(-xs[:, g_off + h])))[:, None]
    want = want.reshape(tokens, -1)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == want.shape
    close(got, want, 1.2e-2, "batched products per head")          # two roundings to bfloat16 with a gate, one without
    close(alone, want, 6e-3, "products per head")


# ---------------------------------------------------------------- the latent attention on the matrix cores
@pytest.mark.parametrize("heads", [3, 20])
def test_latent_attention_on_the_matrix_cores_is_the_general_kernel(ops, heads):
    """bfloat16, key rows of 160 and value rows of 128: tokens at the start of a sequence, at a page's border and inside a
    page, of two sequences whose pages lie in shuffled order, with sinks; against the general kernel on the same pages."""
    rng = np.random.default_rng(11)
    dk, rank, pages = 160, 128, 12
    k_pages = guarded((torch.randn((pages, 1, PAGE, dk), device=DEV) * 0.5).to(torch.bfloat16))
    v_pages = guarded(k_pages[:, :, :, :rank].transpose(2, 3).contiguous())
    table = t([[5, 2, 9, 0], [7, 1, 3, 11]], torch.int32)
    tok_seq, tok_pos = t([0, 0, 0, 1, 1, 1, 1], torch.int32), t([0, 31, 32, 5, 63, 64, 100], torch.int32)
    q = guarded((torch.randn((7, heads * dk), device=DEV) * 0.5).to(torch.bfloat16))
    sinks = t(rng.standard_normal(heads))
    for sink in (sinks, None):
        want = ops.attention(q, k_pages, v_pages, tok_pos, tok_seq, table, heads, 1, dk, None, 0.11, sinks=sink)
        got = ops.latent_attention_mfma(q, k_pages, v_pages, tok_pos, tok_seq, table, heads, 0.11, sink)
        close(got, f64(want), 1.2e-2, "matrix cores against the general kernel")
        for bound in (101, 128, 1024):                    # chunks of one page, of one page with more room than pages, of eight
            got = ops.latent_attention_mfma(q, k_pages, v_pages, tok_pos, tok_seq, table, heads, 0.11, sink, bound)
            close(got, f64(want), 1.2e-2, f"in chunks, sequences of up to {bound}")


@pytest.mark.parametrize("heads, kv_heads, dim, window", [(8, 2, 32, 40), (16, 16, 32, None), (8, 1, 64, 33)])
def test_talking_attention_on_the_matrix_cores_is_the_general_kernel(ops, heads, kv_heads, dim, window):
    """bfloat16: two sequences whose pages lie in shuffled order, one that goes on from 37 cached tokens with 21 new ones
    (two tiles, the second partial) and one that starts with 50; with the distance bias and the mixing matrix, and without;
    against the general kernels on the same pages."""
    rng = np.random.default_rng(12)
    pages = 10
    k_pages = guarded((torch.randn((pages, kv_heads, PAGE, dim), device=DEV) * 0.6).to(torch.bfloat16))
    v_pages = guarded((torch.randn((pages, kv_heads, dim, PAGE), device=DEV) * 0.6).to(torch.bfloat16))
    table = t([[5, 2, 9], [7, 1, 3]], torch.int32)
    counts, starts = [21, 50], [37, 0]
    tok_seq = t([0] * 21 + [1] * 50, torch.int32)
    tok_pos = t(list(range(37, 58)) + list(range(50)), torch.int32)
    cu = t([0, 21, 71], torch.int32)
    proj = guarded((torch.randn((71, heads * dim + 16), device=DEV) * 0.6).to(torch.bfloat16))
    r1, r2 = t(rng.random(heads)), t(rng.random(heads) * 3)
    talk = t(np.eye(heads) + 0.3 * rng.standard_normal((heads, heads)))
    for a, b, c in ((r1, r2, talk), (None, None, None)):
        want = ops.talking_attention(proj, 8, k_pages, v_pages, tok_pos, tok_seq, table, heads, kv_heads, dim, window, 0.2, a, b, c)
        got = ops.talking_attention_mfma(proj, 8, k_pages, v_pages, tok_pos, cu, counts, table, heads, kv_heads, dim, window, 0.2,
                                         a, b, c)
        close(got, f64(want), 1.5e-2, "matrix cores against the general kernels")
