"""The kernels of the Zakelorn design alone, each against the plain function of its mechanism
(tests/plain/zakelorn_plain.py), at sizes that are no power of two and differ from one another.

Like tests/test_kernels_gpu.py these run without a GPU when the environment says RI_TEST_KERNELS=emulated
(tests/test_kernels_emulated.py starts that run): the CPU build of the same sources between guard pages."""
import math
import os

import numpy as np
import pytest
import torch

from plain import zakelorn_plain as P

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


def bf16_round(a):
    return torch.tensor(a).to(torch.bfloat16).to(torch.float64).numpy()


F32 = 3e-6
BF16_OUT = 7.5e-3


# ---------------------------------------------------------------- embedding, norm on a sublayer's output
@pytest.mark.parametrize("act", [None, torch.bfloat16])
def test_the_embedding_times_a_constant(ops, act):
    rng = np.random.default_rng(0)
    table = bf16_round(rng.normal(size=(37, 52)))
    ids = [5, 0, 36, 5]
    odd, _ = ops.embed_scaled(t(table[:, :51].copy(), torch.bfloat16), t(ids, torch.int32), 6.25, act)
    close(odd, table[ids, :51] * 6.25, 1e-7)
    out, rows = ops.embed_scaled(t(table, torch.bfloat16), t(ids, torch.int32), 6.25, act)
    close(out, table[ids] * 6.25, 1e-7)
    assert (rows is None) == (act is None)
    if act is not None:
        close(rows, table[ids] * 6.25, BF16_OUT)


@pytest.mark.parametrize("dim, rows, parts, act", [(52, 5, 1, None), (200, 3, 3, torch.bfloat16), (1030, 2, 1, torch.bfloat16),
                                                   (1300, 2, 2, torch.bfloat16), (4096, 2, 4, torch.bfloat16), (5000, 1, 1, None),
                                                   (8196, 1, 2, torch.bfloat16)])
def test_the_norm_on_a_sublayers_output_with_the_layer_scale(ops, dim, rows, parts, act):
    """residual += ls * layernorm(y): a mean far from zero and a small spread, which a variance taken as the mean of
    the squares minus the squared mean would lose in float32."""
    rng = np.random.default_rng(dim)
    x = rng.normal(size=(rows, dim)) * 3
    y = rng.normal(size=(parts, rows, dim)) * 0.01 + 40.0 / parts
    y = y.astype(np.float32).astype(np.float64)
    w, b, ls = 1 + 0.2 * rng.normal(size=dim), rng.normal(size=dim), rng.normal(size=dim)
    want = x.astype(np.float32).astype(np.float64) + ls * P.layer_norm(y.sum(0), w, b, 1e-5)
    from rust_inference_amd.kernels import ops as real
    res = t(x)
    rows_act = ops.branch_norm_add(res, t(y if parts > 1 else y[0]), t(w), t(b), 1e-5, real.NORM_LAYER, t(ls), act)
    close(res, want, 2e-4, "residual")                       # (the spread is 1e-4 of the mean: float32 keeps three digits of it)
    if act is not None:
        close(rows_act, want, BF16_OUT, "the copy for the products")
    # the same without bias and layer scale, as an RMS norm
    res = t(x)
    y1 = rng.normal(size=(rows, dim))
    ops.branch_norm_add(res, t(y1), t(w), None, 1e-5, real.NORM_RMS, None, None)
    y1 = y1.astype(np.float32).astype(np.float64)
    close(res, x.astype(np.float32) + P.rms_unit(y1, 1e-5) * w, F32, "rms")


# ---------------------------------------------------------------- rotation of neighbours, unit norm, the cache write
def paged(k, v, order, dtype):
    """Keys ``[T, G, dim]`` and values ``[T, G, vdim]`` of one sequence in pages handed out in ``order``."""
    T, G, dim = k.shape
    vdim = v.shape[2]
    pages = -(-T // PAGE)
    kp = torch.zeros((len(order), G, PAGE, dim), dtype=dtype)
    vp = torch.zeros((len(order), G, vdim, PAGE), dtype=dtype)
    for j in range(T):
        kp[order[j // PAGE], :, j % PAGE] = torch.tensor(k[j]).to(dtype)
        vp[order[j // PAGE], :, :, j % PAGE] = torch.tensor(v[j]).to(dtype)
    table = torch.tensor([list(order[:pages]) + [-1] * 2], dtype=torch.int32)
    return guarded(kp.to(DEV)), guarded(vp.to(DEV)), guarded(table.to(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv, dim, vdim, rot, lens", [(4, 2, 24, 40, 10, (35, 1, 3)), (3, 3, 64, 64, 64, (70,)),
                                                            (2, 1, 6, 4, 0, (2, 33)), (8, 2, 128, 128, 32, (5, 1)),
                                                            (2, 2, 64, 32, 12, (40, 3)), (1, 1, 512, 8, 500, (2,))])
def test_rotation_unit_norm_and_cache_write(ops, dtype, heads, kv, dim, vdim, rot, lens):
    """q and k turn in neighbouring pairs over their first ``rot`` elements, then every head is divided by its root mean
    square; q stays in the projection's rows, k and v go to the pages.  The mixer's columns start inside a wider row
    (another mixer's columns before them), and the sequences start at positions of their own."""
    rng = np.random.default_rng(heads + dim)
    T, base, eps, before = sum(lens), 700.0, 1e-5, 16
    row = before + (heads + kv) * dim + kv * vdim + 8
    proj = rng.normal(size=(T, row)).astype(np.float32).astype(np.float64)
    if dtype == torch.bfloat16:
        proj = bf16_round(proj)
    starts = [40, 0, 31][:len(lens)]
    pos = np.concatenate([np.arange(s, s + n) for s, n in zip(starts, lens)])
    seq = np.repeat(np.arange(len(lens)), lens)
    cu = np.concatenate([[0], np.cumsum(lens)])
    q_at, k_at, v_at = before, before + heads * dim, before + (heads + kv) * dim
    q = proj[:, q_at:k_at].reshape(T, heads, dim)
    k = proj[:, k_at:v_at].reshape(T, kv, dim)
    v = proj[:, v_at:v_at + kv * vdim].reshape(T, kv, vdim)
    want_q = P.rms_unit(P.rotate_pairs(q, pos.astype(np.float64), rot, base), eps)
    want_k = P.rms_unit(P.rotate_pairs(k, pos.astype(np.float64), rot, base), eps)
    n_pages = sum(-(-(s + n) // PAGE) for s, n in zip(starts, lens)) + 1
    order = rng.permutation(n_pages)
    width = max(-(-(s + n) // PAGE) for s, n in zip(starts, lens)) + 1
    table = np.full((len(lens), width), -1, dtype=np.int32)
    nxt = 0
    for b, (s, n) in enumerate(zip(starts, lens)):
        for p in range(-(-(s + n) // PAGE)):
            table[b, p] = order[nxt]
            nxt += 1
    kp = guarded(torch.zeros((n_pages, kv, PAGE, dim), dtype=dtype, device=DEV))
    vp = guarded(torch.zeros((n_pages, kv, vdim, PAGE), dtype=dtype, device=DEV))
    inv = t([base ** (-2.0 * i / rot) for i in range(rot // 2)]) if rot else None
    dev = t(proj, dtype)
    ops.qk_pairs_norm_kv_write(dev, q_at, k_at, v_at, inv, None, None, True, eps, t(pos, torch.int32), t(seq, torch.int32),
                               t(table, torch.int32), kp, vp, heads, kv, dim, vdim, t(cu, torch.int32), max(lens))
    tol = 5e-6 if dtype == torch.float32 else BF16_OUT      # (float32 angles at positions up to 110)
    got = f64(dev)
    close(dev[:, q_at:k_at], want_q.reshape(T, -1), tol, "q")
    # what is not q stays as it was: the columns before, the gate's columns behind
    assert np.array_equal(got[:, :before], proj[:, :before]) and np.array_equal(got[:, -8:], proj[:, -8:])
    for i in range(T):
        page, at = table[seq[i], pos[i] // PAGE], pos[i] % PAGE
        close(kp[page, :, at], want_k[i], tol, "k in its page")
        close(vp[page, :, :, at], v[i], 1e-7, "v in its page")


# ---------------------------------------------------------------- attention: window, kept first tokens, sinks
def plain_attention(q, k, v, new, scale, window, keep, sinks):
    pos = np.arange(k.shape[0], dtype=np.float64)
    return P.sink_attention(q, k, v, pos[new], pos, scale, window if window else math.inf, keep, sinks)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv, dim, vdim, window, keep, T", [(6, 2, 24, 24, 7, 3, 75), (3, 3, 16, 40, None, 0, 70),
                                                                  (4, 1, 64, 64, 33, 40, 300), (2, 2, 20, 12, 1, 1, 40),
                                                                  (2, 1, 8, 8, 5, 0, 50), (4, 4, 48, 16, 40, 33, 130)])
def test_generic_attention_with_kept_first_tokens_and_sinks(ops, dtype, heads, kv, dim, vdim, window, keep, T):
    rng = np.random.default_rng(heads * 10 + dim)
    q, k, v = rng.normal(size=(T, heads, dim)), rng.normal(size=(T, kv, dim)), rng.normal(size=(T, kv, vdim))
    sinks = rng.normal(size=heads) * 2
    if dtype == torch.bfloat16:
        q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    new = sorted(set(list(range(T - 9, T)) + [0, 1, keep, (window or 3), (window or 3) + keep, T // 2]))
    want = plain_attention(q[new], k, v, new, 0.31, window, keep, sinks)
    order = list(rng.permutation(-(-T // PAGE) + 2))
    kp, vp, table = paged(k, v, order, dtype)
    # the queries start at a column of their own inside wider rows
    rows = np.concatenate([np.zeros((len(new), 8)), q[new].reshape(len(new), -1), np.ones((len(new), 5))], 1)
    got = ops.attention(t(rows, dtype), kp, vp, t(new, torch.int32), t([0] * len(new), torch.int32), table, heads, kv, dim,
                        window, 0.31, None, None, keep_first=keep, sinks=t(sinks), q_off=8)
    close(got, want.reshape(len(new), -1), F32 if dtype == torch.float32 else BF16_OUT)


def loud_case(T, heads, dim, window, keep):
    """Every key has the same product with every query, so all visible keys weigh the same, and the values are one-hot
    in the key's position (modulo the value size): the result counts the visible keys by their places, and a key
    more or less moves it by one part in the number of keys seen."""
    q = np.zeros((T, heads, dim)); q[..., 0] = 2.0
    k = np.zeros((T, 1, dim)); k[..., 0] = 1.5
    v = np.zeros((T, 1, dim))
    v[np.arange(T), 0, np.arange(T) % dim] = 1.0
    return q, k, v


@pytest.mark.parametrize("window, keep", [(32, 0), (33, 1), (31, 32), (64, 33), (7, 31), (1, 2), (40, 64), (96, 5)])
def test_keys_at_the_edges_of_window_and_kept_tokens_generic(ops, window, keep):
    T, heads, dim = 200, 2, 16
    q, k, v = loud_case(T, heads, dim, window, keep)
    sinks = np.array([-30.0, 0.0])
    new = list(range(T))
    want = plain_attention(q, k, v, new, 1.0, window, keep, sinks)
    # the plain form itself tells the edges: a wider window or one kept token more gives another result
    assert np.abs(plain_attention(q, k, v, new, 1.0, window + 1, keep, sinks) - want).max() > 1e-3
    assert np.abs(plain_attention(q, k, v, new, 1.0, window, keep + 1, sinks) - want).max() > 1e-3
    kp, vp, table = paged(k, v, list(np.random.default_rng(window).permutation(9)), torch.float32)
    got = ops.attention(t(q.reshape(T, -1)), kp, vp, t(new, torch.int32), t([0] * T, torch.int32), table, heads, 1, dim,
                        window, 1.0, None, None, keep_first=keep, sinks=t(sinks))
    close(got, want.reshape(T, -1), F32)


def paged_batch(k, v, lens, seed):
    """Keys and values of several sequences (flat, one after the other) in pages handed out in shuffled order."""
    G, dk, dv = k.shape[1], k.shape[2], v.shape[2]
    width = max(-(-n // PAGE) for n in lens) + 1
    n_pages = sum(-(-n // PAGE) for n in lens) + 2
    order = np.random.default_rng(seed).permutation(n_pages)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    kp = torch.zeros((n_pages, G, PAGE, dk), dtype=torch.bfloat16)
    vp = torch.zeros((n_pages, G, dv, PAGE), dtype=torch.bfloat16)
    nxt = at = 0
    for b, n in enumerate(lens):
        for p in range(-(-n // PAGE)):
            table[b, p] = order[nxt]
            nxt += 1
        for j in range(n):
            kp[table[b, j // PAGE], :, j % PAGE] = torch.tensor(k[at + j]).bfloat16()
            vp[table[b, j // PAGE], :, :, j % PAGE] = torch.tensor(v[at + j]).bfloat16()
        at += n
    return guarded(kp.to(DEV)), guarded(vp.to(DEV)), t(table, torch.int32)


@pytest.mark.parametrize("form", ["prompts", "single tokens", "portions"])
@pytest.mark.parametrize("dh, heads, kv_heads, window, keep", [(64, 8, 4, 41, 20), (128, 4, 1, None, 0), (32, 2, 2, 33, 32),
                                                               (64, 6, 3, 70, 3), (64, 16, 1, 7, 70), (128, 2, 2, 64, 33)])
def test_matrix_core_attention_with_kept_first_tokens_and_sinks(ops, form, dh, heads, kv_heads, window, keep):
    """bfloat16, heads of 32, 64 and 128: prompts of unequal lengths; one new token each after them; the last tokens of
    each as a portion.  Kept tokens that end inside a page, at a page's end, behind the window's first page."""
    rng = np.random.default_rng(dh + heads)
    lens = [75, 1, 40] if form == "prompts" else [300, 33, 164]
    T = sum(lens)
    q, k, v = (bf16_round(rng.normal(size=(T, heads, dh))), bf16_round(rng.normal(size=(T, kv_heads, dh))),
               bf16_round(rng.normal(size=(T, kv_heads, dh))))
    sinks = rng.normal(size=heads) * 2
    kp, vp, table = paged_batch(k, v, lens, dh)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    want = np.concatenate([plain_attention(q[a:b], k[a:b], v[a:b], list(range(b - a)), 0.21, window, keep, sinks).reshape(b - a, -1)
                           for a, b in zip(cu[:-1], cu[1:])])
    tail = {"prompts": None, "single tokens": 1, "portions": 19}[form]
    rows, pos, new_cu = [], [], [0]
    for a, b in zip(cu[:-1], cu[1:]):
        first = a if tail is None else max(a, b - tail)
        rows += list(range(first, b))
        pos += list(range(first - a, b - a))
        new_cu.append(len(rows))
    counts = np.diff(new_cu)
    # the queries sit behind 16 other columns of a wider row
    wide = np.concatenate([np.zeros((len(rows), 16)), q[rows].reshape(len(rows), -1), np.zeros((len(rows), 8))], 1)
    got = ops.attention_prefill_bf16(t(wide, torch.bfloat16), kp, vp, t(new_cu, torch.int32), t(pos, torch.int32), table,
                                     len(lens), int(counts.max()), heads, kv_heads, dh, window, 0.21, None, None, keep, t(sinks), 16)
    close(got, want[rows], BF16_OUT, form)
    if form == "single tokens":                                # the same through the chunks side by side and their join
        got = ops.attention_decode_bf16(t(wide, torch.bfloat16), kp, vp, t(new_cu, torch.int32), t(pos, torch.int32), table,
                                        len(lens), max(lens), heads, kv_heads, dh, window, 0.21, keep_first=keep,
                                        sinks=t(sinks), q_off=16)
        close(got, want[rows], BF16_OUT, "chunks and join")


def test_kept_keys_and_a_sink_in_the_join_of_thousands_of_keys(ops):
    """5,000 keys (more chunks than the short join takes at once), a window of 300 and 40 kept keys of which one answers
    loudly: the join adds the first chunk to the window's two, and the sink to the denominator."""
    rng = np.random.default_rng(12)
    T, dh, window, keep, heads = 5000, 64, 300, 40, 4
    q, k, v = rng.normal(size=(1, heads, dh)) * 0.3, rng.normal(size=(T, 2, dh)) * 0.3, rng.normal(size=(T, 2, dh))
    q[0, :, 5] = 4.0
    k[keep - 1, :, 5] = k[keep, :, 5] = 3.0                   # the last kept key, and the first that is not
    q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    sinks = np.array([-20.0, 0.0, 3.0, 12.0])
    want = plain_attention(q, k, v, [T - 1], 1.0, window, keep, sinks).reshape(1, -1)
    assert np.abs(want[0, :dh] - v[keep - 1, 0]).max() < 0.05 * np.abs(v[keep - 1, 0]).max()
    assert np.abs(want[0, 3 * dh:]).max() < 0.6 * np.abs(want[0, :dh]).max()          # the large sink takes most of the weight
    kp, vp, table = paged_batch(k, v, [T], 3)
    row = t(q.reshape(1, -1), torch.bfloat16)
    got = ops.attention_decode_bf16(row, kp, vp, t([0, 1], torch.int32), t([T - 1], torch.int32), table, 1, T, heads, 2, dh,
                                    window, 1.0, keep_first=keep, sinks=t(sinks))
    close(got, want, BF16_OUT, "chunks and join")
    got = ops.attention_prefill_bf16(row, kp, vp, t([0, 1], torch.int32), t([T - 1], torch.int32), table, 1, 1, heads, 2, dh,
                                     window, 1.0, None, None, keep, t(sinks))
    close(got, want, BF16_OUT, "prompt kernel")


@pytest.mark.parametrize("dh", [32, 64])
@pytest.mark.parametrize("window, keep", [(32, 0), (33, 1), (31, 32), (64, 33), (7, 31), (1, 2), (40, 64), (96, 5)])
def test_keys_at_the_edges_of_window_and_kept_tokens_matrix_cores(ops, dh, window, keep):
    T, heads = 200, 2
    q, k, v = loud_case(T, heads, dh, window, keep)
    sinks = np.array([-30.0, 0.0])
    want = plain_attention(q, k, v, list(range(T)), 1.0, window, keep, sinks).reshape(T, -1)
    kp, vp, table = paged_batch(k, v, [T], window)
    for what, first in (("a prompt", 0), ("the last 70", T - 70), ("one token", T - 1), ("one token at 101", 101)):
        last = T if what != "one token at 101" else 102
        rows = list(range(first if what != "one token at 101" else 101, last))
        got = ops.attention_prefill_bf16(t(q[rows].reshape(len(rows), -1), torch.bfloat16), kp, vp, t([0, len(rows)], torch.int32),
                                         t(rows, torch.int32), table, 1, len(rows), heads, 1, dh, window, 1.0, None, None, keep,
                                         t(sinks))
        close(got, want[rows], 4e-3, what)
        if len(rows) == 1:
            got = ops.attention_decode_bf16(t(q[rows].reshape(1, -1), torch.bfloat16), kp, vp, t([0, 1], torch.int32),
                                            t(rows, torch.int32), table, 1, T, heads, 1, dh, window, 1.0, keep_first=keep,
                                            sinks=t(sinks))
            close(got, want[rows], 4e-3, what + ", chunks and join")


def test_one_far_kept_key_among_hundreds(ops):
    """One of the kept first tokens answers the last query loudly from 700 positions back, another just behind the
    kept ones as loudly but unseen: generic and matrix-core kernel give the kept one's value."""
    rng = np.random.default_rng(9)
    T, dh, window, keep = 720, 64, 50, 11
    q, k, v = rng.normal(size=(T, 2, dh)) * 0.1, rng.normal(size=(T, 1, dh)) * 0.1, rng.normal(size=(T, 1, dh))
    q[-1, :, 3] = 6.0
    k[keep - 1, 0, 3] = k[keep, 0, 3] = 5.0
    q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    sinks = np.zeros(2)
    want = plain_attention(q[-1:], k, v, [T - 1], 1.0, window, keep, sinks).reshape(1, -1)
    assert np.abs(want[0, :dh] - v[keep - 1, 0]).max() < 0.05 * np.abs(v[keep - 1, 0]).max()
    kp, vp, table = paged_batch(k, v, [T], 3)
    row = t(q[-1:].reshape(1, -1), torch.bfloat16)
    got = ops.attention_prefill_bf16(row, kp, vp, t([0, 1], torch.int32), t([T - 1], torch.int32), table, 1, 1, 2, 1, dh, window,
                                     1.0, None, None, keep, t(sinks))
    close(got, want, BF16_OUT, "matrix cores")
    got = ops.attention(row, kp, vp, t([T - 1], torch.int32), t([0], torch.int32), table, 2, 1, dh, window, 1.0, None, None,
                        keep_first=keep, sinks=t(sinks))
    close(got, want, BF16_OUT, "generic")


# ---------------------------------------------------------------- gates
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_gate_on_the_heads_and_the_norm_over_all_heads(ops, dtype):
    rng = np.random.default_rng(2)
    T, w, row = 5, 44, 120
    x, proj = rng.normal(size=(T, w)), rng.normal(size=(T, row)) * 2
    gain = 1 + 0.3 * rng.normal(size=w)
    if dtype == torch.bfloat16:
        proj = bf16_round(proj)
    xd = bf16_round(x) if dtype == torch.bfloat16 else x.astype(np.float32).astype(np.float64)
    out = t(np.full((T, 100), 7.0), dtype)
    ops.gate_rows(out, 8, t(x, dtype), t(proj, dtype), 60, 0.6)
    tol = F32 if dtype == torch.float32 else BF16_OUT
    close(out[:, 8:8 + w], 0.6 * xd * P.sigmoid(proj[:, 60:60 + w]), tol, "gate")
    assert (f64(out[:, :8]) == 7).all() and (f64(out[:, 8 + w:]) == 7).all()
    x32 = x.astype(np.float32).astype(np.float64)
    for g_off in (3, 12):                                     # columns that 16-byte loads do not take, and columns they do
        ops.row_norm_gate(out, 52, t(x), t(gain), 1e-5, t(proj, dtype), g_off, 0.9)
        close(out[:, 52:52 + w], 0.9 * P.rms_unit(x32, 1e-5) * gain * P.sigmoid(proj[:, g_off:g_off + w]), tol, "norm and gate")
        assert (f64(out[:, 8 + w:52]) == 7).all() and (f64(out[:, 52 + w:]) == 7).all()
    ops.gate_rows(out, 1, t(x, dtype), t(proj, dtype), 61, 0.6)              # odd columns: one element a thread
    close(out[:, 1:1 + w], 0.6 * xd * P.sigmoid(proj[:, 61:61 + w]), tol, "gate at odd columns")
    ops.gate_rows(out, 4, t(x, dtype), None, 0, 2.0)
    close(out[:, 4:4 + w], 2.0 * xd, tol, "no gate")


# ---------------------------------------------------------------- linear attention with a fixed decay
def plain_decay(proj, q_at, k_at, v_at, H, dk, dv, decay, lens, slots, state):
    out, at = [], 0
    for b, n in enumerate(lens):
        x = proj[at:at + n]
        q = P.silu(x[:, q_at:q_at + H * dk]).reshape(n, H, dk)
        k = P.silu(x[:, k_at:k_at + H * dk]).reshape(n, H, dk)
        v = P.silu(x[:, v_at:v_at + H * dv]).reshape(n, H, dv)
        out.append(P.decayed_state_walk(q, k, v, decay, state[slots[b]]).reshape(n, -1))
        at += n
    return np.concatenate(out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, dk, dv, lens", [(4, 12, 20, (1, 7, 3)), (2, 64, 48, (45,)), (3, 5, 70, (2, 18)), (1, 100, 130, (20,)),
                                             (2, 33, 8, (17, 1)), (2, 128, 128, (9, 1, 1)), (1, 256, 16, (3,))])
def test_decay_scan(ops, dtype, H, dk, dv, lens):
    rng = np.random.default_rng(H * 11 + dk)
    T = sum(lens)
    before = 8
    row = before + 2 * H * dk + 2 * H * dv
    proj = rng.normal(size=(T, row))
    if dtype == torch.bfloat16:
        proj = bf16_round(proj)
    decay = np.concatenate([[1.0], rng.uniform(0.3, 0.999, size=H)])[:H].astype(np.float32).astype(np.float64)
    slots = [2, 0, 3][:len(lens)]
    state = (rng.normal(size=(4, H, dk, dv)) * 0.5).astype(np.float32).astype(np.float64)
    want_state = state.copy()
    q_at, k_at, v_at = before, before + H * dk, before + 2 * H * dk
    want = plain_decay(proj, q_at, k_at, v_at, H, dk, dv, decay, lens, slots, want_state)
    cu = np.concatenate([[0], np.cumsum(lens)])
    dev_state = t(state)
    got = ops.decay_scan(t(proj, dtype), q_at, k_at, v_at, t(decay), 1.0, dev_state, t(cu, torch.int32), t(slots, torch.int32),
                         H, dk, dv)
    close(got, want, 1e-5, "outputs")
    close(dev_state, want_state, 1e-5, "state")
    assert np.array_equal(f64(dev_state[1]), state[1])        # a slot that no sequence of the step has


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, dk, dv, seqs", [(4, 12, 20, 3), (2, 64, 48, 1), (1, 100, 128, 2), (2, 128, 128, 5), (3, 33, 8, 2),
                                             (1, 256, 16, 1), (2, 128, 64, 2)])
def test_decay_step(ops, dtype, H, dk, dv, seqs):
    """One new token a sequence on states that are not zero, at slots in another order: the step kernel where it takes
    the head sizes, against the plain walk and against the scan."""
    if not ops.gla_step_fits(dk, dv):
        pytest.skip("head sizes that the scan takes for single tokens too")
    rng = np.random.default_rng(H * 13 + dk)
    before = 4
    row = before + 2 * H * dk + 2 * H * dv
    proj = rng.normal(size=(seqs, row)).astype(np.float32).astype(np.float64)
    if dtype == torch.bfloat16:
        proj = bf16_round(proj)
    decay = np.concatenate([[1.0], rng.uniform(0.3, 0.999, size=H)])[:H].astype(np.float32).astype(np.float64)
    slots = [4, 0, 2, 5, 1][:seqs]
    state = (rng.normal(size=(6, H, dk, dv)) * 0.5).astype(np.float32).astype(np.float64)
    want_state = state.copy()
    q_at, k_at, v_at = before, before + H * dk, before + 2 * H * dk
    want = plain_decay(proj, q_at, k_at, v_at, H, dk, dv, decay, [1] * seqs, slots, want_state)
    dev_state = t(state)
    got = ops.decay_step(t(proj, dtype), q_at, k_at, v_at, t(decay), 1.0, dev_state, t(slots, torch.int32), H, dk, dv)
    close(got, want, 1e-5, "outputs")
    close(dev_state, want_state, 1e-5, "state")
    assert np.array_equal(f64(dev_state[3]), state[3])
    scan_state = t(state)
    scan = ops.decay_scan(t(proj, dtype), q_at, k_at, v_at, t(decay), 1.0, scan_state, t(np.arange(seqs + 1), torch.int32),
                          t(slots, torch.int32), H, dk, dv)
    close(got, f64(scan), 2e-6, "step against scan")


def test_decay_scan_token_by_token_is_the_walk_in_blocks(ops):
    """The same 37 tokens in one step, in portions, and one at a time from the state the step before left."""
    rng = np.random.default_rng(5)
    H, dk, dv, T = 2, 24, 40, 37
    proj = rng.normal(size=(T, 2 * H * dk + H * dv))
    decay = t([0.9, 0.999])
    slot = t([1], torch.int32)
    one = t(np.zeros((2, H, dk, dv)))
    whole = ops.decay_scan(t(proj), 0, H * dk, 2 * H * dk, decay, 1.0, one, t([0, T], torch.int32), slot, H, dk, dv)
    for cuts in ([1] * T, [2, 17, 16, 2], [33, 4]):
        two, rows, at = t(np.zeros((2, H, dk, dv))), [], 0
        for n in cuts:
            rows.append(ops.decay_scan(t(proj[at:at + n]), 0, H * dk, 2 * H * dk, decay, 1.0, two, t([0, n], torch.int32), slot,
                                       H, dk, dv))
            at += n
        close(torch.cat([r.cpu() for r in rows]), f64(whole), 2e-6, f"cuts {cuts[:3]}")
        close(two, f64(one), 2e-6, "state")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, dk, dv, lens", [(2, 64, 32, (200,)), (3, 12, 20, (64, 1, 130)), (1, 128, 128, (65, 63)),
                                             (2, 4, 8, (129,)), (2, 100, 36, (2, 191, 128))])
def test_decay_scan_in_chunks(ops, dtype, H, dk, dv, lens):
    """The chunked form of the walk on states that are not zero, at slots in another order: lengths on, one below and one
    above a chunk's edge, a head that does not decay and one that decays to nothing inside a chunk; against the plain
    walk and against the walk token by token."""
    assert ops.decay_chunks_fit(dk, dv, 8, (0,))
    rng = np.random.default_rng(H * 17 + dk)
    T = sum(lens)
    before = 8
    row = before + 2 * H * dk + 2 * H * dv
    proj = rng.normal(size=(T, row))
    if dtype == torch.bfloat16:
        proj = bf16_round(proj)
    decay = np.array([1.0, 0.05, 0.97][:H]).astype(np.float32).astype(np.float64)
    slots = [2, 0, 3][:len(lens)]
    state = (rng.normal(size=(4, H, dk, dv)) * 0.5).astype(np.float32).astype(np.float64)
    want_state = state.copy()
    q_at, k_at, v_at = before, before + H * dk, before + 2 * H * dk
    want = plain_decay(proj, q_at, k_at, v_at, H, dk, dv, decay, lens, slots, want_state)
    cu = np.concatenate([[0], np.cumsum(lens)])
    dev_state, walk_state = t(state), t(state)
    args = (t(proj, dtype), q_at, k_at, v_at, t(decay), 1.0)
    got = ops.decay_scan_chunked(*args, dev_state, t(cu, torch.int32), t(slots, torch.int32), H, dk, dv, max(lens))
    close(got, want, 1e-5, "outputs")
    close(dev_state, want_state, 1e-5, "state")
    assert np.array_equal(f64(dev_state[1]), state[1])        # a slot that no sequence of the step has
    walk = ops.decay_scan(*args, walk_state, t(cu, torch.int32), t(slots, torch.int32), H, dk, dv)
    close(got, f64(walk), 1e-5, "chunks against the walk")


def test_chunks_go_on_from_the_state_that_portions_left(ops):
    """300 tokens in one step and in portions that end inside chunks, each portion from the state the one before left."""
    rng = np.random.default_rng(8)
    H, dk, dv, T = 2, 32, 64, 300
    proj = rng.normal(size=(T, 2 * H * dk + H * dv))
    decay, slot = t([1.0, 0.9]), t([1], torch.int32)
    one = t(np.zeros((2, H, dk, dv)))
    whole = ops.decay_scan_chunked(t(proj), 0, H * dk, 2 * H * dk, decay, 1.0, one, t([0, T], torch.int32), slot, H, dk, dv, T)
    two, rows, at = t(np.zeros((2, H, dk, dv))), [], 0
    for n in (130, 1, 150, 19):
        rows.append(ops.decay_scan_chunked(t(proj[at:at + n]), 0, H * dk, 2 * H * dk, decay, 1.0, two, t([0, n], torch.int32),
                                           slot, H, dk, dv, n))
        at += n
    close(torch.cat([r.cpu() for r in rows]), f64(whole), 1e-5, "portions")
    close(two, f64(one), 1e-5, "state")


# ---------------------------------------------------------------- the general router, the experts' closing sum
def plain_route(z, corr, experts, identity, top, groups, keep):
    router = {"experts": experts, "identity": identity, "top": top, "groups": {"count": groups, "keep": keep}}
    n = experts + identity
    return P.route(z, {"r.router": np.eye(n), "r.correction": corr}, "r.", router)


@pytest.mark.parametrize("experts, identity, top, groups, keep, T", [(8, 2, 3, 5, 2, 50), (5, 0, 5, 1, 1, 3), (12, 4, 1, 4, 1, 9),
                                                                    (60, 10, 4, 7, 3, 65), (3, 3, 2, 2, 1, 20), (6, 0, 2, 3, 3, 10)])
def test_general_router(ops, experts, identity, top, groups, keep, T):
    from rust_inference_amd.kernels import ops as real
    rng = np.random.default_rng(experts)
    n = experts + identity
    z = (rng.normal(size=(T, n + 1)) * 2).astype(np.float32).astype(np.float64)          # one more column: the shared expert's gate
    corr = (rng.normal(size=n) * 0.2).astype(np.float32).astype(np.float64)
    chosen, weights, gaps = plain_route(z[:, :n], corr, experts, identity, top, groups, keep)
    ids, w, dense, extra = ops.experts_route_general(t(z), t(corr), n, experts, top, real.ROUTE_SOFTMAX, False, groups, keep)
    sure = gaps > 1e-5
    assert sure.sum() >= T - 2
    got_ids = f64(ids).astype(int)
    for i in np.nonzero(sure)[0]:
        assert sorted(got_ids[i]) == sorted(chosen[i]), f"token {i}"
        by_id = dict(zip(chosen[i], weights[i]))
        close(w[i], [by_id[e] for e in got_ids[i]], F32, "weights")
        want_dense = np.zeros(n)
        want_dense[chosen[i]] = weights[i]
        close(dense[i, :experts], want_dense[:experts], F32, "dense")
        assert f64(extra[i, 0]) == pytest.approx(want_dense[experts:].sum(), rel=1e-5, abs=1e-7)
        assert f64(extra[i, 1]) == pytest.approx(P.sigmoid(z[i, n]), rel=1e-5)


def test_a_dropped_groups_outputs_lose_to_negative_choice_scores(ops):
    """Corrections make every choice score negative; the group with the best one stays, and both of its outputs are
    chosen although every output of the other group has a larger score."""
    from rust_inference_amd.kernels import ops as real
    z = np.log(np.array([[0.05, 0.10, 0.40, 0.45]]))
    corr = np.array([-0.06, -3.0, -0.5, -0.6])
    ids, w, dense, extra = ops.experts_route_general(t(z), t(corr), 4, 4, 2, real.ROUTE_SOFTMAX, False, 2, 1)
    assert sorted(f64(ids).astype(int)[0]) == [0, 1]
    close(dense, [[0.05, 0.10, 0.0, 0.0]], 1e-5)


@pytest.mark.parametrize("dim", [40, 41, 2052])
def test_the_experts_closing_sum(ops, dim):
    rng = np.random.default_rng(1)
    T = 6
    routed, shared = rng.normal(size=(3, T, dim)), rng.normal(size=(2, T, dim))
    x = bf16_round(rng.normal(size=(T, dim)))
    extra = rng.uniform(size=(T, 2))
    f = lambda a: a.astype(np.float32).astype(np.float64)
    got = ops.experts_finish(t(routed), t(x, torch.bfloat16), t(shared), t(extra))
    close(got, f(routed).sum(0) + f(extra)[:, :1] * x + f(extra)[:, 1:] * f(shared).sum(0), F32)
    got = ops.experts_finish(t(routed[0]), None, t(shared[0]), t(extra))
    close(got, f(routed[0]) + f(extra)[:, 1:] * f(shared[0]), F32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_plain_gated_experts_activation(ops, dtype):
    rng = np.random.default_rng(3)
    T, E, ff = 6, 5, 13
    gu = rng.normal(size=(T, E, 2, ff)) * 1.5
    if dtype == torch.bfloat16:
        gu = bf16_round(gu)
    dense = rng.uniform(0.1, 1, size=(T, E)) * (rng.uniform(size=(T, E)) < 0.5)
    want = dense[:, :, None] * P.silu(gu[:, :, 0]) * gu[:, :, 1]
    got = ops.experts_activate(t(gu.reshape(T, -1), dtype), t(dense), ff, 0.0)
    close(got, want.reshape(T, -1), F32 if dtype == torch.float32 else BF16_OUT)
    assert (f64(got).reshape(T, E, ff)[dense == 0] == 0).all()
