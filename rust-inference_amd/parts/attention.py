"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from .. import profiler
from ..cache import KVNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import build_part, register_part
from .spec import PartSpec


# Up to this many sequences a decode step norms and rotates q and k inside the attention kernel (one launch
# less per layer); beyond it the many workgroups each repeating that work are taken to cost more than the launch
# (up to 56 sequences of 8 kv heads they do not: 1 to 2.4% of the step).  Steps that the attention takes with its
# streaming kernel repeat little of it and are fused at any size.
FUSED_DECODE_MAX_SEQS = 64


@register_part("mixer", "attention")
class GroupedQueryAttention(Mixer):
    """q/k/v projections (no bias), optional per-head RMSNorm of q and k with one
    gain of ``head_dim`` shared by all heads, position encoding of q and k, write of
    k and v into the sequence's pages, causal attention of every new token over its
    sequence (all keys, or the last ``window``), output projection
    (the reference: src/models/qwen3.rs:71-100; src/attention.rs:33-150).

    Query head ``h`` reads kv head ``h // (heads / kv_heads)``; the score is
    ``(q . k) / sqrt(head_dim)``; softmax statistics and the accumulator are float32.
    The three projections are one product with the row-concatenated weight
    ``[q; k; v]``: every output row's dot product is the same as with three products.

    ``qkv_bias`` and ``o_bias`` add ``{q,k,v}_proj.bias`` and ``o_proj.bias`` to the products (the
    reference's family has no bias anywhere, src/models/qwen3.rs:60-69; families that differ from it in
    this alone need no other mixer).  A biased output product adds into the stream the plain way.

    For families without a rotation whose attention differs in its constants: ``v_dim`` is the size of a value
    head where it is not ``head_dim`` (the output product then reads ``heads * v_dim``); ``scale`` replaces
    ``1 / sqrt(head_dim)``; ``softcap = c`` turns a score ``s`` into ``c tanh(s / c)`` before the softmax;
    ``q_temper = (coef, every)`` multiplies the normed query at position ``p`` by
    ``1 + coef * ln(floor((p + 1) / every) + 1)``, all in float32; ``distance_slopes`` (one per query head) takes
    ``slope_h * (i - j)`` off the score of the query at position ``i`` for the key at ``j``, after scale and cap;
    ``window`` holds on this path as on the other.  ``names`` gives the checkpoint names of
    ``q, k, v, o, q_norm, k_norm`` where they are not ``<prefix>q_proj.weight`` and so on.  A mixer with any of
    ``v_dim``, ``softcap`` or ``q_temper`` takes no position encoding; its q/k norm, temperature and cache write
    are one kernel (``ops.qk_norm_temper_kv_write``).

    A third family, with a position encoding that turns neighbouring elements (``position`` of a kind whose
    ``pairs`` is true, for instance ``"rotate_pairs"``): q and k are rotated first and normed afterwards,
    ``qk_norm="unit"`` norms them without gains (a head divided by its root mean square); ``keep_first`` keeps
    a sequence's first tokens visible behind the ``window`` (position ``i`` sees ``j <= i`` with ``i - j < window`` or
    ``j < keep_first``; kept tokens keep their own positions); ``sinks`` reads one number per query head
    (``names["sink"]``) whose exponential joins the softmax's denominator, with no key and no value, unscaled;
    ``gate="sigmoid"`` multiplies the heads side by side by ``sigmoid(W_g h)`` (``names["g"]``, read from the mixer's own
    input) before the output product.  Any of these sends the mixer through ``ops.qk_pairs_norm_kv_write``; value
    heads of their own size are welcome there.  Such a mixer can also run beside another one on one input and one
    output product (``parts.parallel.ParallelMixers``): ``in_matrix``, ``core`` and ``out_matrix`` are its three
    steps taken apart.
    """

    links_norms = True

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, prefix: str, qk_norm: bool = True,
                 eps: float = 1e-6, position: PartSpec | None = None, window: int | None = None,
                 qkv_bias: bool = False, o_bias: bool = False, v_dim: int | None = None, scale: float | None = None,
                 softcap: float | None = None, q_temper: tuple | None = None, names: dict | None = None,
                 distance_slopes: tuple | None = None, keep_first: int = 0, sinks: bool = False, gate: str | None = None):
        if heads < 1 or kv_heads < 1 or heads % kv_heads:
            raise ConfigError(f"{heads} attention heads not divisible by {kv_heads} kv heads")
        if not 1 <= head_dim <= ops.MAX_HEAD_DIM:
            raise ConfigError(f"head_dim {head_dim}: the attention kernels take 1 to {ops.MAX_HEAD_DIM}")
        if window is not None and window < 1:
            raise ConfigError(f"window {window} must be positive")
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.prefix, self.qk_norm, self.eps, self.window = prefix, qk_norm, eps, window
        self.qkv_bias, self.o_bias = qkv_bias, o_bias
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)      # src/attention.rs:28
        self.v_dim = head_dim if v_dim is None else int(v_dim)
        self.softcap = float(softcap) if softcap else None
        self.q_temper = (float(q_temper[0]), int(q_temper[1])) if q_temper else None
        if not 1 <= self.v_dim <= ops.MAX_HEAD_DIM:
            raise ConfigError(f"value heads of {self.v_dim}: the attention kernels take 1 to {ops.MAX_HEAD_DIM}")
        if self.q_temper is not None and self.q_temper[1] < 1:
            raise ConfigError(f"a query temperature every {self.q_temper[1]} positions")
        # what the rotary kernels do not know goes through the kernels that do
        # a distance bias: the score of head h at position i for the key at j loses distance_slopes[h] * (i - j)
        self.distance_slopes = tuple(float(v) for v in distance_slopes) if distance_slopes is not None else None
        if self.distance_slopes is not None and len(self.distance_slopes) != heads:
            raise ConfigError(f"{len(self.distance_slopes)} distance slopes for {heads} heads")
        self.tempered = self.v_dim != head_dim or self.q_temper is not None or self.distance_slopes is not None
        self.position = build_part("position", position or PartSpec("none"))
        self.keep_first, self.sinks, self.gate = int(keep_first or 0), bool(sinks), gate
        if gate not in (None, "sigmoid", "silu"):
            raise ConfigError(f"an output gate {gate!r} is neither 'sigmoid' nor 'silu'")
        if self.keep_first < 0 or (self.keep_first and window is None):
            raise ConfigError(f"{keep_first} first tokens kept behind a window of {window}")
        # rotation of neighbours, unit norm, kept first tokens, sinks or a gate: the third family
        self.paired = (getattr(self.position, "pairs", False) or qk_norm == "unit" or self.keep_first > 0 or self.sinks
                       or gate is not None)
        if self.paired and (self.q_temper is not None or qkv_bias or o_bias):
            raise ConfigError("an attention with a rotation of neighbours, kept first tokens, sinks or a gate takes no "
                              "query temperature and no biases")
        if self.paired and position is not None and position.kind != "none" and not getattr(self.position, "pairs", False):
            raise ConfigError("an attention with kept first tokens, sinks or a gate rotates neighbours or not at all")
        if self.paired and head_dim > 512:
            raise ConfigError(f"head_dim {head_dim}: the kernel that rotates neighbours takes up to 512")
        if not self.paired and (self.tempered or self.softcap is not None) and (position is not None and position.kind != "none"):
            raise ConfigError("an attention with a score cap, a query temperature or value heads of their own size "
                              "takes no position encoding")
        if (self.tempered or self.softcap is not None) and (qkv_bias or o_bias):
            raise ConfigError("an attention with a score cap, a query temperature or value heads of their own size "
                              "takes no biases")
        p = prefix
        self.names = {"q": p + "q_proj.weight", "k": p + "k_proj.weight", "v": p + "v_proj.weight",
                      "o": p + "o_proj.weight", "q_norm": p + "q_norm.weight", "k_norm": p + "k_norm.weight",
                      "sink": p + "sink", "g": p + "g_proj.weight"}
        self.names.update(names or {})
        self.unit_norm = qk_norm == "unit"
        self.q_width, self.k_width, self.v_width = heads * head_dim, kv_heads * head_dim, kv_heads * self.v_dim
        self.out_width = heads * self.v_dim
        # the columns of this mixer's input product: q, k, v and, with a gate, g
        self.in_width = self.q_width + self.k_width + self.v_width + (self.out_width if gate else 0)

    def tensors(self):
        p, d, dh, n = self.prefix, self.hidden, self.head_dim, self.names
        t = {
            n["q"]: TensorSpec((self.heads * dh, d), MATRIX),
            n["k"]: TensorSpec((self.kv_heads * dh, d), MATRIX),
            n["v"]: TensorSpec((self.kv_heads * self.v_dim, d), MATRIX),
            n["o"]: TensorSpec((d, self.heads * self.v_dim), MATRIX),
        }
        if self.qk_norm and not self.unit_norm:
            t[n["q_norm"]] = TensorSpec((dh,), GAIN)
            t[n["k_norm"]] = TensorSpec((dh,), GAIN)
        if self.sinks:
            t[n["sink"]] = TensorSpec((self.heads,), GAIN)
        if self.gate:
            t[n["g"]] = TensorSpec((self.heads * self.v_dim, d), MATRIX)
        if self.qkv_bias:
            t[p + "q_proj.bias"] = TensorSpec((self.heads * dh,), BIAS)
            t[p + "k_proj.bias"] = TensorSpec((self.kv_heads * dh,), BIAS)
            t[p + "v_proj.bias"] = TensorSpec((self.kv_heads * dh,), BIAS)
        if self.o_bias:
            t[p + "o_proj.bias"] = TensorSpec((d,), BIAS)
        t.update(self.position.tensors())
        return t

    def in_matrix(self, weights):
        """The rows of this mixer's input product, ``[q; k; v]`` and, with a gate, ``g``."""
        n = self.names
        return torch.cat([weights[n[x]] for x in (("q", "k", "v", "g") if self.gate else ("q", "k", "v"))], 0)

    def out_matrix(self, weights):
        return weights[self.names["o"]]

    def bind(self, weights, rt, alone: bool = True):
        """``alone`` False: another part owns the products before and after (mixers side by side); this one binds
        what its ``core`` needs."""
        self.rt = rt
        p, n = self.prefix, self.names
        if alone:
            self.w_qkv = rt.pack(rt.place_matrix(self.in_matrix(weights)), always=self.gate is not None)
            self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=(p + "o_proj.bias") not in weights)
        gains = self.qk_norm and not self.unit_norm
        self.q_gain = rt.place_gain(weights[n["q_norm"]]) if gains else None
        self.k_gain = rt.place_gain(weights[n["k_norm"]]) if gains else None
        self.sink = rt.place_gain(weights[n["sink"]]) if self.sinks else None
        self.b_qkv = self.b_o = None
        if self.qkv_bias:
            self.b_qkv = rt.place_gain(torch.cat([weights[p + n + "_proj.bias"] for n in "qkv"], 0))
        if self.o_bias:
            self.b_o = rt.place_gain(weights[p + "o_proj.bias"])
        self.position.bind(weights, rt)
        self.slopes = (torch.tensor(self.distance_slopes, dtype=torch.float32, device=rt.device)
                       if self.distance_slopes is not None else None)

    def bind_plain(self, weights):
        if self.tempered or self.softcap is not None:
            raise ConfigError("an attention with a score cap, a query temperature or value heads of their own size has "
                              "no plain form")
        f32 = lambda name: weights[self.prefix + name].to(torch.float32).numpy()
        self.plain_w = {n: weights[self.names[n]].to(torch.float32).numpy() for n in "qkvo"}
        self.plain_gain = {n: weights[self.names[n + "_norm"]].to(torch.float32).numpy() for n in "qk"} if self.qk_norm else {}
        self.plain_bias = {n: f32(n + "_proj.bias") for n in ("qkv" if self.qkv_bias else "") + ("o" if self.o_bias else "")}
        if getattr(self.position, "acts_after_norm", False) or not hasattr(self.position, "plain"):
            raise ConfigError(f"the position encoding {type(self.position).__name__} has no plain form")
        self.position.bind_plain(weights)

    def plain(self, x, ctx, store, page_table):
        """The same over numpy arrays and the plain C++ twins: three products, per-head norm, rotation, the new keys
        and values into their pages (``store = (k_pages, v_pages)``, values transposed inside a page), attention
        over the pages, output product."""
        from ..kernels import plain
        t, dh, page = x.shape[0], self.head_dim, store[0].shape[2]
        heads = {}
        for n, count in (("q", self.heads), ("k", self.kv_heads), ("v", self.kv_heads)):
            y = plain.linear(x, self.plain_w[n])
            if n in self.plain_bias:
                y = y + self.plain_bias[n]
            heads[n] = y.reshape(t, count, dh)
        for n in "qk":
            if self.qk_norm:
                heads[n] = plain.rms_norm(heads[n], self.plain_gain[n], self.eps)
            heads[n] = self.position.plain(heads[n], ctx.tok_pos)
        phys = page_table[ctx.tok_seq, ctx.tok_pos // page]
        store[0][phys, :, ctx.tok_pos % page, :] = heads["k"]
        store[1][phys, :, :, ctx.tok_pos % page] = heads["v"]
        o = plain.attention(heads["q"], store[0], store[1], ctx.tok_pos, ctx.tok_seq, page_table, self.window, self.scale)
        y = plain.linear(o.reshape(t, self.heads * dh), self.plain_w["o"])
        return y + self.plain_bias["o"] if "o" in self.plain_bias else y

    def takes_tiled_at(self, m: int) -> bool:
        """Whether this part's first product reads ``m`` rows in the matrix cores' order."""
        return self.rt.takes_tiled(self.w_qkv, m)

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window, None if self.v_dim == self.head_dim else self.v_dim,
                      self.keep_first or None)

    def forward(self, x, ctx, store, page_table, link=None):
        rt = self.rt
        with profiler.section(profiler.QKV_PROJECTION):
            qkv = rt.linear_packed(x, self.w_qkv)
            if self.b_qkv is not None:
                ops.add_bias(qkv, self.b_qkv)
        if self.paired:
            proj = ops.as_rows(qkv)
            heads = torch.empty((proj.shape[0], self.out_width), dtype=proj.dtype, device=proj.device)
            self.core(proj, 0, ctx, store, page_table, heads, 0, 1.0)
            with profiler.section(profiler.OUT_PROJECTION):
                return rt.linear_packed(heads, self.w_o, out_dtype=torch.float32, parts_ok=True)
        if self.tempered or self.softcap is not None:
            return self.forward_tempered(qkv, ctx, store, page_table, link)
        self.position.apply(qkv, ctx, self.heads, self.kv_heads, self.head_dim)
        group = self.heads // self.kv_heads
        table = self.position.rotation_table()
        whole = table is None or 2 * table.shape[0] == self.head_dim      # the fused kernel rotates whole heads
        after_norm = getattr(self.position, "acts_after_norm", False)
        if (ctx.is_decode and whole and not after_norm and not rt.invariant
                and ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, True)
                and (ctx.B <= FUSED_DECODE_MAX_SEQS
                     or ops.decode_attention_streams(ctx.B, self.kv_heads, ctx.max_len))):
            # one token per sequence: norm, rotation, cache write and attention are one kernel
            with profiler.section(profiler.ATTENTION):
                o = ops.attention_decode_fused_bf16(qkv, self.q_gain, self.k_gain, self.eps, table, store.k_pages,
                                                    store.v_pages, ctx.tok_pos, page_table, ctx.B, ctx.max_len,
                                                    self.heads, self.kv_heads, self.head_dim, self.window, self.scale,
                                                    tiled_out=rt.takes_tiled(self.w_o, ctx.B, self.b_o is None))
            return self.project_out(o, link)
        with profiler.section(profiler.QK_NORM_ROPE_APPEND):
            shape = (self.heads, self.kv_heads, self.head_dim)
            if after_norm:
                # an encoding that acts on the normed q and k: norm (and rotation) in place, the encoding,
                # then the move of k and v into their pages
                ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, table, ctx.tok_pos, ctx.tok_seq,
                                          page_table, None, None, *shape)
                self.position.apply_normed(qkv, ctx, *shape)
                ops.qk_norm_rope_kv_write(qkv, None, None, self.eps, None, ctx.tok_pos, ctx.tok_seq, page_table,
                                          store.k_pages, store.v_pages, *shape, ctx.cu_seqlens, ctx.max_new)
            elif rt.invariant:
                # the kernel of one wavefront per token and head, whatever the step looks like
                ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, table, ctx.tok_pos, ctx.tok_seq,
                                          page_table, store.k_pages, store.v_pages, *shape)
            else:
                ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, self.eps, table, ctx.tok_pos, ctx.tok_seq,
                                          page_table, store.k_pages, store.v_pages, *shape, ctx.cu_seqlens, ctx.max_new)
        with profiler.section(profiler.ATTENTION):
            o = self.attend(qkv, ctx, store, page_table)
        return self.project_out(o, link)

    def core(self, proj, col0: int, ctx, store, page_table, out, out_col: int, out_scale: float) -> None:
        """The mixer between its two products: ``proj [T, row]`` holds this mixer's q, k, v (and g) from column
        ``col0`` on; the rotated and normed q stay there, k and v go to the pages, and the heads' results, times the
        gate and ``out_scale``, are written into the columns ``out_col ..`` of ``out``."""
        q_at, k_at = col0, col0 + self.q_width
        v_at = k_at + self.k_width
        with profiler.section(profiler.QK_NORM_ROPE_APPEND):
            ops.qk_pairs_norm_kv_write(proj, q_at, k_at, v_at, self.position.rotation_table(), self.q_gain, self.k_gain,
                                       bool(self.qk_norm), self.eps, ctx.tok_pos, ctx.tok_seq, page_table, store.k_pages,
                                       store.v_pages, self.heads, self.kv_heads, self.head_dim, self.v_dim,
                                       ctx.cu_seqlens, ctx.max_new)
        with profiler.section(profiler.ATTENTION):
            o = self.attend_kept(proj, col0, ctx, store, page_table)
            ops.gate_rows(out, out_col, o, proj if self.gate else None, v_at + self.v_width, out_scale,
                          ops.GATE_SILU if self.gate == "silu" else ops.GATE_SIGMOID)

    def attend_kept(self, proj, q_at, ctx, store, page_table):
        """The attention of the third family: window with kept first tokens, sinks, value heads of any size."""
        slopes = getattr(self, "slopes", None)
        group = self.heads // self.kv_heads
        fits = self.v_dim == self.head_dim and proj.shape[1] % 8 == 0 and q_at % 8 == 0
        if (fits and ctx.is_decode and not self.rt.invariant
                and ops.mfma_attention_fits(proj.dtype, self.head_dim, group, store.page_size, True)
                and not ops.decode_attention_streams(ctx.B, self.kv_heads, ctx.max_len)):
            # one new token a sequence in a step that does not fill the machine: the keys in chunks side by side, then
            # the join, which adds the kept keys' chunks and the sink
            return ops.attention_decode_bf16(proj, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos, page_table,
                                             ctx.B, ctx.max_len, self.heads, self.kv_heads, self.head_dim, self.window,
                                             self.scale, softcap=self.softcap, slopes=slopes, keep_first=self.keep_first,
                                             sinks=self.sink, q_off=q_at)
        if fits and ops.mfma_attention_fits(proj.dtype, self.head_dim, group, store.page_size, False):
            # the matrix cores' prompt kernel, also for the single tokens of a step that fills the machine: a
            # wavefront walks a sequence's pages in their order
            return ops.attention_prefill_bf16(proj, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos, page_table,
                                              ctx.B, ctx.max_new, self.heads, self.kv_heads, self.head_dim, self.window,
                                              self.scale, self.softcap, slopes, self.keep_first, self.sink, q_at)
        return ops.attention(proj, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, self.heads,
                             self.kv_heads, self.head_dim, self.window, self.scale, self.softcap, slopes,
                             keep_first=self.keep_first, sinks=self.sink, q_off=q_at)

    def forward_tempered(self, qkv, ctx, store, page_table, link):
        """No rotation: per-head norm, query temperature and the write of k and v in one kernel, then the attention
        with the score cap."""
        with profiler.section(profiler.QK_NORM_ROPE_APPEND):
            ops.qk_norm_temper_kv_write(qkv, self.q_gain, self.k_gain, self.eps, self.q_temper, ctx.tok_pos, ctx.tok_seq,
                                        page_table, store.k_pages, store.v_pages, self.heads, self.kv_heads,
                                        self.head_dim, self.v_dim, ctx.cu_seqlens, ctx.max_new)
        with profiler.section(profiler.ATTENTION):
            o = self.attend(qkv, ctx, store, page_table)
        with profiler.section(profiler.OUT_PROJECTION):          # float32 into the residual: one rounding less a layer
            return self.rt.linear_packed(o, self.w_o, out_dtype=torch.float32, parts_ok=True, link=link)

    def project_out(self, o, link):
        with profiler.section(profiler.OUT_PROJECTION):
            if self.b_o is None:
                return self.rt.linear_packed(o, self.w_o, parts_ok=True, link=link)
            return ops.add_bias(self.rt.linear_packed(o, self.w_o), self.b_o)

    def attend(self, qkv, ctx, store, page_table):
        """The attention kernel that fits the step: matrix cores for bfloat16 (one new token per
        sequence, or any number), the generic kernel for everything else."""
        args = (self.heads, self.kv_heads, self.head_dim, self.window, self.scale)
        group = self.heads // self.kv_heads
        cap = self.softcap
        slopes = getattr(self, "slopes", None)
        if self.v_dim != self.head_dim:          # value heads of their own size: the generic kernel alone takes them
            return ops.attention(qkv, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, *args, cap, slopes)
        if self.rt.invariant:
            # one kernel for prompts and single tokens alike: in the prompt kernel a token's sums run over its
            # sequence's pages in order whatever the other rows of its tile are (a page that a row does not
            # see changes none of its bits); the generic kernel where that one does not take the sizes
            if ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, False):
                return ops.attention_prefill_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                                  page_table, ctx.B, ctx.max_new, *args, cap, slopes)
            return ops.attention(qkv, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, *args, cap, slopes)
        if ops.mfma_attention_fits(qkv.dtype, self.head_dim, group, store.page_size, ctx.is_decode):
            if ctx.is_decode:
                return ops.attention_decode_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                                 page_table, ctx.B, ctx.max_len, *args,
                                                 tiled_out=self.rt.takes_tiled(self.w_o, ctx.B, self.b_o is None),
                                                 softcap=cap, slopes=slopes)
            return ops.attention_prefill_bf16(qkv, store.k_pages, store.v_pages, ctx.cu_seqlens, ctx.tok_pos,
                                              page_table, ctx.B, ctx.max_new, *args, cap, slopes)
        return ops.attention(qkv, store.k_pages, store.v_pages, ctx.tok_pos, ctx.tok_seq, page_table, *args, cap, slopes)
