"""Mixer parts.

"attention": grouped-query causal attention over a paged cache
(nanovllm/models/qwen3.py:14-88, nanovllm/layers/attention.py:43-75):
    qkv = x Wqkv^T (+ b)            rows of Wqkv: q heads, k heads, v heads (linear.py:111-128)
    q, k <- per-head RMS norm       when qk_norm (qwen3.py:68-70,82-84)
    q, k <- position encoding       (qwen3.py:85)
    cache <- k, v                   (attention.py:62-63)
    o = softmax(scale q K^T) V      causal, over the request's cached keys, optionally a window
    out = o Wo^T                    (qwen3.py:87)
Options beyond the reference's attention, each a parameter:
    v_head_dim                      values of a size of their own (the output heads have that size)
    qk_norm_scope "projection"      q and k normed over the whole projection, all heads at once, with
                                    weights of that size, before the split into heads
    q_temperature (coef, every)     q *= 1 + coef * ln(floor((p + 1) / every) + 1) at position p
    sink                            a learned number per head whose exponential joins the softmax's
                                    denominator: a key without a value that every query sees once
    chunk                           a query at position p reads the keys of positions floor(p / chunk) *
                                    chunk ... p only: the sequence is cut into chunks counted from its
                                    position 0, wherever a prompt was cut for processing
    o_bias                          a bias on the output projection
    softcap                         scores capped smoothly: s <- softcap * tanh(s / softcap), after the scale
    keep_first (with a window)      every query also reads the first keep_first positions of its sequence,
                                    however far back they lie; they keep their own positions
    sink_value                      a sink that is a constant (0: the softmax's denominator gains 1), no tensor
    gate "sigmoid"                  the heads' outputs are multiplied, entry by entry, with sigmoid(x Wg^T)
                                    before the output projection; Wg [heads * v_head_dim, hidden] is packed
                                    below q, k and v into the one projection
    v_norm                          every value head is divided by its root mean square (eps inside the root, no
                                    weight) before it is cached
    v_mix (a name)                  the layers of a model that give the same name mix their values: the first of them
                                    in the order keeps its values of the step's tokens (after the norm), every later
                                    one caches (1 - lam) v + lam v_first, lam a learned number of its own
    weights "sigmoid"               no softmax: a visible key weighs sigmoid(score + b_head), b a learned number per
                                    head, and the weights are not normalised over the keys
An encoding that says `interleaved` rotates the neighbours (2i, 2i + 1) instead of the pairs (i, i + R/2).
With values of their own size (or whole-projection norms, or a temperature) the position encoding's
rotation is applied by the same preparation kernel, from the cosines and sines of the step's tokens
(position_encoding.step_table): such a model needs no table of all positions.

Interface of a mixer:
    cache_need()                 -> PagedKV | FixedState | None
    forward(x [T, hidden], batch, cache) -> [T, hidden]
`cache` is the run's LayerCache (its tensors and the index of its group in batch.groups).
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part
from .spec import PagedKV


class Attention(Part):
    """params: hidden_size, num_heads, num_kv_heads, head_dim, qk_norm (bool), eps, bias (bool),
    position_encoding (a name in the model's position encodings, or None), window (None or
    keys), scale (None: head_dim^-0.5), reads_shared_cache (bool: the run owns no cache, it
    projects q only and reads another run's keys and values), v_head_dim (None: head_dim),
    qk_norm_scope ("head" | "projection"), q_temperature (None or {"coef", "every"}), sink (bool),
    chunk (None or positions), o_bias (bool), step_rotation (bool: rotate from the step's own table
    also where the per-head kernel could serve), softcap (None or a positive number), keep_first (positions),
    sink_value (None or a number), gate (None or "sigmoid"), v_norm (bool), v_mix (None or a name shared by the layers
    that mix), weights ("softmax" | "sigmoid"), and the names of the checkpoint tensors (q_name, ..., q_norm_name,
    k_norm_name, sink_name, g_name, v_mix_name, score_bias_name)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        if self.heads % self.kv_heads:
            raise ValueError(f"attention: {self.heads} heads do not divide into {self.kv_heads} kv heads")
        self.qk_norm = bool(p.get("qk_norm", False))
        self.eps = float(p.get("eps", 1e-6))
        self.bias = bool(p.get("bias", False))
        self.window = p.get("window")
        self.chunk = p.get("chunk")
        if self.chunk is not None and int(self.chunk) <= 0:
            raise ValueError(f"attention: a chunk of {self.chunk} positions")
        self.o_bias = bool(p.get("o_bias", False))
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5     # qwen3.py:39
        self.shared = bool(p.get("reads_shared_cache", False))
        name = p.get("position_encoding")
        self.position_encoding = build.position_encodings[name] if name else None
        self.q_name, self.k_name, self.v_name = (p.get("q_name", "q_proj"), p.get("k_name", "k_proj"),
                                                 p.get("v_name", "v_proj"))
        self.o_name = p.get("o_name", "o_proj")
        self.q_norm_name, self.k_norm_name = p.get("q_norm_name", "q_norm"), p.get("k_norm_name", "k_norm")
        self.sink_name = p.get("sink_name", "sinks")
        v = p.get("v_head_dim")
        self.v_head_dim = self.head_dim if v is None else int(v)
        self.norm_scope = p.get("qk_norm_scope", "head")
        if self.norm_scope not in ("head", "projection"):
            raise ValueError(f"attention: qk_norm_scope must be 'head' or 'projection', got {self.norm_scope!r}")
        temp = p.get("q_temperature")
        self.temp_coef = float(temp["coef"]) if temp else 0.0
        self.temp_every = int(temp["every"]) if temp else 1
        self.sink = bool(p.get("sink", False))
        sink_value = p.get("sink_value")
        self.sink_value = None if sink_value is None else float(sink_value)
        if self.sink and self.sink_value is not None:
            raise ValueError("attention: a learned sink and a constant one exclude each other")
        cap = p.get("softcap")
        self.softcap = None if cap is None else float(cap)
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError(f"attention: a softcap of {self.softcap}")
        self.keep_first = int(p.get("keep_first") or 0) if self.window is not None else 0
        if self.keep_first < 0:
            raise ValueError(f"attention: keep_first {self.keep_first}")
        self.gate = p.get("gate")
        if self.gate not in (None, "sigmoid"):
            raise ValueError(f"attention: gate must be 'sigmoid' or absent, got {self.gate!r}")
        self.g_name = p.get("g_name", "g_proj")
        self.v_norm = bool(p.get("v_norm", False))
        self.v_mix = p.get("v_mix")
        self.v_mix_name = p.get("v_mix_name", "v_mix")
        self.weighting = p.get("weights", "softmax")
        if self.weighting not in ("softmax", "sigmoid"):
            raise ValueError(f"attention: weights must be 'softmax' or 'sigmoid', got {self.weighting!r}")
        self.score_bias_name = p.get("score_bias_name", "score_bias")
        if self.weighting == "sigmoid" and (self.sink or self.sink_value is not None or self.softcap is not None
                                            or self.keep_first or self.chunk is not None):
            raise ValueError("attention: sigmoid weights go without sink, softcap, kept positions and chunks")
        if (self.v_norm or self.v_mix) and self.shared:
            raise ValueError("attention: a value norm or mixed values go with a cache of the run's own")
        self.interleaved = bool(getattr(build.position_encodings.get(p.get("position_encoding")), "interleaved", False))
        self._device = build.device
        self._sink_tensor = None
        # The whole-projection preparation has its own kernel, which also scales q by its temperature
        # and stores values of their own size; the per-head one rotates.  Each does what its model needs.
        self.row_prepare = self.norm_scope == "projection" or self.temp_coef != 0.0 or self.v_head_dim != self.head_dim \
            or bool(p.get("step_rotation", False)) or self.gate is not None or self.v_norm or bool(self.v_mix) \
            or self.interleaved
        if self.row_prepare and self.position_encoding is not None and not hasattr(self.position_encoding, "step_table"):
            raise ValueError("attention: with whole-projection norms, a query temperature or values of their own "
                             "size the position encoding must offer step_table")
        if self.gate is not None and (self.shared or self.bias):
            raise ValueError("attention: an output gate goes with a cache of the run's own and no biases")

    @property
    def kernel_modules(self):
        prepare = "qk_rownorm" if self.row_prepare else "rope"
        rope = ("rope",) if self.row_prepare and self.position_encoding else ()
        if self.v_head_dim != self.head_dim:
            return (prepare, "attn_generic") + rope
        return (prepare, "attn_generic", "attn_decode", "attn_prefill") + \
            (("rope",) if self.row_prepare and self.position_encoding else ())

    # ------------------------------------------------------------------ declaration
    def param_decls(self) -> Dict[str, ParamDecl]:
        q, kv, h = self.heads * self.head_dim, self.kv_heads * self.head_dim, self.hidden
        vv = self.kv_heads * self.v_head_dim
        d: Dict[str, ParamDecl] = {}
        if self.shared:
            shards = ((self.q_name, 0, q),)
            rows = q
        else:
            shards = ((self.q_name, 0, q), (self.k_name, q, kv), (self.v_name, q + kv, vv))
            rows = q + kv + vv
            if self.gate is not None:
                shards += ((self.g_name, rows, self.heads * self.v_head_dim),)
                rows += self.heads * self.v_head_dim
        d["qkv_proj.weight"] = ParamDecl((rows, h), sources=tuple(Source(f"{n}.weight", r, c) for n, r, c in shards))
        if self.bias:
            d["qkv_proj.bias"] = ParamDecl((rows,), sources=tuple(Source(f"{n}.bias", r, c) for n, r, c in shards))
        if self.qk_norm:
            whole = self.norm_scope == "projection"
            qn, kn = (q, kv) if whole else (self.head_dim, self.head_dim)
            d["q_norm.weight"] = ParamDecl((qn,), dtype="stored32", init="norm",
                                           sources=(Source(f"{self.q_norm_name}.weight", 0, qn),))
            if not self.shared:
                d["k_norm.weight"] = ParamDecl((kn,), dtype="stored32", init="norm",
                                               sources=(Source(f"{self.k_norm_name}.weight", 0, kn),))
        if self.sink:
            d["sinks"] = ParamDecl((self.heads,), dtype="float32", sources=(Source(self.sink_name, 0, self.heads),))
        if self.v_mix:
            d[self.v_mix_name] = ParamDecl((), dtype="float32")        # (one number: the tensor goes by its own name)
        if self.weighting == "sigmoid":
            d["score_bias"] = ParamDecl((self.heads,), dtype="float32", sources=(Source(self.score_bias_name, 0, self.heads),))
        d[f"{self.o_name}.weight"] = ParamDecl((h, self.heads * self.v_head_dim))
        if self.o_bias:
            d[f"{self.o_name}.bias"] = ParamDecl((h,))
        return d

    def cache_need(self):
        if self.shared:
            return None
        return PagedKV(self.kv_heads, self.head_dim, self.window,
                       None if self.v_head_dim == self.head_dim else self.v_head_dim,
                       None if self.chunk is None else int(self.chunk), self.keep_first)

    def _sinks(self):
        if self.sink:
            return self.weights.get("sinks")
        if self.sink_value is None:
            return None
        if self._sink_tensor is None:          # made on first use: building a part touches no device
            self._sink_tensor = torch.full((self.heads,), self.sink_value, dtype=torch.float32, device=self._device)
        return self._sink_tensor

    # ------------------------------------------------------------------ forward
    def forward(self, x, batch, cache):
        k = self.kernels
        w = self.weights
        kv_heads = 0 if self.shared else self.kv_heads
        # deferred: the products below are handed to the q/k preparation and to the block's norm only
        pe = self.position_encoding
        table = pe.rotary_table() if pe is not None and not self.row_prepare else None
        # (with a gate the row also holds the gate's columns, which outlive the preparation: a tensor, not partial sums)
        qkv = k.linear(x, w["qkv_proj.weight"], w.get("qkv_proj.bias"),
                       deferred=self.gate is None and (self.row_prepare or pe is None or table is not None))
        gate = None
        if self.gate is not None:
            qkv_width = (self.heads + self.kv_heads) * self.head_dim + self.kv_heads * self.v_head_dim
            gate, qkv = qkv[:, qkv_width:], qkv[:, :qkv_width]
        group = batch.groups[cache.group]
        slots = None if self.shared else group.slot_mapping
        kc, vc = (None, None) if self.shared else (cache.k, cache.v)
        qw = w.get("q_norm.weight")
        kw = w.get("k_norm.weight")
        if self.row_prepare:
            extra = {"rot_table": pe.step_table(batch)} if pe is not None else {}
            if self.qk_norm and self.norm_scope == "head":
                extra["norm_per_head"] = True
            if self.interleaved:
                extra["rot_interleaved"] = True
            if self.v_norm:
                extra["v_norm"] = True
            if self.v_mix:
                # the first layer of the name to run in a step leaves its values for the others
                kept = batch.step_cache
                first = kept.get(("v_first", self.v_mix))
                if first is None:
                    first = kept[("v_first", self.v_mix)] = torch.empty(
                        (x.shape[0], self.kv_heads * self.v_head_dim), dtype=torch.float32, device=x.device)
                    extra["v_first_out"] = first
                else:
                    extra["v_first_in"], extra["v_mix"] = first, w[self.v_mix_name]
            q = k.qk_rownorm_store(qkv, self.heads, kv_heads, self.head_dim, self.v_head_dim, qw, kw, self.eps,
                                   batch.positions, self.temp_coef, self.temp_every, slots, kc, vc, **extra)
        elif pe is None or table is not None:
            q = k.qk_norm_rope_store(qkv, self.heads, kv_heads, self.head_dim, qw, kw, self.eps, table,
                                     batch.positions, slots, kc, vc, max_position=batch.max_kv_len)
        else:
            # an encoding without a table: norm, the part's own encoding, then the store
            q = k.qk_norm_rope_store(qkv, self.heads, kv_heads, self.head_dim, qw, kw, self.eps, None, None,
                                     None, None, None)
            qd = self.heads * self.head_dim
            pe.apply(q, qkv[:, qd: qd + kv_heads * self.head_dim], batch.positions, self.heads, kv_heads,
                     self.head_dim)
            if not self.shared:
                k.qk_norm_rope_store(qkv, self.heads, kv_heads, self.head_dim, None, None, self.eps, None, None,
                                     slots, kc, vc)
        extra = {"chunk": int(self.chunk)} if self.chunk is not None else {}
        if self.softcap is not None:
            extra["softcap"] = self.softcap
        if self.keep_first:
            extra["keep_first"] = self.keep_first
        sinks = self._sinks()
        if self.weighting == "sigmoid":
            extra["sigmoid_bias"] = w["score_bias"]
        if sinks is not None or self.v_head_dim != self.head_dim:
            o = k.paged_attention(q, self.heads, self.kv_heads, self.head_dim, cache.k, cache.v, batch, cache.group,
                                  self.scale, self.window, v_head_dim=self.v_head_dim, sinks=sinks, **extra)
        else:
            o = k.paged_attention(q, self.heads, self.kv_heads, self.head_dim, cache.k, cache.v, batch, cache.group,
                                  self.scale, self.window, **extra)
        if gate is not None:
            o = k.sigmoid_mul(o, gate)
        return k.linear(o, w[f"{self.o_name}.weight"], w.get(f"{self.o_name}.bias"), deferred=True)


register_part("mixer", "attention", Attention)
