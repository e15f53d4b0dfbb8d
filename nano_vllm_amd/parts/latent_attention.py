"""Mixer "latent_attention": causal attention whose keys and values of all heads are made from one small
latent row per token, which is all that is cached.

    q = x Wq^T                         H heads of [D plain | R turned] entries
    [c | kr] = x Wdkv^T                c: C entries, kr: R entries, one for all heads
    c <- c / sqrt(mean(c^2) + eps) * w
    kr and every head's turned part are rotated by the position (the mixer's position encoding, R channels)
    per head h:  key_j = [Wuk_h c_j | kr_j],  value_j = Wuv_h c_j
    s_ij = scale * (q_plain_i . Wuk_h c_j + q_turned_i . kr_j),  j <= i
    weights = softmax over j, optionally with a learned sink per head in the denominator
    out = (heads' outputs side by side) Wo^T

Since q_plain . (Wuk_h c) = (Wuk_h^T q_plain) . c, neither keys nor values are ever formed: the cache holds one key
row [c | kr] and one value row c per token (one key/value head of C + R and C entries), a head's query becomes
[Wuk_h^T q_plain | q_turned], the attention runs on that (kernels.latent_attention), and Wuv_h is applied to its output.
The two small products per head are kernels.heads_linear.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part
from .spec import PagedKV


class LatentAttention(Part):
    """params: hidden_size, num_heads, head_dim (plain entries of a head's query and key), rot_dim (turned entries),
    v_head_dim, kv_rank (the latent's size), eps, scale (None: (head_dim + rot_dim)^-0.5), sink (bool),
    position_encoding (a name in the model's position encodings; it offers step_table and pairs neighbours), and the
    names of the checkpoint tensors: q_name, dkv_name, dkv_norm_name, uk_name, uv_name, sink_name, o_name."""

    kernel_modules = ("latent", "rope", "attn_generic")

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.dim = int(p["head_dim"])
        self.rot = int(p["rot_dim"])
        self.vdim = int(p["v_head_dim"])
        self.rank = int(p["kv_rank"])
        if min(self.heads, self.dim, self.rot, self.vdim, self.rank) <= 0 or self.rot % 2:
            raise ValueError(f"latent_attention: sizes heads={self.heads} dim={self.dim} rot={self.rot} vdim={self.vdim} "
                             f"rank={self.rank} (all positive, an even number of turned entries)")
        self.eps = float(p.get("eps", 1e-6))
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else (self.dim + self.rot) ** -0.5
        self.sink = bool(p.get("sink", False))
        name = p.get("position_encoding")
        self.position_encoding = build.position_encodings[name] if name else None
        pe = self.position_encoding
        if pe is None or not getattr(pe, "interleaved", False) or not hasattr(pe, "step_table") or pe.rotary_dim != self.rot:
            raise ValueError("latent_attention: the position encoding turns neighbouring pairs of rot_dim channels and "
                             "offers step_table")
        self.q_name, self.dkv_name = p.get("q_name", "q_proj"), p.get("dkv_name", "kv_down_proj")
        self.dkv_norm_name = p.get("dkv_norm_name", "kv_norm")
        self.uk_name, self.uv_name = p.get("uk_name", "k_up_proj"), p.get("uv_name", "v_up_proj")
        self.sink_name = p.get("sink_name", "sinks")
        self.o_name = p.get("o_name", "o_proj")

    def param_decls(self) -> Dict[str, ParamDecl]:
        H, D, R, C, V, h = self.heads, self.dim, self.rot, self.rank, self.vdim, self.hidden
        q = H * (D + R)
        d = {
            # q and the latent's projection in one product
            "qc_proj.weight": ParamDecl((q + C + R, h), sources=(Source(f"{self.q_name}.weight", 0, q),
                                                                  Source(f"{self.dkv_name}.weight", q, C + R))),
            "c_norm.weight": ParamDecl((C,), dtype="stored32", init="norm",
                                       sources=(Source(f"{self.dkv_norm_name}.weight", 0, C),)),
            f"{self.uk_name}.weight": ParamDecl((H * D, C)),
            f"{self.uv_name}.weight": ParamDecl((H * V, C)),
            f"{self.o_name}.weight": ParamDecl((h, H * V)),
        }
        if self.sink:
            d["sinks"] = ParamDecl((H,), dtype="float32", sources=(Source(self.sink_name, 0, H),))
        return d

    def cache_need(self):
        return PagedKV(1, self.rank + self.rot, None, self.rank)

    def on_weights_loaded(self) -> None:
        # Wuk_h^T, one below the other: [heads * rank, head_dim], the rows of the product that takes the queries' plain
        # parts into the latent's space (made once; the checkpoint's own layout serves the keys, which are never formed)
        uk = self.weights[f"{self.uk_name}.weight"]
        self._uk_t = uk.view(self.heads, self.dim, self.rank).transpose(1, 2).contiguous().view(self.heads * self.rank, self.dim)

    def forward(self, x, batch, cache):
        k, w = self.kernels, self.weights
        H, D, R, C, V = self.heads, self.dim, self.rot, self.rank, self.vdim
        proj = k.linear(x, w["qc_proj.weight"])
        group = batch.groups[cache.group]
        q2 = k.latent_prepare(proj, H, D, R, C, w["c_norm.weight"], self.eps, self.position_encoding.step_table(batch),
                              group.slot_mapping, cache.k, cache.v)
        # the plain parts of the queries into the latent's space: q2[t, h, :C] = Wuk_h^T q[t, h, :D]
        k.heads_linear(proj, D + R, self._uk_t, H, C, D, False, q2, C + R)
        o = k.latent_attention(q2, H, C, R, cache.k, cache.v, batch, cache.group, self.scale, sinks=w.get("sinks"))
        # and the outputs out of it: heads[t, h, :V] = Wuv_h o[t, h, :C]
        heads = o.new_empty((o.shape[0], H * V))
        k.heads_linear(o, C, w[f"{self.uv_name}.weight"], H, V, C, False, heads, V)
        return k.linear(heads, w[f"{self.o_name}.weight"], deferred=True)


register_part("mixer", "latent_attention", LatentAttention)
