"""Kirisun as data: config.json -> typed configuration -> ModelSpec.

Every layer is the sandwich residual block on a float32 stream: an RMS norm before and one after each
sublayer, the normed output times a constant added to the stream.  The mixer is, entry by entry of the
configuration's list, attention (grouped, per-head query and key norms, a partial rotation with linearly
scaled frequencies, scores capped by a tanh, a window that also keeps a sequence's first positions in
sight, a sink of score 0 in the softmax, a sigmoid gate on the heads' outputs) or the channel-wise delta
rule (short convolutions, unit-norm queries and keys, a decay per key channel, a state of fixed size).
The feed-forward is a mixture of gated experts chosen by the largest router logits and weighted by the
softmax over the chosen, or absent.  The embedding is multiplied by a constant; the head is untied.

Checkpoint tensors: "embed", "head", "final.norm", and below "l<i>.": "norm1", "norm1b", "norm2", "norm2b",
"mix.<q|k|v|g|o>", "mix.<q|k>.norm" (attention), "mix.<q|k|v>.conv", "mix.<b|a1|a2|g1|g2|o>", "mix.norm",
"mix.dt_bias", "mix.A_log" (delta rule), "mlp.router", "mlp.router.b", "mlp.e<n>.<gate|up|down>": a matrix is
called by its part's name alone and a bias ".b", which ModelSpec.checkpoint_names says.
"""
from __future__ import annotations

from ..config.model_config import KirisunConfig, KirisunLayer
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MAX_POSITION = 1 << 30          # the design names no longest sequence and keeps no table of positions


def _rotary_name(m) -> str:
    return f"rotary-{m.dim}-{m.rot_dims}-{m.rot_base!r}-{m.rot_factor!r}"


def _mixer(cfg: KirisunConfig, layer: KirisunLayer) -> PartSpec:
    m = layer.mixer
    if layer.kind == "attention":
        return PartSpec("attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
            "v_head_dim": m.vdim, "qk_norm": True, "qk_norm_scope": "head", "eps": cfg.eps, "bias": False,
            "position_encoding": _rotary_name(m) if m.rot_dims else None, "step_rotation": True,
            "window": m.window, "keep_first": m.keep_first, "scale": m.scale, "softcap": m.softcap,
            "sink_value": 0.0, "gate": "sigmoid",
            "q_name": "q", "k_name": "k", "v_name": "v", "g_name": "g", "o_name": "o",
            "q_norm_name": "q.norm", "k_norm_name": "k.norm"})
    return PartSpec("channel_delta", {
        "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
        "v_head_dim": m.vdim, "conv_taps": m.conv, "eps": cfg.eps,
        "decay_rank": getattr(m, "decay_rank", None), "gate_rank": getattr(m, "gate_rank", None),
        **{f"{n}_name": n for n in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o")},
        "conv_suffix": "conv", "norm_name": "norm", "dt_bias_name": "dt_bias", "a_log_name": "A_log"})


def _feed_forward(cfg: KirisunConfig, layer: KirisunLayer) -> PartSpec:
    f = layer.mlp
    return PartSpec("moe", {
        "hidden_size": cfg.width, "num_experts": f.experts, "top": f.top, "intermediate_size": f.ff,
        "routing": "softmax_top", "router_bias": True, "gated": True, "activation": "silu",
        "router_name": "router", "expert_name": "e{}", "gate_name": "gate", "up_name": "up", "down_name": "down"})


def build_spec(cfg: KirisunConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"dim": cfg.width, "eps": cfg.eps})
    layers, encodings = [], {}
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer_norm": norm, "mixer": _mixer(cfg, layer), "mixer_post_norm": norm}
        if layer.mlp is not None:
            parts.update(feed_forward_norm=norm, feed_forward=_feed_forward(cfg, layer), feed_forward_post_norm=norm)
        m = layer.mixer
        if layer.kind == "attention" and m.rot_dims:
            encodings[_rotary_name(m)] = PartSpec("rotary_neox", {
                "head_dim": m.dim, "rotary_dim": m.rot_dims, "theta": m.rot_base, "scaling_factor": m.rot_factor,
                "max_position": MAX_POSITION})
        layers.append(LayerSpec(block=PartSpec("sandwich_residual", {"residual_mult": cfg.residual_mult}), parts=parts,
                                name=f"l{i}", names={"mixer_norm": "norm1", "mixer": "mix", "mixer_post_norm": "norm1b",
                                                     "feed_forward_norm": "norm2", "feed_forward": "mlp",
                                                     "feed_forward_post_norm": "norm2b"}))
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=cfg.width, vocab_size=cfg.vocab, max_position=MAX_POSITION,
        dtype=cfg.dtype,
        embedding=PartSpec("token_embedding", {"name": "embed", "scale": cfg.embedding_scale}),
        layers=tuple(layers),
        order=tuple(LayerRun(i) for i in range(len(layers))),
        final_norm=PartSpec("rms_norm", {**norm.params, "name": "final.norm"}),
        head=PartSpec("output_head", {"name": "head", "tied": False}),
        position_encodings=encodings,
        eos_token_ids=cfg.eos_token_id or (),
        checkpoint_names=((".weight", ""), (".bias", ".b")),
    )


register_architecture("Kirisun", KirisunConfig.from_dict, build_spec, replace=True)
