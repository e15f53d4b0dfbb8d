"""Pemuvik as data: config.json -> typed configuration -> ModelSpec.

Every layer is the parallel residual block on a float32 stream with a norm for each sublayer (both read the
same stream) and a learned vector on each sublayer's output (layer scale).  The mixer is, entry by entry of the
configuration's list, a grouped window attention without a softmax (biases, neighbouring pairs rotated, normed
values, values mixed with the first such layer's, a key's weight sigmoid(score + a number per head)) or an
attention through a shared latent (a normed latent row and one rotated key part per token, a sink in the
softmax).  The feed-forward is the gated dense layer with the tanh form of gelu, a mixture of gated silu experts
chosen by softmax scores plus a correction within the best groups (with identity outputs and a gated shared
expert), or absent.  The head is the embedding table.

Checkpoint tensors: "embed", "final.norm", and below "l<i>.": "norm1", "norm2", "ls1", "ls2", "mix.<q|k|v|o>" with
".b", "mix.vmix", "mix.pb" (window attention), "mix.<q|dkv|uk|uv|o>", "mix.dkv.norm", "mix.sink" (latent attention),
"mlp.<gate|up|down>" (dense), "mlp.router", "mlp.correction", "mlp.e<n>.<gate|up|down>", "mlp.shared.<gate|up|down|sg>":
a matrix is called by its part's name alone and a bias ".b", which ModelSpec.checkpoint_names says.
"""
from __future__ import annotations

from ..config.model_config import PemuvikConfig, PemuvikLayer
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MAX_POSITION = 1 << 30          # the design names no longest sequence and keeps no table of positions


def _rotary_name(dims: int, base: float) -> str:
    return f"pairs-{dims}-{base!r}"


def _mixer(cfg: PemuvikConfig, layer: PemuvikLayer) -> PartSpec:
    m = layer.mixer
    if layer.kind == "attention":
        return PartSpec("attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
            "v_head_dim": m.vdim, "qk_norm": False, "eps": cfg.eps, "bias": True, "o_bias": True,
            "position_encoding": _rotary_name(m.rot_dims, m.rot_base) if m.rot_dims else None, "step_rotation": True,
            "window": m.window, "scale": m.scale, "weights": "sigmoid", "score_bias_name": "pb",
            "v_norm": True, "v_mix": "values" if m.v_mix else None, "v_mix_name": "vmix",
            "q_name": "q", "k_name": "k", "v_name": "v", "o_name": "o"})
    return PartSpec("latent_attention", {
        "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "v_head_dim": m.vdim,
        "kv_rank": m.kv_rank, "eps": cfg.eps, "scale": m.scale, "sink": True,
        "position_encoding": _rotary_name(m.rot_dim, m.rot_base),
        "q_name": "q", "dkv_name": "dkv", "dkv_norm_name": "dkv.norm", "uk_name": "uk", "uv_name": "uv",
        "sink_name": "sink", "o_name": "o"})


_GATED = {"gate_name": "gate", "up_name": "up", "down_name": "down"}


def _feed_forward(cfg: PemuvikConfig, layer: PemuvikLayer) -> PartSpec:
    f = layer.mlp
    if isinstance(f, int):
        return PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": f, "activation": "gelu_tanh", **_GATED})
    shared = None
    if f.shared_ff is not None:
        shared = PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": f.shared_ff, "activation": "silu", **_GATED})
    return PartSpec("moe", {
        "hidden_size": cfg.width, "num_experts": f.experts, "identity": f.identity, "top": f.top, "intermediate_size": f.ff,
        "routing": "softmax_choice", "group_count": f.group_count, "group_keep": f.group_keep, "gated": True,
        "activation": "silu", "shared": shared, "shared_gate": shared is not None, "shared_gate_name": "sg",
        "router_name": "router", "correction_name": "correction", "shared_name": "shared", "expert_name": "e{}", **_GATED})


def build_spec(cfg: PemuvikConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"dim": cfg.width, "eps": cfg.eps})
    layers, encodings = [], {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        dims = m.rot_dims if layer.kind == "attention" else m.rot_dim
        if dims:
            encodings[_rotary_name(dims, m.rot_base)] = PartSpec("rotary_interleaved", {
                "head_dim": dims, "rotary_dim": dims, "theta": m.rot_base, "max_position": MAX_POSITION})
        parts = {"norm": norm, "mixer": _mixer(cfg, layer)}
        if layer.mlp is not None:
            parts.update(feed_forward_norm=norm, feed_forward=_feed_forward(cfg, layer))
        layers.append(LayerSpec(
            block=PartSpec("parallel_residual", {"layer_scale": True, "mixer_scale_name": "ls1", "feed_forward_scale_name": "ls2"}),
            parts=parts, name=f"l{i}",
            names={"norm": "norm1", "mixer": "mix", "feed_forward_norm": "norm2", "feed_forward": "mlp"}))
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=cfg.width, vocab_size=cfg.vocab, max_position=MAX_POSITION,
        dtype=cfg.dtype,
        embedding=PartSpec("token_embedding", {"name": "embed"}),
        layers=tuple(layers),
        order=tuple(LayerRun(i) for i in range(len(layers))),
        final_norm=PartSpec("rms_norm", {**norm.params, "name": "final.norm"}),
        head=PartSpec("output_head", {"name": "head", "tied": True}),
        position_encodings=encodings,
        eos_token_ids=cfg.eos_token_id or (),
        checkpoint_names=((".weight", ""), (".bias", ".b")),
    )


register_architecture("Pemuvik", PemuvikConfig.from_dict, build_spec, replace=True)
