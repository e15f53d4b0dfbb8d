"""Named config.json contents for runs with random weights (there is no checkpoint to read
them from): two tiny test shapes and the Qwen3 dense sizes that the benchmarks use, three
Nozurax shapes (a tiny one, and layers of the Qwen3 1.7B and 8B sizes), two Mafarax shapes (a tiny
one, and layers of the Qwen3 1.7B sizes) and two Kirisun and two Pemuvik shapes of the same kind.  These are
inputs, as a model folder's config.json is; nothing in the model code reads them.

    python -m nano_vllm_amd.cli random-model --shape qwen3-8b --config-only --out DIR
    python -m nano_vllm_amd.cli throughput --model DIR --random-weights 0
"""
from __future__ import annotations

from typing import Dict


def _qwen3(layers, hidden, heads, kv_heads, head_dim, inner, vocab, theta=1e6, eps=1e-6, tied=False,
           max_position=40960, dtype="bfloat16") -> dict:
    return {"architectures": ["Qwen3ForCausalLM"], "hidden_size": hidden, "num_hidden_layers": layers,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
            "intermediate_size": inner, "vocab_size": vocab, "rms_norm_eps": eps, "rope_theta": theta,
            "max_position_embeddings": max_position, "tie_word_embeddings": tied, "attention_bias": False,
            "hidden_act": "silu", "torch_dtype": dtype}


def _nozurax(layers, width, heads, kv_heads, dim, vdim, inner, vocab, eps=1e-6, every=256, dtype="bfloat16",
             ret_heads=None, rot=None, pattern=("attention", "retention")) -> dict:
    """Layers that follow `pattern` in turn, each with tensors of its own: attention (sinks, whole-projection
    norms, a query temperature) and retention (decays 1 - 2^-6 ... 1 - 2^-10 over the heads, rotation of `rot`
    channels, default the whole head)."""
    rh = ret_heads or heads
    kinds = {
        "attention": {"type": "attention", "mlp": {"kind": "dense", "ff": inner},
                      "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                                "q_temp": {"coef": 0.1, "every": every}}},
        "retention": {"type": "retention", "mlp": {"kind": "dense", "ff": inner},
                      "mixer": {"heads": rh, "dim": dim, "vdim": vdim, "rot": {"dims": rot or dim, "base": 1e6},
                                "decay": [1.0 - 2.0 ** (-6 - 4.0 * h / rh) for h in range(rh)]}},
    }
    return {"architecture": "Nozurax", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [kinds[pattern[i % len(pattern)]] for i in range(layers)], "torch_dtype": dtype}


def _mafarax(layers, width, heads, kv_heads, dim, vdim, inner, vocab, chunk, eps=1e-6, dtype="bfloat16", rot=None,
             factor=4.0, ssm_heads=None, ssm_vdim=64, state=128, groups=8, conv=4, norm_groups=1, experts=32, top=6,
             group_count=8, group_keep=4, logit_scale=1.0) -> dict:
    """Layers of a chunked attention and a state-space layer side by side and a routed feed-forward: `top` of
    `experts` experts of inner / 8 each and a shared expert of inner / 4 (a token runs the dense layer's inner size)."""
    layer = {"type": "parallel",
             "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                                "mask": {"size": chunk},
                                "rot": {"dims": rot or dim // 2, "base": 1e6, "scaling": {"factor": factor}}},
                       "right": {"heads": ssm_heads or 2 * width // ssm_vdim, "vdim": ssm_vdim, "state": state,
                                 "groups": groups, "conv": conv, "norm_groups": norm_groups}},
             "mlp": {"kind": "moe", "expert": {"ff": max(1, inner // 8)}, "shared": {"ff": max(1, inner // 4)},
                     "router": {"experts": experts, "top": top, "scale": 1.0,
                                "groups": {"count": group_count, "keep": group_keep}}}}
    return {"architecture": "Mafarax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": [layer] * layers, "torch_dtype": dtype}


def _kirisun(layers, width, heads, kv_heads, dim, vdim, inner, vocab, window, keep_first=4, eps=1e-6, dtype="bfloat16",
             rot=None, factor=4.0, softcap=30.0, delta_heads=None, delta_kv_heads=None, delta_dim=None, delta_vdim=None, conv=4,
             rank=None, experts=32, top=8, residual_mult=0.5, pattern=("channel_delta", "attention")) -> dict:
    """Layers that follow `pattern` in turn: the gated window attention (a cap on the scores, kept first positions,
    half the head rotated) and the channel-wise delta rule (as many value heads of the same size as the attention's
    query heads unless named), each with `top` of `experts` gated experts of inner / top each (a token runs the dense
    layer's inner size)."""
    dh, dd, dv = delta_heads or heads, delta_dim or dim, delta_vdim or vdim
    mlp = {"kind": "moe", "expert": {"ff": max(1, inner // top)}, "router": {"experts": experts, "top": top}}
    kinds = {
        "attention": {"type": "attention", "mlp": mlp,
                      "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                                "softcap": softcap, "mask": {"size": window, "keep_first": keep_first},
                                "rot": {"dims": rot or dim // 2, "base": 1e6, "scaling": {"factor": factor}}}},
        "channel_delta": {"type": "channel_delta", "mlp": mlp,
                          "mixer": {"heads": dh, "kv_heads": delta_kv_heads or dh, "dim": dd, "vdim": dv, "conv": conv,
                                    "decay_rank": rank or max(1, dd // 2), "gate_rank": rank or max(1, dd // 2)}},
    }
    return {"architecture": "Kirisun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": residual_mult,
            "embedding": {"scale": 8.0}, "layers": [kinds[pattern[i % len(pattern)]] for i in range(layers)],
            "torch_dtype": dtype}


def _pemuvik(layers, width, heads, kv_heads, dim, vdim, inner, vocab, window, eps=1e-6, dtype="bfloat16", rot=None,
             latent_heads=None, latent_dim=None, latent_rot=None, latent_vdim=None, kv_rank=None, experts=32, top=8, identity=2,
             group_count=1, group_keep=1, pattern=(("attention", "moe"), ("latent_attention", "dense"))) -> dict:
    """Layers that follow `pattern` in turn: the window attention with sigmoid weights (half the head rotated, values
    normed and mixed with the first such layer's) and the attention through a latent (as many heads as the other has
    query heads, a latent of kv_rank entries and a rotated key part of half a head unless named), each with a dense
    gated layer of `inner` or with `top` of `experts` gated experts of inner / top each (and `identity` outputs that
    give the input back) beside a shared expert of inner / 4."""
    lh, ld, lv = latent_heads or heads, latent_dim or dim, latent_vdim or vdim
    lr = latent_rot or max(2, dim // 2)
    mixers = {
        "attention": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "v_mix": True,
                      "mask": {"size": window}, "rot": {"dims": rot or dim // 2, "base": 1e6}},
        "latent_attention": {"heads": lh, "dim": ld, "rot_dim": lr, "vdim": lv, "kv_rank": kv_rank or 3 * dim,
                             "scale": (ld + lr) ** -0.5, "rot": {"dims": lr, "base": 1e4}},
    }
    mlps = {
        "dense": {"kind": "dense", "ff": inner},
        "moe": {"kind": "moe", "expert": {"ff": max(1, inner // top)}, "shared": {"ff": max(1, inner // 4)},
                "router": {"experts": experts, "top": top, "identity": identity,
                           "groups": {"count": group_count, "keep": group_keep}}},
        None: None,
    }
    return {"architecture": "Pemuvik", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [{"type": pattern[i % len(pattern)][0], "mixer": mixers[pattern[i % len(pattern)][0]],
                        "mlp": mlps[pattern[i % len(pattern)][1]]} for i in range(layers)],
            "torch_dtype": dtype}


SHAPES: Dict[str, dict] = {
    "pemuvik-tiny": _pemuvik(4, 64, 4, 2, 16, 24, 96, 256, window=12, eps=1e-5, dtype="float32", rot=8, latent_heads=2, latent_dim=12,
                             latent_rot=4, latent_vdim=8, kv_rank=20, experts=6, top=2, identity=2, group_count=4, group_keep=2),
    "pemuvik-1b": _pemuvik(16, 2048, 16, 8, 128, 128, 6144, 32768, window=1024, experts=30, group_count=4, group_keep=2),
    "kirisun-tiny": _kirisun(4, 64, 4, 2, 16, 24, 96, 256, window=12, keep_first=3, eps=1e-5, dtype="float32", rot=8, softcap=5.0,
                             delta_heads=4, delta_kv_heads=2, delta_dim=12, delta_vdim=8, conv=3, rank=3, experts=6, top=2),
    "kirisun-1b": _kirisun(16, 2048, 16, 8, 128, 128, 6144, 32768, window=1024),
    "mafarax-tiny": _mafarax(3, 64, 4, 2, 16, 24, 96, 256, chunk=12, eps=1e-5, dtype="float32", rot=8, ssm_heads=4,
                             ssm_vdim=8, state=12, groups=2, conv=3, norm_groups=2, experts=6, top=2, group_count=3,
                             group_keep=2, logit_scale=1.5),
    "mafarax-1b": _mafarax(16, 2048, 16, 8, 128, 128, 6144, 32768, chunk=1024),
    "nozurax-tiny": _nozurax(4, 64, 4, 2, 16, 24, 96, 256, eps=1e-5, every=8, dtype="float32", ret_heads=2, rot=8),
    "nozurax-1b": _nozurax(16, 2048, 16, 8, 128, 128, 6144, 32768),
    "nozurax-8b": _nozurax(32, 4096, 32, 8, 128, 128, 12288, 32768),
    "tiny-a": _qwen3(2, 64, 4, 2, 16, 128, 256, theta=1e4, tied=True, max_position=128, dtype="float32"),
    "tiny-b": _qwen3(3, 96, 8, 2, 32, 160, 384, eps=1e-5, max_position=256, dtype="float32"),
    "qwen3-0.6b": _qwen3(28, 1024, 16, 8, 128, 3072, 151936, tied=True),     # the model of the reference's README benchmark
    "qwen3-1.7b": _qwen3(28, 2048, 16, 8, 128, 6144, 151936, tied=True),
    "qwen3-4b": _qwen3(36, 2560, 32, 8, 128, 9728, 151936, tied=True),
    "qwen3-8b": _qwen3(36, 4096, 32, 8, 128, 12288, 151936),
    "qwen3-14b": _qwen3(40, 5120, 40, 8, 128, 17408, 151936),
    "qwen3-32b": _qwen3(64, 5120, 64, 8, 128, 25600, 151936),
}


def shape(name: str) -> dict:
    if name not in SHAPES:
        raise KeyError(f"unknown shape {name!r}; known: {sorted(SHAPES)}")
    return dict(SHAPES[name])
