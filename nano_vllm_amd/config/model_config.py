"""Typed model configuration, read from the architecture's own config.json keys.

Reference: the keys that nanovllm/models/qwen3.py:128-144,169-171,201-202 and
nanovllm/engine/model_runner.py:29,110-112 read from the Hugging Face config object.
Nothing here imports transformers: config.json is parsed as plain JSON.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict, fields
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value the engine cannot honour."""


_DTYPE_NAMES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16", "torch.bfloat16": "bfloat16",
    "float32": "float32", "fp32": "float32", "float": "float32", "torch.float32": "float32",
    "float16": "float16", "fp16": "float16", "half": "float16", "torch.float16": "float16",
}


def canonical_dtype(name: str) -> str:
    try:
        return _DTYPE_NAMES[str(name)]
    except KeyError:
        raise ConfigError(f"unknown dtype {name!r}; known: {sorted(set(_DTYPE_NAMES.values()))}")


def _require(d: Mapping[str, Any], key: str, typ, where: str):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key {key!r} is missing")
    v = d[key]
    if typ is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"{where}: key {key!r} must be an integer, got {v!r}")
    if typ is float and (isinstance(v, bool) or not isinstance(v, (int, float))):
        raise ConfigError(f"{where}: key {key!r} must be a number, got {v!r}")
    return typ(v)


@dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense decoder.  Field names are config.json's own."""
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    hidden_act: str = "silu"
    dtype: str = "bfloat16"
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Qwen3ForCausalLM"

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen3Config":
        where = "config.json"
        hidden = _require(d, "hidden_size", int, where)
        heads = _require(d, "num_attention_heads", int, where)
        kv_heads = _require(d, "num_key_value_heads", int, where)
        # head_dim absent or null -> hidden // heads (qwen3.py:36,134)
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(f"{where}: head_dim is absent and hidden_size {hidden} is "
                                  f"not a multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        # rope_theta default 1e6 (qwen3.py:135); a rope_scaling dict may carry only a
        # rope_theta of its own (qwen3.py:54-55) - the reference applies no other scaling.
        theta = d.get("rope_theta", 1000000.0)
        scaling = d.get("rope_scaling")
        if isinstance(scaling, dict):
            other = {k: v for k, v in scaling.items()
                     if k not in ("rope_theta", "rope_type", "type") and v is not None}
            kind = scaling.get("rope_type", scaling.get("type", "default"))
            if other or kind not in ("default", None):
                raise ConfigError(f"{where}: rope_scaling {scaling!r} asks for scaled rotary "
                                  "frequencies, which this architecture's engine does not apply")
            theta = scaling.get("rope_theta", theta)
        elif scaling is not None:
            raise ConfigError(f"{where}: rope_scaling must be null or an object, got {scaling!r}")
        if d.get("use_sliding_window"):
            raise ConfigError(f"{where}: use_sliding_window=true is not honoured by this "
                              "architecture (the reference reads no window key); refusing "
                              "rather than attending to all keys silently")
        act = d.get("hidden_act", "silu")
        if act != "silu":                                          # qwen3.py:110
            raise ConfigError(f"{where}: hidden_act must be 'silu', got {act!r}")
        dtype = canonical_dtype(d.get("dtype") or d.get("torch_dtype") or "bfloat16")
        eos = d.get("eos_token_id")
        if isinstance(eos, int):
            eos = (eos,)
        elif isinstance(eos, (list, tuple)):
            eos = tuple(int(x) for x in eos)
        else:
            eos = None
        cfg = cls(
            vocab_size=_require(d, "vocab_size", int, where),
            hidden_size=hidden,
            num_hidden_layers=_require(d, "num_hidden_layers", int, where),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=int(head_dim),
            intermediate_size=_require(d, "intermediate_size", int, where),
            rms_norm_eps=_require(d, "rms_norm_eps", float, where),
            rope_theta=float(theta),
            max_position_embeddings=_require(d, "max_position_embeddings", int, where),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            # The reference's getattr default is True (qwen3.py:133); every Qwen3 file
            # states false, so an absent key means no bias here.
            attention_bias=bool(d.get("attention_bias", False)),
            hidden_act=act,
            dtype=dtype,
            eos_token_id=eos,
            architecture=(d.get("architectures") or ["Qwen3ForCausalLM"])[0],
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for f in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "intermediate_size",
                  "max_position_embeddings"):
            if getattr(self, f) <= 0:
                raise ConfigError(f"config.json: {f} must be positive, got {getattr(self, f)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple "
                f"of num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary pairs")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")

    def to_dict(self) -> dict:
        """The config.json that describes this configuration."""
        d = asdict(self)
        arch = d.pop("architecture")
        dtype = d.pop("dtype")
        eos = d.pop("eos_token_id")
        out = {"architectures": [arch], "model_type": "qwen3"}
        out.update(d)
        out["torch_dtype"] = dtype
        out["rope_scaling"] = None
        out["use_sliding_window"] = False
        if eos is not None:
            out["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        return out

    def replace(self, **kw) -> "Qwen3Config":
        d = {f.name: getattr(self, f.name) for f in fields(self)}
        d.update(kw)
        return Qwen3Config(**d)


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder!r} holds no config.json")
    with open(path) as f:
        return json.load(f)


# ---------------------------------------------------------------------------- Nozurax
def _section(d: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    v = d.get(key)
    if not isinstance(v, Mapping):
        raise ConfigError(f"{where}: key {key!r} must be an object")
    return v


@dataclass(frozen=True)
class NozuraxLayer:
    """One entry of config.json's "layers".  kind: "attention" | "retention".  weights_of: the
    entry whose tensors this one runs (itself where it has its own).  ff: the feed-forward's inner
    size, None for a layer without one.  The mixer's sizes and constants by their config names:
    attention  heads, kv_heads, dim, vdim, scale, temp_coef, temp_every (temp_coef 0: no temperature)
    retention  heads, dim, vdim, decay (one per head), rot_dims, rot_base (rot_dims 0: no rotation)"""
    kind: str
    weights_of: int
    ff: Optional[int]
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0
    scale: float = 1.0
    temp_coef: float = 0.0
    temp_every: int = 1
    decay: Tuple[float, ...] = ()
    rot_dims: int = 0
    rot_base: float = 10000.0


@dataclass(frozen=True)
class NozuraxConfig:
    """Nozurax: a decoder whose layers add a mixer and a feed-forward that read the same norm, with
    retention and sink-attention mixers in an order the configuration gives, and layers that may run
    another layer's tensors again.  config.json gives every size and constant."""
    vocab: int
    width: int
    eps: float
    layers: Tuple[NozuraxLayer, ...]
    dtype: str = "bfloat16"
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Nozurax"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "NozuraxConfig":
        where = "config.json"
        entries = d.get("layers")
        if not isinstance(entries, (list, tuple)):
            raise ConfigError(f"{where}: key 'layers' must be a list")
        layers = []
        for i, entry in enumerate(entries):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at} must be an object")
            kind = entry.get("type")
            m = _section(entry, "mixer", at)
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{at}: mlp must be null or an object of kind 'dense', got {mlp!r}")
                ff = _require(mlp, "ff", int, at + ".mlp")
            common = dict(kind=kind, weights_of=int(entry.get("weights_of", i)), ff=ff,
                          heads=_require(m, "heads", int, at + ".mixer"), dim=_require(m, "dim", int, at + ".mixer"),
                          vdim=_require(m, "vdim", int, at + ".mixer"))
            if kind == "attention":
                temp = m.get("q_temp")
                coef, every = 0.0, 1
                if temp is not None:
                    coef = _require(temp, "coef", float, at + ".mixer.q_temp")
                    every = temp.get("every")
                    if isinstance(every, bool) or not isinstance(every, (int, float)) or every != int(every) or every <= 0:
                        raise ConfigError(f"{at}.mixer.q_temp: 'every' must be a positive whole number, got {every!r}")
                layers.append(NozuraxLayer(**common, kv_heads=_require(m, "kv_heads", int, at + ".mixer"),
                                           scale=_require(m, "scale", float, at + ".mixer"), temp_coef=coef,
                                           temp_every=int(every)))
            elif kind == "retention":
                decay = m.get("decay")
                if not isinstance(decay, (list, tuple)) or any(isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay):
                    raise ConfigError(f"{at}.mixer: 'decay' must be a list of numbers, one per head")
                rot = m.get("rot")
                dims, base = 0, 10000.0
                if rot is not None:
                    dims = _require(rot, "dims", int, at + ".mixer.rot")
                    base = _require(rot, "base", float, at + ".mixer.rot")
                layers.append(NozuraxLayer(**common, decay=tuple(float(x) for x in decay), rot_dims=dims, rot_base=base))
            else:
                raise ConfigError(f"{at}: type must be 'attention' or 'retention', got {kind!r}")
        norm = _section(d, "norm", where)
        eos = d.get("eos_token_id")
        eos = (eos,) if isinstance(eos, int) else tuple(int(x) for x in eos) if isinstance(eos, (list, tuple)) else None
        cfg = cls(vocab=_require(d, "vocab", int, where), width=_require(d, "width", int, where),
                  eps=_require(norm, "eps", float, where + ": norm"), layers=tuple(layers),
                  dtype=canonical_dtype(d.get("dtype") or d.get("torch_dtype") or "bfloat16"), eos_token_id=eos,
                  architecture=d.get("architecture") or (d.get("architectures") or ["Nozurax"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"config.json: vocab and width must be positive, got {self.vocab} and {self.width}")
        if not (self.eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.eps}")
        for i, layer in enumerate(self.layers):
            at = f"config.json: layers[{i}]"
            if min(layer.heads, layer.dim, layer.vdim) <= 0 or (layer.ff is not None and layer.ff <= 0):
                raise ConfigError(f"{at}: heads, dim, vdim and ff must be positive")
            j = layer.weights_of
            if j != i:
                if not 0 <= j < len(self.layers) or self.layers[j].weights_of != j:
                    raise ConfigError(f"{at}: weights_of names layer {j}, which must exist and have tensors of its own")
                own = self.layers[j]
                if (own.kind, own.heads, own.dim, own.vdim, own.kv_heads, own.ff) != \
                        (layer.kind, layer.heads, layer.dim, layer.vdim, layer.kv_heads, layer.ff):
                    raise ConfigError(f"{at}: its sizes differ from those of layer {j}, whose tensors it runs")
            if layer.kind == "attention":
                if layer.kv_heads <= 0 or layer.heads % layer.kv_heads:
                    raise ConfigError(f"{at}: {layer.heads} heads do not divide into {layer.kv_heads} kv_heads")
            else:
                if len(layer.decay) != layer.heads:
                    raise ConfigError(f"{at}: {len(layer.decay)} decays for {layer.heads} heads")
                if any(not 0.0 <= x <= 1.0 for x in layer.decay):
                    raise ConfigError(f"{at}: a decay must lie in [0, 1]")
                if layer.rot_dims % 2 or not 0 <= layer.rot_dims <= layer.dim or (layer.rot_dims and not layer.rot_base > 0):
                    raise ConfigError(f"{at}: rot.dims {layer.rot_dims} must be even and at most dim {layer.dim}, rot.base positive")

    def to_dict(self) -> dict:
        """The config.json that describes this configuration."""
        entries = []
        for i, layer in enumerate(self.layers):
            if layer.kind == "attention":
                mixer = {"heads": layer.heads, "kv_heads": layer.kv_heads, "dim": layer.dim, "vdim": layer.vdim,
                         "scale": layer.scale}
                if layer.temp_coef:
                    mixer["q_temp"] = {"coef": layer.temp_coef, "every": layer.temp_every}
            else:
                mixer = {"heads": layer.heads, "dim": layer.dim, "vdim": layer.vdim, "decay": list(layer.decay)}
                if layer.rot_dims:
                    mixer["rot"] = {"dims": layer.rot_dims, "base": layer.rot_base}
            entry = {"type": layer.kind, "mixer": mixer,
                     "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}}
            if layer.weights_of != i:
                entry["weights_of"] = layer.weights_of
            entries.append(entry)
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "layers": entries, "torch_dtype": self.dtype}
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


# ---------------------------------------------------------------------------- Mafarax
def _whole(d: Mapping[str, Any], key: str, where: str, default=None) -> int:
    """A positive whole number (config files may write 4 as 4.0)."""
    v = d.get(key, default)
    if v is None or isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v) or int(v) <= 0:
        raise ConfigError(f"{where}: key {key!r} must be a positive whole number, got {v!r}")
    return int(v)


@dataclass(frozen=True)
class ChunkAttentionConfig:
    """The attention half of a side-by-side mixer: grouped keys and values, values of a size of their
    own, biases, rotation of the first rot_dims channels of a head with every frequency divided by
    rot_factor, a scale of its own, and a mask that lets a query read its own chunk of `chunk`
    positions only.  rot_dims 0: no rotation."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_factor: float = 1.0


@dataclass(frozen=True)
class StateSpaceConfig:
    """The state-space half: heads of vdim channels, a state of `state` rows per head, B and C shared
    by the heads of a group, a causal convolution of `conv` taps, a gated norm in norm_groups parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class ExpertsConfig:
    """A routed feed-forward: `experts` experts of inner size ff, `top` per token, chosen among the
    `keep` best of `group_count` groups of neighbouring experts; weights are the sigmoid scores
    times `scale`; shared_ff: the inner size of the expert every token runs (None: no such expert)."""
    experts: int
    top: int
    ff: int
    scale: float
    group_count: int = 1
    group_keep: int = 1
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class MafaraxLayer:
    left: ChunkAttentionConfig
    right: StateSpaceConfig
    mlp: Optional[ExpertsConfig]


@dataclass(frozen=True)
class MafaraxConfig:
    """Mafarax: pre-norm layers on a float32 residual stream with Dynamic Tanh norms; every mixer is a
    chunked attention and a state-space layer side by side on the same input, their outputs normed
    and averaged; the feed-forward is a mixture of experts with a shared expert, or absent.
    config.json gives every size and constant, layer by layer."""
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: Tuple[MafaraxLayer, ...]
    dtype: str = "bfloat16"
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Mafarax"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "MafaraxConfig":
        where = "config.json"
        entries = d.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: key 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(entries):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at} must be an object")
            if entry.get("type") != "parallel":
                raise ConfigError(f"{at}: type must be 'parallel', got {entry.get('type')!r}")
            mixer = _section(entry, "mixer", at)
            l, r = _section(mixer, "left", at + ".mixer"), _section(mixer, "right", at + ".mixer")
            la, ra = at + ".mixer.left", at + ".mixer.right"
            rot = l.get("rot")
            dims, base, factor = 0, 10000.0, 1.0
            if rot is not None:
                dims = _whole(rot, "dims", la + ".rot")
                base = _require(rot, "base", float, la + ".rot")
                scaling = rot.get("scaling")
                if scaling is not None:
                    factor = _require(scaling, "factor", float, la + ".rot.scaling")
            mask = _section(l, "mask", la)
            left = ChunkAttentionConfig(
                heads=_whole(l, "heads", la), kv_heads=_whole(l, "kv_heads", la), dim=_whole(l, "dim", la),
                vdim=_whole(l, "vdim", la), scale=_require(l, "scale", float, la), chunk=_whole(mask, "size", la + ".mask"),
                rot_dims=dims, rot_base=base, rot_factor=factor)
            right = StateSpaceConfig(
                heads=_whole(r, "heads", ra), vdim=_whole(r, "vdim", ra), state=_whole(r, "state", ra),
                groups=_whole(r, "groups", ra, 1), conv=_whole(r, "conv", ra),
                norm_groups=_whole(r, "norm_groups", ra, 1))
            mlp = entry.get("mlp")
            experts = None
            if mlp is not None:
                ma = at + ".mlp"
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "moe":
                    raise ConfigError(f"{ma} must be null or an object of kind 'moe', got {mlp!r}")
                router = _section(mlp, "router", ma)
                groups = router.get("groups")
                shared = mlp.get("shared")
                experts = ExpertsConfig(
                    experts=_whole(router, "experts", ma + ".router"), top=_whole(router, "top", ma + ".router"),
                    ff=_whole(_section(mlp, "expert", ma), "ff", ma + ".expert"),
                    scale=float(router["scale"]) if router.get("scale") is not None else 1.0,
                    group_count=1 if groups is None else _whole(groups, "count", ma + ".router.groups"),
                    group_keep=1 if groups is None else _whole(groups, "keep", ma + ".router.groups"),
                    shared_ff=None if shared is None else _whole(shared, "ff", ma + ".shared"))
            layers.append(MafaraxLayer(left, right, experts))
        norm = _section(d, "norm", where)
        eos = d.get("eos_token_id")
        eos = (eos,) if isinstance(eos, int) else tuple(int(x) for x in eos) if isinstance(eos, (list, tuple)) else None
        cfg = cls(vocab=_whole(d, "vocab", where), width=_whole(d, "width", where),
                  eps=_require(norm, "eps", float, where + ": norm"),
                  logit_scale=float(d["logit_scale"]) if d.get("logit_scale") is not None else 1.0,
                  layers=tuple(layers), dtype=canonical_dtype(d.get("dtype") or d.get("torch_dtype") or "bfloat16"),
                  eos_token_id=eos, architecture=d.get("architecture") or (d.get("architectures") or ["Mafarax"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not (self.eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.eps}")
        for i, layer in enumerate(self.layers):
            at = f"config.json: layers[{i}]"
            l, r, m = layer.left, layer.right, layer.mlp
            if l.heads % l.kv_heads:
                raise ConfigError(f"{at}: {l.heads} heads do not divide into {l.kv_heads} kv_heads")
            if l.rot_dims % 2 or l.rot_dims > l.dim or (l.rot_dims and not (l.rot_base > 0 and l.rot_factor > 0)):
                raise ConfigError(f"{at}: rot.dims {l.rot_dims} must be even and at most dim {l.dim}, rot.base and "
                                  f"the scaling factor positive")
            if r.heads % r.groups:
                raise ConfigError(f"{at}: {r.heads} state-space heads do not divide into {r.groups} groups")
            if (r.heads * r.vdim) % r.norm_groups:
                raise ConfigError(f"{at}: {r.heads * r.vdim} inner channels do not divide into {r.norm_groups} norm groups")
            if m is not None:
                if m.experts % m.group_count or not 1 <= m.group_keep <= m.group_count:
                    raise ConfigError(f"{at}: {m.experts} experts in {m.group_count} groups, of which {m.group_keep} are kept")
                if m.top > m.group_keep * (m.experts // m.group_count):
                    raise ConfigError(f"{at}: {m.top} experts a token cannot be chosen from {m.group_keep} groups of "
                                      f"{m.experts // m.group_count}")

    def to_dict(self) -> dict:
        """The config.json that describes this configuration."""
        entries = []
        for layer in self.layers:
            l, r, m = layer.left, layer.right, layer.mlp
            left = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                    "mask": {"size": l.chunk}}
            if l.rot_dims:
                left["rot"] = {"dims": l.rot_dims, "base": l.rot_base, "scaling": {"factor": l.rot_factor}}
            right = {"heads": r.heads, "vdim": r.vdim, "state": r.state, "groups": r.groups, "conv": r.conv,
                     "norm_groups": r.norm_groups}
            mlp = None
            if m is not None:
                mlp = {"kind": "moe", "expert": {"ff": m.ff},
                       "router": {"experts": m.experts, "top": m.top, "scale": m.scale,
                                  "groups": {"count": m.group_count, "keep": m.group_keep}},
                       "shared": None if m.shared_ff is None else {"ff": m.shared_ff}}
            entries.append({"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "logit_scale": self.logit_scale, "layers": entries, "torch_dtype": self.dtype}
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


# ---------------------------------------------------------------------------- Kirisun
def _count(d: Mapping[str, Any], key: str, where: str, default=None) -> int:
    """A whole number that may be zero."""
    v = d.get(key, default)
    if v is None or isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v) or int(v) < 0:
        raise ConfigError(f"{where}: key {key!r} must be a whole number, zero or more, got {v!r}")
    return int(v)


@dataclass(frozen=True)
class GatedAttentionConfig:
    """Grouped attention with normed query and key heads, a rotation of the first rot_dims channels of a head
    (every frequency divided by rot_factor; rot_dims 0: none), scores scale * q.k capped smoothly at +-softcap
    (None: no cap), a window of `window` positions that also keeps the first keep_first positions of the
    sequence in sight (window None: every earlier position), a sink of score 0 in the softmax, and an
    output gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float] = None
    window: Optional[int] = None
    keep_first: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_factor: float = 1.0


@dataclass(frozen=True)
class ChannelDeltaConfig:
    """The delta-rule mixer with a decay per key channel: `heads` value heads of vdim, kv_heads query/key heads
    of dim, short convolutions of `conv` taps; the ranks of the two-step projections of the decay and of the
    output gate are read from the tensors' shapes unless the mixer names them (decay_rank, gate_rank: what a
    folder of random weights is drawn with)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None


@dataclass(frozen=True)
class SoftmaxExpertsConfig:
    """A routed feed-forward of gated experts: `top` of `experts` experts of inner size ff, weighted by the
    softmax over the chosen router logits."""
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class KirisunLayer:
    kind: str                                    # "attention" | "channel_delta"
    mixer: Any                                   # GatedAttentionConfig | ChannelDeltaConfig
    mlp: Optional[SoftmaxExpertsConfig]


@dataclass(frozen=True)
class KirisunConfig:
    """Kirisun: layers with a norm before and after each sublayer on a float32 residual stream that takes each
    sublayer's normed output times residual_mult; the mixer is, layer by layer, a gated window attention or
    the channel-wise delta rule; the feed-forward a mixture of gated experts, or absent; the embedding is
    multiplied by embedding_scale.  config.json gives every size and constant, layer by layer."""
    vocab: int
    width: int
    eps: float
    residual_mult: float
    embedding_scale: float
    layers: Tuple[KirisunLayer, ...]
    dtype: str = "bfloat16"
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Kirisun"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "KirisunConfig":
        where = "config.json"
        entries = d.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: key 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(entries):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at} must be an object")
            kind = entry.get("type")
            m = _section(entry, "mixer", at)
            ma = at + ".mixer"
            sizes = dict(heads=_whole(m, "heads", ma), kv_heads=_whole(m, "kv_heads", ma), dim=_whole(m, "dim", ma),
                         vdim=_whole(m, "vdim", ma))
            if kind == "attention":
                rot, mask = m.get("rot"), m.get("mask")
                dims, base, factor = 0, 10000.0, 1.0
                if rot is not None:
                    dims = _whole(rot, "dims", ma + ".rot")
                    base = _require(rot, "base", float, ma + ".rot")
                    if rot.get("scaling") is not None:
                        factor = _require(rot["scaling"], "factor", float, ma + ".rot.scaling")
                cap = m.get("softcap")
                mixer = GatedAttentionConfig(
                    **sizes, scale=_require(m, "scale", float, ma),
                    softcap=None if cap is None else _require(m, "softcap", float, ma),
                    window=None if mask is None else _whole(mask, "size", ma + ".mask"),
                    keep_first=0 if mask is None else _count(mask, "keep_first", ma + ".mask", 0),
                    rot_dims=dims, rot_base=base, rot_factor=factor)
            elif kind == "channel_delta":
                mixer = ChannelDeltaConfig(**sizes, conv=_whole(m, "conv", ma),
                                           decay_rank=None if m.get("decay_rank") is None else _whole(m, "decay_rank", ma),
                                           gate_rank=None if m.get("gate_rank") is None else _whole(m, "gate_rank", ma))
            else:
                raise ConfigError(f"{at}: type must be 'attention' or 'channel_delta', got {kind!r}")
            mlp = entry.get("mlp")
            experts = None
            if mlp is not None:
                fa = at + ".mlp"
                if not isinstance(mlp, Mapping) or mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"{fa} must be null or an object of kind 'moe', got {mlp!r}")
                router = _section(mlp, "router", fa)
                experts = SoftmaxExpertsConfig(experts=_whole(router, "experts", fa + ".router"),
                                               top=_whole(router, "top", fa + ".router"),
                                               ff=_whole(_section(mlp, "expert", fa), "ff", fa + ".expert"))
            layers.append(KirisunLayer(kind, mixer, experts))
        norm = _section(d, "norm", where)
        embedding = d.get("embedding") or {}
        eos = d.get("eos_token_id")
        eos = (eos,) if isinstance(eos, int) else tuple(int(x) for x in eos) if isinstance(eos, (list, tuple)) else None
        cfg = cls(vocab=_whole(d, "vocab", where), width=_whole(d, "width", where),
                  eps=_require(norm, "eps", float, where + ": norm"),
                  residual_mult=float(d["residual_mult"]) if d.get("residual_mult") is not None else 1.0,
                  embedding_scale=float(embedding["scale"]) if embedding.get("scale") is not None else 1.0,
                  layers=tuple(layers), dtype=canonical_dtype(d.get("dtype") or d.get("torch_dtype") or "bfloat16"),
                  eos_token_id=eos, architecture=d.get("architecture") or (d.get("architectures") or ["Kirisun"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not (self.eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.eps}")
        for i, layer in enumerate(self.layers):
            at = f"config.json: layers[{i}]"
            m, f = layer.mixer, layer.mlp
            if m.heads % m.kv_heads:
                raise ConfigError(f"{at}: {m.heads} heads do not divide into {m.kv_heads} kv_heads")
            if layer.kind == "attention":
                if m.rot_dims % 2 or m.rot_dims > m.dim or (m.rot_dims and not (m.rot_base > 0 and m.rot_factor > 0)):
                    raise ConfigError(f"{at}: rot.dims {m.rot_dims} must be even and at most dim {m.dim}, rot.base and "
                                      f"the scaling factor positive")
                if not (m.scale > 0) or (m.softcap is not None and not (m.softcap > 0)):
                    raise ConfigError(f"{at}: scale and softcap must be positive, got {m.scale} and {m.softcap}")
            if f is not None and f.top > f.experts:
                raise ConfigError(f"{at}: {f.top} experts a token out of {f.experts}")

    def to_dict(self) -> dict:
        """The config.json that describes this configuration."""
        entries = []
        for layer in self.layers:
            m, f = layer.mixer, layer.mlp
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim}
            if layer.kind == "attention":
                mixer["scale"] = m.scale
                if m.softcap is not None:
                    mixer["softcap"] = m.softcap
                if m.window is not None:
                    mixer["mask"] = {"size": m.window, "keep_first": m.keep_first}
                if m.rot_dims:
                    mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base, "scaling": {"factor": m.rot_factor}}
            else:
                mixer["conv"] = m.conv
                for key in ("decay_rank", "gate_rank"):
                    if getattr(m, key) is not None:
                        mixer[key] = getattr(m, key)
            mlp = None if f is None else {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
            entries.append({"type": layer.kind, "mixer": mixer, "mlp": mlp})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "residual_mult": self.residual_mult, "embedding": {"scale": self.embedding_scale}, "layers": entries,
               "torch_dtype": self.dtype}
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


# ---------------------------------------------------------------------------- Pemuvik
@dataclass(frozen=True)
class SigmoidAttentionConfig:
    """Grouped attention without a softmax: a visible key weighs sigmoid(scale q.k + a learned number per head).
    Biases on all four projections; the first rot_dims channels of every q and k head rotated in neighbouring
    pairs (0: none); every value head divided by its root mean square; window None: every earlier position;
    v_mix: the layer mixes its values with those of the model's first such layer."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    v_mix: bool = False


@dataclass(frozen=True)
class LatentAttentionConfig:
    """Causal softmax attention whose keys and values are made from a latent row of kv_rank entries per token and
    one rotated key part of rot_dim entries shared by the heads; a head's query has dim plain and rot_dim rotated
    entries; a learned sink per head."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float = 10000.0


@dataclass(frozen=True)
class ChoiceExpertsConfig:
    """A routed feed-forward: `top` of experts + identity router outputs (the last `identity` of them give the input
    back) in group_count groups of which group_keep can be chosen from; gated experts of inner size ff; shared_ff:
    the inner size of a shared expert behind a sigmoid gate, or None."""
    experts: int
    top: int
    ff: int
    identity: int = 0
    group_count: int = 1
    group_keep: int = 1
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class PemuvikLayer:
    kind: str                                    # "attention" | "latent_attention"
    mixer: Any                                   # SigmoidAttentionConfig | LatentAttentionConfig
    mlp: Any                                     # None | int (a dense layer's inner size) | ChoiceExpertsConfig


@dataclass(frozen=True)
class PemuvikConfig:
    """Pemuvik: layers whose mixer and feed-forward read a norm each of the same float32 residual stream and are
    added to it through a learned vector each; the mixer is, layer by layer, a window attention with sigmoid
    weights or an attention through a shared latent; the feed-forward a dense gated layer, a mixture of gated
    experts, or absent; the head is the embedding table.  config.json gives every size and constant, layer by layer."""
    vocab: int
    width: int
    eps: float
    layers: Tuple[PemuvikLayer, ...]
    dtype: str = "bfloat16"
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Pemuvik"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "PemuvikConfig":
        where = "config.json"
        entries = d.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: key 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(entries):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at} must be an object")
            kind = entry.get("type")
            m = _section(entry, "mixer", at)
            ma = at + ".mixer"
            rot = m.get("rot")
            dims, base = 0, 10000.0
            if rot is not None:
                dims = _whole(rot, "dims", ma + ".rot")
                base = _require(rot, "base", float, ma + ".rot")
            if kind == "attention":
                mask = m.get("mask")
                mixer = SigmoidAttentionConfig(
                    heads=_whole(m, "heads", ma), kv_heads=_whole(m, "kv_heads", ma), dim=_whole(m, "dim", ma),
                    vdim=_whole(m, "vdim", ma), scale=_require(m, "scale", float, ma),
                    window=None if mask is None else _whole(mask, "size", ma + ".mask"),
                    rot_dims=dims, rot_base=base, v_mix=bool(m.get("v_mix", False)))
            elif kind == "latent_attention":
                mixer = LatentAttentionConfig(
                    heads=_whole(m, "heads", ma), dim=_whole(m, "dim", ma), rot_dim=_whole(m, "rot_dim", ma),
                    vdim=_whole(m, "vdim", ma), kv_rank=_whole(m, "kv_rank", ma), scale=_require(m, "scale", float, ma),
                    rot_base=base)
                if rot is None or dims != mixer.rot_dim:
                    raise ConfigError(f"{ma}: rot.dims must be there and equal rot_dim {mixer.rot_dim}, got {dims}")
            else:
                raise ConfigError(f"{at}: type must be 'attention' or 'latent_attention', got {kind!r}")
            mlp = entry.get("mlp")
            ff: Any = None
            if mlp is not None:
                fa = at + ".mlp"
                if not isinstance(mlp, Mapping) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"{fa} must be null or an object of kind 'dense' or 'moe', got {mlp!r}")
                if mlp["kind"] == "dense":
                    ff = _whole(mlp, "ff", fa)
                else:
                    router = _section(mlp, "router", fa)
                    groups = router.get("groups") or {}
                    shared = mlp.get("shared")
                    ff = ChoiceExpertsConfig(
                        experts=_whole(router, "experts", fa + ".router"), top=_whole(router, "top", fa + ".router"),
                        ff=_whole(_section(mlp, "expert", fa), "ff", fa + ".expert"),
                        identity=_count(router, "identity", fa + ".router", 0),
                        group_count=_whole(groups, "count", fa + ".router.groups", 1),
                        group_keep=_whole(groups, "keep", fa + ".router.groups", 1) if groups else 1,
                        shared_ff=None if shared is None else _whole(shared, "ff", fa + ".shared"))
            layers.append(PemuvikLayer(kind, mixer, ff))
        norm = _section(d, "norm", where)
        eos = d.get("eos_token_id")
        eos = (eos,) if isinstance(eos, int) else tuple(int(x) for x in eos) if isinstance(eos, (list, tuple)) else None
        cfg = cls(vocab=_whole(d, "vocab", where), width=_whole(d, "width", where),
                  eps=_require(norm, "eps", float, where + ": norm"), layers=tuple(layers),
                  dtype=canonical_dtype(d.get("dtype") or d.get("torch_dtype") or "bfloat16"),
                  eos_token_id=eos, architecture=d.get("architecture") or (d.get("architectures") or ["Pemuvik"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not (self.eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.eps}")
        mixed = None
        for i, layer in enumerate(self.layers):
            at = f"config.json: layers[{i}]"
            m, f = layer.mixer, layer.mlp
            if not (m.scale > 0):
                raise ConfigError(f"{at}: scale must be positive, got {m.scale}")
            if not (m.rot_base > 0):
                raise ConfigError(f"{at}: rot.base must be positive, got {m.rot_base}")
            if layer.kind == "attention":
                if m.heads % m.kv_heads:
                    raise ConfigError(f"{at}: {m.heads} heads do not divide into {m.kv_heads} kv_heads")
                if m.rot_dims % 2 or m.rot_dims > m.dim:
                    raise ConfigError(f"{at}: rot.dims {m.rot_dims} must be even and at most dim {m.dim}")
                if m.v_mix:
                    if mixed is not None and mixed != (m.kv_heads, m.vdim):
                        raise ConfigError(f"{at}: layers that mix values have the same kv_heads and vdim, got "
                                          f"{(m.kv_heads, m.vdim)} after {mixed}")
                    mixed = (m.kv_heads, m.vdim)
            elif m.rot_dim % 2:
                raise ConfigError(f"{at}: rot_dim {m.rot_dim} must be even")
            if isinstance(f, ChoiceExpertsConfig):
                routed = f.experts + f.identity
                if routed % f.group_count or not 1 <= f.group_keep <= f.group_count:
                    raise ConfigError(f"{at}: {routed} router outputs in {f.group_count} groups of which {f.group_keep} are kept")
                if not 1 <= f.top <= f.group_keep * (routed // f.group_count):
                    raise ConfigError(f"{at}: {f.top} experts a token out of {f.group_keep} groups of {routed // f.group_count}")

    def to_dict(self) -> dict:
        """The config.json that describes this configuration."""
        entries = []
        for layer in self.layers:
            m, f = layer.mixer, layer.mlp
            if layer.kind == "attention":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                         "v_mix": m.v_mix}
                if m.window is not None:
                    mixer["mask"] = {"size": m.window}
                if m.rot_dims:
                    mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                         "scale": m.scale, "rot": {"dims": m.rot_dim, "base": m.rot_base}}
            if f is None:
                mlp = None
            elif isinstance(f, int):
                mlp = {"kind": "dense", "ff": f}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.ff},
                       "router": {"experts": f.experts, "top": f.top, "identity": f.identity,
                                  "groups": {"count": f.group_count, "keep": f.group_keep}}}
                if f.shared_ff is not None:
                    mlp["shared"] = {"ff": f.shared_ff}
            entries.append({"type": layer.kind, "mixer": mixer, "mlp": mlp})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "layers": entries, "torch_dtype": self.dtype}
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out
