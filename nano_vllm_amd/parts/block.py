"""Blocks: the arrangement of a layer's parts.

"pre_norm_residual": the pre-norm residual layer with the residual sum deferred into the
next norm (nanovllm/models/qwen3.py:146-159):
    first layer:  r = h;           x = norm1(h)
    later layers: r = h + r;       x = norm1(r)
    a = mixer(x);  r = a + r;  y = norm2(r);  m = feed_forward(y);  returns (m, r)
The caller adds the last m to r inside the final norm (qwen3.py:182).
With the parameter stream = "float32" the residual stream r is kept in float32 whatever the element
type: every sublayer's output travels as a list of one addend, which the next norm adds to the stream
(the norms of such a block take lists: rms_norm and dynamic_tanh do), and the layer may have no
feed-forward (then it has no second norm either).

"parallel_residual": one norm whose output both sublayers read, their sum added to the stream:
    x = norm(r);  r <- r + (mixer(x) + feed_forward(x))
The residual stream r is float32 whatever the element type.  The sum is deferred into the next
norm as well: the block returns the two sublayer outputs as a list of addends with the stream as
it was before them, and the next block's norm (or the model's final norm) adds them.  The first
block gets the embedding as its one addend.  A layer may have no feed-forward.
With a part in the role "feed_forward_norm" the feed-forward reads a norm of its own of the same stream
(x = norm(r), y = feed_forward_norm(r), both made in one pass over r), and with layer_scale = True the
two outputs are multiplied, channel by channel, by learned vectors of the block's own before they are added:
    r <- r + (s1 * mixer(x) + s2 * feed_forward(y))
(the vectors' names in the checkpoint: mixer_scale_name, feed_forward_scale_name).

"sandwich_residual": a norm before and a norm after every sublayer, the normed output times a
constant added to the stream:
    r <- r + c * post1(mixer(pre1(r)));   r <- r + c * post2(feed_forward(pre2(r)))
The residual stream r is float32 whatever the element type.  The sum is deferred here too: a
sublayer's output leaves the block as a NormedAddend (the output, the post-norm's weight and eps,
the constant c), and the norm that follows norms it, adds it to the stream and norms the stream in
one pass.  The first block gets the float32 stream itself from the embedding (an embedding with a
scale gives one).  A layer may have no feed-forward.

Interface of a block: forward(h, residual | None, batch, cache) -> (h, residual); h is a tensor,
or a list of addends for a float32 stream.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import BuildContext, NormedAddend, ParamDecl, Part, ScaledAddend
from .registry import make_part, register_part


class PreNormResidualBlock(Part):
    ROLES = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        parts = params["parts"]            # role -> PartSpec
        names = params["names"]            # role -> name in checkpoint tensor names
        stream = params.get("stream")
        if stream not in (None, "float32"):
            raise ValueError(f"pre_norm_residual block: stream must be 'float32' or absent, got {stream!r}")
        self.float_stream = stream == "float32"
        optional = ("feed_forward_norm", "feed_forward") if self.float_stream and not parts.get("feed_forward") else ()
        missing = [r for r in self.ROLES if r not in parts and r not in optional]
        if missing:
            raise ValueError(f"pre_norm_residual block: missing parts {missing}")
        self.mixer_norm = make_part("norm", parts["mixer_norm"], build)
        self.mixer = make_part("mixer", parts["mixer"], build)
        self.feed_forward_norm = self.feed_forward = None
        if parts.get("feed_forward"):
            self.feed_forward_norm = make_part("norm", parts["feed_forward_norm"], build)
            self.feed_forward = make_part("feed_forward", parts["feed_forward"], build)
        self._children = {names[r]: getattr(self, r) for r in self.ROLES if getattr(self, r) is not None}

    def children(self) -> Dict[str, Part]:
        return self._children

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def replays_state_steps(self):
        return self.mixer.replays_state_steps

    def forward(self, h, residual, batch, cache):
        if self.float_stream:
            addends = tuple(h) if isinstance(h, (tuple, list)) else (h,)
            x, residual = self.mixer_norm.forward_add(addends, residual)
            a = self.mixer.forward(x, batch, cache)
            if self.feed_forward is None:
                return (a,), residual
            y, residual = self.feed_forward_norm.forward_add((a,), residual)
            return (self.feed_forward.forward(y, batch),), residual
        if residual is None:
            x, residual = self.mixer_norm.forward(h), h
        else:
            x, residual = self.mixer_norm.forward_add(h, residual)
        a = self.mixer.forward(x, batch, cache)
        y, residual = self.feed_forward_norm.forward_add(a, residual)
        m = self.feed_forward.forward(y, batch)
        return m, residual


class ParallelResidualBlock(Part):
    """params: layer_scale (bool), mixer_scale_name, feed_forward_scale_name; parts and names by role: norm, mixer,
    and optionally feed_forward and feed_forward_norm."""
    ROLES = ("norm", "mixer", "feed_forward_norm", "feed_forward")

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        parts = params["parts"]
        names = params["names"]
        missing = [r for r in ("norm", "mixer") if r not in parts]
        if missing:
            raise ValueError(f"parallel_residual block: missing parts {missing}")
        self.norm = make_part("norm", parts["norm"], build)
        self.mixer = make_part("mixer", parts["mixer"], build)
        self.feed_forward = make_part("feed_forward", parts["feed_forward"], build) if parts.get("feed_forward") else None
        self.feed_forward_norm = None
        if parts.get("feed_forward_norm"):
            if self.feed_forward is None:
                raise ValueError("parallel_residual block: a feed-forward norm without a feed-forward")
            self.feed_forward_norm = make_part("norm", parts["feed_forward_norm"], build)
            if getattr(self.feed_forward_norm, "offset", 0.0) or getattr(self.norm, "offset", 0.0) or \
                    self.feed_forward_norm.eps != self.norm.eps:
                raise ValueError("parallel_residual block: two norms of one stream share their eps and have plain weights")
        self.layer_scale = bool(params.get("layer_scale", False))
        self.mixer_scale_name = params.get("mixer_scale_name", "mixer_scale")
        self.feed_forward_scale_name = params.get("feed_forward_scale_name", "feed_forward_scale")
        self.width = build.hidden_size
        self.dtype = build.dtype
        self._children = {names[r]: getattr(self, r) for r in self.ROLES if getattr(self, r) is not None}

    def children(self) -> Dict[str, Part]:
        return self._children

    def param_decls(self):
        if not self.layer_scale:
            return {}
        d = {self.mixer_scale_name: ParamDecl((self.width,), dtype="stored32", init="norm")}
        if self.feed_forward is not None:
            d[self.feed_forward_scale_name] = ParamDecl((self.width,), dtype="stored32", init="norm")
        return d

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def replays_state_steps(self):
        return self.mixer.replays_state_steps

    def _out(self, x, scale_name):
        return ScaledAddend(x, self.weights[scale_name]) if self.layer_scale else x

    def forward(self, h, residual, batch, cache):
        addends = h if isinstance(h, (tuple, list)) else (h,)
        if self.feed_forward_norm is not None:
            x, y, residual = self.kernels.stream_scaled_norm(
                [(a.x, a.scale) if hasattr(a, "scale") else (a, None) for a in addends], residual,
                self.norm.weights["weight"], self.norm.eps, weight2=self.feed_forward_norm.weights["weight"],
                dtype=self.dtype)
        else:
            x, residual = self.norm.forward_add(addends, residual)
            y = x
        a = self._out(self.mixer.forward(x, batch, cache), self.mixer_scale_name)
        if self.feed_forward is None:
            return (a,), residual
        return (a, self._out(self.feed_forward.forward(y, batch), self.feed_forward_scale_name)), residual


class SandwichResidualBlock(Part):
    """params: residual_mult (default 1), parts and names by role: mixer_norm, mixer, mixer_post_norm, and,
    where the layer has a feed-forward, feed_forward_norm, feed_forward, feed_forward_post_norm."""
    ROLES = ("mixer_norm", "mixer", "mixer_post_norm", "feed_forward_norm", "feed_forward", "feed_forward_post_norm")

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        parts = params["parts"]
        names = params["names"]
        self.mult = float(params.get("residual_mult", 1.0))
        self.dtype = build.dtype
        has_ff = bool(parts.get("feed_forward"))
        missing = [r for r in self.ROLES if r not in parts and (has_ff or not r.startswith("feed_forward"))]
        if missing:
            raise ValueError(f"sandwich_residual block: missing parts {missing}")
        self.mixer_norm = make_part("norm", parts["mixer_norm"], build)
        self.mixer = make_part("mixer", parts["mixer"], build)
        self.mixer_post_norm = make_part("norm", parts["mixer_post_norm"], build)
        self.feed_forward_norm = self.feed_forward = self.feed_forward_post_norm = None
        if has_ff:
            self.feed_forward_norm = make_part("norm", parts["feed_forward_norm"], build)
            self.feed_forward = make_part("feed_forward", parts["feed_forward"], build)
            self.feed_forward_post_norm = make_part("norm", parts["feed_forward_post_norm"], build)
        self._children = {names[r]: getattr(self, r) for r in self.ROLES if getattr(self, r) is not None}

    def children(self) -> Dict[str, Part]:
        return self._children

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def replays_state_steps(self):
        return self.mixer.replays_state_steps

    def _through(self, post_norm, x) -> NormedAddend:
        return NormedAddend(x, post_norm.weights["weight"], post_norm.eps, self.mult)

    def forward(self, h, residual, batch, cache):
        if residual is None:
            # the first layer: h is the stream itself, float32, as the embedding made it
            if not torch.is_tensor(h) or h.dtype != torch.float32:
                raise ValueError("sandwich_residual block: the first layer takes the float32 stream from the embedding")
            out = torch.empty(h.shape, dtype=self.dtype, device=h.device)
            x, residual = self.mixer_norm.forward_add((), h, out=out)
        else:
            x, residual = self.mixer_norm.forward_add(tuple(h), residual)
        a = self._through(self.mixer_post_norm, self.mixer.forward(x, batch, cache))
        if self.feed_forward is None:
            return (a,), residual
        y, residual = self.feed_forward_norm.forward_add((a,), residual)
        return (self._through(self.feed_forward_post_norm, self.feed_forward.forward(y, batch)),), residual


register_part("block", "sandwich_residual", SandwichResidualBlock)
register_part("block", "pre_norm_residual", PreNormResidualBlock)
register_part("block", "parallel_residual", ParallelResidualBlock)
