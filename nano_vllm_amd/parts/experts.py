"""Feed-forward parts without a gate, and a mixture of them.

"mlp": m = act(y Wu^T) Wd^T, act one of relu2 (the square of relu), relu, silu, gelu_tanh.

"moe": every token runs `top` of `experts` such layers (no biases) and, optionally, a shared one:
    s = sigmoid(y Wr^T)                       router scores, float
    experts form group_count equal groups of neighbours; a group's score is the sum of its two largest
    scores (of its one score where groups hold one expert); only experts of the group_keep best groups
    can be chosen; of those the `top` with the largest scores are
    m = sum over the chosen e of (scale * s_e) expert_e(y)  +  shared(y)
The weights are the scores themselves, not renormalised.
With routing "softmax_top" the router's logits (plus a bias, with router_bias) are compared as they are: the
`top` largest are chosen and weighted by the softmax over the chosen logits alone (no groups, no scale).
With routing "softmax_choice" s = softmax(y Wr^T) over all experts; an expert is chosen by s_e + c_e with a learned
correction c (a float per expert); a group counts by the largest such choice score in it and only the group_keep best
groups' experts can be chosen; the weights are the chosen experts' s (without the correction) over their sum (+ 1e-20).
With identity = n the router has n more outputs after the experts', which take part in the softmax, the groups and the
choice like experts; they have no tensors, and the output of one that is chosen is y itself.
With shared_gate = True the shared layer's output is multiplied by sigmoid(wg . y), one number per token.
With gated = True an expert is the gated layer  Wd (act(Wg y) * (Wu y)).
Routing is decided on the device and the
experts' products run over the tokens sorted by expert, so a step never asks the host how many
tokens an expert got: the same launches whatever the routing.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part, Source
from .registry import make_part, register_part

ACTIVATIONS = ("relu2", "relu", "silu", "gelu_tanh")


class PlainMLP(Part):
    """params: hidden_size, intermediate_size, activation (default relu2), up_name, down_name."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.hidden = int(params["hidden_size"])
        self.inner = int(params["intermediate_size"])
        self.up_name = params.get("up_name", "up_proj")
        self.down_name = params.get("down_name", "down_proj")
        self.activation = params.get("activation", "relu2")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"mlp: unknown activation {self.activation!r}")

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {f"{self.up_name}.weight": ParamDecl((self.inner, self.hidden)),
                f"{self.down_name}.weight": ParamDecl((self.hidden, self.inner))}

    def forward(self, x, batch=None):
        z = self.kernels.act(self.kernels.linear(x, self.weights[f"{self.up_name}.weight"]), self.activation)
        return self.kernels.linear(z, self.weights[f"{self.down_name}.weight"], deferred=True)


class MixtureOfExperts(Part):
    """params: hidden_size, num_experts, top, intermediate_size, scale, group_count, group_keep,
    activation, shared (a PartSpec of a feed-forward, or None), routing ("sigmoid_groups" | "softmax_top" |
    "softmax_choice"), router_bias (bool), gated (bool), identity (router outputs without an expert), shared_gate (bool),
    and names: correction_name, shared_gate_name (below the shared layer's), router_name, shared_name, expert_name (a format with {} for
    the expert's number), gate_name, up_name, down_name."""

    kernel_modules = ("moe",)

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.experts = int(p["num_experts"])
        self.top = int(p["top"])
        self.inner = int(p["intermediate_size"])
        self.scale = float(p.get("scale", 1.0))
        self.group_count = int(p.get("group_count", 1))
        self.group_keep = int(p.get("group_keep", self.group_count))
        self.activation = p.get("activation", "relu2")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"moe: unknown activation {self.activation!r}")
        self.routing = p.get("routing", "sigmoid_groups")
        if self.routing not in ("sigmoid_groups", "softmax_top", "softmax_choice"):
            raise ValueError(f"moe: unknown routing {self.routing!r}")
        self.router_bias = bool(p.get("router_bias", False))
        self.gated = bool(p.get("gated", False))
        self.gate_name = p.get("gate_name", "gate_proj")
        self.identity = int(p.get("identity", 0))
        self.shared_gate = bool(p.get("shared_gate", False))
        if self.identity < 0 or (self.identity and self.routing != "softmax_choice"):
            raise ValueError("moe: identity outputs go with the routing 'softmax_choice'")
        if self.shared_gate and not p.get("shared"):
            raise ValueError("moe: a gate on the shared layer without a shared layer")
        self.routed = self.experts + self.identity       # the router's outputs
        if self.routed % self.group_count or not 1 <= self.group_keep <= self.group_count:
            raise ValueError(f"moe: {self.routed} experts in {self.group_count} groups of which {self.group_keep} are kept")
        if not 1 <= self.top <= self.group_keep * (self.routed // self.group_count):
            raise ValueError(f"moe: {self.top} experts a token out of {self.group_keep} groups of "
                             f"{self.routed // self.group_count}")
        self.correction_name = p.get("correction_name", "correction")
        self.shared_gate_name = p.get("shared_gate_name", "gate")
        self.router_name = p.get("router_name", "router")
        self.shared_name = p.get("shared_name", "shared")
        self.expert_name = p.get("expert_name", "experts.{}")
        self.up_name, self.down_name = p.get("up_name", "up_proj"), p.get("down_name", "down_proj")
        self.shared = make_part("feed_forward", p["shared"], build) if p.get("shared") else None

    def children(self) -> Dict[str, Part]:
        return {self.shared_name: self.shared} if self.shared is not None else {}

    def param_decls(self) -> Dict[str, ParamDecl]:
        e, i, h = self.experts, self.inner, self.hidden
        name = self.expert_name.format
        if self.gated:
            # an expert's gate rows, then its up rows: the first product makes both and gates in its epilogue
            up = tuple(s for n in range(e) for s in (Source(f"{name(n)}.{self.gate_name}.weight", 2 * n * i, i),
                                                     Source(f"{name(n)}.{self.up_name}.weight", (2 * n + 1) * i, i)))
        else:
            up = tuple(Source(f"{name(n)}.{self.up_name}.weight", n * i, i) for n in range(e))
        router = (Source(f"{self.router_name}.weight", 0, self.routed),)
        if self.shared_gate:
            # the gate's one row lies below the router's: one product makes the logits and the gate's
            router += (Source(f"{self.shared_name}.{self.shared_gate_name}.weight", self.routed, 1),)
        decls = {
            f"{self.router_name}.weight": ParamDecl((self.routed + (1 if self.shared_gate else 0), h), sources=router),
            # the experts' matrices one below the other: expert n's rows are [n * rows, (n + 1) * rows)
            "up.weight": ParamDecl(((2 if self.gated else 1) * e * i, h), sources=up),
            "down.weight": ParamDecl((e * h, i), sources=tuple(
                Source(f"{name(n)}.{self.down_name}.weight", n * h, h) for n in range(e))),
        }
        if self.router_bias:
            decls[f"{self.router_name}.bias"] = ParamDecl((e,), dtype="float32")
        if self.routing == "softmax_choice":
            decls["correction"] = ParamDecl((self.routed,), dtype="float32", sources=(Source(self.correction_name, 0, self.routed),))
        return decls

    def forward(self, x, batch=None):
        k, w = self.kernels, self.weights
        logits = k.linear(x, w[f"{self.router_name}.weight"], out_float32=True)
        gate = None
        if self.shared_gate:
            gate, logits = logits[:, self.routed], logits[:, :self.routed]
        if self.routing == "softmax_choice":
            ids, weights = k.moe_route(logits, self.top, self.group_count, self.group_keep, 1.0, routing="softmax_choice",
                                       bias=w["correction"])
        elif self.routing == "softmax_top":
            ids, weights = k.moe_route(logits, self.top, 1, 1, 1.0, routing="softmax_top",
                                       bias=w.get(f"{self.router_name}.bias"))
        else:
            ids, weights = k.moe_route(logits, self.top, self.group_count, self.group_keep, self.scale)
        shared = self.shared.forward(x, batch) if self.shared is not None else None
        if gate is not None:
            return k.moe_experts(x, ids, weights, w["up.weight"], w["down.weight"], self.experts, self.activation,
                                 add=shared, gated=self.gated, add_gate=gate)
        if self.gated:
            return k.moe_experts(x, ids, weights, w["up.weight"], w["down.weight"], self.experts, self.activation,
                                 add=shared, gated=True)
        return k.moe_experts(x, ids, weights, w["up.weight"], w["down.weight"], self.experts, self.activation, add=shared)


register_part("feed_forward", "mlp", PlainMLP)
register_part("feed_forward", "moe", MixtureOfExperts)
