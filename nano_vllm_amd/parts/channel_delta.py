"""Mixer "channel_delta": the gated delta rule with a decay per key channel, over a state of fixed
size per request (a linear attention whose state forgets channel by channel and is corrected, at
every token, towards the value that its key should read out).

    q = h Wq^T, k = h Wk^T             kv_heads heads of head_dim;  v = h Wv^T: num_heads heads of v_head_dim
    q, k, v <- silu(causal convolution over the last `taps` tokens, per channel, no bias)
    q <- q / sqrt(sum(q^2) + 1e-6) * head_dim^-1/2,  k <- k / sqrt(sum(k^2) + 1e-6)         per head
    beta = sigmoid(h Wb^T)                                                one number per head
    a = exp(-exp(A_log_head) * softplus((h Wa1^T) Wa2^T + dt_bias))       per head and key channel
    per head, with its query/key head floor(head / (num_heads / kv_heads)):
        S <- diag(a) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          S [head_dim, v_head_dim]
    y = o / sqrt(mean(o^2) + eps) * w_norm * sigmoid((h Wg1^T) Wg2^T)     per head; w_norm shared by the heads
    out = y Wo^T

Per request the layer keeps S and the last taps - 1 inputs of the three convolutions in its state slot
(FixedState), both float32, zero at a request's start.  Everything after the projections (the
convolutions' sums, the unit norms, beta, the decay, the state, the read-out, the norm and the gate) is
float whatever the element type.  The ranks of the two-step projections (Wa1/Wa2, Wg1/Wg2) are the
checkpoint's: its tensors' shapes decide them unless the parameters name them.  The step's metadata is
read on the device only, so single-token steps can be captured and replayed.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part
from .spec import FixedState


class ChannelDelta(Part):
    """params: hidden_size, num_heads, num_kv_heads, head_dim, v_head_dim, conv_taps, eps, decay_rank and
    gate_rank (None: the checkpoint's tensors decide; random weights then take head_dim / 4, at least 1), and
    the names of the checkpoint tensors (q_name, k_name, v_name, b_name, a1_name, a2_name, g1_name, g2_name,
    o_name, norm_name, conv_suffix, dt_bias_name, a_log_name)."""

    replays_state_steps = True
    kernel_modules = ("delta",)

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p.get("num_kv_heads") or self.heads)
        self.dim = int(p["head_dim"])
        self.vdim = int(p.get("v_head_dim") or self.dim)
        self.taps = int(p["conv_taps"])
        self.eps = float(p.get("eps", 1e-6))
        if self.heads % self.kv_heads:
            raise ValueError(f"channel_delta: {self.heads} heads do not divide into {self.kv_heads} query/key heads")
        if self.taps < 1:
            raise ValueError("channel_delta: a convolution has at least one tap (the token's own)")
        self.decay_rank = None if p.get("decay_rank") is None else int(p["decay_rank"])
        self.gate_rank = None if p.get("gate_rank") is None else int(p["gate_rank"])
        self.names = {n: p.get(f"{n}_name", f"{n}_proj") for n in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o")}
        self.conv_suffix = p.get("conv_suffix", "conv")
        self.norm_name = p.get("norm_name", "norm")
        self.dt_bias_name = p.get("dt_bias_name", "dt_bias")
        self.a_log_name = p.get("a_log_name", "A_log")
        self.qk_channels = self.kv_heads * self.dim
        self.v_channels = self.heads * self.vdim
        self.conv_channels = 2 * self.qk_channels + self.v_channels
        self._low = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        n, qk, vv, h = self.names, self.qk_channels, self.v_channels, self.hidden
        rows = ((n["q"], 0, qk), (n["k"], qk, qk), (n["v"], 2 * qk, vv))
        fallback = max(1, self.dim // 4)
        ra, rg = self.decay_rank or -1, self.gate_rank or -1
        da, dg = self.decay_rank or fallback, self.gate_rank or fallback
        return {
            # q, k, v and beta in one product; the two narrow first steps in another (made when the weights are in)
            "proj.weight": ParamDecl((self.conv_channels + self.heads, h), sources=tuple(
                Source(f"{name}.weight", r, c) for name, r, c in rows + ((n["b"], self.conv_channels, self.heads),))),
            "conv.weight": ParamDecl((self.conv_channels, self.taps), sources=tuple(
                Source(f"{name}.{self.conv_suffix}.weight", r, c) for name, r, c in rows)),
            f"{n['a1']}.weight": ParamDecl((ra, h), default_shape=(da, h)),
            f"{n['a2']}.weight": ParamDecl((self.heads * self.dim, ra), default_shape=(self.heads * self.dim, da)),
            f"{n['g1']}.weight": ParamDecl((rg, h), default_shape=(dg, h)),
            f"{n['g2']}.weight": ParamDecl((vv, rg), default_shape=(vv, dg)),
            self.dt_bias_name: ParamDecl((self.heads * self.dim,), dtype="float32"),
            self.a_log_name: ParamDecl((self.heads,), dtype="float32"),
            f"{self.norm_name}.weight": ParamDecl((self.vdim,), dtype="float32", init="norm"),
            f"{n['o']}.weight": ParamDecl((h, vv)),
        }

    def on_weights_loaded(self) -> None:
        w, n = self.weights, self.names
        a1, a2, g1, g2 = (w[f"{n[x]}.weight"] for x in ("a1", "a2", "g1", "g2"))
        if a1.shape[0] != a2.shape[1] or g1.shape[0] != g2.shape[1]:
            raise ValueError(f"channel_delta: the two steps of a narrow projection differ in rank "
                             f"({tuple(a1.shape)} and {tuple(a2.shape)}, {tuple(g1.shape)} and {tuple(g2.shape)})")
        self._low = torch.cat((a1, g1), dim=0).contiguous()

    def cache_need(self):
        return FixedState({"conv": ((self.conv_channels, self.taps - 1), "float32"),
                           "s": ((self.heads, self.dim, self.vdim), "float32")})

    def forward(self, x, batch, cache):
        k, w, n = self.kernels, self.weights, self.names
        proj = k.linear(x, w["proj.weight"])
        low = k.linear(x, self._low)
        ra = w[f"{n['a1']}.weight"].shape[0]
        decay_in = k.linear(low[:, :ra], w[f"{n['a2']}.weight"], out_float32=True)
        gate_in = k.linear(low[:, ra:], w[f"{n['g2']}.weight"])
        y = k.channel_delta(proj, decay_in, gate_in, self.heads, self.kv_heads, self.dim, self.vdim, self.taps,
                            w["conv.weight"], w[self.dt_bias_name], w[self.a_log_name], w[f"{self.norm_name}.weight"],
                            self.eps, cache.state["conv"], cache.state["s"], batch)
        return k.linear(y, w[f"{n['o']}.weight"], deferred=True)


register_part("mixer", "channel_delta", ChannelDelta)
