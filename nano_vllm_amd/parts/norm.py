"""Norm parts.

"rms_norm": y = cast(x * rsqrt(mean(x^2) + eps)) * weight, and the same fused with the
residual sum (nanovllm/layers/layernorm.py:16-40).  Sizes and eps are parameters.

With weight_offset c the factor is (c + weight): c = 1 is the weight stored around zero.  A norm
with an offset, and every norm that is handed a list of addends instead of one tensor, works on a
residual stream kept in float32: the stream takes the sum of the addends, the norm is computed in
float and rounded once to the element type.  An addend may be a NormedAddend (parts.base): a sublayer's
output that enters the stream through a norm of its own and a constant factor; the same pass does both norms.
Or a ScaledAddend: an output that is multiplied, channel by channel, by a learned vector on its way into the stream.

"dynamic_tanh": y = tanh(alpha * x) * weight + bias with one learned number alpha per norm: no mean,
no variance, every entry by itself.  It works on a float32 residual stream (a list of addends, as
above); tanh, products and sums in float, rounded once.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part
from .registry import register_part


class RMSNorm(Part):
    """params: dim, eps, weight_offset (default 0)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        self.offset = float(params.get("weight_offset", 0.0))

    def param_decls(self) -> Dict[str, ParamDecl]:
        # vectors stay in float32 when the checkpoint stores them so
        # (a weight that is stored around zero is drawn around zero in random-weights mode)
        return {"weight": ParamDecl((self.dim,), dtype="stored32", init="norm" if self.offset == 0.0 else "normal")}

    def forward(self, x, out=None):
        if self.offset != 0.0:
            return self.kernels.stream_rms_norm((x,), None, self.weights["weight"], self.eps, self.offset, out=out)[0]
        return self.kernels.rms_norm(x, self.weights["weight"], self.eps, out=out)

    def forward_add(self, x, residual, out=None):
        """residual <- x + residual; returns (norm(residual), residual).  x may be a list of one or
        two addends: the residual is then a float32 stream (None: it starts as their sum)."""
        if isinstance(x, (tuple, list)):
            if any(hasattr(a, "scale") for a in x):
                if self.offset != 0.0:
                    raise ValueError("rms_norm: scaled addends go with a plain weight")
                y, _, residual = self.kernels.stream_scaled_norm(
                    [(a.x, a.scale) if hasattr(a, "scale") else (a, None) for a in x], residual, self.weights["weight"],
                    self.eps, out=out)
                return y, residual
            return self.kernels.stream_rms_norm(tuple(x), residual, self.weights["weight"], self.eps, self.offset, out=out)
        if self.offset != 0.0:
            raise ValueError("rms_norm: a weight offset goes with a float32 residual stream (a list of addends)")
        return self.kernels.add_rms_norm(x, residual, self.weights["weight"], self.eps, out=out)


class DynamicTanh(Part):
    """params: dim; optional names of the checkpoint tensors below the norm's own (bias_name, alpha_name)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.dim = int(params["dim"])
        self.bias_name = params.get("bias_name", "bias")
        self.alpha_name = params.get("alpha_name", "alpha")

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.dim,), dtype="float32", init="norm"),
                self.bias_name: ParamDecl((self.dim,), dtype="float32"),
                self.alpha_name: ParamDecl((), dtype="float32", init="norm")}

    def forward(self, x, out=None):
        return self.forward_add((x,), None, out=out)[0]

    def forward_add(self, x, residual, out=None):
        """residual <- residual + sum of the addends x (None: the stream starts as their sum);
        returns (tanh(alpha * residual) * weight + bias, residual)."""
        addends = tuple(x) if isinstance(x, (tuple, list)) else (x,)
        w = self.weights
        return self.kernels.stream_dyt(addends, residual, w["weight"], w[self.bias_name], w[self.alpha_name], out=out)


register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "dynamic_tanh", DynamicTanh)
