"""RMS norm (``llama4/llama4_jax/model.py:885-888``): ``x / sqrt(mean(x^2) + eps) * weight``,
statistics in float32, eps inside the root, the weight used as it is (not ``1 + weight``).  With the option
``unit_offset`` the checkpoint stores the weight as its distance from one: the part adds the one when the weights
are in place (in float32, as a kernel that formed ``1 + weight`` would), and the kernels see a plain weight."""
from __future__ import annotations

from .base import Norm, ParamSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, spec) -> None:
        super().__init__()
        self.eps = float(spec.eps)
        self.weighted = bool(spec.get("weighted", True))
        self.size = spec.get("size")
        self.unit_offset = bool(spec.get("unit_offset", False))
        self._offset_added = False

    graph_safe = True

    def param_specs(self):
        if not self.weighted:
            return {}
        init = ("normal", 0.1) if self.unit_offset else ("ones",)
        return {"weight": ParamSpec((int(self.size),), policy="float32", init=init)}

    def finalize(self) -> None:
        if self.unit_offset and self.weighted and not self._offset_added:
            self.params["weight"].add_(1.0)
            self._offset_added = True

    def forward(self, residual, ctx, want32: bool = False, defer: bool = False):
        return residual.normed(ctx, self.params.get("weight"), self.eps, want32, defer)
