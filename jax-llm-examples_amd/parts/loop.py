"""What happens to the residual stream where a stretch of layers is run several times in a row with the same
weights (every pass with caches and state of its own: the plan's order names the layers once per pass).

``pass_entry``: before the first layer of pass ``t`` the stream becomes ``x + x_0 + step[t]`` for ``t > 0`` and
``x + step[0]`` for the first pass, ``x_0`` being the embedding's output and ``step`` a learned vector per pass.
The part only says so: the sum is made by the kernel that forms the next norm's rows.
"""
from __future__ import annotations

from .base import ParamSpec, Part

_LOOPS = {}


def register_loop(kind: str):
    def deco(cls):
        _LOOPS[kind] = cls
        return cls

    return deco


def build_loop(spec):
    try:
        return _LOOPS[spec.kind](spec)
    except KeyError:
        raise KeyError(f"unknown loop kind {spec.kind!r}; registered: {sorted(_LOOPS)}") from None


@register_loop("pass_entry")
class PassEntry(Part):
    graph_safe = True

    @property
    def needs_embedding_output(self) -> bool:
        """Whether the model has to keep a copy of the embedding's output for it (a single pass adds none)."""
        return self.times > 1

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden, self.times = int(spec.hidden_size), int(spec.times)

    def param_specs(self):
        return {"step": ParamSpec((self.times, self.hidden), policy="float32", init=("normal", 0.3))}

    def flops_per_token(self) -> float:
        return 0.0

    def enter(self, residual, embedded, number: int, ctx) -> None:
        """Pass ``number`` begins: what is to be added stays pending on the residual."""
        if not 0 <= number < self.times:
            raise ValueError(f"pass {number} of a loop of {self.times}")
        residual.inject(embedded if number > 0 else None, self.params["step"][number])
