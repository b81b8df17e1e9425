"""Mixer "side_by_side": two mixers that read the same input, each output normed over the model
width and the two averaged:

    a = left(x);  b = right(x)
    out = ( a / sqrt(mean(a^2) + eps) * w_left  +  b / sqrt(mean(b^2) + eps) * w_right ) / 2

with plain weights (not one-plus) of the model width; the norms and the sum are float.  Either half
is any registered mixer.  The run's cache holds what both need: at most one of them keeps paged keys
and values and at most one keeps fixed state, each in its own place of the run's LayerCache
(spec.CombinedNeed), so that the halves are called with the same cache object.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part
from .registry import make_part, register_part
from .spec import CombinedNeed


class SideBySide(Part):
    """params: hidden_size, eps, parts {"left": PartSpec, "right": PartSpec} (mixers), names {"left":
    name, "right": name} below the mixer's own name, out_name (the name of a half's norm weight below
    the half's name)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.hidden = int(params["hidden_size"])
        self.eps = float(params["eps"])
        parts, names = params["parts"], params.get("names", {"left": "left", "right": "right"})
        self.left = make_part("mixer", parts["left"], build)
        self.right = make_part("mixer", parts["right"], build)
        self.names = (names["left"], names["right"])
        self.out_name = params.get("out_name", "out")
        self._children = {self.names[0]: self.left, self.names[1]: self.right}

    def children(self) -> Dict[str, Part]:
        return self._children

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {f"{n}.{self.out_name}.weight": ParamDecl((self.hidden,), dtype="float32", init="norm") for n in self.names}

    @property
    def replays_state_steps(self):
        return all(m.cache_need() is None or not hasattr(m.cache_need(), "tensors") or m.replays_state_steps
                   for m in (self.left, self.right))

    def cache_need(self):
        needs = tuple(n for n in (self.left.cache_need(), self.right.cache_need()) if n is not None)
        if not needs:
            return None
        return needs[0] if len(needs) == 1 else CombinedNeed(needs)

    def forward(self, x, batch, cache):
        a = self.left.forward(x, batch, cache)
        b = self.right.forward(x, batch, cache)
        w = self.weights
        return self.kernels.pair_norm_mean(a, w[f"{self.names[0]}.{self.out_name}.weight"],
                                           b, w[f"{self.names[1]}.{self.out_name}.weight"], self.eps)


register_part("mixer", "side_by_side", SideBySide)
