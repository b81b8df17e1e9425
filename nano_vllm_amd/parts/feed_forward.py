"""Feed-forward parts.

"swiglu": m = (silu(y Wg^T) * (y Wu^T)) Wd^T with gate and up packed into one matrix
[2*inner, hidden], gate rows first (nanovllm/models/qwen3.py:91-117, linear.py:87-93,
activation.py:8-11).  Dense: no experts, no routing.  The parameter `activation` puts relu or
the tanh form of gelu in silu's place (the same gated layout).
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part


class SwiGLU(Part):
    """params: hidden_size, intermediate_size; optional activation (silu, relu, gelu_tanh) and names
    of the checkpoint tensors."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.hidden = int(params["hidden_size"])
        self.inner = int(params["intermediate_size"])
        self.gate_name = params.get("gate_name", "gate_proj")
        self.up_name = params.get("up_name", "up_proj")
        self.down_name = params.get("down_name", "down_proj")
        self.activation = params.get("activation", "silu")
        if self.activation not in ("silu", "relu", "gelu_tanh"):
            raise ValueError(f"swiglu: unknown activation {self.activation!r}")

    def param_decls(self) -> Dict[str, ParamDecl]:
        i, h = self.inner, self.hidden
        return {
            "gate_up_proj.weight": ParamDecl((2 * i, h), sources=(
                Source(f"{self.gate_name}.weight", 0, i), Source(f"{self.up_name}.weight", i, i))),
            f"{self.down_name}.weight": ParamDecl((h, i)),
        }

    def forward(self, x, batch=None):
        if self.activation == "silu":
            z = self.kernels.linear_silu_mul(x, self.weights["gate_up_proj.weight"])
        else:
            z = self.kernels.linear_act_mul(x, self.weights["gate_up_proj.weight"], self.activation)
        # deferred: the block hands this to the next norm only
        return self.kernels.linear(z, self.weights[f"{self.down_name}.weight"], deferred=True)


register_part("feed_forward", "swiglu", SwiGLU)
