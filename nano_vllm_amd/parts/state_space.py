"""Mixer "state_space": a selective state-space layer with a scalar decay per head and token
(the dual form of such layers is a linear attention whose decay depends on the input).

    [z | x | B | C | dt] = h W_in^T        z, x: heads * vdim; B, C: groups * state; dt: heads
    x, B, C <- silu(causal convolution over the last `taps` tokens, per channel, with a bias)
    dt <- softplus(dt + dt_bias)                                     per head, no clamp
    S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T               per head, S [state, vdim] float32
    y_t = S_t^T C_t + D_h x_t                                        head h reads group floor(h / (heads / groups))
    y <- y * silu(z), then RMS norm in norm_groups equal parts of the heads * vdim channels, times a weight
    out = y W_o^T

Per request the layer keeps S and the last taps - 1 inputs of the convolution in its state slot
(FixedState), both float32, zero at a request's start.  Everything after the projection and the
convolution (step sizes, decays, state, sums, gate and norm) is float whatever the element type.
The step's metadata is read on the device only, so single-token steps can be captured and replayed.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part
from .registry import register_part
from .spec import FixedState


class StateSpace(Part):
    """params: hidden_size, num_heads, v_head_dim, state_size, groups, conv_taps, norm_groups, eps, and
    the names of the checkpoint tensors (in_name, conv_name, norm_name, o_name, dt_bias_name, a_log_name,
    d_name)."""

    replays_state_steps = True
    kernel_modules = ("ssd",)

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.vdim = int(p["v_head_dim"])
        self.state = int(p["state_size"])
        self.groups = int(p.get("groups", 1))
        self.taps = int(p["conv_taps"])
        self.norm_groups = int(p.get("norm_groups", 1))
        self.eps = float(p.get("eps", 1e-6))
        if self.heads % self.groups:
            raise ValueError(f"state_space: {self.heads} heads do not divide into {self.groups} groups")
        self.inner = self.heads * self.vdim
        if self.inner % self.norm_groups:
            raise ValueError(f"state_space: {self.inner} channels do not divide into {self.norm_groups} norm groups")
        if self.taps < 1:
            raise ValueError("state_space: the convolution has at least one tap (the token's own)")
        self.conv_channels = self.inner + 2 * self.groups * self.state
        self.in_name = p.get("in_name", "in_proj")
        self.conv_name = p.get("conv_name", "conv1d")
        self.norm_name = p.get("norm_name", "norm")
        self.o_name = p.get("o_name", "out_proj")
        self.dt_bias_name = p.get("dt_bias_name", "dt_bias")
        self.a_log_name = p.get("a_log_name", "A_log")
        self.d_name = p.get("d_name", "D")

    def param_decls(self) -> Dict[str, ParamDecl]:
        rows = 2 * self.inner + 2 * self.groups * self.state + self.heads
        return {
            f"{self.in_name}.weight": ParamDecl((rows, self.hidden)),
            f"{self.conv_name}.weight": ParamDecl((self.conv_channels, self.taps)),
            f"{self.conv_name}.bias": ParamDecl((self.conv_channels,)),
            self.dt_bias_name: ParamDecl((self.heads,), dtype="float32"),
            self.a_log_name: ParamDecl((self.heads,), dtype="float32"),
            self.d_name: ParamDecl((self.heads,), dtype="float32", init="norm"),
            f"{self.norm_name}.weight": ParamDecl((self.inner,), dtype="float32", init="norm"),
            f"{self.o_name}.weight": ParamDecl((self.hidden, self.inner)),
        }

    def cache_need(self):
        return FixedState({"conv": ((self.conv_channels, self.taps - 1), "float32"),
                           "ssm": ((self.heads, self.state, self.vdim), "float32")})

    def forward(self, x, batch, cache):
        k, w = self.kernels, self.weights
        proj = k.linear(x, w[f"{self.in_name}.weight"])
        y = k.state_space(proj, self.heads, self.vdim, self.state, self.groups, self.taps,
                          w[f"{self.conv_name}.weight"], w[f"{self.conv_name}.bias"], w[self.dt_bias_name],
                          w[self.a_log_name], w[self.d_name], w[f"{self.norm_name}.weight"], self.norm_groups, self.eps,
                          cache.state["conv"], cache.state["ssm"], batch)
        return k.linear(y, w[f"{self.o_name}.weight"], deferred=True)


register_part("mixer", "state_space", StateSpace)
