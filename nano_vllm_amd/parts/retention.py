"""Mixer "retention": linear attention with a fixed decay per head, no softmax and no denominator,
over a state of fixed size per request.

    [q | k | v | g] = x W^T                  heads of dim (q, k) and of v_head_dim (v, g)
    q, k <- rotation of the first rotary_dim channels of a head, pairs (i, i + rotary_dim/2), by the
            angle p * theta^(-2i/rotary_dim) at position p (rotary_dim 0: none)
    k    <- k * head_dim^(-1/2)              (parameter k_scale)
    S_t  = decay_h S_(t-1) + k_t v_t^T       per head, S [head_dim, v_head_dim] float32, zero at the start
    o_t  = S_t^T q_t
    y    = o / sqrt(mean(o^2) + eps) * silu(g)          per head, no weight
    out  = y Wo^T

The state lives in the request's state slot (FixedState) and is carried from step to step; a step
may bring one token or a portion of a prompt, which the kernel takes in chunks.  Rotation, scores,
decay powers, state and sums are float32 whatever the element type.  The step's metadata is read on
the device only, so single-token steps can be captured and replayed.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part
from .spec import FixedState


class Retention(Part):
    """params: hidden_size, num_heads, head_dim, v_head_dim, decay (one per head), eps, rotary_dim
    (0: no rotation), theta, k_scale (None: head_dim^-0.5), and the names of the checkpoint tensors
    (q_name, k_name, v_name, g_name, o_name)."""

    replays_state_steps = True
    kernel_modules = ("retention",)

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.v_head_dim = int(p.get("v_head_dim") or self.head_dim)
        self.decay = tuple(float(x) for x in p["decay"])
        if len(self.decay) != self.heads:
            raise ValueError(f"retention: {len(self.decay)} decays for {self.heads} heads")
        self.eps = float(p.get("eps", 1e-6))
        self.rotary_dim = int(p.get("rotary_dim") or 0)
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"retention: {self.rotary_dim} rotated channels of a head of {self.head_dim}: the number "
                             f"must be even and at most the head's")
        self.theta = float(p.get("theta", 10000.0))
        k_scale = p.get("k_scale")
        self.k_scale = float(k_scale) if k_scale is not None else self.head_dim ** -0.5
        self.names = tuple(p.get(f"{n}_name", f"{n}_proj") for n in ("q", "k", "v", "g"))
        self.o_name = p.get("o_name", "o_proj")
        self._device = build.device
        self._tables = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        qk, vv = self.heads * self.head_dim, self.heads * self.v_head_dim
        rows = (0, qk, 2 * qk, 2 * qk + vv)
        sizes = (qk, qk, vv, vv)
        return {
            "proj.weight": ParamDecl((2 * qk + 2 * vv, self.hidden), sources=tuple(
                Source(f"{n}.weight", r, c) for n, r, c in zip(self.names, rows, sizes))),
            f"{self.o_name}.weight": ParamDecl((self.hidden, vv)),
        }

    def cache_need(self):
        return FixedState({"s": ((self.heads, self.head_dim, self.v_head_dim), "float32")})

    def _constants(self):
        """The powers decay_h^m for m up to the kernel's chunk, and the rotation's frequencies, both
        worked out in double and rounded once (made on first use: building a part touches no device)."""
        if self._tables is None:
            chunk = int(self.kernels.RETENTION_CHUNK)
            powers = torch.tensor(self.decay, dtype=torch.float64)[:, None] ** torch.arange(chunk + 1, dtype=torch.float64)[None, :]
            inv_freq = None
            if self.rotary_dim:
                i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
                inv_freq = (self.theta ** (-2.0 * i / self.rotary_dim)).to(torch.float32).to(self._device)
            self._tables = (powers.to(torch.float32).contiguous().to(self._device), inv_freq)
        return self._tables

    def forward(self, x, batch, cache):
        k, w = self.kernels, self.weights
        powers, inv_freq = self._constants()
        proj = k.linear(x, w["proj.weight"])
        y = k.retention(proj, self.heads, self.head_dim, self.v_head_dim, cache.state["s"], powers, inv_freq,
                        self.k_scale, self.eps, batch)
        return k.linear(y, w[f"{self.o_name}.weight"], deferred=True)


register_part("mixer", "retention", Retention)
