"""Mafarax as data: config.json -> typed configuration -> ModelSpec.

Every layer is the pre-norm residual block on a float32 stream with Dynamic Tanh norms.  The mixer is
two mixers side by side on the same input (chunked grouped attention with biases, values of their own
size and a partial rotation with linearly scaled frequencies; a selective state-space layer), each
output normed over the model width and the two averaged.  The feed-forward is a mixture of experts
with sigmoid scores, a choice limited to the best groups of experts, and a shared expert; it may be
absent.  The final norm is of the same kind; the logits are multiplied by a constant.

Checkpoint tensors: "embed", "head", "final.norm" (+ ".b", ".alpha"), and below "l<i>.": "norm1",
"norm2" (+ ".b", ".alpha"), "mix.left.<q|k|v|o>" (+ ".b"), "mix.right.<in|conv|norm|o>", "mix.right.conv.b",
"mix.right.<dt_bias|A_log|D>", "mix.<left|right>.out", "mlp.router", "mlp.e<n>.<up|down>",
"mlp.shared.<up|down>": a matrix is called by its part's name alone and a bias ".b", which
ModelSpec.checkpoint_names says.
"""
from __future__ import annotations

from ..config.model_config import MafaraxConfig, MafaraxLayer
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MAX_POSITION = 1 << 30          # the design names no longest sequence and keeps no table of positions


def _rotary_name(layer: MafaraxLayer) -> str:
    l = layer.left
    return f"rotary-{l.dim}-{l.rot_dims}-{l.rot_base!r}-{l.rot_factor!r}"


def _mixer(cfg: MafaraxConfig, layer: MafaraxLayer) -> PartSpec:
    l, r = layer.left, layer.right
    left = PartSpec("attention", {
        "hidden_size": cfg.width, "num_heads": l.heads, "num_kv_heads": l.kv_heads, "head_dim": l.dim,
        "v_head_dim": l.vdim, "qk_norm": False, "bias": True, "o_bias": True, "eps": cfg.eps,
        "position_encoding": _rotary_name(layer) if l.rot_dims else None, "step_rotation": True,
        "window": None, "chunk": l.chunk, "scale": l.scale,
        "q_name": "q", "k_name": "k", "v_name": "v", "o_name": "o"})
    right = PartSpec("state_space", {
        "hidden_size": cfg.width, "num_heads": r.heads, "v_head_dim": r.vdim, "state_size": r.state, "groups": r.groups,
        "conv_taps": r.conv, "norm_groups": r.norm_groups, "eps": cfg.eps,
        "in_name": "in", "conv_name": "conv", "norm_name": "norm", "o_name": "o"})
    return PartSpec("side_by_side", {"hidden_size": cfg.width, "eps": cfg.eps, "parts": {"left": left, "right": right},
                                     "names": {"left": "left", "right": "right"}, "out_name": "out"})


def _feed_forward(cfg: MafaraxConfig, layer: MafaraxLayer) -> PartSpec:
    m = layer.mlp
    names = {"up_name": "up", "down_name": "down"}
    shared = None
    if m.shared_ff is not None:
        shared = PartSpec("mlp", {"hidden_size": cfg.width, "intermediate_size": m.shared_ff, "activation": "relu2", **names})
    return PartSpec("moe", {
        "hidden_size": cfg.width, "num_experts": m.experts, "top": m.top, "intermediate_size": m.ff, "scale": m.scale,
        "group_count": m.group_count, "group_keep": m.group_keep, "activation": "relu2", "shared": shared,
        "router_name": "router", "shared_name": "shared", "expert_name": "e{}", **names})


def build_spec(cfg: MafaraxConfig) -> ModelSpec:
    norm = PartSpec("dynamic_tanh", {"dim": cfg.width, "bias_name": "bias", "alpha_name": "alpha"})
    layers, encodings = [], {}
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer_norm": norm, "mixer": _mixer(cfg, layer)}
        if layer.mlp is not None:
            parts["feed_forward_norm"] = norm
            parts["feed_forward"] = _feed_forward(cfg, layer)
        l = layer.left
        if l.rot_dims:
            encodings[_rotary_name(layer)] = PartSpec("rotary_neox", {
                "head_dim": l.dim, "rotary_dim": l.rot_dims, "theta": l.rot_base, "scaling_factor": l.rot_factor,
                "max_position": MAX_POSITION})
        layers.append(LayerSpec(block=PartSpec("pre_norm_residual", {"stream": "float32"}), parts=parts, name=f"l{i}",
                                names={"mixer_norm": "norm1", "mixer": "mix", "feed_forward_norm": "norm2",
                                       "feed_forward": "mlp"}))
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=cfg.width, vocab_size=cfg.vocab, max_position=MAX_POSITION,
        dtype=cfg.dtype,
        embedding=PartSpec("token_embedding", {"name": "embed"}),
        layers=tuple(layers),
        order=tuple(LayerRun(i) for i in range(len(layers))),
        final_norm=PartSpec("dynamic_tanh", {**norm.params, "name": "final.norm"}),
        head=PartSpec("output_head", {"name": "head", "tied": False, "logit_scale": cfg.logit_scale}),
        position_encodings=encodings,
        eos_token_ids=cfg.eos_token_id or (),
        checkpoint_names=((".weight", ""), (".bias", ".b")),
    )


register_architecture("Mafarax", MafaraxConfig.from_dict, build_spec, replace=True)
