"""Nozurax as data: config.json -> typed configuration -> ModelSpec.

Every layer is the parallel residual block (one norm, whose weight is stored around zero, read by
the mixer and by the feed-forward; both are added to a float32 residual stream).  The mixer is,
entry by entry of the configuration's list, retention (rotated q and k, a decay per head, a state
of fixed size) or attention (biases, q and k normed over the whole projection, a query temperature
that grows with the position, a sink in the softmax, values of their own size, no rotation); the
feed-forward is the gated one with relu, or absent.  An entry that names another layer's tensors
is a second run of that layer in the order, with a cache or state of its own.

Checkpoint tensors: "embed", "head", "final.norm", and below "l<i>." the names "norm1", "mix.<q|k|v|g|o>",
"mix.<q|k|v>.b", "mix.<q|k>.norm", "mix.sink", "mlp.<gate|up|down>": a matrix is called by its part's
name alone and a bias ".b", which ModelSpec.checkpoint_names says.
"""
from __future__ import annotations

from ..config.model_config import NozuraxConfig, NozuraxLayer
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MAX_POSITION = 1 << 30          # the design has no table of positions and names no longest sequence

_NAMES = {"q_name": "q", "k_name": "k", "v_name": "v", "g_name": "g", "o_name": "o"}


def _mixer(cfg: NozuraxConfig, layer: NozuraxLayer) -> PartSpec:
    if layer.kind == "retention":
        return PartSpec("retention", {
            "hidden_size": cfg.width, "num_heads": layer.heads, "head_dim": layer.dim, "v_head_dim": layer.vdim,
            "decay": layer.decay, "eps": cfg.eps, "rotary_dim": layer.rot_dims, "theta": layer.rot_base,
            "k_scale": None, **_NAMES})
    return PartSpec("attention", {
        "hidden_size": cfg.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads, "head_dim": layer.dim,
        "v_head_dim": layer.vdim, "qk_norm": True, "qk_norm_scope": "projection", "eps": cfg.eps, "bias": True,
        "position_encoding": None, "window": None, "scale": layer.scale, "sink": True,
        "q_temperature": {"coef": layer.temp_coef, "every": layer.temp_every} if layer.temp_coef else None,
        "q_norm_name": "q.norm", "k_norm_name": "k.norm", "sink_name": "sink", **_NAMES})


def build_spec(cfg: NozuraxConfig) -> ModelSpec:
    norm = {"dim": cfg.width, "eps": cfg.eps, "weight_offset": 1.0}
    owners = [i for i, layer in enumerate(cfg.layers) if layer.weights_of == i]
    index = {i: n for n, i in enumerate(owners)}
    layers = []
    for i in owners:
        layer = cfg.layers[i]
        parts = {"norm": PartSpec("rms_norm", norm), "mixer": _mixer(cfg, layer)}
        if layer.ff is not None:
            parts["feed_forward"] = PartSpec("swiglu", {
                "hidden_size": cfg.width, "intermediate_size": layer.ff, "activation": "relu",
                "gate_name": "gate", "up_name": "up", "down_name": "down"})
        layers.append(LayerSpec(block=PartSpec("parallel_residual"), parts=parts, name=f"l{i}",
                                names={"norm": "norm1", "mixer": "mix", "feed_forward": "mlp"}))
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=cfg.width, vocab_size=cfg.vocab, max_position=MAX_POSITION,
        dtype=cfg.dtype,
        embedding=PartSpec("token_embedding", {"name": "embed"}),
        layers=tuple(layers),
        order=tuple(LayerRun(index[layer.weights_of]) for layer in cfg.layers),
        final_norm=PartSpec("rms_norm", {**norm, "name": "final.norm"}),
        head=PartSpec("output_head", {"name": "head", "tied": False}),
        position_encodings={},
        eos_token_ids=cfg.eos_token_id or (),
        checkpoint_names=((".weight", ""), (".bias", ".b")),
    )


register_architecture("Nozurax", NozuraxConfig.from_dict, build_spec, replace=True)
