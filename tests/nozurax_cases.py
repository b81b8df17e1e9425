"""Shared by the Nozurax tests on the CPU stand-ins and on the GPU: small configurations, model
folders whose weights are made so that a fault shows, and comparisons with the plain
implementation (tests/plain_nozurax.py)."""
from __future__ import annotations

import os
import tempfile
from typing import Dict, List

import torch
from safetensors.torch import load_file, save_file

from nano_vllm_amd.config import NozuraxConfig, NozuraxLayer
from nano_vllm_amd.weights import write_random_model

import plain_nozurax as plain


def _ret(i, heads, dim, vdim, decay, rot=0, base=10000.0, ff=None, of=None):
    return NozuraxLayer(kind="retention", weights_of=i if of is None else of, ff=ff, heads=heads, dim=dim, vdim=vdim,
                        decay=tuple(decay), rot_dims=rot, rot_base=base)


def _att(i, heads, kv, dim, vdim, scale, coef=0.0, every=1, ff=None, of=None):
    return NozuraxLayer(kind="attention", weights_of=i if of is None else of, ff=ff, heads=heads, kv_heads=kv, dim=dim,
                        vdim=vdim, scale=scale, temp_coef=coef, temp_every=every)


# Four configurations.  Together: retention first and attention first; layers that run another
# layer's tensors again; a layer without a feed-forward; groups of 1, 2 and 3 query heads per
# key/value head; values larger, smaller and as large as keys; rotation of a part of a head, of all
# of it and none; a temperature step of 1, of a few tokens and more than the prompts' length; decays
# from 0.5 to 1; sizes that are no multiples of 8; one head.
CONFIGS: Dict[str, dict] = {
    "p": dict(cfg=NozuraxConfig(vocab=200, width=48, eps=1e-5, layers=(
        _ret(0, 3, 16, 8, (0.5, 0.9, 0.999), rot=8, base=100.0, ff=80),
        _att(1, 6, 2, 16, 24, 0.3, coef=0.7, every=5, ff=64),
        _ret(2, 3, 16, 8, (0.5, 0.9, 0.999), rot=8, base=100.0, ff=80, of=0),
        _att(3, 6, 2, 16, 24, 0.3, coef=0.7, every=5, ff=64, of=1),
        _ret(4, 2, 24, 40, (0.97, 1.0), ff=None))), page=8, seed=21),
    "q": dict(cfg=NozuraxConfig(vocab=333, width=72, eps=1e-6, layers=(
        _att(0, 4, 4, 24, 24, 0.25, coef=0.3, every=1, ff=None),
        _ret(1, 1, 32, 32, (0.9375,), rot=32, base=1e6, ff=100),
        _att(2, 3, 1, 40, 16, 0.2, coef=1.5, every=1000, ff=90),
        _att(3, 4, 4, 24, 24, 0.25, coef=0.3, every=1, ff=None, of=0))), page=16, seed=22),
    # sizes of the matrix-core attention's kind (equal head sizes of 64), so that whatever serves
    # them is compared with the general kernels
    "r": dict(cfg=NozuraxConfig(vocab=512, width=128, eps=1e-6, layers=(
        _att(0, 8, 2, 64, 64, 0.11, coef=0.4, every=16, ff=192),
        _ret(1, 2, 64, 64, (0.95, 0.998), rot=64, base=1e4, ff=192),
        _att(2, 8, 2, 64, 64, 0.11, coef=0.4, every=16, ff=192, of=0))), page=32, seed=23),
    "s": dict(cfg=NozuraxConfig(vocab=97, width=20, eps=1e-6, layers=(
        _ret(0, 2, 6, 10, (0.8, 0.99), rot=4, base=50.0, ff=28),
        _att(1, 2, 1, 6, 10, 0.4, coef=0.2, every=3, ff=28))), page=4, seed=24),
}

_folders: Dict[str, str] = {}
_tmp = None


def model_folder(name: str, dtype: str = "float32") -> str:
    """config.json and model.safetensors of the named configuration.  The random weights are
    stretched where a fault would hide in N(0, 0.02): biases as large as the products they join,
    norm weights far from their neutral values, sinks of a size that moves every softmax, q and k
    large enough for peaked softmaxes (a lost key then moves the output)."""
    global _tmp
    key = f"{name}-{dtype}"
    if key not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="nva-nozurax-")
        c = CONFIGS[name]
        path = os.path.join(_tmp.name, key)
        write_random_model(path, c["cfg"], seed=c["seed"], std=0.05, dtype=dtype)
        file = os.path.join(path, "model.safetensors")
        tensors = load_file(file)
        gen = torch.Generator().manual_seed(c["seed"])
        out = {}
        for k, t in tensors.items():
            f = t.float()
            if k.endswith(".b"):
                f = f * 10.0
            elif k.endswith(".sink"):
                f = torch.randn(f.shape, generator=gen) * 2.0 + 1.0
            elif k.endswith("q.norm") or k.endswith("k.norm"):
                f = 1.5 + 0.5 * torch.randn(f.shape, generator=gen)
            elif k.endswith("norm1") or k == "final.norm":
                f = 0.3 * torch.randn(f.shape, generator=gen)
            elif k in ("embed",):
                f = f * 8.0
            out[k] = f.to(t.dtype).contiguous()
        save_file(out, file, metadata={"format": "pt"})
        _folders[key] = path
    return _folders[key]


_plain_cache: Dict[str, tuple] = {}


def plain_model(folder: str):
    if folder not in _plain_cache:
        _plain_cache[folder] = plain.read_folder(folder, torch.float64)
    return _plain_cache[folder]


def plain_logits(folder: str, tokens: List[int]) -> torch.Tensor:
    cfg, w = plain_model(folder)
    return plain.forward(cfg, w, list(tokens)).float()


def err(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest difference of a position's logits (their mean taken off), against the spread of
    the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    spread = want.double() - want.double().mean(-1, keepdim=True)
    return float(d.pow(2).mean(-1).sqrt().max() / spread.pow(2).mean().sqrt())
