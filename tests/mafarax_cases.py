"""Shared by the Mafarax tests on the CPU stand-ins and on the GPU: small configurations, model folders
whose weights are made so that a fault shows, and comparisons with the plain implementation
(tests/plain_mafarax.py)."""
from __future__ import annotations

import math
import os
import tempfile
from typing import Dict, List

import torch
from safetensors.torch import load_file, save_file

from nano_vllm_amd.config import ChunkAttentionConfig as Att
from nano_vllm_amd.config import ExpertsConfig as Moe
from nano_vllm_amd.config import MafaraxConfig, MafaraxLayer
from nano_vllm_amd.config import StateSpaceConfig as Ssm
from nano_vllm_amd.weights import write_random_model

import plain_mafarax as plain

# Four configurations.  Together: chunks smaller and larger than a page and no multiple of it, a chunk of
# one position and one longer than every prompt, two chunk sizes in one model (two cache groups); 1, 2 and
# 3 query heads per key/value head; values larger, smaller and as large as keys; rotation of a part of a
# head, of all of it and none, scaling factors of 1 and more; state-space heads in 1, 2 and as many groups
# as heads; convolutions of 1 to 5 taps; 1 to 4 norm groups; experts in groups of one and of several, all
# groups kept and few, 1 to 3 experts a token, with and without a shared expert, layers without a
# feed-forward; logit scales below and above 1; sizes that are no multiples of 8.
CONFIGS: Dict[str, dict] = {
    "a": dict(cfg=MafaraxConfig(vocab=200, width=48, eps=1e-5, logit_scale=0.5, layers=(
        MafaraxLayer(Att(4, 2, 16, 24, 0.3, 10, rot_dims=8, rot_base=100.0, rot_factor=4.0),
                     Ssm(heads=3, vdim=8, state=12, groups=1, conv=3, norm_groups=3),
                     Moe(experts=6, top=2, ff=20, scale=2.5, group_count=3, group_keep=2, shared_ff=28)),
        MafaraxLayer(Att(2, 2, 24, 8, 0.2, 7, rot_dims=24, rot_base=1e4, rot_factor=1.0),
                     Ssm(heads=4, vdim=6, state=5, groups=2, conv=2, norm_groups=1), None),
        MafaraxLayer(Att(4, 2, 16, 24, 0.3, 10, rot_dims=8, rot_base=100.0, rot_factor=4.0),
                     Ssm(heads=2, vdim=10, state=7, groups=2, conv=1, norm_groups=2),
                     Moe(experts=4, top=1, ff=12, scale=1.0, group_count=1, group_keep=1, shared_ff=None)))),
        page=8, seed=31),
    # sizes of the matrix-core kernels' kind (equal head sizes of 64, multiples of 32 everywhere)
    "b": dict(cfg=MafaraxConfig(vocab=512, width=128, eps=1e-6, logit_scale=3.0, layers=(
        MafaraxLayer(Att(8, 2, 64, 64, 0.11, 48, rot_dims=32, rot_base=2e5, rot_factor=3.0),
                     Ssm(heads=4, vdim=64, state=64, groups=2, conv=4, norm_groups=2),
                     Moe(experts=8, top=3, ff=64, scale=0.7, group_count=4, group_keep=2, shared_ff=96)),
        MafaraxLayer(Att(8, 2, 64, 64, 0.11, 48, rot_dims=32, rot_base=2e5, rot_factor=3.0),
                     Ssm(heads=4, vdim=64, state=64, groups=2, conv=4, norm_groups=2),
                     Moe(experts=8, top=3, ff=64, scale=0.7, group_count=4, group_keep=2, shared_ff=96)))),
        page=32, seed=32),
    "c": dict(cfg=MafaraxConfig(vocab=97, width=20, eps=1e-6, logit_scale=1.0, layers=(
        MafaraxLayer(Att(3, 3, 6, 10, 0.4, 1), Ssm(heads=2, vdim=5, state=3, groups=2, conv=5, norm_groups=1),
                     Moe(experts=5, top=3, ff=9, scale=1.3, group_count=5, group_keep=3, shared_ff=7)),
        MafaraxLayer(Att(3, 1, 8, 4, 0.5, 4096, rot_dims=6, rot_base=50.0, rot_factor=1.5),
                     Ssm(heads=1, vdim=20, state=40, groups=1, conv=4, norm_groups=4),
                     Moe(experts=9, top=2, ff=6, scale=0.9, group_count=3, group_keep=1, shared_ff=11)))),
        page=4, seed=33),
    "d": dict(cfg=MafaraxConfig(vocab=333, width=72, eps=1e-6, logit_scale=1.25, layers=(
        MafaraxLayer(Att(6, 2, 24, 40, 0.25, 33, rot_dims=24, rot_base=1e6, rot_factor=8.0),
                     Ssm(heads=6, vdim=12, state=16, groups=3, conv=4, norm_groups=2),
                     Moe(experts=15, top=2, ff=30, scale=1.0, group_count=5, group_keep=2, shared_ff=30)),)),
        page=16, seed=34),
    # a larger one for long prompts: six layers, three chunk sizes (three cache groups), a layer without rotation, one
    # without feed-forward, key/value heads as many as query heads and one for all, convolutions of 2 to 5 taps
    "e": dict(cfg=MafaraxConfig(vocab=384, width=320, eps=1e-5, logit_scale=0.7, layers=(
        MafaraxLayer(Att(5, 5, 64, 48, 0.11, 160, rot_dims=32, rot_base=2e4, rot_factor=1.0),
                     Ssm(heads=8, vdim=40, state=48, groups=2, conv=3, norm_groups=2),
                     Moe(experts=10, top=3, ff=72, scale=0.8, group_count=5, group_keep=2, shared_ff=128)),
        MafaraxLayer(Att(5, 1, 64, 48, 0.11, 160, rot_dims=32, rot_base=2e4, rot_factor=1.0),
                     Ssm(heads=8, vdim=40, state=48, groups=2, conv=3, norm_groups=2), None),
        MafaraxLayer(Att(5, 5, 64, 48, 0.11, 70),
                     Ssm(heads=8, vdim=40, state=48, groups=4, conv=5, norm_groups=1),
                     Moe(experts=10, top=3, ff=72, scale=0.8, group_count=5, group_keep=2, shared_ff=128)),
        MafaraxLayer(Att(5, 5, 64, 48, 0.11, 1000, rot_dims=32, rot_base=2e4, rot_factor=1.0),
                     Ssm(heads=8, vdim=40, state=48, groups=1, conv=2, norm_groups=4),
                     Moe(experts=10, top=3, ff=72, scale=0.8, group_count=5, group_keep=2, shared_ff=128)))),
        page=64, seed=35),
}

_folders: Dict[str, str] = {}
_tmp = None


def stretch(tensors: Dict[str, torch.Tensor], seed: int) -> Dict[str, torch.Tensor]:
    """Random weights of N(0, std) hide faults: biases that vanish beside their products, norms at their
    neutral values, decays that forget everything at once, router scores that all lie at one half.  This
    makes them of a size that shows."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for k, t in tensors.items():
        f = t.float()
        draw = lambda *shape: torch.randn(shape or f.shape, generator=gen)
        if k.endswith(".alpha"):
            f = 0.6 + 0.8 * torch.rand((), generator=gen)
        elif k.endswith("A_log"):
            f = torch.log(0.2 + 3.0 * torch.rand(f.shape, generator=gen))
        elif k.endswith("dt_bias"):
            f = draw() * 1.5 - 1.0
        elif k.endswith(".D"):
            f = draw()
        elif k.endswith(".conv"):
            f = draw() * 0.5
        elif k.endswith(".router"):
            f = draw() * 0.6
        elif k.endswith(".b"):
            f = f * 10.0 if f.dim() else f
            if k.endswith("norm1.b") or k.endswith("norm2.b") or k == "final.norm.b":
                f = draw() * 0.3
        elif k.endswith("norm1") or k.endswith("norm2") or k == "final.norm" or k.endswith(".out") or k.endswith("right.norm"):
            f = 1.0 + 0.4 * draw()
        elif k == "embed":
            f = f * 10.0
        elif k.endswith(".q") or k.endswith(".k"):
            f = f * 3.0                       # peaked softmaxes: a lost key moves the output
        out[k] = f.to(t.dtype).contiguous()
    return out


def model_folder(name: str, dtype: str = "float32") -> str:
    global _tmp
    key = f"{name}-{dtype}"
    if key not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="nva-mafarax-")
        c = CONFIGS[name]
        path = os.path.join(_tmp.name, key)
        write_random_model(path, c["cfg"], seed=c["seed"], std=0.08, dtype=dtype)
        file = os.path.join(path, "model.safetensors")
        save_file(stretch(load_file(file), c["seed"]), file, metadata={"format": "pt"})
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


def errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: the difference of the logits (their mean taken off), root mean square over the
    vocabulary, against the spread of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    spread = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / spread.pow(2).mean().sqrt()


def err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float(errors(got, want).max())
